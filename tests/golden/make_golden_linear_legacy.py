"""Writes tests/golden/ref_linear_legacy.npz: inputs and outputs of the reference's own legacy
`linear_generic` (utils_functional.py:955-1081), a pure-torch bit-by-bit simulation that no compiled-extension
vector pins (different seeds, different quantisation rule from the extension's linear op).

The reference module is imported from /root/reference in this container only, the way make_golden_calib.py
does it: its top-level imports name four extension modules; the two CPU ones are the reference's own sources
compiled by oracle/build.py into oracle/_ref/, the two CUDA ones cannot exist here and are not touched by the
function, so empty placeholder modules stand in for their names during the import.  Only data is stored:
float32 operands, the call's parameters and the float result (the reference returns float16; stored as float32).

    python oracle/build.py && python tests/golden/make_golden_linear_legacy.py
"""
import json
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle", "_ref"))
sys.path.insert(0, "/root/reference")
for name in ("sc_extension_cuda", "fixed_extension_cuda"):
    sys.modules[name] = types.ModuleType(name)

import utils_functional as ref  # noqa: E402

CASES = [
    # name, B, C, O, bit_length, forward, operand kind, density
    ("or_L128_q7", 6, 100, 9, 128, "full_or", "q7", 0.2),     # what Linear_Or runs: operands quantised to 1/128
    ("or_L32_q7", 5, 64, 8, 32, "full_or", "q7", 0.25),        # quarter-grid products, values reaching 32
    ("or_L64_plain", 7, 130, 6, 64, "full_or", "plain", 0.15), # plain floats: float16 rounding of the products
    ("or_L16_q7", 4, 33, 5, 16, "full_or", "q7", 0.3),
    ("or_L8_q7", 3, 20, 4, 8, "full_or", "q7", 0.4),
    ("bin_L32_q7", 5, 70, 7, 32, "full_bin", "q7", 0.5),
    ("bin_L128_plain", 4, 200, 5, 128, "full_bin", "plain", 0.7),
    ("or_L128_dense_ones", 3, 40, 4, 128, "full_or", "ones", 0.25),  # activations of exactly 1.0, weights of +-1.0
    # share=False: one generator per weight and per activation element, seeds running over the whole tensors (:996-998)
    ("or_L32_q7_noshare", 5, 64, 8, 32, "full_or", "q7", 0.25, False),
    ("or_L128_q7_noshare", 6, 100, 9, 128, "full_or", "q7", 0.2, False),
    ("bin_L64_plain_noshare", 4, 70, 17, 64, "full_bin", "plain", 0.5, False),   # 17 outputs: a ragged group of 16
    ("or_L16_q7_noshare", 3, 33, 5, 16, "full_or", "q7", 0.3, False),
]


def operands(rng, kind, B, C, O, dens):
    if kind == "plain":
        x = rng.uniform(-0.2, 1.1, size=(B, C))
        w = rng.uniform(-1.2, 1.2, size=(O, C))
    else:
        x = np.round(rng.uniform(0, 1, size=(B, C)) * 128).clip(0, 127) / 128
        w = np.round(rng.uniform(-1, 1, size=(O, C)) * 128).clip(-127, 127) / 128
        if kind == "ones":
            x = np.where(rng.uniform(size=x.shape) < 0.5, 1.0, x)
            w = np.where(rng.uniform(size=w.shape) < 0.3, np.sign(w), w)
    x = x * (rng.uniform(size=x.shape) < dens)
    w = w * (rng.uniform(size=w.shape) < dens)
    return x.astype(np.float32), w.astype(np.float32)


def main():
    rng = np.random.default_rng(6737)
    out, meta = {}, []
    for case in CASES:
        (name, B, C, O, L, forward, kind, dens), share = case[:8], (case[8] if len(case) > 8 else True)
        x, w = operands(rng, kind, B, C, O, dens)
        y = ref.linear_generic(torch.from_numpy(x), torch.from_numpy(w), bit_length=L, forward=forward, generator="lfsr",
                               share=share)
        y = y.detach().float().numpy()
        out[name + "/x"], out[name + "/w"], out[name + "/y"] = x, w, y
        meta.append(dict(name=name, bit_length=L, forward=forward, share=share))
        print(name, "out", y.shape, "min %.4f max %.4f nonzero %.2f" % (y.min(), y.max(), (y != 0).mean()))
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    path = os.path.join(HERE, "ref_linear_legacy.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
