"""Writes tests/golden/ref_calib.npz: inputs and outputs of the reference's own
`compute_bias_std_coef` (utils_functional.py:900-949), the one function of the path that no
compiled-extension vector pins.

The reference module is imported from /root/reference in this container only.  Its top-level imports
name four extension modules: the two CPU ones are the reference's own sources compiled by
oracle/build.py into oracle/_ref/; the two CUDA ones cannot exist here and are not touched by the
function, so empty placeholder modules stand in for their names during the import.  Only data is
stored: the float32 input vectors, (or_n, order) and the two float32 coefficient vectors.

    python oracle/build.py && python tests/golden/make_golden_calib.py
"""
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


def orn(x, n):
    e = np.exp(-x)
    if n == 1:
        return 1 - e
    if n == 2:
        return 2 - 2 * e - x * e
    if n == 3:
        return 3 - 3 * e - 2 * x * e - 0.5 * x * x * e
    return 4 - 4 * e - 3 * x * e - x * x * e - x ** 3 * e / 6


def main():
    rng = np.random.default_rng(2025)
    out = {}
    cases = []
    # (name, n, or_n, order, spread of the surrogate values, noise, planted bias)
    for name, n, or_n, order, hi, noise, bias in [
            ("or2_o5_wide", 40000, 2, 5, 6.0, 0.04, (0.02, -0.03, 0.004)),
            ("or3_o4_wide", 30000, 3, 4, 7.0, 0.03, (0.0, 0.02, -0.002)),
            ("or2_o5_narrow", 10000, 2, 5, 1.5, 0.05, (0.01, 0.0, 0.0)),      # few valid windows: bias fit suppressed
            ("or1_o2", 20000, 1, 2, 5.0, 0.02, (-0.01, 0.01, 0.0)),
            ("or4_o3_sparse", 3000, 4, 3, 8.0, 0.05, (0.0, 0.01, 0.0)),
            ("neg_orn", 1000, -1, 5, 3.0, 0.05, (0.0, 0.0, 0.0))]:
        x = rng.uniform(0, hi, n)
        act = orn(x, max(or_n, 1)).astype(np.float32)
        a64 = act.astype(np.float64)
        bit = (a64 + bias[0] + bias[1] * a64 + bias[2] * a64 * a64 +
               noise * (0.5 + 0.3 * a64) * rng.normal(size=n)).astype(np.float32)
        b, s = ref.compute_bias_std_coef(or_n, torch.from_numpy(bit), torch.from_numpy(act), order)
        out[name + "_bit"] = bit
        out[name + "_act"] = act
        out[name + "_bias"] = b.detach().cpu().numpy().astype(np.float32)
        out[name + "_std"] = s.detach().cpu().numpy().astype(np.float32)
        cases.append("%s,%d,%d" % (name, or_n, order))
        print(name, or_n, order, out[name + "_bias"], out[name + "_std"])
    out["cases"] = np.array(cases)
    np.savez_compressed(os.path.join(HERE, "ref_calib.npz"), **out)


if __name__ == "__main__":
    main()
