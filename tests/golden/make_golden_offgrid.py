"""Writes tests/golden/ref_cpu_ext_offgrid.npz: operands that do NOT lie on the 1/S quantisation grid,
run through the reference's own compiled CPU extension (oracle/_ref/, built by oracle/build.py from
/root/reference), in the key layout of ref_cpu_ext.npz.

    python oracle/build.py && python tests/golden/make_golden_offgrid.py

The other two fixtures use operands rounded onto the 1/S grid, where ceil, round and floor agree.
The layers feed the op values quantised to 1/128 (prec 7) with 32- or 64-bit streams, and callers may
pass any float: here the wrappers' ceil(clamp(x*S, 0, S-1)) (sc_conv.cpp:318-320, sc_matmul.cpp:586-590)
and the fixed-point conv's round(clamp(...)) (fixed.cpp:207-210) are exercised on
  * values on the 1/128 grid with S = 32 and S = 64,
  * plain uniform floats, including activations below 0 and above 1 - 1/S and weights beyond +-1.
Only data is stored: float32 operands, integer parameters, integer outputs.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "oracle", "_ref"))

import fixed_extension  # noqa: E402  (compiled reference)
import sc_extension  # noqa: E402  (compiled reference)


def grid128(rng, shape, density, lo, hi):
    v = np.round(rng.uniform(lo, hi, size=shape) * 128) / 128
    v *= rng.uniform(size=shape) < density
    return v.astype(np.float32)


def plain(rng, shape, density, lo, hi):
    v = rng.uniform(lo, hi, size=shape)
    v *= rng.uniform(size=shape) < density
    return v.astype(np.float32)


CONV = [
    # name, maker, N,C,H,W, O,K, stride, pad, L, lfsr, bin_config, gen, cl_act, cl_w, density, (act lo, hi), (w lo, hi)
    ("g128_L32_or2", grid128, 2, 32, 8, 8, 12, 3, (1, 1), (1, 1), 32, -1, 1, 1, False, False, 0.25, (0, 1), (-1, 1)),
    ("g128_L64_or3_cl", grid128, 2, 40, 7, 7, 9, 3, (1, 1), (1, 1), 64, -1, 2, 1, True, False, 0.2, (0, 1), (-1, 1)),
    ("g128_L32_or2_c3", grid128, 2, 3, 10, 10, 8, 3, (1, 1), (1, 1), 32, -1, 1, 1, False, False, 1.0, (0, 1), (-1, 1)),
    ("g128_L32_or1_s2_1x1", grid128, 2, 64, 8, 8, 16, 1, (2, 2), (0, 0), 32, -1, 0, 1, True, True, 0.15, (0, 1), (-1, 1)),
    ("plain_L32_or2", plain, 2, 32, 8, 8, 12, 3, (1, 1), (1, 1), 32, -1, 1, 1, False, False, 0.25, (-0.3, 1.2), (-1.3, 1.3)),
    ("plain_L64_or2_cl", plain, 1, 33, 7, 9, 10, 3, (1, 2), (1, 0), 64, -1, 1, 1, True, True, 0.25, (-0.3, 1.2), (-1.3, 1.3)),
    ("plain_L16_or4_5x5", plain, 1, 20, 9, 9, 6, 5, (1, 1), (2, 2), 16, -1, 3, 1, False, False, 0.1, (-0.2, 1.1), (-1.1, 1.1)),
    ("plain_L32_lfsr7_and2", plain, 1, 16, 6, 6, 8, 3, (1, 1), (1, 1), 32, 7, 1, 2, False, False, 0.4, (-0.2, 1.1), (-1.1, 1.1)),
    ("plain_L128_fullbin", plain, 1, 16, 6, 6, 8, 3, (1, 1), (1, 1), 128, -1, 51200, 1, False, False, 0.6, (-0.2, 1.1), (-1.1, 1.1)),
    ("tiny_values_L32", plain, 1, 32, 6, 6, 8, 3, (1, 1), (1, 1), 32, -1, 1, 1, False, False, 1.0, (0, 0.04), (-0.04, 0.04)),
]

LINEAR = [
    # name, maker, B,C,O, L, lfsr, bin_config, gen, density, (act lo, hi), (w lo, hi)
    ("g128_L64_or2", grid128, 9, 100, 12, 64, -1, 1, 1, 0.15, (0, 1), (-1, 1)),
    ("g128_L32_or2", grid128, 33, 64, 10, 32, -1, 1, 1, 0.2, (0, 1), (-1, 1)),
    ("plain_L64_or2", plain, 17, 200, 14, 64, -1, 1, 1, 0.08, (-0.3, 1.2), (-1.3, 1.3)),
    ("plain_L32_orno2", plain, 8, 70, 9, 32, -1, -1, 1, 0.2, (-0.3, 1.2), (-1.3, 1.3)),
    ("plain_L128_fullbin_and2", plain, 5, 33, 7, 128, -1, 51200, 2, 0.5, (-0.2, 1.1), (-1.1, 1.1)),
]

FIXED = [
    # name, N,C,H,W, O,K, stride, pad, add_config, pin, pout, density, (act lo, hi), (w lo, hi)
    ("plain_p5_24", 2, 16, 7, 7, 6, 3, (1, 1), (1, 1), 0, 5, 24, 0.6, (-0.3, 1.2), (-1.3, 1.3)),
    ("plain_p6_10", 1, 33, 6, 6, 5, 3, (2, 1), (1, 0), 0, 6, 10, 0.07, (-0.2, 1.1), (-1.1, 1.1)),
    ("plain_p4_add1", 1, 8, 6, 6, 4, 3, (1, 1), (1, 1), 1, 4, 24, 0.8, (-0.2, 1.1), (-1.1, 1.1)),
    ("g128_p5_24", 2, 32, 6, 6, 8, 3, (1, 1), (1, 1), 0, 5, 24, 0.7, (0, 1), (-1, 1)),
]


def main():
    rng = np.random.default_rng(4242)
    out, meta = {}, {"conv": [], "linear": [], "fixed": []}
    for (name, mk, N, C, H, W, O, K, stride, pad, L, lfsr, bc, gen, cla, clw, dens, ar, wr) in CONV:
        name = "off_" + name
        x = mk(rng, (N, C, H, W), dens, *ar)
        w = mk(rng, (O, C, K, K), dens, *wr)
        xt, wt = torch.from_numpy(x), torch.from_numpy(w)
        if cla:
            xt = xt.contiguous(memory_format=torch.channels_last)
        if clw:
            wt = wt.contiguous(memory_format=torch.channels_last)
        y = sc_extension.conv2d_generic_general(xt, wt, L, lfsr, 16, pad, stride, (7, 8, 1), bc, gen, True, False)
        y = y.contiguous().numpy()
        S = (1 << lfsr) if lfsr > 0 else L
        off = float(np.mean((x * S) != np.round(x * S)))
        out["conv/%s/x" % name], out["conv/%s/w" % name], out["conv/%s/y" % name] = x, w, y
        meta["conv"].append(dict(name=name, stride=stride, padding=pad, bit_length=L, lfsr_length=lfsr, bin_config=bc,
                                 gen_config=gen, channels_last_activation=cla, channels_last_weight=clw,
                                 prog_load=(7, 8, 1)))
        print("conv %s out %s nonzero %.2f off-grid activations %.2f" % (name, y.shape, (y != 0).mean(), off))
    for (name, mk, B, C, O, L, lfsr, bc, gen, dens, ar, wr) in LINEAR:
        name = "off_" + name
        x = mk(rng, (B, C), dens, *ar)
        w = mk(rng, (O, C), dens, *wr)
        pos, neg = sc_extension.linear_generic_general(torch.from_numpy(x), torch.from_numpy(w), (7, 8, 1), L, lfsr, bc,
                                                       gen, True, False)
        out["linear/%s/x" % name], out["linear/%s/w" % name] = x, w
        out["linear/%s/pos" % name], out["linear/%s/neg" % name] = pos.numpy(), neg.numpy()
        meta["linear"].append(dict(name=name, bit_length=L, lfsr_length=lfsr, bin_config=bc, gen_config=gen,
                                   prog_load=(7, 8, 1)))
        print("linear %s pos max %d neg max %d" % (name, pos.max(), neg.max()))
    for (name, N, C, H, W, O, K, stride, pad, add, pin, pout, dens, ar, wr) in FIXED:
        mk = grid128 if name.startswith("g128") else plain
        name = "off_" + name
        x = mk(rng, (N, C, H, W), dens, *ar)
        w = mk(rng, (O, C, K, K), dens, *wr)
        y = fixed_extension.conv2d_saturate(torch.from_numpy(x), torch.from_numpy(w), add, pin, pout, pad, stride)
        out["fixed/%s/x" % name], out["fixed/%s/w" % name], out["fixed/%s/y" % name] = x, w, y.numpy()
        meta["fixed"].append(dict(name=name, stride=stride, padding=pad, add_config=add, precision_in=pin,
                                  precision_out=pout))
        print("fixed %s nonzero %.2f min %d max %d" % (name, (y.numpy() != 0).mean(), y.min(), y.max()))
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    path = os.path.join(HERE, "ref_cpu_ext_offgrid.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
