"""Writes tests/golden/ref_cpu_ext.npz: inputs and outputs of the reference's own CPU extension.

The reference ships no tests and no golden vectors, so the vectors are made here, once, by
running the reference's C++ CPU extension (sc_extension / fixed_extension, compiled from
/root/reference by oracle/build.py into oracle/_ref/) on small seeded inputs.  Only data
is stored: float32 operands, the call's integer parameters and the integer outputs.

    python oracle/build.py && python tests/golden/make_golden.py

Cases are chosen so that a plausible mistake changes the output: sparse operands (so OR-n
counts do not all saturate), odd channel counts (tail words), both memory orders for
operands, strides and asymmetric padding, every stream length, both generators, the
"nth-bit" rule of the linear op, progressive loading, int16 wrap-around (full_bin), and for
the fixed-point conv every add_config with and without accumulator truncation.
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


def sparse_uniform(rng, shape, density, lo, hi, grid):
    """Values on the 1/grid lattice in [lo, hi], a fraction `density` of them non-zero."""
    v = rng.uniform(lo, hi, size=shape)
    v = np.round(v * grid) / grid
    v *= rng.uniform(size=shape) < density
    return v.astype(np.float32)


CONV_CASES = [
    # name, N,C,H,W, O,KH,KW, stride, padding, L, lfsr_length, bin_config, gen, cl_act, cl_w, prog_load, density
    ("or1_c32", 2, 32, 8, 8, 16, 3, 3, (1, 1), (1, 1), 32, -1, 0, 1, False, False, (7, 8, 1), 0.15),
    ("or2_c3", 2, 3, 9, 7, 5, 3, 3, (1, 1), (1, 1), 32, -1, 1, 1, False, False, (7, 8, 1), 0.9),
    ("or3_c33_s2_L64", 1, 33, 6, 6, 7, 3, 3, (2, 2), (1, 1), 64, -1, 2, 1, False, False, (7, 8, 1), 0.3),
    ("or4_c64_1x1_L16", 2, 64, 6, 6, 8, 1, 1, (1, 1), (0, 0), 16, -1, 3, 1, False, False, (7, 8, 1), 0.3),
    ("or2_c40_5x5_L128_cla", 2, 40, 7, 7, 8, 5, 5, (1, 1), (2, 2), 128, -1, 1, 1, True, False, (7, 8, 1), 0.1),
    ("or2_c40_s21_p10_cla_clw", 2, 40, 7, 7, 8, 3, 3, (2, 1), (1, 0), 32, -1, 1, 1, True, True, (7, 8, 1), 0.2),
    ("or2_c16_clw", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 32, -1, 1, 1, False, True, (7, 8, 1), 0.4),
    ("or2_and2", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 32, -1, 1, 2, False, False, (7, 8, 1), 0.5),
    ("or3_and2_L64_c70", 1, 70, 5, 5, 6, 3, 3, (1, 1), (1, 1), 64, -1, 2, 2, False, False, (7, 8, 1), 0.3),
    ("fullbin_L8", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 8, -1, 51200, 1, False, False, (7, 8, 1), 1.0),
    ("fullbin_wrap_L256", 1, 96, 4, 4, 4, 3, 3, (1, 1), (1, 1), 256, -1, 51200, 1, False, False, (7, 8, 1), 1.0),
    ("or1_L4", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 4, -1, 0, 1, False, False, (7, 8, 1), 0.5),
    ("or1_L2", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 2, -1, 0, 1, False, False, (7, 8, 1), 0.5),
    ("orno2", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 32, -1, -1, 1, False, False, (7, 8, 1), 0.4),
    ("or2_prog_2_4", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 32, -1, 1, 1, False, False, (7, 2, 4), 0.5),
    ("or2_prog_3_2_L64", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 64, -1, 1, 1, False, False, (7, 3, 2), 0.5),
    ("or2_L256", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 256, -1, 1, 1, False, False, (7, 8, 1), 0.3),
    ("or2_L16", 1, 20, 6, 6, 8, 3, 3, (1, 1), (1, 1), 16, -1, 1, 1, False, False, (7, 8, 1), 0.3),
    ("or2_L32_lfsr7", 1, 16, 6, 6, 8, 3, 3, (1, 1), (1, 1), 32, 7, 1, 1, False, False, (7, 8, 1), 0.4),
    ("or2_7x7_s2_c3", 1, 3, 15, 15, 8, 7, 7, (2, 2), (3, 3), 32, -1, 1, 1, False, False, (7, 8, 1), 0.8),
    ("or2_c128_o40", 1, 128, 5, 5, 40, 3, 3, (1, 1), (1, 1), 32, -1, 1, 1, True, False, (7, 8, 1), 0.08),
]

LINEAR_CASES = [
    # name, B, C, O, L, lfsr_length, bin_config, gen, prog_load, density
    ("or1", 4, 64, 8, 32, -1, 0, 1, (7, 8, 1), 0.1),
    ("or2_c100_L64", 5, 100, 7, 64, -1, 1, 1, (7, 8, 1), 0.15),
    ("or2_blockedge", 130, 96, 130, 64, -1, 1, 1, (7, 8, 1), 0.15),
    ("orno2_L16", 3, 32, 3, 16, -1, -1, 1, (7, 8, 1), 0.4),
    ("or3_and2_L128", 3, 96, 3, 128, -1, 2, 2, (7, 8, 1), 0.2),
    ("fullbin", 3, 40, 5, 32, -1, 51200, 1, (7, 8, 1), 1.0),
    ("or2_prog_3_2", 3, 64, 5, 32, -1, 1, 1, (7, 3, 2), 0.3),
    ("or2_c512", 6, 512, 9, 64, -1, 1, 1, (7, 8, 1), 0.03),
]

FIXED_CASES = [
    # name, N,C,H,W, O,KH,KW, stride, padding, add_config, precision_in, precision_out, density
    ("add0_5_24", 2, 8, 6, 6, 4, 3, 3, (1, 1), (1, 1), 0, 5, 24, 1.0),
    ("add0_5_8_s2", 2, 8, 6, 6, 4, 3, 3, (2, 2), (1, 1), 0, 5, 8, 0.2),
    ("add0_5_9_sat", 1, 32, 5, 5, 4, 3, 3, (1, 1), (1, 1), 0, 5, 9, 0.6),
    ("add0_7_12", 1, 16, 6, 7, 4, 3, 3, (1, 1), (1, 1), 0, 7, 12, 0.15),
    ("add0_7_10", 1, 16, 6, 7, 4, 3, 3, (1, 1), (1, 1), 0, 7, 10, 0.1),
    ("add0_4_6_p10_s12", 1, 6, 7, 8, 5, 3, 2, (1, 2), (1, 0), 0, 4, 6, 0.5),
    ("add0_6_12_sat", 1, 64, 4, 4, 3, 3, 3, (1, 1), (1, 1), 0, 6, 12, 1.0),
    ("add1_5_24", 1, 5, 6, 7, 4, 3, 3, (1, 1), (1, 1), 1, 5, 24, 1.0),
    ("add1_6_8", 1, 5, 6, 7, 4, 3, 3, (1, 1), (1, 1), 1, 6, 8, 0.5),
    ("add2_5_24", 1, 5, 6, 7, 4, 3, 3, (1, 1), (1, 1), 2, 5, 24, 1.0),
    ("add2_5_24_even", 1, 4, 5, 5, 3, 2, 2, (1, 1), (0, 0), 2, 5, 24, 1.0),
]


def main():
    rng = np.random.default_rng(20240607)
    out = {}
    meta = {"conv": [], "linear": [], "fixed": []}
    for (name, N, C, H, W, O, KH, KW, stride, pad, L, lfsr, bc, gen, cla, clw, prog, dens) in CONV_CASES:
        S = (1 << lfsr) if lfsr > 0 else L
        x = sparse_uniform(rng, (N, C, H, W), dens, 0.0, 1.0, S)
        w = sparse_uniform(rng, (O, C, KH, KW), dens, -1.0, 1.0, S)
        xt, wt = torch.from_numpy(x), torch.from_numpy(w)
        if cla:
            xt = xt.contiguous(memory_format=torch.channels_last)
        if clw:
            wt = wt.contiguous(memory_format=torch.channels_last)
        y = sc_extension.conv2d_generic_general(xt, wt, L, lfsr, 16, pad, stride, prog, bc, gen, True, False)
        y = y.contiguous().numpy()
        assert y.dtype == np.int16
        out["conv/%s/x" % name] = x
        out["conv/%s/w" % name] = w
        out["conv/%s/y" % name] = y
        meta["conv"].append(dict(name=name, stride=stride, padding=pad, bit_length=L, lfsr_length=lfsr,
                                 bin_config=bc, gen_config=gen, channels_last_activation=cla,
                                 channels_last_weight=clw, prog_load=prog))
        print("conv %-28s out %s  nonzero %.2f  min %d max %d" % (name, y.shape, (y != 0).mean(), y.min(), y.max()))
    for (name, B, C, O, L, lfsr, bc, gen, prog, dens) in LINEAR_CASES:
        S = (1 << lfsr) if lfsr > 0 else L
        x = sparse_uniform(rng, (B, C), dens, 0.0, 1.0, S)
        w = sparse_uniform(rng, (O, C), dens, -1.0, 1.0, S)
        pos, neg = sc_extension.linear_generic_general(torch.from_numpy(x), torch.from_numpy(w), prog, L, lfsr,
                                                       bc, gen, True, False)
        out["linear/%s/x" % name] = x
        out["linear/%s/w" % name] = w
        out["linear/%s/pos" % name] = pos.numpy()
        out["linear/%s/neg" % name] = neg.numpy()
        meta["linear"].append(dict(name=name, bit_length=L, lfsr_length=lfsr, bin_config=bc, gen_config=gen,
                                   prog_load=prog))
        print("linear %-26s pos max %d neg max %d" % (name, pos.max(), neg.max()))
    for (name, N, C, H, W, O, KH, KW, stride, pad, add, pin, pout, dens) in FIXED_CASES:
        P2 = 1 << pin
        x = sparse_uniform(rng, (N, C, H, W), dens, 0.0, 1.0, 2 * P2)  # half-grid values exercise round()
        w = sparse_uniform(rng, (O, C, KH, KW), dens, -1.0, 1.0, 2 * P2)
        y = fixed_extension.conv2d_saturate(torch.from_numpy(x), torch.from_numpy(w), add, pin, pout, pad, stride)
        out["fixed/%s/x" % name] = x
        out["fixed/%s/w" % name] = w
        out["fixed/%s/y" % name] = y.numpy()
        meta["fixed"].append(dict(name=name, stride=stride, padding=pad, add_config=add, precision_in=pin,
                                  precision_out=pout))
        print("fixed %-26s nonzero %.2f min %d max %d" % (name, (y.numpy() != 0).mean(), y.min(), y.max()))
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    path = os.path.join(HERE, "ref_cpu_ext.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
