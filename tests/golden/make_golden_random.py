"""Writes tests/golden/ref_cpu_ext_random.npz: seeded random configurations run through the
reference's own compiled CPU extension (oracle/_ref/, built by oracle/build.py from
/root/reference), in the key layout of ref_cpu_ext.npz.

    python oracle/build.py && python tests/golden/make_golden_random.py

make_golden.py holds hand-picked cases; these add breadth: random shapes with channel tails,
kernel sizes 1..5 (also non-square), strides, asymmetric padding, stream lengths 8..256, explicit
LFSR lengths, every OR-n / "nth-bit" / full_bin rule, both generators, progressive loading, both
memory orders for both operands; and for the fixed-point conv random precisions and adders.
Configurations on which the reference itself writes out of bounds or faults are left out (linear
op with a gen_config that does not divide the stream length, sc_matmul.cpp:336-337; linear op with
an 8-bit LFSR, see below).
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


def lattice(rng, shape, density, lo, hi, grid):
    v = np.round(rng.uniform(lo, hi, size=shape) * grid) / grid
    v *= rng.uniform(size=shape) < density
    return v.astype(np.float32)


def pick(rng, seq):
    return seq[int(rng.integers(0, len(seq)))]


def main():
    rng = np.random.default_rng(777)
    out, meta = {}, {"conv": [], "linear": [], "fixed": []}
    for i in range(48):
        L = pick(rng, [8, 16, 32, 32, 32, 64, 64, 128, 256])
        lb = L.bit_length() - 1
        lfsr = pick(rng, [-1, -1, -1, min(8, lb + 1), min(8, lb + 2)])
        S = (1 << lfsr) if lfsr > 0 else L
        N, C = int(rng.integers(1, 3)), pick(rng, [1, 3, 16, 31, 32, 33, 40, 64, 70])
        KH, KW = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        if rng.uniform() < 0.6:
            KW = KH
        pad = (int(rng.integers(0, KW // 2 + 2)), int(rng.integers(0, KH // 2 + 2)))  # (last axis, axis 2)
        stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        H = int(rng.integers(max(1, KH - 2 * pad[1]), KH + 6))
        W = int(rng.integers(max(1, KW - 2 * pad[0]), KW + 6))
        O = int(rng.integers(1, 13))
        bc = pick(rng, [0, 1, 1, 2, 3, -1, -2, 51200])
        gen = pick(rng, [1, 1, 2])
        prog = pick(rng, [(7, 8, 1), (7, 8, 1), (7, 2, 4), (7, 3, 2), (7, 4, 1)])
        cla, clw = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        dens = pick(rng, [0.05, 0.2, 0.5, 1.0])
        name = "rnd%02d" % i
        x = lattice(rng, (N, C, H, W), dens, 0.0, 1.0, S)
        w = lattice(rng, (O, C, KH, KW), dens, -1.0, 1.0, S)
        xt, wt = torch.from_numpy(x), torch.from_numpy(w)
        if cla:
            xt = xt.contiguous(memory_format=torch.channels_last)
        if clw:
            wt = wt.contiguous(memory_format=torch.channels_last)
        y = sc_extension.conv2d_generic_general(xt, wt, L, lfsr, 16, pad, stride, prog, bc, gen, True, False)
        y = y.contiguous().numpy()
        out["conv/%s/x" % name], out["conv/%s/w" % name], out["conv/%s/y" % name] = x, w, y
        meta["conv"].append(dict(name=name, stride=stride, padding=pad, bit_length=L, lfsr_length=lfsr,
                                 bin_config=bc, gen_config=gen, channels_last_activation=cla,
                                 channels_last_weight=clw, prog_load=prog))
        print("conv %s N%d C%d %dx%d O%d k%dx%d s%s p%s L%d lfsr%d bc%d g%d %s cl%d%d  out %s nonzero %.2f"
              % (name, N, C, H, W, O, KH, KW, stride, pad, L, lfsr, bc, gen, prog, cla, clw, y.shape,
                 (y != 0).mean()))
    for i in range(24):
        # Built with AVX-512 (this host), the reference's linear generators pick their vector LFSR step
        # from a switch without a case for 8 bits (sc_matmul.cpp:48-70, 258-279) and call the pointer
        # uninitialised: 256-bit streams and lfsr_length 8 fault there, so LFSRs stay at 7 bits or below.
        # (Built without AVX-512 the same sources run, but their linear op then returns different
        # numbers on repeated calls with the same operands, for every LFSR length: no use as a reference.)
        L = pick(rng, [8, 16, 32, 64, 64, 128])
        lb = L.bit_length() - 1
        lfsr = pick(rng, [-1, -1, min(7, lb + 1)])
        S = (1 << lfsr) if lfsr > 0 else L
        B, C, O = int(rng.integers(1, 70)), pick(rng, [1, 5, 32, 33, 64, 100, 200, 513]), int(rng.integers(1, 40))
        bc = pick(rng, [0, 1, 1, 2, 3, -1, -2, 51200])
        gen = pick(rng, [1, 1, 2])  # both divide every stream length used here
        prog = pick(rng, [(7, 8, 1), (7, 8, 1), (7, 3, 2), (7, 2, 4)])
        dens = pick(rng, [0.03, 0.15, 0.5])
        name = "rnd%02d" % i
        x = lattice(rng, (B, C), dens, 0.0, 1.0, S)
        w = lattice(rng, (O, C), dens, -1.0, 1.0, S)
        pos, neg = sc_extension.linear_generic_general(torch.from_numpy(x), torch.from_numpy(w), prog, L, lfsr, bc,
                                                       gen, True, False)
        out["linear/%s/x" % name], out["linear/%s/w" % name] = x, w
        out["linear/%s/pos" % name], out["linear/%s/neg" % name] = pos.numpy(), neg.numpy()
        meta["linear"].append(dict(name=name, bit_length=L, lfsr_length=lfsr, bin_config=bc, gen_config=gen,
                                   prog_load=prog))
        print("linear %s B%d C%d O%d L%d lfsr%d bc%d g%d %s  pos max %d neg max %d"
              % (name, B, C, O, L, lfsr, bc, gen, prog, pos.max(), neg.max()))
    for i in range(24):
        pin = int(rng.integers(2, 8))
        pout = pick(rng, [24, 24, 2 * pin + 2, 2 * pin, 2 * pin - 2, pin + 3])
        add = pick(rng, [0, 0, 0, 1, 2])
        N, C = int(rng.integers(1, 3)), pick(rng, [1, 4, 5, 16, 32, 33])
        KH, KW = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        pad = (int(rng.integers(0, 2)), int(rng.integers(0, 2)))
        stride = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        H, W, O = int(rng.integers(KH, KH + 5)), int(rng.integers(KW, KW + 5)), int(rng.integers(1, 8))
        dens = pick(rng, [0.15, 0.5, 1.0])
        name = "rnd%02d" % i
        P2 = 1 << pin
        x = lattice(rng, (N, C, H, W), dens, 0.0, 1.0, 2 * P2)  # half-grid values exercise round()
        w = lattice(rng, (O, C, KH, KW), dens, -1.0, 1.0, 2 * P2)
        y = fixed_extension.conv2d_saturate(torch.from_numpy(x), torch.from_numpy(w), add, pin, pout, pad, stride)
        out["fixed/%s/x" % name], out["fixed/%s/w" % name], out["fixed/%s/y" % name] = x, w, y.numpy()
        meta["fixed"].append(dict(name=name, stride=stride, padding=pad, add_config=add, precision_in=pin,
                                  precision_out=pout))
        print("fixed %s N%d C%d %dx%d O%d k%dx%d s%s p%s add%d pin%d pout%d  nonzero %.2f min %d max %d"
              % (name, N, C, H, W, O, KH, KW, stride, pad, add, pin, pout, (y.numpy() != 0).mean(), y.min(), y.max()))
    out["meta"] = np.frombuffer(json.dumps(meta).encode(), dtype=np.uint8)
    path = os.path.join(HERE, "ref_cpu_ext_random.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
