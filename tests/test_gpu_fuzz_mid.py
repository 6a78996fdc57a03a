"""Seeded random configurations at layer-like sizes (up to 512 channels, 30x30 planes, 4096-wide
linear layers, every stream length, both generators, all three bitstream-generator modes) of the SC
conv / linear and fixed-point conv ops against the oracle.  One test per op family: the cases are
printed as they run, so a failure names its configuration."""
import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu


def test_conv_mid_sizes(monkeypatch):
    import _ops
    import sc_extension_cuda
    rng = np.random.default_rng(31337)
    for it in range(60):
        KH, KW = [(1, 1), (3, 3), (3, 3), (3, 3), (5, 5), (7, 7)][rng.integers(0, 6)]
        C = int(rng.choice([32, 64, 96, 128, 200, 256, 384, 512]))
        if KH >= 5:
            C = min(C, 128)
        O = int(rng.choice([16, 48, 64, 100, 128, 256]))
        H = int(rng.integers(KH + 3, 30))
        W = int(rng.integers(KW + 3, 30))
        N = int(rng.choice([1, 2, 3, 8]))
        s = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
        pad = (int(rng.integers(0, KW // 2 + 1)), int(rng.integers(0, KH // 2 + 1)))
        L = int(rng.choice([8, 16, 32, 32, 64, 128, 256]))
        if L >= 128:
            N, H, W = 1, min(H, 12), min(W, 12)
        gen = int(rng.choice([1, 1, 1, 2]))
        bc = int(rng.choice([0, 1, 1, 2, 3]))
        cla, clw = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        mode = str(rng.choice(["0", "1", "2"]))
        monkeypatch.setenv("REXSC_SNG_MODE", mode)
        dens = min(1.0, 8.0 / (C * KH * KW) + 0.03)
        x = (rng.integers(0, L + 1, size=(N, C, H, W)) / L * (rng.uniform(size=(N, C, H, W)) < 3 * dens)).astype(np.float32)
        w = (rng.integers(-L, L + 1, size=(O, C, KH, KW)) / L * (rng.uniform(size=(O, C, KH, KW)) < 3 * dens)).astype(np.float32)
        xt, wt = torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()
        if cla:
            xt = xt.contiguous(memory_format=torch.channels_last)
        if clw:
            wt = wt.contiguous(memory_format=torch.channels_last)
        ce, we = _ops.is_channels_last(xt), _ops.is_channels_last(wt)
        print("conv", it, (N, C, H, W, O, KH, KW, s, pad, L, gen, bc, cla, clw, mode), flush=True)
        pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(xt, wt, L, -1, 16, pad, s, (7, 8, 1), bc, gen, True, False)
        op, on = orc.conv2d_generic_general_split(x, w, L, -1, 16, pad, s, (7, 8, 1), bc, gen,
                                                  channels_last_activation=ce, channels_last_weight=we)
        assert np.array_equal(pos.cpu().numpy(), op) and np.array_equal(neg.cpu().numpy(), on)


def test_linear_mid_sizes(monkeypatch):
    import sc_extension
    rng = np.random.default_rng(4242)
    for it in range(30):
        B = int(rng.choice([7, 64, 100, 256, 513]))
        C = int(rng.choice([64, 300, 1024, 2048, 4096]))
        O = int(rng.choice([10, 64, 200, 1000]))
        L = int(rng.choice([16, 32, 64, 128]))
        gen = int(rng.choice([1, 1, 2]))
        bc = int(rng.choice([0, 1, 2, -2, 51200]))
        mode = str(rng.choice(["0", "1", "2"]))
        monkeypatch.setenv("REXSC_SNG_MODE", mode)
        dens = 1.0 if bc > 100 else min(1.0, 8.0 / C + 0.02)
        x = (rng.integers(0, L + 1, size=(B, C)) / L * (rng.uniform(size=(B, C)) < 2 * dens)).astype(np.float32)
        w = (rng.integers(-L, L + 1, size=(O, C)) / L * (rng.uniform(size=(O, C)) < 2 * dens)).astype(np.float32)
        print("linear", it, (B, C, O, L, gen, bc, mode), flush=True)
        pos, neg = sc_extension.linear_generic_general(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), (7, 8, 1), L,
                                                       -1, bc, gen, True, False)
        op, on = orc.linear_generic_general(x, w, (7, 8, 1), L, -1, bc, gen)
        assert np.array_equal(pos.cpu().numpy(), op) and np.array_equal(neg.cpu().numpy(), on)


def test_fixed_conv_mid_sizes():
    import fixed_extension_cuda
    rng = np.random.default_rng(777)
    for it in range(24):
        C = int(rng.choice([16, 64, 100, 256]))
        O = int(rng.choice([8, 64, 130]))
        H = int(rng.integers(5, 20))
        N = int(rng.choice([1, 4]))
        K = int(rng.choice([1, 3, 5]))
        pin = int(rng.choice([4, 5, 6]))
        pout = int(rng.choice([8, 16, 24]))
        add = int(rng.choice([0, 0, 1, 2]))
        x = (rng.integers(0, 1 << pin, size=(N, C, H, H)) / (1 << pin)).astype(np.float32)
        w = (rng.integers(-(1 << pin) + 1, 1 << pin, size=(O, C, K, K)) / (1 << pin)).astype(np.float32)
        print("fixed", it, (N, C, H, O, K, pin, pout, add), flush=True)
        y = fixed_extension_cuda.conv2d_saturate_acc(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), add, pin, pout,
                                                     (K // 2, K // 2), (1, 1))
        oy = orc.conv2d_saturate(x, w, add, pin, pout, (K // 2, K // 2), (1, 1))
        assert np.array_equal(y.cpu().numpy(), oy)
