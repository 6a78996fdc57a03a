"""Seeded random configurations of the SC conv / linear ops against the oracle: small shapes with
awkward sizes (fewer pixels than a wave, channel tails, stream lengths from 2 to 256, both
generators, both layouts for both operands, strides, asymmetric padding, progressive loading).
Every configuration runs with both bitstream generators of the library (REXSC_SNG_MODE: 1 = lane
ballot, 2 = bit-sliced); left alone the library picks one per problem size."""
import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu


def _rand_conv_cfg(rng):
    KH, KW = [(1, 1), (3, 3), (3, 3), (5, 5), (7, 7), (2, 2), (1, 3), (3, 1)][rng.integers(0, 8)]
    C = int(rng.choice([1, 3, 16, 31, 32, 33, 64, 65, 96, 128, 130, 260]))
    O = int(rng.choice([1, 2, 15, 16, 17, 33, 64]))
    H = int(rng.integers(KH, KH + 9))
    W = int(rng.integers(KW, KW + 9))
    N = int(rng.choice([1, 1, 2, 5]))
    s = (int(rng.integers(1, 3)), int(rng.integers(1, 3)))
    pad = (int(rng.integers(0, 3)), int(rng.integers(0, 3)))
    L = int(rng.choice([2, 4, 8, 16, 32, 32, 64, 128, 256]))
    gen = int(rng.choice([1, 1, 1, 2]))
    bc = int(rng.choice([0, 1, 1, 2, 3, -1, -2, 51200]))
    prog = [(7, 8, 1), (7, 8, 1), (7, 8, 1), (7, 2, 4), (7, 3, 2), (5, 1, 3)][rng.integers(0, 6)]
    cla, clw = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    if 32 * KH * KW * ((C + 31) // 32) >= 65536:
        C = 32
    return (N, C, H, W, O, KH, KW, s, pad, L, gen, bc, prog, cla, clw)


_rng = np.random.default_rng(2024)
CONV_CFGS = [_rand_conv_cfg(_rng) for _ in range(120)]


SNG_MODES = {"ballot": "1", "sliced": "2"}


@pytest.mark.parametrize("sng", sorted(SNG_MODES))
@pytest.mark.parametrize("idx", range(len(CONV_CFGS)))
def test_conv_fuzz(idx, sng, monkeypatch):
    import sc_extension_cuda
    monkeypatch.setenv("REXSC_SNG_MODE", SNG_MODES[sng])
    cfg = CONV_CFGS[idx]
    N, C, H, W, O, KH, KW, s, pad, L, gen, bc, prog, cla, clw = cfg
    print("conv fuzz", idx, sng, cfg, flush=True)
    rng = np.random.default_rng(1000 + idx)
    dens = min(1.0, 6.0 / (C * KH * KW) + 0.05)
    x = (rng.integers(0, L + 1, size=(N, C, H, W)) / L * (rng.uniform(size=(N, C, H, W)) < 3 * dens)).astype(np.float32)
    w = (rng.integers(-L, L + 1, size=(O, C, KH, KW)) / L * (rng.uniform(size=(O, C, KH, KW)) < 3 * dens)).astype(np.float32)
    xt = torch.from_numpy(x).cuda()
    wt = torch.from_numpy(w).cuda()
    if cla:
        xt = xt.contiguous(memory_format=torch.channels_last)
    if clw:
        wt = wt.contiguous(memory_format=torch.channels_last)
    # the memory order the op sees is decided by the reference's stride test, which size-1 dims can flip
    import _ops
    cla_eff, clw_eff = _ops.is_channels_last(xt), _ops.is_channels_last(wt)
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(xt, wt, L, -1, 16, pad, s, prog, bc, gen, True, False)
    opos, oneg = orc.conv2d_generic_general_split(x, w, L, -1, 16, pad, s, prog, bc, gen,
                                                  channels_last_activation=cla_eff, channels_last_weight=clw_eff)
    assert pos.shape == opos.shape
    assert np.array_equal(pos.cpu().numpy(), opos)
    assert np.array_equal(neg.cpu().numpy(), oneg)


@pytest.mark.parametrize("sng", sorted(SNG_MODES))
@pytest.mark.parametrize("cla", [False, True])
def test_conv_batch_chunks(cla, sng, monkeypatch):
    """Batches whose activation streams exceed the cap are processed in chunks (weight streams and the
    state table are made once): force a 1 MiB cap and compare with the oracle."""
    import sc_extension_cuda
    import _lib
    import ctypes
    monkeypatch.setenv("REXSC_SNG_MODE", SNG_MODES[sng])
    monkeypatch.setenv("REXSC_TUNE_ACT_CAP_MB", "1")
    N, C, H, W, O, L = 7, 70, 25, 23, 20, 32
    d = _lib.ConvDesc(N, C, H, W, O, 3, 3, 1, 1, 1, 1, L, -1, 1, 1, 7, 8, 1, int(cla), 0)
    info = (ctypes.c_int64 * 16)()
    _lib.check(_lib.lib().rexsc_conv2d_plan_info(ctypes.byref(d), info), "plan_info")
    assert 1 <= info[11] < N, "the cap should split this batch (n_chunk=%d)" % info[11]
    print("chunked conv", cla, sng, "n_chunk", info[11], flush=True)
    rng = np.random.default_rng(77)
    x = (rng.integers(0, L + 1, size=(N, C, H, W)) / L * (rng.uniform(size=(N, C, H, W)) < 0.2)).astype(np.float32)
    w = (rng.integers(-L, L + 1, size=(O, C, 3, 3)) / L * (rng.uniform(size=(O, C, 3, 3)) < 0.2)).astype(np.float32)
    xt = torch.from_numpy(x).cuda()
    if cla:
        xt = xt.contiguous(memory_format=torch.channels_last)
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(xt, torch.from_numpy(w).cuda(), L, -1, 16, (1, 1), (1, 1),
                                                                  (7, 8, 1), 1, 1, True, False)
    opos, oneg = orc.conv2d_generic_general_split(x, w, L, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1,
                                                  channels_last_activation=cla)
    assert np.array_equal(pos.cpu().numpy(), opos)
    assert np.array_equal(neg.cpu().numpy(), oneg)


def _rand_lin_cfg(rng):
    B = int(rng.choice([1, 3, 63, 64, 65, 130, 300]))
    C = int(rng.choice([1, 31, 32, 33, 100, 256, 257, 1000]))
    O = int(rng.choice([1, 15, 16, 17, 40, 100]))
    L = int(rng.choice([2, 8, 16, 32, 64, 128, 256]))
    gen = int(rng.choice([1, 1, 2, 3]))
    bc = int(rng.choice([0, 1, 2, 3, -1, -3, 51200]))
    prog = [(7, 8, 1), (7, 8, 1), (7, 2, 4), (6, 3, 1)][rng.integers(0, 4)]
    return (B, C, O, L, gen, bc, prog)


LIN_CFGS = [_rand_lin_cfg(_rng) for _ in range(60)]


@pytest.mark.parametrize("sng", sorted(SNG_MODES))
@pytest.mark.parametrize("idx", range(len(LIN_CFGS)))
def test_linear_fuzz(idx, sng, monkeypatch):
    import sc_extension
    monkeypatch.setenv("REXSC_SNG_MODE", SNG_MODES[sng])
    B, C, O, L, gen, bc, prog = LIN_CFGS[idx]
    print("linear fuzz", idx, sng, LIN_CFGS[idx], flush=True)
    rng = np.random.default_rng(5000 + idx)
    dens = 1.0 if bc > 100 else min(1.0, 8.0 / C + 0.05)
    x = (rng.integers(0, L + 1, size=(B, C)) / L * (rng.uniform(size=(B, C)) < 2 * dens)).astype(np.float32)
    w = (rng.integers(-L, L + 1, size=(O, C)) / L * (rng.uniform(size=(O, C)) < 2 * dens)).astype(np.float32)
    pos, neg = sc_extension.linear_generic_general(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda(), prog, L, -1,
                                                   bc, gen, True, False)
    opos, oneg = orc.linear_generic_general(x, w, prog, L, -1, bc, gen)
    assert np.array_equal(pos.cpu().numpy(), opos)
    assert np.array_equal(neg.cpu().numpy(), oneg)
