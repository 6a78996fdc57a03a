"""HIP path (through the C ABI of librexsc.so, via the drop-in extension modules) against the
golden vectors of the reference CPU extension and against the CPU oracle -- bit-exact."""
import json
import os

import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


class _Golden:
    """The fixtures written by the reference's compiled CPU extension: hand-picked cases (make_golden.py),
    seeded random configurations (make_golden_random.py) and operands off the quantisation grid
    (make_golden_offgrid.py), as one key space."""

    def __init__(self):
        self.files = [np.load(os.path.join(ROOT, "tests", "golden", f), allow_pickle=False)
                      for f in ("ref_cpu_ext.npz", "ref_cpu_ext_random.npz", "ref_cpu_ext_offgrid.npz")]
        self.meta = {"conv": [], "linear": [], "fixed": []}
        for f in self.files:
            m = json.loads(bytes(f["meta"]).decode())
            for kind in self.meta:
                self.meta[kind] += m[kind]

    def __getitem__(self, key):
        for f in self.files:
            if key in f.files:
                return f[key]
        raise KeyError(key)


_data = _Golden()
_meta = _data.meta


def _dev(a, channels_last=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to("cuda")
    if channels_last:
        t = t.contiguous(memory_format=torch.channels_last)
    return t


@pytest.mark.parametrize("case", _meta["conv"], ids=lambda c: c["name"])
def test_conv_golden(case):
    import sc_extension_cuda
    x, w, y = (_data["conv/%s/%s" % (case["name"], k)] for k in ("x", "w", "y"))
    xt = _dev(x, case["channels_last_activation"])
    wt = _dev(w, case["channels_last_weight"])
    print("conv golden", case["name"], flush=True)
    args = (xt, wt, case["bit_length"], case["lfsr_length"], 16, tuple(case["padding"]), tuple(case["stride"]),
            tuple(case["prog_load"]), case["bin_config"], case["gen_config"], True, False)
    diff = sc_extension_cuda.conv2d_generic_general_acc(*args)
    assert diff.dtype == torch.int16
    # the result follows the activation's memory order as the reference reads it off the strides
    # (sc_conv.cpp:326-331, 467-471; a one-channel tensor never counts as channels-last)
    st = xt.stride()
    if st[1] == 1 and st[1] * st[2] * st[3] != 1:
        assert diff.permute(0, 2, 3, 1).is_contiguous()
    else:
        assert diff.is_contiguous()
    assert np.array_equal(diff.cpu().numpy(), y)
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(*args)
    opos, oneg = orc.conv2d_generic_general_split(
        x, w, case["bit_length"], case["lfsr_length"], 16, case["padding"], case["stride"], case["prog_load"],
        case["bin_config"], case["gen_config"],
        channels_last_activation=case["channels_last_activation"], channels_last_weight=case["channels_last_weight"])
    assert np.array_equal(pos.cpu().numpy(), opos)
    assert np.array_equal(neg.cpu().numpy(), oneg)


@pytest.mark.parametrize("case", _meta["linear"], ids=lambda c: c["name"])
def test_linear_golden(case):
    import sc_extension
    n = case["name"]
    print("linear golden", n, flush=True)
    pos, neg = sc_extension.linear_generic_general(
        _dev(_data["linear/%s/x" % n]), _dev(_data["linear/%s/w" % n]), tuple(case["prog_load"]), case["bit_length"],
        case["lfsr_length"], case["bin_config"], case["gen_config"], True, False)
    assert pos.dtype == torch.int32
    assert np.array_equal(pos.cpu().numpy(), _data["linear/%s/pos" % n])
    assert np.array_equal(neg.cpu().numpy(), _data["linear/%s/neg" % n])


@pytest.mark.parametrize("case", _meta["fixed"], ids=lambda c: c["name"])
def test_fixed_golden(case):
    import fixed_extension_cuda
    n = case["name"]
    print("fixed golden", n, flush=True)
    out = fixed_extension_cuda.conv2d_saturate_acc(
        _dev(_data["fixed/%s/x" % n]), _dev(_data["fixed/%s/w" % n]), case["add_config"], case["precision_in"],
        case["precision_out"], tuple(case["padding"]), tuple(case["stride"]))
    assert out.dtype == torch.int32
    assert np.array_equal(out.cpu().numpy(), _data["fixed/%s/y" % n])


# ---- seeded random shapes against the oracle --------------------------------------------------
RANDOM_CONV = [
    # N, C, H, W, O, KH, KW, stride, padding, L, bin_config, gen, cl_act, cl_w
    (3, 64, 14, 14, 48, 3, 3, (1, 1), (1, 1), 32, 1, 1, False, False),   # ResNet-like, px=1
    (2, 64, 56, 56, 64, 3, 3, (1, 1), (1, 1), 32, 1, 1, True, False),    # layer1 shape, channels_last
    (2, 64, 56, 56, 128, 3, 3, (2, 2), (1, 1), 32, 1, 1, True, False),   # stride-2 3x3
    (2, 64, 56, 56, 128, 1, 1, (2, 2), (0, 0), 32, 1, 1, True, False),   # 1x1 downsample
    (1, 512, 7, 7, 512, 3, 3, (1, 1), (1, 1), 32, 1, 1, True, False),    # layer4 shape: slot splits
    (2, 256, 14, 14, 256, 3, 3, (1, 1), (1, 1), 32, 1, 1, False, False),
    (4, 32, 32, 32, 64, 3, 3, (1, 1), (1, 1), 32, 0, 1, False, False),   # config-1 shape, OR-1
    (2, 3, 32, 32, 32, 3, 3, (1, 1), (1, 1), 64, 2, 1, False, False),    # TinyConv first layer, OR-3 L=64
    (2, 32, 16, 16, 64, 5, 5, (1, 1), (2, 2), 64, 2, 1, False, False),   # 5x5
    (1, 100, 9, 11, 33, 3, 3, (1, 2), (0, 1), 128, 3, 1, False, True),   # odd everything
    (1, 24, 10, 10, 20, 2, 2, (1, 1), (0, 0), 32, 1, 1, False, False),   # no tuned instance -> generic kernel
    (1, 160, 8, 8, 24, 7, 7, (1, 1), (3, 3), 32, 1, 2, True, True),      # 7x7, and_2 generator
]


@pytest.mark.parametrize("cfg", RANDOM_CONV, ids=lambda c: "x".join(str(v) for v in c[:7]) + "_L%d_b%d" % (c[9], c[10]))
def test_conv_random_vs_oracle(cfg):
    import sc_extension_cuda
    N, C, H, W, O, KH, KW, stride, pad, L, bc, gen, cla, clw = cfg
    print("conv random", cfg, flush=True)
    rng = np.random.default_rng(hash(cfg) & 0xFFFF)
    dens = min(1.0, 24.0 / (C * KH * KW) + 0.02)
    x = (rng.integers(0, L, size=(N, C, H, W)) / L * (rng.uniform(size=(N, C, H, W)) < 4 * dens)).astype(np.float32)
    w = (rng.integers(-L + 1, L, size=(O, C, KH, KW)) / L * (rng.uniform(size=(O, C, KH, KW)) < 4 * dens)).astype(np.float32)
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(
        _dev(x, cla), _dev(w, clw), L, -1, 16, pad, stride, (7, 8, 1), bc, gen, True, False)
    opos, oneg = orc.conv2d_generic_general_split(x, w, L, -1, 16, pad, stride, (7, 8, 1), bc, gen,
                                                  channels_last_activation=cla, channels_last_weight=clw)
    assert pos.shape == opos.shape
    assert opos.max() > 0 and (opos != oneg).any()
    assert np.array_equal(pos.cpu().numpy(), opos)
    assert np.array_equal(neg.cpu().numpy(), oneg)


RANDOM_LINEAR = [
    (256, 4096, 64, 64, 1, 1),     # config-2 K and batch, fewer outputs
    (7, 1000, 50, 32, 0, 1),
    (300, 96, 40, 128, 3, 1),
    (16, 2048, 24, 256, 51200, 1),  # full_bin with sums above 65535: wide accumulators
    (5, 64, 9, 32, -2, 2),          # nth-bit rule, and_2 slot interleave
]


@pytest.mark.parametrize("cfg", RANDOM_LINEAR, ids=lambda c: "_".join(str(v) for v in c))
def test_linear_random_vs_oracle(cfg):
    import sc_extension
    B, C, O, L, bc, gen = cfg
    print("linear random", cfg, flush=True)
    rng = np.random.default_rng(hash(cfg) & 0xFFFF)
    dens = 1.0 if bc > 100 else min(1.0, 40.0 / C)
    x = (rng.integers(0, L, size=(B, C)) / L * (rng.uniform(size=(B, C)) < dens)).astype(np.float32)
    w = (rng.integers(-L + 1, L, size=(O, C)) / L * (rng.uniform(size=(O, C)) < dens)).astype(np.float32)
    pos, neg = sc_extension.linear_generic_general(_dev(x), _dev(w), (7, 8, 1), L, -1, bc, gen, True, False)
    opos, oneg = orc.linear_generic_general(x, w, (7, 8, 1), L, -1, bc, gen)
    if bc > 100:
        assert opos.max() > 65535
    assert np.array_equal(pos.cpu().numpy(), opos)
    assert np.array_equal(neg.cpu().numpy(), oneg)


def test_conv_rejects_bad_arguments():
    import sc_extension_cuda
    x = torch.rand(1, 8, 6, 6, device="cuda")
    w = torch.rand(4, 8, 3, 3, device="cuda")
    with pytest.raises(RuntimeError, match="stream length"):
        sc_extension_cuda.conv2d_generic_general_split_acc(x, w, 48, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1, True, False)
    with pytest.raises(RuntimeError, match="gen_config"):
        sc_extension_cuda.conv2d_generic_general_split_acc(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 3, True, False)
    with pytest.raises(RuntimeError, match="equal C"):
        sc_extension_cuda.conv2d_generic_general_split_acc(x, w[:, :4], 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1,
                                                           True, False)
    with pytest.raises(RuntimeError, match="HIP device"):
        sc_extension_cuda.conv2d_generic_general_split_acc(x.cpu(), w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1,
                                                           True, False)


def test_empty_batch_gives_empty_results():
    """N = 0 (B = 0) is not an error: the ops return empty tensors of the right shape, dtype and device."""
    import fixed_extension_cuda
    import sc_extension
    import sc_extension_cuda
    import sc_functional as uf
    w = torch.rand(4, 8, 3, 3, device="cuda")
    x = torch.rand(0, 8, 6, 6, device="cuda").contiguous(memory_format=torch.channels_last)
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(x, w, 32, -1, 16, (1, 1), (2, 2), (7, 8, 1), 1, 1,
                                                                  True, False)
    assert pos.shape == neg.shape == (0, 4, 3, 3) and pos.dtype == torch.int16 and pos.is_cuda
    assert sc_extension_cuda.conv2d_generic_general_acc(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1, True,
                                                        False).shape == (0, 4, 6, 6)
    lp, ln = sc_extension.linear_generic_general(torch.rand(0, 40, device="cuda"), torch.rand(5, 40, device="cuda"),
                                                 (7, 8, 1), 32, -1, 1, 1, True, False)
    assert lp.shape == ln.shape == (0, 5) and lp.dtype == torch.int32
    y = fixed_extension_cuda.conv2d_saturate_acc(x, w, 0, 5, 24, (1, 1), (1, 1))
    assert y.shape == (0, 4, 6, 6) and y.dtype == torch.int32
    for sync in (1, 3):
        out = uf.conv2d_generic(x.requires_grad_(False), w.clone().requires_grad_(True), (1, 1), (1, 1), bit_length=32,
                                generator="lfsr", forward="or_2", sync=sync, order=5)
        assert out.shape == (0, 4, 6, 6)
    assert uf.quantize(x, 7).shape == x.shape


RANDOM_FIXED = [
    # N, C, H, W, O, KH, KW, stride, padding, add_config, pin, pout
    (2, 64, 14, 14, 64, 3, 3, (1, 1), (1, 1), 0, 5, 24),     # int8 MFMA closed form, ResNet-like
    (1, 20, 9, 11, 70, 3, 3, (2, 1), (1, 0), 0, 5, 24),      # odd channels / outputs / strides
    (3, 8, 12, 12, 130, 1, 1, (1, 1), (0, 0), 0, 6, 24),     # 1x1, three output tiles
    (1, 33, 8, 8, 5, 5, 5, (1, 1), (2, 2), 0, 7, 31),        # 7-bit operands, 5x5
    (2, 128, 28, 28, 128, 3, 3, (1, 1), (1, 1), 0, 5, 24),   # config-4 stage 2 at batch 2
    (1, 512, 7, 7, 512, 3, 3, (1, 1), (1, 1), 0, 5, 24),     # config-4 stage 4 at batch 1
    (1, 16, 8, 8, 8, 3, 3, (1, 1), (1, 1), 0, 5, 8, 0.1),    # d > 0: VALU closed form with rounding (sparse operands)
    (1, 64, 6, 6, 4, 3, 3, (1, 1), (1, 1), 0, 6, 12, 0.06),  # clamp fires for some outputs: VALU closed form
    (1, 6, 7, 7, 5, 3, 3, (1, 1), (1, 1), 1, 5, 24),         # OR adder, sequential
    (1, 7, 6, 6, 4, 3, 3, (1, 1), (1, 1), 3, 5, 24),         # pairwise OR2 adder, odd product count
]


@pytest.mark.parametrize("cfg", RANDOM_FIXED, ids=lambda c: "_".join(str(v) for v in c).replace(" ", ""))
def test_fixed_random_vs_oracle(cfg):
    import fixed_extension_cuda
    N, C, H, W, O, KH, KW, stride, pad, add, pin, pout = cfg[:12]
    dens = cfg[12] if len(cfg) > 12 else 1.0
    print("fixed random", cfg, flush=True)
    rng = np.random.default_rng(hash(cfg) & 0xFFFF)
    P2 = 1 << pin
    x = (rng.integers(0, 2 * P2, size=(N, C, H, W)) / (2 * P2)).astype(np.float32)   # half-grid: exercises round()
    w = (rng.integers(-2 * P2 + 1, 2 * P2, size=(O, C, KH, KW)) / (2 * P2)).astype(np.float32)
    x *= rng.uniform(size=x.shape) < dens
    w *= rng.uniform(size=w.shape) < dens
    out = fixed_extension_cuda.conv2d_saturate_acc(_dev(x), _dev(w), add, pin, pout, pad, stride)
    want = orc.conv2d_saturate(x, w, add, pin, pout, pad, stride)
    assert out.shape == want.shape and np.abs(want).max() > 0
    assert np.array_equal(out.cpu().numpy(), want)


FUSED_FIXED = [
    # N, C, H, W, O: 3x3 / stride 1 / padding 1 shapes of the single-pass MFMA kernel, ragged in every direction
    (5, 20, 7, 7, 70),      # several images per tile, batch not a multiple of the group, ragged channels and outputs
    (3, 40, 30, 30, 64),    # row tiles that do not divide the plane
    (2, 33, 57, 57, 10),    # wide rows: four rows per tile, three rounds of tile entries per thread
    (1, 16, 13, 90, 64),    # two rows per tile
    (7, 96, 14, 14, 192),   # one image per tile, three output tiles
    (70, 8, 5, 9, 8),       # small planes, one image per tile
    (600, 8, 5, 9, 8),      # small planes, two images per tile
    (2, 12, 20, 20, 5),     # few channels, few outputs: all weights stay in LDS, channel tail inside a half
    (2, 64, 24, 24, 64),    # exactly one output tile and two channel pairs
    (3, 40, 12, 36, 70),    # rows of a multiple of four pixels (16-byte loads), ragged row tiles, two output tiles
    (2, 33, 10, 16, 64),    # 16-byte loads with a channel tail of one
    (600, 8, 4, 8, 8),      # small planes of a multiple of four pixels per row: two images per tile with 16-byte loads
    (3, 130, 14, 14, 70),   # five channel groups over four waves (2, 2, 1, 0), channel tail of two, ragged row tiles
    (2, 256, 14, 14, 256),  # config-4 stage 3 at batch 2
]


@pytest.mark.parametrize("path", ["planner", "single_pass", "single_pass_tiled_weights", "two_pass", "split_reduction"])
@pytest.mark.parametrize("cfg", FUSED_FIXED, ids=lambda c: "_".join(str(v) for v in c))
def test_fixed_fused_shapes_and_out_of_range_operands(cfg, path, monkeypatch):
    """Activations below zero, above one, at rounding ties and near-ties; weights likewise.  Once with the
    library's own choice between the single-pass and the two-pass MFMA path, once with each forced (the single
    pass also without its weights-in-LDS variant, and the single pass whose waves split the reduction wherever its
    tiling exists -- rows of at most 64 pixels; other shapes fall through to the two passes)."""
    import fixed_extension_cuda
    N, C, H, W, O = cfg
    print("fixed fused", cfg, path, flush=True)
    if path != "planner":
        monkeypatch.setenv("REXSC_TUNE_FIXED_FUSED", {"two_pass": "0", "split_reduction": "3"}.get(path, "2"))
    if path == "single_pass_tiled_weights":   # never the variant that keeps all weights in LDS
        monkeypatch.setenv("REXSC_TUNE_FIXED_WS", "0")
    rng = np.random.default_rng(sum(cfg))
    x = (rng.integers(-8, 80, size=(N, C, H, W)) / 64).astype(np.float32)            # [-1/8, 5/4) on the half grid
    x += (rng.integers(-1, 2, size=x.shape) * 2.0 ** -20).astype(np.float32)         # just below / at / above
    w = (rng.integers(-80, 80, size=(O, C, 3, 3)) / 64).astype(np.float32)
    w += (rng.integers(-1, 2, size=w.shape) * 2.0 ** -20).astype(np.float32)
    out = fixed_extension_cuda.conv2d_saturate_acc(_dev(x), _dev(w), 0, 5, 24, (1, 1), (1, 1))
    want = orc.conv2d_saturate(x, w, 0, 5, 24, (1, 1), (1, 1))
    assert out.shape == want.shape and np.abs(want).max() > 0
    assert np.array_equal(out.cpu().numpy(), want)


# ---- REXSC_XNOR_MODE=cuda_ref: the generators of the reference's CUDA conv kernels ---------------------------
XNOR_CONV = [
    # N, C, H, W, O, K, stride, L, lfsr_length, bin_config, gen, cl_act, cl_w
    (2, 64, 14, 14, 48, 3, 1, 32, -1, 1, 1, True, False),
    (2, 64, 56, 56, 64, 3, 1, 32, -1, 1, 1, True, False),    # ResNet-18 layer1 shape: bit-sliced generator, shift table
    (1, 33, 9, 11, 20, 3, 2, 64, -1, 2, 1, False, True),
    (2, 3, 32, 32, 32, 3, 1, 64, -1, 2, 1, False, False),
    (1, 40, 8, 8, 24, 5, 1, 16, -1, 0, 2, False, False),     # and_2 with the XNOR LFSR (no "_acc" variant on CUDA)
    (1, 16, 6, 6, 8, 1, 1, 32, 7, 3, 2, True, False),
    (1, 8, 5, 5, 4, 3, 1, 8, -1, 1, 1, False, False),
    (1, 512, 7, 7, 64, 3, 1, 128, -1, 1, 1, True, False),
]


@pytest.mark.parametrize("sng_mode", ["0", "1", "2"])
@pytest.mark.parametrize("cfg", XNOR_CONV, ids=lambda c: "_".join(str(v) for v in c))
def test_conv_cuda_xnor_mode_vs_oracle(cfg, sng_mode, monkeypatch):
    import sc_extension
    import sc_extension_cuda
    N, C, H, W, O, K, stride, L, lfsr, bc, gen, cla, clw = cfg
    print("conv cuda_xnor", cfg, "sng mode", sng_mode, flush=True)
    monkeypatch.setenv("REXSC_XNOR_MODE", "cuda_ref")
    monkeypatch.setenv("REXSC_SNG_MODE", sng_mode)
    rng = np.random.default_rng(hash(cfg) & 0xFFFF)
    S = (1 << lfsr) if lfsr > 0 else L
    dens = min(1.0, 96.0 / (C * K * K) + 0.02)
    x = (rng.integers(0, S, size=(N, C, H, W)) / S * (rng.uniform(size=(N, C, H, W)) < dens)).astype(np.float32)
    w = (rng.integers(-S + 1, S, size=(O, C, K, K)) / S * (rng.uniform(size=(O, C, K, K)) < dens)).astype(np.float32)
    pad = (K // 2, K // 2)
    args = (_dev(x, cla), _dev(w, clw), L, lfsr, 16, pad, (stride, stride), (7, 8, 1), bc, gen)
    pos, neg = sc_extension_cuda.conv2d_generic_general_split_acc(*args, True, False)
    opos, oneg = orc.conv2d_generic_general_split(x, w, L, lfsr, 16, pad, (stride, stride), (7, 8, 1), bc, gen,
                                                  channels_last_activation=cla, channels_last_weight=clw, cuda_xnor=True)
    assert opos.max() > 0
    assert np.array_equal(pos.cpu().numpy(), opos) and np.array_equal(neg.cpu().numpy(), oneg)
    # xnor=False in the same mode, and the CPU-named module in any mode, keep the CPU extension's generator
    cpos, cneg = orc.conv2d_generic_general_split(x, w, L, lfsr, 16, pad, (stride, stride), (7, 8, 1), bc, gen,
                                                  channels_last_activation=cla, channels_last_weight=clw)
    assert not np.array_equal(cpos, opos)
    p0, n0 = sc_extension_cuda.conv2d_generic_general_split_acc(*args, False, False)
    assert np.array_equal(p0.cpu().numpy(), cpos) and np.array_equal(n0.cpu().numpy(), cneg)
    d0 = sc_extension.conv2d_generic_general(*args, True, False)
    assert np.array_equal(d0.cpu().numpy(), (cpos.astype(np.int32) - cneg).astype(np.int16))


def test_cuda_xnor_mode_rejections_and_default(monkeypatch):
    import _ops
    import sc_extension_cuda
    x = torch.rand(1, 8, 6, 6, device="cuda")
    w = torch.rand(4, 8, 3, 3, device="cuda")
    monkeypatch.delenv("REXSC_XNOR_MODE", raising=False)
    assert _ops.xnor_mode() == "cpu_oracle"
    monkeypatch.setenv("REXSC_XNOR_MODE", "cuda_ref")
    with pytest.raises(RuntimeError, match="8-bit"):
        sc_extension_cuda.conv2d_generic_general_split_acc(x, w, 256, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1, True, False)
    monkeypatch.setenv("REXSC_XNOR_MODE", "something")
    with pytest.raises(RuntimeError, match="REXSC_XNOR_MODE"):
        sc_extension_cuda.conv2d_generic_general_split_acc(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1, True, False)
