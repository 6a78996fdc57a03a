"""conv2d_generic with the two surrogate convolutions merged (polarity-pair layout) against the
two-convolution path it replaces: forward values, gradients, noise stream, layouts, fallbacks."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _operands(seed, N, C, H, W, O, K, L=32, dens=0.4):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randint(0, L, (N, C, H, W), generator=g).float() / L) * (torch.rand(N, C, H, W, generator=g) < dens)
    w = (torch.randint(-L + 1, L, (O, C, K, K), generator=g).float() / L) * (torch.rand(O, C, K, K, generator=g) < dens)
    return x, w


def _run(monkeypatch, merged, x, w, pad, stride, forward, sync, channels_last, need_x=True, seed=11, bias=None,
         std=None):
    import sc_functional as uf
    monkeypatch.setenv("REXSC_MERGED_SURROGATE", "1" if merged else "0")
    xt = x.cuda()
    if channels_last:
        xt = xt.contiguous(memory_format=torch.channels_last)
    xt.requires_grad_(need_x)
    wt = w.cuda().requires_grad_(True)
    torch.manual_seed(seed)
    kw = dict(bit_length=32, generator="lfsr", forward=forward, sync=sync, order=5)
    if bias is not None:
        kw.update(bias_coef=bias.cuda(), std_coef=std.cuda())
    out = uf.conv2d_generic(xt, wt, pad, stride, **kw)
    g = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).cuda()
    out.backward(g)
    return out.detach().cpu(), (xt.grad.cpu() if need_x else None), wt.grad.cpu()


def _close(a, b, what):
    scale = float(b.abs().max()) + 1e-30
    err = float((a - b).abs().max())
    assert err <= 1e-5 * scale, "%s: max error %g against scale %g" % (what, err, scale)


CASES = [
    # N, C, H, W, O, K, pad, stride, channels_last
    (2, 16, 10, 10, 12, 3, (1, 1), (1, 1), False),
    (2, 16, 10, 10, 12, 3, (1, 1), (1, 1), True),
    (3, 24, 9, 7, 8, 3, (1, 1), (2, 2), True),
    (2, 8, 8, 8, 6, 1, (0, 0), (1, 1), False),     # O % 4 != 0, O*Ho*Wo % 4 == 0: NCHW pair layout
    (2, 8, 8, 8, 6, 1, (0, 0), (1, 1), True),      # channels-last sums re-laid out as NCHW
    (1, 40, 12, 12, 20, 5, (2, 2), (1, 1), True),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("forward", ["or_2", "or_3", "full_or"])
def test_sync1_merged_equals_two_convolutions(case, forward, monkeypatch):
    N, C, H, W, O, K, pad, stride, cl = case
    print("merged sync1", case, forward, flush=True)
    x, w = _operands(21, N, C, H, W, O, K)
    ya, gxa, gwa = _run(monkeypatch, True, x, w, pad, stride, forward, 1, cl)
    yb, gxb, gwb = _run(monkeypatch, False, x, w, pad, stride, forward, 1, cl)
    assert torch.equal(ya, yb)   # the SC result, exactly
    _close(gxa, gxb, "grad x")
    _close(gwa, gwb, "grad w")


@pytest.mark.parametrize("case", CASES[:4])
def test_sync3_merged_equals_two_convolutions(case, monkeypatch):
    N, C, H, W, O, K, pad, stride, cl = case
    print("merged sync3", case, flush=True)
    x, w = _operands(22, N, C, H, W, O, K)
    bias = torch.tensor([0.01, -0.02, 0.005, 0.001, 0, 0])
    std = torch.tensor([0.02, 0.01, 0, 0, 0, 0])
    ya, gxa, gwa = _run(monkeypatch, True, x, w, pad, stride, "or_2", 3, cl, bias=bias, std=std)
    yb, gxb, gwb = _run(monkeypatch, False, x, w, pad, stride, "or_2", 3, cl, bias=bias, std=std)
    # same seed, same element order: the same noise draws, so the values agree to float rounding
    _close(ya, yb, "forward")
    _close(gxa, gxb, "grad x")
    _close(gwa, gwb, "grad w")


def test_first_layer_needs_no_activation_gradient(monkeypatch):
    x, w = _operands(23, 2, 16, 8, 8, 8, 3)
    ya, gxa, gwa = _run(monkeypatch, True, x, w, (1, 1), (1, 1), "or_2", 1, True, need_x=False)
    yb, gxb, gwb = _run(monkeypatch, False, x, w, (1, 1), (1, 1), "or_2", 1, True, need_x=False)
    assert gxa is None and torch.equal(ya, yb)
    _close(gwa, gwb, "grad w")


def test_shapes_without_a_vector_view_fall_back(monkeypatch):
    # O = 5 and 5*3*3 = 45 outputs per image: no inner % 4 == 0 view in either layout
    import sc_functional as uf
    x, w = _operands(24, 2, 8, 3, 3, 5, 1)
    calls = []
    orig = uf.Merged_Surrogate_Conv.apply
    monkeypatch.setattr(uf.Merged_Surrogate_Conv, "apply", lambda *a: calls.append(1) or orig(*a))
    ya, gxa, gwa = _run(monkeypatch, True, x, w, (0, 0), (1, 1), "or_2", 1, False)
    assert not calls
    x2, w2 = _operands(24, 2, 8, 3, 3, 8, 1)
    _run(monkeypatch, True, x2, w2, (0, 0), (1, 1), "or_2", 1, False)
    assert calls


def test_weight_split_and_merge_follow_clamp(monkeypatch):
    import _ops
    w = torch.tensor([-200.0, -100.0, -0.5, 0.0, 0.25, 100.0, 150.0, float("nan")]).reshape(8, 1, 1, 1).cuda()
    w2 = _ops.split_weight(w)
    want = torch.cat([w.clamp(0, 100), -(w.clamp(-100, 0))])
    assert torch.equal(torch.nan_to_num(w2, nan=7.0), torch.nan_to_num(want, nan=7.0))
    wr = w.clone().requires_grad_(True)
    d2 = torch.arange(1.0, 17.0).reshape(16, 1, 1, 1).cuda()
    torch.cat([wr.clamp(0, 100), -(wr.clamp(-100, 0))]).backward(d2)
    assert torch.equal(_ops.merge_weight_grad(d2, w), wr.grad)


@pytest.mark.parametrize("w_cl", [False, True])
@pytest.mark.parametrize("out_cl", [False, True])
def test_weight_split_and_merge_in_both_memory_orders(w_cl, out_cl):
    import _ops
    g = torch.Generator().manual_seed(9)
    w = (torch.rand(6, 5, 3, 2, generator=g) * 2 - 1).cuda()
    if w_cl:
        w = w.contiguous(memory_format=torch.channels_last)
    w2 = _ops.split_weight(w, channels_last=out_cl)
    assert w2.is_contiguous(memory_format=torch.channels_last if out_cl else torch.contiguous_format)
    assert torch.equal(w2, torch.cat([w.clamp(0, 100), -(w.clamp(-100, 0))]))
    d2 = torch.randn(12, 5, 3, 2, generator=g).cuda()
    if out_cl:
        d2 = d2.contiguous(memory_format=torch.channels_last)
    wr = w.clone().requires_grad_(True)
    torch.cat([wr.clamp(0, 100), -(wr.clamp(-100, 0))]).backward(d2)
    got = _ops.merge_weight_grad(d2, w)
    assert got.stride() == w.stride() and torch.equal(got, wr.grad)


def test_counts_to_float_odd_length():
    import _ops
    g = torch.Generator().manual_seed(3)
    pos = torch.randint(-32768, 32767, (3, 5, 7, 3), generator=g, dtype=torch.int16).cuda()
    neg = torch.randint(-32768, 32767, (3, 5, 7, 3), generator=g, dtype=torch.int16).cuda()
    for L in (32, 48):
        assert torch.equal(_ops.sc_counts_to_float(pos, neg, L), pos.float() / L - neg.float() / L)


def test_inference_skips_the_surrogate(monkeypatch):
    """Without gradients sync 1 returns the SC result and never runs the float convolution."""
    import sc_functional as uf
    import torch.nn.functional as F
    x, w = _operands(25, 2, 16, 8, 8, 8, 3)
    xt, wt = x.cuda(), w.cuda().requires_grad_(True)
    want = uf.conv2d_generic(xt, wt, (1, 1), (1, 1), bit_length=32, generator="lfsr", forward="or_2", sync=1).detach()
    calls = []
    orig = F.conv2d
    monkeypatch.setattr(uf.F, "conv2d", lambda *a, **k: calls.append(1) or orig(*a, **k))
    with torch.no_grad():
        got = uf.conv2d_generic(xt, wt, (1, 1), (1, 1), bit_length=32, generator="lfsr", forward="or_2", sync=1)
    assert torch.equal(got, want) and not calls and not got.requires_grad


def test_side_stream_overlap_changes_nothing(monkeypatch):
    """The SC forward on a second stream (default) and on the caller's stream give the same step."""
    x, w = _operands(26, 4, 32, 14, 14, 32, 3)
    monkeypatch.setenv("REXSC_OVERLAP_SURROGATE", "1")
    ya, gxa, gwa = _run(monkeypatch, True, x, w, (1, 1), (1, 1), "or_2", 1, True)
    monkeypatch.setenv("REXSC_OVERLAP_SURROGATE", "0")
    yb, gxb, gwb = _run(monkeypatch, True, x, w, (1, 1), (1, 1), "or_2", 1, True)
    assert torch.equal(ya, yb)
    _close(gxa, gxb, "grad x")   # MIOpen's gradient kernels accumulate with atomics: not bit-reproducible
    _close(gwa, gwb, "grad w")


@pytest.mark.parametrize("forward", ["or_2", "or_1", "full_or"])
def test_linear_merged_equals_two_gemms(forward, monkeypatch):
    import sc_functional as uf
    g = torch.Generator().manual_seed(31)
    L = 64
    x = torch.randint(0, L, (37, 200), generator=g).float() / L
    w = torch.randint(-L + 1, L, (24, 200), generator=g).float() / L
    gout = torch.randn(37, 24, generator=g).cuda()
    res = []
    for merged in ("1", "0"):
        monkeypatch.setenv("REXSC_MERGED_SURROGATE", merged)
        xt, wt = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
        y = uf.linear_generic_sc(xt, wt, bit_length=L, forward=forward, generator="lfsr", sync=1)
        y.backward(gout)
        res.append((y.detach().cpu(), xt.grad.cpu(), wt.grad.cpu()))
    assert torch.equal(res[0][0], res[1][0])
    _close(res[0][1], res[1][1], "grad x")
    _close(res[0][2], res[1][2], "grad w")


@pytest.mark.parametrize("cl", [False, True])
def test_sync2_merged_equals_two_convolutions(cl, monkeypatch):
    """Calibration step: same fitted polynomials, same gradients; the forward values differ only by the
    noise realisation (another generator), so their difference is zero-mean with the fitted spread."""
    import sc_functional as uf
    x, w = _operands(27, 4, 32, 16, 16, 32, 3, dens=0.3)
    res = []
    for merged in ("1", "0"):
        monkeypatch.setenv("REXSC_MERGED_SURROGATE", merged)
        xt = x.cuda()
        if cl:
            xt = xt.contiguous(memory_format=torch.channels_last)
        xt.requires_grad_(True)
        wt = w.cuda().requires_grad_(True)
        bias, std = torch.zeros(6, device="cuda"), torch.zeros(6, device="cuda")
        torch.manual_seed(3)
        out, b2, s2 = uf.conv2d_generic(xt, wt, (1, 1), (1, 1), bit_length=32, generator="lfsr", forward="or_2", sync=2,
                                        order=5, bias_coef=bias, std_coef=std)
        assert b2 is bias and s2 is std and std.abs().sum() > 0   # updated in place (the bias fit may be suppressed)
        g = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).cuda()
        out.backward(g)
        res.append((out.detach().cpu().double(), xt.grad.cpu(), wt.grad.cpu(), bias.cpu(), std.cpu()))
    (ya, gxa, gwa, ba, sa), (yb, gxb, gwb, bb, sb) = res
    xs = torch.linspace(0, 1.5, 16)
    poly = lambda c: sum(float(c[i]) * xs ** i for i in range(6))
    assert torch.allclose(poly(ba), poly(bb), atol=2e-4) and torch.allclose(poly(sa), poly(sb), atol=2e-4)
    _close(gxa, gxb, "grad x")
    _close(gwa, gwb, "grad w")
    d = ya - yb
    spread = float(d.std())
    assert 0 < spread < 0.5 and abs(float(d.mean())) < 6 * spread / d.numel() ** 0.5


def _run_autocast(monkeypatch, merged, lowp, x, w, pad, stride, forward, sync, channels_last, half_input, bias=None,
                  std=None):
    """conv2d_generic inside an autocast region (the reference's reduced-precision step, utils_own.py:127-131)."""
    import sc_functional as uf
    monkeypatch.setenv("REXSC_MERGED_SURROGATE", "1" if merged else "0")
    xt = x.cuda()
    if half_input:  # what a layer sees behind a reduced-precision convolution and a ReLU
        xt = xt.to(lowp)
    if channels_last:
        xt = xt.contiguous(memory_format=torch.channels_last)
    xt.requires_grad_(True)
    wt = w.cuda().requires_grad_(True)
    torch.manual_seed(11)
    kw = dict(bit_length=32, generator="lfsr", forward=forward, sync=sync, order=5)
    if bias is not None:
        kw.update(bias_coef=bias.cuda(), std_coef=std.cuda())
    with torch.autocast("cuda", dtype=lowp):
        out = uf.conv2d_generic(xt, wt, pad, stride, **kw)
    g = torch.randn(out.shape, generator=torch.Generator().manual_seed(5)).cuda().to(out.dtype)
    out.backward(g)
    assert xt.grad.dtype == xt.dtype and wt.grad.dtype == torch.float32
    return out.detach(), xt.grad.float().cpu(), wt.grad.cpu()


def _close_lowp(a, b, what, tol):
    scale = float(b.abs().max()) + 1e-30
    err = float((a - b).abs().max())
    assert err <= tol * scale, "%s: max error %g against scale %g" % (what, err, scale)


@pytest.mark.parametrize("case", [CASES[1], CASES[2], CASES[3]])
@pytest.mark.parametrize("half_input", [False, True])
def test_merged_path_inside_a_float16_autocast_region(case, half_input, monkeypatch):
    """Inside an autocast region the merged path runs its convolutions in float16, as the two-convolution path does
    there; the SC value is the same number and the gradients agree to float16 rounding (both paths round the sums and
    the convolutions' results to float16; they differ in where the two polarities' data gradients are added)."""
    N, C, H, W, O, K, pad, stride, cl = case
    print("merged autocast", case, half_input, flush=True)
    x, w = _operands(31, N, C, H, W, O, K)
    import sc_functional as uf
    calls = []
    orig = uf.Merged_Surrogate_Conv.apply
    monkeypatch.setattr(uf.Merged_Surrogate_Conv, "apply", lambda *a: calls.append(1) or orig(*a))
    ya, gxa, gwa = _run_autocast(monkeypatch, True, torch.float16, x, w, pad, stride, "or_2", 1, cl, half_input)
    assert calls, "the merged path was not taken inside the autocast region"
    yb, gxb, gwb = _run_autocast(monkeypatch, False, torch.float16, x, w, pad, stride, "or_2", 1, cl, half_input)
    assert ya.dtype == torch.float16 and yb.dtype == torch.float16
    assert torch.equal(ya, yb)  # the SC result: k / 32, exact in float16
    _close_lowp(gxa, gxb, "grad x", 4e-3)
    _close_lowp(gwa, gwb, "grad w", 4e-3)
    # and against the float32 run of the same layer: float16 rounding of sums and gradients only
    yc, gxc, gwc = _run(monkeypatch, True, x, w, pad, stride, "or_2", 1, cl)
    assert torch.equal(ya.float().cpu(), yc)
    _close_lowp(gxa, gxc, "grad x against float32", 1e-2)
    _close_lowp(gwa, gwc, "grad w against float32", 1e-2)


@pytest.mark.parametrize("sync", [3, 2])
def test_merged_path_autocast_error_injection_and_calibration(sync, monkeypatch):
    N, C, H, W, O, K, pad, stride, cl = CASES[1]
    x, w = _operands(32, N, C, H, W, O, K)
    bias = torch.tensor([0.01, -0.02, 0.005, 0.001, 0, 0])
    std = torch.zeros(6)  # no noise: the two paths index their noise streams differently per polarity tensor
    import sc_functional as uf
    if sync == 3:
        ya, gxa, gwa = _run_autocast(monkeypatch, True, torch.float16, x, w, pad, stride, "or_2", 3, cl, True, bias, std)
        yb, gxb, gwb = _run_autocast(monkeypatch, False, torch.float16, x, w, pad, stride, "or_2", 3, cl, True, bias, std)
        _close_lowp(ya.float().cpu(), yb.float().cpu(), "forward", 4e-3)
        _close_lowp(gxa, gxb, "grad x", 4e-3)
        _close_lowp(gwa, gwb, "grad w", 4e-3)
        return
    monkeypatch.setenv("REXSC_MERGED_SURROGATE", "1")
    xt = x.cuda().half().contiguous(memory_format=torch.channels_last).requires_grad_(True)
    wt = w.cuda().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.float16):
        out, b, s = uf.conv2d_generic(xt, wt, pad, stride, bit_length=32, generator="lfsr", forward="or_2", sync=2, order=5)
    out.float().sum().backward()
    assert out.dtype == torch.float16 and torch.isfinite(out).all()
    assert torch.isfinite(b).all() and torch.isfinite(s).all() and s.abs().sum() > 0
    assert torch.isfinite(xt.grad).all() and torch.isfinite(wt.grad).all()


def test_merged_path_inside_a_bfloat16_autocast_region(monkeypatch):
    N, C, H, W, O, K, pad, stride, cl = CASES[1]
    x, w = _operands(33, N, C, H, W, O, K)
    ya, gxa, gwa = _run_autocast(monkeypatch, True, torch.bfloat16, x, w, pad, stride, "or_2", 1, cl, True)
    yc, gxc, gwc = _run(monkeypatch, True, x, w, pad, stride, "or_2", 1, cl)
    assert ya.dtype == torch.float16  # the reference returns float16 inside any autocast region (utils_functional.py:1148-1150)
    assert torch.equal(ya.float().cpu(), yc)
    _close_lowp(gxa, gxc, "grad x against float32", 4e-2)
    _close_lowp(gwa, gwc, "grad w against float32", 4e-2)


@pytest.mark.parametrize("or_n", [1, 2, 3, 4])
@pytest.mark.parametrize("cl", [False, True])
def test_pair_backward_on_float16_tensors_equals_widen_compute_round(or_n, cl):
    """rexsc_orn_pair_backward_f16 (all three tensors binary16) = widen, rexsc_orn_pair_backward, round: bit for bit."""
    import _ops
    g = torch.Generator().manual_seed(40 + or_n)
    N, O, H, W = 3, 8, 5, 6
    s2 = (torch.rand(N, 2 * O, H, W, generator=g) * 6).half().cuda()
    go = (torch.randn(N, O, H, W, generator=g) * 3).half().cuda()
    if cl:
        s2 = s2.contiguous(memory_format=torch.channels_last)
        go = go.contiguous(memory_format=torch.channels_last)
    s2h, outer, inner, c = _ops.pair_layout(s2, keep_half=True)
    assert s2h.dtype == torch.float16
    got = _ops.orn_pair_backward(go, s2h, outer, inner, c, or_n)
    s2f, outer2, inner2, c2 = _ops.pair_layout(s2)
    assert s2f.dtype == torch.float32 and (outer2, inner2, c2) == (outer, inner, c)
    want = _ops.orn_pair_backward(go, s2f, outer2, inner2, c2, or_n)
    assert got.dtype == torch.float16 and want.dtype == torch.float32
    assert torch.equal(got, want.half()) and float(want.abs().max()) > 0
