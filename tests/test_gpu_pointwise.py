"""Pointwise HIP kernels (through the C ABI) against the oracle's float32 restatement.

Tolerance: 1e-5 relative plus a few ulps of the leading constant n (the functions subtract
exp(-x) terms from n, so tiny outputs carry the rounding of n itself)."""
import numpy as np
import pytest
import torch

import oracle as orc

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def _close(got, want, atol):
    got = got.detach().cpu().numpy() if isinstance(got, torch.Tensor) else got
    err = np.abs(got.astype(np.float64) - want.astype(np.float64))
    assert (err <= atol + RTOL * np.abs(want)).all(), "max err %g" % err.max()


def _x(n_elem, seed):
    rng = np.random.default_rng(seed)
    x = np.concatenate([rng.uniform(0, 8, n_elem - 6), [0.0, 1e-3, 0.5, 11.0, 30.0, 88.0]]).astype(np.float32)
    return x


@pytest.mark.parametrize("n", [1, 2, 3, 4])
@pytest.mark.parametrize("size", [1, 7, 4099, 1 << 20])
def test_orn_forward_backward(n, size):
    import sc_extension_cuda
    print("orn fwd/bwd", n, size, flush=True)
    x = _x(size + 6, n)[:size] if size < 7 else _x(size, n)
    xt = torch.from_numpy(x).cuda()
    y = sc_extension_cuda.or_approx_n_forward_acc(xt, n)
    assert y.dtype == torch.float32 and y.shape == xt.shape
    _close(y, orc.or_approx_n_forward(x, n), atol=4 * n * 1.2e-7)
    g = np.random.default_rng(5).normal(size=x.shape).astype(np.float32)
    gx = sc_extension_cuda.or_approx_n_backward_acc(torch.from_numpy(g).cuda(), xt, n)
    _close(gx, orc.or_approx_n_backward(g, x, n, half_input=True), atol=1e-7)


def test_orn_accepts_half_and_channels_last():
    import sc_extension_cuda
    x = torch.rand(2, 8, 5, 5, device="cuda").contiguous(memory_format=torch.channels_last) * 3
    y = sc_extension_cuda.or_approx_n_forward_acc(x, 2)
    assert y.stride() == x.stride()
    _close(y.contiguous(), orc.or_approx_n_forward(x.contiguous().cpu().numpy(), 2), atol=1e-6)
    yh = sc_extension_cuda.or_approx_n_forward_acc(x.half(), 2)
    assert yh.dtype == torch.float32
    _close(yh.contiguous(), orc.or_approx_n_forward(x.half().float().contiguous().cpu().numpy(), 2), atol=1e-6)
    with pytest.raises(RuntimeError, match="or_n"):
        sc_extension_cuda.or_approx_n_forward_acc(x, 5)


@pytest.mark.parametrize("n", [1, 2, 3, 4])
@pytest.mark.parametrize("size", [5, 4096, 100003])
def test_fused_both_forward_backward(n, size):
    import _ops
    import sc_extension_cuda
    print("fused both", n, size, flush=True)
    rng = np.random.default_rng(n * 7 + size)
    xp = rng.uniform(0, 5, size).astype(np.float32)
    xn = rng.uniform(0, 5, size).astype(np.float32)
    # coefficients decay with the power so that every term stays O(1) for OR_n values up to n = 4:
    # the result is a difference of the two polarities and is compared at 1e-5 of ITS magnitude
    decay = 0.4 ** np.arange(6)
    b = (rng.normal(size=6) * 0.05 * decay).astype(np.float32)
    s = (np.abs(rng.normal(size=6)) * 0.02 * decay).astype(np.float32)
    tp, tn = torch.from_numpy(xp).cuda(), torch.from_numpy(xn).cuda()
    tb, ts = torch.from_numpy(b).cuda(), torch.from_numpy(s).cuda()
    # the draws are returned so that the deterministic part can be checked exactly
    y, zp, zn = _ops.orn_bias_std_both_forward(tp, tn, tb, ts, n, seed=1234, offset=10, return_noise=True)
    want = orc.or_approx_n_forward_bias_std_both(xp, xn, b, s, n, zp.cpu().numpy(), zn.cpu().numpy())
    _close(y, want, atol=4e-6)
    # same (seed, offset) -> same draws; another offset -> other draws
    ya, _, _ = _ops.orn_bias_std_both_forward(tp, tn, tb, ts, n, seed=1234, offset=10, return_noise=True)
    assert torch.equal(y, ya)
    # without the noise outputs: one draw per output (the first stream's), scaled by the root of the summed variances
    y2 = _ops.orn_bias_std_both_forward(tp, tn, tb, ts, n, seed=1234, offset=10)
    assert torch.equal(y2, _ops.orn_bias_std_both_forward(tp, tn, tb, ts, n, seed=1234, offset=10))
    vp, vn = orc.or_approx_n_forward(xp, n).astype(np.float64), orc.or_approx_n_forward(xn, n).astype(np.float64)
    poly = lambda c, v: sum(float(c[k]) * v ** k for k in range(6))
    want2 = (vp + poly(b, vp)) - (vn + poly(b, vn)) + np.sqrt(poly(s, vp) ** 2 + poly(s, vn) ** 2) * zp.cpu().numpy()
    _close(y2, want2.astype(np.float32), atol=4e-6)
    if size > 100:
        y3 = _ops.orn_bias_std_both_forward(tp, tn, tb, ts, n, seed=1234, offset=11)
        assert not torch.equal(y2, y3)
    # zero std coefficients: fully deterministic
    y0 = sc_extension_cuda.or_approx_n_forward_bias_std_both_acc(tp, tn, tb, torch.zeros(6, device="cuda"), n)
    want0 = orc.or_approx_n_forward_bias_std_both(xp, xn, b, np.zeros(6, np.float32), n, np.zeros(size, np.float32),
                                                  np.zeros(size, np.float32))
    _close(y0, want0, atol=4e-6)
    g = rng.normal(size=size).astype(np.float32)
    gp, gn = sc_extension_cuda.or_approx_n_backward_bias_std_both_acc(torch.from_numpy(g).cuda(), tp, tn, tb, n)
    wp, wn = orc.or_approx_n_backward_bias_std_both(g, xp, xn, b, n, half_input=True)
    _close(gp, wp, atol=1e-6)
    _close(gn, wn, atol=1e-6)


def test_noise_statistics():
    """The injected noise is N(0,1): moments, tails and independence of the two polarities."""
    import _ops
    n = 1 << 22
    z = torch.zeros(n, device="cuda")
    coef0 = torch.zeros(6, device="cuda")
    _, zp, zn = _ops.orn_bias_std_both_forward(z, z, coef0, coef0, 1, seed=99, offset=0, return_noise=True)
    for d in (zp, zn):
        d = d.double()
        assert abs(d.mean().item()) < 3e-3
        assert abs(d.var().item() - 1) < 5e-3
        assert abs((d ** 3).mean().item()) < 1e-2
        assert abs((d ** 4).mean().item() - 3) < 3e-2
        assert abs((d.abs() > 1.959964).double().mean().item() - 0.05) < 1e-3
        assert d.abs().max().item() < 6.5
    assert abs((zp.double() * zn.double()).mean().item()) < 3e-3
    # Kolmogorov-Smirnov against the normal CDF on a subsample
    from scipy import stats
    ks = stats.kstest(zp[:200000].cpu().numpy().astype(np.float64), "norm")
    assert ks.pvalue > 1e-3


def test_single_draw_noise_has_the_variance_of_the_two_draw_form():
    """Without the noise outputs the fused forward draws one normal per output scaled by
    sqrt(std(v_pos)^2 + std(v_neg)^2): per bin of (v_pos, v_neg) the result has the mean of the deterministic part
    and the variance std_p^2 + std_n^2 of the reference's two-draw form (sc_cuda_pw.cu:219-373), and so has the
    pair-layout kernel, which draws the same noise."""
    import _ops
    n = 1 << 22
    bias = torch.tensor([0.01, -0.02, 0.004, 0.0, 0.001, 0.0], device="cuda")
    std = torch.tensor([0.05, 0.03, -0.004, 0.0, 0.0, 0.0], device="cuda")
    poly = lambda c, v: sum(c[k].item() * v ** k for k in range(6))
    for xp_v, xn_v in ((0.3, 2.0), (1.5, 0.0), (3.0, 3.0)):
        xp = torch.full((n,), xp_v, device="cuda")
        xn = torch.full((n,), xn_v, device="cuda")
        y = _ops.orn_bias_std_both_forward(xp, xn, bias, std, 2, seed=7, offset=0).double()
        vp = float(orc.or_approx_n_forward(np.array([xp_v], np.float32), 2)[0])
        vn = float(orc.or_approx_n_forward(np.array([xn_v], np.float32), 2)[0])
        mean = (vp + poly(bias, vp)) - (vn + poly(bias, vn))
        var = poly(std, vp) ** 2 + poly(std, vn) ** 2
        assert abs(y.mean().item() - mean) < 4 * (var / n) ** 0.5 + 1e-6
        assert abs(y.var().item() / var - 1) < 5e-3
        z = (y - mean) / var ** 0.5
        assert abs((z ** 3).mean().item()) < 1e-2 and abs((z ** 4).mean().item() - 3) < 3e-2
        # the two-draw form (noise outputs requested) has the same moments
        y2, _, _ = _ops.orn_bias_std_both_forward(xp, xn, bias, std, 2, seed=7, offset=0, return_noise=True)
        assert abs(y2.double().mean().item() - mean) < 4 * (var / n) ** 0.5 + 1e-6
        assert abs(y2.double().var().item() / var - 1) < 5e-3
        # pair layout: same values as the two-tensor kernel, element for element
        s2 = torch.stack((xp.view(-1, 64), xn.view(-1, 64)), dim=1).contiguous()
        yp = _ops.orn_bias_std_pair_forward(s2.view(-1, 128), n // 64, 64, False, bias, std, 2, seed=7, offset=0)
        assert torch.equal(yp.reshape(-1), y.float())


def test_single_polarity_variants():
    import _ops
    import sc_extension_cuda
    rng = np.random.default_rng(2)
    x = rng.uniform(0, 4, 3001).astype(np.float32)
    b = (rng.normal(size=6) * 0.05).astype(np.float32)
    tb = torch.from_numpy(b).cuda()
    y = sc_extension_cuda.or_approx_n_forward_bias_std_acc(torch.from_numpy(x).cuda(), tb, torch.zeros(6, device="cuda"), 3)
    assert y.dtype == torch.float16
    xh = x.astype(np.float16).astype(np.float32)
    want = orc.or_approx_n_forward_bias_std_both(xh, np.zeros_like(xh), b, np.zeros(6, np.float32), 3,
                                                 np.zeros_like(xh), np.zeros_like(xh))
    want = want + orc.or_approx_n_forward_bias_std_both(np.zeros_like(xh), np.zeros_like(xh), b, np.zeros(6, np.float32),
                                                        3, np.zeros_like(xh), np.zeros_like(xh))[0] * 0 \
        + (b[0])  # f(OR(0)) = b0 was subtracted by the "both" form
    assert np.allclose(y.float().cpu().numpy(), want, rtol=2e-3, atol=2e-3)
    g = rng.normal(size=x.shape).astype(np.float32)
    gx = sc_extension_cuda.or_approx_n_backward_bias_std_acc(torch.from_numpy(g).cuda(), torch.from_numpy(x).cuda(), tb, 3)
    wp, _ = orc.or_approx_n_backward_bias_std_both(g, x, x, b, 3, half_input=True)
    _close(gx, wp, atol=1e-6)


def test_calib_stats_kernel():
    import _ops
    rng = np.random.default_rng(8)
    n = 300007
    a_act = rng.uniform(0, 2.5, n).astype(np.float32)
    a_bit = (a_act + 0.03 + 0.05 * rng.normal(size=n)).astype(np.float32)
    starts = np.linspace(0, float(a_bit.max()), 30)
    lo = [np.float32(s) for s in starts]
    hi = [np.float32(s + 0.1) for s in starts]
    st = _ops.calib_stats(torch.from_numpy(a_bit).cuda(), torch.from_numpy(a_act).cuda(), lo, hi).cpu().numpy()
    for k in range(30):
        sel = (a_act >= lo[k]) & (a_act < hi[k])
        err = (a_bit[sel] - a_act[sel]).astype(np.float64)
        assert st[k, 0] == sel.sum()
        # sums and sums of squares are carried in float64 from the first term on (the reference works in float32
        # throughout)
        assert abs(st[k, 1] - err.sum()) <= 1e-12 * np.abs(err).sum() + 1e-12
        assert np.isclose(st[k, 2], (err * err).sum(), rtol=1e-12, atol=1e-12)


def test_calib_stats_variance_survives_a_large_bias():
    """A spread a thousand times smaller than the bias: the variance formed from the returned sums as
    s2/n - (s1/n)^2 still agrees with the float64 variance of the float32 errors."""
    import _ops
    rng = np.random.default_rng(9)
    n = 1 << 20
    a_act = rng.uniform(0, 1, n).astype(np.float32)
    a_bit = (a_act + 1.0 + 1e-3 * rng.normal(size=n)).astype(np.float32)
    st = _ops.calib_stats(torch.from_numpy(a_bit).cuda(), torch.from_numpy(a_act).cuda(), [np.float32(0)],
                          [np.float32(2)]).cpu().numpy()
    err = (a_bit - a_act).astype(np.float64)
    cnt, s1, s2 = st[0]
    assert cnt == n
    var = s2 / cnt - (s1 / cnt) ** 2
    assert np.isclose(var, err.var(), rtol=1e-6)


def test_noise_stream_follows_the_torch_generator():
    """Seed and offset come from the device's torch generator: re-seeding restarts the noise,
    consecutive calls draw from disjoint parts of the stream."""
    import sc_extension_cuda
    x = torch.rand(5000, device="cuda")
    coef0 = torch.zeros(6, device="cuda")
    std = torch.tensor([0.5, 0, 0, 0, 0, 0], device="cuda")
    torch.manual_seed(7)
    a = sc_extension_cuda.or_approx_n_forward_bias_std_both_acc(x, x, coef0, std, 2)
    b = sc_extension_cuda.or_approx_n_forward_bias_std_both_acc(x, x, coef0, std, 2)
    torch.manual_seed(7)
    c = sc_extension_cuda.or_approx_n_forward_bias_std_both_acc(x, x, coef0, std, 2)
    assert torch.equal(a, c)
    assert not torch.equal(a, b)
    assert abs(float(((a - b) / 0.5).var()) - 4.0) < 0.4   # four independent N(0,1) draws per element
