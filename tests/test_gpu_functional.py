"""The host-side counterpart of utils_functional / utils_class on the GPU: mode logic (sync 1/2/3),
what .data holds, gradients of the surrogate, calibration, layers and one training step."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle as orc

pytestmark = pytest.mark.gpu


def _operands(seed, N=2, C=16, H=10, O=12, L=32, dens=0.35):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randint(0, L, (N, C, H, H), generator=g).float() / L) * (torch.rand(N, C, H, H, generator=g) < dens)
    w = (torch.randint(-L + 1, L, (O, C, 3, 3), generator=g).float() / L) * (torch.rand(O, C, 3, 3, generator=g) < dens)
    return x, w


def _orn64(s, n):
    e = torch.exp(-s)
    fact = [1, 1, 2, 6]
    return n - e * sum((n - i) * s ** i / fact[i] for i in range(n))


@pytest.mark.parametrize("forward,n", [("or_1", 1), ("or_2", 2), ("or_3", 3), ("full_or", 1)])
def test_sync1_forward_is_sc_and_backward_is_surrogate(forward, n):
    import sc_functional as uf
    print("sync1", forward, flush=True)
    L = 32
    x, w = _operands(1)
    xt = x.cuda().requires_grad_(True)
    wt = w.cuda().requires_grad_(True)
    out = uf.conv2d_generic(xt, wt, (1, 1), (1, 1), bit_length=L, generator="lfsr", forward=forward, sync=1, order=5)
    bc = 0 if forward == "full_or" else n - 1
    pos, neg = orc.conv2d_generic_general_split(x.numpy(), w.numpy(), L, -1, 16, (1, 1), (1, 1), (7, 8, 1), bc, 1)
    want = pos.astype(np.float32) / L - neg.astype(np.float32) / L
    assert np.array_equal(out.detach().cpu().numpy(), want)      # forward values are the SC result, exactly
    g = torch.randn(out.shape, generator=torch.Generator().manual_seed(3)).cuda()
    out.backward(g)
    # the gradient is that of the float surrogate, evaluated on the fp16-rounded saved sums
    x64 = x.double().requires_grad_(True)
    w64 = w.double().requires_grad_(True)
    sp = F.conv2d(x64, w64.clamp(0, 100), padding=1)
    sn = F.conv2d(x64, -(w64.clamp(-100, 0)), padding=1)
    # d OR_n / ds at the rounded s, chained by hand so that the rounding does not enter autograd
    def dorn(s):
        sh = s.detach().float().half().double()
        return torch.exp(-sh) * sum(sh ** i / [1, 1, 2, 6][i] for i in range(n))
    (sp * (dorn(sp) * g.cpu().double())).sum().backward(retain_graph=True)
    gx_pos, gw_pos = x64.grad.clone(), w64.grad.clone()
    x64.grad = None; w64.grad = None
    (sn * (dorn(sn) * (-g.cpu().double()))).sum().backward()
    gx = gx_pos + x64.grad
    gw = gw_pos + w64.grad
    # 1e-5 relative to the largest gradient entry (float32 convolutions against float64)
    assert (xt.grad.cpu().double() - gx).abs().max() <= 1e-5 * gx.abs().max()
    assert (wt.grad.cpu().double() - gw).abs().max() <= 1e-5 * gw.abs().max()


def test_sync3_is_error_injection_only():
    import sc_functional as uf
    x, w = _operands(2)
    xt, wt = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    bias = torch.tensor([0.01, -0.02, 0.005, 0, 0, 0], device="cuda")
    out = uf.conv2d_generic(xt, wt, (1, 1), (1, 1), bit_length=32, generator="lfsr", forward="or_2", sync=3,
                            bias_coef=bias, std_coef=torch.zeros(6, device="cuda"), order=5)
    sp = F.conv2d(x.double(), w.double().clamp(0, 100), padding=1).float().numpy()
    sn = F.conv2d(x.double(), -(w.double().clamp(-100, 0)), padding=1).float().numpy()
    want = orc.or_approx_n_forward_bias_std_both(sp, sn, bias.cpu().numpy(), np.zeros(6, np.float32), 2,
                                                 np.zeros_like(sp), np.zeros_like(sp))
    assert np.abs(out.detach().cpu().numpy() - want).max() <= 1e-5 * np.abs(want).max()
    out.sum().backward()
    assert torch.isfinite(xt.grad).all() and xt.grad.abs().sum() > 0


def test_sync2_calibrates_in_place():
    import sc_functional as uf
    L = 32
    x, w = _operands(4, N=4, C=32, H=16, O=32, dens=0.3)
    xt, wt = x.cuda(), w.cuda()
    bias = torch.zeros(6, device="cuda")
    std = torch.zeros(6, device="cuda")
    out, b2, s2 = uf.conv2d_generic(xt, wt, (1, 1), (1, 1), bit_length=L, generator="lfsr", forward="or_2", sync=2,
                                    bias_coef=bias, std_coef=std, order=5)
    assert b2 is bias and s2 is std and std.abs().sum() > 0      # buffers are updated in place
    pos, neg = orc.conv2d_generic_general_split(x.numpy(), w.numpy(), L, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1)
    sp = F.conv2d(x, w.clamp(0, 100), padding=1).numpy()
    sn = F.conv2d(x, -(w.clamp(-100, 0)), padding=1).numpy()
    a_bit = np.concatenate([pos.reshape(-1) / np.float32(L), neg.reshape(-1) / np.float32(L)]).astype(np.float32)
    a_act = np.concatenate([orc.or_approx_n_forward(sp, 2).reshape(-1), orc.or_approx_n_forward(sn, 2).reshape(-1)])
    wb, ws = orc.compute_bias_std_coef(2, a_bit, a_act, 5)
    grid = np.linspace(0, float(a_bit.max()), 9)
    ev = lambda c: sum(c[k] * grid ** k for k in range(6))
    assert np.allclose(ev(bias.cpu().numpy()), ev(wb), atol=2e-3)
    assert np.allclose(ev(std.cpu().numpy()), ev(ws), atol=2e-3)
    assert torch.isfinite(out).all()


def test_fixed_generator_mode():
    import sc_functional as uf
    L = 32
    x, w = _operands(5)
    out = uf.conv2d_generic(x.cuda(), w.cuda(), (1, 1), (1, 1), bit_length=L, generator="fixed", forward="full_bin",
                            sync=1, order=5)
    want = orc.conv2d_saturate(x.numpy(), w.numpy(), 0, 5, 24, (1, 1), (1, 1)).astype(np.float32) / L / L
    assert np.allclose(out.detach().cpu().numpy(), want, rtol=0, atol=0)


def test_fixed_generator_backward_is_the_float_conv():
    """generator 'fixed' / forward 'full_bin': the forward value is the saturating fixed-point conv, the gradient
    that of conv(x, clamp(w, -100, 100)) (utils_functional.py:1184-1188, 1244-1246)."""
    import sc_functional as uf
    L = 32
    x, w = _operands(6, N=3, C=24, H=12, O=20)
    xt, wt = x.cuda().requires_grad_(True), w.cuda().requires_grad_(True)
    out = uf.conv2d_generic(xt, wt, (1, 1), (2, 2), bit_length=L, generator="fixed", forward="full_bin", sync=1, order=5)
    want = orc.conv2d_saturate(x.numpy(), w.numpy(), 0, 5, 24, (1, 1), (2, 2)).astype(np.float32) / L / L
    assert np.array_equal(out.detach().cpu().numpy(), want)
    g = torch.randn(out.shape, generator=torch.Generator().manual_seed(8))
    out.backward(g.cuda())
    x64, w64 = x.double().requires_grad_(True), w.double().requires_grad_(True)
    F.conv2d(x64, w64.clamp(-100, 100), padding=1, stride=2).backward(g.double())
    assert (xt.grad.cpu().double() - x64.grad).abs().max() <= 1e-5 * x64.grad.abs().max()
    assert (wt.grad.cpu().double() - w64.grad).abs().max() <= 1e-5 * w64.grad.abs().max()


def test_layer_matches_reference_defaults_and_groups():
    from sc_layers import Conv2d_Add_Partial
    torch.manual_seed(0)
    layer = Conv2d_Add_Partial(8, 12, kernel_size=3, padding=1, groups=2, bias=False, forward="or_2", err=5).cuda()
    assert layer.run_args["bit_length"] == 32 and layer.run_args["prec"] == 7 and layer.run_args["order"] == 5
    assert set(dict(layer.named_buffers())) == {"weight_flag", "prune", "bias_coef", "std_coef"}
    x = torch.rand(2, 8, 6, 6, device="cuda")
    y = layer(x)
    assert y.shape == (2, 12, 6, 6)
    # group g of the output only depends on group g of the input; the reference stacks the group
    # results along dim 2 before flattening (utils_class.py:75-76), so output channel
    # o_in_group * groups + g belongs to group g
    x2 = x.clone()
    x2[:, 4:] = 0
    y2 = layer(x2)
    assert torch.equal(y[:, 0::2], y2[:, 0::2]) and not torch.equal(y[:, 1::2], y2[:, 1::2])
    # values: quantise (prec 7) then the SC op per group
    xq = orc.quantize(x.cpu().numpy(), 7)
    wq = orc.quantize(layer.weight.detach().cpu().numpy(), 7)
    pos, neg = orc.conv2d_generic_general_split(xq[:, :4], wq[:6], 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 1, 1)
    assert np.array_equal(y[:, 0::2].detach().cpu().numpy(), (pos / np.float32(32) - neg / np.float32(32)))


def test_linear_layer_forward_and_grad():
    from sc_layers import Linear_Or
    torch.manual_seed(1)
    layer = Linear_Or(64, 10, bias=False, forward="or_2", err=6).cuda()
    x = torch.rand(5, 64, device="cuda", requires_grad=True)
    y = layer(x)
    xq = orc.quantize(x.detach().cpu().numpy(), 7)
    wq = orc.quantize(layer.weight.detach().cpu().numpy(), 7)
    pos, neg = orc.linear_generic_general(xq, wq, (7, 8, 1), 64, -1, 1, 1)
    assert np.array_equal(y.detach().cpu().numpy(), pos.astype(np.float32) / 64 - neg.astype(np.float32) / 64)
    y.sum().backward()
    assert torch.isfinite(x.grad).all() and layer.weight.grad.abs().sum() > 0


@pytest.mark.parametrize("sync", [1, 3, 2])
def test_tinyconv_training_step(sync):
    """One optimiser step of the TinyConv-style net in each step flavour: finite, and the SC flavours
    are reproducible bit for bit."""
    from sc_models import TinyConvSC
    print("tinyconv step sync", sync, flush=True)

    def run():
        torch.manual_seed(0)
        net = TinyConvSC(forward="or_3", err=6).cuda()
        opt = torch.optim.Adam(net.parameters(), lr=8e-3, weight_decay=1e-4)
        g = torch.Generator().manual_seed(3)
        x = torch.randn(8, 3, 32, 32, generator=g).clamp(-1, 1).cuda()
        y = torch.randint(0, 10, (8,), generator=g).cuda()
        net.sync = sync
        loss = F.cross_entropy(net(x), y)
        loss.backward()
        opt.step()
        return loss.item(), [p.detach().clone() for p in net.parameters()]

    l1, p1 = run()
    assert np.isfinite(l1)
    assert all(torch.isfinite(p).all() for p in p1)
    if sync == 1:
        l2, _ = run()
        assert l1 == l2


def test_calibration_fit_matches_reference_python_on_gpu():
    """sc_functional.compute_bias_std_coef (statistics kernel + host fit) against the vectors written
    by the reference's own function."""
    import sc_functional as uf
    from test_oracle_golden import check_calib_against_reference

    def fit(or_n, bit, act, order):
        b, s = uf.compute_bias_std_coef(or_n, torch.from_numpy(bit).cuda(), torch.from_numpy(act).cuda(), order)
        return b.cpu().numpy(), s.cpu().numpy()

    check_calib_against_reference(fit)


@pytest.mark.parametrize("prec", [0, 1, 5, 7, 8, 16])
def test_fused_quantize_equals_the_four_torch_passes(prec):
    """quantize (utils_functional.py:93-104) as one kernel: bit-equal to mul / round / clamp / div."""
    import _ops
    import sc_functional as uf
    g = torch.Generator().manual_seed(prec)
    s = 2.0 ** prec
    x = torch.cat([
        torch.randn(100003, generator=g) * 0.7,
        (torch.arange(-40, 41).float() + 0.5) / s,            # ties: round half to even
        torch.tensor([0.0, -0.0, 1.0, -1.0, 3.0, -3.0, 1 - 1 / s, 1e-30, -1e-30, 1e30, float("inf"), -float("inf"),
                      float("nan")]),
    ]).cuda()
    want = (x * s).round().clamp(-s + 1, s - 1) / s
    got = _ops.quantize(x, prec)
    assert torch.equal(torch.nan_to_num(got, nan=9.0), torch.nan_to_num(want, nan=9.0))
    assert torch.equal(torch.signbit(got), torch.signbit(want))
    # through QuantizeGrad: same values, straight-through gradient, channels_last kept
    x4 = torch.randn(2, 8, 5, 5, generator=g).cuda().contiguous(memory_format=torch.channels_last).requires_grad_(True)
    y4 = uf.QuantizeGrad.apply(x4, prec)
    assert y4.stride() == x4.stride()
    assert torch.equal(y4, (x4.detach() * s).round().clamp(-s + 1, s - 1) / s)
    y4.backward(torch.ones_like(y4))
    assert torch.equal(x4.grad, torch.ones_like(x4))


@pytest.mark.parametrize("prec", [0, 1, 5, 7, 10])
def test_fused_quantize_on_float16_equals_the_four_float16_passes(prec):
    """Inside a float16 autocast region QuantizeGrad sees float16 activations: every float16 bit pattern through
    rexsc_quantize_f16 against mul / round / clamp / div on the float16 tensor, bit for bit."""
    import _ops
    import sc_functional as uf
    s = 2.0 ** prec
    x = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16).view(torch.float16).cuda()  # all 65536 patterns
    want = (x * s).round().clamp(-s + 1, s - 1) / s
    got = _ops.quantize(x, prec)
    assert got.dtype == torch.float16
    assert torch.equal(torch.nan_to_num(got.float(), nan=9.0), torch.nan_to_num(want.float(), nan=9.0))
    assert torch.equal(torch.signbit(got), torch.signbit(want))
    # ragged length (scalar tail), channels_last, through QuantizeGrad
    assert torch.equal(_ops.quantize(x[5:1008], prec), want[5:1008])
    g = torch.Generator().manual_seed(prec)
    x4 = torch.randn(2, 8, 5, 5, generator=g).half().cuda().contiguous(memory_format=torch.channels_last).requires_grad_(True)
    y4 = uf.QuantizeGrad.apply(x4, prec)
    assert y4.dtype == torch.float16 and y4.stride() == x4.stride()
    assert torch.equal(y4, (x4.detach() * s).round().clamp(-s + 1, s - 1) / s)
    # a precision beyond the kernel's range takes the tensor passes
    assert torch.equal(uf.quantize(x4.detach(), 12), (x4.detach() * 4096).round().clamp(-4095, 4095) / 4096)
