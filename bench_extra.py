"""The other reference configurations, reported next to the headline of bench.py.

Each entry states its workload, the time of one pass, a rate in the unit that fits it and, where
one kernel dominates, the fraction of the roofline that bounds it (VALU integer throughput for the
AND/popcount kernels, HBM bandwidth for the streaming kernels).  Everything runs on one GPU with
synthetic data; the train steps follow the reference's step structure (utils_own.py:96-171):
forward, label-smoothed cross entropy, backward, Adam step, in the three flavours the training
loop alternates between (sync 1 = SC forward, 3 = error injection only, 2 = calibration on half
a batch).
"""
import time

VALU_PEAK_LANEOPS = 256 * 64 * 2.4e9
HBM_PEAK = 8.0e12


def _time(torch, fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def config1_sc_conv_or1(torch, dev):
    import sc_extension_cuda
    L = 32
    g = torch.Generator().manual_seed(1)
    x = (torch.randint(0, 32, (32, 32, 32, 32), generator=g).float() / 32).to(dev)
    w = ((torch.rand(64, 32, 3, 3, generator=g) * 2 - 1) * 32).round().clamp(-31, 31).div(32).to(dev)
    fn = lambda: sc_extension_cuda.conv2d_generic_general_split_acc(x, w, L, -1, 16, (1, 1), (1, 1), (7, 8, 1), 0, 1,
                                                                    True, False)
    sec = _time(torch, fn, 50, 5)
    mac = 32 * 32 * 32 * 64 * 32 * 9
    return {"workload": "SC conv2d forward OR-1, 32-bit streams, N32 C32 32x32 -> 64, 3x3 s1 p1, NCHW",
            "ms": sec * 1e3, "bit_mac_per_s": mac * L / sec, "images_per_s": 32 / sec,
            "valu_frac": mac * L * 4 / 32 / sec / VALU_PEAK_LANEOPS}


def config2_sc_linear(torch, dev):
    import sc_functional as uf
    L = 64
    g = torch.Generator().manual_seed(2)
    x = (torch.randint(0, 64, (256, 4096), generator=g).float() / 64).to(dev).requires_grad_(True)
    w = ((torch.rand(1024, 4096, generator=g) * 2 - 1) * 64).round().clamp(-63, 63).div(64).to(dev).requires_grad_(True)
    gout = torch.randn(256, 1024, generator=g).to(dev)

    def fwd():
        return uf.linear_generic_sc(x, w, bit_length=L, forward="or_2", generator="lfsr", sync=1)

    def fwd_bwd():
        x.grad = None
        w.grad = None
        fwd().backward(gout)

    with torch.no_grad():
        import sc_extension_cuda
        sc_only = lambda: sc_extension_cuda.linear_generic_general_acc(x, w, (7, 8, 1), L, -1, 1, 1, True, False)
        sec_sc = _time(torch, sc_only, 20, 3)
    sec_fb = _time(torch, fwd_bwd, 20, 3)
    mac = 256 * 4096 * 1024
    return {"workload": "SC linear OR-2, 64-bit streams, 256x4096 . (1024x4096)^T; backward through the float surrogate",
            "sc_forward_ms": sec_sc * 1e3, "forward_backward_ms": sec_fb * 1e3,
            "bit_mac_per_s": mac * L / sec_sc, "samples_per_s_fwd_bwd": 256 / sec_fb,
            "valu_frac": mac * L * 4 / 32 / sec_sc / VALU_PEAK_LANEOPS}


def _train_flavours(torch, dev, net, make_batch, batch, steps, lr):
    import torch.nn.functional as F
    opt = torch.optim.Adam(net.parameters(), lr=lr, weight_decay=1e-4)
    out = {}
    for name, sync, frac in (("sync1_sc_forward", 1, 1.0), ("sync3_error_injection", 3, 1.0),
                             ("sync2_calibration_half_batch", 2, 0.5)):
        n = max(1, int(batch * frac))
        x, y = make_batch(n)

        def step():
            net.sync = sync
            opt.zero_grad(set_to_none=True)
            loss = F.cross_entropy(net(x), y, label_smoothing=0.1)
            loss.backward()
            opt.step()
            return loss

        sec = _time(torch, step, steps, 2)
        out[name] = {"ms_per_step": sec * 1e3, "images_per_s": n / sec, "batch": n}
    return out


def config3_tinyconv_step(torch, dev):
    from sc_models import TinyConvSC
    torch.manual_seed(3)
    net = TinyConvSC(forward="or_3", err=6).to(dev)
    g = torch.Generator().manual_seed(3)

    def make_batch(n):
        return (torch.randn(n, 3, 32, 32, generator=g).clamp(-1, 1).to(dev),
                torch.randint(0, 10, (n,), generator=g).to(dev))

    res = _train_flavours(torch, dev, net, make_batch, 256, 10, 8e-3)
    res["workload"] = ("TinyConv-style training step, batch 256, 3x32x32, conv3x3 3-32-32-pool-64-64-pool-fc10, "
                       "OR-3, 64-bit streams, Adam")
    return res


def config4_fixed_conv(torch, dev):
    import fixed_extension_cuda
    import sc_functional as uf
    out = {"workload": "saturating fixed-point conv (add_config 0, 5-bit operands, 24-bit accumulator), batch 64, "
                       "conv3x3 s1 p1: forward kernel alone, and forward + backward through the float conv", "shapes": {}}
    for C, H in ((64, 56), (128, 28), (256, 14), (512, 7)):
        g = torch.Generator().manual_seed(4)
        x = (torch.randint(0, 32, (64, C, H, H), generator=g).float() / 32).to(dev)
        w = (torch.randint(-31, 32, (C, C, 3, 3), generator=g).float() / 32).to(dev)
        fn = lambda: fixed_extension_cuda.conv2d_saturate_acc(x, w, 0, 5, 24, (1, 1), (1, 1))
        sec = _time(torch, fn, 10, 2)
        # forward + backward as the training path runs it: fixed-point forward values over the float
        # conv, whose backward supplies the gradients (generator 'fixed', forward 'full_bin')
        xg, wg = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        gout = torch.randn(64, C, H, H, generator=g).to(dev)

        def fwd_bwd():
            xg.grad = None
            wg.grad = None
            uf.conv2d_generic(xg, wg, (1, 1), (1, 1), bit_length=32, forward="full_bin", generator="fixed",
                              sync=1).backward(gout)

        sec_fb = _time(torch, fwd_bwd, 10, 3)
        nbytes = 4 * x.numel() + 4 * w.numel() + 4 * 64 * C * H * H
        mac = 64 * H * H * C * C * 9
        out["shapes"]["%dx%dx%d" % (C, H, H)] = {"ms": sec * 1e3, "GB_per_s": nbytes / sec / 1e9,
                                               "hbm_frac": nbytes / sec / HBM_PEAK, "mac_per_s": mac / sec,
                                               "images_per_s": 64 / sec, "forward_backward_ms": sec_fb * 1e3,
                                               "images_per_s_fwd_bwd": 64 / sec_fb}
    return out


def config5_resnet18_step(torch, dev, batch=64):
    from sc_models import ResNet18SC
    torch.manual_seed(5)
    net = ResNet18SC(forward="or_2", err=5).to(dev).to(memory_format=torch.channels_last)
    g = torch.Generator().manual_seed(5)

    def make_batch(n):
        return (torch.randn(n, 3, 224, 224, generator=g).to(dev).contiguous(memory_format=torch.channels_last),
                torch.randint(0, 1000, (n,), generator=g).to(dev))

    res = _train_flavours(torch, dev, net, make_batch, batch, 5, 1e-3)
    res["workload"] = ("ResNet-18 SC training step, batch %d, 3x224x224, channels_last, OR-2, 32-bit streams, "
                       "float stem/fc, Adam" % batch)
    return res


def resnet18_sc_conv_fwd_bwd(torch, dev, batch=64):
    """The 19 SC conv layers of ResNet-18 through conv2d_generic (sync 1): integer SC forward over the
    float OR-2 surrogate, backward through the surrogate (two float convs and the OR-n kernels)."""
    import sc_functional as uf
    from bench import RESNET18_SC_LAYERS, make_conv_operands
    layers = []
    for i, (C, H, O, K, s) in enumerate(RESNET18_SC_LAYERS):
        x, w = make_conv_operands(torch, batch, C, H, O, K, 32, seed=900 + i)
        x = x.to(dev).contiguous(memory_format=torch.channels_last).requires_grad_(True)
        w = (w.to(dev) * 0.1).requires_grad_(True)
        Ho = (H + 2 * (K // 2) - K) // s + 1
        gout = torch.randn(batch, O, Ho, Ho, device=dev).contiguous(memory_format=torch.channels_last)
        layers.append((x, w, K, s, gout))

    def step():
        for (x, w, K, s, gout) in layers:
            x.grad = None
            w.grad = None
            uf.conv2d_generic(x, w, (K // 2, K // 2), (s, s), bit_length=32, forward="or_2", generator="lfsr",
                              sync=1).backward(gout)

    sec = _time(torch, step, 5, 2)
    return {"workload": "19 ResNet-18 SC conv layers, batch %d, OR-2, 32-bit streams, channels_last: SC forward + "
                        "backward through the float surrogate (conv2d_generic, sync 1)" % batch,
            "ms_per_step": sec * 1e3, "images_per_s": batch / sec}


def pointwise(torch, dev):
    import _ops
    n = 64 * 64 * 56 * 56  # one ResNet-18 layer1 activation tensor
    x = torch.rand(n, device=dev) * 4
    x2 = torch.rand(n, device=dev) * 4
    gout = torch.randn(n, device=dev)
    coef = torch.tensor([0.01, -0.01, 0.002, 0.0, 0.0, 0.0], device=dev)
    res = {"workload": "pointwise kernels on %d float32 elements (64x64x56x56)" % n}
    for name, fn, bpe in (
            ("orn_forward", lambda: _ops.orn_forward(x, 2), 8),
            ("orn_backward", lambda: _ops.orn_backward(gout, x, 2), 12),
            ("orn_bias_std_both_forward", lambda: _ops.orn_bias_std_both_forward(x, x2, coef, coef, 2), 12),
            ("orn_bias_std_both_backward", lambda: _ops.orn_bias_std_both_backward(gout, x, x2, coef, 2), 20)):
        sec = _time(torch, fn, 20, 3)
        res[name] = {"ms": sec * 1e3, "GB_per_s": bpe * n / sec / 1e9, "hbm_frac": bpe * n / sec / HBM_PEAK}
    # the kernels of the merged surrogate: both polarities in one [pixels][2][channels] tensor
    outer, inner = 64 * 56 * 56, 64
    s2 = (torch.rand(64, 2 * inner, 56, 56, device=dev) * 4).contiguous(memory_format=torch.channels_last)
    g4 = gout.view(64, 56, 56, inner).permute(0, 3, 1, 2)
    pos = torch.randint(0, 64, (64, inner, 56, 56), device=dev, dtype=torch.int16).contiguous(memory_format=torch.channels_last)
    neg = torch.randint(0, 64, (64, inner, 56, 56), device=dev, dtype=torch.int16).contiguous(memory_format=torch.channels_last)
    for name, fn, bpe in (
            ("orn_pair_backward", lambda: _ops.orn_pair_backward(g4, s2, outer, inner, True, 2), 20),
            ("orn_bias_std_pair_forward", lambda: _ops.orn_bias_std_pair_forward(s2, outer, inner, True, coef, coef, 2), 12),
            ("orn_bias_std_pair_backward", lambda: _ops.orn_bias_std_pair_backward(g4, s2, outer, inner, True, coef, 2), 20),
            ("sc_counts_to_float", lambda: _ops.sc_counts_to_float(pos, neg, 32), 8),
            ("quantize", lambda: _ops.quantize(x, 7), 8)):
        sec = _time(torch, fn, 20, 3)
        res[name] = {"ms": sec * 1e3, "GB_per_s": bpe * n / sec / 1e9, "hbm_frac": bpe * n / sec / HBM_PEAK}
    return res


def run(torch, dev):
    out = {}
    for name, fn in (("config1_sc_conv_or1", config1_sc_conv_or1), ("config2_sc_linear", config2_sc_linear),
                     ("config3_tinyconv_train", config3_tinyconv_step), ("config4_fixed_conv", config4_fixed_conv),
                     ("config5_resnet18_train", config5_resnet18_step),
                     ("resnet18_sc_conv_fwd_bwd", resnet18_sc_conv_fwd_bwd), ("pointwise", pointwise)):
        try:
            out[name] = fn(torch, dev)
        except Exception as e:
            out[name] = {"error": "%s: %s" % (type(e).__name__, e)}
        torch.cuda.empty_cache()
    return out
