"""The other reference configurations, reported next to the headline of bench.py.

Each entry states its workload, the time of one pass, a rate in the unit that fits it and the fraction
of the roofline that bounds its kernels (VALU integer throughput for the AND/popcount kernels, HBM
bandwidth for the streaming kernels).  Everything runs on one GPU with synthetic data; the train steps
follow the reference's step structure (utils_own.py:96-171): forward, label-smoothed cross entropy,
backward, Adam step, in the three flavours the training loop alternates between (sync 1 = SC forward,
3 = error injection only, 2 = calibration on half a batch).

Kernel-level figures come from the library's own HIP-event brackets (rexsc_profile_begin / _end) in a
pass separate from the wall-clock timing.  The streaming kernels are timed twice: on one set of buffers
(which the 256 MB memory-side cache can partly hold) and rotating through more than 1 GiB of distinct
buffers, so that every byte comes from and goes to HBM; `hbm_frac` is the rotating figure.
"""
import ctypes
import gc
import json
import os
import time

# integer VALU roofs, lane-ops/s (see bench.py): and + popcount pair at 2 + 4 cycles per wave64 and SIMD; single
# instructions of the 4-cycle class (v_and_or_b32, the OR-1 kernels)
VALU_PEAK_LANEOPS = 256 * 4 * (2 * 64 / 6) * 2.4e9
VALU_PEAK_4CYCLE = 256 * 4 * 16 * 2.4e9
HBM_PEAK = 8.0e12
ROTATE_BYTES = 1.25 * 2 ** 30  # distinct bytes touched before a buffer is used again

SC_KERNELS = ("sc_compute", "sc_finalize", "sng_", "fold_")
STREAM_KERNELS = ("orn_", "sc_counts_to_float", "quantize", "split_weight", "merge_weight_grad", "calib_stats",
                  "fixed_")


def _time(torch, fn, steps, warmup):
    """Seconds per call of fn over `steps` calls after `warmup` untimed ones; Python's cyclic garbage collector is
    held off during the timed calls, as timeit does (a full collection is tens of milliseconds in this process)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    gc_was_on = gc.isenabled()
    gc.disable()
    try:
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps
    finally:
        if gc_was_on:
            gc.enable()


def _profile(torch, fn, reps):
    """Per-kernel records of `reps` passes of fn: {name: dict(calls, total_ms, total_work)} per pass."""
    import _lib
    fn()
    torch.cuda.synchronize()
    _lib.profile_begin()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    prof = _lib.profile_end(max_records=128)
    return {k: dict(calls=v["calls"] / reps, ms=v["total_ms"] / reps, work=v["total_work"] / reps) for k, v in prof.items()}


def _breakdown(prof, step_ms):
    """Library time of one step by kernel class, with the roofline fraction of each class."""
    sc = {k: v for k, v in prof.items() if k.startswith(SC_KERNELS)}
    comp = {k: v for k, v in sc.items() if k.startswith("sc_compute")}
    pw = {k: v for k, v in prof.items() if k.startswith(STREAM_KERNELS)}
    sc_ms = sum(v["ms"] for v in sc.values())
    comp_ms = sum(v["ms"] for v in comp.values())
    comp_ops = sum(v["work"] for v in comp.values())
    pw_ms = sum(v["ms"] for v in pw.values())
    pw_bytes = sum(v["work"] for v in pw.values())
    lib_ms = sc_ms + pw_ms
    out = {
        "sc_kernels_ms": round(sc_ms, 4), "sc_compute_ms": round(comp_ms, 4),
        "sc_compute_valu_frac": comp_ops / (comp_ms * 1e-3) / VALU_PEAK_LANEOPS if comp_ms else None,
        "sc_kernels_valu_frac": comp_ops / (sc_ms * 1e-3) / VALU_PEAK_LANEOPS if sc_ms else None,
        "streaming_kernels_ms": round(pw_ms, 4),
        "streaming_kernels_hbm_frac": pw_bytes / (pw_ms * 1e-3) / HBM_PEAK if pw_ms else None,
        "library_ms": round(lib_ms, 4),
        # kernels of this library against the step's wall clock; at sync 1 the SC forward runs on a second stream
        # beside the float convolution, so the two shares can add up to more than one
        "share_outside_library": max(0.0, 1.0 - lib_ms / step_ms),
        "kernel_ms": {k: round(v["ms"], 4) for k, v in sorted(prof.items())},
    }
    return out


def config1_sc_conv_or1(torch, dev):
    import sc_extension_cuda
    L = 32
    g = torch.Generator().manual_seed(1)
    xc = torch.randint(0, 32, (32, 32, 32, 32), generator=g).float() / 32
    wc = ((torch.rand(64, 32, 3, 3, generator=g) * 2 - 1) * 32).round().clamp(-31, 31).div(32)
    x, w = xc.to(dev), wc.to(dev)
    fn = lambda: sc_extension_cuda.conv2d_generic_general_split_acc(x, w, L, -1, 16, (1, 1), (1, 1), (7, 8, 1), 0, 1,
                                                                    True, False)
    sec = _time(torch, fn, 50, 5)
    prof = _profile(torch, fn, 5)
    mac = 32 * 32 * 32 * 64 * 32 * 9
    words = mac * L / 32  # 32-channel stream words ANDed per polarity
    comp_ms = sum(v["ms"] for k, v in prof.items() if k.startswith("sc_compute"))
    out = {"workload": "SC conv2d forward OR-1, 32-bit streams, N32 C32 32x32 -> 64, 3x3 s1 p1, NCHW",
           "ms": sec * 1e3, "bit_mac_per_s": mac * L / sec, "images_per_s": 32 / sec,
           # op model: the AND/popcount formulation costs 2 VALU ops per word and polarity; saturation at one needs no
           # count, and this kernel issues ONE v_and_or_b32 per word and polarity -- both fractions are stated
           "op_model": "kernel issues 1 op/word/polarity (v_and_or_b32); the 2-op figure prices the and+popcount formulation",
           # 2-op model against the pair roof (52.43 T); 1-op model against the roof of the instruction issued (39.32 T)
           "valu_frac_2op": words * 4 / sec / VALU_PEAK_LANEOPS, "valu_frac_1op": words * 2 / sec / VALU_PEAK_4CYCLE,
           "sc_compute_ms": comp_ms,
           "sc_compute_valu_frac_1op": words * 2 / (comp_ms * 1e-3) / VALU_PEAK_4CYCLE if comp_ms else None,
           "kernel_ms": {k: round(v["ms"], 4) for k, v in sorted(prof.items())}}
    return out


def config2_sc_linear(torch, dev):
    import sc_extension_cuda
    import sc_functional as uf
    L = 64
    g = torch.Generator().manual_seed(2)
    xc = torch.randint(0, 64, (256, 4096), generator=g).float() / 64
    wc = ((torch.rand(1024, 4096, generator=g) * 2 - 1) * 64).round().clamp(-63, 63).div(64)
    x = xc.to(dev).requires_grad_(True)
    w = wc.to(dev).requires_grad_(True)
    gout = torch.randn(256, 1024, generator=g).to(dev)

    def fwd_bwd():
        x.grad = None
        w.grad = None
        uf.linear_generic_sc(x, w, bit_length=L, forward="or_2", generator="lfsr", sync=1).backward(gout)

    with torch.no_grad():
        sc_only = lambda: sc_extension_cuda.linear_generic_general_acc(x, w, (7, 8, 1), L, -1, 1, 1, True, False)
        sec_sc = _time(torch, sc_only, 20, 3)
        prof = _profile(torch, sc_only, 5)
        # evaluation: the layer under no_grad keeps its weight bitstreams while the parameter does not change
        from sc_layers import Linear_Or
        layer = Linear_Or(4096, 1024, bias=False, forward="or_2", err=6).to(dev)
        layer.weight.copy_(w)
        sec_eval = _time(torch, lambda: layer(x), 20, 3)
    sec_fb = _time(torch, fwd_bwd, 20, 3)
    mac = 256 * 4096 * 1024
    comp_ms = sum(v["ms"] for k, v in prof.items() if k.startswith("sc_compute"))
    out = {"workload": "SC linear OR-2, 64-bit streams, 256x4096 . (1024x4096)^T; backward through the float surrogate",
           "sc_forward_ms": sec_sc * 1e3, "forward_backward_ms": sec_fb * 1e3,
           "eval_layer_forward_ms": sec_eval * 1e3,   # Linear_Or.forward: quantise input + SC op on cached weight streams + counts to float
           "bit_mac_per_s": mac * L / sec_sc, "samples_per_s_fwd_bwd": 256 / sec_fb,
           "valu_frac": mac * L * 4 / 32 / sec_sc / VALU_PEAK_LANEOPS,
           "sc_compute_valu_frac": mac * L * 4 / 32 / (comp_ms * 1e-3) / VALU_PEAK_LANEOPS if comp_ms else None,
           "kernel_ms": {k: round(v["ms"], 4) for k, v in sorted(prof.items())}}
    return out


def _train_flavours(torch, dev, net, make_batch, batch, steps, lr, only=None):
    """Training steps as utils_own.py:96-171 runs them: sync 1 / 3 / 2 in float32; only="autocast": sync 1 under
    float16 autocast with a gradient scaler instead (the reference's `torch_type != torch.float32` branch,
    :127-131,156-165); only="sync1": the float32 sync-1 flavour alone (for profiler runs)."""
    import torch.nn.functional as F
    opt = torch.optim.Adam(net.parameters(), lr=lr, weight_decay=1e-4)
    only_autocast = only == "autocast"
    scaler = torch.amp.GradScaler("cuda") if only_autocast else None
    out = {}
    flavours = ((("sync1_sc_forward_autocast_fp16", 1, 1.0),) if only_autocast else
                (("sync1_sc_forward", 1, 1.0),) if only == "sync1" else
                (("sync1_sc_forward", 1, 1.0), ("sync3_error_injection", 3, 1.0), ("sync2_calibration_half_batch", 2, 0.5)))
    for name, sync, frac in flavours:
        n = max(1, int(batch * frac))
        x, y = make_batch(n)

        def step():
            net.sync = sync
            opt.zero_grad(set_to_none=True)
            if only_autocast:
                with torch.autocast("cuda", dtype=torch.float16):
                    output = net(x)
                loss = F.cross_entropy(output, y, label_smoothing=0.1)
                scaler.scale(loss).backward()
                scaler.step(opt)
                scaler.update()
                return loss
            loss = F.cross_entropy(net(x), y, label_smoothing=0.1)
            loss.backward()
            opt.step()
            return loss

        # two timed runs of `steps` steps, the faster one reported: on these boxes one step in a few dozen stalls for
        # tens of milliseconds on the host side (seen in any of the three flavours, never in the kernels' own times)
        runs = [_time(torch, step, steps, 2), _time(torch, step, steps, 0)]
        sec = min(runs)
        out[name] = {"ms_per_step": sec * 1e3, "ms_per_step_runs": [r * 1e3 for r in runs], "images_per_s": n / sec,
                     "batch": n}
        out[name].update(_breakdown(_profile(torch, step, 2), sec * 1e3))
    return out


def config3_tinyconv_step(torch, dev, only=None):
    from sc_models import TinyConvSC
    torch.manual_seed(3)
    net = TinyConvSC(forward="or_3", err=6).to(dev)
    g = torch.Generator().manual_seed(3)

    def make_batch(n):
        return (torch.randn(n, 3, 32, 32, generator=g).clamp(-1, 1).to(dev),
                torch.randint(0, 10, (n,), generator=g).to(dev))

    res = _train_flavours(torch, dev, net, make_batch, 256, 10, 8e-3, only)
    res["workload"] = ("TinyConv-style training step, batch 256, 3x32x32, conv3x3 3-32-32-pool-64-64-pool-fc10, "
                       "OR-3, 64-bit streams, Adam")
    return res


def config3_tinyconv_autocast_step(torch, dev):
    return config3_tinyconv_step(torch, dev, only="autocast")


def _rotating_sets(nbytes_per_set):
    return max(2, int(ROTATE_BYTES // max(1, nbytes_per_set)) + 1)


def config4_fixed_conv(torch, dev):
    import _lib
    import fixed_extension_cuda
    import sc_functional as uf
    L_ = _lib.lib()
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    out = {"workload": "saturating fixed-point conv (add_config 0, 5-bit operands, 24-bit accumulator), batch 64, "
                       "conv3x3 s1 p1: forward op alone (one buffer set, and rotating through >1 GiB of distinct "
                       "buffers), and forward + backward through the float conv", "shapes": {}}
    for C, H in ((64, 56), (128, 28), (256, 14), (512, 7)):
        g = torch.Generator().manual_seed(4)
        xc = torch.randint(0, 32, (64, C, H, H), generator=g).float() / 32
        wc = torch.randint(-31, 32, (C, C, 3, 3), generator=g).float() / 32
        x, w = xc.to(dev), wc.to(dev)
        fn = lambda: fixed_extension_cuda.conv2d_saturate_acc(x, w, 0, 5, 24, (1, 1), (1, 1))
        sec = _time(torch, fn, 10, 2)
        nbytes = 4 * x.numel() + 4 * w.numel() + 4 * 64 * C * H * H
        # rotating: distinct input / weight / output / workspace per call, through the C ABI
        d = _lib.FixedDesc(64, C, H, H, C, 3, 3, 1, 1, 1, 1, 0, 5, 24)
        ws_bytes = L_.rexsc_fixed_conv2d_workspace_bytes(ctypes.byref(d))
        nset = _rotating_sets(nbytes)
        sets = [(x.clone(), w.clone(), torch.empty((64, C, H, H), dtype=torch.int32, device=dev)) for _ in range(nset)]
        ws = torch.empty(max(ws_bytes, 256), dtype=torch.uint8, device=dev)
        state = {"i": 0}

        def rot():
            xs, wsx, os_ = sets[state["i"] % nset]
            state["i"] += 1
            _lib.check(L_.rexsc_fixed_conv2d(ctypes.byref(d), ptr(xs), ptr(wsx), ptr(os_), ptr(ws), ws.numel(), stream()),
                       "rexsc_fixed_conv2d")

        sec_rot = _time(torch, rot, 2 * nset, nset)
        prof = _profile(torch, rot, nset)
        del sets
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
        mac = 64 * H * H * C * C * 9
        kern_ms = sum(v["ms"] for v in prof.values())
        entry = {"ms": sec * 1e3, "ms_rotating": sec_rot * 1e3, "rotating_sets": nset,
                 "kernel_ms_rotating": {k: round(v["ms"], 4) for k, v in sorted(prof.items())},
                 "GB_per_s": nbytes / sec_rot / 1e9, "hbm_frac": nbytes / sec_rot / HBM_PEAK,
                 "hbm_frac_kernels_only": nbytes / (kern_ms * 1e-3) / HBM_PEAK if kern_ms else None,
                 "hbm_frac_one_buffer_set": nbytes / sec / HBM_PEAK,
                 "mac_per_s": mac / sec_rot, "images_per_s": 64 / sec_rot, "forward_backward_ms": sec_fb * 1e3,
                 "images_per_s_fwd_bwd": 64 / sec_fb}
        out["shapes"]["%dx%dx%d" % (C, H, H)] = entry
        del x, w, xg, wg
        torch.cuda.empty_cache()
    return out


def config5_resnet18_autocast_step(torch, dev):
    return config5_resnet18_step(torch, dev, only="autocast")


def config5_resnet18_sync1_step(torch, dev):
    return config5_resnet18_step(torch, dev, only="sync1")


def config3_tinyconv_sync1_step(torch, dev):
    return config3_tinyconv_step(torch, dev, only="sync1")


def config5_resnet18_step(torch, dev, batch=64, only=None):
    from sc_models import ResNet18SC
    torch.manual_seed(5)
    net = ResNet18SC(forward="or_2", err=5).to(dev).to(memory_format=torch.channels_last)
    g = torch.Generator().manual_seed(5)

    def make_batch(n):
        return (torch.randn(n, 3, 224, 224, generator=g).to(dev).contiguous(memory_format=torch.channels_last),
                torch.randint(0, 1000, (n,), generator=g).to(dev))

    res = _train_flavours(torch, dev, net, make_batch, batch, 5, 1e-3, only)
    res["workload"] = ("ResNet-18 SC training step, batch %d, 3x224x224, channels_last, OR-2, 32-bit streams, "
                       "float stem/fc, Adam" % batch)
    if only:
        return res
    # evaluation: weights frozen, the layers reuse their weight streams from call to call
    net.eval()
    net.sync = 1
    x, _ = make_batch(batch)
    with torch.no_grad():
        sec = _time(torch, lambda: net(x), 5, 2)
    res["eval_forward_no_grad"] = {"ms": sec * 1e3, "images_per_s": batch / sec}
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
    res = {"workload": "19 ResNet-18 SC conv layers, batch %d, OR-2, 32-bit streams, channels_last: SC forward + "
                       "backward through the float surrogate (conv2d_generic, sync 1)" % batch,
           "ms_per_step": sec * 1e3, "images_per_s": batch / sec}
    res.update(_breakdown(_profile(torch, step, 2), sec * 1e3))
    return res


def pointwise(torch, dev):
    """The streaming kernels on one ResNet-18 layer1 activation tensor, through the C ABI with preallocated
    outputs: on one buffer set, and rotating through more than 1 GiB of distinct inputs and outputs."""
    import _lib
    L_ = _lib.lib()
    n = 64 * 64 * 56 * 56
    outer, inner = 64 * 56 * 56, 64
    coef = torch.tensor([0.01, -0.01, 0.002, 0.0, 0.0, 0.0], device=dev)
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    f32 = lambda k: torch.rand(k, device=dev) * 4
    i16 = lambda k: torch.randint(0, 64, (k,), device=dev, dtype=torch.int16)
    e32 = lambda k: torch.empty(k, dtype=torch.float32, device=dev)
    # name -> (bytes per element of y, buffer makers, call)
    kernels = {
        "orn_forward": (8, lambda: (f32(n), e32(n)),
                        lambda b: L_.rexsc_orn_forward(p(b[0]), p(b[1]), n, 2, stream())),
        "orn_backward": (12, lambda: (f32(n), f32(n), e32(n)),
                         lambda b: L_.rexsc_orn_backward(p(b[0]), p(b[1]), p(b[2]), n, 2, 1, stream())),
        "orn_bias_std_both_forward": (12, lambda: (f32(n), f32(n), e32(n)),
                                      lambda b: L_.rexsc_orn_bias_std_both_forward(p(b[0]), p(b[1]), p(coef), p(coef), p(b[2]), n, 2,
                                                                                   1234, 0, None, None, None, stream())),
        "orn_bias_std_both_backward": (20, lambda: (f32(n), f32(n), f32(n), e32(n), e32(n)),
                                       lambda b: L_.rexsc_orn_bias_std_both_backward(p(b[0]), p(b[1]), p(b[2]), p(coef), p(b[3]),
                                                                                     p(b[4]), n, 2, 1, stream())),
        "orn_pair_backward": (20, lambda: (f32(n), f32(2 * n), e32(2 * n)),
                              lambda b: L_.rexsc_orn_pair_backward(p(b[0]), p(b[1]), p(b[2]), outer, inner, 2, 1, stream())),
        "orn_bias_std_pair_forward": (12, lambda: (f32(2 * n), e32(n)),
                                      lambda b: L_.rexsc_orn_bias_std_pair_forward(p(b[0]), p(coef), p(coef), p(b[1]), outer, inner, 2,
                                                                                   1234, 0, None, stream())),
        "orn_bias_std_pair_backward": (20, lambda: (f32(n), f32(2 * n), e32(2 * n)),
                                       lambda b: L_.rexsc_orn_bias_std_pair_backward(p(b[0]), p(b[1]), p(coef), p(b[2]), outer, inner,
                                                                                     2, 1, stream())),
        "sc_counts_to_float": (8, lambda: (i16(n), i16(n), e32(n)),
                               lambda b: L_.rexsc_sc_counts_to_float(p(b[0]), p(b[1]), p(b[2]), n, 32, stream())),
        "quantize": (8, lambda: (f32(n), e32(n)),
                     lambda b: L_.rexsc_quantize(p(b[0]), p(b[1]), n, 7, stream())),
    }
    res = {"workload": "streaming kernels on %d float32 elements (64x64x56x56); hbm_frac: rotating through >1 GiB of "
                       "distinct buffers; hbm_frac_one_buffer_set: the same buffers every call" % n}
    for name, (bpe, make, call) in kernels.items():
        one = make()
        sec_one = _time(torch, lambda: _lib.check(call(one), name), 20, 3)
        set_bytes = sum(t.numel() * t.element_size() for t in one)
        nset = _rotating_sets(set_bytes)
        sets = [one] + [make() for _ in range(nset - 1)]
        state = {"i": 0}

        def rot():
            b = sets[state["i"] % nset]
            state["i"] += 1
            _lib.check(call(b), name)

        sec = _time(torch, rot, 2 * nset, nset)
        prof = _profile(torch, rot, nset)
        kms = prof.get(name, {}).get("ms")
        res[name] = {"ms": sec * 1e3, "kernel_ms": kms, "rotating_sets": nset, "GB_per_s": bpe * n / sec / 1e9,
                     "hbm_frac": bpe * n / sec / HBM_PEAK,
                     "hbm_frac_kernel_only": bpe * n / (kms * 1e-3) / HBM_PEAK if kms else None,
                     "hbm_frac_one_buffer_set": bpe * n / sec_one / HBM_PEAK}
        del sets, one
        torch.cuda.empty_cache()
    return res


def _in_child_process(name, timeout=240):
    """One function of this file in a process of its own (python bench.py --only-extra NAME), so that whatever happens
    in it cannot take the benchmark's JSON line with it; returns its entry or {"error": ...}."""
    import subprocess
    import sys
    cmd = [sys.executable, os.path.join(os.path.dirname(os.path.abspath(__file__)), "bench.py"), "--only-extra", name]
    try:
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout)
        if proc.returncode != 0:
            return {"error": "exit code %d: %s" % (proc.returncode, proc.stderr.strip()[-300:])}
        return json.loads(proc.stdout.strip().splitlines()[-1])[name]
    except Exception as e:
        return {"error": "%s: %s" % (type(e).__name__, e)}


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
    # the reduced-precision step of both networks: float16 convolutions of the vendor library, searched and compiled
    # per shape on first use -- kept out of this process
    for name, child in (("config3_tinyconv_train", "config3_tinyconv_autocast_step"),
                        ("config5_resnet18_train", "config5_resnet18_autocast_step")):
        res = _in_child_process(child)
        if isinstance(out.get(name), dict) and "error" not in out[name]:
            out[name]["sync1_sc_forward_autocast_fp16"] = res.get("sync1_sc_forward_autocast_fp16", res)
    return out
