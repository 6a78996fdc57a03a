#!/usr/bin/env python3
"""Benchmark of the SC hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extra]

A "step" is one forward pass of all 19 stochastic-computing conv layers of ResNet-18
(16 conv3x3 + 3 conv1x1; resnet_sc.py:33-44,246-271 of the reference) at batch 64, OR-2
accumulation, 32-bit streams, channels_last activations, synthetic operands uniform on the
5-bit quantisation grid -- float operands in HBM in, int16 positive/negative results in HBM out,
i.e. exactly what sc_extension_cuda.conv2d_generic_general_split_acc does for each layer.
The headline value is bit-MAC/s = MAC * stream length / time (one activation bit times one
split-unipolar weight bit-pair counts as one bit-MAC).

The one JSON line printed at the end also carries
  roofline      the dominant kernel (AND/popcount compute) against the VALU integer peak:
                achieved = algorithmic lane-ops / duration measured with HIP events on the launch
                stream, peak = 256 CU x 64 lanes/clk x 2.4 GHz;
  cpu_baseline  the reference's own CPU extension (compiled into oracle/_ref/) on a bounded sample
                of the same workload, timed on this host; the C restatement in oracle/ (OpenMP)
                beside it, and instead of it where the reference build is absent;
  extra         the other reference configurations (SC conv OR-1, SC linear fwd+bwd, fixed-point
                conv, pointwise kernels, training steps), each with its own rate.
"""
import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "rex-sc_amd"))

# Integer VALU roofs (lane-ops/s) at 256 CUs x 4 SIMDs x 2.4 GHz.  Measured per wave64 instruction and SIMD on this
# part (profiles/valu_instruction_rates_gfx950.md): v_and_b32 2 cycles, v_bcnt_u32_b32 / v_and_or_b32 / v_pk_*_u16 4
# cycles.  The and + popcount pair therefore retires in 6 cycles: 2 x 64 lane-ops / 6 cycles per SIMD.
VALU_PEAK_4CYCLE = 256 * 4 * 16 * 2.4e9          # every instruction at 4 cycles: 39.32 T lane-op/s
VALU_PEAK_LANEOPS = 256 * 4 * (2 * 64 / 6) * 2.4e9  # the and + popcount pair: 52.43 T lane-op/s
HBM_PEAK = 8.0e12

# (C_in, H_in, C_out, K, stride) for the 19 SC convs of ResNet-18 at 224x224 input
RESNET18_SC_LAYERS = (
    [(64, 56, 64, 3, 1)] * 4 +
    [(64, 56, 128, 3, 2), (128, 28, 128, 3, 1), (64, 56, 128, 1, 2), (128, 28, 128, 3, 1), (128, 28, 128, 3, 1)] +
    [(128, 28, 256, 3, 2), (256, 14, 256, 3, 1), (128, 28, 256, 1, 2), (256, 14, 256, 3, 1), (256, 14, 256, 3, 1)] +
    [(256, 14, 512, 3, 2), (512, 7, 512, 3, 1), (256, 14, 512, 1, 2), (512, 7, 512, 3, 1), (512, 7, 512, 3, 1)]
)


def layer_macs(N, C, H, O, K, s):
    Ho = (H + 2 * (K // 2) - K) // s + 1
    return N * Ho * Ho * O * C * K * K


def make_conv_operands(torch, N, C, H, O, K, L, seed, channels_last=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randint(0, L, (N, C, H, H), generator=g).float() / L
    w = torch.randint(-L + 1, L, (O, C, K, K), generator=g).float() / L
    return x, w


def time_gpu(torch, fn, steps, warmup):
    """Seconds per call: `warmup` untimed calls, then exactly `steps` calls between two device synchronisations
    (Python's cyclic garbage collector held off meanwhile, as timeit does)."""
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--cpu-sample-batch", type=int, default=64)
    ap.add_argument("--only-layer", default=None, metavar="C,H,O,K,S",
                    help="run a single SC conv layer shape instead of the 19 (for per-kernel counter runs)")
    ap.add_argument("--only-extra", default=None, metavar="NAME",
                    help="run one function of bench_extra.py (e.g. pointwise, config4_fixed_conv) and exit (for profiler runs)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="run three 256 MiB device-to-device copies and exit (scales the rocprofv3 byte counters)")
    ap.add_argument("--valu-probe", action="store_true",
                    help="run the library's register-only VALU probe in all its modes, print the rates and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the SC path has no collectives); use --gpus 1",
              file=sys.stderr)
        return 2

    import torch
    import _lib
    import _ops
    import sc_extension_cuda

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, OR_N, N = 32, 2, args.batch
    if args.copy_probe:
        a = torch.zeros(64 * 1024 * 1024, dtype=torch.float32, device=dev)
        b = torch.empty_like(a)
        for _ in range(3):
            b.copy_(a)
        torch.cuda.synchronize()
        return 0
    _lib.check(_lib.lib().rexsc_init(None), "rexsc_init")
    if args.valu_probe:
        modes = {0: "v_and_b32 (SGPR operand); s_nop 0; v_bcnt_u32_b32 accumulate -- the compute kernel's pair",
                 1: "v_and_or_b32 (SGPR operand) -- the OR-1 form",
                 2: "v_and_b32 (SGPR operand); v_bcnt_u32_b32 accumulate -- the pair without the scalar instruction",
                 3: "v_and_b32, vector registers only", 4: "v_bcnt_u32_b32 accumulate alone"}
        res = {}
        for m, text in modes.items():
            rate = max(_lib.valu_probe(m, 2000) for _ in range(3))
            # cycles one wave64 instruction occupies its SIMD at the nominal 2.4 GHz
            res["mode%d" % m] = {"what": text, "Tlane_op_per_s": rate / 1e12,
                                 "cycles_per_instruction": 256 * 4 * 64 * 2.4e9 / rate}
        print(json.dumps({"valu_probe": res, "device": torch.cuda.get_device_name(0)}))
        return 0
    if args.only_extra:
        import bench_extra
        fn = getattr(bench_extra, args.only_extra, None)  # a function of bench_extra.py, e.g. pointwise
        if not callable(fn) or args.only_extra.startswith("_") or args.only_extra == "run":
            print("bench.py: no configuration named %r in bench_extra.py" % args.only_extra, file=sys.stderr)
            return 2
        print(json.dumps({args.only_extra: fn(torch, dev)}))
        return 0

    shapes = RESNET18_SC_LAYERS
    if args.only_layer:
        shapes = [tuple(int(v) for v in args.only_layer.split(","))]
    layers = []
    for i, (C, H, O, K, s) in enumerate(shapes):
        x, w = make_conv_operands(torch, N, C, H, O, K, L, seed=500 + i)
        layers.append((x.to(dev).contiguous(memory_format=torch.channels_last), w.to(dev), K, s))
    total_mac = sum(layer_macs(N, C, H, O, K, s) for (C, H, O, K, s) in shapes)

    def step():
        """The 19 layers through the reference's own entry point, one call after the other.  (Generating every layer's
        weight bitstreams on a second stream while earlier layers compute -- rexsc_conv2d_prepare_weights -- was
        measured here and lost: 10.43 ms against 10.35, the generators' blocks displace blocks of the VALU-bound
        compute kernel.)"""
        for (x, w, K, s) in layers:
            sc_extension_cuda.conv2d_generic_general_split_acc(
                x, w, L, -1, 16, (K // 2, K // 2), (s, s), (7, 8, 1), OR_N - 1, 1, True, False)

    sec = time_gpu(torch, step, args.steps, args.warmup)
    value = total_mac * L / sec

    # per-kernel durations with HIP events on the launch stream (separate pass: the event
    # bookkeeping is kept out of the headline timing)
    _lib.profile_begin()
    for _ in range(3):
        step()
    prof = _lib.profile_end()
    comp = {k: v for k, v in prof.items() if k.startswith("sc_compute")}
    dom_name = max(comp, key=lambda k: comp[k]["total_ms"])
    dom = comp[dom_name]
    achieved = dom["total_work"] / (dom["total_ms"] * 1e-3)
    comp_ms = sum(v["total_ms"] for v in comp.values())
    comp_ops = sum(v["total_work"] for v in comp.values())
    # what the register-only and/popcount probe kernel sustains on this machine, beside the nominal peak
    peak_measured = max(_lib.valu_probe(0, 2000) for _ in range(2))
    traffic = quoted_traffic()
    roofline = {
        "bound": "valu", "kernel": dom_name,
        "achieved": achieved / 1e12, "peak": VALU_PEAK_LANEOPS / 1e12, "unit": "Tlane-op/s",
        "frac": achieved / VALU_PEAK_LANEOPS,
        "peak_model": "and+popcount pair at its measured instruction costs (v_and_b32 2 cycles + v_bcnt_u32_b32 4 cycles per "
                      "wave64 and SIMD); every instruction at 4 cycles would be %.2f" % (VALU_PEAK_4CYCLE / 1e12),
        "peak_measured": peak_measured / 1e12, "frac_of_peak_measured": achieved / peak_measured,
        "peak_measured_and_or": _lib.valu_probe(1, 2000) / 1e12,
        # HBM bytes per launch of this kernel: quoted from the committed rocprofv3 counter summary (FETCH_SIZE +
        # WRITE_SIZE on one layer shape), not measured in this run; null when the summary is absent
        "traffic": traffic.get("bytes"), "traffic_shape": traffic.get("shape"), "traffic_source": traffic.get("source"),
        "avg_launch_us": dom["total_ms"] * 1e3 / dom["calls"], "launches": dom["calls"],
        "all_compute_kernels_frac": comp_ops / (comp_ms * 1e-3) / VALU_PEAK_LANEOPS,
        "whole_step_frac": (total_mac * L * 4 / 32) / sec / VALU_PEAK_LANEOPS,
        "kernel_ms_per_step": {k: round(v["total_ms"] / 3, 4) for k, v in sorted(prof.items())},
    }

    out = {
        "metric": "sc_bit_mac_per_s", "value": value, "unit": "bit-MAC/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": sec * 1e3,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u32",
        "data": "synthetic",
        "config": {"workload": ("resnet18_sc_conv_forward: 19 SC conv layers (16 3x3 + 3 1x1), batch %d, OR-%d, "
                                "%d-bit streams, channels_last, float in / int16 pos+neg out" % (N, OR_N, L))
                               if not args.only_layer else "single SC conv layer C,H,O,K,S=%s, batch %d" % (args.only_layer, N),
                   "batch": N, "bit_length": L, "or_n": OR_N, "images_per_s": N / sec,
                   "xnor_mode": _ops.xnor_mode()},
        "roofline": roofline,
    }

    # the same step with the stream generators of the reference's CUDA kernels (REXSC_XNOR_MODE=cuda_ref: other
    # sequence tables and seed offsets, the same kernels)
    prev_mode = os.environ.get("REXSC_XNOR_MODE")
    os.environ["REXSC_XNOR_MODE"] = "cuda_ref"
    try:
        sec_xnor = time_gpu(torch, step, max(3, args.steps // 2), 2)
        out["config"]["xnor_mode_cuda_ref"] = {"ms_per_step": sec_xnor * 1e3, "bit_mac_per_s": total_mac * L / sec_xnor,
                                               "relative_to_headline": sec_xnor / sec}
    finally:
        if prev_mode is None:
            os.environ.pop("REXSC_XNOR_MODE", None)
        else:
            os.environ["REXSC_XNOR_MODE"] = prev_mode

    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.cpu_sample_batch, L, OR_N, full_batch=N)
    if not args.no_extra:
        try:
            import bench_extra
            out["extra"] = bench_extra.run(torch, dev)
            if not args.no_cpu_baseline:
                for name, base in cpu_baselines_other_configs(torch).items():
                    target = out["extra"].get(name.split("/")[0], {})
                    if "/" in name:
                        target = target.get("shapes", {}).get(name.split("/")[1], {})
                    if isinstance(target, dict) and "error" not in target:
                        target["cpu_baseline"] = base
        except Exception as e:  # the headline must survive a failure of an auxiliary config
            out["extra"] = {"error": "%s: %s" % (type(e).__name__, e)}
    print(json.dumps(out))
    return 0


def quoted_traffic():
    """HBM bytes per launch of the dominant compute kernel as the committed counter summary states them (a line
    `traffic_bytes_per_launch: <number>` and a line `traffic_shape: <text>`)."""
    import re
    path = os.path.join(ROOT, "profiles", "sc_compute_3x3_c128_hbm_traffic.md")
    try:
        text = open(path).read()
        m = re.search(r"^traffic_bytes_per_launch:\s*([0-9.eE+]+)", text, re.M)
        sh = re.search(r"^traffic_shape:\s*(.+)$", text, re.M)
        if m:
            return {"bytes": float(m.group(1)), "shape": sh.group(1).strip() if sh else None,
                    "source": "profiles/" + os.path.basename(path)}
    except OSError:
        pass
    return {}


_REF_CHILD = r"""
import json, sys, time
sys.path.insert(0, sys.argv[1])
import numpy as np, torch
import sc_extension
layers = json.loads(sys.argv[2]); batch = int(sys.argv[3]); L = int(sys.argv[4]); or_n = int(sys.argv[5])
full = int(sys.argv[6])
ops = []
for i, (C, H, O, K, s) in enumerate(layers):
    g = torch.Generator().manual_seed(500 + i)   # the tensors of the GPU leg, first `batch` images
    x = (torch.randint(0, L, (full, C, H, H), generator=g).float() / L)[:batch]
    w = torch.randint(-L + 1, L, (O, C, K, K), generator=g).float() / L
    ops.append((x.contiguous(memory_format=torch.channels_last), w, K, s))
t0 = time.perf_counter()
for (x, w, K, s) in ops:
    sc_extension.conv2d_generic_general(x, w, L, -1, 16, (K // 2, K // 2), (s, s), (7, 8, 1), or_n - 1, 1, True, False)
print(json.dumps({"sec": time.perf_counter() - t0, "threads": torch.get_num_threads()}))
"""


def cpu_baseline(sample_batch, L, or_n, full_batch=64):
    """CPU rate of the same 19 layers on this host, on a bounded sample (bit-MAC/s scales linearly
    with batch for this embarrassingly parallel op).  Preferred: the reference's own CPU extension,
    compiled from its sources into oracle/_ref/ (kind "reference"), run in a child process so that a
    missing build or an instruction this host lacks cannot take the benchmark down.  Otherwise the C
    restatement in oracle/ (kind "port"), which is also timed and reported as port_value."""
    import subprocess
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import numpy as np
    import oracle as orc
    import torch
    cores = orc.num_threads()
    sample_batch = min(sample_batch, full_batch)
    mac = 0
    sec = 0.0
    for i, (C, H, O, K, s) in enumerate(RESNET18_SC_LAYERS):
        # the same tensors as the GPU leg (same seeds, same generator calls), first sample_batch images
        xt, wt = make_conv_operands(torch, full_batch, C, H, O, K, L, seed=500 + i)
        x, w = xt[:sample_batch].numpy(), wt.numpy()
        t0 = time.perf_counter()
        orc.conv2d_generic_general_split(x, w, L, -1, 16, (K // 2, K // 2), (s, s), (7, 8, 1), or_n - 1, 1,
                                         channels_last_activation=True)
        sec += time.perf_counter() - t0
        mac += layer_macs(sample_batch, C, H, O, K, s)
    port = {"value": mac * L / sec, "unit": "bit-MAC/s", "cores": cores, "kind": "port",
            "sample": "the GPU leg's tensors, same 19 ResNet-18 SC conv layers, first %d images (%.1f s of CPU time on %d threads)"
                      % (sample_batch, sec, cores)}
    ref_dir = os.path.join(ROOT, "oracle", "_ref")
    ref_batch = max(1, sample_batch // 4)
    if not os.path.exists(os.path.join(ref_dir, "sc_extension.so")):
        port["reference_skipped"] = "oracle/_ref/sc_extension.so not built"
        return port
    try:
        out = subprocess.run([sys.executable, "-c", _REF_CHILD, ref_dir, json.dumps(RESNET18_SC_LAYERS), str(ref_batch),
                              str(L), str(or_n), str(full_batch)], capture_output=True, text=True, timeout=180)
        res = json.loads(out.stdout.strip().splitlines()[-1])
        rmac = sum(layer_macs(ref_batch, C, H, O, K, s) for (C, H, O, K, s) in RESNET18_SC_LAYERS)
        return {"value": rmac * L / res["sec"], "unit": "bit-MAC/s", "cores": res["threads"], "kind": "reference",
                "sample": "the GPU leg's tensors, same 19 ResNet-18 SC conv layers, first %d images, through the reference's "
                          "compiled CPU extension (%.1f s on %d threads)" % (ref_batch, res["sec"], res["threads"]),
                "port_value": port["value"], "port_sample": port["sample"]}
    except Exception as e:  # missing build, illegal instruction, timeout: report the port
        port["reference_skipped"] = "%s: %s" % (type(e).__name__, str(e)[:200])
        return port


def cpu_baselines_other_configs(torch):
    """The C restatement in oracle/ (kind "port", OpenMP) on the tensors bench_extra.py builds for configurations 1, 2
    and 4 (same seeds, same generator calls): configurations 1 and 2 at full size, the fixed-point conv on the first two
    images of each shape; configuration 3: its four SC conv layers at full batch on synthetic operands."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    import oracle as orc
    cores = orc.num_threads()
    res = {}
    g = torch.Generator().manual_seed(1)
    x = (torch.randint(0, 32, (32, 32, 32, 32), generator=g).float() / 32).numpy()
    w = ((torch.rand(64, 32, 3, 3, generator=g) * 2 - 1) * 32).round().clamp(-31, 31).div(32).numpy()
    t0 = time.perf_counter()
    orc.conv2d_generic_general_split(x, w, 32, -1, 16, (1, 1), (1, 1), (7, 8, 1), 0, 1)
    sec = time.perf_counter() - t0
    res["config1_sc_conv_or1"] = {"value": 32 * 32 * 32 * 64 * 32 * 9 * 32 / sec, "unit": "bit-MAC/s", "cores": cores,
                                  "kind": "port", "sample": "the same tensors at full size (%.2f s)" % sec}
    g = torch.Generator().manual_seed(2)
    x = (torch.randint(0, 64, (256, 4096), generator=g).float() / 64).numpy()
    w = ((torch.rand(1024, 4096, generator=g) * 2 - 1) * 64).round().clamp(-63, 63).div(64).numpy()
    t0 = time.perf_counter()
    orc.linear_generic_general(x, w, (7, 8, 1), 64, -1, 1, 1)
    sec = time.perf_counter() - t0
    res["config2_sc_linear"] = {"value": 256 * 4096 * 1024 * 64 / sec, "unit": "bit-MAC/s", "cores": cores, "kind": "port",
                                "sample": "the same tensors at full size (%.2f s)" % sec}
    # configuration 3: the four SC conv layers of the TinyConv net (OR-3, 64-bit streams) at its batch of 256, on
    # synthetic operands of the layers' shapes (the net's own activations exist only inside its forward pass)
    g = torch.Generator().manual_seed(3)
    sec = 0.0
    for C, H, O in ((3, 32, 32), (32, 32, 32), (32, 16, 64), (64, 16, 64)):
        x = (torch.randint(0, 64, (256, C, H, H), generator=g).float() / 64).numpy()
        w = ((torch.randn(O, C, 3, 3, generator=g) * (2.0 / (O * 9)) ** 0.5) * 64).round().clamp(-63, 63).div(64).numpy()
        t0 = time.perf_counter()
        orc.conv2d_generic_general_split(x, w, 64, -1, 16, (1, 1), (1, 1), (7, 8, 1), 2, 1)
        sec += time.perf_counter() - t0
    res["config3_tinyconv_train"] = {
        "value": 256 / sec, "unit": "images/s", "cores": cores, "kind": "port",
        "sample": "the SC forward of the net's four SC conv layers alone (3-32-32 at 32x32, 32-64-64 at 16x16; OR-3, "
                  "64-bit streams), batch 256, synthetic operands of the layers' shapes (%.2f s)" % sec}
    for C, H in ((64, 56), (128, 28), (256, 14), (512, 7)):
        g = torch.Generator().manual_seed(4)
        x = (torch.randint(0, 32, (64, C, H, H), generator=g).float() / 32)[:2].numpy()
        w = (torch.randint(-31, 32, (C, C, 3, 3), generator=g).float() / 32).numpy()
        t0 = time.perf_counter()
        orc.conv2d_saturate(x, w, 0, 5, 24, (1, 1), (1, 1))
        sec = time.perf_counter() - t0
        res["config4_fixed_conv/%dx%dx%d" % (C, H, H)] = {
            "value": 2 / sec, "unit": "images/s", "cores": cores, "kind": "port",
            "sample": "the first 2 images of the same tensors (%.2f s)" % sec}
    return res


if __name__ == "__main__":
    sys.exit(main())
