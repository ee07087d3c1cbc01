#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME]

Default (the line the headline metric is quoted on): APRConv 3x3x3 forward, Cin = Cout = 32, fp32, on the APR of
the seeded 512 x 512 x 256 blob volume (BASELINE.json configs[1], ``--config blobs512``) as ``value``; ``extra`` carries
the second half of the metric, the forward latency of the 4-level APR-UNet on the APR of the whole 1024^3 volume
(configs[3], ``apr_unet_1024_*``, fp32 and bfloat16), the same network on the configs[1] APR
(``apr_unet_blobs512_*``), and the results of configs[2] and configs[4], whose full lines go to stderr.  The other
BASELINE configurations are also selected by name and print one JSON line each, with the measured particle count per
level:

  spheres128   configs[0]  APRConv 3x3x3 1 -> 16 fp32 forward with bias on the 128^3 volume          (HBM-bound)
  blobs512     configs[1]  APRConv 3x3x3 32 -> 32 fp32 forward (+ --chain: conv -> ReLU -> pool -> upsample, fwd + bwd)
  nuclei2048   configs[2]  tree fill + APRConv 3x3x3 16 -> 16 fp32 forward on the 2048 x 2048 x 512 volume
  nuclei1024   configs[3]  4-level APR-UNet forward, fp32 and bfloat16 features, on the 1024^3 volume
  spots16k     configs[4]  APRConv 1x5x5 64 -> 64, bfloat16 features, forward + backward, 16384^2 image

A step is one pass of the configuration's operator(s) over device-resident features.  ``value`` is particles/s of
the whole step (latency in ms for the network); ``roofline`` prices the dominant kernel alone (its duration is
measured with HIP events recorded around the launch on its own stream, see aprnet_profile_enable in
include/aprnet_hip.h); ``cpu_baseline`` times the CPU oracle (a restatement of the reference's OpenMP code) on a
bounded sample of the same workload: one warm-up run, then the median of five, with one thread and with all cores.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "apr-cnn_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_BF16_MATRIX_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
# HBM-side bytes of one launch of the convolution kernel on the default workload: FETCH_SIZE + WRITE_SIZE of two
# profiler passes, scaled by what the same counters read for a device-to-device copy of known size
# (profiles/conv333_fwd_32x32_f32_blobs512_hbm_traffic.txt).  Counters cannot be read from inside this script: the
# figure is a constant taken from that profile and only reported when the workload is the one it was measured on.
PROFILED_TRAFFIC_BYTES = {23245996: 27.18e9 + 3.91e9}


# ------------------------------------------------------------------------------------------------ workloads
def build_volume(name):
    from pyapr.synthetic import CONFIGS, synth_volume
    shape, kind, n, axes, amp, bg, iso, _rel = CONFIGS[name]
    return synth_volume(shape, 0, kind, n, axes, amp, bg, iso)


def centre_crop(img, crop):
    import numpy as np
    sl = []
    for s, c in zip(img.shape, crop):
        c = min(c, s)
        a = (s - c) // 2
        sl.append(slice(a, a + c))
    return np.ascontiguousarray(img[tuple(sl)])


def build_workload(name, crop=None, img=None, with_parts=False):
    """APR of a named configuration (optionally of a centre crop of its volume)."""
    from pyapr.synthetic import CONFIGS, pipeline_parameters
    from pyapr.converter import get_apr
    if img is None:
        img = build_volume(name)
    if crop is not None:
        img = centre_crop(img, crop)
    apr, parts = get_apr(img, params=pipeline_parameters(CONFIGS[name][7]))
    return (apr, parts) if with_parts else apr


def level_counts(apr):
    it, tr = apr.iterator(), apr.tree_iterator()
    out = {"particles": {}, "tree_nodes": {}}
    for l in range(it.level_min(), it.level_max() + 1):
        out["particles"][str(l)] = it.particles_level_end(l) - it.particles_level_begin(l)
    for l in range(tr.level_min(), tr.level_max() + 1):
        out["tree_nodes"][str(l)] = tr.particles_level_end(l) - tr.particles_level_begin(l)
    return out


def say(msg):
    """Progress line on stderr (long configurations would otherwise be silent for minutes)."""
    print("# " + msg, file=sys.stderr, flush=True)


def host_cores():
    return int(os.environ.get("OMP_NUM_THREADS", 0)) or len(os.sched_getaffinity(0))


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline_conv(apr, cin, cout, ksize, nstencils, sample, budget_s=25.0):
    """The CPU oracle (port of pyapr/aprnet/src/conv.hpp + helpers.hpp, OpenMP over z) on `apr`: weight expansion +
    convolution forward, output allocation excluded.  1 warm-up + median of five, with one thread and with all cores.
    When one single-thread run is longer than a fifth of the budget, fewer runs are taken and the line says so."""
    import torch
    from oracle import oracle
    n = apr.total_number_particles()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, cin, n, generator=g)
    w = torch.randn(cin, nstencils, cout, *ksize, generator=g) * 0.1
    ld = torch.zeros(1, dtype=torch.int32)
    levels = apr.level_max() - apr.level_min() + 1

    def run():
        oracle.conv_forward([apr], x, oracle.restrict_kernel_forward(w, levels), ld)

    cores = host_cores()
    res = {}
    for threads in (cores, 1):
        before = oracle.set_threads(threads)
        say(f"cpu baseline: {n} particles on {threads} thread(s)")
        t0 = time.perf_counter()
        run()                                       # warm-up, also sizes the number of timed runs
        first = time.perf_counter() - t0
        runs = 5 if first * 6 < budget_s else (3 if first * 4 < budget_s else (1 if first * 2 < budget_s else 0))
        ts = []
        for _ in range(runs):
            t0 = time.perf_counter()
            run()
            ts.append(time.perf_counter() - t0)
        oracle.set_threads(before)
        # a run too long for the budget is its own (un-warmed) measurement
        res[threads] = (statistics.median(ts), f"1 warm-up + median of {runs}") if runs else (first, "one run without warm-up")
    t_all, r_all = res[cores]
    t_one, r_one = res[1]
    return {"value": n / t_all, "unit": "particles/s", "cores": cores, "kind": "port",
            "value_1_thread": n / t_one, "cpu": cpu_model(),
            "sample": f"{sample}, {n} particles, conv {ksize[0]}x{ksize[1]}x{ksize[2]} {cin}->{cout} fp32 forward incl. weight "
                      f"expansion; {cores} threads: {r_all}, {t_all:.2f} s per run; 1 thread: {r_one}, {t_one:.2f} s per run"}


def _time(fn, iters=10, warmup=2):
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def _steps(fn, steps, warmup):
    """The timed region of the contract: W untimed steps, then exactly K steps between two synchronisations."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def _kernel_ms(lib, fn, repeats):
    """Average duration of the convolution kernel inside fn(): HIP events around its launch, on its stream."""
    lib.aprnet_profile_enable(1)
    kms = []
    for _ in range(repeats):
        fn()
        kms.append(float(lib.aprnet_profile_last_ms()))
    lib.aprnet_profile_enable(0)
    return sum(kms) / len(kms)


def make_unet(dev):
    import torch
    from apr_models.unet import APRUNet, fold_norms
    torch.manual_seed(0)
    net = APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch")
    for m in net.modules():                          # He initialisation of the convolution weights, seed 0
        if hasattr(m, "weight") and getattr(m, "weight") is not None and m.weight.dim() == 6:
            fan_in = m.weight.shape[2] * m.weight.shape[3] * m.weight.shape[4] * m.weight.shape[5]
            torch.nn.init.normal_(m.weight, 0.0, (2.0 / fan_in) ** 0.5)
    return fold_norms(net.eval()).to(dev)


def base_line(metric, value, unit, args, ms_per_step, dtype, config, higher=True):
    return {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": ms_per_step, "higher_is_better": higher, "scaling": "weak", "vs_baseline": None,
            "dtype": dtype, "data": "synthetic", "config": config}


def mfma_roofline(flop, kernel_ms, peak, kernel, hbm_bytes, traffic=None):
    tflops = flop / (kernel_ms * 1e-3) / 1e12
    gbs = hbm_bytes / (kernel_ms * 1e-3) / 1e9
    return {"bound": "mfma", "achieved": tflops, "peak": peak, "unit": "TFLOP/s", "frac": tflops / peak,
            "traffic": traffic, "traffic_source": "constant from the committed profiler summary, not read in this run" if traffic else None,
            "kernel": kernel, "kernel_ms": kernel_ms, "hbm_achieved_GBs": gbs, "hbm_frac": gbs / PEAK_HBM_GBS}


def hbm_roofline(nbytes, kernel_ms, kernel, flop=None):
    gbs = nbytes / (kernel_ms * 1e-3) / 1e9
    out = {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": gbs / PEAK_HBM_GBS, "traffic": None,
           "kernel": kernel, "kernel_ms": kernel_ms}
    if flop is not None:
        out["fp32_TFLOPs"] = flop / (kernel_ms * 1e-3) / 1e12
    return out


# ------------------------------------------------------------------------------------------------ configs
def run_blobs512(args, dev, lib):
    """configs[1]: the 32 -> 32 layer (headline metric) and the APR-UNet forward latency on the same APR."""
    import torch
    from pyapr import aprnet
    CIN, COUT = args.channels
    flop_pp, bytes_pp = 2 * 27 * CIN * COUT, 4 * (CIN + COUT) + 2
    nstencils = 2
    t0 = time.perf_counter()
    img = build_volume("blobs512")
    apr = build_workload("blobs512", img=img)
    t_build = time.perf_counter() - t0
    t0 = time.perf_counter()
    apr.init_cuda()
    t_plan = time.perf_counter() - t0
    n = apr.total_number_particles()
    bf16 = args.features in ("bf16", "bf16g")
    torch.manual_seed(0)
    x = torch.randn(1, CIN, n, device=dev)
    if bf16:
        x = x.to(torch.bfloat16)
    conv = aprnet.cuda.APRConv(CIN, COUT, nstencils=nstencils, kernel_size=(3, 3, 3), bias=True).to(dev)
    ld = torch.zeros(1, dtype=torch.int32)
    if args.features == "bf16g":
        # the same layer between two layers of a network that keeps its tensors grouped by eight channels
        from pyapr.aprnet import _ops, grouped
        xg = grouped.regroup(x)
        levels = apr.level_max() - apr.level_min() + 1

        def step():
            return grouped.conv_forward([apr], xg, _ops.restrict_kernel_forward(conv.weight.detach(), levels), ld, conv.bias.detach())
    else:
        def step():
            return conv(x, [apr], ld)
    e = 2 if bf16 else 4
    if args.backward:
        # the backward pass of the same layer (input and weight gradient) as the timed step: the call a profiler run traces
        if args.features == "bf16g":
            sys.exit("bench.py: --backward runs on channel planes (--features f32 or bf16)")
        xg = x.clone().requires_grad_(True)
        yb = conv(xg, [apr], ld)
        go = torch.randn_like(yb)

        def bstep():
            return torch.autograd.grad(yb, (xg, conv.weight, conv.bias), go, retain_graph=True)
        sec = _steps(bstep, args.steps, args.warmup)
        out = base_line(f"APRConv 3x3x3 bwd particles/s (Cin={CIN}, Cout={COUT})", n / sec, "particles/s", args, sec * 1e3,
                        "bf16" if bf16 else "f32",
                        {"workload": f"APRConv 3x3x3 {CIN}->{COUT} {'bf16' if bf16 else 'fp32'} backward (input, weight and bias gradient, "
                                     "tree-fill and restriction backward), batch 1, blobs512 APR", "n_particles": n})
        out["roofline"] = mfma_roofline(2 * flop_pp * n, sec * 1e3, PEAK_BF16_MATRIX_TFLOPS if bf16 else PEAK_FP32_MATRIX_TFLOPS,
                                        "whole backward call (input-gradient and weight-gradient kernels on two streams)",
                                        (e * 2 * (CIN + COUT)) * n)
        if args.calibrate_copy:
            torch.empty_like(x).copy_(x)
            torch.cuda.synchronize()
        return out
    with torch.no_grad():
        sec = _steps(step, args.steps, args.warmup)
        kernel_ms = _kernel_ms(lib, step, args.steps)
        y = step()
    y = y.data if args.features == "bf16g" else y
    assert torch.isfinite(y.float()).all()
    del y
    metric = "APRConv 3x3x3 fwd particles/s (Cin=Cout=32) + APR-UNet fwd latency, 1 GPU"
    if (CIN, COUT) != (32, 32):
        metric = f"APRConv 3x3x3 fwd particles/s (Cin={CIN}, Cout={COUT})"
    out = base_line(metric, n / sec, "particles/s", args,
                    sec * 1e3, "bf16" if bf16 else "f32",
                    {"workload": f"APRConv 3x3x3 {CIN}->{COUT} {'bf16' if bf16 else 'fp32'} forward (restrict + tree fill + conv + bias"
                                 f"{', input and output grouped by eight channels' if args.features == 'bf16g' else ''}), batch 1, "
                                 "APR of the seeded 512x512x256 volume with 2000 ellipsoidal blobs (configs[1]); extra: 4-level "
                                 "APR-UNet forward on the same APR",
                     "n_particles": n, "levels": level_counts(apr), "nstencils": nstencils, "level_max": apr.level_max(),
                     "apr_build_s": round(t_build, 2), "plan_create_s": round(t_plan, 2)})
    peak = PEAK_BF16_MATRIX_TFLOPS if bf16 else PEAK_FP32_MATRIX_TFLOPS
    alg_bytes = (e * (CIN + COUT) + 2) * n
    if flop_pp / (e * (CIN + COUT) + 2) < peak * 1e12 / (PEAK_HBM_GBS * 1e9):      # fewer flops per byte than the machine: HBM bounds it
        out["roofline"] = hbm_roofline(alg_bytes, kernel_ms, "conv_narrow_kernel" if CIN <= 3 else "conv kernel", flop_pp * n)
    else:
        out["roofline"] = mfma_roofline(flop_pp * n, kernel_ms, peak, "conv_mfma_bf16_kernel" if bf16 else "conv_mfma16_kernel",
                                        alg_bytes, None if bf16 or (CIN, COUT) != (32, 32) else PROFILED_TRAFFIC_BYTES.get(n))
    if not args.no_extra:                  # (profiler runs pass --no-extra: the convolution step only)
        # second half of the metric: forward latency of the 4-level network (16-32-64-128, norms folded) on this APR
        net = make_unet(dev)
        xin = x[:, :1].float().contiguous()
        extra = {"apr_unet_blobs512_n_particles": n}
        with torch.no_grad():
            # (the network on the configs[1] APR; the latency on the configs[3] APR, the one the metric names, is added
            # to this dictionary by main() as apr_unet_1024_*)
            net.prepare_inference([apr])
            extra["apr_unet_blobs512_fwd_ms_f32"] = _time(lambda: net(xin, [apr]), iters=5, warmup=2)
            xinb = xin.to(torch.bfloat16)
            extra["apr_unet_blobs512_fwd_ms_bf16"] = _time(lambda: net(xinb, [apr]), iters=5, warmup=2)
            # the narrow first layer of the network (1 -> 16 with bias and ReLU folded in): bound by HBM, 68 bytes per particle
            first = net.encoder[0].blocks[0].conv
            k1 = _kernel_ms(lib, lambda: first.forward_fused(xin, [apr], ld, relu=True), 5)
            extra["conv333_1to16_kernel_ms"] = k1
            extra["conv333_1to16_hbm_frac"] = 68 * n / (k1 * 1e-3) / 1e9 / PEAK_HBM_GBS
        out["extra"] = extra
    if args.calibrate_copy:
        torch.empty_like(x).copy_(x)
        torch.cuda.synchronize()
        print(json.dumps({"calibration_copy_bytes_read": x.numel() * e, "calibration_copy_bytes_written": x.numel() * e}),
              file=sys.stderr, flush=True)
    if args.chain:
        print(json.dumps(chain_step(apr, x.float(), dev)), file=sys.stderr, flush=True)
    if args.ops or args.ops_mem:
        for line in memory_ops(apr, x.float() if bf16 else x, dev):
            print(json.dumps(line), file=sys.stderr, flush=True)
    if args.ops:
        for line in other_ops(apr, x.float() if bf16 else x, dev):
            print(json.dumps(line), file=sys.stderr, flush=True)
    if not args.no_cpu_baseline:
        crop = (128, 256, 256)
        out["cpu_baseline"] = cpu_baseline_conv(build_workload("blobs512", crop=crop, img=img), CIN, COUT, (3, 3, 3), nstencils,
                                                f"centre crop {crop[0]}x{crop[1]}x{crop[2]} of the 256x512x512 volume")
    return out


def chain_step(apr, x, dev):
    """configs[1] in full: APRConv(32 -> 32) -> ReLU -> MaxPool -> UpSampleConst, forward + backward (dX, dW)."""
    import torch
    from pyapr import aprnet
    C = x.shape[1]
    conv = aprnet.cuda.APRConv(C, C, nstencils=2).to(dev)
    pool, up = aprnet.cuda.MaxPool(), aprnet.cuda.UpSampleConst()
    xg = x.clone().requires_grad_(True)
    n = x.shape[2]

    def step():
        ld = torch.zeros(1, dtype=torch.int32)
        xg.grad = None
        conv.weight.grad = None
        u = up(pool(torch.relu(conv(xg, [apr], ld)), [apr], ld), [apr], ld)
        u.backward(torch.ones_like(u))
    ms = _time(step, iters=3, warmup=1)
    return {"op": "chain_conv_relu_pool_upsample_fwd_bwd", "ms": ms, "particles_per_s": n / ms * 1e3,
            "note": f"configs[1] chain, {C}->{C} fp32, forward + backward (grad input, grad weight)"}


def spheres128_inputs():
    """configs[0]: the APR of the 128^3 sphere volume, its sampled intensities as the one input channel, and the
    seeded layer (weights N(0, 0.1), seed 0, one stencil, bias)."""
    import torch
    apr, parts = build_workload("spheres128", with_parts=True)
    x = (torch.from_numpy(parts).float() / 1000.0).view(1, 1, -1).contiguous()
    g = torch.Generator().manual_seed(0)
    w = torch.randn(1, 16, 1, 3, 3, 3, generator=g) * 0.1           # device layout [S, Cout, Cin, kz, kx, ky]
    b = torch.randn(16, generator=g) * 0.1
    return apr, x, w, b


def run_spheres128(args, dev, lib):
    import torch
    from pyapr.aprnet import _ops
    apr, x, w, b = spheres128_inputs()
    apr.init_cuda()
    n = apr.total_number_particles()
    levels = apr.level_max() - apr.level_min() + 1
    xd, wd, bd = x.to(dev), w.to(dev), b.to(dev)
    ld = torch.zeros(1, dtype=torch.int32)

    def step():
        return _ops.conv_forward([apr], xd, _ops.restrict_kernel_forward(wd, levels), ld, bias=bd)
    with torch.no_grad():
        sec = _steps(step, args.steps, args.warmup)
        kernel_ms = _kernel_ms(lib, step, args.steps)
        y = step()
    out = base_line("APRConv 3x3x3 fwd particles/s (Cin=1, Cout=16)", n / sec, "particles/s", args, sec * 1e3, "f32",
                    {"workload": "APRConv 3x3x3 1->16 fp32 forward with bias, batch 1, APR of the seeded 128^3 volume with 200 Gaussian "
                                 "spheres (configs[0]); the launch is too small to fill the GPU: the same layer shape on the "
                                 "23 M-particle APR is in the default line's extra",
                     "n_particles": n, "levels": level_counts(apr), "nstencils": 1, "level_max": apr.level_max()})
    out["roofline"] = hbm_roofline(68 * n, kernel_ms, "conv_narrow_kernel", flop=864 * n)
    # cross-machine golden check of this configuration (tests/golden/spheres128_conv_1to16.json)
    gold = os.path.join(ROOT, "tests", "golden", "spheres128_conv_1to16.json")
    if os.path.exists(gold):
        ref = json.load(open(gold))
        yc = y[0].cpu().double()
        scale = max(abs(v) for v in ref["abs_max"])
        ok = ref["n_particles"] == n
        for c in range(16):
            ok = ok and abs(float(yc[c].sum()) - ref["sum"][c]) <= 1e-5 * scale * n
            ok = ok and max(abs(a - r) for a, r in zip(yc[c, :64].tolist(), ref["first64"][c])) <= 1e-5 * scale
            ok = ok and max(abs(a - r) for a, r in zip(yc[c, -64:].tolist(), ref["last64"][c])) <= 1e-5 * scale
        out["config"]["golden_check"] = "ok" if ok else "MISMATCH"
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_conv(apr, 1, 16, (3, 3, 3), 1, "the whole configuration (128^3 volume)")
    return out


def _largest_apr(name, img, limit=(1 << 30) - 1):
    say(f"{name}: volume {img.shape} synthesised, building the APR")
    """The APR of the whole volume when it stays within the particle limit of a plan, otherwise of the largest
    centre crop (halving z, then x, then y) that does.  -> (apr, description)."""
    import numpy as np
    crop = list(img.shape)
    axis = 0
    while True:
        apr = build_workload(name, crop=tuple(crop) if tuple(crop) != img.shape else None, img=img)
        if apr.total_number_particles() <= limit:
            desc = "whole volume" if tuple(crop) == img.shape else f"centre crop {crop[0]}x{crop[1]}x{crop[2]} (the whole volume exceeds 2^30 particles)"
            return apr, desc
        while crop[axis % 3] <= 1:
            axis += 1
        crop[axis % 3] //= 2
        axis += 1


def run_nuclei2048(args, dev, lib):
    """configs[2]: bottom-up tree fill, then a 3x3x3 convolution that reads tree parents, 16 channels fp32."""
    import torch
    from pyapr import aprnet
    from pyapr.aprnet import _ops
    C = 16
    t0 = time.perf_counter()
    say("nuclei2048: synthesising the 512x2048x2048 volume")
    img = build_volume("nuclei2048")
    apr, what = _largest_apr("nuclei2048", img)
    t_build = time.perf_counter() - t0
    apr.init_cuda()
    n, nt = apr.total_number_particles(), _ops.tree_parts(apr, 0)
    say(f"nuclei2048: {n} particles ({what}), {nt} tree nodes, built in {t_build:.0f} s")
    torch.manual_seed(0)
    x = torch.randn(1, C, n, device=dev)
    conv = aprnet.cuda.APRConv(C, C, nstencils=2).to(dev)
    ld = torch.zeros(1, dtype=torch.int32)
    with torch.no_grad():
        sec = _steps(lambda: conv(x, [apr], ld), args.steps, args.warmup)
        kernel_ms = _kernel_ms(lib, lambda: conv(x, [apr], ld), min(args.steps, 5))
        tree = torch.empty(C, max(nt, 1), device=dev)
        plan, st = apr.plan(0), torch.cuda.current_stream().cuda_stream
        fill_ms = _time(lambda: lib.aprnet_fill_tree_mean_f32(plan, 0, x.data_ptr(), n, C, tree.data_ptr(), tree.shape[1], st), iters=5)
    out = base_line("tree fill + APRConv 3x3x3 fwd particles/s (16 ch fp32)", n / sec, "particles/s", args, sec * 1e3, "f32",
                    {"workload": f"tree fill (mean of children) + APRConv 3x3x3 16->16 fp32 forward reading tree parents, batch 1, APR of the "
                                 f"seeded 2048x2048x512 nuclei volume (configs[2]), {what}",
                     "n_particles": n, "tree_nodes": nt, "levels": level_counts(apr), "apr_build_s": round(t_build, 1)})
    out["roofline"] = mfma_roofline(2 * 27 * C * C * n, kernel_ms, PEAK_FP32_MATRIX_TFLOPS, "conv_mfma16_kernel", (8 * C + 2) * n)
    fill_bytes = 4 * C * (n + 2 * nt)
    out["extra"] = {"fill_tree_mean_ms": fill_ms, "fill_tree_mean_GBs": fill_bytes / fill_ms / 1e6,
                    "fill_tree_mean_hbm_frac": fill_bytes / fill_ms / 1e6 / PEAK_HBM_GBS,
                    "fill_tree_mean_algorithmic_bytes": fill_bytes}
    if not args.no_cpu_baseline:
        crop = (128, 256, 256)
        out["cpu_baseline"] = cpu_baseline_conv(build_workload("nuclei2048", crop=crop, img=img), C, C, (3, 3, 3), 2,
                                                f"centre crop {crop[0]}x{crop[1]}x{crop[2]} of the 512x2048x2048 volume")
    return out


def run_nuclei1024(args, dev, lib):
    """configs[3]: forward of the 4-level APR-UNet (16-32-64-128, norms folded, He init seed 0), fp32 and bfloat16."""
    import torch
    t0 = time.perf_counter()
    say("nuclei1024: synthesising the 1024^3 volume")
    img = build_volume("nuclei1024")
    apr, what = _largest_apr("nuclei1024", img)
    t_build = time.perf_counter() - t0
    apr.init_cuda()
    n = apr.total_number_particles()
    say(f"nuclei1024: {n} particles ({what}), built in {t_build:.0f} s")
    parts = torch.randn(1, 1, n, device=dev)
    net = make_unet(dev).prepare_inference([apr])
    res = {}
    with torch.no_grad():
        for name, xin in (("bf16", parts.to(torch.bfloat16)), ("f32", parts)):
            try:
                torch.cuda.reset_peak_memory_stats()
                sec = _steps(lambda: net(xin, [apr]), max(1, min(args.steps, 3)), 1)
                y = net(xin, [apr])
                assert torch.isfinite(y.float()).all()
                res[name] = {"ms": sec * 1e3, "peak_device_GB": torch.cuda.max_memory_allocated() / 1e9}
                del y
            except RuntimeError as e:           # torch.OutOfMemoryError, or a failed allocation inside the library
                res[name] = {"ms": None, "error": str(e).split("\n")[0][:200]}
            torch.cuda.empty_cache()
            say(f"nuclei1024 {name}: {res[name]}")
    ms = res["bf16"]["ms"] or res["f32"]["ms"]
    out = base_line("APR-UNet fwd latency (ms), 4 levels 16-32-64-128", ms, "ms", args, ms, "bf16",
                    {"workload": f"APR-UNet forward, 4 levels 16-32-64-128, two 3x3x3 convolutions + ReLU per level, norms folded, 1x1x1 head "
                                 f"to 3 classes, batch 1, APR of the seeded 1024^3 nuclei volume (configs[3]), {what}",
                     "n_particles": n, "levels": level_counts(apr), "apr_build_s": round(t_build, 1)}, higher=False)
    out["steps"] = max(1, min(args.steps, 3))
    out["warmup"] = 1
    out["extra"] = {"apr_unet_fwd_bf16": res["bf16"], "apr_unet_fwd_f32": res["f32"],
                    "particles_per_s_bf16": n / res["bf16"]["ms"] * 1e3 if res["bf16"]["ms"] else None}
    out["roofline"] = None
    return out


def run_spots16k(args, dev, lib):
    """configs[4]: APRConv 1x5x5 64 -> 64, bfloat16 features with fp32 accumulation, forward + backward."""
    import torch
    from pyapr import aprnet
    C = 64
    t0 = time.perf_counter()
    img = build_volume("spots16k")
    apr = build_workload("spots16k", img=img)
    t_build = time.perf_counter() - t0
    apr.init_cuda()
    n = apr.total_number_particles()
    say(f"spots16k: {n} particles, built in {t_build:.0f} s")
    conv = aprnet.cuda.APRConv(C, C, nstencils=2, kernel_size=(1, 5, 5)).to(dev)
    ld = torch.zeros(1, dtype=torch.int32)
    x = torch.randn(1, C, n, device=dev).to(torch.bfloat16)
    steps = max(1, min(args.steps, 5))
    with torch.no_grad():
        sec = _steps(lambda: conv(x, [apr], ld), steps, 1)
        kernel_ms = _kernel_ms(lib, lambda: conv(x, [apr], ld), 3)
    extra = {"fwd_ms": sec * 1e3, "fwd_peak_device_GB": torch.cuda.max_memory_allocated() / 1e9}
    say(f"spots16k forward: {sec * 1e3:.1f} ms per step, kernel {kernel_ms:.1f} ms")
    # the same layer between two layers of a network that keeps its tensors grouped by eight channels: no regrouping
    # pass per call, 8-byte output stores instead of 2-byte ones
    try:
        from pyapr.aprnet import _ops, grouped
        xg8 = grouped.regroup(x)
        levels = apr.level_max() - apr.level_min() + 1
        with torch.no_grad():
            gstep = lambda: grouped.conv_forward([apr], xg8, _ops.restrict_kernel_forward(conv.weight.detach(), levels), ld, conv.bias.detach())
            gsec = _steps(gstep, steps, 1)
            gk = _kernel_ms(lib, gstep, 3)
        extra["fwd_grouped_ms"] = gsec * 1e3
        extra["fwd_grouped_kernel_ms"] = gk
        extra["fwd_grouped_frac_of_bf16_matrix_peak"] = 2 * 25 * C * C * n / (gk * 1e-3) / 1e12 / PEAK_BF16_MATRIX_TFLOPS
        say(f"spots16k forward on grouped tensors: {gsec * 1e3:.1f} ms per step, kernel {gk:.1f} ms")
        del xg8
        torch.cuda.empty_cache()
    except RuntimeError as err:                 # out of device memory, or the grouped layout's size limit
        extra["fwd_grouped_ms"] = None
        extra["fwd_grouped_note"] = str(err).splitlines()[0][:200]
        torch.cuda.empty_cache()
    # the backward of the layer at full size needs the features, two gradients and an fp32 gradient work space at
    # 64 channels: run when it fits, otherwise on the 4096^2 corner of the same image
    try:
        xg = x.requires_grad_(True)
        y = conv(xg, [apr], ld)
        go = torch.randn_like(y)
        extra["bwd_ms"] = _time(lambda: torch.autograd.grad(y, (xg, conv.weight), go, retain_graph=True), iters=2, warmup=1)
        extra["bwd_sample"] = "whole image"
        say(f"spots16k backward (whole image): {extra['bwd_ms']:.1f} ms")
        del y, go
    except RuntimeError:                        # out of device memory
        xg = y = go = None
        torch.cuda.empty_cache()
        say("spots16k backward does not fit at full size: 4096^2 crop")
        small = build_workload("spots16k", crop=(1, 4096, 4096), img=img)
        ns = small.total_number_particles()
        xs = torch.randn(1, C, ns, device=dev).to(torch.bfloat16).requires_grad_(True)
        ys = conv(xs, [small], ld)
        gs = torch.randn_like(ys)
        extra["bwd_ms"] = _time(lambda: torch.autograd.grad(ys, (xs, conv.weight), gs, retain_graph=True), iters=2, warmup=1)
        extra["bwd_sample"] = f"centre crop 4096x4096 ({ns} particles): the whole image's backward does not fit the device"
    out = base_line("APRConv 1x5x5 fwd particles/s (Cin=Cout=64, bf16)", n / sec, "particles/s", args, sec * 1e3, "bf16",
                    {"workload": "APRConv 1x5x5 64->64 forward, bfloat16 features, fp32 accumulation, batch 1, APR of the seeded 16384^2 "
                                 "image with 1M Gaussian spots (configs[4]); backward in extra",
                     "n_particles": n, "levels": level_counts(apr), "apr_build_s": round(t_build, 1)})
    out["steps"], out["warmup"] = steps, 1
    out["roofline"] = mfma_roofline(2 * 25 * C * C * n, kernel_ms, PEAK_BF16_MATRIX_TFLOPS, "conv_mfma_bf16_kernel", (2 * 2 * C + 2) * n)
    out["extra"] = extra
    if not args.no_cpu_baseline:
        crop = (1, 1024, 1024)
        out["cpu_baseline"] = cpu_baseline_conv(build_workload("spots16k", crop=crop, img=img), C, C, (1, 5, 5), 2,
                                                "centre crop 1024x1024 of the 16384^2 image")
    return out


def memory_ops(apr, x, dev):
    """Memory-bound operators at 32 channels on the benchmark APR, priced with their algorithmic bytes against the HBM
    peak (hbm_frac), a device-to-device copy of the same tensor (copy_frac) and the best streaming rate measured
    here (stream_frac).  fp32 channel planes, bfloat16 channel planes, and bfloat16 grouped by eight channels."""
    import torch
    from pyapr.aprnet import _ops, grouped
    C, e = x.shape[1], 4
    ld0, ld1 = torch.zeros(1, dtype=torch.int32), torch.ones(1, dtype=torch.int32)
    n0, n1 = _ops.number_particles(apr, 0), _ops.number_particles(apr, 1)
    nt = _ops.tree_parts(apr, 0)
    res = []

    # Two reference rates for the memory-bound operators: a plain device-to-device copy of the same tensor, and the
    # best streaming rate this library itself reaches on it (the norm kernels: mostly reads, 16 bytes per lane).
    dst = torch.empty_like(x)
    ms = _time(lambda: dst.copy_(x))
    copy_gbs = 2 * x.numel() * e / ms / 1e6
    res.append({"op": "copy_d2d", "ms": ms, "algorithmic_GB": 2 * x.numel() * e / 1e9, "GBps": copy_gbs,
                "hbm_frac": copy_gbs / PEAK_HBM_GBS, "note": "torch copy of the input features, read + write"})
    ms = _time(lambda: dst.fill_(1.0))
    res.append({"op": "fill", "ms": ms, "algorithmic_GB": x.numel() * e / 1e9, "GBps": x.numel() * e / ms / 1e6,
                "hbm_frac": x.numel() * e / ms / 1e6 / PEAK_HBM_GBS, "note": "torch fill of a tensor of the same size: writes only"})
    ms = _time(lambda: torch.sum(x, dim=2))
    res.append({"op": "row_sum", "ms": ms, "algorithmic_GB": x.numel() * e / 1e9, "GBps": x.numel() * e / ms / 1e6,
                "hbm_frac": x.numel() * e / ms / 1e6 / PEAK_HBM_GBS, "note": "torch sum over the particles: reads only"})
    del dst
    from apr_models.unet.particle_norm import ParticleBatchNorm
    bn = ParticleBatchNorm(C).to(dev).train()
    with torch.no_grad():
        ms_nf = _time(lambda: bn(x, relu=True))
    xn = x.detach().clone().requires_grad_(True)
    yn = bn(xn, relu=True)
    gn = torch.randn_like(yn)
    ms_nb = _time(lambda: torch.autograd.grad(yn, xn, gn, retain_graph=True))
    del xn, yn, gn, bn
    stream_gbs = max(copy_gbs, e * 3 * C * n0 / ms_nf / 1e6, e * 7 * C * n0 / ms_nb / 1e6)

    def line(op, ms, nbytes, note):
        res.append({"op": op, "ms": ms, "algorithmic_GB": nbytes / 1e9, "GBps": nbytes / ms / 1e6,
                    "hbm_frac": nbytes / ms / 1e6 / PEAK_HBM_GBS, "copy_frac": nbytes / ms / 1e6 / copy_gbs,
                    "stream_frac": nbytes / ms / 1e6 / stream_gbs, "note": note})

    line("norm_relu_fwd", ms_nf, e * 3 * C * n0, f"C={C}: one pass for the moments, one read + one write to normalise")
    line("norm_relu_bwd", ms_nb, e * 7 * C * n0, "gradient, input and output read twice (sums, then result), one write")
    lib, plan, st = _ops._lib(), apr.plan(0), torch.cuda.current_stream().cuda_stream
    with torch.no_grad():
        pooled, idx = _ops.maxpool_forward([apr], x, ld0, 0.0)
        ms = _time(lambda: _ops.maxpool_forward([apr], x, ld0, 0.0))
        line("maxpool_fwd", ms, e * C * n0 + (e + 8) * C * n1, f"C={C}, N {n0} -> {n1}, int64 argmax written")
        ms = _time(lambda: _ops.maxpool_backward([apr], pooled, idx, ld0))
        line("maxpool_bwd", ms, (e + 8) * C * n1 + e * C * n0, "reads grad + argmax, writes grad_input")
        ms = _time(lambda: _ops.upsample_const_forward([apr], pooled, ld1))
        line("upsample_fwd", ms, e * C * (n1 + n0), f"C={C}, N {n1} -> {n0}")
        ms = _time(lambda: _ops.upsample_const_backward([apr], x, ld1))
        line("upsample_bwd", ms, e * C * (n1 + n0), "sum of child gradients")
        tree = torch.empty(C, max(nt, 1), device=dev)
        ms = _time(lambda: lib.aprnet_fill_tree_mean_f32(plan, 0, x.data_ptr(), x.shape[2], C, tree.data_ptr(), tree.shape[1], st))
        line("fill_tree_mean", ms, e * C * (n0 + 2 * nt), f"C={C}, {nt} tree nodes")
        gxt, gtt = torch.zeros_like(x[0]), torch.randn(C, max(nt, 1), device=dev)
        ms = _time(lambda: lib.aprnet_fill_tree_mean_bwd_f32(plan, 0, gxt.data_ptr(), gxt.shape[1], C, gtt.data_ptr(), gtt.shape[1], st))
        line("fill_tree_mean_bwd", ms, e * C * (2 * n0 + 3 * nt), "children read and written in place, tree gradient read and written")
        del gxt, gtt, tree
        w1 = torch.randn(1, C, C, 1, 1, 1, device=dev) * 0.1
        ms = _time(lambda: _ops.conv_forward([apr], x, w1, ld0))
        line("conv111_fwd", ms, e * 2 * C * n0, f"{C}->{C}")
        # bfloat16 channel planes
        xb = x.to(torch.bfloat16)
        pooled_b, idx_b = _ops.maxpool_forward([apr], xb, ld0, 0.0)
        ms = _time(lambda: _ops.maxpool_forward([apr], xb, ld0, 0.0))
        line("maxpool_fwd_bf16", ms, 2 * C * n0 + (2 + 8) * C * n1, "bfloat16 planes, int64 argmax")
        ms = _time(lambda: _ops.upsample_const_forward([apr], pooled_b, ld1))
        line("upsample_fwd_bf16", ms, 2 * C * (n1 + n0), "bfloat16 planes")
        ms = _time(lambda: _ops.conv_forward([apr], xb, w1, ld0))
        line("conv111_fwd_bf16", ms, 2 * 2 * C * n0, f"{C}->{C}, bfloat16 planes")
        del idx_b, idx
        # bfloat16 grouped by eight channels (the layout a network keeps between its layers at inference)
        if grouped.supported([apr], (C,)):
            xg8 = grouped.regroup(xb)
            ms = _time(lambda: grouped.regroup(xb))
            line("regroup8_bf16", ms, 2 * 2 * C * n0, "channel planes -> groups of eight")
            pg8 = grouped.maxpool_forward([apr], xg8, ld0)
            ms = _time(lambda: grouped.maxpool_forward([apr], xg8, ld0))
            line("maxpool_fwd_bf16g", ms, 2 * C * (n0 + n1), "values only (no argmax at inference)")
            ms = _time(lambda: grouped.upsample_const_forward([apr], pg8, ld1))
            line("upsample_fwd_bf16g", ms, 2 * C * (n1 + n0), "")
            ms = _time(lambda: grouped.conv111_forward([apr], xg8, w1, ld0))
            line("conv111_fwd_bf16g", ms, 2 * 2 * C * n0, f"{C}->{C}, grouped in and out")
            treeg = torch.empty((C // 8) * max(nt, 1) * 8, dtype=torch.bfloat16, device=dev)
            ms = _time(lambda: lib.aprnet_fill_tree_mean_bf16g(plan, 0, xg8.data.data_ptr(), n0, C, treeg.data_ptr(), max(nt, 1), st))
            line("fill_tree_mean_bf16g", ms, 2 * C * (n0 + 2 * nt), "")
    return res


def other_ops(apr, x, dev):
    """The backward pass of the convolution, the wide 2-D stencil, and the 4-level APR-UNet (forward, HIP graph, training
    step) on the benchmark APR."""
    import torch
    from pyapr import aprnet
    from pyapr.aprnet import _ops
    from apr_models.unet import APRUNet, fold_norms
    C = x.shape[1]
    ld0 = torch.zeros(1, dtype=torch.int32)
    n0 = _ops.number_particles(apr, 0)
    res = []
    conv = aprnet.cuda.APRConv(C, C, nstencils=2).to(dev)
    xg = x.clone().requires_grad_(True)
    y = conv(xg, [apr], ld0)
    go = torch.randn_like(y)
    ms = _time(lambda: torch.autograd.grad(y, (xg, conv.weight), go, retain_graph=True), iters=3, warmup=1)
    fl = 2 * 2 * 27 * C * C * n0
    res.append({"op": "conv333_bwd", "ms": ms, "particles_per_s": n0 / ms * 1e3, "TFLOPs": fl / ms / 1e9,
                "mfma_frac": fl / ms / 1e9 / PEAK_FP32_MATRIX_TFLOPS, "note": f"{C}->{C} grad_input + grad_weight"})
    del y, go, xg
    torch.manual_seed(0)
    net = fold_norms(APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch").eval()).to(dev)
    xin = x[:, :1].contiguous()
    with torch.no_grad():
        ms = _time(lambda: net(xin, [apr]), iters=3, warmup=1)
    res.append({"op": "apr_unet_fwd", "ms": ms, "note": f"4 levels 16-32-64-128, fp32, {n0} particles, norms folded"})
    # the same forward captured once into a HIP graph and replayed (no host work between the ~250 launches)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            net(xin, [apr])
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_graph = net(xin, [apr])
        ms = _time(graph.replay, iters=3, warmup=1)
    res.append({"op": "apr_unet_fwd_graph", "ms": ms, "note": "the fp32 forward replayed from a HIP graph"})
    del graph, y_graph
    # the reference's default configuration: GroupNorm with one group per channel, which cannot be folded away
    torch.manual_seed(0)
    gnet = APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="group").eval().to(dev)
    with torch.no_grad():
        ms = _time(lambda: gnet(xin, [apr]), iters=3, warmup=1)
    res.append({"op": "apr_unet_fwd_groupnorm", "ms": ms, "note": "same architecture with GroupNorm layers (norm + ReLU in one pass of the streaming norm kernels)"})
    del gnet
    # one training step of the same architecture (unfolded BatchNorm in training mode): forward, loss, backward
    torch.manual_seed(0)
    tnet = APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch").to(dev).train()
    target = torch.randn(1, 3, xin.shape[2], device=dev)

    def train_step():
        for p_ in tnet.parameters():
            p_.grad = None
        torch.nn.functional.mse_loss(tnet(xin, [apr]), target).backward()
    ms = _time(train_step, iters=2, warmup=1)
    res.append({"op": "apr_unet_train_step", "ms": ms, "particles_per_s": n0 / ms * 1e3,
                "note": "forward + backward of the 4-level network, fp32, BatchNorm in training mode, MSE loss, no optimizer"})
    del tnet, target
    # the same step on an APR of the size training crops have (64 x 128 x 128 centre crop): bound by the host, ~850 launches
    small = build_workload("blobs512", crop=(64, 128, 128))
    ns = small.total_number_particles()
    torch.manual_seed(0)
    snet = APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch").to(dev).train()
    xs, ts = torch.randn(1, 1, ns, device=dev), torch.randn(1, 3, ns, device=dev)

    def small_step():
        for p_ in snet.parameters():
            p_.grad = None
        torch.nn.functional.mse_loss(snet(xs, [small]), ts).backward()
    ms = _time(small_step, iters=10, warmup=3)
    res.append({"op": "apr_unet_train_step_small", "ms": ms, "particles_per_s": ns / ms * 1e3,
                "note": f"the same training step on a 64x128x128 crop, {ns} particles, ~590 short launches on two streams"})
    # the same step captured once into a HIP graph (forward, loss, backward) and replayed
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        small_step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for p_ in snet.parameters():
        p_.grad = None
    sgraph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(sgraph):
        torch.nn.functional.mse_loss(snet(xs, [small]), ts).backward()
    ms = _time(sgraph.replay, iters=10, warmup=3)
    res.append({"op": "apr_unet_train_step_small_graph", "ms": ms, "particles_per_s": ns / ms * 1e3,
                "note": "that step replayed from a HIP graph: no host work between the launches"})
    del sgraph, snet, xs, ts, small
    # the wide 2-D stencil of configs[4] (1x5x5, 64 -> 64), here on the 3-D benchmark APR, fp32
    conv5 = aprnet.cuda.APRConv(64, 64, nstencils=2, kernel_size=(1, 5, 5)).to(dev)
    x64 = torch.randn(1, 64, x.shape[2], device=dev)
    with torch.no_grad():
        ms = _time(lambda: conv5(x64, [apr], ld0), iters=3, warmup=1)
    fl = 2 * 25 * 64 * 64 * n0
    res.append({"op": "conv155_fwd", "ms": ms, "particles_per_s": n0 / ms * 1e3, "TFLOPs": fl / ms / 1e9,
                "mfma_frac": fl / ms / 1e9 / PEAK_FP32_MATRIX_TFLOPS, "note": "1x5x5 64->64 fp32, whole APRConv.forward"})
    x64.requires_grad_(True)
    y5 = conv5(x64, [apr], ld0)
    go5 = torch.randn_like(y5)
    ms = _time(lambda: torch.autograd.grad(y5, (x64, conv5.weight), go5, retain_graph=True), iters=2, warmup=1)
    res.append({"op": "conv155_bwd", "ms": ms, "particles_per_s": n0 / ms * 1e3, "note": "1x5x5 64->64 grad_input + grad_weight"})
    del y5, go5, x64, conv5
    # bfloat16 features (convolutions: bfloat16 matrix instructions with fp32 accumulation)
    xb = x.to(torch.bfloat16)
    with torch.no_grad():
        ms = _time(lambda: conv(xb, [apr], ld0), iters=5, warmup=1)
        res.append({"op": "conv333_fwd_bf16", "ms": ms, "particles_per_s": n0 / ms * 1e3,
                    "note": f"{C}->{C}, bfloat16 features and matrix math (fp32 accumulate), whole APRConv.forward"})
        x64b = torch.randn(1, 64, x.shape[2], device=dev).to(torch.bfloat16)
        conv5b = aprnet.cuda.APRConv(64, 64, nstencils=2, kernel_size=(1, 5, 5)).to(dev)
        ms = _time(lambda: conv5b(x64b, [apr], ld0), iters=3, warmup=1)
        res.append({"op": "conv155_fwd_bf16", "ms": ms, "particles_per_s": n0 / ms * 1e3, "TFLOPs": 2 * 25 * 64 * 64 * n0 / ms / 1e9,
                    "note": "1x5x5 64->64, bfloat16 features and matrix math (configs[4] layer), whole APRConv.forward"})
    x64b.requires_grad_(True)
    y5b = conv5b(x64b, [apr], ld0)
    go5b = torch.randn_like(y5b)
    ms = _time(lambda: torch.autograd.grad(y5b, (x64b, conv5b.weight), go5b, retain_graph=True), iters=2, warmup=1)
    res.append({"op": "conv155_bwd_bf16", "ms": ms, "particles_per_s": n0 / ms * 1e3,
                "note": "1x5x5 64->64 backward, bfloat16 features and gradients: input and weight gradient on the bfloat16 "
                        "matrix cores, fp32 accumulation"})
    del y5b, go5b, x64b, conv5b
    with torch.no_grad():
        xinb = xin.to(torch.bfloat16)
        ms = _time(lambda: net(xinb, [apr]), iters=3, warmup=1)
    res.append({"op": "apr_unet_fwd_bf16", "ms": ms, "note": "same network, bfloat16 features"})
    torch.manual_seed(0)
    tnet = APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch").to(dev).train()
    target = torch.randn(1, 3, xin.shape[2], device=dev)
    torch.cuda.empty_cache()          # the step allocates other sizes than the inference runs before it left cached

    def train_step_bf16():
        for p_ in tnet.parameters():
            p_.grad = None
        torch.nn.functional.mse_loss(tnet(xinb, [apr]).float(), target).backward()
    ms = _time(train_step_bf16, iters=3, warmup=2)
    res.append({"op": "apr_unet_train_step_bf16", "ms": ms, "particles_per_s": n0 / ms * 1e3,
                "note": "the training step with bfloat16 features and feature gradients (fp32 parameters and accumulation)"})
    return res


RUNNERS = {"spheres128": run_spheres128, "blobs512": run_blobs512, "nuclei2048": run_nuclei2048,
           "nuclei1024": run_nuclei1024, "spots16k": run_spots16k}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", choices=sorted(RUNNERS), default="blobs512",
                    help="BASELINE configuration to run (default: the one the headline metric is quoted on)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true",
                    help="blobs512: only the convolution step (no APR-UNet latency, no CPU baseline): for profiler runs")
    ap.add_argument("--features", choices=["f32", "bf16", "bf16g"], default="f32",
                    help="blobs512: element type of the feature tensors; bf16 runs the bfloat16 matrix-core kernel on channel "
                         "planes, bf16g on tensors grouped by eight channels, as a network keeps them between its layers "
                         "(the headline figure is the f32 one)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="blobs512: run one device-to-device copy of the input features (a kernel of known traffic, "
                         "used to scale the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--ops", action="store_true",
                    help="blobs512: also time the memory-bound operators, the backward pass and the networks (extra JSON lines on stderr)")
    ap.add_argument("--channels", type=int, nargs=2, default=[32, 32], metavar=("CIN", "COUT"),
                    help="blobs512: channel counts of the timed layer (default 32 32, the layer the metric is quoted on)")
    ap.add_argument("--backward", action="store_true",
                    help="blobs512: time the backward pass of the layer instead of the forward pass")
    ap.add_argument("--ops-mem", action="store_true",
                    help="blobs512: also time the memory-bound operators only (fp32, bfloat16 planes, bfloat16 grouped by eight)")
    ap.add_argument("--chain", action="store_true",
                    help="blobs512: also time the conv -> ReLU -> pool -> upsample chain of configs[1], forward + backward (stderr)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
                 "(the path would shard by batch item, or by z-slabs with a one-row halo per level)")

    import threading
    import torch
    from pyapr import _native
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    if args.config != "blobs512":
        # the large configurations spend minutes in native host code (volume synthesis, APR build, CPU baseline)
        t_start = time.perf_counter()

        def heartbeat():
            while True:
                time.sleep(60)
                say(f"{args.config}: working, {time.perf_counter() - t_start:.0f} s")
        threading.Thread(target=heartbeat, daemon=True).start()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    out = RUNNERS[args.config](args, dev, _native.hip())
    headline = (args.config == "blobs512" and not args.no_extra and not args.backward and args.features == "f32"
                and tuple(args.channels) == (32, 32))
    if headline:
        # The second half of the metric on the configuration it is quoted on: APR-UNet forward on the APR of the whole
        # 1024^3 volume (configs[3]), fp32 and bfloat16, into extra.apr_unet_1024_*; then the lines of configs[2] and
        # configs[4] on stderr with their rooflines.  A failure here (device memory on a smaller card) is reported in
        # the line and does not take the headline measurement with it.
        import gc
        sub = argparse.Namespace(**vars(args))
        sub.no_cpu_baseline = True
        for name in ("nuclei1024", "nuclei2048", "spots16k"):
            gc.collect()
            torch.cuda.empty_cache()
            t0 = time.perf_counter()
            try:
                line = RUNNERS[name](sub, dev, _native.hip())
            except Exception as err:                 # noqa: BLE001 - reported, not hidden
                line = {"config": {"workload": name}, "error": f"{type(err).__name__}: {str(err).splitlines()[0][:300]}"}
            line["wall_s"] = round(time.perf_counter() - t0, 1)
            print(json.dumps(line), file=sys.stderr, flush=True)
            if name == "nuclei1024":
                ex, cfg = line.get("extra", {}), line.get("config", {})
                for key, tag in (("apr_unet_fwd_f32", "f32"), ("apr_unet_fwd_bf16", "bf16")):
                    r = ex.get(key) or {}
                    out["extra"][f"apr_unet_1024_fwd_ms_{tag}"] = r.get("ms")
                    out["extra"][f"apr_unet_1024_peak_device_GB_{tag}"] = r.get("peak_device_GB")
                    if r.get("error"):
                        out["extra"][f"apr_unet_1024_error_{tag}"] = r["error"]
                out["extra"]["apr_unet_1024_n_particles"] = cfg.get("n_particles")
                out["extra"]["apr_unet_1024_workload"] = cfg.get("workload", line.get("error"))
                out["extra"]["apr_unet_1024_apr_build_s"] = cfg.get("apr_build_s")
                out["extra"]["apr_unet_1024_particles_per_s_bf16"] = ex.get("particles_per_s_bf16")
            else:
                key = "conv333_16x16_nuclei2048" if name == "nuclei2048" else "conv155_64x64_bf16_spots16k"
                out["extra"][key] = {"value": line.get("value"), "unit": line.get("unit"), "ms_per_step": line.get("ms_per_step"),
                                     "n_particles": line.get("config", {}).get("n_particles"), "roofline": line.get("roofline"),
                                     "extra": line.get("extra"), "error": line.get("error")}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
