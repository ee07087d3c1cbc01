#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X: APRConv 3x3x3 forward, Cin = Cout = 32, fp32, on the APR of the
seeded 512 x 512 x 256 blob volume (BASELINE.json configs[1]).

  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one `aprnet.cuda.APRConv.forward` on device-resident features: weight expansion
(restrict kernel), tree fill of the 32 input channels and the convolution kernel (bias fused into its store).
Prints ONE JSON line.  `value` = particles/s of the whole step; `roofline` prices the convolution
kernel alone (its duration is measured with HIP events recorded around the launch on its own stream,
see aprnet_profile_enable in include/aprnet_hip.h); `cpu_baseline` times the CPU oracle (a restatement
of the reference's OpenMP code) on a centre crop of the same volume.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "apr-cnn_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

CIN = COUT = 32
K_TAPS = 27
FLOP_PER_PARTICLE = 2 * K_TAPS * CIN * COUT          # 55 296
BYTES_PER_PARTICLE = 4 * (CIN + COUT) + 2            # features in + out, y_vec
PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_BF16_MATRIX_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
# HBM-side bytes of one launch of the convolution kernel on this workload: FETCH_SIZE + WRITE_SIZE of two
# profiler passes, scaled by what the same counters read for a device-to-device copy of known size
# (profiles/conv333_fwd_32x32_f32_blobs512_hbm_traffic.txt).  Counters cannot be read from inside this
# script; the figure is only reported when the workload is the one it was measured on.
MEASURED_TRAFFIC_BYTES = {23245996: 30.18e9 + 4.10e9}


def build_workload(name, crop=None):
    import numpy as np
    from pyapr.synthetic import CONFIGS, synth_volume, pipeline_parameters
    from pyapr.converter import get_apr
    shape, kind, n, axes, amp, bg, iso, rel = CONFIGS[name]
    img = synth_volume(shape, 0, kind, n, axes, amp, bg, iso)
    if crop is not None:
        z, x, y = (s // 2 for s in shape)
        cz, cx, cy = (c // 2 for c in crop)
        img = np.ascontiguousarray(img[z - cz:z + cz, x - cx:x + cx, y - cy:y + cy])
    apr, _parts = get_apr(img, params=pipeline_parameters(rel))
    return apr


def cpu_baseline(nstencils):
    """CPU oracle (port of pyapr/aprnet/src/conv.hpp + helpers.hpp, OpenMP over z) on a 128 x 256 x 256 centre
    crop of the benchmark volume, same layer shape; a few seconds to tens of seconds of CPU work."""
    import torch
    from oracle import oracle
    crop = (128, 256, 256)
    apr = build_workload("blobs512", crop=crop)
    n = apr.total_number_particles()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, CIN, n, generator=g)
    w = torch.randn(CIN, nstencils, COUT, 3, 3, 3, generator=g) * 0.1
    ld = torch.zeros(1, dtype=torch.int32)
    t0 = time.perf_counter()
    w_exp = oracle.restrict_kernel_forward(w, apr.level_max() - apr.level_min() + 1)
    oracle.conv_forward([apr], x, w_exp, ld)
    dt = time.perf_counter() - t0
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or len(os.sched_getaffinity(0))
    return {"value": n / dt, "unit": "particles/s", "cores": cores, "kind": "port",
            "sample": f"centre crop {crop[0]}x{crop[1]}x{crop[2]} of the 256x512x512 volume, {n} particles, "
                      f"conv 3x3x3 {CIN}->{COUT} fp32, 1 run, {dt:.1f} s"}


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


def other_ops(apr, x, dev):
    """Memory-bound operators at 32 channels on the same APR, priced against the HBM roofline with their
    algorithmic bytes, the backward pass of the convolution, and the 4-level APR-UNet forward."""
    import torch
    from pyapr import aprnet
    from pyapr.aprnet import _ops
    from apr_models.unet import APRUNet, fold_norms
    C, e = x.shape[1], 4
    ld0, ld1 = torch.zeros(1, dtype=torch.int32), torch.ones(1, dtype=torch.int32)
    n0, n1 = _ops.number_particles(apr, 0), _ops.number_particles(apr, 1)
    nt = _ops.tree_parts(apr, 0)
    res = []

    # what a plain device-to-device copy of the same tensor reaches on this GPU: the practical ceiling that the
    # memory-bound operators are also priced against
    dst = torch.empty_like(x)
    ms = _time(lambda: dst.copy_(x))
    copy_gbs = 2 * x.numel() * e / ms / 1e6
    res.append({"op": "copy_d2d", "ms": ms, "algorithmic_GB": 2 * x.numel() * e / 1e9, "GBps": copy_gbs,
                "hbm_frac": copy_gbs / PEAK_HBM_GBS, "note": "torch copy of the input features, read + write"})
    del dst

    def line(op, ms, nbytes, note):
        res.append({"op": op, "ms": ms, "algorithmic_GB": nbytes / 1e9, "GBps": nbytes / ms / 1e6,
                    "hbm_frac": nbytes / ms / 1e6 / PEAK_HBM_GBS, "copy_frac": nbytes / ms / 1e6 / copy_gbs, "note": note})

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
        lib, plan, st = _ops._lib(), apr.plan(0), torch.cuda.current_stream().cuda_stream
        ms = _time(lambda: lib.aprnet_fill_tree_mean_f32(plan, 0, x.data_ptr(), x.shape[2], C, tree.data_ptr(), tree.shape[1], st))
        line("fill_tree_mean", ms, e * C * (n0 + 2 * nt), f"C={C}, {nt} tree nodes")
        w1 = torch.randn(1, C, C, 1, 1, 1, device=dev) * 0.1
        ms = _time(lambda: _ops.conv_forward([apr], x, w1, ld0))
        line("conv111_fwd", ms, e * 2 * C * n0, f"{C}->{C}")
    # BatchNorm1d + ReLU over the particle axis in training mode (statistics of the batch), forward and backward
    from apr_models.unet.particle_norm import ParticleBatchNorm
    bn = ParticleBatchNorm(C).to(dev).train()
    with torch.no_grad():
        ms = _time(lambda: bn(x, relu=True))
    line("norm_relu_fwd", ms, e * 3 * C * n0, f"C={C}: one pass for the moments, one read + one write to normalise")
    xn = x.detach().clone().requires_grad_(True)
    yn = bn(xn, relu=True)
    gn = torch.randn_like(yn)
    ms = _time(lambda: torch.autograd.grad(yn, xn, gn, retain_graph=True))
    line("norm_relu_bwd", ms, e * 7 * C * n0, "gradient, input and output read twice (sums, then result), one write")
    del xn, yn, gn, bn
    conv = aprnet.cuda.APRConv(C, C, nstencils=2).to(dev)
    xg = x.clone().requires_grad_(True)
    y = conv(xg, [apr], ld0)
    go = torch.randn_like(y)
    ms = _time(lambda: torch.autograd.grad(y, (xg, conv.weight), go, retain_graph=True), iters=3, warmup=1)
    res.append({"op": "conv333_bwd", "ms": ms, "particles_per_s": n0 / ms * 1e3, "note": f"{C}->{C} grad_input + grad_weight"})
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
        ms = _time(lambda: _ops.maxpool_forward([apr], xb, ld0, 0.0))
        line("maxpool_fwd_bf16", ms, 2 * C * n0 + (2 + 8) * C * n1, "bfloat16 values, int64 argmax")
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

    def train_step_bf16():
        for p_ in tnet.parameters():
            p_.grad = None
        torch.nn.functional.mse_loss(tnet(xinb, [apr]).float(), target).backward()
    ms = _time(train_step_bf16, iters=2, warmup=1)
    res.append({"op": "apr_unet_train_step_bf16", "ms": ms, "particles_per_s": n0 / ms * 1e3,
                "note": "the training step with bfloat16 features and feature gradients (fp32 parameters and accumulation)"})
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--features", choices=["f32", "bf16"], default="f32",
                    help="element type of the feature tensors; bf16 runs the bfloat16 matrix-core kernel "
                         "(the headline figure is the f32 one)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run one device-to-device copy of the input features (a kernel of known traffic, "
                         "used to scale the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--ops", action="store_true",
                    help="also time the memory-bound operators and the APR-UNet forward (extra JSON lines on stderr)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
                 "(the path would shard by batch item, or by z-slabs with a one-row halo per level)")

    import torch
    from pyapr import aprnet, _native
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    nstencils = 2
    t0 = time.perf_counter()
    apr = build_workload("blobs512")
    t_build = time.perf_counter() - t0
    t0 = time.perf_counter()
    apr.init_cuda()
    t_plan = time.perf_counter() - t0
    n = apr.total_number_particles()

    torch.manual_seed(0)
    x = torch.randn(1, CIN, n, device=dev)
    if args.features == "bf16":
        x = x.to(torch.bfloat16)
    conv = aprnet.cuda.APRConv(CIN, COUT, nstencils=nstencils, kernel_size=(3, 3, 3), bias=True).to(dev)
    ld = torch.zeros(1, dtype=torch.int32)
    lib = _native.hip()

    with torch.no_grad():
        for _ in range(args.warmup):
            y = conv(x, [apr], ld)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            y = conv(x, [apr], ld)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0

        # duration of the convolution kernel alone: HIP events around its launch, on its stream
        lib.aprnet_profile_enable(1)
        kms = []
        for _ in range(args.steps):
            y = conv(x, [apr], ld)
            kms.append(float(lib.aprnet_profile_last_ms()))
        lib.aprnet_profile_enable(0)
    kernel_ms = sum(kms) / len(kms)
    assert torch.isfinite(y.float()).all()
    bf16 = args.features == "bf16"

    ms_per_step = dt / args.steps * 1e3
    value = n / (dt / args.steps)
    tflops = FLOP_PER_PARTICLE * n / (kernel_ms * 1e-3) / 1e12
    gbs = (BYTES_PER_PARTICLE if args.features == "f32" else BYTES_PER_PARTICLE // 2 + 1) * n / (kernel_ms * 1e-3) / 1e9
    out = {
        "metric": "APRConv 3x3x3 fwd particles/s (Cin=Cout=32)",
        "value": value, "unit": "particles/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f32", "data": "synthetic",
        "config": {"workload": f"APRConv 3x3x3 32->32 {'bf16' if bf16 else 'fp32'} forward (restrict + tree fill + conv + bias), batch 1, "
                               "APR of the seeded 512x512x256 volume with 2000 ellipsoidal blobs (configs[1])",
                   "n_particles": n, "nstencils": nstencils, "level_max": apr.level_max(),
                   "apr_build_s": round(t_build, 2), "plan_create_s": round(t_plan, 2)},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK_BF16_MATRIX_TFLOPS if bf16 else PEAK_FP32_MATRIX_TFLOPS,
                     "unit": "TFLOP/s", "frac": tflops / (PEAK_BF16_MATRIX_TFLOPS if bf16 else PEAK_FP32_MATRIX_TFLOPS),
                     "traffic": None if bf16 else MEASURED_TRAFFIC_BYTES.get(n),
                     "kernel": "conv_mfma_bf16_kernel" if bf16 else "conv_mfma16_kernel", "kernel_ms": kernel_ms,
                     "hbm_achieved_GBs": gbs, "hbm_frac": gbs / PEAK_HBM_GBS},
    }
    if args.calibrate_copy:
        torch.empty_like(x).copy_(x)
        torch.cuda.synchronize()
        print(json.dumps({"calibration_copy_bytes_read": x.numel() * 4, "calibration_copy_bytes_written": x.numel() * 4}),
              file=sys.stderr, flush=True)
    if args.ops:
        for line in other_ops(apr, x, dev):
            print(json.dumps(line), file=sys.stderr, flush=True)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(nstencils)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
