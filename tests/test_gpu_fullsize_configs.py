"""BASELINE configs[2] and configs[4] at their full size (360 M and 246 M particles), where the CPU oracle cannot be
the checker: properties that hold at any size and that a wrong index, a dropped window or a 32-bit overflow at these
particle counts would break.  (configs[0] and configs[1] run at full size in test_gpu_configs.py / test_gpu_fullsize.py,
configs[3] in test_gpu_configs.py; scaled replicas of every configuration are compared with the oracle there.)
Needs a device with about 200 GB of free memory; skipped otherwise."""
import pytest
import torch

from pyapr.aprnet import _ops, grouped as g8
from pyapr.synthetic import make_config

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _need(gb):
    free, _total = torch.cuda.mem_get_info()
    if free < gb * 1e9:
        pytest.skip(f"needs about {gb} GB of free device memory, {free / 1e9:.0f} GB available")


def _dot(a, b):
    """<a, b> in float64 without a float64 copy of the whole tensors (one channel at a time)."""
    return sum(float((a[0, c].double() * b[0, c].double()).sum()) for c in range(a.shape[1]))


def _absdot(a, b):
    return sum(float((a[0, c].double().abs() * b[0, c].double().abs()).sum()) for c in range(a.shape[1]))


def test_nuclei2048_whole_volume_tree_fill_and_conv_properties():
    """configs[2], whole 2048 x 2048 x 512 volume, 16 channels fp32: the tree mean of a constant field is that constant
    on every node, bit for bit; the identity stencil returns its input exactly (every particle is visited once and
    reads its own cell); the parent-reading convolution is finite and repeats bit for bit."""
    _need(150)
    apr, _ = make_config("nuclei2048")
    apr.init_cuda()
    n, c = apr.total_number_particles(), 16
    assert n > 300_000_000
    nt = _ops.tree_parts(apr, 0)
    lib, plan, st = _ops._lib(), apr.plan(0), torch.cuda.current_stream().cuda_stream
    x = torch.full((1, c, n), 3.25, device=DEV)
    tree = torch.empty(c, nt, device=DEV)
    assert lib.aprnet_fill_tree_mean_f32(plan, 0, x.data_ptr(), n, c, tree.data_ptr(), nt, st) == 0
    assert bool((tree == 3.25).all())
    del tree
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    g = torch.Generator(device=DEV).manual_seed(2)
    x.normal_(generator=g)
    wi = torch.zeros(levels, c, c, 3, 3, 3)
    for i in range(c):
        wi[:, i, i, 1, 1, 1] = 1
    y = _ops.conv_forward([apr], x, wi.to(DEV), ld)
    assert torch.equal(y, x)
    wr = (torch.randn(levels, c, c, 3, 3, 3, generator=torch.Generator().manual_seed(3)) * 0.1).to(DEV)
    y = _ops.conv_forward([apr], x, wr, ld)
    assert bool(torch.isfinite(y).all()) and float(y.abs().max()) > 0
    y2 = _ops.conv_forward([apr], x, wr, ld)
    assert torch.equal(y, y2)


def test_spots16k_whole_image_identity_adjoint_and_grouped_equals_planes():
    """configs[4], whole 16384^2 image, 1x5x5 64 -> 64 with bfloat16 features: the identity stencil copies the features
    exactly; the kernel on tensors grouped by eight channels returns bit for bit what the kernel on channel planes
    returns; <conv(x), gy> = <x, dX> = <w, dW> to the bfloat16 rounding of the stored tensors."""
    _need(230)
    apr, _ = make_config("spots16k")
    apr.init_cuda()
    n, c = apr.total_number_particles(), 64
    assert n > 200_000_000
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    g = torch.Generator(device=DEV).manual_seed(5)
    x = torch.empty(1, c, n, device=DEV, dtype=torch.bfloat16).normal_(generator=g)
    wi = torch.zeros(levels, c, c, 1, 5, 5)
    for i in range(c):
        wi[:, i, i, 0, 2, 2] = 1
    y = _ops.conv_forward([apr], x, wi.to(DEV), ld)
    assert torch.equal(y, x)
    del y
    w = (torch.randn(levels, c, c, 1, 5, 5, generator=torch.Generator().manual_seed(6)) * 0.05).to(torch.bfloat16).float().to(DEV)
    y = _ops.conv_forward([apr], x, w, ld)
    assert bool(torch.isfinite(y[0, 0].float()).all()) and bool(torch.isfinite(y[0, c - 1].float()).all())
    xg = g8.regroup(x)
    yg = g8.conv_forward([apr], xg, w, ld)
    del xg
    for q in range(c // 8):                                  # group q of the grouped result = planes 8 q .. 8 q + 7
        assert torch.equal(yg.data[0, q].transpose(0, 1), y[0, 8 * q:8 * q + 8])
    del yg
    torch.cuda.empty_cache()
    gy = torch.empty(1, c, n, device=DEV, dtype=torch.bfloat16).normal_(generator=g)
    lhs, ref = _dot(y, gy), _absdot(y, gy)
    del y
    torch.cuda.empty_cache()
    gx, gw = _ops.conv_backward([apr], x, w, gy, ld)
    assert abs(lhs - _dot(x, gx)) <= 1e-2 * ref
    assert abs(lhs - float((w.double() * gw.double()).sum())) <= 1e-2 * ref
