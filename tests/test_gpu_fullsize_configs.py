"""BASELINE configs[2], configs[3] and configs[4] at their full size (360 M, 844 M and 246 M particles).  At 16 to 64
channels the CPU oracle cannot be the checker there: properties that hold at any size and that a wrong index, a
dropped window or a 32-bit overflow at these particle counts would break.  With 1 to 8 channels it can: configs[3] is
compared with it on every particle, for the forward kernel families, the tree operators and the gradients.
(configs[0] and configs[1] run at full size in test_gpu_configs.py / test_gpu_fullsize.py; scaled replicas of every
configuration are compared with the oracle there.)  Needs a device with about 200 GB of free memory; skipped otherwise."""
import pytest
import torch

from pyapr.aprnet import _ops, grouped as g8
from pyapr.synthetic import make_config

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _need(gb):
    import gc
    gc.collect()
    torch.cuda.empty_cache()                  # what earlier tests left in torch's cache counts as free
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
    reads its own cell); the parent-reading convolution is finite and repeats bit for bit; with four channels it is
    compared with the CPU oracle on every particle."""
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
    del y, y2
    # with four channels the CPU oracle finishes in seconds at this size: every particle, rel 1e-5 of the output scale
    from oracle import oracle
    w4 = torch.randn(4, levels, 4, 3, 3, 3, generator=torch.Generator().manual_seed(4)) * 0.2
    x4 = x[:, :4].contiguous()
    got = _ops.conv_forward([apr], x4, w4.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld).cpu()
    ref = oracle.conv_forward([apr], x4.cpu(), w4, ld)
    for ch in range(4):
        assert float((got[0, ch] - ref[0, ch]).abs().max()) <= 1e-5 * float(ref[0, ch].abs().max())


def test_spots16k_whole_image_identity_adjoint_and_grouped_equals_planes():
    """configs[4], whole 16384^2 image, 1x5x5 64 -> 64 with bfloat16 features: the identity stencil copies the features
    exactly; the kernel on tensors grouped by eight channels returns bit for bit what the kernel on channel planes
    returns; <conv(x), gy> = <x, dX> = <w, dW> to the bfloat16 rounding of the stored tensors; with eight channels the
    grouped kernel is compared with the CPU oracle on every particle."""
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
    del gx, gy
    torch.cuda.empty_cache()
    # eight channels against the CPU oracle on every particle (grouped tensors; stored values within 1e-2 of the scale of
    # the fp32 result on the same bfloat16 inputs)
    from oracle import oracle
    x8 = x[:, :8].contiguous()
    w8 = (torch.randn(8, levels, 8, 1, 5, 5, generator=torch.Generator().manual_seed(7)) * 0.1).to(torch.bfloat16).float()
    got = g8.ungroup(g8.conv_forward([apr], g8.regroup(x8), w8.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld)).cpu()
    ref8 = oracle.conv_forward([apr], x8.float().cpu(), w8, ld)
    for ch in range(8):
        assert float((got[0, ch].float() - ref8[0, ch]).abs().max()) <= 1e-2 * float(ref8[0, ch].abs().max())


def test_nuclei1024_whole_volume_conv_matches_the_oracle():
    """configs[3], whole 1024^3 volume (844 M particles): with few channels the CPU oracle finishes in seconds at this
    size too, so the three forward kernel families are compared with it on EVERY particle of the full-size APR -
    the pipelined kernel for narrow inputs (1 -> 4, fp32), the general matrix-core kernel (4 -> 4, fp32; rel 1e-5 of the
    output scale, the tolerance of the parity tests) and the bfloat16 kernel on grouped tensors in its 64-bit-address
    form, which only APRs of 2^28 particles and more take (8 -> 8; every stored value within 1e-2 of the scale of the
    fp32 result on the same bfloat16 inputs)."""
    from oracle import oracle
    _need(70)
    apr, _ = make_config("nuclei1024")
    apr.init_cuda()
    n = apr.total_number_particles()
    assert n >= 1 << 28
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    g = torch.Generator(device=DEV).manual_seed(11)
    gw = torch.Generator().manual_seed(12)

    def compare(got, ref, tol):
        for c in range(ref.shape[1]):                     # one channel at a time: no second copy of the tensors
            scale = max(float(ref[0, c].abs().max()), 1e-30)
            err = float((got[0, c].float() - ref[0, c]).abs().max())
            assert err <= tol * scale, f"channel {c}: max abs err {err:.3e} vs scale {scale:.3e}"

    x = torch.empty(1, 4, n, device=DEV).normal_(generator=g)
    xc = x.cpu()
    for cin, cout in ((1, 4), (4, 4)):
        w = torch.randn(cin, levels, cout, 3, 3, 3, generator=gw) * 0.2          # oracle layout, one stencil per level
        got = _ops.conv_forward([apr], x[:, :cin].contiguous(), w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld).cpu()
        ref = oracle.conv_forward([apr], xc[:, :cin].contiguous(), w, ld)
        compare(got, ref, 1e-5)
        del got, ref
    del x, xc
    torch.cuda.empty_cache()
    xb = torch.empty(1, 8, n, device=DEV, dtype=torch.bfloat16).normal_(generator=g)
    w = (torch.randn(8, levels, 8, 3, 3, 3, generator=gw) * 0.2).to(torch.bfloat16).float()
    yg = g8.conv_forward([apr], g8.regroup(xb), w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld)
    got = g8.ungroup(yg).cpu()
    del yg
    ref = oracle.conv_forward([apr], xb.float().cpu(), w, ld)
    compare(got, ref, 1e-2)


def test_nuclei1024_whole_volume_tree_operators_and_gradients_match_the_oracle():
    """configs[3], whole volume, against the oracle on every element: the mean-filled tree, max pool with its argmax
    and the upsampling of the pooled tensor are bit-identical (same candidate and summation order); the gradients of
    the 4 -> 4 fp32 stencil convolution are compared with the oracle run in float64 on the same values: input gradient to
    rel 1e-5 of its scale, weight gradient (8.4e8 terms per element) to 1e-4."""
    from oracle import oracle
    _need(70)
    apr, _ = make_config("nuclei1024")
    apr.init_cuda()
    n, c = apr.total_number_particles(), 2
    levels = apr.level_max() - apr.level_min() + 1
    ld0, ld1 = torch.zeros(1, dtype=torch.int32), torch.ones(1, dtype=torch.int32)
    g = torch.Generator(device=DEV).manual_seed(21)
    x = torch.empty(1, c, n, device=DEV).normal_(generator=g)
    xc = x.cpu()
    lib, plan, st = _ops._lib(), apr.plan(0), torch.cuda.current_stream().cuda_stream
    nt = _ops.tree_parts(apr, 0)
    tree = torch.empty(c, nt, device=DEV)
    assert lib.aprnet_fill_tree_mean_f32(plan, 0, x.data_ptr(), n, c, tree.data_ptr(), nt, st) == 0
    for ch in range(c):
        assert torch.equal(tree[ch].cpu(), oracle.fill_tree_mean(apr, xc[0, ch], 0))
    del tree
    pooled, idx = _ops.maxpool_forward([apr], x, ld0)
    ref, ref_idx = oracle.maxpool_forward([apr], xc, ld0)
    assert torch.equal(pooled.cpu(), ref) and torch.equal(idx.cpu(), ref_idx)
    del idx, ref_idx
    up = _ops.upsample_const_forward([apr], pooled, ld1)
    assert torch.equal(up.cpu(), oracle.upsample_const_forward([apr], ref, ld1))
    del up, pooled, ref, x, xc
    torch.cuda.empty_cache()
    x = torch.empty(1, 4, n, device=DEV).normal_(generator=g)
    gy = torch.empty(1, 4, n, device=DEV).normal_(generator=g)
    w = torch.randn(4, levels, 4, 3, 3, 3, generator=torch.Generator().manual_seed(22)) * 0.2
    gx, gw = _ops.conv_backward([apr], x, w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), gy, ld0)
    # the oracle in float64 on the same fp32 values: a weight gradient is a sum of 8.4e8 terms per element, which the
    # oracle's own fp32 running sums hold to about 2e-4 of its scale only
    gx_ref, gw_ref = oracle.conv_backward([apr], x.cpu().double(), w.double(), gy.cpu().double(), ld0)
    for ch in range(4):
        scale = float(gx_ref[0, ch].abs().max())
        assert float((gx[0, ch].cpu().double() - gx_ref[0, ch]).abs().max()) <= 1e-5 * scale
    gw = gw.permute(2, 0, 1, 3, 4, 5).cpu().double()
    # every element sums 8.4e8 products of fp32 values: 1e-4 of the scale (measured 1.7e-5; the reference's fp32 order 2e-4)
    assert float((gw - gw_ref).abs().max()) <= 1e-4 * float(gw_ref.abs().max())
