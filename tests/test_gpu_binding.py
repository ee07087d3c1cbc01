"""The compiled pybind11 module `_pyaprwrapper` exposes the reference's native function names
(wrappers/pythonBind.cpp:144-182) over the C ABI.  Every function is called by that name with the reference's
argument order; results must equal the ctypes host layer's bit for bit (same C entry points) and a sample is held
to the oracle."""
import pytest
import torch

import apr_cases
from oracle import oracle
from pyapr.aprnet import _ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def w():
    import _pyaprwrapper
    return _pyaprwrapper.aprnet


def _case(c, dtype=torch.float32):
    aprs = [apr_cases.get("3d_s"), apr_cases.get("3d_t")]
    ld = torch.tensor([0, 1], dtype=torch.int32)
    sizes = [oracle.number_parts(a, int(d)) for a, d in zip(aprs, ld)]
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, c, max(sizes), dtype=dtype, generator=g)
    for i, n in enumerate(sizes):
        x[i, :, n:] = 0
    return aprs, ld, x, g


def test_cuda_flavour_convolutions_by_reference_name(w):
    aprs, ld, x, g = _case(5)
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    wt = torch.randn(2, 7, 5, 3, 3, 3, generator=g).to(DEV)              # [S, Cout, Cin, 3, 3, 3]
    xd = x.to(DEV)
    w_exp = w.cuda.restrict_kernel333_forward(wt, levels)
    assert torch.equal(w_exp, _ops.restrict_kernel_forward(wt, levels))
    y = w.cuda.conv333_forward(aprs, xd, w_exp, ld)
    assert torch.equal(y, _ops.conv_forward(aprs, xd, w_exp, ld))
    ref = oracle.conv_forward(aprs, x, w_exp.cpu().permute(2, 0, 1, 3, 4, 5).contiguous(), ld)
    assert float((y.cpu() - ref).abs().max()) <= 1e-5 * float(ref.abs().max())
    gy = torch.randn(y.shape, generator=g).to(DEV)
    gx, gw = w.cuda.conv333_backward(aprs, xd, w_exp, gy, ld)
    gx2, gw2 = _ops.conv_backward(aprs, xd, w_exp, gy, ld)
    assert torch.equal(gx, gx2) and torch.equal(gw, gw2)
    gw_small = w.cuda.restrict_kernel333_backward(gw, 2)
    assert torch.equal(gw_small, _ops.restrict_kernel_backward(gw, 2))
    w1 = torch.randn(2, 4, 5, 1, 1, 1, generator=g).to(DEV)
    y1 = w.cuda.conv111_forward(aprs, xd, w1, ld)
    assert torch.equal(y1, _ops.conv_forward(aprs, xd, w1, ld))
    g1 = torch.randn(y1.shape, generator=g).to(DEV)
    a, b = w.cuda.conv111_backward(aprs, xd, w1, g1, ld)
    a2, b2 = _ops.conv_backward(aprs, xd, w1, g1, ld)
    assert torch.equal(a, a2) and float((b - b2).abs().max()) <= 1e-5 * float(b2.abs().max())     # 1x1x1 weight gradient adds atomically


def test_cuda_flavour_pool_upsample_pixels_by_reference_name(w):
    aprs, ld, x, g = _case(3)
    xd = x.to(DEV)
    out, idx = w.cuda.maxpool_forward_cuda(aprs, xd, ld)
    o2, i2 = _ops.maxpool_forward(aprs, xd, ld, 0.0)
    assert torch.equal(out, o2) and torch.equal(idx, i2)
    pr, ir = oracle.maxpool_forward(aprs, x, ld)
    n1 = [oracle.number_parts(a, int(d) + 1) for a, d in zip(aprs, ld)]
    for b, n in enumerate(n1):
        assert torch.equal(out[b, :, :n].cpu(), pr[b, :, :n]) and torch.equal(idx[b, :, :n].cpu(), ir[b, :, :n])
    go = torch.randn(out.shape, generator=g).to(DEV)
    assert torch.equal(w.cuda.maxpool_backward_cuda(aprs, go, idx, ld), _ops.maxpool_backward(aprs, go, idx, ld))
    ld1 = ld + 1
    up = w.cuda.upsample_const_forward(aprs, out, ld1)
    assert torch.equal(up, _ops.upsample_const_forward(aprs, out, ld1))
    assert torch.equal(w.cuda.upsample_const_backward(aprs, xd, ld1), _ops.upsample_const_backward(aprs, xd, ld1))
    with pytest.raises(ValueError, match="level_delta > 0"):
        w.cuda.upsample_const_forward(aprs, xd, ld)
    one = [aprs[0]]
    ld0 = torch.zeros(1, dtype=torch.int32)
    x0 = xd[:1, :, :aprs[0].total_number_particles()].contiguous()
    img = w.cuda.reconstruct_forward(one, x0, ld0)
    assert torch.equal(img, _ops.reconstruct_forward(one, x0, ld0))
    back = w.cuda.sample_particles_forward(one, img, ld0)
    torch.testing.assert_close(back, x0, rtol=1e-6, atol=1e-6)           # sample(reconstruct(x)) == x, test_aprnet.py:272-285
    gi = torch.randn(img.shape, generator=g).to(DEV)
    assert torch.equal(w.cuda.reconstruct_backward(one, gi, ld0), _ops.reconstruct_backward(one, gi, ld0))
    assert torch.equal(w.cuda.sample_particles_backward(one, x0, ld0), _ops.sample_particles_backward(one, x0, ld0))


@pytest.mark.parametrize("k", [(1, 1, 1), (3, 3, 3), (1, 3, 3), (5, 5, 5), (1, 5, 5)], ids=lambda k: "%d%d%d" % k)
def test_cpu_flavour_names_take_the_reference_weight_layout(w, k):
    """aprnet.conv.convolve###_forward / _backward and restrict_kernel### with weights [Cin, S, Cout, kz, kx, ky]
    (conv.py:164), against the oracle, which follows the same layout."""
    aprs, ld, x, g = _case(3, torch.float64)
    name = "%d%d%d" % k
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    wt = torch.randn(3, 2, 4, *k, dtype=torch.float64, generator=g)       # [Cin, S, Cout, k]
    if k == (1, 1, 1):
        w_exp, w_exp_ref = wt.to(DEV), wt
    else:
        w_exp = getattr(w.conv, f"restrict_kernel{name}_forward")(wt.to(DEV), levels)
        w_exp_ref = oracle.restrict_kernel_forward(wt, levels)
        torch.testing.assert_close(w_exp.cpu(), w_exp_ref, rtol=1e-12, atol=1e-12)
    y = getattr(w.conv, f"convolve{name}_forward")(aprs, x.to(DEV), w_exp, ld)
    ref = oracle.conv_forward(aprs, x, w_exp_ref, ld)
    torch.testing.assert_close(y.cpu(), ref, rtol=1e-11, atol=1e-11 * float(ref.abs().max()))
    gy = torch.randn(y.shape, dtype=torch.float64, generator=g)
    gx, gw = getattr(w.conv, f"convolve{name}_backward")(aprs, x.to(DEV), w_exp, gy.to(DEV), ld)
    gx_ref, gw_ref = oracle.conv_backward(aprs, x, w_exp_ref, gy, ld)
    torch.testing.assert_close(gx.cpu(), gx_ref, rtol=1e-10, atol=1e-10 * float(gx_ref.abs().max()))
    torch.testing.assert_close(gw.cpu(), gw_ref, rtol=1e-10, atol=1e-10 * float(gw_ref.abs().max()))
    if k != (1, 1, 1):
        back = getattr(w.conv, f"restrict_kernel{name}_backward")(gw, 2)
        torch.testing.assert_close(back.cpu(), oracle.restrict_kernel_backward(gw_ref, 2), rtol=1e-10, atol=1e-10 * float(gw_ref.abs().max()))


def test_cpu_flavour_pool_upsample_utils(w):
    aprs, ld, x, g = _case(2)
    out, idx = w.pool.maxpool_forward(aprs, x.to(DEV), ld)
    pr, ir = oracle.maxpool_forward(aprs, x, ld)
    assert torch.equal(out.cpu(), pr) and torch.equal(idx.cpu(), ir)          # padding slots hold -1e17 (maxpool.hpp:51)
    go = torch.randn(out.shape, generator=g)
    assert torch.equal(w.pool.maxpool_backward(aprs, go.to(DEV), idx, ld).cpu(), oracle.maxpool_backward(aprs, go, ir, ld))
    up = w.upsample.upsample_const_forward(aprs, out, ld + 1)
    assert torch.equal(up.cpu(), oracle.upsample_const_forward(aprs, pr, ld + 1))
    gb = w.upsample.upsample_const_backward(aprs, x.to(DEV), ld + 1)
    torch.testing.assert_close(gb.cpu(), oracle.upsample_const_backward(aprs, x, ld + 1), rtol=1e-6, atol=1e-6)
    for a in aprs:
        for d in range(2):
            assert w.utils.number_particles(a, d) == w.utils.number_parts(a, d) == oracle.number_parts(a, d)
            assert w.utils.number_particles_after_pooling(a, d) == oracle.number_parts(a, d + 1)
            assert w.utils.number_particles_after_upsampling(a, d + 1) == oracle.number_parts(a, d)
    with pytest.raises(RuntimeError, match="CUDA tensor"):
        w.pool.maxpool_forward(aprs, x, ld)
    with pytest.raises(ValueError, match="does not match"):
        w.cuda.conv333_forward(aprs, x.to(DEV), torch.zeros(1, 4, 7, 3, 3, 3, device=DEV), ld)
