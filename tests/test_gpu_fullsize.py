"""Size-independent properties at the benchmark size (BASELINE configs[1]: APR of the seeded 256x512x512 blob
volume, 23 M particles), where the CPU oracle is too slow to be the checker: identity stencils, linearity,
adjointness of forward and backward, gather consistency of the pooling argmax, pool/upsample round trips.
A centre crop of the same volume is compared with the oracle directly."""
import pytest
import torch

from bench import build_workload
from pyapr import aprnet
from pyapr.aprnet import _ops
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def apr():
    a = build_workload("blobs512")
    a.init_cuda()
    return a


def _identity_weights(c, ksize, dtype=torch.float32):
    kz, kx, ky = ksize
    w = torch.zeros(1, c, c, kz, kx, ky, dtype=dtype)           # [S, Cout, Cin, k], one stencil for all levels
    for i in range(c):
        w[0, i, i, kz // 2, kx // 2, ky // 2] = 1
    return w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 5, 5)], ids=["333", "155"])
def test_identity_stencil_returns_input(apr, ksize, dtype):
    """A stencil whose only non-zero tap is the centre copies every particle and every downsampled particle:
    exact in both element types (one product with 1.0 per output)."""
    n, c = apr.total_number_particles(), 20
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, c, n, generator=g).to(dtype).to(DEV)
    levels = apr.level_max() - apr.level_min() + 1
    w = _identity_weights(c, ksize).expand(levels, -1, -1, -1, -1, -1).contiguous().to(DEV)
    for d in (0, 1):
        nd = _ops.number_particles(apr, d)
        xd = x[:, :, :nd].contiguous()
        y = _ops.conv_forward([apr], xd, w, torch.tensor([d], dtype=torch.int32))
        assert torch.equal(y, xd)


def test_forward_is_linear_and_backward_is_its_adjoint(apr):
    n, cin, cout = apr.total_number_particles(), 8, 24
    g = torch.Generator().manual_seed(1)
    ld = torch.zeros(1, dtype=torch.int32)
    levels = apr.level_max() - apr.level_min() + 1
    w = (torch.randn(levels, cout, cin, 3, 3, 3, generator=g) * 0.2).to(DEV)
    x1 = torch.randn(1, cin, n, generator=g).to(DEV)
    x2 = torch.randn(1, cin, n, generator=g).to(DEV)
    y1, y2 = _ops.conv_forward([apr], x1, w, ld), _ops.conv_forward([apr], x2, w, ld)
    y12 = _ops.conv_forward([apr], 2 * x1 - 3 * x2, w, ld)
    scale = float(y12.abs().max())
    assert float((y12 - (2 * y1 - 3 * y2)).abs().max()) <= 2e-5 * scale
    gy = torch.randn(1, cout, n, generator=g).to(DEV)
    gx, gw = _ops.conv_backward([apr], x1, w, gy, ld)
    # <conv(x), gy> == <x, conv'(gy)> == <w, dW>   (float64 accumulation of the inner products)
    lhs = float((y1.double() * gy.double()).sum())
    rhs_x = float((x1.double() * gx.double()).sum())
    rhs_w = float((w.double() * gw.double()).sum())
    ref = float((y1.double().abs() * gy.double().abs()).sum())
    assert abs(lhs - rhs_x) <= 1e-5 * ref
    assert abs(lhs - rhs_w) <= 1e-5 * ref


def test_fused_forward_equals_separate_passes(apr):
    """relu(conv(cat([x, x2])) + bias) from the fused entry point is bit-equal to the plain kernel on the
    concatenated tensor followed by a clamp (same products in the same order), fp32 and bfloat16 features."""
    n, c1, c2, cout = apr.total_number_particles(), 16, 16, 16
    g = torch.Generator().manual_seed(4)
    ld = torch.zeros(1, dtype=torch.int32)
    levels = apr.level_max() - apr.level_min() + 1
    w = (torch.randn(levels, cout, c1 + c2, 3, 3, 3, generator=g) * 0.1).to(DEV)
    bias = torch.randn(cout, generator=g).to(DEV)
    for dtype in (torch.float32, torch.bfloat16):
        xa = torch.randn(1, c1, n, generator=g).to(dtype).to(DEV)
        xb = torch.randn(1, c2, n, generator=g).to(dtype).to(DEV)
        fused = _ops.conv_forward([apr], xa, w, ld, bias, relu=True, x2=xb)
        plain = _ops.conv_forward([apr], torch.cat([xa, xb], dim=1), w, ld, bias)
        assert torch.equal(fused, torch.relu(plain))
        assert float(fused.float().abs().max()) > 0


def test_bf16_backward_is_adjoint_of_bf16_forward(apr):
    """bfloat16 features: <conv(x), gy> against <x, dX> and <w, dW> with the input gradient on the bfloat16 matrix
    cores; the three inner products agree to the bfloat16 rounding of the stored values (1e-2 of the absolute sum)."""
    n, cin, cout = apr.total_number_particles(), 16, 24
    g = torch.Generator().manual_seed(5)
    ld = torch.zeros(1, dtype=torch.int32)
    levels = apr.level_max() - apr.level_min() + 1
    w = (torch.randn(levels, cout, cin, 3, 3, 3, generator=g) * 0.2).to(torch.bfloat16).float().to(DEV)   # exact in bf16
    x = torch.randn(1, cin, n, generator=g).to(torch.bfloat16).to(DEV)
    gy = torch.randn(1, cout, n, generator=g).to(torch.bfloat16).to(DEV)
    y = _ops.conv_forward([apr], x, w, ld)
    gx, gw = _ops.conv_backward([apr], x, w, gy, ld)
    assert gx.dtype == torch.bfloat16 and gw.dtype == torch.float32
    lhs = float((y.double() * gy.double()).sum())
    rhs_x = float((x.double() * gx.double()).sum())
    rhs_w = float((w.double() * gw.double()).sum())
    ref = float((y.double().abs() * gy.double().abs()).sum())
    assert abs(lhs - rhs_x) <= 1e-2 * ref
    assert abs(lhs - rhs_w) <= 1e-2 * ref


def test_pool_argmax_gathers_and_upsample_round_trip(apr):
    n, c = apr.total_number_particles(), 6
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, c, n, generator=g).to(DEV)
    ld = torch.zeros(1, dtype=torch.int32)
    out, idx = _ops.maxpool_forward([apr], x, ld, 0.0)
    n1, ncopy = _ops.number_particles(apr, 1), apr.iterator().particles_level_end(apr.level_max() - 1)
    assert out.shape[2] == n1
    assert torch.equal(out[:, :, :ncopy], x[:, :, :ncopy])                     # coarser particles pass through
    pooled = out[:, :, ncopy:]
    assert torch.equal(pooled, torch.gather(x, 2, idx[:, :, ncopy:]))          # the value at the reported argmax
    up = _ops.upsample_const_forward([apr], out, torch.ones(1, dtype=torch.int32))
    assert up.shape[2] == n
    assert torch.equal(up[:, :, :ncopy], x[:, :, :ncopy])
    assert bool((up[:, :, ncopy:] >= x[:, :, ncopy:]).all())                   # every child sees its block's maximum
    again, idx2 = _ops.maxpool_forward([apr], up, ld, 0.0)
    assert torch.equal(again, out)                                             # pool(upsample(pool(x))) == pool(x)
    # backward of the pool scatters exactly the pooled gradients: sums agree per channel
    go = torch.randn(1, c, n1, generator=g).to(DEV)
    gi = _ops.maxpool_backward([apr], go, idx, ld)
    torch.testing.assert_close(gi.double().sum(dim=2), go.double().sum(dim=2), rtol=1e-9, atol=1e-6)


@pytest.mark.parametrize("kind", ["batch", "group"])
def test_particle_norm_at_full_size(apr, kind):
    """The streaming norm kernels on 16 x 23 M elements: the normalised rows have mean 0 and variance 1 in float64,
    outputs and input gradients agree with torch's own GPU modules (a different implementation and summation order)
    to 1e-5 / 1e-4 of the tensors' scale, and the input gradient is orthogonal to the constant and to the normalised
    input, as the derivative of a normalisation must be."""
    from apr_models.unet.particle_norm import ParticleBatchNorm, ParticleGroupNorm
    n, c = apr.total_number_particles(), 16
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(1, c, n, generator=g) * 2.5 + 7.0).to(DEV).requires_grad_(True)
    go = torch.randn(1, c, n, generator=g).to(DEV)
    if kind == "batch":
        mine, ref = ParticleBatchNorm(c).to(DEV), torch.nn.BatchNorm1d(c).to(DEV)
    else:
        mine, ref = ParticleGroupNorm(c, c).to(DEV), torch.nn.GroupNorm(c, c).to(DEV)
    y = mine(x)
    yd = y.detach().double()
    assert float(yd.mean(dim=2).abs().max()) < 1e-5 and float((yd.var(dim=2, unbiased=False) - 1).abs().max()) < 1e-4
    y.backward(go)
    gx = x.grad.detach().clone()
    x.grad = None
    yr = ref(x)
    yr.backward(go)
    assert float((y.detach() - yr.detach()).abs().max()) <= 1e-5 * float(yr.detach().abs().max())
    assert float((gx - x.grad).abs().max()) <= 1e-4 * float(x.grad.abs().max())
    gxd = gx.double()
    scale = float(gxd.abs().sum(dim=2).max())
    assert float(gxd.sum(dim=2).abs().max()) <= 1e-5 * scale
    assert float((gxd * yd).sum(dim=2).abs().max()) <= 1e-5 * scale * float(yd.abs().max())


def test_centre_crop_against_oracle():
    """The benchmark's CPU-baseline sample (128x256x256 crop, 3 M particles) through both implementations."""
    apr = build_workload("blobs512", crop=(128, 256, 256))
    apr.init_cuda()
    n, cin, cout = apr.total_number_particles(), 4, 6
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, cin, n, generator=g)
    w = torch.randn(cin, 2, cout, 3, 3, 3, generator=g) * 0.2
    ld = torch.zeros(1, dtype=torch.int32)
    w_exp = oracle.restrict_kernel_forward(w, apr.level_max() - apr.level_min() + 1)
    ref = oracle.conv_forward([apr], x, w_exp, ld)
    got = _ops.conv_forward([apr], x.to(DEV), w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld)
    assert float((got.cpu() - ref).abs().max()) <= 1e-5 * float(ref.abs().max())


def test_backward_repeats_bit_for_bit(apr):
    """Gradients do not depend on scheduling: the weight gradient is summed from per-workgroup partial sums in a
    fixed order, every element of the input gradient receives at most two atomic contributions (fp32 addition of
    two values onto zero is commutative) before the tree gradient is pushed down in a fixed order.  Two runs of the
    32 -> 32 backward on the 23 M-particle APR are compared with torch.equal."""
    n, c = apr.total_number_particles(), 32
    g = torch.Generator().manual_seed(7)
    ld = torch.zeros(1, dtype=torch.int32)
    levels = apr.level_max() - apr.level_min() + 1
    w = (torch.randn(levels, c, c, 3, 3, 3, generator=g) * 0.1).to(DEV)
    x = torch.randn(1, c, n, generator=g).to(DEV)
    gy = torch.randn(1, c, n, generator=g).to(DEV)
    gx1, gw1 = _ops.conv_backward([apr], x, w, gy, ld)
    gx2, gw2 = _ops.conv_backward([apr], x, w, gy, ld)
    assert torch.equal(gw1, gw2)
    assert torch.equal(gx1, gx2)
