"""Every BASELINE configuration through the HIP path.

configs[0] (spheres128) runs at its full size against the oracle and against the committed golden summary.  The other
four are too large for the CPU oracle (and, at full size, for a test's time budget: `bench.py --config NAME` runs
them whole), so each is exercised twice: a scaled replica of the configuration (same generator, same blob density,
every dimension shrunk by the stated factor) at a size of millions of particles through size-independent properties,
and a smaller replica compared with the oracle directly."""
import json
import os

import pytest
import torch

from bench import build_workload, spheres128_inputs
from oracle import oracle
from oracle_modules import OracleConv, OracleMaxPool, OracleUpSample
from pyapr import aprnet
from pyapr.aprnet import _ops
from pyapr.synthetic import make_config

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "spheres128_conv_1to16.json")


def _rel(got, ref):
    return float((got - ref).abs().max()) / max(float(ref.abs().max()), 1e-30)


# ------------------------------------------------------------------------------------------------ configs[0]
def test_spheres128_full_size_against_oracle_and_golden():
    """APRConv 3x3x3 1 -> 16 fp32 with bias on the whole 128^3 configuration: every output value against the oracle
    (1e-5 of the output scale) and the committed summary (sums, first / last 64 values per channel)."""
    apr, x, w, b = spheres128_inputs()
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    w_cpu = w.permute(2, 0, 1, 3, 4, 5).contiguous()
    ref = oracle.conv_forward([apr], x, oracle.restrict_kernel_forward(w_cpu, levels), ld) + b.view(1, -1, 1)
    got = _ops.conv_forward([apr], x.to(DEV), _ops.restrict_kernel_forward(w.to(DEV), levels), ld, bias=b.to(DEV)).cpu()
    assert _rel(got, ref) <= 1e-5
    gold = json.load(open(GOLD))
    n = apr.total_number_particles()
    assert gold["n_particles"] == n
    scale = max(gold["abs_max"])
    gd = got[0].double()
    for c in range(16):
        assert abs(float(gd[c].sum()) - gold["sum"][c]) <= 1e-5 * scale * n ** 0.5 * 16
        assert float((gd[c, :64] - torch.tensor(gold["first64"][c], dtype=torch.float64)).abs().max()) <= 1e-5 * scale
        assert float((gd[c, -64:] - torch.tensor(gold["last64"][c], dtype=torch.float64)).abs().max()) <= 1e-5 * scale


# ------------------------------------------------------------------------------------------------ configs[1]
def test_blobs512_chain_on_a_crop_against_oracle():
    """conv(32 -> 32) -> ReLU -> MaxPool -> UpSampleConst, forward and backward (grad input, grad weight), on the
    64 x 128 x 128 centre crop of the configs[1] volume against the oracle chain.  Both sides are fed the same
    intermediate tensors (the oracle's), because a 1e-6 difference in the convolution output may flip a ReLU mask or a
    pooling argmax and move a whole gradient entry: forward values to 1e-5 of their scale, argmax and the pool /
    upsample gradients bit-exact, convolution gradients to 1e-5."""
    apr = build_workload("blobs512", crop=(64, 128, 128))
    n, c = apr.total_number_particles(), 32
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, c, n, generator=g)
    conv = aprnet.cuda.APRConv(c, c, nstencils=2).to(DEV)
    ld0, ld1 = torch.zeros(1, dtype=torch.int32), torch.ones(1, dtype=torch.int32)
    # oracle chain, forward and backward
    xc = x.clone().requires_grad_(True)
    wc = conv.weight.detach().cpu().permute(2, 0, 1, 3, 4, 5).contiguous().requires_grad_(True)
    yr = OracleConv.apply(xc, wc, conv.bias.detach().cpu(), [apr], ld0.clone())
    ar = torch.relu(yr)
    pr, ir = oracle.maxpool_forward([apr], ar.detach(), ld0)
    ur = oracle.upsample_const_forward([apr], pr, ld1)
    go = torch.randn(ur.shape, generator=g)
    gpr = oracle.upsample_const_backward([apr], go, ld1)
    gar = oracle.maxpool_backward([apr], gpr, ir, ld0)
    gyr = gar * (yr.detach() > 0)
    yr.backward(gyr)
    # HIP chain on the same inputs
    xd = x.to(DEV).requires_grad_(True)
    y = conv(xd, [apr], ld0.clone())
    assert _rel(y.detach().cpu(), yr.detach()) <= 1e-5
    p, idx = _ops.maxpool_forward([apr], ar.detach().to(DEV), ld0)
    assert torch.equal(p.cpu(), pr) and torch.equal(idx.cpu(), ir)
    u = _ops.upsample_const_forward([apr], p, ld1)
    assert torch.equal(u.cpu(), ur)
    gp = _ops.upsample_const_backward([apr], go.to(DEV), ld1)
    assert _rel(gp.cpu(), gpr) <= 1e-6
    ga = _ops.maxpool_backward([apr], gp, idx, ld0)
    assert torch.equal(ga.cpu(), oracle.maxpool_backward([apr], gp.cpu(), ir, ld0))
    y.backward(gyr.to(DEV))
    assert _rel(xd.grad.cpu(), xc.grad) <= 1e-5
    assert _rel(conv.weight.grad.cpu(), wc.grad.permute(1, 2, 0, 3, 4, 5)) <= 1e-5
    # and the modules composed end to end run, with the in-place level_deltas contract
    ld = torch.zeros(1, dtype=torch.int32)
    out = aprnet.cuda.UpSampleConst()(aprnet.cuda.MaxPool()(torch.relu(conv(xd, [apr], ld)), [apr], ld), [apr], ld)
    assert int(ld[0]) == 0 and out.shape == (1, c, n)
    out.sum().backward()
    assert torch.isfinite(xd.grad).all()


# ------------------------------------------------------------------------------------------------ configs[2]
@pytest.fixture(scope="module")
def nuclei2048_quarter():
    apr, _ = make_config("nuclei2048", scale=0.25)            # 128 x 512 x 512 replica, ~5 M particles
    apr.init_cuda()
    return apr


def test_nuclei2048_tree_fill_and_parent_reading_conv_properties(nuclei2048_quarter):
    """Tree fill + 3x3x3 convolution at 16 channels fp32 on the quarter-scale replica of configs[2]: the mean fill of a
    constant is that constant on every tree node, bit for bit; a convolution with the all-ones / 27 stencil of a
    constant field returns the constant away from the image faces (it reads coarser particles and filled tree parents
    alike); the identity stencil copies the input; repeats are bit-identical."""
    apr = nuclei2048_quarter
    n, c = apr.total_number_particles(), 16
    nt = _ops.tree_parts(apr, 0)
    lib, plan, st = _ops._lib(), apr.plan(0), torch.cuda.current_stream().cuda_stream
    x = torch.full((1, c, n), 3.25, device=DEV)
    tree = torch.empty(c, nt, device=DEV)
    assert lib.aprnet_fill_tree_mean_f32(plan, 0, x.data_ptr(), n, c, tree.data_ptr(), nt, st) == 0
    assert bool((tree == 3.25).all())
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    w = torch.zeros(levels, c, c, 3, 3, 3)
    for i in range(c):
        w[:, i, i] = 1.0 / 27
    y = _ops.conv_forward([apr], x, w.to(DEV), ld)
    # interior particles see 27 cells of the constant; particles on a face see fewer (zero padding): never more
    assert float(y.max()) <= 3.25 * (1 + 1e-6)
    interior = (y[0, 0] - 3.25).abs() <= 1e-5 * 3.25
    assert float(interior.float().mean()) > 0.9
    g = torch.Generator().manual_seed(2)
    xr = torch.randn(1, c, n, generator=g).to(DEV)
    wi = torch.zeros(levels, c, c, 3, 3, 3)
    for i in range(c):
        wi[:, i, i, 1, 1, 1] = 1
    assert torch.equal(_ops.conv_forward([apr], xr, wi.to(DEV), ld), xr)
    wr = (torch.randn(levels, c, c, 3, 3, 3, generator=g) * 0.1).to(DEV)
    assert torch.equal(_ops.conv_forward([apr], xr, wr, ld), _ops.conv_forward([apr], xr, wr, ld))


def test_nuclei2048_small_replica_against_oracle():
    """The same pair of operators on the 1/16-scale replica (32 x 128 x 128, sinusoidal background included): tree
    means bit-identical to the oracle, convolution to 1e-5 of the output scale."""
    apr, _ = make_config("nuclei2048", scale=0.0625)
    n, c = apr.total_number_particles(), 16
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, c, n, generator=g)
    nt = _ops.tree_parts(apr, 0)
    apr.init_cuda()
    lib, plan, st = _ops._lib(), apr.plan(0), torch.cuda.current_stream().cuda_stream
    xd = x.to(DEV)
    tree = torch.empty(c, nt, device=DEV)
    assert lib.aprnet_fill_tree_mean_f32(plan, 0, xd.data_ptr(), n, c, tree.data_ptr(), nt, st) == 0
    for ch in (0, c - 1):
        assert torch.equal(tree[ch].cpu(), oracle.fill_tree_mean(apr, x[0, ch].contiguous(), 0)[:nt])
    w = torch.randn(c, 2, c, 3, 3, 3, generator=g) * 0.1
    ld = torch.zeros(1, dtype=torch.int32)
    w_exp = oracle.restrict_kernel_forward(w, apr.level_max() - apr.level_min() + 1)
    ref = oracle.conv_forward([apr], x, w_exp, ld)
    got = _ops.conv_forward([apr], xd, w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld)
    assert _rel(got.cpu(), ref) <= 1e-5


# ------------------------------------------------------------------------------------------------ configs[3]
def _unet():
    from bench import make_unet
    return make_unet("cpu")


def test_nuclei1024_unet_on_the_eighth_scale_replica_against_oracle():
    """APR-UNet forward (16-32-64-128, He init seed 0, norms folded) on the 128^3 replica of configs[3], 1.5 M particles:
    fp32 against the network composed from oracle operators (2e-5 of the output scale after 18 layers), bfloat16
    features against the same reference (2e-2)."""
    from test_gpu_unet import reference_forward
    apr, parts = make_config("nuclei1024", scale=0.125)
    x = (torch.from_numpy(parts).float() / 1000.0).view(1, 1, -1)
    model = _unet()
    with torch.no_grad():
        ref = reference_forward(model, x, [apr])
        model = model.to(DEV)
        got = model(x.to(DEV), [apr]).cpu()
        gotb = model(x.to(DEV).to(torch.bfloat16), [apr]).float().cpu()
    assert _rel(got, ref) <= 2e-5
    assert _rel(gotb, ref) <= 2e-2


def test_nuclei1024_unet_on_the_quarter_scale_replica_properties():
    """The same network on the 256^3 replica (13 M particles): finite, bit-identical from run to run, bfloat16 features
    within 2e-2 of the fp32 result, and every intermediate tensor released (peak memory far below the sum of all
    stage outputs)."""
    apr, parts = make_config("nuclei1024", scale=0.25)
    n = apr.total_number_particles()
    x = (torch.from_numpy(parts).float() / 1000.0).view(1, 1, -1).to(DEV)
    model = _unet().to(DEV)
    with torch.no_grad():
        y1 = model(x, [apr])
        y2 = model(x, [apr])
        yb = model(x.to(torch.bfloat16), [apr])
    assert y1.shape == (1, 3, n) and torch.isfinite(y1).all()
    assert torch.equal(y1, y2)
    assert _rel(yb.float(), y1) <= 2e-2


def test_nuclei1024_whole_volume_grouped_path_against_plane_path():
    """The whole 1024^3 volume (844 M particles): with bfloat16 features the network keeps its tensors grouped by eight
    channels, and from 2^28 particles on the convolution addresses its 16-byte items with 64 bits.  Checked against the
    plane path of the same build over the whole particle range (the two differ in the summation order and the weight
    rounding of the 1x1x1 convolutions: 2e-2 of the output scale, as for the small replicas)."""
    if torch.cuda.get_device_properties(0).total_memory < 200e9:
        pytest.skip("needs about 100 GB of device memory")
    apr, parts = make_config("nuclei1024")
    n = apr.total_number_particles()
    assert n >= (1 << 28)
    x = (torch.from_numpy(parts).float() / 1000.0).view(1, 1, -1).to(DEV).to(torch.bfloat16)
    model = _unet().to(DEV)
    with torch.no_grad():
        model.use_grouped = True
        yg = model(x, [apr])
        model.use_grouped = False
        yp = model(x, [apr])
    assert yg.shape == (1, 3, n) and yg.dtype == torch.bfloat16
    scale = float(yp.float().abs().max())
    assert scale > 0 and torch.isfinite(yg.float()).all()
    step = 1 << 26
    worst = max(float((yg[:, :, lo:lo + step].float() - yp[:, :, lo:lo + step].float()).abs().max()) for lo in range(0, n, step))
    assert worst <= 2e-2 * scale


# ------------------------------------------------------------------------------------------------ configs[4]
def test_spots16k_small_replica_against_oracle():
    """APRConv 1x5x5 64 -> 64 with bfloat16 features on the 256^2 replica of configs[4] (59 k particles): forward,
    input gradient and weight gradient against the fp32 oracle, 2e-2 of each tensor's scale (inputs and weights are
    exact in bfloat16, so only the stored outputs and gradients are rounded)."""
    apr, _ = make_config("spots16k", scale=1 / 64)
    n, c = apr.total_number_particles(), 64
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, c, n, generator=g).to(torch.bfloat16)
    gy = torch.randn(1, c, n, generator=g).to(torch.bfloat16)
    w = (torch.randn(c, 2, c, 1, 5, 5, generator=g) * 0.05).to(torch.bfloat16).float()
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    w_exp = oracle.restrict_kernel_forward(w, levels).to(torch.bfloat16).float()
    ref = oracle.conv_forward([apr], x.float(), w_exp, ld)
    rgx, rgw = oracle.conv_backward([apr], x.float(), w_exp, gy.float(), ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    got = _ops.conv_forward([apr], x.to(DEV), wd, ld)
    gx, gw = _ops.conv_backward([apr], x.to(DEV), wd, gy.to(DEV), ld)
    assert got.dtype == torch.bfloat16 and gx.dtype == torch.bfloat16
    assert _rel(got.float().cpu(), ref) <= 2e-2
    assert _rel(gx.float().cpu(), rgx) <= 2e-2
    assert _rel(gw.cpu(), rgw.permute(1, 2, 0, 3, 4, 5)) <= 2e-2


def test_spots16k_eighth_scale_replica_adjoint_and_identity():
    """The layer on the 2048^2 replica (3.8 M particles, level_max 11): the identity stencil copies bfloat16 features
    exactly, and <conv(x), gy> = <x, dX> = <w, dW> to the bfloat16 rounding of the stored tensors."""
    apr, _ = make_config("spots16k", scale=0.125)
    n, c = apr.total_number_particles(), 64
    levels = apr.level_max() - apr.level_min() + 1
    ld = torch.zeros(1, dtype=torch.int32)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(1, c, n, generator=g).to(torch.bfloat16).to(DEV)
    wi = torch.zeros(levels, c, c, 1, 5, 5)
    for i in range(c):
        wi[:, i, i, 0, 2, 2] = 1
    assert torch.equal(_ops.conv_forward([apr], x, wi.to(DEV), ld), x)
    w = (torch.randn(levels, c, c, 1, 5, 5, generator=g) * 0.05).to(torch.bfloat16).float().to(DEV)
    gy = torch.randn(1, c, n, generator=g).to(torch.bfloat16).to(DEV)
    y = _ops.conv_forward([apr], x, w, ld)
    gx, gw = _ops.conv_backward([apr], x, w, gy, ld)
    lhs = float((y.double() * gy.double()).sum())
    ref = float((y.double().abs() * gy.double().abs()).sum())
    assert abs(lhs - float((x.double() * gx.double()).sum())) <= 1e-2 * ref
    assert abs(lhs - float((w.double() * gw.double()).sum())) <= 1e-2 * ref
