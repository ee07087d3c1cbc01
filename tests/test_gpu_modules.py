"""GPU tests of the module layer, shaped like the reference's own tests (pyapr/tests/test_aprnet.py):
float64 gradchecks of the device modules, the CPU-flavour vs device-flavour comparison with Cin = Cout =
33 and three stencils (:133-179, here both flavours run on the GPU and the oracle is the third party), the
Reconstruct/SampleParticles round trip (:272-285), the in-place level_deltas contract, and error behaviour."""
import pytest
import torch
from torch.autograd import gradcheck

import apr_cases
from oracle import oracle
from pyapr import aprnet

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _batch(names_d, channels, dtype=torch.float64, seed=0):
    aprs = [apr_cases.get(n) for n, _ in names_d]
    ld = torch.tensor([d for _, d in names_d], dtype=torch.int32)
    sizes = [oracle.number_parts(a, int(d)) for a, d in zip(aprs, ld)]
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(len(aprs), channels, max(sizes), dtype=dtype, generator=g)
    for i, n in enumerate(sizes):
        x[i, :, n:] = 0
    for a in aprs:
        a.init_cuda()
    return x.to(DEV).requires_grad_(True), aprs, ld


CASES_2D = [[("2d_a", 0)], [("2d_a", 1), ("2d_b", 2)]]
CASES_3D = [[("3d_a", 0)], [("3d_b", 1)], [("3d_a", 2), ("3d_c", 2)]]
IDS = lambda b: "+".join(f"{n}@{d}" for n, d in b)


@pytest.mark.parametrize("bt", CASES_2D + CASES_3D, ids=IDS)
def test_maxpool_gradcheck(bt):
    model = aprnet.cuda.MaxPool().double()
    model.increment_level_deltas = False
    x, aprs, ld = _batch(bt, 2)
    with torch.no_grad():
        x += 10 * torch.arange(x.shape[2], dtype=torch.float64, device=DEV)
    assert gradcheck(model, (x, aprs, ld), eps=1e-3)


@pytest.mark.parametrize("bt", CASES_3D, ids=IDS)
@pytest.mark.parametrize("k", [1, 3, 5])
def test_conv3d_gradcheck(bt, k):
    x, aprs, ld = _batch(bt, 2)
    model = aprnet.cuda.APRConv(2, 1, kernel_size=(k, k, k), nstencils=6 if k == 1 else 2).double().to(DEV)
    assert gradcheck(model, (x, aprs, ld), eps=1e-5)
    params = [model.weight, model.bias]
    assert gradcheck(lambda w, b: aprnet.functional.ConvFunction.apply(x.detach(), w, b, aprs, ld, model.weight_layout),
                     params, eps=1e-5)


@pytest.mark.parametrize("bt", CASES_2D, ids=IDS)
@pytest.mark.parametrize("k", [1, 3, 5])
def test_conv2d_gradcheck_cpu_flavour_layout(bt, k):
    """the (commented-out) CPU-flavour gradchecks of test_aprnet.py:94-104: kernel (1,k,k), nstencils 3"""
    x, aprs, ld = _batch(bt, 2)
    model = aprnet.APRConv(in_channels=2, out_channels=2, nstencils=3, kernel_size=(1, k, k), bias=True).double().to(DEV)
    assert gradcheck(model, (x, aprs, ld), eps=1e-6)
    assert gradcheck(lambda w: aprnet.functional.ConvFunction.apply(x.detach(), w, None, aprs, ld, model.weight_layout),
                     [model.weight], eps=1e-6)


@pytest.mark.parametrize("bt", [[("3d_a", 1)], [("3d_b", 1), ("3d_c", 2)], [("2d_a", 1), ("2d_b", 2)]], ids=IDS)
def test_upsample_gradcheck(bt):
    x, aprs, ld = _batch(bt, 2)
    model = aprnet.cuda.UpSampleConst().double()
    model.decrement_level_deltas = False
    assert gradcheck(model, (x, aprs, ld), eps=1e-3)


@pytest.mark.parametrize("bt", [[("3d_a", 0)], [("3d_b", 1)], [("3d_c", 2), ("3d_c", 2)]], ids=IDS)
def test_reconstruct_sample_gradcheck_and_roundtrip(bt):
    x, aprs, ld = _batch(bt, 2)
    recon, sample = aprnet.cuda.Reconstruct(), aprnet.cuda.SampleParticles()
    assert gradcheck(recon, (x, aprs, ld), eps=1e-5)
    img = torch.rand_like(recon(x.detach(), aprs, ld)).requires_grad_(True)
    assert gradcheck(sample, (img, aprs, ld), eps=1e-5)
    assert torch.allclose(sample(recon(x, aprs, ld), aprs, ld), x)


@pytest.mark.parametrize("bt", CASES_3D, ids=IDS)
def test_conv333_device_flavour_vs_cpu_flavour_vs_oracle(bt):
    cin = cout = 33
    x, aprs, ld = _batch(bt, cin)
    model_dev = aprnet.cuda.APRConv(cin, cout, nstencils=3).double().to(DEV)
    out_dev = model_dev(x, aprs, ld)
    go = torch.rand_like(out_dev)
    out_dev.backward(go, inputs=(x, model_dev.weight, model_dev.bias))
    dx_dev, dw_dev, db_dev = x.grad.clone(), model_dev.weight.grad.clone(), model_dev.bias.grad.clone()

    model_cpu = aprnet.APRConv(cin, cout, nstencils=3).double().to(DEV)
    model_cpu.weight = torch.nn.Parameter(model_dev.weight.detach().permute(2, 0, 1, 3, 4, 5).contiguous())
    model_cpu.bias = torch.nn.Parameter(model_dev.bias.detach().clone())
    x.grad = None
    out_cpu = model_cpu(x, aprs, ld)
    out_cpu.backward(go, inputs=(x, model_cpu.weight, model_cpu.bias))
    assert torch.allclose(out_dev, out_cpu)
    assert torch.allclose(dw_dev, model_cpu.weight.grad.permute(1, 2, 0, 3, 4, 5))
    assert torch.allclose(db_dev, model_cpu.bias.grad)
    assert torch.allclose(dx_dev, x.grad)

    # third party: the CPU oracle with the reference's arithmetic
    w_cpu = model_cpu.weight.detach().cpu()
    num_levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    w_exp = oracle.restrict_kernel_forward(w_cpu, num_levels)
    ref = oracle.conv_forward(aprs, x.detach().cpu(), w_exp, ld) + model_cpu.bias.detach().cpu().view(1, -1, 1)
    gx_ref, gw_exp_ref = oracle.conv_backward(aprs, x.detach().cpu(), w_exp, go.cpu(), ld)
    gw_ref = oracle.restrict_kernel_backward(gw_exp_ref, 3)
    torch.testing.assert_close(out_cpu.detach().cpu(), ref, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(x.grad.cpu(), gx_ref, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(model_cpu.weight.grad.cpu(), gw_ref, rtol=1e-10, atol=1e-9)


def test_level_deltas_are_mutated_in_place_after_the_call():
    """pool.py:13-14 / upsample.py:13-14: the network shares one level_deltas tensor."""
    x, aprs, ld = _batch([("3d_a", 0), ("3d_c", 1)], 2, dtype=torch.float32)
    pool, up = aprnet.cuda.MaxPool(), aprnet.cuda.UpSampleConst()
    y = pool(x, aprs, ld)
    assert ld.tolist() == [1, 2]
    assert y.shape[2] == max(oracle.number_parts(aprs[0], 1), oracle.number_parts(aprs[1], 2))
    z = up(y, aprs, ld)
    assert ld.tolist() == [0, 1]
    assert z.shape == x.shape
    # backward uses the pre-mutation clones
    z.sum().backward()
    assert x.grad is not None and x.grad.shape == x.shape
    pool.increment_level_deltas = False
    pool(x, aprs, ld)
    assert ld.tolist() == [0, 1]


def test_error_behaviour():
    x, aprs, ld = _batch([("3d_a", 0)], 2, dtype=torch.float32)
    with pytest.raises(ValueError, match="does not match"):               # conv.hpp:63-66
        aprnet.cuda.APRConv(3, 2).to(DEV)(x, aprs, ld)
    with pytest.raises(ValueError, match="downsampled"):                  # upsample.hpp:49-54
        aprnet.cuda.UpSampleConst()(x, aprs, ld)
    with pytest.raises(RuntimeError, match="contiguous"):                 # CHECK_CONTIGUOUS
        aprnet._ops.maxpool_forward(aprs, x.detach().transpose(1, 2).contiguous().transpose(1, 2), ld)
    big = torch.tensor([aprs[0].level_max()], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="level delta"):                # CHECK_LEVEL_DELTA
        aprnet._ops.conv_forward(aprs, x.detach(), torch.zeros(1, 2, 2, 3, 3, 3, device=DEV), big)


def test_maxpool_padding_values_per_flavour():
    """Slots behind a batch item's last particle: -1e17 in the CPU flavour (maxpool.hpp:51), 0 in the CUDA
    flavour (wrap_maxpool_gpu.hpp:42)."""
    x, aprs, ld = _batch([("3d_a", 0), ("3d_s", 0)], 1, dtype=torch.float32)
    n0 = oracle.number_parts(aprs[0], 1)
    a, b = aprnet.MaxPool(), aprnet.cuda.MaxPool()
    a.increment_level_deltas = b.increment_level_deltas = False
    ya, yb = a(x, aprs, ld), b(x, aprs, ld)
    assert torch.all(ya[0, :, n0:] == -1e17) and torch.all(yb[0, :, n0:] == 0)
    assert torch.equal(ya[:, :, :n0], yb[:, :, :n0])


def test_aprconv_bf16_training_step():
    """APRConv with bfloat16 features end to end through autograd: fp32 parameters get fp32 gradients, the input
    gets a bfloat16 gradient, all within bfloat16 tolerance of the fp32 run."""
    apr = apr_cases.get("3d_b")
    n = oracle.number_parts(apr, 0)
    torch.manual_seed(3)
    model = aprnet.cuda.APRConv(6, 5, nstencils=2).to(DEV)
    x32 = torch.randn(1, 6, n, device=DEV).to(torch.bfloat16).float().requires_grad_(True)
    xb = x32.detach().to(torch.bfloat16).requires_grad_(True)
    ld = torch.zeros(1, dtype=torch.int32)
    go = torch.randn(1, 5, n, device=DEV).to(torch.bfloat16)
    y32 = model(x32, [apr], ld)
    g32 = torch.autograd.grad(y32, (x32, model.weight, model.bias), go.float())
    yb = model(xb, [apr], ld)
    gb = torch.autograd.grad(yb, (xb, model.weight, model.bias), go)
    assert yb.dtype == torch.bfloat16 and gb[0].dtype == torch.bfloat16
    assert gb[1].dtype == torch.float32 and gb[2].dtype == torch.float32
    for a, b in zip(gb, g32):
        assert float((a.float() - b).abs().max()) <= 1e-2 * float(b.abs().max())
