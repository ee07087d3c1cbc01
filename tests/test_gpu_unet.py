"""APRUNet forward on the GPU against the same network evaluated op by op with the CPU oracle
(4 levels, 16-32-64-128 channels, two 3x3x3 convolutions per stage, BatchNorm folded into the
convolutions, 1x1x1 head; BASELINE configs[3] at reduced size)."""
import numpy as np
import pytest
import torch

import apr_cases
from oracle import oracle
from oracle_modules import OracleConv, OracleMaxPool, OracleUpSample
from apr_models.unet import APRUNet, fold_norms

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cpu_conv(conv, x, aprs, ld):
    w = conv.weight.detach().cpu().permute(2, 0, 1, 3, 4, 5).contiguous()       # -> [Cin, S, Cout, k]
    b = None if conv.bias is None else conv.bias.detach().cpu()
    return OracleConv.apply(x, w, b, aprs, ld)


def _cpu_block(block, x, aprs, ld):
    for bb in block.blocks:
        x = torch.relu(_cpu_conv(bb.conv, x, aprs, ld))
    return x


def reference_forward(model, x, aprs):
    ld = torch.zeros(len(aprs), dtype=torch.int32)
    skips = [_cpu_block(model.encoder[0], x, aprs, ld)]
    for stage in model.encoder[1:]:
        y = OracleMaxPool.apply(skips[-1], aprs, ld)
        ld += 1
        skips.append(_cpu_block(stage.conv, y, aprs, ld))
    y = skips[-1]
    for i, stage in enumerate(model.decoder):
        y = torch.relu(_cpu_conv(stage.reduce_ch.conv, y, aprs, ld))
        y = OracleUpSample.apply(y, aprs, ld)
        ld -= 1
        y = _cpu_block(stage.conv, torch.cat([skips[-(i + 2)], y], dim=1), aprs, ld)
    return _cpu_conv(model.head, y, aprs, ld)


@pytest.mark.parametrize("shape,seed", [((33, 29, 37), 11), ((1, 130, 257), 14)])
def test_unet_forward_matches_oracle(shape, seed):
    apr = apr_cases.random_apr(shape, seed, density=0.02)
    assert apr.level_max() >= 5
    torch.manual_seed(0)
    model = APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch",
                    dims=2 if shape[0] == 1 else 3).eval()
    for m in model.modules():                      # non-trivial running statistics to fold
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.uniform_(-0.2, 0.2); m.running_var.uniform_(0.5, 1.5)
            m.weight.data.uniform_(0.5, 1.5); m.bias.data.uniform_(-0.1, 0.1)
    fold_norms(model)
    n = apr.total_number_particles()
    x = torch.randn(1, 1, n)
    ref = reference_forward(model, x, [apr])
    with torch.no_grad():
        got = model.to(DEV)(x.to(DEV), [apr])
    assert got.shape == ref.shape == (1, 3, n)
    err = float((got.cpu() - ref).abs().max()) / float(ref.abs().max())
    assert err < 2e-5, f"rel err {err:.2e}"      # 18 fp32 layers deep; single ops agree to 1e-5


def test_fold_norms_equals_eval_batchnorm():
    apr = apr_cases.get("3d_s")
    torch.manual_seed(1)
    model = APRUNet(2, 2, depth=1, n_filters_base=4, norm="batch").eval().to(DEV)
    for m in model.modules():
        if isinstance(m, torch.nn.BatchNorm1d):
            m.running_mean.uniform_(-0.5, 0.5); m.running_var.uniform_(0.5, 2.0)
    x = torch.randn(1, 2, apr.total_number_particles(), device=DEV)
    with torch.no_grad():
        a = model(x, [apr])
        b = fold_norms(model)(x, [apr])
    torch.testing.assert_close(a, b, rtol=1e-4, atol=1e-5)


def test_unet_forward_bf16_features():
    """The same network with bfloat16 features (fp32 weights and arithmetic inside every operator) against
    the fp32 oracle: 2e-2 of the output scale after 18 layers (BASELINE configs[3], bf16 leg, reduced size)."""
    apr = apr_cases.random_apr((33, 29, 37), 11, density=0.02)
    torch.manual_seed(0)
    model = fold_norms(APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch").eval())
    n = apr.total_number_particles()
    x = torch.randn(1, 1, n).to(torch.bfloat16)
    ref = reference_forward(model, x.float(), [apr])
    with torch.no_grad():
        got = model.to(DEV)(x.to(DEV), [apr])
    assert got.dtype == torch.bfloat16 and got.shape == ref.shape
    err = float((got.float().cpu() - ref).abs().max()) / float(ref.abs().max())
    assert err < 2e-2, f"rel err {err:.2e}"
