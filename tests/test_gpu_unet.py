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
from pyapr.aprnet import _ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cpu_conv(conv, x, aprs, ld):
    w = conv.weight.detach().cpu().permute(2, 0, 1, 3, 4, 5).contiguous()       # -> [Cin, S, Cout, k]
    b = None if conv.bias is None else conv.bias.detach().cpu()
    return OracleConv.apply(x, w, b, aprs, ld)


def _cpu_norm(norm, x):
    """The block's norm evaluated by torch on the CPU (a CPU copy of the module; nn.Identity when folded away)."""
    import copy
    return copy.deepcopy(norm).cpu()(x)


def _cpu_basic(bb, x, aprs, ld):
    return torch.relu(_cpu_norm(bb.norm, _cpu_conv(bb.conv, x, aprs, ld)))


def _cpu_block(block, x, aprs, ld):
    for bb in block.blocks:
        x = _cpu_basic(bb, x, aprs, ld)
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
        y = _cpu_basic(stage.reduce_ch, y, aprs, ld)
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


@pytest.mark.parametrize("norm,train", [("group", False), ("batch", True), ("batch", False)])
def test_unet_forward_with_norm_layers_matches_oracle(norm, train):
    """The network as the reference builds it (GroupNorm with one group per channel by default, or BatchNorm1d in
    training / eval mode, nothing folded) on a batch of two APRs of different sizes: convolutions, norms over the padded
    particle axis, pool and upsample on the GPU against the same composition on the CPU (oracle operators, torch norms)."""
    aprs = [apr_cases.random_apr((24, 40, 36), 5, density=0.05), apr_cases.random_apr((20, 33, 28), 6, density=0.04)]
    n = max(a.total_number_particles() for a in aprs)
    torch.manual_seed(3)
    model = APRUNet(1, 2, depth=2, n_filters_base=8, n_stencils=2, norm=norm)
    with torch.no_grad():
        for m in model.modules():
            if isinstance(m, (torch.nn.BatchNorm1d, torch.nn.GroupNorm)):
                m.weight.uniform_(0.5, 1.5); m.bias.uniform_(-0.5, 0.5)
            if isinstance(m, torch.nn.BatchNorm1d):
                m.running_mean.uniform_(-0.2, 0.2); m.running_var.uniform_(0.5, 2.0)
    model.train(train)
    x = torch.randn(2, 1, n)
    for b, a in enumerate(aprs):
        x[b, :, a.total_number_particles():] = 0
    with torch.no_grad():
        ref = reference_forward(model, x, aprs)
        got = model.to(DEV)(x.to(DEV), aprs)
    err = float((got.cpu() - ref).abs().max()) / float(ref.abs().max())
    assert err < 2e-5, f"rel err {err:.2e}"


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


# ----------------------------------------------------------------------------------------------- hybrid network
def reference_forward_hybrid(model, x, aprs):
    """HybridAPRUNet evaluated with the CPU oracle for every particle operator (and the model's own dense torch
    blocks, on the CPU) in the order of apr_models/apr_models/unet/hybrid_model.py:123-139."""
    from apr_models.unet import DownConv, UpConv, TransitionDownConv, TransitionUpConv
    from oracle_modules import OracleReconstruct, OracleSample
    ld = torch.zeros(len(aprs), dtype=torch.int32)
    skips = [_cpu_block(model.encoder[0], x, aprs, ld)]
    for stage in model.encoder[1:]:
        if isinstance(stage, DownConv):
            y = OracleMaxPool.apply(skips[-1], aprs, ld); ld += 1
            skips.append(_cpu_block(stage.conv, y, aprs, ld))
        elif isinstance(stage, TransitionDownConv):
            y = OracleMaxPool.apply(skips[-1], aprs, ld); ld += 1
            skips.append(stage.conv(OracleReconstruct.apply(y, aprs, ld)))
        else:
            skips.append(stage(skips[-1]))
    y = skips[-1]
    for i, stage in enumerate(model.decoder):
        skip = skips[-(i + 2)]
        if isinstance(stage, UpConv):
            y = torch.relu(_cpu_conv(stage.reduce_ch.conv, y, aprs, ld))
            y = OracleUpSample.apply(y, aprs, ld); ld -= 1
            y = _cpu_block(stage.conv, torch.cat([skip, y], dim=1), aprs, ld)
        elif isinstance(stage, TransitionUpConv):
            y = OracleSample.apply(stage.reduce_ch(y), aprs, ld)
            y = OracleUpSample.apply(y, aprs, ld); ld -= 1
            y = _cpu_block(stage.conv, torch.cat([skip, y], dim=1), aprs, ld)
        else:
            y = stage(y, skip)
    return _cpu_conv(model.head, y, aprs, ld)


@pytest.mark.parametrize("apr_depth", [0, 1, 2])
def test_hybrid_unet_forward_matches_oracle(apr_depth):
    """Particle stages above, dense stages below the transition (Reconstruct / SampleParticles), norms folded;
    odd volume dimensions exercise the padding of the dense decoder."""
    import copy
    from apr_models.unet import HybridAPRUNet
    apr = apr_cases.random_apr((33, 29, 37), 11, density=0.02)
    torch.manual_seed(0)
    model = HybridAPRUNet(1, 3, depth=3, apr_depth=apr_depth, n_filters_base=8, n_stencils=2, norm="batch").eval()
    for m in model.modules():
        if isinstance(m, (torch.nn.BatchNorm1d, torch.nn.BatchNorm3d)):
            m.running_mean.uniform_(-0.2, 0.2); m.running_var.uniform_(0.5, 1.5)
            m.weight.data.uniform_(0.5, 1.5); m.bias.data.uniform_(-0.1, 0.1)
    fold_norms(model)
    n = apr.total_number_particles()
    x = torch.randn(1, 1, n)
    with torch.no_grad():
        ref = reference_forward_hybrid(copy.deepcopy(model), x, [apr])
        got = model.to(DEV)(x.to(DEV), [apr])
    assert got.shape == ref.shape == (1, 3, n)
    err = float((got.cpu() - ref).abs().max()) / float(ref.abs().max())
    assert err < 5e-5, f"rel err {err:.2e}"      # dense convolutions of the two sides differ in summation order too


def test_hybrid_unet_training_step_matches_oracle_gradients():
    """One backward pass through particle and dense stages (GroupNorm, not folded): gradients of the first
    particle convolution and of a dense convolution against the oracle-composed network's autograd."""
    import copy
    from apr_models.unet import HybridAPRUNet
    apr = apr_cases.random_apr((20, 24, 28), 5, density=0.03)
    torch.manual_seed(3)
    model = HybridAPRUNet(2, 2, depth=2, apr_depth=1, n_filters_base=4, n_stencils=1, norm="batch").train()
    for m in model.modules():                       # batch statistics would differ through the padded tails: eval norms
        if isinstance(m, (torch.nn.BatchNorm1d, torch.nn.BatchNorm3d)):
            m.eval()
    n = apr.total_number_particles()
    x = torch.randn(1, 2, n)
    ref_model = copy.deepcopy(model)

    def conv_g(conv, y, aprs, ld):                  # oracle convolution that keeps the graph to the parameters
        return OracleConv.apply(y, conv.weight.permute(2, 0, 1, 3, 4, 5).contiguous(), conv.bias, aprs, ld)

    def cpu_block_bn(block, y, aprs, ld):           # particle blocks with their (eval) norms, on the oracle
        for bb in block.blocks:
            y = torch.relu(bb.norm(conv_g(bb.conv, y, aprs, ld)))
        return y

    from oracle_modules import OracleReconstruct, OracleSample
    ld = torch.zeros(1, dtype=torch.int32)
    e0 = cpu_block_bn(ref_model.encoder[0], x, [apr], ld)
    y = OracleMaxPool.apply(e0, [apr], ld); ld += 1
    e1 = cpu_block_bn(ref_model.encoder[1].conv, y, [apr], ld)
    y = OracleMaxPool.apply(e1, [apr], ld); ld += 1
    e2 = ref_model.encoder[2].conv(OracleReconstruct.apply(y, [apr], ld))
    d = ref_model.decoder[0]
    y = OracleUpSample.apply(OracleSample.apply(d.reduce_ch(e2), [apr], ld), [apr], ld); ld -= 1
    y = cpu_block_bn(d.conv, torch.cat([e1, y], 1), [apr], ld)
    d = ref_model.decoder[1]
    y = torch.relu(d.reduce_ch.norm(conv_g(d.reduce_ch.conv, y, [apr], ld)))
    y = OracleUpSample.apply(y, [apr], ld); ld -= 1
    y = cpu_block_bn(d.conv, torch.cat([e0, y], 1), [apr], ld)
    ref = conv_g(ref_model.head, y, [apr], ld)
    ref.square().sum().backward()

    model.to(DEV)
    got = model(x.to(DEV), [apr])
    got.square().sum().backward()
    assert float((got.detach().cpu() - ref.detach()).abs().max()) <= 5e-5 * float(ref.detach().abs().max())
    for name in ["encoder.0.blocks.0.conv.weight", "encoder.2.conv.blocks.0.conv.weight", "decoder.0.conv.blocks.0.conv.weight",
                 "head.bias"]:
        g = dict(model.named_parameters())[name].grad.cpu()
        r = dict(ref_model.named_parameters())[name].grad
        assert float((g - r).abs().max()) <= 2e-4 * float(r.abs().max()) + 1e-7, name


@pytest.mark.parametrize("out_delta,after", [(0, None), (1, 12)])
def test_stardist_unet_heads_match_oracle(out_delta, after):
    """APRStardistUNet: probability and ray-distance heads on the particles left at output_level_delta, against the
    oracle composition (stardist_model.py:113-132)."""
    from apr_models.unet import APRStardistUNet
    apr = apr_cases.random_apr((33, 29, 37), 11, density=0.02)
    torch.manual_seed(2)
    model = fold_norms(APRStardistUNet(1, 8, depth=2, n_filters_base=8, n_stencils=2, norm="batch",
                                       output_level_delta=out_delta, net_conv_after_unet=after).eval())
    x = torch.randn(1, 1, apr.total_number_particles())
    aprs, ld = [apr], torch.zeros(1, dtype=torch.int32)
    skips = [_cpu_block(model.encoder[0], x, aprs, ld)]
    for stage in model.encoder[1:]:
        y = OracleMaxPool.apply(skips[-1], aprs, ld); ld += 1
        skips.append(_cpu_block(stage.conv, y, aprs, ld))
    y = skips[-1]
    for i, stage in enumerate(model.decoder):
        y = torch.relu(_cpu_conv(stage.reduce_ch.conv, y, aprs, ld))
        y = OracleUpSample.apply(y, aprs, ld); ld -= 1
        y = _cpu_block(stage.conv, torch.cat([skips[-(i + 2)], y], dim=1), aprs, ld)
    if after is not None:
        y = _cpu_block(model.conv_after_unet, y, aprs, ld)
    ref_prob = torch.sigmoid(_cpu_conv(model.output_prob.conv, y, aprs, ld))
    ref_dist = _cpu_conv(model.output_dist, y, aprs, ld)
    assert int(ld[0]) == out_delta
    with torch.no_grad():
        prob, dist = model.to(DEV)(x.to(DEV), [apr])
    n_out = oracle.number_parts(apr, out_delta)
    assert prob.shape == (1, 1, n_out) and dist.shape == (1, 8, n_out)
    assert float((prob.cpu() - ref_prob).abs().max()) < 2e-5
    assert float((dist.cpu() - ref_dist).abs().max()) < 2e-5 * float(ref_dist.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_unet_forward_replays_from_a_hip_graph(dtype):
    """After one eager call (which builds the plan's lists) the operators neither allocate, copy nor synchronise, so
    the whole network forward can be captured into a HIP graph.  Replays with new inputs, interleaved with eager
    calls and synchronisations, reproduce the eager results bit for bit (the forward is deterministic)."""
    apr = apr_cases.random_apr((33, 29, 37), 11, density=0.02)
    torch.manual_seed(0)
    model = fold_norms(APRUNet(1, 3, depth=3, n_filters_base=16, n_stencils=2, norm="batch").eval()).to(DEV)
    n = apr.total_number_particles()
    g = torch.Generator().manual_seed(1)
    x_static = torch.randn(1, 1, n, generator=g).to(dtype).to(DEV)
    with torch.no_grad():
        model(x_static, [apr])                                   # eager warm-up: lists, tile tables, scratch
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model(x_static, [apr])
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static = model(x_static, [apr])
        for k in range(3):
            x_new = torch.randn(1, 1, n, generator=g).to(dtype).to(DEV)
            eager = model(x_new, [apr])
            torch.cuda.synchronize()
            x_static.copy_(x_new)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y_static, eager), f"replay {k}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_unet_training_step_replays_from_a_hip_graph(dtype):
    """Forward, loss and backward of the network in training mode (BatchNorm statistics of the batch, running
    statistics updated) captured into one HIP graph: the backward operators fork the weight gradient onto the
    plan's second stream and join it again, clear their work space with fill kernels and neither allocate outside
    torch's allocator nor synchronise.  Every replay, with new inputs and with eager steps and synchronisations in
    between, gives the loss, the parameter gradients and the running statistics of the same step run eagerly
    (to the 1e-4 that the order of the atomic additions of the gradients leaves open; 2e-2 with bfloat16 features)."""
    import copy
    apr = apr_cases.random_apr((33, 29, 37), 11, density=0.02)
    torch.manual_seed(0)
    model = APRUNet(1, 3, depth=3, n_filters_base=8, n_stencils=2, norm="batch").to(DEV).train()
    ref = copy.deepcopy(model)
    n = apr.total_number_particles()
    g = torch.Generator().manual_seed(1)
    x_static = torch.randn(1, 1, n, generator=g).to(dtype).to(DEV)
    t_static = torch.randn(1, 3, n, generator=g).to(DEV)

    def step(m, x, t):
        for p in m.parameters():
            p.grad = None
        loss = torch.nn.functional.mse_loss(m(x, [apr]).float(), t)
        loss.backward()
        return loss

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):                                       # eager warm-up: lists, tile tables, scratch
            step(model, x_static, t_static)
            step(ref, x_static, t_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for p in model.parameters():
        p.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        loss_static = step(model, x_static, t_static)
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    for k in range(3):
        x_new = torch.randn(1, 1, n, generator=g).to(dtype).to(DEV)
        t_new = torch.randn(1, 3, n, generator=g).to(DEV)
        loss_eager = step(ref, x_new, t_new)
        torch.cuda.synchronize()
        x_static.copy_(x_new)
        t_static.copy_(t_new)
        graph.replay()
        torch.cuda.synchronize()
        assert abs(float(loss_static) - float(loss_eager)) <= tol * abs(float(loss_eager)), f"replay {k}"
        scale = max(float(q.grad.abs().max()) for q in ref.parameters())
        for (name, p), q in zip(model.named_parameters(), ref.parameters()):
            assert p.grad is not None and torch.isfinite(p.grad).all(), name
            # a convolution's bias in front of a norm layer has a zero gradient up to rounding: absolute term
            bound = tol * float(q.grad.abs().max()) + 0.02 * tol * scale
            assert float((p.grad - q.grad).abs().max()) <= bound, f"replay {k}: {name}"
        for (name, b), c in zip(model.named_buffers(), ref.named_buffers()):
            assert name == c[0]
            assert torch.allclose(b.float(), c[1].float(), rtol=tol, atol=tol * 1e-2), f"replay {k}: {name}"


def test_hybrid_stardist_unet_matches_oracle():
    """HybridStardistUNet (stardist_hybrid_model.py:24-199): dense stages below the transition, decoder back to the
    particles at output_level_delta = 1, probability and distance heads there; against the oracle composition."""
    import copy
    from apr_models.unet import HybridStardistUNet
    from oracle_modules import OracleReconstruct, OracleSample
    apr = apr_cases.random_apr((33, 29, 37), 11, density=0.02)
    torch.manual_seed(4)
    model = fold_norms(HybridStardistUNet(1, 6, depth=3, apr_depth=1, n_filters_base=8, n_stencils=2, norm="batch",
                                          output_level_delta=1, net_conv_after_unet=10).eval())
    with pytest.raises(ValueError):
        HybridStardistUNet(1, 6, depth=3, apr_depth=1, output_level_delta=2)
    ref_model = copy.deepcopy(model)
    x = torch.randn(1, 1, apr.total_number_particles())
    aprs, ld = [apr], torch.zeros(1, dtype=torch.int32)
    with torch.no_grad():
        e0 = _cpu_block(ref_model.encoder[0], x, aprs, ld)
        y = OracleMaxPool.apply(e0, aprs, ld); ld += 1
        e1 = _cpu_block(ref_model.encoder[1].conv, y, aprs, ld)                       # DownConv (particles)
        y = OracleMaxPool.apply(e1, aprs, ld); ld += 1
        e2 = ref_model.encoder[2].conv(OracleReconstruct.apply(y, aprs, ld))          # TransitionDownConv
        e3 = ref_model.encoder[3](e2)                                                 # PixelDownConv
        y = ref_model.decoder[0](e3, e2)                                              # PixelUpConv
        d = ref_model.decoder[1]                                                      # TransitionUpConv
        y = OracleUpSample.apply(OracleSample.apply(d.reduce_ch(y), aprs, ld), aprs, ld); ld -= 1
        y = _cpu_block(d.conv, torch.cat([e1, y], 1), aprs, ld)
        y = _cpu_block(ref_model.conv_after_unet, y, aprs, ld)
        ref_prob = torch.sigmoid(_cpu_conv(ref_model.output_prob.conv, y, aprs, ld))
        ref_dist = _cpu_conv(ref_model.output_dist, y, aprs, ld)
        assert int(ld[0]) == 1
        prob, dist = model.to(DEV)(x.to(DEV), [apr])
    n1 = oracle.number_parts(apr, 1)
    assert prob.shape == (1, 1, n1) and dist.shape == (1, 6, n1)
    assert float((prob.cpu() - ref_prob).abs().max()) < 5e-5
    assert float((dist.cpu() - ref_dist).abs().max()) < 5e-5 * float(ref_dist.abs().max())


# ---------------------------------------------------------------------------- normalisation over the particle axis
def _norm_pair(kind, C, groups, dtype, seed):
    from apr_models.unet.particle_norm import ParticleBatchNorm, ParticleGroupNorm
    torch.manual_seed(seed)
    if kind == "batch":
        mine, ref = ParticleBatchNorm(C, momentum=0.1), torch.nn.BatchNorm1d(C, momentum=0.1)
    else:
        mine, ref = ParticleGroupNorm(groups, C), torch.nn.GroupNorm(groups, C)
    with torch.no_grad():
        mine.weight.copy_(torch.randn(C) * 0.5 + 1.0)
        mine.bias.copy_(torch.randn(C))
    ref.load_state_dict(mine.state_dict())            # interchangeable state
    return mine.to(DEV), ref.double()


@pytest.mark.gpu
@pytest.mark.parametrize("kind,C,groups", [("batch", 6, 1), ("group", 6, 6), ("group", 8, 2), ("group", 5, 1)])
@pytest.mark.parametrize("B,N", [(1, 4099), (3, 1021), (2, 3)])
@pytest.mark.parametrize("relu", [False, True])
def test_particle_norm_matches_torch(kind, C, groups, B, N, relu):
    """Forward, input / weight / bias gradients and running statistics of the streaming-kernel norms against the
    torch modules the reference uses (float64 on the CPU).  Tolerance 1e-5 relative to the tensor's largest entry."""
    mine, ref = _norm_pair(kind, C, groups, torch.float32, 7)
    g = torch.Generator().manual_seed(B * 1000 + N)
    x = torch.randn(B, C, N, generator=g) * 3.0 + 10.0            # a mean well away from zero
    go = torch.randn(B, C, N, generator=g)
    for step in range(2):                                          # two steps: running statistics accumulate
        xm = x.to(DEV).requires_grad_(True)
        xr = x.double().requires_grad_(True)
        ym = mine(xm, relu=relu)
        yr = ref(xr)
        if relu:
            yr = torch.relu(yr)
        ym.backward(go.to(DEV)); yr.backward(go.double())

        def close(a, b, tol=1e-5):
            a, b = a.detach().double().cpu(), b.detach().double()
            assert a.shape == b.shape
            assert (a - b).abs().max().item() <= tol * max(b.abs().max().item(), 1.0), (a - b).abs().max().item()
        close(ym, yr); close(xm.grad, xr.grad)
        close(mine.weight.grad, ref.weight.grad, 2e-5); close(mine.bias.grad, ref.bias.grad, 2e-5)
        if kind == "batch":
            close(mine.running_mean, ref.running_mean); close(mine.running_var, ref.running_var)
            assert int(mine.num_batches_tracked) == int(ref.num_batches_tracked) == step + 1
        mine.zero_grad(); ref.zero_grad()
    if kind == "batch":                                            # eval mode: running statistics, no batch terms
        mine.eval(); ref.eval()
        xm = x.to(DEV).requires_grad_(True); xr = x.double().requires_grad_(True)
        ym, yr = mine(xm, relu=relu), ref(xr)
        if relu:
            yr = torch.relu(yr)
        ym.backward(go.to(DEV)); yr.backward(go.double())
        close(ym, yr); close(xm.grad, xr.grad); close(mine.weight.grad, ref.weight.grad, 2e-5)


@pytest.mark.gpu
def test_particle_norm_bf16_and_repeatability():
    mine, ref = _norm_pair("group", 8, 4, torch.bfloat16, 3)
    x = (torch.randn(2, 8, 2050) * 2 + 1).to(torch.bfloat16)
    go = torch.randn(2, 8, 2050).to(torch.bfloat16)
    xm = x.to(DEV).requires_grad_(True); xr = x.double().requires_grad_(True)
    ym = mine(xm, relu=True); yr = torch.relu(ref(xr))
    ym.backward(go.to(DEV)); yr.backward(go.double())
    assert ym.dtype == torch.bfloat16 and xm.grad.dtype == torch.bfloat16
    assert (ym.double().cpu() - yr).abs().max() <= 2e-2 * yr.abs().max()
    assert (xm.grad.double().cpu() - xr.grad).abs().max() <= 2e-2 * xr.grad.abs().max()
    # fixed summation order: bit-identical on repetition
    x32 = torch.randn(1, 4, 100003, device=DEV)
    a = _ops.row_moments(x32); b = _ops.row_moments(x32)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    # closed forms: a constant row has m2 = 0 and mean = the constant; a ramp 0..n-1 has mean (n-1)/2, m2 = n(n^2-1)/12
    n = 4097
    rows = torch.stack([torch.full((n,), 3.25), torch.arange(n, dtype=torch.float32)]).unsqueeze(0).to(DEV).contiguous()
    mean, m2 = _ops.row_moments(rows)
    assert mean[0, 0].item() == 3.25 and m2[0, 0].item() == 0.0
    assert abs(mean[0, 1].item() - (n - 1) / 2) < 1e-6 * n and abs(m2[0, 1].item() / (n * (n * n - 1) / 12) - 1) < 1e-6
    with pytest.raises(ValueError):
        _ops.norm_apply(x32, torch.zeros(3, device=DEV), torch.zeros(4, device=DEV), torch.zeros(4, device=DEV), False)


@pytest.mark.gpu
@pytest.mark.parametrize("norm", ["batch", "group"])
def test_unet_training_step_bf16_follows_fp32(norm):
    """A whole training step (forward, MSE loss, backward) with bfloat16 features runs on the native kernels - stencil and
    1x1x1 convolutions, norm + ReLU, pool, upsample - and its gradients point the way of the fp32 step's: cosine
    similarity above 0.9 for every convolution weight (the first layer's gradient has crossed every layer's bfloat16
    storage twice; observed 0.96 there, above 0.99 near the head).  The norm parameters and the head's bias have a
    handful of entries that are sums of nearly cancelling terms, below the bfloat16 noise of those terms: they are
    only required to be finite here (their arithmetic is pinned by the norm tests above)."""
    apr = apr_cases.random_apr((24, 40, 36), 5, density=0.05)
    n = apr.total_number_particles()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 1, n, generator=g).to(DEV)
    target = torch.randn(1, 2, n, generator=g).to(DEV)
    torch.manual_seed(2)
    net = APRUNet(1, 2, depth=2, n_filters_base=8, n_stencils=2, norm=norm).to(DEV).train()

    def grads(dtype):
        net.zero_grad()
        out = net(x.to(dtype), [apr])
        assert out.dtype == dtype
        torch.nn.functional.mse_loss(out.float(), target).backward()
        return {k: p.grad.detach().clone() for k, p in net.named_parameters()}
    ref, got = grads(torch.float32), grads(torch.bfloat16)
    for k in ref:
        assert got[k].dtype == ref[k].dtype and torch.isfinite(got[k]).all()
        a, b = got[k].flatten().double(), ref[k].flatten().double()
        if k.endswith("conv.weight") or k == "head.weight":
            cos = torch.nn.functional.cosine_similarity(a, b, dim=0)
            assert cos > 0.9, (k, float(cos))

