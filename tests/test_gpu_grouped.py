"""bfloat16 features grouped by eight channels ([B, C / 8, N, 8]): every grouped operator against its plane twin
(bit-identical where the arithmetic and its order are the same, which is everywhere but the 1x1x1 convolution) and
the grouped network forward against the fp32 oracle."""
import pytest
import torch

import apr_cases
from oracle import oracle
from pyapr import _native
from pyapr.aprnet import _ops, grouped as g8

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _batch(c, seed=0):
    aprs = [apr_cases.get("3d_s"), apr_cases.get("3d_t")]
    ld = torch.tensor([0, 1], dtype=torch.int32)
    sizes = [oracle.number_parts(a, int(d)) for a, d in zip(aprs, ld)]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(2, c, max(sizes), generator=g).to(torch.bfloat16)
    for i, n in enumerate(sizes):
        x[i, :, n:] = 0
    return aprs, ld, x.to(DEV), g


def test_regroup_roundtrip_and_padding():
    _, _, x, _ = _batch(24)
    g = g8.regroup(x)
    assert g.data.shape == (2, 3, x.shape[2], 8) and g.channels == 24
    assert torch.equal(g8.ungroup(g), x)
    assert torch.equal(g.data[:, 1, :, 3], x[:, 11, :])
    odd = x[:, :13].contiguous()                       # 13 channels: the last group is padded with zeros
    go = g8.regroup(odd)
    assert go.channels == 16 and torch.equal(g8.ungroup(go, 13), odd) and float(go.data[:, 1, :, 5:].abs().max()) == 0


def test_tree_fill_pool_upsample_equal_the_plane_kernels():
    aprs, ld, x, _ = _batch(16, seed=1)
    g = g8.regroup(x)
    lib = _native.hip()
    st = torch.cuda.current_stream().cuda_stream
    for b, apr in enumerate(aprs):
        d = int(ld[b])
        nt = _ops.tree_parts(apr, d)
        n = x.shape[2]
        tp = torch.zeros(16, nt, dtype=torch.bfloat16, device=DEV)
        tg = torch.zeros(2, nt, 8, dtype=torch.bfloat16, device=DEV)
        assert lib.aprnet_fill_tree_mean_bf16(apr.plan(0), d, x[b].data_ptr(), n, 16, tp.data_ptr(), nt, st) == 0
        assert lib.aprnet_fill_tree_mean_bf16g(apr.plan(0), d, g.data[b].data_ptr(), n, 16, tg.data_ptr(), nt, st) == 0
        assert torch.equal(tg.permute(0, 2, 1).reshape(16, nt), tp)
    pooled = g8.maxpool_forward(aprs, g, ld)
    ref, _ = _ops.maxpool_forward(aprs, x, ld, 0.0)
    assert torch.equal(g8.ungroup(pooled), ref)
    up = g8.upsample_const_forward(aprs, pooled, ld + 1)
    assert torch.equal(g8.ungroup(up), _ops.upsample_const_forward(aprs, ref, ld + 1))


@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3), (1, 5, 5)], ids=["333", "133", "155"])
@pytest.mark.parametrize("c1,c2,cout", [(16, 0, 16), (8, 24, 40), (32, 0, 8), (32, 32, 64), (64, 0, 72), (8, 0, 16)])
def test_grouped_convolution_equals_the_plane_kernel(c1, c2, cout, ksize):
    """Grouped input (with and without a second input), grouped and plane output, bias and ReLU: bit-identical to the
    fused plane entry point, which stages the same values from a regrouped copy."""
    aprs, ld, x, g = _batch(c1 + c2, seed=2)
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    w = (torch.randn(levels, cout, c1 + c2, *ksize, generator=g) * 0.1).to(DEV)
    bias = torch.randn(cout, generator=g).to(DEV)
    xa, xb = x[:, :c1].contiguous(), (x[:, c1:].contiguous() if c2 else None)
    ref = _ops.conv_forward(aprs, xa, w, ld, bias, relu=True, x2=xb)
    got = g8.conv_forward(aprs, g8.regroup(xa), w, ld, bias, relu=True, x2=g8.regroup(xb) if c2 else None)
    assert torch.equal(g8.ungroup(got), ref)
    planes = g8.conv_forward(aprs, g8.regroup(xa), w, ld, bias, relu=False, x2=g8.regroup(xb) if c2 else None, grouped_output=False)
    assert torch.equal(planes, _ops.conv_forward(aprs, xa, w, ld, bias, x2=xb))


@pytest.mark.parametrize("c1,c2,cout", [(16, 0, 16), (8, 24, 40)])
def test_grouped_convolution_with_64_bit_addresses(c1, c2, cout):
    """Tensors of 2^28 particles and more make the kernel address its 16-byte items with 64 bits instead of 32-bit
    byte offsets; forced here on a small batch (tiles with and without tree items, a second input, lanes without an
    item): bit-identical to the default."""
    aprs, ld, x, g = _batch(c1 + c2, seed=6)
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    w = (torch.randn(levels, cout, c1 + c2, 3, 3, 3, generator=g) * 0.1).to(DEV)
    bias = torch.randn(cout, generator=g).to(DEV)
    xa, xb = g8.regroup(x[:, :c1].contiguous()), (g8.regroup(x[:, c1:].contiguous()) if c2 else None)
    ref = g8.conv_forward(aprs, xa, w, ld, bias, relu=True, x2=xb)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(15) == 0
    try:
        got = g8.conv_forward(aprs, xa, w, ld, bias, relu=True, x2=xb)
        planes = g8.conv_forward(aprs, xa, w, ld, bias, relu=False, x2=xb, grouped_output=False)
    finally:
        assert lib.aprnet_set_conv_path(14) == 0
    assert torch.equal(got.data, ref.data)
    assert torch.equal(planes, g8.conv_forward(aprs, xa, w, ld, bias, relu=False, x2=xb, grouped_output=False))


@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 5, 5)], ids=["333", "155"])
@pytest.mark.parametrize("c1,c2,cout,hc,hs", [(16, 0, 16, 3, 1), (16, 16, 16, 1, 2), (8, 0, 8, 4, 3), (24, 8, 16, 2, 1)])
def test_convolution_with_fused_head_equals_the_two_operators(c1, c2, cout, hc, hs, ksize):
    """The last stencil convolution and the 1x1x1 head in one kernel: the head sees the layer's result rounded to
    bfloat16, as the stored tensor would hold it, and sums in fp32; against the same sums in float64 over the stored
    result of the unfused layer the outputs agree to bfloat16 rounding (half a unit in the 8th mantissa bit of the
    value, here 2^-8 of the row's absolute sum), also with 64-bit item addresses, where they are bit-identical."""
    aprs, ld, x, g = _batch(c1 + c2, seed=9)
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    w = (torch.randn(levels, cout, c1 + c2, *ksize, generator=g) * 0.1).to(DEV)
    bias = torch.randn(cout, generator=g).to(DEV)
    hw = torch.randn(hs, hc, cout, 1, 1, 1, generator=g).to(DEV)
    hb = torch.randn(hc, generator=g).to(DEV)
    xa, xb = g8.regroup(x[:, :c1].contiguous()), (g8.regroup(x[:, c1:].contiguous()) if c2 else None)
    mid = g8.ungroup(g8.conv_forward(aprs, xa, w, ld, bias, relu=True, x2=xb))            # [B, cout, N] bfloat16
    got = g8.conv_head_forward(aprs, xa, w, ld, bias, hw, hb, relu=True, x2=xb)
    assert got.shape == (2, hc, x.shape[2]) and got.dtype == torch.bfloat16
    # the oracle's 1x1x1 convolution in float64 on the stored result of the unfused layer, and the same on absolute values
    hw_cpu = hw.permute(2, 0, 1, 3, 4, 5).contiguous().double().cpu()
    m = mid.double().cpu()
    want = oracle.conv_forward(aprs, m, hw_cpu, ld) + hb.double().cpu().view(1, -1, 1)
    bound = oracle.conv_forward(aprs, m.abs(), hw_cpu.abs(), ld) + hb.double().cpu().abs().view(1, -1, 1)
    for b, apr in enumerate(aprs):
        n = oracle.number_parts(apr, int(ld[b]))
        err = (got[b, :, :n].double().cpu() - want[b, :, :n]).abs()
        assert bool((err <= 2.0 ** -8 * bound[b, :, :n] + 1e-30).all()), float((err / (bound[b, :, :n] + 1e-30)).max())
        tail = got[b, :, n:].float().cpu()
        assert torch.equal(tail, hb.to(torch.bfloat16).float().cpu().view(-1, 1).expand_as(tail))
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(15) == 0
    try:
        big = g8.conv_head_forward(aprs, xa, w, ld, bias, hw, hb, relu=True, x2=xb)
    finally:
        assert lib.aprnet_set_conv_path(14) == 0
    assert torch.equal(big, got)


@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3)], ids=["333", "133"])
@pytest.mark.parametrize("fill", [16, 17], ids=["needed-nodes", "whole-tree"])
def test_tree_of_an_upsampled_second_input_is_read_off_its_source(fill, ksize):
    """The second input of a decoder's first convolution is an upsampled tensor; its mean tree holds the values it was
    upsampled from (a mean of equal values), so the convolution may read that tree off the source tensor instead of
    computing it: bit-identical outputs, with the restricted and with the whole tree fill, with and without the head."""
    aprs, ld, x, g = _batch(16, seed=4)
    ld1 = ld + 1
    n1 = max(oracle.number_parts(a, int(d)) for a, d in zip(aprs, ld1))
    z = torch.randn(2, 24, n1, generator=g).to(torch.bfloat16)
    for b, (a, d) in enumerate(zip(aprs, ld1)):
        z[b, :, oracle.number_parts(a, int(d)):] = 0
    zg = g8.regroup(z.to(DEV))
    u = g8.upsample_const_forward(aprs, zg, ld1)
    assert u.data.shape[2] == x.shape[2]
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    w = (torch.randn(levels, 16, 40, *ksize, generator=g) * 0.1).to(DEV)
    bias = torch.randn(16, generator=g).to(DEV)
    hw = torch.randn(1, 3, 16, 1, 1, 1, generator=g).to(DEV)
    xa = g8.regroup(x)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(fill) == 0
    try:
        ref = g8.conv_forward(aprs, xa, w, ld, bias, relu=True, x2=u)
        got = g8.conv_forward(aprs, xa, w, ld, bias, relu=True, x2=u, x2_coarse=zg)
        href = g8.conv_head_forward(aprs, xa, w, ld, bias, hw, None, relu=True, x2=u)
        hgot = g8.conv_head_forward(aprs, xa, w, ld, bias, hw, None, relu=True, x2=u, x2_coarse=zg)
    finally:
        assert lib.aprnet_set_conv_path(16) == 0
    assert torch.equal(got.data, ref.data)
    assert torch.equal(hgot, href)
    with pytest.raises(ValueError):
        g8.conv_forward(aprs, xa, w, ld, bias, relu=True, x2=u, x2_coarse=g8.regroup(z[:, :16].contiguous().to(DEV)))


def test_fused_head_refuses_what_it_does_not_take():
    aprs, ld, x, g = _batch(32, seed=2)
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    xa = g8.regroup(x)
    w32 = torch.randn(levels, 32, 32, 3, 3, 3, generator=g).to(DEV)
    with pytest.raises(ValueError):
        g8.conv_head_forward(aprs, xa, w32, ld, None, torch.randn(1, 2, 32, 1, 1, 1).to(DEV))       # 32 channels in between
    w16 = torch.randn(levels, 16, 32, 3, 3, 3, generator=g).to(DEV)
    with pytest.raises(ValueError):
        g8.conv_head_forward(aprs, xa, w16, ld, None, torch.randn(1, 5, 16, 1, 1, 1).to(DEV))       # five outputs


@pytest.mark.parametrize("cin", [1, 3])
def test_first_layer_planes_in_grouped_out(cin):
    aprs, ld, x, g = _batch(cin, seed=3)
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    w = (torch.randn(levels, 16, cin, 3, 3, 3, generator=g) * 0.2).to(DEV)
    bias = torch.randn(16, generator=g).to(DEV)
    got = g8.conv_forward(aprs, x, w, ld, bias, relu=True)
    assert torch.equal(g8.ungroup(got), _ops.conv_forward(aprs, x, w, ld, bias, relu=True))


# small layers run on the vector-ALU kernel, the others on the matrix-core kernel: whole and partial blocks of 16 input
# channels and of 32 outputs, one and two output blocks per workgroup, 128 inputs, plane output
@pytest.mark.parametrize("cin,cout,grouped_out,relu", [(16, 8, True, False), (64, 32, True, False), (16, 3, False, False),
                                                       (24, 40, True, True), (32, 64, True, False), (128, 16, True, True),
                                                       (48, 19, False, True), (8, 64, True, False)])
def test_grouped_conv111_against_oracle(cin, cout, grouped_out, relu):
    aprs, ld, x, g = _batch(cin, seed=4)
    w = torch.randn(2, cout, cin, 1, 1, 1, generator=g) * 0.2
    bias = torch.randn(cout, generator=g)
    ref = oracle.conv_forward(aprs, x.float().cpu(), w.permute(2, 0, 1, 3, 4, 5).contiguous(), ld) + bias.view(1, -1, 1)
    if relu:
        ref = ref.clamp_min(0)
    got = g8.conv111_forward(aprs, g8.regroup(x), w.to(DEV), ld, bias.to(DEV), relu=relu, grouped_output=grouped_out)
    got = g8.ungroup(got) if grouped_out else got
    for b, a in enumerate(aprs):
        n = oracle.number_parts(a, int(ld[b]))
        err = float((got[b, :, :n].float().cpu() - ref[b, :, :n]).abs().max())
        assert err <= 1e-2 * float(ref.abs().max())


def test_unet_grouped_forward_against_oracle_and_plane_path():
    """The 4-level network with bfloat16 features: the grouped path (default for inference with folded norms) against
    the fp32 oracle composition (2e-2 of the output scale) and against the plane path of the same build (the two differ
    only in the summation order of the 1x1x1 convolutions)."""
    from bench import make_unet
    from test_gpu_unet import reference_forward
    apr = apr_cases.random_apr((33, 29, 37), 11, density=0.02)
    n = apr.total_number_particles()
    x = torch.randn(1, 1, n, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    model = make_unet("cpu")
    with torch.no_grad():
        ref = reference_forward(model, x.float(), [apr])
        model = model.to(DEV)
        assert model._grouped_ok(x.to(DEV), [apr])
        got = model(x.to(DEV), [apr])
        model.use_grouped = False
        planes = model(x.to(DEV), [apr])
    assert got.shape == planes.shape == (1, 3, n) and got.dtype == torch.bfloat16
    scale = float(ref.abs().max())
    assert float((got.float().cpu() - ref).abs().max()) <= 2e-2 * scale
    assert float((got.float() - planes.float()).abs().max()) <= 1e-2 * scale


def test_unet_grouped_forward_follows_weight_updates():
    """Without prepare_inference() the grouped forward restricts its stencils in every pass, so every kind of weight
    update shows in the next forward pass: in place (w.mul_), and through .data (which autograd's version counter
    does not see).  With prepare_inference() the stencils are kept until they are dropped: by
    invalidate_inference_cache(), load_state_dict(), train() or a move of the module."""
    from bench import make_unet
    apr = apr_cases.random_apr((20, 24, 22), 3, density=0.05)
    x = torch.randn(1, 1, apr.total_number_particles(), generator=torch.Generator().manual_seed(7)).to(torch.bfloat16).to(DEV)
    model = make_unet(DEV)
    conv = model.encoder[0].blocks[1].conv
    with torch.no_grad():
        assert model._grouped_ok(x, [apr])
        y0 = model(x, [apr]).clone()
        assert torch.equal(model(x, [apr]), y0)
        w = conv.weight
        w.mul_(0.5)
        y1 = model(x, [apr]).clone()
        assert not torch.equal(y1, y0)
        w.mul_(2.0)
        assert torch.equal(model(x, [apr]), y0)
        w.data.mul_(0.5)                                   # leaves w._version and w.data_ptr() unchanged
        assert torch.equal(model(x, [apr]), y1)
        w.data.mul_(2.0)
        # kept stencils
        model.prepare_inference([apr])
        assert hasattr(conv, "_inference_stencils")
        assert torch.equal(model(x, [apr]), y0)
        w.data.mul_(0.5)
        assert torch.equal(model(x, [apr]), y0)            # stale by contract ...
        model.invalidate_inference_cache()
        assert torch.equal(model(x, [apr]), y1)            # ... until invalidated
        w.data.mul_(2.0)
        model.prepare_inference([apr])
        state = {k: v.clone() for k, v in model.state_dict().items()}
        state["encoder.0.blocks.1.conv.weight"] *= 0.5
        model.load_state_dict(state)
        assert not hasattr(conv, "_inference_stencils")
        assert torch.equal(model(x, [apr]), y1)
        model.prepare_inference([apr])
        model.train()
        assert not hasattr(conv, "_inference_stencils")
        model.eval()
        model.prepare_inference(levels=apr.level_max() - apr.level_min() + 1)
        model.float()
        assert not hasattr(conv, "_inference_stencils")


def test_unet_grouped_limits_fall_back_to_the_plane_path():
    """A network whose 1x1x1 reduction sees 512 channels is beyond the grouped 1x1x1 kernel (256 inputs): the model
    must notice before any layer runs and compute the same result on channel planes.  The same when the plan's
    window lists are switched off (the grouped convolution then reports "unsupported" from inside the forward pass),
    and when a submodule carries a forward hook, which the grouped path would skip."""
    from apr_models.unet import APRUNet, fold_norms
    apr = apr_cases.random_apr((12, 10, 14), 5, density=0.08)
    x = torch.randn(1, 1, apr.total_number_particles(), generator=torch.Generator().manual_seed(9)).to(torch.bfloat16).to(DEV)
    torch.manual_seed(3)
    wide = fold_norms(APRUNet(1, 2, depth=3, n_filters_base=64, n_stencils=1, norm="batch").eval()).to(DEV)
    assert g8.limits()["conv111_max_cin"] == 256
    with torch.no_grad():
        assert not wide._grouped_ok(x, [apr])
        got = wide(x, [apr])
        wide.use_grouped = False
        assert torch.equal(wide(x, [apr]), got)
    from bench import make_unet
    model = make_unet(DEV)
    lib = _native.hip()
    with torch.no_grad():
        assert model._grouped_ok(x, [apr])
        grouped_out = model(x, [apr])
        model.use_grouped = False
        planes = model(x, [apr])
        model.use_grouped = True
        ld = torch.zeros(1, dtype=torch.int32)
        assert lib.aprnet_set_conv_path(5) == 0            # no window lists: the grouped convolution refuses
        try:
            fallback = model(x, [apr], ld)
        finally:
            assert lib.aprnet_set_conv_path(4) == 0
        assert int(ld[0]) == 0                             # level deltas restored and walked down and up again
        lib.aprnet_set_conv_path(5)
        try:
            model.use_grouped = False
            planes_nolists = model(x, [apr])
        finally:
            lib.aprnet_set_conv_path(4)
            model.use_grouped = True
        assert torch.equal(fallback, planes_nolists)
        scale = float(planes.float().abs().max())
        assert float((fallback.float() - grouped_out.float()).abs().max()) <= 1e-2 * scale
        seen = []
        h = model.encoder[1].pool.register_forward_hook(lambda m, i, o: seen.append(1))
        assert not model._grouped_ok(x, [apr])
        assert torch.equal(model(x, [apr]), planes) and seen
        h.remove()
        assert model._grouped_ok(x, [apr])
        model.encoder[1].pool.increment_level_deltas = False
        assert not model._grouped_ok(x, [apr])
        model.encoder[1].pool.increment_level_deltas = True
        del model.use_grouped                              # a whole-model pickle from before the attribute existed
        assert model._grouped_ok(x, [apr])
