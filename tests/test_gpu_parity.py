"""GPU parity tests: the HIP operators (through pyapr.aprnet -> C ABI of libaprnet_hip.so) against the
CPU oracle on the same seeded inputs.  Bit-exact for index maps and pooling argmax; float64 to 1e-11
and float32 to rel 1e-5 of the output scale for values (the sides differ in summation order only)."""
import ctypes as C

import numpy as np
import pytest
import torch

import apr_cases
from oracle import oracle
from pyapr import _native
from pyapr.aprnet import _ops

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ALL_CASES = list(apr_cases.TINY) + list(apr_cases.SMALL)
KID = lambda k: "k%d%d%d" % tuple(k)


def close(got, ref, dtype):
    got = got.detach().cpu()
    if dtype == torch.float64:
        torch.testing.assert_close(got, ref, rtol=1e-11, atol=1e-11 * max(1.0, float(ref.abs().max())))
    else:
        # rel 1e-5 of the output scale (fp32 sums of up to a few thousand terms in a different order)
        scale = max(float(ref.abs().max()), 1e-30)
        err = float((got - ref).abs().max())
        assert err <= 1e-5 * scale, f"max abs err {err:.3e} vs scale {scale:.3e}"


def batch(names_d, channels, dtype, seed=0):
    aprs = [apr_cases.get(n) for n, _ in names_d]
    ld = torch.tensor([d for _, d in names_d], dtype=torch.int32)
    sizes = [oracle.number_parts(a, int(d)) for a, d in zip(aprs, ld)]
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(len(aprs), channels, max(sizes), dtype=dtype, generator=g)
    for i, n in enumerate(sizes):
        x[i, :, n:] = 0
    return x, aprs, ld


def max_delta(apr):
    return min(2, apr.level_max() - 1)


@pytest.mark.parametrize("name", ALL_CASES)
def test_child_table_matches_reference_parent_walk(name):
    """The index map behind pool / upsample / tree fill is bit-exact against the merge walk of
    helpers.hpp:185-194 (restated in the oracle)."""
    apr = apr_cases.get(name)
    apr.init_cuda()
    nt = apr.total_number_tree_particles()
    ch = np.zeros((8, nt), np.int32)
    assert _native.hip().aprnet_plan_children(apr.plan(0), ch.ctypes.data) == 0
    parent_of_part = np.full(apr.total_number_particles(), -1, np.int64)
    parent_of_tree = np.full(nt, -1, np.int64)
    for s in range(8):
        for t in range(nt):
            v = int(ch[s, t])
            if v == -2 ** 31:
                continue
            if v >= 0:
                assert parent_of_part[v] == -1
                parent_of_part[v] = t
            else:
                assert parent_of_tree[~v] == -1
                parent_of_tree[~v] = t
    it, tr = apr.iterator(), apr.tree_iterator()
    for level in range(1, apr.level_max() + 1):
        ref = oracle.parent_index(apr, 0, level)
        b, e = it.particles_level_begin(level), it.particles_level_end(level)
        assert np.array_equal(parent_of_part[b:e], ref[b:e])
    for level in range(1, apr.level_max()):
        ref = oracle.parent_index(apr, 1, level)
        b, e = tr.particles_level_begin(level), tr.particles_level_end(level)
        assert np.array_equal(parent_of_tree[b:e], ref[b:e])


@pytest.mark.parametrize("name", ALL_CASES)
def test_number_parts(name):
    apr = apr_cases.get(name)
    apr.init_cuda()
    lib = _native.hip()
    for d in range(apr.level_max()):
        assert lib.aprnet_number_parts(apr.plan(0), d) == oracle.number_parts(apr, d) == _ops.number_particles(apr, d)
        assert lib.aprnet_tree_offset(apr.plan(0), apr.level_max() - d) == oracle.tree_offset(apr, apr.level_max() - d)
        assert lib.aprnet_tree_parts(apr.plan(0), d) == oracle.tree_parts(apr, d)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("name", ALL_CASES)
def test_fill_tree_mean(name, dtype):
    apr = apr_cases.get(name)
    apr.init_cuda()
    lib = _native.hip()
    sfx = "f32" if dtype == torch.float32 else "f64"
    for d in range(max_delta(apr) + 1):
        n, nt = oracle.number_parts(apr, d), oracle.tree_parts(apr, d)
        g = torch.Generator().manual_seed(d)
        x = torch.randn(2, n, dtype=dtype, generator=g)
        xd = x.to(DEV)
        tree = torch.zeros(2, max(nt, 1), dtype=dtype, device=DEV)
        rc = getattr(lib, "aprnet_fill_tree_mean_" + sfx)(apr.plan(0), d, xd.data_ptr(), n, 2, tree.data_ptr(), max(nt, 1),
                                                         torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.aprnet_last_error()
        for c in range(2):
            ref = oracle.fill_tree_mean(apr, x[c], d)
            # same summation order as the reference -> identical bits
            assert torch.equal(tree[c, :nt].cpu(), ref)
        # backward: adjoint of the forward
        gt = torch.randn(2, max(nt, 1), dtype=dtype, generator=g)
        gtd, gx = gt.to(DEV), torch.zeros(2, n, dtype=dtype, device=DEV)
        rc = getattr(lib, "aprnet_fill_tree_mean_bwd_" + sfx)(apr.plan(0), d, gx.data_ptr(), n, 2, gtd.data_ptr(), max(nt, 1),
                                                             torch.cuda.current_stream().cuda_stream)
        assert rc == 0, lib.aprnet_last_error()
        for c in range(2):
            close(gx[c], oracle.fill_tree_mean_backward(apr, gt[c, :nt], n, d), dtype)


CONV_BATCHES = [
    [("3d_a", 0)], [("3d_b", 1)], [("3d_a", 2), ("3d_c", 2)], [("3d_s", 0), ("3d_a", 1)], [("3d_t", 1)],
    [("2d_a", 0)], [("2d_a", 1), ("2d_b", 2)], [("2d_s", 0)], [("2d_t", 0), ("2d_t", 2)], [("1d_a", 0), ("1d_s", 1)],
]


def _conv_case(bt, ksize, nstencils, cin, cout, dtype):
    x, aprs, ld = batch(bt, cin, dtype, seed=nstencils)
    g = torch.Generator().manual_seed(17)
    w = torch.randn(cin, nstencils, cout, *ksize, dtype=dtype, generator=g)      # CPU layout
    num_levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    w_exp = w if ksize == (1, 1, 1) else oracle.restrict_kernel_forward(w, num_levels)
    return x, aprs, ld, w_exp


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3), (1, 5, 5), (5, 5, 5), (1, 1, 1)], ids=KID)
@pytest.mark.parametrize("bt", CONV_BATCHES, ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_conv_forward(bt, ksize, dtype):
    cin, cout, S = 5, 7, 3
    x, aprs, ld, w_exp = _conv_case(bt, ksize, S, cin, cout, dtype)
    ref = oracle.conv_forward(aprs, x, w_exp, ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)                    # -> [S, Cout, Cin, k]
    got = _ops.conv_forward(aprs, x.to(DEV), wd, ld)
    close(got, ref, dtype)


@pytest.mark.parametrize("path", [0, 1], ids=["mfma", "valu"])
@pytest.mark.parametrize("cin,cout", [(1, 16), (32, 32), (33, 33), (16, 3), (64, 40)])
def test_conv333_forward_channel_shapes(cin, cout, path):
    """Channel counts of the benchmark configurations and of the reference's CUDA-vs-CPU test
    (33 -> 33, pyapr/tests/test_aprnet.py:137-138), on both fp32 kernels (matrix cores / VALU)."""
    x, aprs, ld, w_exp = _conv_case([("3d_s", 0), ("3d_t", 1)], (3, 3, 3), 2, cin, cout, torch.float32)
    ref = oracle.conv_forward(aprs, x, w_exp, ld)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(path) == 0
    try:
        got = _ops.conv_forward(aprs, x.to(DEV), w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld)
    finally:
        lib.aprnet_set_conv_path(0)
    close(got, ref, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 5, 5)], ids=KID)
def test_conv_forward_without_plan_lists(ksize, dtype):
    """The forward matrix-core kernels scanning the access arrays per call (the path taken when the plan's
    window lists are switched off or do not fit) give the same result as with the lists."""
    x, aprs, ld, w_exp = _conv_case([("3d_s", 0), ("3d_t", 1)], ksize, 2, 12, 20, torch.float32)
    xd = x.to(dtype).to(DEV)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    lib = _native.hip()
    with_lists = _ops.conv_forward(aprs, xd, wd, ld)
    assert lib.aprnet_set_conv_path(5) == 0
    try:
        scanned = _ops.conv_forward(aprs, xd, wd, ld)
    finally:
        lib.aprnet_set_conv_path(4)
    ref = oracle.conv_forward(aprs, xd.float().cpu(), w_exp, ld)
    if dtype == torch.float32:
        assert torch.equal(with_lists, scanned)            # same kernel body, same summation order
        close(scanned, ref, torch.float32)
    else:
        close_bf16(scanned, ref)                           # fp32 products here, bfloat16 products with the lists
        close_bf16(with_lists, ref)


def test_conv333_forward_dense_windows():
    """A fully refined APR: every window holds the maximum number of output positions (all four column
    blocks per wave of the matrix-core kernel), plus run-to-run bit equality (no atomics in the forward)."""
    import numpy as np
    from pyapr import APR
    shape = (6, 10, 140)
    apr = APR.from_level_field(shape, np.full(tuple((s + 1) // 2 for s in shape), 8, np.uint8))
    assert apr.total_number_particles() == 6 * 10 * 140
    g = torch.Generator().manual_seed(4)
    x = torch.randn(1, 6, apr.total_number_particles(), generator=g)
    w = torch.randn(6, 1, 10, 3, 3, 3, generator=g)
    ld = torch.zeros(1, dtype=torch.int32)
    w_exp = oracle.restrict_kernel_forward(w, apr.level_max() - apr.level_min() + 1)
    ref = oracle.conv_forward([apr], x, w_exp, ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    got = _ops.conv_forward([apr], x.to(DEV), wd, ld)
    close(got, ref, torch.float32)
    again = _ops.conv_forward([apr], x.to(DEV), wd, ld)
    assert torch.equal(got, again)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3), (1, 5, 5), (5, 5, 5), (1, 1, 1)], ids=KID)
@pytest.mark.parametrize("bt", [[("3d_a", 0)], [("3d_b", 1), ("3d_c", 2)], [("2d_a", 1), ("2d_b", 0)], [("3d_s", 0)]],
                         ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_conv_backward(bt, ksize, dtype):
    cin, cout, S = 3, 4, 2
    x, aprs, ld, w_exp = _conv_case(bt, ksize, S, cin, cout, dtype)
    g = torch.Generator().manual_seed(5)
    go = torch.randn(x.size(0), cout, x.size(2), dtype=dtype, generator=g)
    gx_ref, gw_ref = oracle.conv_backward(aprs, x, w_exp, go, ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    gx, gw = _ops.conv_backward(aprs, x.to(DEV), wd, go.to(DEV), ld)
    # the reference leaves gradients of padding slots at zero
    close(gx, gx_ref, dtype)
    close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, dtype)


@pytest.mark.parametrize("path", [0, 1], ids=["mfma", "valu"])
@pytest.mark.parametrize("cin,cout", [(1, 16), (32, 32), (33, 33), (16, 3), (40, 64)])
def test_conv333_backward_channel_shapes(cin, cout, path):
    """Gradients of input and weights on both fp32 kernel families, at channel counts that fill, straddle and
    underfill the 32-channel blocks and the 16-channel groups of the matrix-core kernels."""
    x, aprs, ld, w_exp = _conv_case([("3d_s", 0), ("3d_t", 1)], (3, 3, 3), 2, cin, cout, torch.float32)
    g = torch.Generator().manual_seed(6)
    go = torch.randn(x.size(0), cout, x.size(2), generator=g)
    gx_ref, gw_ref = oracle.conv_backward(aprs, x, w_exp, go, ld)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(path) == 0
    try:
        gx, gw = _ops.conv_backward(aprs, x.to(DEV), w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), go.to(DEV), ld)
    finally:
        lib.aprnet_set_conv_path(0)
    close(gx, gx_ref, torch.float32)
    close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_conv_backward_on_one_stream(dtype):
    """The backward pass with the weight gradient on the caller's stream (path 7) instead of the plan's second stream
    (default): same gradients, and the switch is accepted both ways."""
    cin, cout = 20, 33
    x, aprs, ld, w_exp = _conv_case([("3d_s", 0), ("3d_t", 1)], (3, 3, 3), 2, cin, cout, torch.float32)
    g = torch.Generator().manual_seed(21)
    go = torch.randn(x.size(0), cout, x.size(2), generator=g)
    if dtype == torch.bfloat16:
        x, go = x.to(dtype).float(), go.to(dtype).float()
    gx_ref, gw_ref = oracle.conv_backward(aprs, x, w_exp, go, ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    lib = _native.hip()
    for path in (7, 6):
        assert lib.aprnet_set_conv_path(path) == 0
        try:
            gx, gw = _ops.conv_backward(aprs, x.to(DEV).to(dtype), wd, go.to(DEV).to(dtype), ld)
        finally:
            lib.aprnet_set_conv_path(6)
        if dtype == torch.bfloat16:
            close_bf16(gx, gx_ref)
            assert float((gw.permute(2, 0, 1, 3, 4, 5).cpu() - gw_ref).abs().max()) <= 1e-2 * float(gw_ref.abs().max())
        else:
            close(gx, gx_ref, dtype)
            close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, dtype)


@pytest.mark.parametrize("path", [0, 1, 3], ids=["mfma", "valu", "fp32math"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cin,cout", [(1, 16), (5, 4), (18, 33)])
def test_conv_backward_weights_only(cin, cout, dtype, path):
    """need_input_grad=False (what autograd asks of the first layer of a network): no input gradient, the same weight
    gradient; channel counts that leave whole input-channel chunks of the weight-gradient kernel empty and that take
    its 16-row and 32-row forms.  bfloat16 features: with bfloat16 and (path 3) with fp32 matrix instructions."""
    if (dtype == torch.bfloat16 and path == 1) or (dtype == torch.float32 and path == 3):
        pytest.skip("bfloat16 features run on the matrix-core kernels only; path 3 concerns bfloat16 features")
    x, aprs, ld, w_exp = _conv_case([("3d_s", 0), ("3d_t", 1)], (3, 3, 3), 2, cin, cout, torch.float32)
    g = torch.Generator().manual_seed(9)
    go = torch.randn(x.size(0), cout, x.size(2), generator=g)
    if dtype == torch.bfloat16:
        x, go = x.to(dtype).float(), go.to(dtype).float()          # the oracle sees the rounded values
    _, gw_ref = oracle.conv_backward(aprs, x, w_exp, go, ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(path) == 0
    try:
        gx, gw = _ops.conv_backward(aprs, x.to(DEV).to(dtype), wd, go.to(DEV).to(dtype), ld, need_input_grad=False)
    finally:
        lib.aprnet_set_conv_path(0); lib.aprnet_set_conv_path(2)
    assert gx is None
    if dtype == torch.bfloat16:      # the mean-filled tree values that the sums read are stored in bfloat16
        assert float((gw.permute(2, 0, 1, 3, 4, 5).cpu() - gw_ref).abs().max()) <= 1e-2 * float(gw_ref.abs().max())
    else:
        close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, torch.float32)


@pytest.mark.parametrize("path", [0, 1], ids=["mfma", "valu"])
@pytest.mark.parametrize("ksize", [(1, 3, 3), (1, 5, 5)], ids=KID)
@pytest.mark.parametrize("bt", [[("2d_a", 0), ("2d_b", 1)], [("3d_s", 0)]], ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_conv_flat_stencils_wide_channels(bt, ksize, path):
    """1x3x3 and 1x5x5 (the 2-D stencils) at channel counts that straddle the blocks of the matrix-core
    kernels, forward and backward, on both fp32 kernel families."""
    cin, cout = 20, 33
    x, aprs, ld, w_exp = _conv_case(bt, ksize, 2, cin, cout, torch.float32)
    g = torch.Generator().manual_seed(8)
    go = torch.randn(x.size(0), cout, x.size(2), generator=g)
    ref = oracle.conv_forward(aprs, x, w_exp, ld)
    gx_ref, gw_ref = oracle.conv_backward(aprs, x, w_exp, go, ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(path) == 0
    try:
        got = _ops.conv_forward(aprs, x.to(DEV), wd, ld)
        gx, gw = _ops.conv_backward(aprs, x.to(DEV), wd, go.to(DEV), ld)
    finally:
        lib.aprnet_set_conv_path(0)
    close(got, ref, torch.float32)
    close(gx, gx_ref, torch.float32)
    close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, torch.float32)


def test_conv333_backward_dense_windows():
    """Fully refined APR: windows with the maximum number of columns (496 > one staged group of 256 in the
    weight-gradient kernel, all column blocks in the input-gradient kernel)."""
    import numpy as np
    from pyapr import APR
    shape = (6, 10, 140)
    apr = APR.from_level_field(shape, np.full(tuple((s + 1) // 2 for s in shape), 8, np.uint8))
    g = torch.Generator().manual_seed(7)
    n = apr.total_number_particles()
    x = torch.randn(1, 6, n, generator=g)
    w = torch.randn(6, 1, 10, 3, 3, 3, generator=g)
    go = torch.randn(1, 10, n, generator=g)
    ld = torch.zeros(1, dtype=torch.int32)
    w_exp = oracle.restrict_kernel_forward(w, apr.level_max() - apr.level_min() + 1)
    gx_ref, gw_ref = oracle.conv_backward([apr], x, w_exp, go, ld)
    gx, gw = _ops.conv_backward([apr], x.to(DEV), w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), go.to(DEV), ld)
    close(gx, gx_ref, torch.float32)
    close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3), (1, 5, 5), (5, 5, 5)], ids=KID)
@pytest.mark.parametrize("s,levels", [(1, 4), (2, 5), (3, 3), (3, 7)])
def test_restrict_kernel(ksize, s, levels, dtype):
    g = torch.Generator().manual_seed(s + levels)
    w = torch.randn(3, s, 4, *ksize, dtype=dtype, generator=g)                   # CPU layout [Cin, S, Cout, k]
    ref = oracle.restrict_kernel_forward(w, levels)
    got = _ops.restrict_kernel_forward(w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), levels)
    close(got.permute(2, 0, 1, 3, 4, 5), ref, dtype)
    gw = torch.randn(3, levels, 4, *ksize, dtype=dtype, generator=g)
    ref_b = oracle.restrict_kernel_backward(gw, s)
    got_b = _ops.restrict_kernel_backward(gw.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), s)
    close(got_b.permute(2, 0, 1, 3, 4, 5), ref_b, dtype)


POOL_BATCHES = [[("3d_a", 0)], [("3d_b", 1)], [("3d_a", 1), ("3d_c", 0)], [("3d_s", 0), ("3d_t", 1)], [("2d_a", 0), ("2d_b", 1)],
                [("2d_t", 2)], [("1d_a", 0), ("1d_s", 1)]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("bt", POOL_BATCHES, ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_maxpool_bit_exact_with_ties(bt, dtype):
    x, aprs, ld = batch(bt, 3, dtype)
    x = torch.clamp(torch.round(x * 1.5), min=0)          # few distinct values, zeros as after a ReLU
    ref, ref_idx = oracle.maxpool_forward(aprs, x, ld)
    out, idx = _ops.maxpool_forward(aprs, x.to(DEV), ld)
    assert torch.equal(out.cpu(), ref)
    assert torch.equal(idx.cpu(), ref_idx)
    g = torch.Generator().manual_seed(3)
    go = torch.randn(ref.shape, dtype=dtype, generator=g)
    gref = oracle.maxpool_backward(aprs, go, ref_idx, ld)
    got = _ops.maxpool_backward(aprs, go.to(DEV), idx, ld)
    assert torch.equal(got.cpu(), gref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("bt", [[("3d_a", 1)], [("3d_b", 2)], [("3d_a", 1), ("3d_c", 2)], [("3d_s", 1), ("3d_t", 2)],
                                [("2d_a", 1), ("2d_b", 2)], [("1d_a", 1), ("1d_s", 2)]],
                         ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_upsample(bt, dtype):
    x, aprs, ld = batch(bt, 3, dtype)
    ref = oracle.upsample_const_forward(aprs, x, ld)
    got = _ops.upsample_const_forward(aprs, x.to(DEV), ld)
    assert torch.equal(got.cpu(), ref)
    g = torch.Generator().manual_seed(9)
    go = torch.randn(ref.shape, dtype=dtype, generator=g)
    sizes = [oracle.number_parts(a, int(d) - 1) for a, d in zip(aprs, ld)]
    for i, n in enumerate(sizes):
        go[i, :, n:] = 0
    close(_ops.upsample_const_backward(aprs, go.to(DEV), ld), oracle.upsample_const_backward(aprs, go, ld), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("bt", [[("3d_a", 0)], [("3d_b", 1)], [("3d_c", 2), ("3d_c", 2)], [("2d_a", 1)], [("3d_s", 0)]],
                         ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_reconstruct_and_sample(bt, dtype):
    x, aprs, ld = batch(bt, 2, dtype)
    xd = x.to(DEV)
    img_ref = oracle.reconstruct_forward(aprs, x, ld)
    img = _ops.reconstruct_forward(aprs, xd, ld)
    assert torch.equal(img.cpu(), img_ref)
    # SampleParticles(Reconstruct(x)) == x  (pyapr/tests/test_aprnet.py:272-285)
    close(_ops.sample_particles_forward(aprs, img, ld), x, dtype)
    g = torch.Generator().manual_seed(2)
    im = torch.randn(img_ref.shape, dtype=dtype, generator=g)
    close(_ops.sample_particles_forward(aprs, im.to(DEV), ld), oracle.sample_particles_forward(aprs, im, ld), dtype)
    close(_ops.reconstruct_backward(aprs, im.to(DEV), ld), oracle.reconstruct_backward(aprs, im, ld), dtype)
    close(_ops.sample_particles_backward(aprs, xd, ld), oracle.sample_particles_backward(aprs, x, ld), dtype)


# ------------------------------------------------------------------------------------------- bfloat16 features
def close_bf16(got, ref):
    """bfloat16 storage, fp32 arithmetic: every stored value is within half a unit in the 8th mantissa bit of
    the fp32 result; 2e-2 of the output scale is the stated bound, 1e-2 is asserted."""
    assert got.dtype == torch.bfloat16
    scale = max(float(ref.abs().max()), 1e-30)
    err = float((got.detach().float().cpu() - ref).abs().max())
    assert err <= 1e-2 * scale, f"max abs err {err:.3e} vs scale {scale:.3e}"


@pytest.mark.parametrize("bt", [[("3d_a", 0)], [("3d_b", 1)], [("3d_c", 2), ("3d_c", 2)], [("2d_a", 1)]],
                         ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_reconstruct_and_sample_bf16(bt):
    """bfloat16 particles and images: the piecewise-constant fill copies bit patterns; sums and means are taken in
    fp32 over bfloat16 inputs and rounded once."""
    x, aprs, ld = batch(bt, 2, torch.float32)
    xb = x.to(torch.bfloat16)
    img = _ops.reconstruct_forward(aprs, xb.to(DEV), ld)
    assert img.dtype == torch.bfloat16
    assert torch.equal(img.float().cpu(), oracle.reconstruct_forward(aprs, xb.float(), ld))
    # SampleParticles(Reconstruct(x)) == x exactly: the mean of equal bfloat16 values is that value
    assert torch.equal(_ops.sample_particles_forward(aprs, img, ld).cpu(), xb)
    g = torch.Generator().manual_seed(2)
    im = torch.randn(img.shape, generator=g).to(torch.bfloat16)
    close_bf16(_ops.sample_particles_forward(aprs, im.to(DEV), ld), oracle.sample_particles_forward(aprs, im.float(), ld))
    close_bf16(_ops.reconstruct_backward(aprs, im.to(DEV), ld), oracle.reconstruct_backward(aprs, im.float(), ld))
    close_bf16(_ops.sample_particles_backward(aprs, xb.to(DEV), ld), oracle.sample_particles_backward(aprs, xb.float(), ld))


@pytest.mark.parametrize("math", [2, 3], ids=["bf16math", "fp32math"])
@pytest.mark.parametrize("cin,cout", [(1, 16), (32, 32), (33, 17)])
@pytest.mark.parametrize("bt", [[("3d_a", 0)], [("3d_b", 1), ("3d_c", 2)], [("3d_s", 0), ("3d_t", 1)]],
                         ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_conv333_forward_bf16(bt, cin, cout, math):
    """bfloat16 features against the fp32 oracle on the same (bfloat16-representable) inputs and fp32 weights,
    with the products on the bfloat16 matrix cores (weights rounded to bfloat16) and on the fp32 ones."""
    x, aprs, ld, w_exp = _conv_case(bt, (3, 3, 3), 2, cin, cout, torch.float32)
    xb = x.to(torch.bfloat16)
    g = torch.Generator().manual_seed(11)
    bias = torch.randn(cout, generator=g)
    ref = oracle.conv_forward(aprs, xb.float(), w_exp, ld) + bias.view(1, -1, 1)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(math) == 0
    try:
        got = _ops.conv_forward(aprs, xb.to(DEV), w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld, bias.to(DEV))
    finally:
        lib.aprnet_set_conv_path(2)
    close_bf16(got, ref)


@pytest.mark.parametrize("ksize", [(1, 3, 3), (1, 5, 5)], ids=KID)
def test_conv_flat_forward_bf16(ksize):
    x, aprs, ld, w_exp = _conv_case([("2d_a", 0), ("2d_b", 1)], ksize, 2, 20, 33, torch.float32)
    xb = x.to(torch.bfloat16)
    ref = oracle.conv_forward(aprs, xb.float(), w_exp, ld)
    got = _ops.conv_forward(aprs, xb.to(DEV), w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld)
    close_bf16(got, ref)


def test_conv111_forward_bf16():
    x, aprs, ld, w = _conv_case([("3d_b", 1), ("3d_c", 0)], (1, 1, 1), 3, 20, 9, torch.float32)
    xb = x.to(torch.bfloat16)
    ref = oracle.conv_forward(aprs, xb.float(), w, ld)
    got = _ops.conv_forward(aprs, xb.to(DEV), w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), ld)
    close_bf16(got, ref)


def test_bf16_results_round_to_nearest_even():
    """What a kernel stores as bfloat16 is its fp32 result rounded to nearest, ties to even, overflow to infinity:
    a 1x1x1 convolution of a channel of ones writes its fp32 weights, so every output equals the
    weight rounded by torch (ties both ways, the last finite value and the first that rounds to infinity, random
    bit patterns of normal numbers)."""
    x, aprs, ld = batch([("3d_b", 0)], 4, torch.float32)
    x[:] = 0
    x[:, 0] = 1.0
    special = [1.0, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 1.0 + 2.0 ** -8 + 2.0 ** -20, 1.0 + 2.0 ** -7 - 2.0 ** -23,
               -1.0 - 2.0 ** -8, -1.0 - 3 * 2.0 ** -8, 3.3895313892515355e38, 3.3961775292304601e38, 3.4e38, -3.4e38,
               0.0, 2.0 ** -126, 2.0 ** -126 * (1 + 2.0 ** -8), 1e-30, 65504.0, 1.0 / 3.0]
    g = torch.Generator().manual_seed(11)
    bits = torch.randint(0x00800000, 0x7f000000, (64 - len(special),), generator=g, dtype=torch.int64)
    bits = bits | (torch.randint(0, 2, bits.shape, generator=g, dtype=torch.int64) << 31)
    rnd = (bits - (bits >> 31 << 32)).to(torch.int32).view(torch.float32)
    w0 = torch.cat([torch.tensor(special, dtype=torch.float32), rnd])
    w = torch.zeros(1, 64, 4, 1, 1, 1)
    w[0, :, 0, 0, 0, 0] = w0
    got = _ops.conv_forward(aprs, x.to(torch.bfloat16).to(DEV), w.to(DEV), ld)
    want = w0.to(torch.bfloat16)
    n = oracle.number_parts(aprs[0], 0)
    for i in (0, n // 2, n - 1):
        assert torch.equal(got[0, :, i].cpu().view(torch.int16), want.view(torch.int16)), i


@pytest.mark.parametrize("bt", POOL_BATCHES[:4], ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_maxpool_upsample_bf16_bit_exact(bt):
    """Pool and upsample move values without arithmetic: bfloat16 results equal the oracle's on the same
    (bfloat16-representable) values bit for bit, argmax included."""
    x, aprs, ld = batch(bt, 5, torch.float32)
    xb = x.to(torch.bfloat16)
    ref, ref_idx = oracle.maxpool_forward(aprs, xb.float(), ld)
    out, idx = _ops.maxpool_forward(aprs, xb.to(DEV), ld)
    assert out.dtype == torch.bfloat16
    ref = ref.to(torch.bfloat16).float()        # the -1e17 fill of padding slots (maxpool.hpp:51) rounds in bfloat16
    assert torch.equal(out.float().cpu(), ref)
    assert torch.equal(idx.cpu(), ref_idx)
    ld1 = ld + 1
    up_ref = oracle.upsample_const_forward(aprs, ref, ld1)
    up = _ops.upsample_const_forward(aprs, out, ld1)
    assert torch.equal(up.float().cpu(), up_ref)
    g = torch.Generator().manual_seed(3)
    go = torch.randn(ref.shape, generator=g).to(torch.bfloat16)
    gref = oracle.maxpool_backward(aprs, go.float(), ref_idx, ld)
    assert torch.equal(_ops.maxpool_backward(aprs, go.to(DEV), idx, ld).float().cpu(), gref)


@pytest.mark.parametrize("math", [2, 3, 5], ids=["bf16math", "fp32math", "nolists"])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 5, 5)], ids=KID)
@pytest.mark.parametrize("bt", [[("3d_b", 1), ("3d_c", 0)], [("2d_a", 0), ("2d_b", 1)], [("3d_s", 0), ("3d_t", 1)]],
                         ids=lambda b: "+".join(f"{n}@{d}" for n, d in b))
def test_conv_backward_bf16(bt, ksize, math):
    """bfloat16 features and output gradient, fp32 weights and accumulation: gradients against the fp32 oracle on
    the same (bfloat16-representable) inputs; the input gradient comes back in bfloat16, the weight gradient in fp32.
    The input gradient runs on the bfloat16 matrix cores from the plan's input-gradient lists (weights rounded to
    bfloat16), or with fp32 products when those are asked for or the lists are switched off."""
    cin, cout = 20, 33
    x, aprs, ld, w_exp = _conv_case(bt, ksize, 2, cin, cout, torch.float32)
    xb = x.to(torch.bfloat16)
    g = torch.Generator().manual_seed(12)
    gob = torch.randn(x.size(0), cout, x.size(2), generator=g).to(torch.bfloat16)
    gx_ref, gw_ref = oracle.conv_backward(aprs, xb.float(), w_exp, gob.float(), ld)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(math) == 0
    try:
        gx, gw = _ops.conv_backward(aprs, xb.to(DEV), w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), gob.to(DEV), ld)
    finally:
        lib.aprnet_set_conv_path(2); lib.aprnet_set_conv_path(4)
    close_bf16(gx, gx_ref)
    assert gw.dtype == torch.float32
    # fp32 sums; the mean-filled tree values they read are stored in bfloat16, hence the bfloat16 tolerance
    gwc = gw.permute(2, 0, 1, 3, 4, 5).cpu()
    assert float((gwc - gw_ref).abs().max()) <= 1e-2 * float(gw_ref.abs().max())


@pytest.mark.parametrize("cin,cout,S", [(20, 9, 3), (3, 40, 1), (64, 3, 2)])
def test_conv111_backward_bf16(cin, cout, S):
    """1x1x1 backward with bfloat16 features and output gradient: fp32 weights, weight gradient and accumulation;
    against the fp32 oracle on the same (bfloat16-representable) inputs."""
    x, aprs, ld, w = _conv_case([("3d_b", 1), ("3d_c", 0)], (1, 1, 1), S, cin, cout, torch.float32)
    xb = x.to(torch.bfloat16)
    g = torch.Generator().manual_seed(13)
    gob = torch.randn(x.size(0), cout, x.size(2), generator=g).to(torch.bfloat16)
    gx_ref, gw_ref = oracle.conv_backward(aprs, xb.float(), w, gob.float(), ld)
    gx, gw = _ops.conv_backward(aprs, xb.to(DEV), w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), gob.to(DEV), ld)
    close_bf16(gx, gx_ref)
    assert gw.dtype == torch.float32
    close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, torch.float32)        # fp32 products of exact inputs, fp32 sums
    with pytest.raises(TypeError):
        _ops.conv_backward(aprs, xb.to(DEV), w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV), gob.float().to(DEV), ld)


# ------------------------------------------------------------------------- fused forward (ReLU, second input)
@pytest.mark.parametrize("path", [0, 1], ids=["mfma", "valu"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16], ids=["f32", "f64", "bf16"])
@pytest.mark.parametrize("ksize,c1,c2,cout", [((3, 3, 3), 16, 16, 16), ((3, 3, 3), 5, 6, 33), ((1, 5, 5), 7, 3, 20),
                                              ((5, 5, 5), 3, 2, 4)], ids=lambda v: KID(v) if isinstance(v, tuple) else str(v))
def test_conv_forward_fused_relu_and_second_input(ksize, c1, c2, cout, dtype, path):
    """aprnet_conv_fwd_fused_*: relu(conv(cat([x, x2])) + bias) in one kernel against the oracle's convolution of the
    concatenated tensor followed by bias and ReLU (unet_parts.py:17-26, 82).  Unequal batch items: the padded
    tails must hold relu(bias) as they would after the reference's separate passes."""
    if dtype == torch.bfloat16 and path == 1 and ksize != (5, 5, 5):
        pytest.skip("bfloat16 features run the matrix-core kernels (5x5x5: the vector-ALU kernel, whatever the path)")
    bt = [("3d_b", 1), ("3d_c", 0)]
    cdt = torch.float32 if dtype == torch.bfloat16 else dtype
    x, aprs, ld, w_exp = _conv_case(bt, ksize, 2, c1 + c2, cout, cdt)
    if dtype == torch.bfloat16:
        x = x.to(torch.bfloat16).float()
    g = torch.Generator().manual_seed(5)
    bias = torch.randn(cout, dtype=cdt, generator=g)
    ref = torch.relu(oracle.conv_forward(aprs, x, w_exp, ld) + bias.view(1, -1, 1))
    xa, xb = x[:, :c1].contiguous().to(dtype).to(DEV), x[:, c1:].contiguous().to(dtype).to(DEV)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(path) == 0
    try:
        got = _ops.conv_forward(aprs, xa, wd, ld, bias.to(DEV), relu=True, x2=xb)
        plain = _ops.conv_forward(aprs, torch.cat([xa, xb], 1), wd, ld, bias.to(DEV))
    finally:
        lib.aprnet_set_conv_path(0)
    if dtype == torch.bfloat16:
        close_bf16(got, ref)
    else:
        close(got, ref, dtype)
        # same kernel, same order of operations: the fusion changes nothing but the clamp
        assert torch.equal(got, torch.relu(plain))


@pytest.mark.parametrize("ksize,c1,c2,cout", [((3, 3, 3), 16, 16, 16), ((3, 3, 3), 5, 6, 33), ((1, 5, 5), 7, 3, 20),
                                              ((1, 3, 3), 1, 0, 8)], ids=lambda v: KID(v) if isinstance(v, tuple) else str(v))
def test_conv_bf16_regrouped_input_equals_channel_planes(ksize, c1, c2, cout):
    """bfloat16 stencil convolutions stage from a copy of the input regrouped as [Cin / 8][particles][8]
    (aprnet_set_conv_path(8), the default) or gather from the channel planes (9).  Same values, same products, same
    order of accumulation: the forward results (with and without a second input tensor and the clamp) are
    bit-identical, and so is the oracle check; the backward's input gradient (fp32 atomics) agrees to rounding."""
    bt = [("3d_b", 1), ("3d_c", 0)]
    x, aprs, ld, w_exp = _conv_case(bt, ksize, 2, c1 + c2, cout, torch.float32)
    x = x.to(torch.bfloat16)
    g = torch.Generator().manual_seed(7)
    bias = torch.randn(cout, generator=g)
    ref = torch.relu(oracle.conv_forward(aprs, x.float(), w_exp, ld) + bias.view(1, -1, 1))
    xa = x[:, :c1].contiguous().to(DEV)
    xb = x[:, c1:].contiguous().to(DEV) if c2 else None
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    go = torch.randn(x.shape[0], cout, x.shape[2], generator=g).to(torch.bfloat16).to(DEV)
    lib = _native.hip()
    res = {}
    try:
        for path in (8, 9):
            assert lib.aprnet_set_conv_path(path) == 0
            fused = _ops.conv_forward(aprs, xa, wd, ld, bias.to(DEV), relu=True, x2=xb)
            plain = _ops.conv_forward(aprs, x.to(DEV), wd, ld, bias.to(DEV))
            gx, gw = _ops.conv_backward(aprs, x.to(DEV), wd, go, ld)
            torch.cuda.synchronize()
            res[path] = (fused, plain, gx, gw)
    finally:
        lib.aprnet_set_conv_path(8)
    close_bf16(res[8][0], ref)
    assert torch.equal(res[8][0], res[9][0]) and torch.equal(res[8][1], res[9][1])
    assert torch.equal(res[8][0], torch.relu(res[8][1]))
    scale = float(res[9][2].float().abs().max())
    assert float((res[8][2].float() - res[9][2].float()).abs().max()) <= 1e-2 * scale      # one bfloat16 rounding step
    assert float((res[8][3] - res[9][3]).abs().max()) <= 1e-5 * float(res[9][3].abs().max())
    assert lib.aprnet_set_conv_path(99) != 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16], ids=["f32", "f64", "bf16"])
def test_conv111_forward_fused_relu(dtype):
    cdt = torch.float32 if dtype == torch.bfloat16 else dtype
    x, aprs, ld, w = _conv_case([("3d_b", 1), ("3d_c", 0)], (1, 1, 1), 3, 20, 9, cdt)
    if dtype == torch.bfloat16:
        x = x.to(torch.bfloat16).float()
    bias = torch.linspace(-1, 1, 9, dtype=cdt)
    ref = torch.relu(oracle.conv_forward(aprs, x, w, ld) + bias.view(1, -1, 1))
    wd = w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    got = _ops.conv_forward(aprs, x.to(dtype).to(DEV), wd, ld, bias.to(DEV), relu=True)
    close_bf16(got, ref) if dtype == torch.bfloat16 else close(got, ref, dtype)
    with pytest.raises(ValueError):
        _ops.conv_forward(aprs, x[:, :10].contiguous().to(dtype).to(DEV), wd, ld, x2=x[:, 10:].contiguous().to(dtype).to(DEV))


# ------------------------------------------------------------------------------- degenerate access structures
DEGENERATE = {
    "dense": ((16, 16, 16), 1, 1.0, 0),        # every particle on the finest level, full tree
    "coarse": ((12, 10, 14), 2, 0.0, 2),       # no cell asks for resolution: a handful of particles on level 1
    "single": ((1, 1, 1), 3, 1.0, 0),          # one particle, one level, no tree level below it
    "sliver": ((2, 3, 1), 4, 1.0, 0),
    "line": ((5, 1, 1), 5, 0.5, 1),
}


@pytest.mark.parametrize("name", list(DEGENERATE))
def test_degenerate_structures(name):
    """Structures at the edges of what the access arrays can describe: all operators against the oracle at every
    level delta they accept (forward and backward of the 3x3x3 convolution on both kernel families, pool with
    argmax, upsample, tree fill through the convolution)."""
    shape, seed, dens, drop = DEGENERATE[name]
    apr = apr_cases.random_apr(shape, seed, dens, drop)
    lib = _native.hip()
    for d in range(max(apr.level_max() - 1, 1)):
        n = oracle.number_parts(apr, d)
        assert _ops.number_particles(apr, d) == n
        ld = torch.tensor([d], dtype=torch.int32)
        g = torch.Generator().manual_seed(7 + d)
        x = torch.randn(1, 3, n, generator=g)
        levels = apr.level_max() - apr.level_min() + 1
        w = torch.randn(3, min(2, levels), 5, 3, 3, 3, generator=g)
        w_exp = oracle.restrict_kernel_forward(w, levels)
        wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
        ref = oracle.conv_forward([apr], x, w_exp, ld)
        go = torch.randn(ref.shape, generator=g)
        ref_gx, ref_gw = oracle.conv_backward([apr], x, w_exp, go, ld)
        for path in (0, 1):
            assert lib.aprnet_set_conv_path(path) == 0
            try:
                got = _ops.conv_forward([apr], x.to(DEV), wd, ld)
                gx, gw = _ops.conv_backward([apr], x.to(DEV), wd, go.to(DEV), ld)
            finally:
                lib.aprnet_set_conv_path(0)
            close(got, ref, torch.float32)
            close(gx, ref_gx, torch.float32)
            close(gw.permute(2, 0, 1, 3, 4, 5), ref_gw, torch.float32)
        if apr.level_max() - d - 1 >= apr.level_min():          # there is a level left to pool into
            rp, ri = oracle.maxpool_forward([apr], x, ld)
            gp, gi = _ops.maxpool_forward([apr], x.to(DEV), ld, -1e17)
            assert torch.equal(gp.cpu(), rp) and torch.equal(gi.cpu(), ri)
            ld1 = ld + 1
            ru = oracle.upsample_const_forward([apr], rp, ld1)
            assert torch.equal(_ops.upsample_const_forward([apr], gp, ld1).cpu(), ru)
    # more stencils than levels: kernel.hpp:70-74 writes out of bounds there; refused on both sides
    levels = apr.level_max() - apr.level_min() + 1
    with pytest.raises(ValueError):
        _ops.restrict_kernel_forward(torch.zeros(levels + 1, 2, 2, 3, 3, 3, device=DEV), levels)
    with pytest.raises(ValueError):
        oracle.restrict_kernel_forward(torch.zeros(2, levels + 1, 2, 3, 3, 3), levels)


# ------------------------------------------------------------------------------------ StarDist utilities
@pytest.mark.parametrize("name", ["3d_c", "3d_s", "2d_a", "1d_a"])
def test_stardist_utilities_match_oracle(name):
    """get_particle_coordinates, sample_image (max pyramid) and labels_to_dist on the device against the oracle's
    restatement of utils.hpp:86-333: bit-exact (integer coordinates, maxima, and the same fp32 ray walk with
    round-half-even), for numpy and tensor inputs, every label type, integer and fractional ray steps."""
    from pyapr.aprnet import stardist_utils as su
    apr = apr_cases.get(name)
    Z, X, Y = apr.shape()
    g = torch.Generator().manual_seed(21)
    img = torch.randn(Z, X, Y, generator=g)
    blobs = (torch.rand(Z, X, Y, generator=g) * 2.2).floor()            # labels 0, 1, 2 in random patches
    lab = torch.nn.functional.interpolate(blobs[None, None, ::3, ::3, ::3], size=(Z, X, Y), mode="nearest")[0, 0]
    rays = torch.tensor([[1, 0, 0], [0, -1, 0], [0, 0, 1], [0.5, 0.5, 0], [-0.7, 0.2, 0.4], [0, 1.5, -1.5], [0.3, 0, 0]],
                        dtype=torch.float32)
    if Z == 1:
        rays[:, 0] = 0
    if X == 1:
        rays[:, 1] = 0
    rays = rays[(rays != 0).any(dim=1)]
    for d in range(max_delta(apr) + 1):
        n = oracle.number_parts(apr, d)
        ref_c = oracle.particle_coords(apr, d)
        got_c = su.get_particle_coordinates(apr, d)
        assert isinstance(got_c, np.ndarray) and got_c.shape == (n, 3) and np.array_equal(got_c, ref_c.numpy())
        assert torch.equal(su.get_particle_coordinates(apr, d, device=DEV).cpu(), ref_c)
        ref_s = oracle.sample_image_max(apr, img, d)
        assert np.array_equal(su.sample_image(apr, img.numpy(), d), ref_s.numpy())
        assert torch.equal(su.sample_image(apr, img.to(DEV), d).cpu(), ref_s)
        for dt in (torch.uint8, torch.uint16, torch.uint32, torch.uint64):
            labels = lab.to(torch.int64).to(dt)
            ref_d = oracle.labels_to_dist(apr, labels, rays[:, 0], rays[:, 1], rays[:, 2], d)
            got_d = su.labels_to_dist(apr, labels.to(DEV), rays.numpy(), level_delta=d)
            assert torch.equal(got_d.cpu(), ref_d), dt
        got_np = su.labels_to_dist(apr, lab.numpy().astype(np.uint16), rays.numpy(), step_factor=(2, 2, 2), level_delta=d)
        ref_np = oracle.labels_to_dist(apr, lab.to(torch.int64).to(torch.uint16), rays[:, 0] / 2, rays[:, 1] / 2, rays[:, 2] / 2, d)
        assert isinstance(got_np, np.ndarray) and np.array_equal(got_np, ref_np.numpy())
    with pytest.raises(ValueError):
        su.labels_to_dist(apr, np.zeros((Z + 1, X, Y), np.uint16), rays.numpy())
    with pytest.raises(ValueError):
        su.labels_to_dist(apr, np.zeros((Z, X, Y), np.uint16), np.zeros((2, 3), np.float32))
    with pytest.raises(TypeError):
        su.labels_to_dist(apr, np.zeros((Z, X, Y), np.float32), rays.numpy())
    with pytest.raises(ImportError):
        su.get_prob_apr(apr, np.zeros((Z, X, Y), np.uint16))            # stardist is not installed here
    prob = su.get_prob_apr(apr, lab.numpy().astype(np.uint16), prob_fn=lambda a: (a > 0).astype(np.float32))
    assert np.array_equal(prob, oracle.sample_image_max(apr, (lab > 0).float(), 0).numpy())


@pytest.mark.parametrize("bt,ksize", [([("3d_t", 0), ("3d_a", 1)], (3, 3, 3)), ([("3d_s", 0)], (3, 3, 3)),
                                      ([("2d_t", 0), ("2d_a", 0)], (1, 3, 3)), ([("2d_s", 1)], (1, 5, 5))],
                         ids=["333-odd", "333-odd-b", "133-2d", "155-2d"])
def test_conv_backward_fp32_repeats_bit_for_bit_on_odd_sizes(bt, ksize):
    """APRs whose levels have odd sizes hold coarse particles that stick out of the far faces of the next finer level.
    Their input gradient comes from the face lists of the plan (a fixed summation order), everything else receives at
    most two atomic contributions, and the weight gradient is summed from per-workgroup partials: three runs give
    identical bits, equal to the oracle within 1e-5, and equal (within 1e-5) to the run with atomic additions."""
    cin, cout = 12, 20
    x, aprs, ld, w_exp = _conv_case(bt, ksize, 2, cin, cout, torch.float32)
    g = torch.Generator().manual_seed(31)
    go = torch.randn(x.size(0), cout, x.size(2), generator=g)
    gx_ref, gw_ref = oracle.conv_backward(aprs, x, w_exp, go, ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    xd, god = x.to(DEV), go.to(DEV)
    runs = [_ops.conv_backward(aprs, xd, wd, god, ld) for _ in range(3)]
    for gx, gw in runs[1:]:
        assert torch.equal(gx, runs[0][0]) and torch.equal(gw, runs[0][1])
    close(runs[0][0], gx_ref, torch.float32)
    close(runs[0][1].permute(2, 0, 1, 3, 4, 5), gw_ref, torch.float32)
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(11) == 0
    try:
        gx_a, gw_a = _ops.conv_backward(aprs, xd, wd, god, ld)
    finally:
        lib.aprnet_set_conv_path(10)
    close(gx_a, gx_ref, torch.float32)
    close(gw_a.permute(2, 0, 1, 3, 4, 5), gw_ref, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64, torch.bfloat16], ids=["f32", "f64", "bf16"])
def test_conv111_backward_repeats_bit_for_bit(dtype):
    """The 1x1x1 weight gradient is summed from per-workgroup partials in a fixed order (each level range adds to its
    stencil's slot in turn) and the input gradient has one writer per element: three runs give identical bits, equal
    within the stated tolerance to the oracle and to the run with atomic additions (aprnet_set_conv_path(11))."""
    cin, cout = 12, 20
    cd = torch.float32 if dtype == torch.bfloat16 else dtype
    x, aprs, ld, w = _conv_case([("3d_t", 0), ("3d_a", 1), ("3d_s", 0)], (1, 1, 1), 2, cin, cout, cd)
    g = torch.Generator().manual_seed(33)
    go = torch.randn(x.size(0), cout, x.size(2), dtype=cd, generator=g)
    if dtype == torch.bfloat16:
        x, go = x.to(dtype).float(), go.to(dtype).float()          # the oracle sees the rounded values
    gx_ref, gw_ref = oracle.conv_backward(aprs, x, w, go, ld)
    wd = w.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    xd, god = x.to(dtype).to(DEV), go.to(dtype).to(DEV)
    runs = [_ops.conv_backward(aprs, xd, wd, god, ld) for _ in range(3)]
    for gx, gw in runs[1:]:
        assert torch.equal(gx, runs[0][0]) and torch.equal(gw, runs[0][1])
    lib = _native.hip()
    assert lib.aprnet_set_conv_path(11) == 0
    try:
        gx_a, gw_a = _ops.conv_backward(aprs, xd, wd, god, ld)
    finally:
        lib.aprnet_set_conv_path(10)
    assert torch.equal(gx_a, runs[0][0])
    for gw in (runs[0][1], gw_a):
        close(gw.permute(2, 0, 1, 3, 4, 5), gw_ref, cd)
    if dtype == torch.bfloat16:
        close_bf16(runs[0][0], gx_ref)
    else:
        close(runs[0][0], gx_ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3), (1, 5, 5)], ids=KID)
@pytest.mark.parametrize("cin,cout", [(1, 16), (1, 32), (2, 5), (3, 24), (2, 40)])
def test_conv_forward_narrow_input(cin, cout, ksize, dtype):
    """Layers of 1 to 3 input channels run on the pipelined kernel with the (tap, channel) axis flattened: against the
    oracle (batch of two APRs at different level deltas, bias, ReLU fused for one of the two runs), against the general
    matrix-core kernel (path 13), and bit-identical from run to run."""
    bt = [("3d_s", 0), ("3d_t", 1)] if ksize[0] == 3 else [("2d_t", 0), ("2d_s", 1), ("3d_s", 0)]
    x, aprs, ld, w_exp = _conv_case(bt, ksize, 2, cin, cout, torch.float32)
    g = torch.Generator().manual_seed(41)
    bias = torch.randn(cout, generator=g)
    xd = x.to(dtype).to(DEV)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    ref = oracle.conv_forward(aprs, xd.float().cpu(), w_exp, ld) + bias.view(1, -1, 1)
    for b, a in enumerate(aprs):                     # the oracle leaves padding slots at zero, the modules add the bias there
        ref[b, :, oracle.number_parts(a, int(ld[b])):] = bias.view(-1, 1)
    lib = _native.hip()
    got = _ops.conv_forward(aprs, xd, wd, ld, bias=bias.to(DEV))
    again = _ops.conv_forward(aprs, xd, wd, ld, bias=bias.to(DEV))
    fused = _ops.conv_forward(aprs, xd, wd, ld, bias=bias.to(DEV), relu=True)
    assert lib.aprnet_set_conv_path(13) == 0
    try:
        general = _ops.conv_forward(aprs, xd, wd, ld, bias=bias.to(DEV))
    finally:
        lib.aprnet_set_conv_path(12)
    assert torch.equal(got, again)
    if dtype == torch.float32:
        close(got, ref, dtype)
        close(general, ref, dtype)
        assert torch.equal(fused, torch.relu(got))
    else:
        close_bf16(got, ref)
        close_bf16(general, ref)
        assert torch.equal(fused, torch.relu(got))


def _tight(got32, ora32, ref64, terms64, what):
    """fp32 parity as a claim the arithmetic fixes, against the oracle run in float64 on the same fp32 inputs:
    (1) element by element, |hip - truth| <= 1e-5 * |truth| + 1e-5 * sum |terms|: the rounding of an fp32 sum is bounded
        by its terms, so an element that is small because large terms cancel is held to the size of the terms and every
        other element to rel 1e-5 (the reference's check is element-wise too: torch.allclose,
        pyapr/tests/test_aprnet.py:176-179);
    (2) the largest deviation from the truth stays within 8 x that of the reference's own fp32 loop order.  The two are
        not equal: the reference forms a dot product per input channel over the taps and adds those to the output (a
        two-level sum whose partial sums stay small), the kernels run one accumulator through all taps and channels
        of an output (864 terms at 32 channels), whose rounding grows with the running sum: measured 3 to 7 x for the
        forward pass on these cases (1.2e-6 of the output scale against 2e-7).  The factor records that; a loss of
        accuracy proper (products rounded to a shorter type, a dropped term) would be 100 x and more."""
    got, ora = got32.detach().cpu().double(), ora32.double()
    bound = 1e-5 * ref64.abs() + 1e-5 * terms64
    worst = float(((got - ref64).abs() - bound).max())
    assert worst <= 0.0, f"{what}: element-wise bound exceeded by {worst:.3e}"
    e_hip, e_ora = float((got - ref64).abs().max()), float((ora - ref64).abs().max())
    floor = 1e-7 * float(ref64.abs().max())             # both at the last bit of fp32
    assert e_hip <= 8.0 * e_ora + floor, f"{what}: HIP fp32 is {e_hip:.3e} from float64, the oracle's fp32 {e_ora:.3e}"
    return e_hip / max(e_ora, 1e-300)


@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 5, 5)], ids=KID)
@pytest.mark.parametrize("cin,cout", [(32, 32), (33, 33)])
def test_conv_fp32_is_as_close_to_float64_as_the_reference_order(cin, cout, ksize):
    """Forward, input gradient and weight gradient in fp32 against the oracle run in float64 on the same fp32 inputs
    and the same expanded stencils (so that only the convolution arithmetic differs)."""
    bt = [("3d_s", 0), ("3d_t", 1)] if ksize[0] == 3 else [("2d_s", 0), ("2d_t", 1)]
    x, aprs, ld, w_exp = _conv_case(bt, ksize, 2, cin, cout, torch.float32)
    go = torch.randn(x.size(0), cout, x.size(2), generator=torch.Generator().manual_seed(8))
    sizes = [oracle.number_parts(a, int(d)) for a, d in zip(aprs, ld)]
    for i, n in enumerate(sizes):
        go[i, :, n:] = 0
    x64, w64, go64 = x.double(), w_exp.double(), go.double()
    y32, y64 = oracle.conv_forward(aprs, x, w_exp, ld), oracle.conv_forward(aprs, x64, w64, ld)
    y_terms = oracle.conv_forward(aprs, x64.abs(), w64.abs(), ld)
    gx32, gw32 = oracle.conv_backward(aprs, x, w_exp, go, ld)
    gx64, gw64 = oracle.conv_backward(aprs, x64, w64, go64, ld)
    gx_terms, gw_terms = oracle.conv_backward(aprs, x64.abs(), w64.abs(), go64.abs(), ld)
    wd = w_exp.permute(1, 2, 0, 3, 4, 5).contiguous().to(DEV)
    y = _ops.conv_forward(aprs, x.to(DEV), wd, ld)
    gx, gw = _ops.conv_backward(aprs, x.to(DEV), wd, go.to(DEV), ld)
    ratios = (_tight(y, y32, y64, y_terms, "forward"), _tight(gx, gx32, gx64, gx_terms, "input gradient"),
              _tight(gw.permute(2, 0, 1, 3, 4, 5), gw32, gw64, gw_terms, "weight gradient"))
    print("deviation from float64, HIP fp32 / oracle fp32 (forward, input gradient, weight gradient): %.2f %.2f %.2f" % ratios)


def test_short_rows_are_refused_before_any_launch():
    """A tensor with fewer elements per channel than the APR has particles at the level delta must come back as
    APRNET_ERR_INVALID_ARGUMENT (-1) from the C ABI, not as an out-of-range device access."""
    apr = apr_cases.get("3d_b")
    apr.init_cuda()
    lib, plan = _native.hip(), apr.plan(0)
    n, n1, nt = oracle.number_parts(apr, 0), oracle.number_parts(apr, 1), _ops.tree_parts(apr, 0)
    x = torch.zeros(4, n, device=DEV)
    y = torch.zeros(4, n, device=DEV)
    w = torch.zeros(1, 4, 4, 3, 3, 3, device=DEV)
    tree = torch.zeros(4, max(nt, 1), device=DEV)
    idx = torch.zeros(4, n1, dtype=torch.int64, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    p = lambda t: C.c_void_p(t.data_ptr())
    torch.cuda.synchronize()
    assert lib.aprnet_conv_fwd_f32(plan, 0, 3, 3, 3, p(x), n - 1, 4, p(w), 1, 4, None, p(y), n, p(tree), max(nt, 1), st) == -1
    assert lib.aprnet_conv_fwd_f32(plan, 0, 3, 3, 3, p(x), n, 4, p(w), 1, 4, None, p(y), n - 1, p(tree), max(nt, 1), st) == -1
    assert b"holds" in lib.aprnet_last_error()
    assert lib.aprnet_conv111_fwd_f32(plan, 0, p(x), n - 1, 4, p(w), 1, 4, None, p(y), n, st) == -1
    assert lib.aprnet_maxpool_fwd_f32(plan, 0, p(x), n - 1, 4, p(y), n1, p(idx), n1, st) == -1
    assert lib.aprnet_maxpool_fwd_f32(plan, 0, p(x), n, 4, p(y), n1 - 1, p(idx), n1, st) == -1
    assert lib.aprnet_maxpool_fwd_f32(plan, 0, p(x), n, 4, p(y), n1, p(idx), n1 - 1, st) == -1
    assert lib.aprnet_upsample_fwd_f32(plan, 1, p(x), n1 - 1, 4, p(y), n, st) == -1
    assert lib.aprnet_upsample_fwd_f32(plan, 1, p(x), n1, 4, p(y), n - 1, st) == -1
    assert lib.aprnet_upsample_bwd_f32(plan, 1, p(x), n - 1, 4, p(y), n1, st) == -1
    assert lib.aprnet_fill_tree_mean_f32(plan, 0, p(x), n - 1, 4, p(tree), max(nt, 1), st) == -1
    xg = torch.zeros(1, n, 8, dtype=torch.bfloat16, device=DEV)
    assert lib.aprnet_conv111_fwd_bf16g(plan, 0, p(xg), n - 1, 8, p(w), 1, 8, None, 0, p(xg), n, 1, st) == -1
    # the reference-named binding: one batch item per APR
    import _pyaprwrapper
    ldt = torch.zeros(1, dtype=torch.int32)
    with pytest.raises(ValueError, match="batch"):
        _pyaprwrapper.aprnet.cuda.conv333_forward([apr, apr], x.view(1, 4, n), w, torch.zeros(2, dtype=torch.int32))
    with pytest.raises(ValueError, match="holds"):
        _pyaprwrapper.aprnet.cuda.conv333_forward([apr], x.view(1, 4, n)[:, :, :n - 1].contiguous(), w, ldt)
    torch.cuda.synchronize()


# ------------------------------------------------------------------------- tree fill restricted to the nodes read
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cin", [2, 8], ids=["narrow", "general"])
@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3), (1, 5, 5)], ids=KID)
def test_conv_forward_fills_only_the_tree_nodes_it_reads(ksize, cin, dtype):
    """Before a forward convolution the library fills the mean tree at the nodes the kernel's window lists name (and
    their descendants), not at every node (aprnet_set_conv_path(16), the default; 17 fills all).  With the work space
    poisoned beforehand: same bits in the output either way, no NaN reaches it, the filled nodes hold the values of the
    full fill, and on APRs with resolved interiors some nodes stay untouched (the restriction is in effect)."""
    lib = _native.hip()
    sfx = "f32" if dtype == torch.float32 else "bf16"
    fn = getattr(lib, "aprnet_conv_fwd_" + sfx)
    untouched = 0
    for name, d in [("3d_s", 0), ("3d_t", 0), ("3d_a", 0), ("3d_b", 1), ("2d_a", 0), ("2d_t", 1)]:
        apr = apr_cases.get(name)
        apr.init_cuda()
        n, nt = oracle.number_parts(apr, d), max(oracle.tree_parts(apr, d), 1)
        g = torch.Generator().manual_seed(n)
        x = torch.randn(cin, n, generator=g).to(dtype).to(DEV)
        S = apr.level_max() - apr.level_min() + 1
        w = torch.randn(S, 5, cin, *ksize, generator=g).to(DEV)
        st = torch.cuda.current_stream().cuda_stream
        outs, trees = [], []
        for path in (16, 17):
            tree = torch.full((cin, nt), float("nan"), dtype=dtype, device=DEV)
            y = torch.zeros(5, n, dtype=dtype, device=DEV)
            assert lib.aprnet_set_conv_path(path) == 0
            try:
                rc = fn(apr.plan(0), d, *ksize, x.data_ptr(), n, cin, w.data_ptr(), S, 5, None, y.data_ptr(), n, tree.data_ptr(), nt, st)
            finally:
                lib.aprnet_set_conv_path(16)
            assert rc == 0, lib.aprnet_last_error()
            outs.append(y.cpu()); trees.append(tree.float().cpu())
        assert not torch.isnan(outs[0]).any() and not torch.isnan(outs[1]).any()
        assert torch.equal(outs[0], outs[1]), (name, d)
        filled = ~torch.isnan(trees[0])
        assert not torch.isnan(trees[1][:, :oracle.tree_parts(apr, d)]).any()
        assert torch.equal(trees[0][filled], trees[1][filled])
        untouched += int((~filled).sum())
    assert untouched > 0
