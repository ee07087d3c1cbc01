"""Pins the oracle's backward passes: float64 torch.autograd.gradcheck with the settings of the
reference's (commented-out) CPU gradchecks, pyapr/tests/test_aprnet.py:86-131 (eps 1e-6, nstencils 3,
kernel sizes 1/3/5 in 2-D and 3-D, mixed level deltas in one batch), plus the tree-fill adjoint identity
and RestrictKernel against the compiled reference header and its closed-form invariants."""
import ctypes as C
import os

import numpy as np
import pytest
import torch
from torch.autograd import gradcheck

import apr_cases
from oracle import oracle
from oracle_modules import OracleConv, OracleMaxPool, OracleUpSample, OracleReconstruct, OracleSample


def _batch(names_d, channels, seed=0):
    aprs = [apr_cases.get(n) for n, _ in names_d]
    ld = torch.tensor([d for _, d in names_d], dtype=torch.int32)
    sizes = [oracle.number_parts(a, int(d)) for a, d in zip(aprs, ld)]
    g = torch.Generator().manual_seed(seed)
    x = torch.rand(len(aprs), channels, max(sizes), dtype=torch.float64, generator=g)
    for i, n in enumerate(sizes):
        x[i, :, n:] = 0
    return x.requires_grad_(True), aprs, ld


BATCHES_2D = [[("2d_a", 0)], [("2d_a", 1), ("2d_b", 2)]]
BATCHES_3D = [[("3d_a", 0)], [("3d_b", 1)], [("3d_a", 2), ("3d_c", 2)]]


@pytest.mark.parametrize("batch", BATCHES_2D + BATCHES_3D)
def test_maxpool_gradcheck(batch):
    x, aprs, ld = _batch(batch, 2)
    with torch.no_grad():                      # distinct values: max-pool is not differentiable at ties
        x += 10 * torch.arange(x.shape[2], dtype=torch.float64)
    assert gradcheck(lambda t: OracleMaxPool.apply(t, aprs, ld), (x,), eps=1e-6)


@pytest.mark.parametrize("batch", BATCHES_2D)
@pytest.mark.parametrize("k", [1, 3, 5])
def test_conv2d_gradcheck(batch, k):
    x, aprs, ld = _batch(batch, 2)
    g = torch.Generator().manual_seed(k)
    w = torch.randn(2, 3, 2, 1, k, k, dtype=torch.float64, generator=g).requires_grad_(True)
    b = torch.randn(2, dtype=torch.float64, generator=g).requires_grad_(True)
    assert gradcheck(lambda xi, wi, bi: OracleConv.apply(xi, wi, bi, aprs, ld), (x, w, b), eps=1e-6)


@pytest.mark.parametrize("batch", BATCHES_3D)
@pytest.mark.parametrize("k", [1, 3, 5])
def test_conv3d_gradcheck(batch, k):
    x, aprs, ld = _batch(batch, 2)
    g = torch.Generator().manual_seed(k)
    w = torch.randn(2, 3, 1, k, k, k, dtype=torch.float64, generator=g).requires_grad_(True)
    b = torch.randn(1, dtype=torch.float64, generator=g).requires_grad_(True)
    assert gradcheck(lambda xi, wi, bi: OracleConv.apply(xi, wi, bi, aprs, ld), (x, w, b), eps=1e-6)


@pytest.mark.parametrize("batch", [[("2d_a", 1)], [("2d_a", 1), ("2d_b", 2)], [("3d_a", 1)], [("3d_b", 1), ("3d_c", 2)]])
def test_upsample_gradcheck(batch):
    x, aprs, ld = _batch(batch, 2)
    assert gradcheck(lambda t: OracleUpSample.apply(t, aprs, ld), (x,), eps=1e-6)


@pytest.mark.parametrize("batch", [[("3d_a", 0)], [("3d_b", 1)], [("3d_c", 2)], [("2d_a", 1)]])
def test_reconstruct_and_sample_gradcheck(batch):
    x, aprs, ld = _batch(batch, 2)
    assert gradcheck(lambda t: OracleReconstruct.apply(t, aprs, ld), (x,), eps=1e-6)
    img = torch.rand_like(oracle.reconstruct_forward(aprs, x.detach(), ld)).requires_grad_(True)
    assert gradcheck(lambda t: OracleSample.apply(t, aprs, ld), (img,), eps=1e-6)


@pytest.mark.parametrize("name", ["3d_a", "2d_b", "1d_a"])
def test_fill_tree_adjoint(name):
    """<fill(x), g> == <x, fill_backward(g)> for the linear tree fill (helpers.hpp:156-350)."""
    apr = apr_cases.get(name)
    for d in range(0, min(2, apr.level_max() - 1) + 1):
        n, nt = oracle.number_parts(apr, d), oracle.tree_parts(apr, d)
        g = torch.Generator().manual_seed(d)
        x = torch.randn(n, dtype=torch.float64, generator=g)
        gt = torch.randn(nt, dtype=torch.float64, generator=g)
        lhs = torch.dot(oracle.fill_tree_mean(apr, x, d), gt)
        rhs = torch.dot(x, oracle.fill_tree_mean_backward(apr, gt, n, d))
        torch.testing.assert_close(lhs, rhs, rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------------------------ RestrictKernel
_REF = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "libref_restrict.so")


def _ref_restrict(backward, w, s_out):
    lib = C.CDLL(_REF)
    cin, s_in, cout, kz, kx, ky = w.shape
    out = torch.zeros(cin, s_out, cout, kz, kx, ky, dtype=torch.float64)
    rc = lib.ref_restrict_kernel(int(backward), kz, kx, ky, C.c_void_p(w.data_ptr()), C.c_void_p(out.data_ptr()),
                                 cin, s_in, s_out, cout)
    assert rc == 0
    return out


@pytest.mark.skipif(not os.path.exists(_REF), reason="oracle/_ref not built (reference tree absent)")
@pytest.mark.parametrize("k", [(3, 3, 3), (1, 3, 3), (1, 5, 5), (5, 5, 5)])
@pytest.mark.parametrize("s,levels", [(1, 4), (2, 5), (3, 3), (3, 7)])
def test_restrict_kernel_matches_compiled_reference(k, s, levels):
    g = torch.Generator().manual_seed(s * 10 + levels)
    w = torch.randn(2, s, 3, *k, dtype=torch.float64, generator=g)
    # equal up to fused-multiply-add contraction (the two sides are built with different -march flags)
    torch.testing.assert_close(oracle.restrict_kernel_forward(w, levels), _ref_restrict(False, w, levels), rtol=1e-14, atol=1e-15)
    gw = torch.randn(2, levels, 3, *k, dtype=torch.float64, generator=g)
    torch.testing.assert_close(oracle.restrict_kernel_backward(gw, s), _ref_restrict(True, gw, s), rtol=1e-14, atol=1e-15)


@pytest.mark.parametrize("k", [(3, 3, 3), (1, 3, 3), (1, 5, 5), (5, 5, 5)])
def test_restrict_kernel_invariants(k):
    """Levels < S are copied; for 3-D stencils the restricted stencil keeps the weight sum, and a
    (1,k,k) stencil gains a factor `step` per expanded level (overlap of the singleton dimension is
    `step` but ndim does not count it, kernel.hpp:59,78-80); backward is the transpose."""
    s, levels = 2, 5
    g = torch.Generator().manual_seed(3)
    w = torch.randn(2, s, 3, *k, dtype=torch.float64, generator=g)
    we = oracle.restrict_kernel_forward(w, levels)
    assert torch.equal(we[:, :s], w)
    base = w[:, s - 1].sum(dim=(-1, -2, -3))
    for j in range(s, levels):
        step = 2 ** (j - (s - 1))
        scale = step if k[0] == 1 else 1
        torch.testing.assert_close(we[:, j].sum(dim=(-1, -2, -3)), base * scale, rtol=1e-12, atol=1e-12)
    gwe = torch.randn_like(we)
    torch.testing.assert_close((we * gwe).sum(), (w * oracle.restrict_kernel_backward(gwe, s)).sum(), rtol=1e-12, atol=1e-12)
    # 3x3x3, one level up (step 2): the centre tap of the restricted stencil collects, per dimension,
    # overlaps (1,2,1)/2 of the source taps -> closed form
    if k == (3, 3, 3):
        src = w[0, s - 1, 0]
        ov = torch.tensor([0.5, 1.0, 0.5], dtype=torch.float64)     # overlap of source tap i with the centre cell / step
        expect = torch.einsum("zxy,z,x,y->", src, ov, ov, ov)
        torch.testing.assert_close(we[0, s, 0, 1, 1, 1], expect, rtol=1e-12, atol=1e-12)


def test_restrict_kernel_refuses_fewer_levels_than_stencils():
    """kernel.hpp:70-74 copies every given stencil into an output that holds num_levels of them, which writes out
    of bounds when num_levels < num_stencils; the restatement raises instead of following it there."""
    w = torch.zeros(2, 3, 2, 3, 3, 3)
    with pytest.raises(ValueError):
        oracle.restrict_kernel_forward(w, 2)
    with pytest.raises(ValueError):
        oracle.restrict_kernel_backward(torch.zeros(2, 2, 2, 3, 3, 3), 3)
    assert tuple(oracle.restrict_kernel_forward(w, 3).shape) == (2, 3, 2, 3, 3, 3)
