"""Pins the CPU oracle (oracle/aprnet_oracle.cpp) against an independent dense formulation
(oracle/dense_ref.py: F.conv3d / block means / brute-force search on dense level views) on tiny
random APRs with odd sizes in 1-D, 2-D and 3-D.  float64, tolerance 1e-12 (the two sides only differ
in summation order)."""
import numpy as np
import pytest
import torch

import apr_cases
from oracle import oracle, dense_ref

CASES = list(apr_cases.TINY)
TOL = dict(rtol=1e-11, atol=1e-12)


@pytest.fixture(scope="module", params=CASES)
def case(request):
    apr = apr_cases.get(request.param)
    return apr, dense_ref.DenseAPR(apr)


def _max_delta(apr):
    return min(2, apr.level_max() - 1)


def test_structure_invariants(case):
    """What the operators silently rely on: partition, complete sibling sets, tree = strict ancestors,
    2:1 balance over the 26-neighbourhood, ascending y per row, level-major order."""
    apr, D = case
    lmax = apr.level_max()
    pset = {tuple(c) for c in D.pc}
    tset = {tuple(c) for c in D.tc}
    assert len(pset) == len(D.pc) and len(tset) == len(D.tc)
    assert not (pset & tset)
    # index order: level-major, then z, x, y
    for arr in (D.pc, D.tc):
        keys = [tuple(c) for c in arr]
        assert keys == sorted(keys)
    # every particle / tree node (level > 0) has its parent in the tree; tree nodes have all in-image children
    for (l, z, x, y) in list(pset) + [t for t in tset if t[0] > 0]:
        assert (l - 1, z // 2, x // 2, y // 2) in tset
    for (l, z, x, y) in tset:
        assert l <= lmax - 1
        dz, dx, dy = apr.level_dims(l + 1)
        for cz in (2 * z, 2 * z + 1):
            for cx in (2 * x, 2 * x + 1):
                for cy in (2 * y, 2 * y + 1):
                    if cz < dz and cx < dx and cy < dy:
                        assert ((l + 1, cz, cx, cy) in pset) != ((l + 1, cz, cx, cy) in tset)
    # partition of the finest grid (views() asserts full coverage) and 2:1 balance: every in-grid
    # neighbour (half-width 2) of a particle of level l is a level-l particle, a level-l tree node or
    # lies inside a level l-1 particle
    D.views(torch.zeros(1, D.n_parts(0), dtype=torch.float64), 0)
    for (l, z, x, y) in pset:
        dz, dx, dy = apr.level_dims(l)
        for nz in range(max(z - 2, 0), min(z + 3, dz)):
            for nx in range(max(x - 2, 0), min(x + 3, dx)):
                for ny in range(max(y - 2, 0), min(y + 3, dy)):
                    c = (l, nz, nx, ny)
                    assert c in pset or c in tset or (l - 1, nz // 2, nx // 2, ny // 2) in pset


def test_number_parts_and_offsets(case):
    apr, D = case
    for d in range(0, apr.level_max()):
        assert oracle.number_parts(apr, d) == D.n_parts(d)
        lc = apr.level_max() - d
        assert oracle.tree_offset(apr, lc) == D.tree_offset(lc)
        assert oracle.tree_parts(apr, d) == int((D.tc[:, 0] < lc).sum())


def test_parent_index_bit_exact(case):
    apr, D = case
    for level in range(1, apr.level_max() + 1):
        got = oracle.parent_index(apr, 0, level)
        assert np.array_equal(got[D.pc[:, 0] == level], D.parent_index(0, level)[D.pc[:, 0] == level])
    for level in range(1, apr.level_max()):
        got = oracle.parent_index(apr, 1, level)
        assert np.array_equal(got[D.tc[:, 0] == level], D.parent_index(1, level)[D.tc[:, 0] == level])


def test_fill_tree_mean(case):
    apr, D = case
    for d in range(0, _max_delta(apr) + 1):
        g = torch.Generator().manual_seed(10 + d)
        x = torch.randn(D.n_parts(d), dtype=torch.float64, generator=g)
        torch.testing.assert_close(oracle.fill_tree_mean(apr, x, d), D.fill_tree_mean(x, d), **TOL)


@pytest.mark.parametrize("ksize", [(3, 3, 3), (1, 3, 3), (1, 5, 5), (5, 5, 5), (1, 1, 1)])
@pytest.mark.parametrize("nstencils", [1, 2, 3])
def test_conv_forward(case, ksize, nstencils):
    apr, D = case
    cin, cout = 2, 3
    num_levels = apr.level_max() - apr.level_min() + 1
    for d in range(0, _max_delta(apr) + 1):
        g = torch.Generator().manual_seed(100 * nstencils + d)
        x = torch.randn(1, cin, D.n_parts(d), dtype=torch.float64, generator=g)
        w = torch.randn(cin, nstencils, cout, *ksize, dtype=torch.float64, generator=g)
        w_exp = w if ksize == (1, 1, 1) else oracle.restrict_kernel_forward(w, num_levels)
        got = oracle.conv_forward([apr], x, w_exp, torch.tensor([d], dtype=torch.int32))
        torch.testing.assert_close(got[0], D.conv(x[0], w_exp, d), **TOL)


def test_conv_linear_in_channels(case):
    """Output accumulates over input channels (conv.hpp:107, helpers.hpp:543): f([x0,x1]) = f(x0) + f(x1)."""
    apr, D = case
    g = torch.Generator().manual_seed(7)
    x = torch.randn(1, 2, D.n_parts(0), dtype=torch.float64, generator=g)
    w = torch.randn(2, 1, 2, 3, 3, 3, dtype=torch.float64, generator=g)
    ld = torch.zeros(1, dtype=torch.int32)
    full = oracle.conv_forward([apr], x, w, ld)
    parts = sum(oracle.conv_forward([apr], x[:, c:c + 1], w[c:c + 1], ld) for c in range(2))
    torch.testing.assert_close(full, parts, **TOL)


def test_maxpool_values_and_argmax_with_ties(case):
    apr, D = case
    for d in range(0, _max_delta(apr)):
        g = torch.Generator().manual_seed(20 + d)
        # few distinct values -> many ties, as after a ReLU
        x = torch.randint(0, 3, (1, 2, D.n_parts(d)), generator=g).to(torch.float64)
        out, idx = oracle.maxpool_forward([apr], x, torch.tensor([d], dtype=torch.int32))
        ref_out, ref_idx = D.maxpool(x[0], d)
        assert torch.equal(out[0], ref_out)
        ncopy = apr.iterator().total_number_particles(apr.level_max() - d - 1) if apr.level_max() - d - 1 >= 1 else 0
        assert torch.equal(idx[0][:, ncopy:], ref_idx[:, ncopy:])
        assert torch.equal(idx[0][:, :ncopy], torch.zeros_like(idx[0][:, :ncopy]))   # zeros, maxpool.hpp:52


def test_upsample(case):
    apr, D = case
    for d in range(1, _max_delta(apr) + 1):
        g = torch.Generator().manual_seed(30 + d)
        x = torch.randn(1, 2, D.n_parts(d), dtype=torch.float64, generator=g)
        out = oracle.upsample_const_forward([apr], x, torch.tensor([d], dtype=torch.int32))
        assert torch.equal(out[0], D.upsample(x[0], d))
    with pytest.raises(ValueError):
        oracle.upsample_const_forward([apr], torch.zeros(1, 1, D.n_parts(0), dtype=torch.float64),
                                      torch.zeros(1, dtype=torch.int32))


def test_reconstruct_and_sample(case):
    apr, D = case
    for d in range(0, _max_delta(apr) + 1):
        g = torch.Generator().manual_seed(40 + d)
        ld = torch.tensor([d], dtype=torch.int32)
        x = torch.randn(1, 2, D.n_parts(d), dtype=torch.float64, generator=g)
        img = oracle.reconstruct_forward([apr], x, ld)
        assert torch.equal(img[0], D.reconstruct(x[0], d))
        # SampleParticles(Reconstruct(x)) == x  (pyapr/tests/test_aprnet.py:272-285)
        torch.testing.assert_close(oracle.sample_particles_forward([apr], img, ld), x, **TOL)
        # sampling an arbitrary image = mean over each particle's cell
        im = torch.randn_like(img)
        s = oracle.sample_particles_forward([apr], im, ld)
        lc = apr.level_max() - d
        for idx, l, z, xx, y in D.outputs(d)[::7]:
            f = 1 << (lc - int(l))
            cell = im[0, :, z * f:(z + 1) * f, xx * f:(xx + 1) * f, y * f:(y + 1) * f]
            torch.testing.assert_close(s[0, :, idx], cell.mean(dim=(1, 2, 3)), **TOL)


# ------------------------------------------------------------------------------------ StarDist utilities
def test_particle_coords_closed_form(case):
    """get_particle_coords: centre of every feature's cell in pixels, floor((c + 0.5) * 2^(lmax - l)), in feature
    order (particles of levels <= Lc, then the tree nodes of level Lc)."""
    apr, D = case
    lmax = apr.level_max()
    for d in range(_max_delta(apr) + 1):
        got = oracle.particle_coords(apr, d)
        outs = D.outputs(d)                      # (feature index, level, z, x, y)
        assert got.shape == (len(outs), 3)
        for i, l, z, x, y in outs:
            f = 2 ** (lmax - l)
            want = [np.floor((c + 0.5) * f) for c in (z, x, y)]
            assert got[i].tolist() == want


def test_sample_image_reads_a_max_pyramid(case):
    """sample_image: every feature takes the entry of its cell in a pyramid built by maxima.  The pyramid here is
    F.max_pool3d(kernel 2, ceil_mode=True) applied level by level (partial blocks at the far faces hold the maximum
    of the pixels that exist)."""
    apr, D = case
    lmax = apr.level_max()
    g = torch.Generator().manual_seed(3)
    img = torch.randn(*apr.shape(), generator=g)
    pyr = {lmax: img}
    for l in range(lmax - 1, -1, -1):
        pyr[l] = torch.nn.functional.max_pool3d(pyr[l + 1][None, None], 2, ceil_mode=True)[0, 0]
    for d in range(_max_delta(apr) + 1):
        got = oracle.sample_image_max(apr, img, d)
        for i, l, z, x, y in D.outputs(d):
            assert float(got[i]) == float(pyr[l][z, x, y])


def test_labels_to_dist_on_a_cuboid():
    """labels_to_dist: inside an axis-aligned cuboid label the distance along +-axis rays is the number of steps to
    the first pixel outside, along a face diagonal sqrt(2) times the smaller of the two; label 0 gives 0."""
    apr = apr_cases.get("3d_c")                                   # 16 x 16 x 16
    Z, X, Y = apr.shape()
    lab = torch.zeros(Z, X, Y, dtype=torch.uint16)
    z0, z1, x0, x1, y0, y1 = 3, 12, 2, 9, 5, 14
    lab[z0:z1, x0:x1, y0:y1] = 7
    lab[0:2, 0:2, 0:2] = 3                                        # a second object, touching the image corner
    rays = torch.tensor([[1, 0, 0], [-1, 0, 0], [0, 1, 0], [0, -1, 0], [0, 0, 1], [0, 0, -1], [1, 1, 0], [0, -1, -1]],
                        dtype=torch.float32)
    for d in (0, 1):
        dist = oracle.labels_to_dist(apr, lab, rays[:, 0], rays[:, 1], rays[:, 2], d)
        coords = oracle.particle_coords(apr, d).long()
        inside = 0
        for n in range(coords.shape[0]):
            i, j, k = coords[n].tolist()
            v = int(lab[i, j, k]) if (i < Z and j < X and k < Y) else 0
            if v == 0:
                assert float(dist[n].abs().max()) == 0.0
                continue
            b = (z0, z1, x0, x1, y0, y1) if v == 7 else (0, 2, 0, 2, 0, 2)
            want = [b[1] - i, i - b[0] + 1, b[3] - j, j - b[2] + 1, b[5] - k, k - b[4] + 1,
                    np.sqrt(2.0) * min(b[1] - i, b[3] - j), np.sqrt(2.0) * min(j - b[2] + 1, k - b[4] + 1)]
            np.testing.assert_allclose(dist[n].numpy(), np.asarray(want, np.float32), rtol=1e-6)
            inside += 1
        assert inside > 0
