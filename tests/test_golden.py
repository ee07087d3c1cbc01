"""Frozen vectors (tests/golden/operators_small.npz, written by tests/golden/make_vectors.py): the CPU oracle must
keep reproducing them, and the HIP path must match them through the C ABI.  The APRs come from the stored access
arrays, so neither side depends on the APR builder."""
import os

import numpy as np
import pytest
import torch

import pyapr
from oracle import oracle

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "operators_small.npz")
STENCILS = {"3d": [(3, 3, 3), (1, 1, 1)], "3d_coarse": [(3, 3, 3), (5, 5, 5)], "2d": [(1, 3, 3), (1, 5, 5)]}
TAGS = list(STENCILS)
DEV = "cuda:0"


@pytest.fixture(scope="module")
def vec():
    with np.load(PATH, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def _apr(vec, tag):
    return pyapr.APR.from_state(vec[f"{tag}/org_dims"], vec[f"{tag}/xz_end_vec"], vec[f"{tag}/y_vec"],
                                vec[f"{tag}/tree_xz_end_vec"], vec[f"{tag}/tree_y_vec"])


def _close(got, want, tol):
    got = got.detach().cpu().numpy() if isinstance(got, torch.Tensor) else np.asarray(got)
    assert got.shape == want.shape and got.dtype == want.dtype
    assert float(np.abs(got.astype(np.float64) - want).max()) <= tol * max(float(np.abs(want).max()), 1e-30)


@pytest.mark.parametrize("tag", TAGS)
def test_oracle_reproduces_the_frozen_vectors(vec, tag):
    apr = _apr(vec, tag)
    d = int(vec[f"{tag}/level_delta"])
    ld = torch.tensor([d], dtype=torch.int32)
    x = torch.from_numpy(vec[f"{tag}/x"])
    assert x.shape[2] == oracle.number_parts(apr, d)
    tol = 1e-6          # same code, same order of operations; the slack covers a different compiler or libm only
    _close(torch.stack([oracle.fill_tree_mean(apr, x[0, c], d) for c in range(x.shape[1])]), vec[f"{tag}/fill_tree_mean"], tol)
    for k in STENCILS[tag]:
        ks = "%d%d%d" % k
        w = torch.from_numpy(vec[f"{tag}/conv{ks}/w"])
        w_exp = w if k == (1, 1, 1) else oracle.restrict_kernel_forward(w, apr.level_max() - apr.level_min() + 1)
        _close(w_exp, vec[f"{tag}/conv{ks}/w_expanded"], tol)
        _close(oracle.conv_forward([apr], x, w_exp, ld), vec[f"{tag}/conv{ks}/y"], tol)
        gx, gw = oracle.conv_backward([apr], x, w_exp, torch.from_numpy(vec[f"{tag}/conv{ks}/grad_y"]), ld)
        _close(gx, vec[f"{tag}/conv{ks}/grad_x"], tol)
        _close(gw, vec[f"{tag}/conv{ks}/grad_w_expanded"], tol)
    pooled, idx = oracle.maxpool_forward([apr], x, ld)
    assert np.array_equal(pooled.numpy(), vec[f"{tag}/maxpool/y"]) and np.array_equal(idx.numpy(), vec[f"{tag}/maxpool/argmax"])
    gp = torch.from_numpy(vec[f"{tag}/maxpool/grad_y"])
    assert np.array_equal(oracle.maxpool_backward([apr], gp, idx, ld).numpy(), vec[f"{tag}/maxpool/grad_x"])
    assert np.array_equal(oracle.upsample_const_forward([apr], pooled, ld + 1).numpy(), vec[f"{tag}/upsample/y"])
    _close(oracle.upsample_const_backward([apr], x, ld + 1), vec[f"{tag}/upsample/grad_x"], tol)
    if f"{tag}/reconstruct/y" in vec:
        img = oracle.reconstruct_forward([apr], x, ld)
        assert np.array_equal(img.numpy(), vec[f"{tag}/reconstruct/y"])
        _close(oracle.sample_particles_forward([apr], img, ld), vec[f"{tag}/sample_particles/y"], tol)


@pytest.mark.gpu
@pytest.mark.parametrize("tag", TAGS)
def test_hip_path_matches_the_frozen_vectors(vec, tag):
    """fp32: 1e-5 of each tensor's scale for the sums, bit-exact for what only moves values (pool, argmax, upsample,
    reconstruct) and for the tree fill, whose sums keep the reference's order."""
    from pyapr.aprnet import _ops
    apr = _apr(vec, tag)
    d = int(vec[f"{tag}/level_delta"])
    ld = torch.tensor([d], dtype=torch.int32)
    x = torch.from_numpy(vec[f"{tag}/x"]).to(DEV)
    tol = 1e-5
    from pyapr import _native
    nt, n, cin = vec[f"{tag}/fill_tree_mean"].shape[-1], x.shape[2], x.shape[1]
    tree = torch.zeros(cin, max(nt, 1), device=DEV)
    rc = _native.hip().aprnet_fill_tree_mean_f32(apr.plan(0), d, x.data_ptr(), n, cin, tree.data_ptr(), max(nt, 1),
                                                torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert np.array_equal(tree[:, :nt].cpu().numpy(), vec[f"{tag}/fill_tree_mean"])
    for k in STENCILS[tag]:
        ks = "%d%d%d" % k
        w = torch.from_numpy(vec[f"{tag}/conv{ks}/w"]).to(DEV)
        wd = w.permute(1, 2, 0, 3, 4, 5).contiguous()                                   # -> [S, Cout, Cin, k]
        if k != (1, 1, 1):
            wd = _ops.restrict_kernel_forward(wd, apr.level_max() - apr.level_min() + 1)
        _close(wd.permute(2, 0, 1, 3, 4, 5).contiguous(), vec[f"{tag}/conv{ks}/w_expanded"], tol)
        _close(_ops.conv_forward([apr], x, wd, ld), vec[f"{tag}/conv{ks}/y"], tol)
        gx, gw = _ops.conv_backward([apr], x, wd, torch.from_numpy(vec[f"{tag}/conv{ks}/grad_y"]).to(DEV), ld)
        _close(gx, vec[f"{tag}/conv{ks}/grad_x"], tol)
        _close(gw.permute(2, 0, 1, 3, 4, 5).contiguous(), vec[f"{tag}/conv{ks}/grad_w_expanded"], tol)
    pooled, idx = _ops.maxpool_forward([apr], x, ld)
    assert np.array_equal(pooled.cpu().numpy(), vec[f"{tag}/maxpool/y"]) and np.array_equal(idx.cpu().numpy(), vec[f"{tag}/maxpool/argmax"])
    gp = torch.from_numpy(vec[f"{tag}/maxpool/grad_y"]).to(DEV)
    assert np.array_equal(_ops.maxpool_backward([apr], gp, idx, ld).cpu().numpy(), vec[f"{tag}/maxpool/grad_x"])
    assert np.array_equal(_ops.upsample_const_forward([apr], pooled, ld + 1).cpu().numpy(), vec[f"{tag}/upsample/y"])
    _close(_ops.upsample_const_backward([apr], x, ld + 1), vec[f"{tag}/upsample/grad_x"], tol)
    if f"{tag}/reconstruct/y" in vec:
        img = _ops.reconstruct_forward([apr], x, ld)
        assert np.array_equal(img.cpu().numpy(), vec[f"{tag}/reconstruct/y"])
        _close(_ops.sample_particles_forward([apr], img, ld), vec[f"{tag}/sample_particles/y"], tol)


def test_spheres128_golden_summary_matches_the_oracle():
    """BASELINE configs[0] on the CPU: the builder reproduces the committed particle counts per level and the oracle
    reproduces the committed per-channel sums and first / last 64 output values (the cross-machine check)."""
    import json
    import os
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    sys.path.insert(0, os.path.join(here, "golden"))
    import make_spheres128
    gold = json.load(open(os.path.join(here, "golden", "spheres128_conv_1to16.json")))
    now = make_spheres128.summary(*make_spheres128.oracle_output())
    assert now["n_particles"] == gold["n_particles"] and now["levels"] == gold["levels"]
    scale = max(gold["abs_max"])
    for c in range(16):
        assert abs(now["sum"][c] - gold["sum"][c]) <= 1e-6 * scale * gold["n_particles"] ** 0.5
        assert max(abs(a - b) for a, b in zip(now["first64"][c], gold["first64"][c])) <= 1e-6 * scale
        assert max(abs(a - b) for a, b in zip(now["last64"][c], gold["last64"][c])) <= 1e-6 * scale
