"""Writes tests/golden/operators_small.npz: frozen inputs and expected outputs of every operator on two small APRs.

The reference keeps no golden vectors for this path (its fixtures are git-ignored upstream, its tests are property
tests), and it cannot be run here, so these vectors were produced by the CPU oracle of this repository after that
oracle had been pinned against closed forms, dense torch operators and brute force (tests/test_oracle_*.py).  They
freeze its answers: a later change to the oracle or to the HIP kernels that moves a result shows up against them.
The APRs are stored as their access arrays (the state of BindAPR.hpp:72-90), not rebuilt, so the vectors do not
depend on the builder either.

    python tests/golden/make_vectors.py        # from the repository root, CPU only
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path[:0] = [ROOT, os.path.join(ROOT, "apr-cnn_amd"), os.path.join(ROOT, "tests")]

import apr_cases                      # noqa: E402
from oracle import oracle             # noqa: E402

CASES = [("3d", "3d_c", 0), ("3d_coarse", "3d_b", 1), ("2d", "2d_a", 1)]          # (tag, APR case, level_delta)
STENCILS = {"3d": [(3, 3, 3), (1, 1, 1)], "3d_coarse": [(3, 3, 3), (5, 5, 5)], "2d": [(1, 3, 3), (1, 5, 5)]}


def main():
    out = {}
    g = torch.Generator().manual_seed(2024)
    for tag, name, d in CASES:
        apr = apr_cases.get(name)
        oy, ox, oz, _par, xze, yv, txze, tyv = apr.get_state()
        out[f"{tag}/org_dims"] = np.array([oy, ox, oz], np.int64)
        out[f"{tag}/xz_end_vec"], out[f"{tag}/y_vec"] = xze, yv
        out[f"{tag}/tree_xz_end_vec"], out[f"{tag}/tree_y_vec"] = txze, tyv
        out[f"{tag}/level_delta"] = np.array(d, np.int32)
        ld = torch.tensor([d], dtype=torch.int32)
        n = oracle.number_parts(apr, d)
        cin, cout, S = 3, 4, 2
        x = torch.randn(1, cin, n, generator=g)
        out[f"{tag}/x"] = x.numpy()
        out[f"{tag}/fill_tree_mean"] = torch.stack([oracle.fill_tree_mean(apr, x[0, c], d) for c in range(cin)]).numpy()
        for k in STENCILS[tag]:
            ks = "%d%d%d" % k
            w = torch.randn(cin, S, cout, *k, generator=g) * 0.3                 # CPU-flavour layout [Cin, S, Cout, k]
            go = torch.randn(1, cout, n, generator=g)
            w_exp = w if k == (1, 1, 1) else oracle.restrict_kernel_forward(w, apr.level_max() - apr.level_min() + 1)
            gx, gw = oracle.conv_backward([apr], x, w_exp, go, ld)
            out[f"{tag}/conv{ks}/w"] = w.numpy()
            out[f"{tag}/conv{ks}/w_expanded"] = w_exp.numpy()
            out[f"{tag}/conv{ks}/y"] = oracle.conv_forward([apr], x, w_exp, ld).numpy()
            out[f"{tag}/conv{ks}/grad_y"] = go.numpy()
            out[f"{tag}/conv{ks}/grad_x"] = gx.numpy()
            out[f"{tag}/conv{ks}/grad_w_expanded"] = gw.numpy()
        pooled, idx = oracle.maxpool_forward([apr], x, ld)
        out[f"{tag}/maxpool/y"], out[f"{tag}/maxpool/argmax"] = pooled.numpy(), idx.numpy()
        gp = torch.randn(pooled.shape, generator=g)
        out[f"{tag}/maxpool/grad_y"] = gp.numpy()
        out[f"{tag}/maxpool/grad_x"] = oracle.maxpool_backward([apr], gp, idx, ld).numpy()
        ld1 = ld + 1
        out[f"{tag}/upsample/y"] = oracle.upsample_const_forward([apr], pooled, ld1).numpy()
        out[f"{tag}/upsample/grad_x"] = oracle.upsample_const_backward([apr], x, ld1).numpy()
        if tag != "3d":          # the dense image of the largest case would be most of the file
            img = oracle.reconstruct_forward([apr], x, ld)
            out[f"{tag}/reconstruct/y"] = img.numpy()
            out[f"{tag}/sample_particles/y"] = oracle.sample_particles_forward([apr], img, ld).numpy()
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "operators_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
