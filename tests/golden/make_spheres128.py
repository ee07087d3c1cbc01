#!/usr/bin/env python3
"""Writes tests/golden/spheres128_conv_1to16.json: the cross-machine check of BASELINE configs[0].

The configuration (APR of the seeded 128^3 sphere volume, APRConv 3x3x3 1 -> 16 with bias, weights N(0, 0.1) seed 0,
input = the sampled particle intensities / 1000) is run through the CPU oracle; per output channel the file keeps the
float64 sum, the maximum magnitude and the first and last 64 values.  The reference holds no vectors for this path
(its fixtures are absent), so these are this repository's own oracle answers, frozen after the oracle was pinned by
the dense level-view identities of tests/test_oracle_dense.py.

  python tests/golden/make_spheres128.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "apr-cnn_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def oracle_output():
    import torch
    from bench import spheres128_inputs, level_counts
    from oracle import oracle
    apr, x, w, b = spheres128_inputs()
    levels = apr.level_max() - apr.level_min() + 1
    w_cpu = w.permute(2, 0, 1, 3, 4, 5).contiguous()                  # CPU layout [Cin, S, Cout, kz, kx, ky]
    y = oracle.conv_forward([apr], x, oracle.restrict_kernel_forward(w_cpu, levels), torch.zeros(1, dtype=torch.int32))
    return apr, (y + b.view(1, -1, 1))[0], level_counts(apr)


def summary(apr, y, levels):
    yd = y.double()
    return {"config": "BASELINE configs[0]: 128^3, 200 Gaussian spheres, APRConv 3x3x3 1->16 fp32 with bias, weights N(0,0.1) seed 0",
            "n_particles": apr.total_number_particles(), "levels": levels,
            "sum": [float(v) for v in yd.sum(dim=1)], "abs_max": [float(v) for v in yd.abs().max(dim=1).values],
            "first64": [[float(v) for v in row[:64]] for row in y], "last64": [[float(v) for v in row[-64:]] for row in y]}


if __name__ == "__main__":
    out = summary(*oracle_output())
    with open(os.path.join(HERE, "spheres128_conv_1to16.json"), "w") as f:
        json.dump(out, f)
    print("wrote", out["n_particles"], "particles")
