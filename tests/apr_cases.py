"""Seeded random valid APRs for the parity tests: odd sizes, 1-D / 2-D / 3-D, several levels.

The reference's own fixtures (sphere_{1,2,3}D.apr, two_objects.apr; pyapr/tests/test_io.py:5-9 gives
their odd shapes (1,1,63), (1,63,63), (65,61,63)) are git-ignored upstream and absent, so the
tests draw APRs with the same flavour of shapes from random required-level fields."""
import numpy as np

from pyapr import APR


def random_apr(shape, seed, density=0.06, max_drop=2):
    """Random required-level field: a fraction `density` of the half-resolution cells ask for a level in
    [level_max - max_drop, level_max]; the builder balances the rest."""
    rng = np.random.default_rng(seed)
    z, x, y = shape
    m, lmax = max(shape), 0
    while (1 << lmax) < m:
        lmax += 1
    lmax = max(lmax, 1)
    dims = tuple((s + 1) // 2 for s in shape)
    field = np.zeros(dims, np.uint8)
    mask = rng.random(dims) < density
    lo = max(lmax - max_drop, 1)
    field[mask] = rng.integers(lo, lmax + 1, size=int(mask.sum()), dtype=np.uint8)
    return APR.from_level_field(shape, field)


# name -> (shape (z, x, y), seed, density)
TINY = {
    "3d_a": ((13, 11, 9), 1, 0.08),
    "3d_b": ((9, 17, 12), 2, 0.05),
    "3d_c": ((16, 16, 16), 3, 0.03),
    "2d_a": ((1, 21, 19), 4, 0.08),
    "2d_b": ((1, 32, 17), 5, 0.04),
    "1d_a": ((1, 1, 63), 6, 0.10),
}

SMALL = {
    "3d_s": ((33, 29, 37), 11, 0.02),
    "3d_t": ((65, 61, 63), 12, 0.004),
    "2d_s": ((1, 63, 63), 13, 0.03),
    "2d_t": ((1, 130, 257), 14, 0.01),
    "1d_s": ((1, 1, 300), 15, 0.05),
}


def get(name):
    shape, seed, dens = (TINY.get(name) or SMALL[name])
    return random_apr(shape, seed, dens)
