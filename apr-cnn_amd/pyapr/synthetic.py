"""Seeded synthetic volumes and APRs for the benchmark configurations (no datasets are used)."""
import numpy as np

from . import _native
from .data_containers import APR, APRParameters
from .converter import get_apr

GAUSSIAN, ELLIPSOID = 0, 1


def synth_volume(shape, seed, kind, n_blobs, axes, amp, background=(100.0, 100.0), isotropic=False, poisson=True):
    """uint16 volume (z, x, y): ``n_blobs`` blobs with semi-axes U[axes] px and amplitude U[amp] on a
    background, plus Poisson noise.  A pure function of its arguments (counter-based RNG)."""
    z, x, y = (int(v) for v in shape)
    img = np.empty((z, x, y), np.uint16)
    _native.core().aprcore_synth_volume_u16(img.ctypes.data, z, x, y, int(seed), int(kind), int(n_blobs),
                                            float(axes[0]), float(axes[1]), int(isotropic), float(amp[0]),
                                            float(amp[1]), float(background[0]), float(background[1]), int(poisson))
    return img


def pipeline_parameters(rel_error=0.1):
    p = APRParameters()
    p.rel_error, p.gradient_smoothing, p.Ip_th, p.sigma_th, p.grad_th = rel_error, 2.0, 110.0, 20.0, 10.0
    return p


# name -> (shape (z,x,y), kind, n_blobs, axes, amplitude, background, isotropic, rel_error)
CONFIGS = {
    # 128^3, 200 Gaussian spheres radius U[3,8] (sigma = radius / 2), peak 1000
    "spheres128": ((128, 128, 128), GAUSSIAN, 200, (1.5, 4.0), (1000.0, 1000.0), (100.0, 100.0), True, 0.1),
    # 512 x 512 x 256, 2000 ellipsoidal blobs, semi-axes U[4,16], intensity U[400,3000]
    "blobs512": ((256, 512, 512), ELLIPSOID, 2000, (4.0, 16.0), (400.0, 3000.0), (100.0, 100.0), False, 0.1),
    # 2048 x 2048 x 512, 50k nucleus-like ellipsoids U[3,10], sinusoidal background 100-300
    "nuclei2048": ((512, 2048, 2048), ELLIPSOID, 50000, (3.0, 10.0), (500.0, 2000.0), (100.0, 300.0), False, 0.1),
    # 1024^3, 200k ellipsoids U[3,12], intensity U[300,4000]
    "nuclei1024": ((1024, 1024, 1024), ELLIPSOID, 200000, (3.0, 12.0), (300.0, 4000.0), (100.0, 100.0), False, 0.1),
    # 16384^2 2-D, 1M Gaussian spots sigma U[1.5,6], peak U[500,5000], rel_error 0.05
    "spots16k": ((1, 16384, 16384), GAUSSIAN, 1000000, (1.5, 6.0), (500.0, 5000.0), (100.0, 100.0), True, 0.05),
}


def make_config(name, seed=0, scale=1.0):
    """Returns (apr, parts) for a named configuration.  ``scale`` < 1 shrinks every dimension and the
    blob count proportionally to the volume (for parity tests at reduced size)."""
    shape, kind, n, axes, amp, bg, iso, rel = CONFIGS[name]
    if scale != 1.0:
        shape = tuple(max(1, int(round(s * scale))) if s > 1 else 1 for s in shape)
        ndim = sum(1 for s in CONFIGS[name][0] if s > 1)
        n = max(1, int(round(n * scale ** ndim)))
    img = synth_volume(shape, seed, kind, n, axes, amp, bg, iso)
    return get_apr(img, params=pipeline_parameters(rel))
