"""Image -> APR.  Same entry point as the reference (pyapr/converter/converter_methods.py:11-72),
own particle-selection pipeline (LibAPR's converter is not part of the reference tree)."""
import numpy as np

from . import _native
from .data_containers import APR, APRParameters


def get_apr(image, converter=None, params=None, verbose=False):
    """Convert a uint16 image of 1-3 dimensions (shape (z, x, y), C-contiguous) to an APR.

    Returns ``(apr, parts)``; ``parts`` are float32 cell means of the image over each particle
    (the reference samples particles the same way, converter_methods.py:64-65)."""
    image = np.asarray(image)
    while image.ndim < 3:
        image = image[None]
    if image.dtype != np.uint16:
        raise TypeError(f"get_apr accepts uint16 images, but {image.dtype} was given")
    image = np.ascontiguousarray(image)
    params = params or APRParameters()
    lib = _native.core()
    z, x, y = image.shape
    h = lib.aprcore_create(z, x, y)
    if not h:
        raise ValueError(lib.aprcore_last_error().decode())
    try:
        lmax = lib.aprcore_level_max(h)
        dims = np.zeros(3, np.int32)
        lib.aprcore_level_dims(h, lmax - 1, dims.ctypes.data)
        field = np.zeros(tuple(int(v) for v in dims), np.uint8)
        lib.aprcore_level_field_u16(h, image.ctypes.data, float(params.rel_error), float(params.gradient_smoothing),
                                    float(params.Ip_th), float(params.sigma_th), float(params.grad_th),
                                    field.ctypes.data)
        lib.aprcore_build_from_levels(h, field.ctypes.data)
        apr = APR._from_handle(h, (z, x, y))
        apr._params = params
        parts = np.zeros(apr.total_number_particles(), np.float32)
        lib.aprcore_sample_mean_u16(h, image.ctypes.data, parts.ctypes.data)
    finally:
        lib.aprcore_destroy(h)
    if verbose:
        print("Total number of particles: {}".format(apr.total_number_particles()))
        print("Computational Ratio: {}".format(apr.computational_ratio()))
    return apr, parts
