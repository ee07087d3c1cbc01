"""Label utilities of the StarDist networks with the names and argument meaning of
pyapr/aprnet/stardist_utils.py:7-33 (``labels_to_dist``, ``get_prob_apr``, ``get_particle_coordinates``), computed by
device kernels instead of the reference's CPU loops (pyapr/aprnet/src/utils.hpp:86-333).

Inputs may be numpy arrays (results come back as numpy arrays, as in the reference) or GPU tensors (results stay
on the device).  There is no CPU path behind these functions."""
import ctypes as C

import numpy as np
import torch

from . import _ops

_LABEL_SFX = {torch.uint8: "u8", torch.uint16: "u16", torch.uint32: "u32", torch.uint64: "u64"}
MAX_RAY_STEPS = 1 << 20       # bound on the walk along one ray (the reference has none: a zero step never ends there)


def _device():
    if not torch.cuda.is_available():
        raise RuntimeError("pyapr.aprnet.stardist_utils needs a GPU: the operators have no CPU path")
    return torch.device("cuda", torch.cuda.current_device())


def _to_device(a, dtype=None):
    """-> (GPU tensor, came_from_numpy)"""
    if isinstance(a, torch.Tensor):
        if not a.is_cuda:
            raise RuntimeError("tensor arguments must live on the GPU")
        return (a if dtype is None else a.to(dtype)).contiguous(), False
    t = torch.from_numpy(np.ascontiguousarray(a))
    return (t if dtype is None else t.to(dtype)).to(_device()), True


def _image3(img, apr, what):
    if img.dim() < 3:
        img = img.reshape((1,) * (3 - img.dim()) + tuple(img.shape))
    if tuple(img.shape) != tuple(apr.shape()):
        raise ValueError(f"{what}: the image must have the shape of the APR, {tuple(apr.shape())}")     # stardist_utils.py:12
    return img


def get_particle_coordinates(apr, level_delta=0, device=None):
    """[N, 3] float32 (z, x, y) centres of the particles at ``level_delta`` in pixels (stardist_utils.py:29-33).
    Returns a numpy array, or a GPU tensor when ``device`` is given."""
    dev = torch.device(device) if device is not None else _device()
    n = _ops.number_particles(apr, level_delta)
    out = torch.zeros((n, 3), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _ops._lib().aprnet_particle_coords(apr.plan(dev.index or 0), int(level_delta), _ops._ptr(out), _ops._stream())
    if rc:
        _ops._raise(rc, "get_particle_coordinates failed")
    return out if device is not None else out.cpu().numpy()


def sample_image(apr, img, level_delta=0):
    """sample_image of the reference (utils.hpp:270-333): every particle takes the maximum of ``img`` over its cell.
    -> [N] float32."""
    t, from_numpy = _to_device(img, torch.float32)
    t = _image3(t, apr, "sample_image")
    n = _ops.number_particles(apr, level_delta)
    out = torch.zeros(n, dtype=torch.float32, device=t.device)
    z, x, y = t.shape
    with torch.cuda.device(t.device):
        rc = _ops._lib().aprnet_sample_image_max_f32(apr.plan(t.device.index or 0), int(level_delta), _ops._ptr(t), z, x, y,
                                                    _ops._ptr(out), _ops._stream())
    if rc:
        _ops._raise(rc, "sample_image failed")
    return out.cpu().numpy() if from_numpy else out


def get_prob_apr(apr, img, level_delta=0, prob_fn=None):
    """Object probabilities of a label image sampled onto the particles (stardist_utils.py:22-26).  ``prob_fn`` maps
    the label image to per-pixel probabilities; by default ``stardist.utils.edt_prob`` as in the reference."""
    if prob_fn is None:
        try:
            from stardist.utils import edt_prob as prob_fn
        except ImportError as e:
            raise ImportError("get_prob_apr needs stardist.utils.edt_prob (or pass prob_fn)") from e
    return sample_image(apr, np.asarray(prob_fn(img), dtype=np.float32), level_delta)


def labels_to_dist(apr, img, rays, step_factor=(1, 1, 1), level_delta=0):
    """Star-convex distances (stardist_utils.py:7-19): for every particle inside an object and every ray, the length of
    the ray up to the border of the object.  ``rays``: an object with ``.vertices`` [n_rays, 3] (columns dz, dx, dy,
    as the reference unpacks them) or such an array.  -> [N, n_rays] float32; rows of particles outside objects are 0."""
    verts = np.asarray(getattr(rays, "vertices", rays), dtype=np.float32)
    if verts.ndim != 2 or verts.shape[1] != 3:
        raise ValueError("labels_to_dist: rays must be [n_rays, 3]")
    steps = verts / np.asarray(step_factor, dtype=np.float32)[None, :]
    if not np.all(np.any(steps != 0, axis=1)):
        raise ValueError("labels_to_dist: a ray with a zero step never leaves its object")
    t, from_numpy = _to_device(img)
    if t.dtype not in _LABEL_SFX:
        raise TypeError("labels_to_dist: label images must be uint8, uint16, uint32 or uint64")      # stardist_utils.py:13
    t = _image3(t, apr, "labels_to_dist")
    dz, dx, dy = (torch.from_numpy(np.ascontiguousarray(steps[:, k])).to(t.device) for k in range(3))
    n = _ops.number_particles(apr, level_delta)
    out = torch.zeros((n, verts.shape[0]), dtype=torch.float32, device=t.device)
    z, x, y = t.shape
    fn = getattr(_ops._lib(), "aprnet_labels_to_dist_" + _LABEL_SFX[t.dtype])
    with torch.cuda.device(t.device):
        rc = fn(apr.plan(t.device.index or 0), int(level_delta), _ops._ptr(t), z, x, y, _ops._ptr(dz), _ops._ptr(dx), _ops._ptr(dy),
                verts.shape[0], MAX_RAY_STEPS, _ops._ptr(out), _ops._stream())
    if rc:
        _ops._raise(rc, "labels_to_dist failed")
    return out.cpu().numpy() if from_numpy else out
