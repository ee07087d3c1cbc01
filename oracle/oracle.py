"""TEST INFRASTRUCTURE — NOT PART OF THE PRODUCT.

Python face of ``liboracle.so`` (oracle/aprnet_oracle.cpp), the CPU restatement of the reference's
operators.  Signatures follow the reference's native functions (`_pyaprwrapper.aprnet.{conv,pool,
upsample,utils}`, wrappers/pythonBind.cpp:144-158): batched CPU tensors, a list of APRs and an int32
``level_deltas`` tensor; outputs are allocated here like the reference's wrappers do.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile liboracle.so with the flags of the reference's CPU build (CMakeLists.txt:70-71,144)."""
    so = os.path.join(_HERE, "liboracle.so")
    src = os.path.join(_HERE, "aprnet_oracle.cpp")
    if force or not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.check_call(["g++", "-O3", "-march=x86-64-v3", "-fopenmp", "-shared", "-fPIC", "-std=c++17",
                               "-o", so, src])
    return so


class _Desc(C.Structure):
    _fields_ = [("level_min", C.c_int32), ("level_max", C.c_int32),
                ("z_num", C.c_void_p), ("x_num", C.c_void_p), ("y_num", C.c_void_p),
                ("level_xz_vec", C.c_void_p), ("xz_end_vec", C.c_void_p), ("y_vec", C.c_void_p),
                ("n_rows", C.c_uint64), ("n_particles", C.c_uint64)]


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(so):
            build()
        _LIB = C.CDLL(so)
        _LIB.oracle_number_parts.restype = C.c_int64
        _LIB.oracle_tree_offset.restype = C.c_int64
    return _LIB


def set_threads(n):
    """Sets the OpenMP thread count of the oracle; returns the previous maximum."""
    return int(lib().oracle_set_threads(int(n)))


def _desc(it):
    d = _Desc()
    d.level_min, d.level_max = it.level_min(), it.level_max()
    d.z_num, d.x_num, d.y_num = it._z.ctypes.data, it._x.ctypes.data, it._y.ctypes.data
    d.level_xz_vec, d.xz_end_vec = it.level_xz_vec.ctypes.data, it.xz_end_vec.ctypes.data
    d.y_vec = it.y_vec.ctypes.data if it.y_vec.shape[0] else None
    d.n_rows, d.n_particles = it.xz_end_vec.shape[0], it.y_vec.shape[0]
    return d


def _descs(apr):
    a, t = _desc(apr.iterator()), _desc(apr.tree_iterator())
    return C.byref(a), C.byref(t), (a, t)


def _sfx(t):
    if t.dtype == torch.float32:
        return "f32"
    if t.dtype == torch.float64:
        return "f64"
    raise TypeError("oracle supports float32 / float64 only (AT_DISPATCH_FLOATING_TYPES, conv.hpp:70)")


def _p(t):
    return C.c_void_p(t.data_ptr())


def _i64(v):
    return C.c_int64(int(v))


# ------------------------------------------------------------------------------------ index helpers
def number_parts(apr, level_delta):
    a, t, _k = _descs(apr)
    return int(lib().oracle_number_parts(a, t, int(level_delta)))


def tree_offset(apr, level):
    a, t, _k = _descs(apr)
    return int(lib().oracle_tree_offset(a, t, int(level)))


def tree_parts(apr, level_delta):
    """tree_it.total_number_particles(Lc-1) (helpers.hpp:166): tree nodes of levels < Lc."""
    lc = apr.level_max() - level_delta
    return apr.tree_iterator().particles_level_end(lc - 1) if lc >= 1 else 0


def parent_index(apr, which, level):
    """Parent tree index of every particle (which=0) / tree node (which=1) of ``level`` (merge walk)."""
    it = apr.tree_iterator() if which else apr.iterator()
    out = np.full(it.total_number_particles(), -1, np.int64)
    a, t, _k = _descs(apr)
    lib().oracle_parent_index(a, t, int(which), int(level), C.c_void_p(out.ctypes.data))
    return out


# ------------------------------------------------------------------------------------ tree fill
def fill_tree_mean(apr, x, level_delta):
    x = x.contiguous()
    td = torch.zeros(max(tree_parts(apr, level_delta), 1), dtype=x.dtype)
    a, t, _k = _descs(apr)
    getattr(lib(), "oracle_fill_tree_mean_" + _sfx(x))(a, t, _p(x), _p(td), int(level_delta))
    return td[:tree_parts(apr, level_delta)]


def fill_tree_mean_backward(apr, grad_tree, n_in, level_delta):
    gt = grad_tree.clone().contiguous()
    gin = torch.zeros(n_in, dtype=gt.dtype)
    a, t, _k = _descs(apr)
    getattr(lib(), "oracle_fill_tree_mean_bwd_" + _sfx(gt))(a, t, _p(gin), _p(gt), int(level_delta))
    return gin


# ------------------------------------------------------------------------------------ convolution
def conv_forward(aprs, x, weights, level_deltas):
    """convolve{111,133,155,333,555}_forward; weights [Cin, S_exp, Cout, kz, kx, ky]."""
    if x.size(1) != weights.size(0):
        raise ValueError("convolve: input tensor shape does not match weights tensor!")
    x, weights = x.contiguous(), weights.contiguous()
    kz, kx, ky = weights.shape[3:]
    out = torch.zeros(x.size(0), weights.size(2), x.size(2), dtype=x.dtype)
    fn = getattr(lib(), "oracle_conv_fwd_" + _sfx(x))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        rc = fn(a, t, kz, kx, ky, _p(x[b]), _i64(x.size(2)), x.size(1), _p(weights), weights.size(1), weights.size(2),
                _p(out[b]), _i64(out.size(2)), int(level_deltas[b]))
        if rc != 0:
            raise ValueError(f"unsupported stencil {(kz, kx, ky)}")
    return out


def conv_backward(aprs, x, weights, grad_output, level_deltas):
    x, weights, grad_output = x.contiguous(), weights.contiguous(), grad_output.contiguous()
    kz, kx, ky = weights.shape[3:]
    gx, gw = torch.zeros_like(x), torch.zeros_like(weights)
    fn = getattr(lib(), "oracle_conv_bwd_" + _sfx(x))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, kz, kx, ky, _p(x[b]), _i64(x.size(2)), x.size(1), _p(weights), weights.size(1), weights.size(2),
           _p(grad_output[b]), _i64(grad_output.size(2)), _p(gx[b]), _i64(gx.size(2)), _p(gw), int(level_deltas[b]))
    return gx, gw


def restrict_kernel_forward(weights, num_levels):
    weights = weights.contiguous()
    cin, s, cout, kz, kx, ky = weights.shape
    if num_levels < s:
        # kernel.hpp:70-74 copies all given stencils into an output of num_levels entries: out of bounds in the
        # reference when there are fewer levels than stencils.  Refused here (the product refuses it too).
        raise ValueError("restrict_kernel_forward: fewer levels than stencils")
    out = torch.zeros(cin, num_levels, cout, kz, kx, ky, dtype=weights.dtype)
    getattr(lib(), "oracle_restrict_fwd_" + _sfx(weights))(_p(weights), _p(out), cin, s, num_levels, cout, kz, kx, ky)
    return out


def restrict_kernel_backward(grad_weights, num_stencils):
    grad_weights = grad_weights.contiguous()
    cin, se, cout, kz, kx, ky = grad_weights.shape
    if se < num_stencils:
        raise ValueError("restrict_kernel_backward: fewer levels than stencils")
    out = torch.zeros(cin, num_stencils, cout, kz, kx, ky, dtype=grad_weights.dtype)
    getattr(lib(), "oracle_restrict_bwd_" + _sfx(grad_weights))(_p(grad_weights), _p(out), cin, num_stencils, se, cout,
                                                                kz, kx, ky)
    return out


# ------------------------------------------------------------------------------------ pool / upsample
def maxpool_forward(aprs, x, level_deltas):
    x = x.contiguous()
    n_out = max(number_parts(a, int(level_deltas[i]) + 1) for i, a in enumerate(aprs))
    out = -1e17 * torch.ones(x.size(0), x.size(1), n_out, dtype=x.dtype)      # maxpool.hpp:51
    idx = torch.zeros(out.shape, dtype=torch.int64)
    fn = getattr(lib(), "oracle_maxpool_fwd_" + _sfx(x))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(x[b]), _i64(x.size(2)), x.size(1), _p(out[b]), _i64(n_out), _p(idx[b]), _i64(n_out),
           int(level_deltas[b]))
    return out, idx


def maxpool_backward(aprs, grad_output, max_indices, level_deltas):
    grad_output, max_indices = grad_output.contiguous(), max_indices.contiguous()
    n_in = max(number_parts(a, int(level_deltas[i])) for i, a in enumerate(aprs))
    gin = torch.zeros(grad_output.size(0), grad_output.size(1), n_in, dtype=grad_output.dtype)
    fn = getattr(lib(), "oracle_maxpool_bwd_" + _sfx(grad_output))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(grad_output[b]), _i64(grad_output.size(2)), grad_output.size(1), _p(gin[b]), _i64(n_in),
           _p(max_indices[b]), _i64(max_indices.size(2)), int(level_deltas[b]))
    return gin


def upsample_const_forward(aprs, x, level_deltas):
    if min(int(v) for v in level_deltas) <= 0:
        raise ValueError("UpSampleConst is only implemented for downsampled particles")     # upsample.hpp:49-54
    x = x.contiguous()
    n_out = max(number_parts(a, int(level_deltas[i]) - 1) for i, a in enumerate(aprs))
    out = torch.zeros(x.size(0), x.size(1), n_out, dtype=x.dtype)
    fn = getattr(lib(), "oracle_upsample_fwd_" + _sfx(x))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(x[b]), _i64(x.size(2)), x.size(1), _p(out[b]), _i64(n_out), int(level_deltas[b]))
    return out


def upsample_const_backward(aprs, grad_output, level_deltas):
    grad_output = grad_output.contiguous()
    n_in = max(number_parts(a, int(level_deltas[i])) for i, a in enumerate(aprs))
    gin = torch.zeros(grad_output.size(0), grad_output.size(1), n_in, dtype=grad_output.dtype)
    fn = getattr(lib(), "oracle_upsample_bwd_" + _sfx(grad_output))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(grad_output[b]), _i64(grad_output.size(2)), grad_output.size(1), _p(gin[b]), _i64(n_in),
           int(level_deltas[b]))
    return gin


# ------------------------------------------------------------------------------------ pixels <-> particles
def _dense_shape(aprs, level_deltas):
    z = x = y = 0
    for i, a in enumerate(aprs):
        lc = a.level_max() - int(level_deltas[i])
        z, x, y = max(z, a.z_num(lc)), max(x, a.x_num(lc)), max(y, a.y_num(lc))
    return z, x, y


def reconstruct_forward(aprs, x, level_deltas):
    assert len(aprs) == 1 or len({a.shape() for a in aprs}) == 1, "oracle: same-shaped APRs only"
    x = x.contiguous()
    z, xx, y = _dense_shape(aprs, level_deltas)
    out = torch.zeros(x.size(0), x.size(1), z, xx, y, dtype=x.dtype)
    fn = getattr(lib(), "oracle_reconstruct_fwd_" + _sfx(x))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(x[b]), _i64(x.size(2)), x.size(1), _p(out[b]), _i64(z * xx * y), int(level_deltas[b]))
    return out


def reconstruct_backward(aprs, grad_output, level_deltas):
    grad_output = grad_output.contiguous()
    n = max(number_parts(a, int(level_deltas[i])) for i, a in enumerate(aprs))
    gin = torch.zeros(grad_output.size(0), grad_output.size(1), n, dtype=grad_output.dtype)
    fn = getattr(lib(), "oracle_reconstruct_bwd_" + _sfx(grad_output))
    plane = grad_output[0, 0].numel()
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(gin[b]), _i64(n), gin.size(1), _p(grad_output[b]), _i64(plane), int(level_deltas[b]))
    return gin


def sample_particles_forward(aprs, img, level_deltas):
    img = img.contiguous()
    n = max(number_parts(a, int(level_deltas[i])) for i, a in enumerate(aprs))
    out = torch.zeros(img.size(0), img.size(1), n, dtype=img.dtype)
    fn = getattr(lib(), "oracle_sample_fwd_" + _sfx(img))
    plane = img[0, 0].numel()
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(out[b]), _i64(n), out.size(1), _p(img[b]), _i64(plane), int(level_deltas[b]))
    return out


def sample_particles_backward(aprs, grad_output, level_deltas):
    grad_output = grad_output.contiguous()
    z, xx, y = _dense_shape(aprs, level_deltas)
    gimg = torch.zeros(grad_output.size(0), grad_output.size(1), z, xx, y, dtype=grad_output.dtype)
    fn = getattr(lib(), "oracle_sample_bwd_" + _sfx(grad_output))
    for b, apr in enumerate(aprs):
        a, t, _k = _descs(apr)
        fn(a, t, _p(grad_output[b]), _i64(grad_output.size(2)), grad_output.size(1), _p(gimg[b]), _i64(z * xx * y),
           int(level_deltas[b]))
    return gimg


# ------------------------------------------------------------------------------------ StarDist utilities
_LABEL_SFX = {torch.uint8: "u8", torch.uint16: "u16", torch.uint32: "u32", torch.uint64: "u64"}


def particle_coords(apr, level_delta):
    """get_particle_coords (utils.hpp:222-267) -> [N_d, 3] float32 (z, x, y)."""
    a, t, _k = _descs(apr)
    out = torch.zeros(number_parts(apr, level_delta), 3, dtype=torch.float32)
    lib().oracle_particle_coords(a, t, int(level_delta), _p(out))
    return out


def sample_image_max(apr, img, level_delta):
    """sample_image (utils.hpp:270-333): maximum of the image over every particle's cell -> [N_d] float32."""
    img = img.contiguous().float()
    a, t, _k = _descs(apr)
    out = torch.zeros(number_parts(apr, level_delta), dtype=torch.float32)
    z, x, y = img.shape
    lib().oracle_sample_image_max(a, t, int(level_delta), _p(img), int(z), int(x), int(y), _p(out))
    return out


def labels_to_dist(apr, labels, dzs, dxs, dys, level_delta, max_steps=1 << 20):
    """labels_to_dist_cpp (utils.hpp:86-219) -> [N_d, n_rays] float32."""
    labels = labels.contiguous()
    dzs, dxs, dys = (v.contiguous().float() for v in (dzs, dxs, dys))
    a, t, _k = _descs(apr)
    out = torch.zeros(number_parts(apr, level_delta), dzs.numel(), dtype=torch.float32)
    z, x, y = labels.shape
    getattr(lib(), "oracle_labels_to_dist_" + _LABEL_SFX[labels.dtype])(
        a, t, int(level_delta), _p(labels), int(z), int(x), int(y), _p(dzs), _p(dxs), _p(dys), int(dzs.numel()), int(max_steps),
        _p(out))
    return out
