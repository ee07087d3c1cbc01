"""Native operator calls: the functions APR-CNN binds on ``_pyaprwrapper.aprnet.{conv,pool,upsample,
utils,cuda}`` (wrappers/pythonBind.cpp:144-182), here implemented on top of the C ABI of
``libaprnet_hip.so``.  Same names, argument order, output allocation and exception types as the
reference's wrappers; every tensor must live on the GPU ("cuda" device of PyTorch-ROCm) — there is no
CPU path behind these functions.

Weight layouts: the ``cuda`` flavour uses [S, Cout, Cin, kz, kx, ky] (cuda/conv.py:77) and is what the
kernels consume; the CPU-flavour names (``convolve333_forward`` ...) take [Cin, S, Cout, kz, kx, ky]
(conv.py:164) and are permuted on the way in and out.
"""
import ctypes as C

import torch

from .. import _native


def _lib():
    return _native.hip()


class UnsupportedError(RuntimeError):
    """APRNET_ERR_UNSUPPORTED: the call is valid but this build has no kernel for it (a size or channel limit, window
    lists that could not be built).  A RuntimeError, as the reference's TORCH_CHECK failures are."""


def _raise(rc, what):
    msg = _lib().aprnet_last_error().decode()
    if rc == -1:
        raise ValueError(msg or what)            # std::invalid_argument -> ValueError (pybind11)
    if rc == -4:
        raise UnsupportedError(msg or what)
    raise RuntimeError(msg or what)              # TORCH_CHECK -> RuntimeError


def _sfx(t, bf16=False):
    """Entry-point suffix of a tensor's element type.  bfloat16 is a storage type of the features for the
    operators that pass bf16=True (forward operators of the network, backward of pool / upsample)."""
    if t.dtype == torch.float32:
        return "f32"
    if t.dtype == torch.float64:
        return "f64"
    if t.dtype == torch.bfloat16 and bf16:
        return "bf16"
    raise TypeError(f"this aprnet operator does not support {t.dtype} tensors")


def _check_input(t, name):
    # CHECK_INPUT (cuda/src/common.hpp:14-16)
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _deltas(level_deltas, n):
    d = [int(v) for v in level_deltas.tolist()]
    if len(d) < n:
        raise ValueError("level_deltas must hold one entry per APR")
    return d


def _plans(aprs, device):
    return [a.plan(device.index if device.index is not None else torch.cuda.current_device()) for a in aprs]


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr())


def _zero_tails(out, sizes):
    """Batch items shorter than the padded length keep zeros behind their last particle, as the
    reference's zero-initialised outputs do (conv.hpp:68)."""
    n = out.shape[-1]
    for b, nb in enumerate(sizes):
        if nb < n:
            out[b, ..., nb:] = 0


# ---------------------------------------------------------------------------------------- utils
def number_particles(apr, level_delta):
    """helpers::number_parts (helpers.hpp:86-101); pure host arithmetic on the row tables."""
    it, tr = apr.iterator(), apr.tree_iterator()
    lc = apr.level_max() - int(level_delta)
    n = it.particles_level_end(lc)
    if tr.level_min() <= lc <= tr.level_max():
        n += tr.particles_level_end(lc) - tr.particles_level_begin(lc)
    return n


number_parts = number_particles


def number_particles_after_pooling(apr, level_delta):
    return number_particles(apr, int(level_delta) + 1)


def number_particles_after_upsampling(apr, level_delta):
    return number_particles(apr, int(level_delta) - 1)


def tree_parts(apr, level_delta):
    lc = apr.level_max() - int(level_delta)
    return apr.tree_iterator().particles_level_end(lc - 1) if lc >= 1 else 0


# ---------------------------------------------------------------------------------------- restrict kernel
def _restrict(weights, n_other, backward):
    _check_input(weights, "weights")
    s_in, cout, cin, kz, kx, ky = weights.shape
    out = torch.empty((n_other, cout, cin, kz, kx, ky), dtype=weights.dtype, device=weights.device)
    fn = getattr(_lib(), f"aprnet_restrict_kernel_{'bwd' if backward else 'fwd'}_{_sfx(weights)}")
    with torch.cuda.device(weights.device):
        rc = fn(_ptr(weights), s_in, cout * cin, kz, kx, ky, n_other, _ptr(out), _stream())
    if rc:
        _raise(rc, "restrict_kernel failed")
    return out


def restrict_kernel_forward(weights, num_levels):
    """[S, Cout, Cin, k] -> [num_levels, Cout, Cin, k] (restrict_kernel333_forward, restrict_gpu.cu:175-203)."""
    return _restrict(weights, int(num_levels), False)


def restrict_kernel_backward(grad_weights, num_stencils):
    return _restrict(grad_weights, int(num_stencils), True)


# ---------------------------------------------------------------------------------------- convolution
class _Fusion(C.Structure):
    """aprnet_conv_fusion of the C ABI."""
    _fields_ = [("x2", C.c_void_p), ("ldx2", C.c_int64), ("C2", C.c_int32), ("relu", C.c_int32),
                ("x2_coarse", C.c_void_p), ("ld_coarse", C.c_int64)]


def conv_forward(aprs, x, weights, level_delta, bias=None, relu=False, x2=None):
    """conv333_forward / conv111_forward (wrap_conv_gpu.hpp:32-66, 170-193) for any supported stencil.
    weights: [S_exp, Cout, Cin, kz, kx, ky] (for 1x1x1: [S, Cout, Cin, 1, 1, 1], not expanded).
    bias ([Cout], optional) is added inside the kernel instead of in a separate pass over the output.
    relu: the result is clamped at zero in the kernel (the ReLU of BasicBlock, unet_parts.py:17-26).
    x2 ([B, C2, N], optional): the kernel reads its channels after those of x, which stands for
    conv(torch.cat([x, x2], dim=1)) (unet_parts.py:82) without writing the concatenated tensor."""
    _check_input(x, "input")
    _check_input(weights, "weights")
    c2 = 0
    if x2 is not None:
        _check_input(x2, "second input")
        if x2.dtype != x.dtype or x2.size(0) != x.size(0) or x2.size(2) != x.size(2):
            raise ValueError("the second input must match the first in dtype, batch size and particle count")
        c2 = x2.size(1)
    if x.dtype == torch.bfloat16:
        # bfloat16 is the storage type of the features only: weights and bias are used in fp32
        weights = weights.float()
        bias = None if bias is None else bias.float()
    elif weights.dtype != x.dtype:
        raise ValueError("weights must have the dtype of the input")
    if bias is not None:
        _check_input(bias, "bias")
        if bias.dtype != weights.dtype or bias.numel() != weights.size(1):
            raise ValueError("bias must hold one value per output channel, in the dtype of the weights")
    bptr = _ptr(bias) if bias is not None else None
    if x.size(1) + c2 != weights.size(2):
        raise ValueError("convolve: input tensor shape does not match weights tensor!")   # conv.hpp:63-66
    s_exp, cout, cin, kz, kx, ky = weights.shape
    c1 = cin - c2
    fused = relu or x2 is not None
    if x2 is not None and (kz, kx, ky) == (1, 1, 1):
        raise ValueError("the 1x1x1 convolution takes a single input")
    B, _, N = x.shape
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    if max(sizes) > N:
        raise ValueError("input holds fewer particles than the APR at this level delta")
    out = torch.empty((B, cout, N), dtype=x.dtype, device=x.device)
    _zero_tails(out, sizes)
    if bias is not None:
        # the reference adds the bias to the whole padded tensor (conv.py:101): tails hold 0 + bias
        for b, nb in enumerate(sizes):
            if nb < N:
                out[b, :, nb:] = (bias.clamp(min=0) if relu else bias).view(-1, 1)
    plans = _plans(aprs, x.device)
    sfx = _sfx(x, bf16=True)
    with torch.cuda.device(x.device):
        st = _stream()
        if fused:
            ld_tree = max(max(tree_parts(a, d[b]) for b, a in enumerate(aprs)), 1)
            tree_ws = torch.empty((cin, ld_tree), dtype=x.dtype, device=x.device)
            fn = getattr(_lib(), "aprnet_conv_fwd_fused_" + sfx)
            for b in range(B):
                fu = _Fusion(_ptr(x2[b]) if x2 is not None else None, N, c2, 1 if relu else 0)
                rc = fn(plans[b], d[b], kz, kx, ky, _ptr(x[b]), N, c1, _ptr(weights), s_exp, cout, bptr, _ptr(out[b]), N,
                        _ptr(tree_ws), ld_tree, C.byref(fu), st)
                if rc:
                    _raise(rc, "conv_forward failed")
        elif (kz, kx, ky) == (1, 1, 1):
            fn = getattr(_lib(), "aprnet_conv111_fwd_" + sfx)
            for b in range(B):
                rc = fn(plans[b], d[b], _ptr(x[b]), N, cin, _ptr(weights), s_exp, cout, bptr, _ptr(out[b]), N, st)
                if rc:
                    _raise(rc, "conv111_forward failed")
        else:
            ld_tree = max(max(tree_parts(a, d[b]) for b, a in enumerate(aprs)), 1)
            tree_ws = torch.empty((cin, ld_tree), dtype=x.dtype, device=x.device)
            fn = getattr(_lib(), "aprnet_conv_fwd_" + sfx)
            for b in range(B):
                rc = fn(plans[b], d[b], kz, kx, ky, _ptr(x[b]), N, cin, _ptr(weights), s_exp, cout, bptr, _ptr(out[b]), N,
                        _ptr(tree_ws), ld_tree, st)
                if rc:
                    _raise(rc, "conv_forward failed")
    return out


def channel_sum(x):
    """sum over batch and positions of a [B, C, N] tensor -> [C] (the bias gradient, conv.py:33), deterministic."""
    _check_input(x, "grad_output")
    B, C, N = x.shape
    acc = torch.float32 if x.dtype == torch.bfloat16 else x.dtype      # bfloat16 is summed in fp32
    out = torch.empty(C, dtype=acc, device=x.device)
    lib = _lib()
    work = torch.empty(lib.aprnet_channel_sum_work_elems(C), dtype=acc, device=x.device)
    fn = getattr(lib, "aprnet_channel_sum_" + _sfx(x, bf16=True))
    with torch.cuda.device(x.device):
        st = _stream()
        for b in range(B):
            rc = fn(_ptr(x[b]), N, C, N, _ptr(out), 1 if b else 0, _ptr(work), st)
            if rc:
                _raise(rc, "channel_sum failed")
    return out


# ---------------------------------------------------------------------------- normalisation over the particle axis
def _norm_sfx(x, name):
    _check_input(x, name)
    if x.dtype not in (torch.float32, torch.bfloat16) or x.dim() != 3:
        raise TypeError(f"{name}: [batch, channels, particles] float32 or bfloat16 tensor expected")
    return "f32" if x.dtype == torch.float32 else "bf16"


def _norm_work(rows, device):
    return torch.empty(_lib().aprnet_norm_work_elems(rows), dtype=torch.float32, device=device)


def _rowvec(v, rows, name):
    if v.dtype != torch.float32 or v.numel() != rows or not v.is_cuda or not v.is_contiguous():
        raise ValueError(f"{name}: contiguous float32 GPU tensor with one value per (batch item, channel) expected")
    return v


def row_moments(x):
    """[B, C, N] -> (mean, m2) float64 [B, C]: mean and sum of squared deviations of every row."""
    sfx = _norm_sfx(x, "input")
    B, Cn, N = x.shape
    mean = torch.empty(B, Cn, dtype=torch.float64, device=x.device)
    m2 = torch.empty_like(mean)
    with torch.cuda.device(x.device):
        rc = getattr(_lib(), "aprnet_row_moments_" + sfx)(_ptr(x), N, B * Cn, N, _ptr(mean), _ptr(m2),
                                                          _ptr(_norm_work(B * Cn, x.device)), _stream())
    if rc:
        _raise(rc, "row_moments failed")
    return mean, m2


def _f32_or_none(v, n, name):
    if v is None:
        return None
    v = v.detach()
    if v.dtype != torch.float32 or not v.is_contiguous():
        v = v.float().contiguous()
    if v.numel() != n or not v.is_cuda:
        raise ValueError(f"{name}: GPU tensor with {n} entries expected")
    return v


def _optr(v):
    return None if v is None else _ptr(v)


def norm_coeffs_forward(shape, groups, eps, row_mean, row_m2, given, gamma, beta, device):
    """The join of the forward pass in one launch.  shape = (B, C, N); groups = 0 for BatchNorm.  Either the row
    moments or ``given`` = (mean[C], var[C]).  -> (mean32, rstd32, scale32, shift32 [B, C]; set_mean, set_var float32,
    [C] or [B, groups], None with given statistics)."""
    B, Cn, N = shape
    out = [torch.empty(B, Cn, dtype=torch.float32, device=device) for _ in range(4)]
    gm, gv = (None, None) if given is None else (_f32_or_none(given[0], Cn, "mean"), _f32_or_none(given[1], Cn, "var"))
    sets = None
    if given is None:
        sets = [torch.empty(Cn if groups == 0 else (B, groups), dtype=torch.float32, device=device) for _ in range(2)]
    gamma, beta = _f32_or_none(gamma, Cn, "weight"), _f32_or_none(beta, Cn, "bias")
    with torch.cuda.device(device):
        rc = _lib().aprnet_norm_coeffs_fwd(B, Cn, groups, N, float(eps), _optr(row_mean), _optr(row_m2), _optr(gm), _optr(gv),
                                           _optr(gamma), _optr(beta), *[_ptr(t) for t in out],
                                           _optr(sets[0] if sets else None), _optr(sets[1] if sets else None), _stream())
    if rc:
        _raise(rc, "norm_coeffs_forward failed")
    return (*out, *(sets or (None, None)))


def norm_coeffs_backward(shape, groups, own_stats, sum_g, sum_gx, gamma, rstd32, want_gamma, want_beta):
    """The join of the backward pass in one launch -> (a, b, c [B, C] float32, grad_gamma, grad_beta [C] float32 or None)."""
    B, Cn, N = shape
    dev = sum_g.device
    a, b, c = (torch.empty(B, Cn, dtype=torch.float32, device=dev) for _ in range(3))
    gg = torch.empty(Cn, dtype=torch.float32, device=dev) if want_gamma else None
    gb = torch.empty(Cn, dtype=torch.float32, device=dev) if want_beta else None
    gamma = _f32_or_none(gamma, Cn, "weight")
    with torch.cuda.device(dev):
        rc = _lib().aprnet_norm_coeffs_bwd(B, Cn, groups, N, 1 if own_stats else 0, _ptr(sum_g), _ptr(sum_gx), _optr(gamma),
                                           _ptr(_rowvec(rstd32, B * Cn, "rstd")), _ptr(a), _ptr(b), _ptr(c), _optr(gg), _optr(gb),
                                           _stream())
    if rc:
        _raise(rc, "norm_coeffs_backward failed")
    return a, b, c, gg, gb


def norm_apply(x, mean, scale, shift, relu):
    """y = (x - mean) * scale + shift per row (float32 [B, C] coefficients), then ReLU if asked."""
    sfx = _norm_sfx(x, "input")
    B, Cn, N = x.shape
    y = torch.empty_like(x)
    with torch.cuda.device(x.device):
        rc = getattr(_lib(), "aprnet_norm_apply_" + sfx)(_ptr(x), N, B * Cn, N, _ptr(_rowvec(mean, B * Cn, "mean")),
                                                         _ptr(_rowvec(scale, B * Cn, "scale")), _ptr(_rowvec(shift, B * Cn, "shift")),
                                                         1 if relu else 0, _ptr(y), N, _stream())
    if rc:
        _raise(rc, "norm_apply failed")
    return y


def norm_backward_sums(gy, x, y, mean, rstd):
    """-> (sum g, sum g * xhat) float64 [B, C];  g = gy masked by y > 0 when the forward output y is given."""
    sfx = _norm_sfx(x, "input")
    _check_input(gy, "grad_output")
    if gy.dtype != x.dtype or gy.shape != x.shape or (y is not None and (y.dtype != x.dtype or y.shape != x.shape or not y.is_contiguous())):
        raise ValueError("norm_backward_sums: grad_output / output must match the input in type and shape")
    B, Cn, N = x.shape
    s_g = torch.empty(B, Cn, dtype=torch.float64, device=x.device)
    s_gx = torch.empty_like(s_g)
    with torch.cuda.device(x.device):
        rc = getattr(_lib(), "aprnet_norm_bwd_sums_" + sfx)(_ptr(gy), N, _ptr(x), N, None if y is None else _ptr(y), N, B * Cn, N,
                                                            _ptr(_rowvec(mean, B * Cn, "mean")), _ptr(_rowvec(rstd, B * Cn, "rstd")),
                                                            _ptr(s_g), _ptr(s_gx), _ptr(_norm_work(B * Cn, x.device)), _stream())
    if rc:
        _raise(rc, "norm_backward_sums failed")
    return s_g, s_gx


def norm_backward_apply(gy, x, y, mean, rstd, a, b, c):
    """gx = a * g + b * xhat + c per row."""
    sfx = _norm_sfx(x, "input")
    _check_input(gy, "grad_output")
    if gy.dtype != x.dtype or gy.shape != x.shape or (y is not None and (y.dtype != x.dtype or y.shape != x.shape or not y.is_contiguous())):
        raise ValueError("norm_backward_apply: grad_output / output must match the input in type and shape")
    B, Cn, N = x.shape
    gx = torch.empty_like(x)
    rows = B * Cn
    with torch.cuda.device(x.device):
        rc = getattr(_lib(), "aprnet_norm_bwd_apply_" + sfx)(_ptr(gy), N, _ptr(x), N, None if y is None else _ptr(y), N, rows, N,
                                                             _ptr(_rowvec(mean, rows, "mean")), _ptr(_rowvec(rstd, rows, "rstd")),
                                                             _ptr(_rowvec(a, rows, "a")), _ptr(_rowvec(b, rows, "b")),
                                                             _ptr(_rowvec(c, rows, "c")), _ptr(gx), N, _stream())
    if rc:
        _raise(rc, "norm_backward_apply failed")
    return gx


def conv_backward(aprs, x, weights, grad_output, level_delta, need_input_grad=True):
    """conv333_backward / conv111_backward (wrap_conv_gpu.hpp:87-133, 216-246) -> [grad_input, grad_weights].
    ``need_input_grad=False`` (stencil convolutions): the input gradient is not computed, grad_input is None."""
    _check_input(x, "input")
    _check_input(weights, "weights")
    _check_input(grad_output, "grad_output")
    s_exp, cout, cin, kz, kx, ky = weights.shape
    B, _, N = x.shape
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    skip_gx = not need_input_grad and (kz, kx, ky) != (1, 1, 1)
    gx = None if skip_gx else torch.empty_like(x)
    if gx is not None:
        _zero_tails(gx, sizes)
    gxp = (lambda b: None) if skip_gx else (lambda b: _ptr(gx[b]))
    plans = _plans(aprs, x.device)
    if x.dtype == torch.bfloat16:
        # bfloat16 features and output gradient; weights and their gradient in fp32, fp32 accumulation
        if grad_output.dtype != torch.bfloat16:
            raise TypeError("bfloat16 features need a bfloat16 output gradient")
        weights = weights.float()
        gw = torch.zeros_like(weights)
        if (kz, kx, ky) == (1, 1, 1):
            with torch.cuda.device(x.device):
                st = _stream()
                for b in range(B):
                    rc = _lib().aprnet_conv111_bwd_bf16(plans[b], d[b], _ptr(x[b]), N, cin, _ptr(weights), s_exp, cout,
                                                        _ptr(grad_output[b]), grad_output.size(2), _ptr(gx[b]), N, _ptr(gw), st)
                    if rc:
                        _raise(rc, "conv111_backward failed")
            return [gx, gw]
        ld_tree = max(max(tree_parts(a, d[b]) for b, a in enumerate(aprs)), 1)
        tree_ws = torch.empty((cin, ld_tree), dtype=x.dtype, device=x.device)
        gtree_ws = None if skip_gx else torch.empty((cin, ld_tree), dtype=torch.float32, device=x.device)
        gx32_ws = None if skip_gx else torch.empty((cin, N), dtype=torch.float32, device=x.device)
        with torch.cuda.device(x.device):
            st = _stream()
            for b in range(B):
                rc = _lib().aprnet_conv_bwd_bf16(plans[b], d[b], kz, kx, ky, _ptr(x[b]), N, cin, _ptr(weights), s_exp, cout,
                                                 _ptr(grad_output[b]), grad_output.size(2), gxp(b), N, _ptr(gw),
                                                 _ptr(tree_ws), ld_tree, None if skip_gx else _ptr(gx32_ws), N,
                                                 None if skip_gx else _ptr(gtree_ws), ld_tree, st)
                if rc:
                    _raise(rc, "conv_backward failed")
        return [gx, gw]
    gw = torch.zeros_like(weights)
    sfx = _sfx(x)
    with torch.cuda.device(x.device):
        st = _stream()
        if (kz, kx, ky) == (1, 1, 1):
            fn = getattr(_lib(), "aprnet_conv111_bwd_" + sfx)
            for b in range(B):
                rc = fn(plans[b], d[b], _ptr(x[b]), N, cin, _ptr(weights), s_exp, cout, _ptr(grad_output[b]),
                        grad_output.size(2), _ptr(gx[b]), N, _ptr(gw), st)
                if rc:
                    _raise(rc, "conv111_backward failed")
        else:
            ld_tree = max(max(tree_parts(a, d[b]) for b, a in enumerate(aprs)), 1)
            tree_ws = torch.empty((cin, ld_tree), dtype=x.dtype, device=x.device)
            gtree_ws = None if skip_gx else torch.empty((cin, ld_tree), dtype=x.dtype, device=x.device)
            fn = getattr(_lib(), "aprnet_conv_bwd_" + sfx)
            for b in range(B):
                rc = fn(plans[b], d[b], kz, kx, ky, _ptr(x[b]), N, cin, _ptr(weights), s_exp, cout,
                        _ptr(grad_output[b]), grad_output.size(2), gxp(b), N, _ptr(gw),
                        _ptr(tree_ws), ld_tree, None if skip_gx else _ptr(gtree_ws), ld_tree, st)
                if rc:
                    _raise(rc, "conv_backward failed")
    return [gx, gw]


# ---------------------------------------------------------------------------------------- pool / upsample
def maxpool_forward(aprs, x, level_delta, pad_value=-1e17):
    """maxpool_forward (maxpool.hpp:43-64) -> [output, max_indices].  Slots behind a batch item's last
    particle hold ``pad_value``: -1e17 in the CPU flavour (maxpool.hpp:51), 0 in the CUDA flavour
    (wrap_maxpool_gpu.hpp:42)."""
    _check_input(x, "input")
    B, Cn, N = x.shape
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b] + 1) for b, a in enumerate(aprs)]
    n_out = max(sizes)
    out = torch.empty((B, Cn, n_out), dtype=x.dtype, device=x.device)
    idx = torch.empty((B, Cn, n_out), dtype=torch.int64, device=x.device)
    for b, nb in enumerate(sizes):
        if nb < n_out:
            out[b, :, nb:] = pad_value
            idx[b, :, nb:] = 0
    plans = _plans(aprs, x.device)
    fn = getattr(_lib(), "aprnet_maxpool_fwd_" + _sfx(x, bf16=True))
    with torch.cuda.device(x.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(x[b]), N, Cn, _ptr(out[b]), n_out, _ptr(idx[b]), n_out, st)
            if rc:
                _raise(rc, "maxpool_forward failed")
    return [out, idx]


def maxpool_backward(aprs, grad_output, max_indices, level_delta):
    _check_input(grad_output, "grad_output")
    _check_input(max_indices, "max_indices")
    B, Cn, n_out = grad_output.shape
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    n_in = max(sizes)
    gx = torch.empty((B, Cn, n_in), dtype=grad_output.dtype, device=grad_output.device)
    _zero_tails(gx, sizes)
    plans = _plans(aprs, grad_output.device)
    fn = getattr(_lib(), "aprnet_maxpool_bwd_" + _sfx(grad_output, bf16=True))
    with torch.cuda.device(grad_output.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(grad_output[b]), n_out, Cn, _ptr(gx[b]), n_in, _ptr(max_indices[b]),
                    max_indices.size(2), st)
            if rc:
                _raise(rc, "maxpool_backward failed")
    return gx


def upsample_const_forward(aprs, x, level_delta):
    _check_input(x, "input")
    B, Cn, N = x.shape
    d = _deltas(level_delta, len(aprs))
    if min(d[:len(aprs)]) <= 0:           # upsample.hpp:49-54
        raise ValueError("UpSampleConst is only implemented for downsampled particles. It is currently "
                         "not possible to go beyond the original resolution. That is, input must have "
                         "`level_delta > 0`.")
    sizes = [number_particles(a, d[b] - 1) for b, a in enumerate(aprs)]
    n_out = max(sizes)
    out = torch.empty((B, Cn, n_out), dtype=x.dtype, device=x.device)
    _zero_tails(out, sizes)
    plans = _plans(aprs, x.device)
    fn = getattr(_lib(), "aprnet_upsample_fwd_" + _sfx(x, bf16=True))
    with torch.cuda.device(x.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(x[b]), N, Cn, _ptr(out[b]), n_out, st)
            if rc:
                _raise(rc, "upsample_const_forward failed")
    return out


def upsample_const_backward(aprs, grad_output, level_delta):
    _check_input(grad_output, "grad_output")
    B, Cn, n_out = grad_output.shape
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    n_in = max(sizes)
    gx = torch.empty((B, Cn, n_in), dtype=grad_output.dtype, device=grad_output.device)
    _zero_tails(gx, sizes)
    plans = _plans(aprs, grad_output.device)
    fn = getattr(_lib(), "aprnet_upsample_bwd_" + _sfx(grad_output, bf16=True))
    with torch.cuda.device(grad_output.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(grad_output[b]), n_out, Cn, _ptr(gx[b]), n_in, st)
            if rc:
                _raise(rc, "upsample_const_backward failed")
    return gx


# ---------------------------------------------------------------------------------------- pixels <-> particles
def _dense_shape(aprs, d):
    z = x = y = 0
    for b, a in enumerate(aprs):
        lc = a.level_max() - d[b]
        z, x, y = max(z, a.z_num(lc)), max(x, a.x_num(lc)), max(y, a.y_num(lc))
    return z, x, y


def _same_dense_shape(aprs, d, shape):
    for b, a in enumerate(aprs):
        lc = a.level_max() - d[b]
        if (a.z_num(lc), a.x_num(lc), a.y_num(lc)) != tuple(shape):
            raise ValueError("reconstruct / sample_particles: all batch items must share the dense shape "
                             f"{tuple(shape)} at their level delta")


def reconstruct_forward(aprs, x, level_delta):
    """reconstruct_forward (wrap_reconstruct_gpu.hpp:30-63): particles [B,C,N_d] -> [B,C,Z,X,Y] at level Lc."""
    _check_input(x, "input")
    B, Cn, N = x.shape
    d = _deltas(level_delta, len(aprs))
    shape = _dense_shape(aprs, d)
    _same_dense_shape(aprs, d, shape)
    out = torch.zeros((B, Cn, *shape), dtype=x.dtype, device=x.device)
    plane = shape[0] * shape[1] * shape[2]
    plans = _plans(aprs, x.device)
    fn = getattr(_lib(), "aprnet_reconstruct_fwd_" + _sfx(x, bf16=True))
    with torch.cuda.device(x.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(x[b]), N, Cn, _ptr(out[b]), plane, st)
            if rc:
                _raise(rc, "reconstruct_forward failed")
    return out


def reconstruct_backward(aprs, grad_output, level_delta):
    _check_input(grad_output, "grad_output")
    B, Cn = grad_output.shape[:2]
    d = _deltas(level_delta, len(aprs))
    _same_dense_shape(aprs, d, grad_output.shape[2:])
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    n = max(sizes)
    gx = torch.empty((B, Cn, n), dtype=grad_output.dtype, device=grad_output.device)
    _zero_tails(gx, sizes)
    plane = grad_output[0, 0].numel()
    plans = _plans(aprs, grad_output.device)
    fn = getattr(_lib(), "aprnet_reconstruct_bwd_" + _sfx(grad_output, bf16=True))
    with torch.cuda.device(grad_output.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(grad_output[b]), plane, Cn, _ptr(gx[b]), n, st)
            if rc:
                _raise(rc, "reconstruct_backward failed")
    return gx


def sample_particles_forward(aprs, img, level_delta):
    """sample_particles_forward (wrap_sample_particles_gpu.hpp:30-63): dense [B,C,Z,X,Y] -> particles (cell means)."""
    _check_input(img, "input")
    B, Cn = img.shape[:2]
    d = _deltas(level_delta, len(aprs))
    _same_dense_shape(aprs, d, img.shape[2:])
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    n = max(sizes)
    out = torch.empty((B, Cn, n), dtype=img.dtype, device=img.device)
    _zero_tails(out, sizes)
    plane = img[0, 0].numel()
    plans = _plans(aprs, img.device)
    fn = getattr(_lib(), "aprnet_sample_particles_fwd_" + _sfx(img, bf16=True))
    with torch.cuda.device(img.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(img[b]), plane, Cn, _ptr(out[b]), n, st)
            if rc:
                _raise(rc, "sample_particles_forward failed")
    return out


def sample_particles_backward(aprs, grad_output, level_delta):
    _check_input(grad_output, "grad_output")
    B, Cn, N = grad_output.shape
    d = _deltas(level_delta, len(aprs))
    shape = _dense_shape(aprs, d)
    _same_dense_shape(aprs, d, shape)
    gimg = torch.zeros((B, Cn, *shape), dtype=grad_output.dtype, device=grad_output.device)
    plane = shape[0] * shape[1] * shape[2]
    plans = _plans(aprs, grad_output.device)
    fn = getattr(_lib(), "aprnet_sample_particles_bwd_" + _sfx(grad_output, bf16=True))
    with torch.cuda.device(grad_output.device):
        st = _stream()
        for b in range(B):
            rc = fn(plans[b], d[b], _ptr(grad_output[b]), N, Cn, _ptr(gimg[b]), plane, st)
            if rc:
                _raise(rc, "sample_particles_backward failed")
    return gimg
