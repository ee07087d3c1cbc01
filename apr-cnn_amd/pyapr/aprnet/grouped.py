"""bfloat16 features grouped by eight channels, ``[B, C / 8, N, 8]``: the layout that the forward pass of a network
keeps between its layers on the GPU (no counterpart in the reference, whose tensors are ``[B, C, N]`` planes,
conv.hpp:68).  A particle's eight channels are one 16-byte word: the convolution stages straight from its input
instead of from a regrouped copy, pool / upsample / tree fill move 16 bytes per access, and every result is
bit-identical to the plane operators'.  Inference only (no autograd), channel counts multiples of eight, at most
2^31 - 1 particles per APR (from 2^28 on the convolution addresses its items with 64 bits instead of 32-bit offsets)."""
import ctypes as C

import torch

from . import _ops
from ._ops import _check_input, _deltas, _lib, _plans, _ptr, _raise, _stream, number_particles, tree_parts

MAX_PARTICLES = (1 << 31) - 1


class Grouped:
    """``data``: contiguous bfloat16 GPU tensor [B, C / 8, N, 8]."""

    def __init__(self, data):
        if data.dtype != torch.bfloat16 or data.dim() != 4 or data.size(3) != 8 or not data.is_cuda or not data.is_contiguous():
            raise ValueError("grouped features: contiguous bfloat16 GPU tensor [B, C / 8, N, 8] expected")
        self.data = data

    @property
    def channels(self):
        return self.data.size(1) * 8

    @property
    def particles(self):
        return self.data.size(2)


def limits():
    """Channel limits of the grouped kernels, read from the library."""
    return {"conv111_max_cin": int(_lib().aprnet_conv111_g8_max_cin())}


def supported(aprs, channels):
    return all(c % 8 == 0 for c in channels) and all(a.total_number_particles() <= MAX_PARTICLES for a in aprs)


def regroup(x):
    """[B, C, N] bfloat16 planes -> Grouped (channels past C pad the last group with zeros)."""
    _check_input(x, "input")
    if x.dtype != torch.bfloat16:
        raise TypeError("grouped features are bfloat16")
    B, Cn, N = x.shape
    out = torch.empty((B, (Cn + 7) // 8, N, 8), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        st = _stream()
        for b in range(B):
            rc = _lib().aprnet_regroup8_bf16(_ptr(x[b]), N, Cn, N, _ptr(out[b]), N, st)
            if rc:
                _raise(rc, "regroup failed")
    return Grouped(out)


def ungroup(g, channels=None):
    """Grouped -> [B, C, N] bfloat16 planes."""
    B, G, N, _ = g.data.shape
    Cn = channels or G * 8
    out = torch.empty((B, Cn, N), dtype=g.data.dtype, device=g.data.device)
    with torch.cuda.device(out.device):
        st = _stream()
        for b in range(B):
            rc = _lib().aprnet_ungroup8_bf16(_ptr(g.data[b]), N, Cn, N, _ptr(out[b]), N, st)
            if rc:
                _raise(rc, "ungroup failed")
    return out


def _fusion(x2, b, N, c2, relu, x2_coarse):
    fu = _ops._Fusion(_ptr(x2.data[b]) if x2 is not None else None, N, c2, 1 if relu else 0)
    if x2_coarse is not None:
        if x2 is None or x2_coarse.channels != c2 or x2_coarse.data.shape[0] != x2.data.shape[0]:
            raise ValueError("x2_coarse goes with a second input of the same batch size and channel count")
        fu.x2_coarse, fu.ld_coarse = _ptr(x2_coarse.data[b]), x2_coarse.data.shape[2]
    return fu


def conv_forward(aprs, x, weights, level_delta, bias=None, relu=False, x2=None, grouped_output=True, x2_coarse=None):
    """Stencil convolution (3x3x3, 1x3x3, 1x5x5) on the bfloat16 matrix cores.  ``x``: Grouped, or a [B, C <= 3, N]
    bfloat16 plane tensor (the first layer of a network); ``x2``: optional Grouped second input whose channels follow
    those of x (the concatenation of a decoder stage).  weights [S_exp, Cout, Cin, kz, kx, ky] fp32.
    ``x2_coarse``: the Grouped tensor at level_delta + 1 that x2 is the upsample_const_forward of; the mean tree of x2
    is then read off it instead of computed from x2 (same values, an eighth of the reads).
    -> Grouped, or [B, Cout, N] planes with ``grouped_output=False``."""
    planes_in = not isinstance(x, Grouped)
    xd = x if planes_in else x.data
    _check_input(weights, "weights")
    weights = weights.float()
    bias = None if bias is None else bias.float().contiguous()
    s_exp, cout, cin, kz, kx, ky = weights.shape
    B, N = xd.shape[0], xd.shape[2]
    c1 = xd.shape[1] if planes_in else x.channels
    c2 = 0 if x2 is None else x2.channels
    if c1 + c2 != cin:
        raise ValueError("convolve: input tensor shape does not match weights tensor!")
    if x2 is not None and (planes_in or x2.data.shape[0] != B or x2.data.shape[2] != N):
        raise ValueError("the second input must be grouped and match the first in batch size and particle count")
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    if max(sizes) > N:
        raise ValueError("input holds fewer particles than the APR at this level delta")
    if grouped_output:
        out = torch.empty((B, cout // 8, N, 8), dtype=torch.bfloat16, device=xd.device)
    else:
        out = torch.empty((B, cout, N), dtype=torch.bfloat16, device=xd.device)
    for b, nb in enumerate(sizes):             # slots behind a batch item's last particle, as conv_forward leaves them
        if nb < N:
            pad = torch.zeros(cout, device=xd.device) if bias is None else (bias.clamp(min=0) if relu else bias)
            if grouped_output:
                out[b, :, nb:, :] = pad.to(torch.bfloat16).view(cout // 8, 1, 8)
            else:
                out[b, :, nb:] = pad.to(torch.bfloat16).view(-1, 1)
    ld_tree = max(max(tree_parts(a, d[b]) for b, a in enumerate(aprs)), 1)
    tree_ws = torch.empty((cin if planes_in else cin // 8, ld_tree, 1 if planes_in else 8), dtype=torch.bfloat16, device=xd.device)
    plans = _plans(aprs, xd.device)
    with torch.cuda.device(xd.device):
        st = _stream()
        for b in range(B):
            fu = _fusion(x2, b, N, c2, relu, x2_coarse)
            rc = _lib().aprnet_conv_fwd_fused_bf16l(plans[b], d[b], kz, kx, ky, _ptr(xd[b]), N, c1, 0 if planes_in else 1, _ptr(weights),
                                                    s_exp, cout, None if bias is None else _ptr(bias), _ptr(out[b]), N,
                                                    1 if grouped_output else 0, _ptr(tree_ws), ld_tree, C.byref(fu), st)
            if rc:
                _raise(rc, "conv_forward failed")
    return Grouped(out) if grouped_output else out


def head_limits_ok(cout, head_weights):
    """Whether conv_head_forward takes a layer of ``cout`` channels followed by this 1x1x1 head."""
    return cout <= 16 and head_weights.shape[1] <= 4 and tuple(head_weights.shape[3:]) == (1, 1, 1) and head_weights.shape[2] == cout


def conv_head_forward(aprs, x, weights, level_delta, bias, head_weights, head_bias=None, relu=True, x2=None, x2_coarse=None):
    """The last stencil convolution of a network and the 1x1x1 convolution that follows it (unet_model.py:94) in one
    kernel: conv111(relu(conv(x) + bias)) without storing the layer's result.  ``x`` (and ``x2``) Grouped, weights
    [S_exp, Cout <= 16, Cin, kz, kx, ky], head_weights [S, C <= 4, Cout, 1, 1, 1] (not expanded), fp32
    -> [B, C, N] bfloat16 planes."""
    _check_input(weights, "weights")
    weights = weights.float()
    bias = None if bias is None else bias.float().contiguous()
    hw = head_weights.float().contiguous()
    hb = None if head_bias is None else head_bias.float().contiguous()
    s_exp, cout, cin, kz, kx, ky = weights.shape
    if not head_limits_ok(cout, hw):
        raise ValueError("the fused head takes at most 16 channels between the two convolutions and at most 4 outputs")
    B, N = x.data.shape[0], x.data.shape[2]
    c1, c2 = x.channels, (0 if x2 is None else x2.channels)
    if c1 + c2 != cin:
        raise ValueError("convolve: input tensor shape does not match weights tensor!")
    if x2 is not None and (x2.data.shape[0] != B or x2.data.shape[2] != N):
        raise ValueError("the second input must match the first in batch size and particle count")
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    if max(sizes) > N:
        raise ValueError("input holds fewer particles than the APR at this level delta")
    hs, hc = hw.shape[0], hw.shape[1]
    out = torch.empty((B, hc, N), dtype=torch.bfloat16, device=x.data.device)
    for b, nb in enumerate(sizes):             # slots behind a batch item's last particle, as conv111_forward leaves them
        if nb < N:
            out[b, :, nb:] = 0 if hb is None else hb.to(torch.bfloat16).view(-1, 1)
    ld_tree = max(max(tree_parts(a, d[b]) for b, a in enumerate(aprs)), 1)
    tree_ws = torch.empty((cin // 8, ld_tree, 8), dtype=torch.bfloat16, device=out.device)
    plans = _plans(aprs, out.device)
    with torch.cuda.device(out.device):
        st = _stream()
        for b in range(B):
            fu = _fusion(x2, b, N, c2, relu, x2_coarse)
            rc = _lib().aprnet_conv_fwd_head_bf16g(plans[b], d[b], kz, kx, ky, _ptr(x.data[b]), N, c1, _ptr(weights), s_exp, cout,
                                                   None if bias is None else _ptr(bias), _ptr(tree_ws), ld_tree, C.byref(fu),
                                                   _ptr(hw), hs, hc, None if hb is None else _ptr(hb), _ptr(out[b]), N, st)
            if rc:
                _raise(rc, "conv_head_forward failed")
    return out


def conv111_forward(aprs, x, weights, level_delta, bias=None, relu=False, grouped_output=True):
    """1x1x1 convolution of Grouped features; weights [S, Cout, Cin, 1, 1, 1] fp32 (not expanded)."""
    _check_input(weights, "weights")
    weights = weights.float().contiguous()
    bias = None if bias is None else bias.float().contiguous()
    s, cout, cin = weights.shape[:3]
    B, _, N, _ = x.data.shape
    if cin != x.channels:
        raise ValueError("convolve: input tensor shape does not match weights tensor!")
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b]) for b, a in enumerate(aprs)]
    if grouped_output:
        out = torch.empty((B, cout // 8, N, 8), dtype=torch.bfloat16, device=x.data.device)
    else:
        out = torch.empty((B, cout, N), dtype=torch.bfloat16, device=x.data.device)
    for b, nb in enumerate(sizes):
        if nb < N:
            pad = torch.zeros(cout, device=out.device) if bias is None else (bias.clamp(min=0) if relu else bias)
            if grouped_output:
                out[b, :, nb:, :] = pad.to(torch.bfloat16).view(cout // 8, 1, 8)
            else:
                out[b, :, nb:] = pad.to(torch.bfloat16).view(-1, 1)
    plans = _plans(aprs, out.device)
    with torch.cuda.device(out.device):
        st = _stream()
        for b in range(B):
            rc = _lib().aprnet_conv111_fwd_bf16g(plans[b], d[b], _ptr(x.data[b]), N, cin, _ptr(weights), s, cout,
                                                 None if bias is None else _ptr(bias), 1 if relu else 0, _ptr(out[b]), N,
                                                 1 if grouped_output else 0, st)
            if rc:
                _raise(rc, "conv111_forward failed")
    return Grouped(out) if grouped_output else out


def maxpool_forward(aprs, x, level_delta):
    """MaxPool forward, values only; padding slots of shorter batch items hold 0 (the CUDA flavour's fill)."""
    B, G, N, _ = x.data.shape
    d = _deltas(level_delta, len(aprs))
    sizes = [number_particles(a, d[b] + 1) for b, a in enumerate(aprs)]
    n_out = max(sizes)
    out = torch.empty((B, G, n_out, 8), dtype=x.data.dtype, device=x.data.device)
    for b, nb in enumerate(sizes):
        if nb < n_out:
            out[b, :, nb:, :] = 0
    plans = _plans(aprs, out.device)
    with torch.cuda.device(out.device):
        st = _stream()
        for b in range(B):
            rc = _lib().aprnet_maxpool_fwd_bf16g(plans[b], d[b], _ptr(x.data[b]), N, G * 8, _ptr(out[b]), n_out, st)
            if rc:
                _raise(rc, "maxpool_forward failed")
    return Grouped(out)


def upsample_const_forward(aprs, x, level_delta):
    B, G, N, _ = x.data.shape
    d = _deltas(level_delta, len(aprs))
    if min(d[:len(aprs)]) <= 0:
        raise ValueError("UpSampleConst is only implemented for downsampled particles. That is, input must have `level_delta > 0`.")
    sizes = [number_particles(a, d[b] - 1) for b, a in enumerate(aprs)]
    n_out = max(sizes)
    out = torch.empty((B, G, n_out, 8), dtype=x.data.dtype, device=x.data.device)
    for b, nb in enumerate(sizes):
        if nb < n_out:
            out[b, :, nb:, :] = 0
    plans = _plans(aprs, out.device)
    with torch.cuda.device(out.device):
        st = _stream()
        for b in range(B):
            rc = _lib().aprnet_upsample_fwd_bf16g(plans[b], d[b], _ptr(x.data[b]), N, G * 8, _ptr(out[b]), n_out, st)
            if rc:
                _raise(rc, "upsample_const_forward failed")
    return Grouped(out)
