"""torch.autograd.Functions of the particle-space operators, with the contracts of the reference's
Functions (pyapr/aprnet/conv.py:18-138, pool.py:7-22, upsample.py:7-22; cuda/conv.py:12-54,
cuda/maxpool.py:8-28, cuda/upsample.py:8-26, cuda/utils.py:10-47):

* convolution: weights are expanded to one stencil per level before every call
  (num_levels = max over the batch of level_max - level_min + 1, conv.py:95), the expanded weights and a
  *clone* of ``level_deltas`` are saved for backward, the bias is added afterwards, backward returns
  ``(grad_input, grad_weights, grad_bias, None, None)``;
* max-pool / upsample mutate ``level_deltas`` in place *after* the native call (pool.py:13-14,
  upsample.py:13-14) and use the saved pre-mutation copy in backward.

One Function per operator, parameterised by the stencil size and the weight layout, instead of one
class per stencil size.
"""
import torch
from torch.autograd import Function

from . import _ops

CPU_LAYOUT = "cin_s_cout"      # [Cin, S, Cout, kz, kx, ky]   pyapr/aprnet/conv.py:164
CUDA_LAYOUT = "s_cout_cin"     # [S, Cout, Cin, kz, kx, ky]   pyapr/aprnet/cuda/conv.py:77

SUPPORTED_KERNELS = {(1, 1, 1), (1, 3, 3), (1, 5, 5), (3, 3, 3), (5, 5, 5)}


def _to_device_layout(w, layout):
    return w if layout == CUDA_LAYOUT else w.permute(1, 2, 0, 3, 4, 5).contiguous()


def _from_device_layout(w, layout):
    return w if layout == CUDA_LAYOUT else w.permute(2, 0, 1, 3, 4, 5).contiguous()


class ConvFunction(Function):
    @staticmethod
    def forward(ctx, inputs, weights, bias, aprs, level_deltas, layout):
        ctx.aprs = aprs
        ctx.layout = layout
        ctx.param_dtypes = (weights.dtype, None if bias is None else bias.dtype)
        w = _to_device_layout(weights, layout).contiguous()
        if inputs.dtype == torch.bfloat16:
            w = w.float()          # bfloat16 stores the features; stencils are restricted and applied in fp32
        ctx.num_stencils = w.shape[0]
        ksize = tuple(w.shape[3:])
        if ksize not in SUPPORTED_KERNELS:
            raise ValueError(f"unsupported kernel size {ksize}")
        ctx.expand = ksize != (1, 1, 1)
        if ctx.expand:
            num_levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
            w = _ops.restrict_kernel_forward(w, num_levels)
        inputs = inputs.contiguous()
        ctx.save_for_backward(inputs, w, bias, level_deltas.clone())
        # the bias add of conv.py:101 is fused into the kernel's store
        return _ops.conv_forward(aprs, inputs, w, level_deltas, None if bias is None else bias.contiguous())

    @staticmethod
    def backward(ctx, grad_output):
        inputs, w_exp, bias, level_deltas = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_input, grad_w = _ops.conv_backward(ctx.aprs, inputs, w_exp, grad_output, level_deltas,
                                                need_input_grad=ctx.needs_input_grad[0])
        grad_bias = None if bias is None else _ops.channel_sum(grad_output)
        if ctx.expand:
            grad_w = _ops.restrict_kernel_backward(grad_w, ctx.num_stencils)
        grad_w = _from_device_layout(grad_w, ctx.layout).to(ctx.param_dtypes[0])     # fp32 sums for bfloat16 features
        if grad_bias is not None:
            grad_bias = grad_bias.to(ctx.param_dtypes[1])
        return grad_input, grad_w, grad_bias, None, None, None


def conv_inference(inputs, weights, bias, aprs, level_deltas, layout, relu=False, inputs2=None, kept_stencils=None):
    """ConvFunction.forward without the autograd record, with the two fusions the kernel offers: the ReLU that
    follows the convolution in BasicBlock (unet_parts.py:17-26, norm folded away) and a second input tensor in
    place of torch.cat([inputs, inputs2], dim=1) (unet_parts.py:82).  For inference under torch.no_grad().
    ``kept_stencils``: (levels, fp32 stencils in the device layout already restricted to that many levels), used when
    the APRs have that many levels."""
    levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
    if (kept_stencils is not None and kept_stencils[0] == levels and inputs.dtype in (torch.float32, torch.bfloat16)
            and kept_stencils[1].device == inputs.device):
        return _ops.conv_forward(aprs, inputs.contiguous(), kept_stencils[1], level_deltas,
                                 None if bias is None else bias.detach().contiguous(),
                                 relu=relu, x2=None if inputs2 is None else inputs2.contiguous())
    w = _to_device_layout(weights.detach(), layout).contiguous()
    if inputs.dtype == torch.bfloat16:
        w = w.float()
    ksize = tuple(w.shape[3:])
    if ksize not in SUPPORTED_KERNELS:
        raise ValueError(f"unsupported kernel size {ksize}")
    if ksize != (1, 1, 1):
        w = _ops.restrict_kernel_forward(w, levels)
    return _ops.conv_forward(aprs, inputs.contiguous(), w, level_deltas, None if bias is None else bias.detach().contiguous(),
                             relu=relu, x2=None if inputs2 is None else inputs2.contiguous())


class NormFunction(Function):
    """Normalisation over the particle axis (+ optional ReLU) of a [B, C, N] tensor with the arithmetic of
    torch.nn.BatchNorm1d (``kind='batch'``: one set of statistics per channel, taken over batch and particles) and
    torch.nn.GroupNorm (``kind='group'``: one per batch item and group), as BasicBlock applies them
    (apr_models/unet/unet_parts.py:17-26).  ``stats`` = (mean[C], var[C]) normalises with given statistics (BatchNorm in
    eval mode) instead of those of the input.  Returns ``(y, mean, var)``: the statistics used (biased variance, float32),
    per channel for 'batch' and [B, groups] for 'group'.  Four launches each way: row moments (two), the join, apply."""

    @staticmethod
    def forward(ctx, x, weight, bias, kind, groups, eps, relu, stats):
        x = x.contiguous()
        g = 0 if kind == "batch" else int(groups)
        row_mean = row_m2 = None
        if stats is None:
            row_mean, row_m2 = _ops.row_moments(x)                  # float64 [B, C]
        mean32, rstd32, scale32, shift32, set_mean, set_var = _ops.norm_coeffs_forward(
            tuple(x.shape), g, eps, row_mean, row_m2, stats, weight, bias, x.device)
        y = _ops.norm_apply(x, mean32, scale32, shift32, relu)
        if stats is not None:
            set_mean, set_var = stats[0].detach().float(), stats[1].detach().float()
        ctx.save_for_backward(x, y if relu else None, mean32, rstd32, weight)
        ctx.cfg = (g, stats is None, None if weight is None else weight.dtype, None if bias is None else bias.dtype)
        ctx.mark_non_differentiable(set_mean, set_var)
        return y, set_mean, set_var

    @staticmethod
    def backward(ctx, grad_y, _gm, _gv):
        x, y, mean32, rstd32, weight = ctx.saved_tensors
        g, own_stats, w_dtype, b_dtype = ctx.cfg
        grad_y = grad_y.contiguous()
        s_g, s_gx = _ops.norm_backward_sums(grad_y, x, y, mean32, rstd32)          # float64 [B, C]
        want_w = w_dtype is not None and ctx.needs_input_grad[1]
        want_b = b_dtype is not None and ctx.needs_input_grad[2]
        a, b, c, grad_w, grad_b = _ops.norm_coeffs_backward(tuple(x.shape), g, own_stats, s_g, s_gx, weight, rstd32, want_w, want_b)
        grad_x = _ops.norm_backward_apply(grad_y, x, y, mean32, rstd32, a, b, c) if ctx.needs_input_grad[0] else None
        if grad_w is not None and grad_w.dtype != w_dtype:
            grad_w = grad_w.to(w_dtype)
        if grad_b is not None and grad_b.dtype != b_dtype:
            grad_b = grad_b.to(b_dtype)
        return grad_x, grad_w, grad_b, None, None, None, None, None


class MaxPoolFunction(Function):
    @staticmethod
    def forward(ctx, inputs, aprs, level_deltas, increment_level_deltas, pad_value):
        ctx.aprs = aprs
        output, max_indices = _ops.maxpool_forward(aprs, inputs.contiguous(), level_deltas, pad_value)
        ctx.save_for_backward(max_indices, level_deltas.clone())
        if increment_level_deltas:
            level_deltas.add_(1)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        max_indices, level_deltas = ctx.saved_tensors
        grad_input = _ops.maxpool_backward(ctx.aprs, grad_output.contiguous(), max_indices, level_deltas)
        return grad_input, None, None, None, None


class UpSampleConstFunction(Function):
    @staticmethod
    def forward(ctx, inputs, aprs, level_deltas, decrement_level_deltas):
        ctx.aprs = aprs
        ctx.save_for_backward(level_deltas.clone())
        output = _ops.upsample_const_forward(aprs, inputs.contiguous(), level_deltas)
        if decrement_level_deltas:
            level_deltas.sub_(1)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        level_deltas, = ctx.saved_tensors
        grad_input = _ops.upsample_const_backward(ctx.aprs, grad_output.contiguous(), level_deltas)
        return grad_input, None, None, None


class ReconstructFunction(Function):
    @staticmethod
    def forward(ctx, inputs, aprs, level_deltas):
        ctx.aprs = aprs
        ctx.save_for_backward(level_deltas.clone())
        return _ops.reconstruct_forward(aprs, inputs.contiguous(), level_deltas)

    @staticmethod
    def backward(ctx, grad_output):
        level_deltas, = ctx.saved_tensors
        return _ops.reconstruct_backward(ctx.aprs, grad_output.contiguous(), level_deltas), None, None


class SampleParticlesFunction(Function):
    @staticmethod
    def forward(ctx, inputs, aprs, level_deltas):
        ctx.aprs = aprs
        ctx.save_for_backward(level_deltas.clone())
        return _ops.sample_particles_forward(aprs, inputs.contiguous(), level_deltas)

    @staticmethod
    def backward(ctx, grad_output):
        level_deltas, = ctx.saved_tensors
        return _ops.sample_particles_backward(ctx.aprs, grad_output.contiguous(), level_deltas), None, None
