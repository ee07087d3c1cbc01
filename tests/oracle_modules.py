"""autograd wrappers over the CPU oracle with the contracts of the reference's CPU-flavour
Functions (pyapr/aprnet/conv.py:18-138, pool.py:7-22, upsample.py:7-22, cuda/utils.py:10-47), so that
torch.autograd.gradcheck can pin the oracle's backward passes."""
import torch
from torch.autograd import Function

from oracle import oracle


class OracleConv(Function):
    @staticmethod
    def forward(ctx, x, weights, bias, aprs, level_deltas):
        ctx.aprs, ctx.S = aprs, weights.shape[1]
        k = tuple(weights.shape[3:])
        if k == (1, 1, 1):
            w_exp = weights
        else:
            num_levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
            w_exp = oracle.restrict_kernel_forward(weights, num_levels)
        ctx.k = k
        ctx.save_for_backward(x, w_exp, bias, level_deltas.clone())
        out = oracle.conv_forward(aprs, x, w_exp, level_deltas)
        return out if bias is None else out + bias.view(1, -1, 1)

    @staticmethod
    def backward(ctx, grad_output):
        x, w_exp, bias, level_deltas = ctx.saved_tensors
        gx, gw_exp = oracle.conv_backward(ctx.aprs, x, w_exp, grad_output, level_deltas)
        gw = gw_exp if ctx.k == (1, 1, 1) else oracle.restrict_kernel_backward(gw_exp, ctx.S)
        gb = None if bias is None else grad_output.sum(dim=(0, 2))
        return gx, gw, gb, None, None


class OracleMaxPool(Function):
    @staticmethod
    def forward(ctx, x, aprs, level_deltas):
        ctx.aprs = aprs
        out, idx = oracle.maxpool_forward(aprs, x, level_deltas)
        ctx.save_for_backward(idx, level_deltas.clone())
        return out

    @staticmethod
    def backward(ctx, grad_output):
        idx, level_deltas = ctx.saved_tensors
        return oracle.maxpool_backward(ctx.aprs, grad_output, idx, level_deltas), None, None


class OracleUpSample(Function):
    @staticmethod
    def forward(ctx, x, aprs, level_deltas):
        ctx.aprs = aprs
        ctx.save_for_backward(level_deltas.clone())
        return oracle.upsample_const_forward(aprs, x, level_deltas)

    @staticmethod
    def backward(ctx, grad_output):
        level_deltas, = ctx.saved_tensors
        return oracle.upsample_const_backward(ctx.aprs, grad_output, level_deltas), None, None


class OracleReconstruct(Function):
    @staticmethod
    def forward(ctx, x, aprs, level_deltas):
        ctx.aprs = aprs
        ctx.save_for_backward(level_deltas.clone())
        return oracle.reconstruct_forward(aprs, x, level_deltas)

    @staticmethod
    def backward(ctx, grad_output):
        level_deltas, = ctx.saved_tensors
        return oracle.reconstruct_backward(ctx.aprs, grad_output, level_deltas), None, None


class OracleSample(Function):
    @staticmethod
    def forward(ctx, img, aprs, level_deltas):
        ctx.aprs = aprs
        ctx.save_for_backward(level_deltas.clone())
        return oracle.sample_particles_forward(aprs, img, level_deltas)

    @staticmethod
    def backward(ctx, grad_output):
        level_deltas, = ctx.saved_tensors
        return oracle.sample_particles_backward(ctx.aprs, grad_output, level_deltas), None, None
