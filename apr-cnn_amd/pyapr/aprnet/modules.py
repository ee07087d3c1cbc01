"""nn.Modules of the particle-space operators.

``APRConv``, ``MaxPool``, ``UpSampleConst`` keep the constructor signatures, parameter names and
initialisation of pyapr/aprnet/conv.py:154-182, pool.py:25-34, upsample.py:25-34.  The class
attribute ``weight_layout`` selects the parameter layout: the CPU flavour stores
[Cin, S, Cout, kz, kx, ky], the ``cuda`` flavour [S, Cout, Cin, kz, kx, ky] (cuda/conv.py:77), so
state_dicts of either flavour load unchanged."""
import math

import torch
from torch import nn
from torch.nn import init

from .functional import (ConvFunction, conv_inference, MaxPoolFunction, UpSampleConstFunction, ReconstructFunction,
                         SampleParticlesFunction, CPU_LAYOUT, CUDA_LAYOUT, SUPPORTED_KERNELS)


class APRConv(nn.Module):
    weight_layout = CPU_LAYOUT
    allowed_kernels = SUPPORTED_KERNELS

    def __init__(self, in_channels, out_channels, nstencils=1, kernel_size=(3, 3, 3), bias=True):
        super().__init__()
        kernel_size = tuple(kernel_size)
        assert len(kernel_size) == 3, "argument 'kernel_size' to APRConv must be of length 3"
        assert kernel_size in self.allowed_kernels, \
            f"APRConv supports kernels of size {sorted(self.allowed_kernels)}, got {kernel_size}"
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.nstencils = nstencils
        self.kernel_size = kernel_size
        shape = (in_channels, nstencils, out_channels) if self.weight_layout == CPU_LAYOUT \
            else (nstencils, out_channels, in_channels)
        self.weight = nn.Parameter(torch.empty(*shape, *kernel_size))
        self.bias = nn.Parameter(torch.empty(out_channels)) if bias else None
        self.reset_parameters()

    def extra_repr(self):
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, "
                f"nstencils={self.nstencils}, bias={self.bias is not None}")

    def reset_parameters(self):
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.weight)
            bound = 1 / math.sqrt(fan_in)
            init.uniform_(self.bias, -bound, bound)

    def forward(self, input_features, aprs, level_deltas):
        return ConvFunction.apply(input_features, self.weight, self.bias, aprs, level_deltas, self.weight_layout)

    def forward_fused(self, input_features, aprs, level_deltas, relu=False, second_input=None):
        """Inference-only forward (no autograd record): optionally clamps the result at zero inside the kernel and
        reads ``second_input`` as the channels that follow those of ``input_features``, i.e.
        relu(self(torch.cat([input_features, second_input], 1))) in one pass."""
        # stencils kept by a network's prepare_inference() (fp32, device layout); only weights that are fp32 themselves
        # would be restricted to the same values here
        kept = getattr(self, "_inference_stencils", None) if self.weight.dtype == torch.float32 else None
        return conv_inference(input_features, self.weight, self.bias, aprs, level_deltas, self.weight_layout,
                              relu=relu, inputs2=second_input, kept_stencils=kept)


class MaxPool(nn.Module):
    pad_value = -1e17        # value of output slots behind a batch item's last particle (maxpool.hpp:51)

    def __init__(self):
        super().__init__()
        # If True, increments the level_deltas tensor after the operation.  Set to False when the module is
        # called repeatedly on the same level_deltas, e.g. for numerical gradient tests.
        self.increment_level_deltas = True

    def forward(self, input_features, aprs, level_deltas):
        return MaxPoolFunction.apply(input_features, aprs, level_deltas, self.increment_level_deltas, self.pad_value)


class UpSampleConst(nn.Module):
    def __init__(self):
        super().__init__()
        self.decrement_level_deltas = True

    def forward(self, input_features, aprs, level_deltas):
        return UpSampleConstFunction.apply(input_features, aprs, level_deltas, self.decrement_level_deltas)


class Reconstruct(nn.Module):
    def forward(self, input_features, aprs, level_deltas=None):
        level_deltas = torch.zeros(len(aprs), dtype=torch.int32) if level_deltas is None else level_deltas
        return ReconstructFunction.apply(input_features, aprs, level_deltas)


class SampleParticles(nn.Module):
    def forward(self, input_features, aprs, level_deltas=None):
        level_deltas = torch.zeros(len(aprs), dtype=torch.int32) if level_deltas is None else level_deltas
        return SampleParticlesFunction.apply(input_features, aprs, level_deltas)
