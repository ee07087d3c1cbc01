"""Building blocks of the particle-space U-Net.  Module tree and parameter names follow
apr_models/apr_models/unet/unet_parts.py:6-83 so that state_dicts are interchangeable:
BasicBlock = {conv, norm, activation}; ConvBlock = {blocks[i]}; DownConv = {pool, conv};
UpConv = {reduce_ch, upsample, conv}."""
import torch
import torch.nn as nn

from pyapr.aprnet import cuda as aprnet
from .particle_norm import ParticleBatchNorm, ParticleGroupNorm


def _make_norm(kind, channels, num_groups, bn_momentum):
    if kind == "group":
        groups = min(num_groups, channels) if num_groups is not None else channels
        return ParticleGroupNorm(num_groups=groups, num_channels=channels)
    if kind == "batch":
        return ParticleBatchNorm(channels, momentum=bn_momentum)
    if kind == "none":          # inference with the normalisation folded into the convolution
        return nn.Identity()
    raise ValueError("norm must be either 'group' or 'batch'")


class BasicBlock(nn.Module):
    """APRConv (no bias) -> norm over [B, C, N] -> activation."""

    def __init__(self, in_channels, out_channels, nstencils=1, kernel_size=(3, 3, 3), activation=nn.ReLU,
                 num_groups=None, norm="group", bn_momentum=0.1):
        super().__init__()
        self.conv = aprnet.APRConv(in_channels=in_channels, out_channels=out_channels, nstencils=nstencils,
                                   kernel_size=kernel_size, bias=False)
        self.norm = _make_norm(norm, out_channels, num_groups, bn_momentum)
        self.activation = activation if isinstance(activation, nn.Module) else activation()

    def forward(self, x, aprs, level_deltas, x2=None):
        """x2: optional second input whose channels follow those of x (the concatenation of UpConv)."""
        # Inference with the norm folded away: ReLU and the concatenation are done inside the convolution kernel
        if (not torch.is_grad_enabled() and isinstance(self.norm, nn.Identity) and type(self.activation) is nn.ReLU
                and x.is_cuda):
            return self.conv.forward_fused(x, aprs, level_deltas, relu=True, second_input=x2)
        if x2 is not None and not torch.is_grad_enabled() and x.is_cuda:
            y = self.conv.forward_fused(x, aprs, level_deltas, relu=False, second_input=x2)      # no concatenated copy
        else:
            if x2 is not None:
                x = torch.cat([x, x2], dim=1)
            y = self.conv(x, aprs, level_deltas)
        if type(self.activation) is nn.ReLU and isinstance(self.norm, (ParticleBatchNorm, ParticleGroupNorm)):
            return self.norm(y, relu=True)          # one pass for norm + ReLU
        return self.activation(self.norm(y))


class ConvBlock(nn.Module):
    def __init__(self, in_channels, out_channels, mid_channels=None, nstencils=1, kernel_size=(3, 3, 3),
                 activation=nn.ReLU, num_blocks=2, num_groups=None, norm="group", bn_momentum=0.1):
        super().__init__()
        mid = mid_channels or out_channels
        widths = [in_channels] + [mid] * (num_blocks - 1) + [out_channels]
        self.blocks = nn.ModuleList(
            BasicBlock(widths[i], widths[i + 1], nstencils=nstencils, kernel_size=kernel_size, activation=activation,
                       num_groups=num_groups, norm=norm, bn_momentum=bn_momentum) for i in range(num_blocks))

    def forward(self, x, aprs, level_deltas, x2=None):
        for i, block in enumerate(self.blocks):
            x = block(x, aprs, level_deltas, x2 if i == 0 else None)
        return x


class DownConv(nn.Module):
    """MaxPool (level_deltas += 1) then ConvBlock."""

    def __init__(self, in_channels, out_channels, mid_channels=None, nstencils=1, kernel_size=(3, 3, 3),
                 activation=nn.ReLU, num_conv_blocks=2, num_groups=None, norm="group", bn_momentum=0.1):
        super().__init__()
        self.pool = aprnet.MaxPool()
        self.conv = ConvBlock(in_channels, out_channels, mid_channels=mid_channels, nstencils=nstencils,
                              kernel_size=kernel_size, activation=activation, num_blocks=num_conv_blocks,
                              num_groups=num_groups, norm=norm, bn_momentum=bn_momentum)

    def forward(self, x, aprs, level_deltas):
        return self.conv(self.pool(x, aprs, level_deltas), aprs, level_deltas)


class UpConv(nn.Module):
    """1x1x1 channel reduction -> UpSampleConst (level_deltas -= 1) -> concat with the skip -> ConvBlock."""

    def __init__(self, in_channels, out_channels, mid_channels=None, nstencils=1, kernel_size=(3, 3, 3),
                 activation=nn.ReLU, num_conv_blocks=2, num_groups=None, norm="group", bn_momentum=0.1):
        super().__init__()
        # the reduction block keeps one group per channel (unet_parts.py:72)
        self.reduce_ch = BasicBlock(in_channels, in_channels // 2, nstencils=nstencils, kernel_size=(1, 1, 1),
                                    activation=activation, norm=norm, bn_momentum=bn_momentum)
        self.upsample = aprnet.UpSampleConst()
        self.conv = ConvBlock(in_channels, out_channels, mid_channels=mid_channels, nstencils=nstencils,
                              kernel_size=kernel_size, activation=activation, num_blocks=num_conv_blocks,
                              num_groups=num_groups, norm=norm, bn_momentum=bn_momentum)

    def forward(self, x1, x2, aprs, level_deltas):
        x1 = self.reduce_ch(x1, aprs, level_deltas)
        x1 = self.upsample(x1, aprs, level_deltas)
        return self.conv(x2, aprs, level_deltas, x1)          # = conv(torch.cat([x2, x1], dim=1)), unet_parts.py:82
