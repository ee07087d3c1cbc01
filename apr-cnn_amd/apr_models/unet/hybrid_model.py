"""HybridAPRUNet (apr_models/apr_models/unet/hybrid_model.py:7-139): the first ``apr_depth`` stages of encoder and
decoder work on particles, the stages below on the dense volume reconstructed at the resolution that is left
after ``apr_depth + 1`` pools.  Same constructor arguments, module tree and parameter names as the reference, plus
``norm`` ('group' as in the reference, 'batch' for models whose norms are folded for inference)."""
import torch
import torch.nn as nn

from pyapr.aprnet import cuda as aprnet
from .unet_parts import ConvBlock, DownConv, UpConv
from .hybrid_unet_parts import TransitionDownConv, TransitionUpConv, PixelDownConv, PixelUpConv


def hybrid_stages(in_channels, widths, stencils, depth, apr_depth, first_decoder_stage, kernel_size, activation, norm,
                  n_conv_per_block, groups):
    """Encoder and decoder of the hybrid networks (hybrid_model.py:47-114, stardist_hybrid_model.py:64-146): stage i
    works on particles for i < apr_depth, crosses between particles and the dense volume at i == apr_depth and is
    dense below.  The decoder holds the stages depth-1 ... first_decoder_stage."""
    common = dict(kernel_size=kernel_size, activation=activation, norm=norm)
    encoder = nn.ModuleList([ConvBlock(in_channels, widths[0], nstencils=stencils[0], num_blocks=n_conv_per_block,
                                       num_groups=groups(widths[0]), **common)])
    for i in range(depth):
        down = dict(num_conv_blocks=n_conv_per_block, num_groups=groups(widths[i + 1]), **common)
        if i < apr_depth:
            encoder.append(DownConv(widths[i], widths[i + 1], nstencils=stencils[i + 1], **down))
        elif i == apr_depth:
            encoder.append(TransitionDownConv(widths[i], widths[i + 1], **down))
        else:
            encoder.append(PixelDownConv(widths[i], widths[i + 1], **down))
    decoder = nn.ModuleList()
    for i in reversed(range(first_decoder_stage, depth)):
        up = dict(num_conv_blocks=n_conv_per_block, num_groups=groups(widths[i]), **common)
        if i < apr_depth:
            decoder.append(UpConv(widths[i + 1], widths[i], nstencils=stencils[i], **up))
        elif i == apr_depth:
            decoder.append(TransitionUpConv(widths[i + 1], widths[i], nstencils=stencils[i], **up))
        else:
            decoder.append(PixelUpConv(widths[i + 1], widths[i], **up))
    return encoder, decoder


def hybrid_forward(encoder, decoder, x, aprs, level_deltas):
    """Runs the stages (hybrid_model.py:123-137): particle stages take (features, aprs, level_deltas), dense ones the
    volume alone."""
    skips = [encoder[0](x, aprs, level_deltas)]
    for stage in encoder[1:]:
        on_particles = isinstance(stage, (DownConv, TransitionDownConv))
        skips.append(stage(skips[-1], aprs, level_deltas) if on_particles else stage(skips[-1]))
    y = skips[-1]
    for i, stage in enumerate(decoder):
        skip = skips[-(i + 2)]
        y = stage(y, skip, aprs, level_deltas) if isinstance(stage, (UpConv, TransitionUpConv)) else stage(y, skip)
    return y


class HybridAPRUNet(nn.Module):
    def __init__(self, in_channels, out_channels, depth=3, apr_depth=2, kernel_size=3, dims=3, activation=nn.ReLU,
                 n_filters_base=16, n_conv_per_block=2, n_stencils=2, decrement_stencils=False, num_groups=None,
                 channels_per_group=None, norm="group"):
        super().__init__()
        if apr_depth < 0:
            raise ValueError("apr_depth must not be negative")
        self.in_channels, self.out_channels, self.depth, self.apr_depth = in_channels, out_channels, depth, apr_depth
        self.num_groups = self.channels_per_group = None
        if num_groups is None and channels_per_group is None:
            self.num_groups = n_filters_base
        elif channels_per_group:
            self.channels_per_group = channels_per_group
        else:
            self.num_groups = num_groups

        ks = (kernel_size,) * dims if isinstance(kernel_size, int) else tuple(kernel_size)
        self.kernel_size = (1,) * (3 - len(ks)) + ks
        stencils = [max(n_stencils - i, 1) if decrement_stencils else max(n_stencils, 1) for i in range(depth + 1)]
        widths = [n_filters_base * 2 ** i for i in range(depth + 1)]

        def groups(c):
            return self.num_groups or c // self.channels_per_group

        self.encoder, self.decoder = hybrid_stages(in_channels, widths, stencils, depth, apr_depth, 0, self.kernel_size,
                                                   activation, norm, n_conv_per_block, groups)
        self.head = aprnet.APRConv(widths[0], out_channels, nstencils=stencils[0], kernel_size=(1, 1, 1))

    def forward(self, x, aprs, level_deltas=None):
        if level_deltas is None:
            level_deltas = torch.zeros(len(aprs), dtype=torch.int32, device=torch.device("cpu"))
        y = hybrid_forward(self.encoder, self.decoder, x, aprs, level_deltas)
        return self.head(y, aprs, level_deltas)
