"""APRStardistUNet (apr_models/apr_models/unet/stardist_model.py:8-132): the particle U-Net with two 1x1x1 heads,
an object probability (sigmoid) and ``n_rays`` radial distances, both evaluated on the particles that are left at
``output_level_delta`` (the decoder stops that many stages short of the input resolution).  Module tree and
parameter names as in the reference: encoder, decoder, conv_after_unet, output_prob = {conv, activation},
output_dist."""
import torch
import torch.nn as nn

from pyapr.aprnet import cuda as aprnet
from .unet_parts import ConvBlock, DownConv, UpConv
from .hybrid_model import hybrid_stages, hybrid_forward


class OutBlock(nn.Module):
    """Bias-free APRConv followed by an activation."""

    def __init__(self, in_channels, out_channels, nstencils=1, kernel_size=(3, 3, 3), activation=nn.ReLU):
        super().__init__()
        self.conv = aprnet.APRConv(in_channels=in_channels, out_channels=out_channels, nstencils=nstencils,
                                   kernel_size=kernel_size, bias=False)
        self.activation = activation if isinstance(activation, nn.Module) else activation()

    def forward(self, x, aprs, level_deltas):
        return self.activation(self.conv(x, aprs, level_deltas))


class APRStardistUNet(nn.Module):
    def __init__(self, in_channels, n_rays, depth=3, kernel_size=3, dims=3, activation=nn.ReLU, n_filters_base=16,
                 n_conv_per_block=2, n_stencils=2, decrement_stencils=False, num_groups=None, channels_per_group=None,
                 output_level_delta=0, net_conv_after_unet=None, norm="group"):
        super().__init__()
        if not 0 <= output_level_delta <= depth:
            raise ValueError("output_level_delta must lie between 0 and depth")
        self.in_channels, self.n_rays, self.depth = in_channels, n_rays, depth
        self.output_level_delta, self.net_conv_after_unet = output_level_delta, net_conv_after_unet
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

        common = dict(kernel_size=self.kernel_size, activation=activation, norm=norm)
        self.encoder = nn.ModuleList([ConvBlock(in_channels, widths[0], nstencils=stencils[0], num_blocks=n_conv_per_block,
                                                num_groups=groups(widths[0]), **common)])
        for i in range(depth):
            self.encoder.append(DownConv(widths[i], widths[i + 1], nstencils=stencils[i + 1],
                                         num_conv_blocks=n_conv_per_block, num_groups=groups(widths[i + 1]), **common))
        self.decoder = nn.ModuleList()
        for i in reversed(range(output_level_delta, depth)):
            self.decoder.append(UpConv(widths[i + 1], widths[i], nstencils=stencils[i], num_conv_blocks=n_conv_per_block,
                                       num_groups=groups(widths[i]), **common))
        n_features = widths[output_level_delta]
        self.conv_after_unet = None
        if net_conv_after_unet is not None:
            self.conv_after_unet = ConvBlock(n_features, net_conv_after_unet, nstencils=stencils[0],
                                             kernel_size=self.kernel_size, num_blocks=1, norm=norm)
            n_features = net_conv_after_unet
        self.output_prob = OutBlock(n_features, 1, nstencils=stencils[0], kernel_size=(1, 1, 1), activation=nn.Sigmoid)
        self.output_dist = aprnet.APRConv(n_features, n_rays, nstencils=stencils[0], kernel_size=(1, 1, 1))

    def forward(self, x, aprs, level_deltas=None):
        """-> (probability [B, 1, N_d], distances [B, n_rays, N_d]) with d = output_level_delta."""
        if level_deltas is None:
            level_deltas = torch.zeros(len(aprs), dtype=torch.int32, device=torch.device("cpu"))
        skips = [self.encoder[0](x, aprs, level_deltas)]
        for stage in self.encoder[1:]:
            skips.append(stage(skips[-1], aprs, level_deltas))
        y = skips[-1]
        for i, stage in enumerate(self.decoder):
            y = stage(y, skips[-(i + 2)], aprs, level_deltas)
        if self.conv_after_unet is not None:
            y = self.conv_after_unet(y, aprs, level_deltas)
        return self.output_prob(y, aprs, level_deltas), self.output_dist(y, aprs, level_deltas)


class HybridStardistUNet(nn.Module):
    """apr_models/apr_models/unet/stardist_hybrid_model.py:24-199: the hybrid particle / dense U-Net with the two
    StarDist heads.  The heads work on particles, so the decoder has to come back to particle space:
    output_level_delta <= apr_depth."""

    def __init__(self, in_channels, n_rays, depth=3, apr_depth=2, kernel_size=3, dims=3, activation=nn.ReLU,
                 n_filters_base=16, n_conv_per_block=2, n_stencils=2, decrement_stencils=False, num_groups=None,
                 channels_per_group=None, output_level_delta=0, net_conv_after_unet=None, norm="group", bn_momentum=0.1):
        super().__init__()
        if apr_depth < 0 or not 0 <= output_level_delta <= min(depth, apr_depth):
            raise ValueError("need 0 <= output_level_delta <= apr_depth: the heads work on particles")
        self.in_channels, self.n_rays, self.depth, self.apr_depth = in_channels, n_rays, depth, apr_depth
        self.output_level_delta, self.net_conv_after_unet = output_level_delta, net_conv_after_unet
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

        self.encoder, self.decoder = hybrid_stages(in_channels, widths, stencils, depth, apr_depth, output_level_delta,
                                                   self.kernel_size, activation, norm, n_conv_per_block, groups)
        n_features = widths[output_level_delta]
        self.conv_after_unet = None
        if net_conv_after_unet is not None:
            self.conv_after_unet = ConvBlock(n_features, net_conv_after_unet, nstencils=stencils[0], kernel_size=self.kernel_size,
                                             activation=activation, num_blocks=1, norm=norm, bn_momentum=bn_momentum)
            n_features = net_conv_after_unet
        self.output_prob = OutBlock(n_features, 1, nstencils=stencils[0], kernel_size=(1, 1, 1), activation=nn.Sigmoid)
        self.output_dist = aprnet.APRConv(n_features, n_rays, nstencils=stencils[0], kernel_size=(1, 1, 1))

    def forward(self, x, aprs, level_deltas=None):
        if level_deltas is None:
            level_deltas = torch.zeros(len(aprs), dtype=torch.int32, device=torch.device("cpu"))
        y = hybrid_forward(self.encoder, self.decoder, x, aprs, level_deltas)
        if self.conv_after_unet is not None:
            y = self.conv_after_unet(y, aprs, level_deltas)
        return self.output_prob(y, aprs, level_deltas), self.output_dist(y, aprs, level_deltas)
