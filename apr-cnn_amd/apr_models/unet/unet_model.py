"""APRUNet (apr_models/apr_models/unet/unet_model.py:7-94): encoder of ConvBlock + `depth` DownConv
stages, decoder of UpConv stages with skip connections, 1x1x1 head with bias.  One int32 CPU
``level_deltas`` tensor is shared and mutated in place by the pool / upsample modules."""
import torch
import torch.nn as nn

from pyapr.aprnet import cuda as aprnet
from .unet_parts import BasicBlock, ConvBlock, DownConv, UpConv


class APRUNet(nn.Module):
    def __init__(self, in_channels, out_channels, depth=3, kernel_size=3, dims=3, activation=nn.ReLU,
                 n_filters_base=16, n_conv_per_block=2, n_stencils=2, decrement_stencils=False, num_groups=None,
                 channels_per_group=None, norm="group"):
        super().__init__()
        self.in_channels, self.out_channels, self.depth = in_channels, out_channels, depth
        self.use_grouped = True         # inference with bfloat16 features: keep tensors grouped by eight channels between layers
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
        for i in reversed(range(depth)):
            self.decoder.append(UpConv(widths[i + 1], widths[i], nstencils=stencils[i], num_conv_blocks=n_conv_per_block,
                                       num_groups=groups(widths[i]), **common))
        self.head = aprnet.APRConv(widths[0], out_channels, nstencils=stencils[0], kernel_size=(1, 1, 1))

    def _grouped_ok(self, x, aprs):
        """Inference with bfloat16 features and every norm folded away runs on tensors grouped by eight channels
        (pyapr.aprnet.grouped): same arithmetic as the plane operators, no regrouping pass per convolution.
        Checked before any layer runs: element type, the channel limits of the grouped kernels, and that no
        submodule carries hooks or non-default level-delta flags (the grouped path calls the operators directly, so
        hooks on the submodules would not fire); anything else takes the module path."""
        from pyapr.aprnet import grouped
        if torch.is_grad_enabled() or not x.is_cuda or x.dtype != torch.bfloat16 or x.size(1) > 3 \
                or not getattr(self, "use_grouped", True):
            return False
        blocks = [b for m in self.modules() if isinstance(m, ConvBlock) for b in m.blocks] + [st.reduce_ch for st in self.decoder]
        limits = grouped.limits()
        for b in blocks:
            if not isinstance(b.norm, nn.Identity) or type(b.activation) is not nn.ReLU:
                return False
            s_, cout, cin = b.conv.weight.shape[:3]
            ks = tuple(b.conv.weight.shape[3:])
            if ks not in ((3, 3, 3), (1, 3, 3), (1, 5, 5), (1, 1, 1)) or cout % 8:
                return False
            if ks == (1, 1, 1) and (cin % 8 or cin > limits["conv111_max_cin"]):
                return False
            if ks != (1, 1, 1) and cin > 3 and cin % 8:
                return False
        hw = self.head.weight
        if tuple(hw.shape[3:]) != (1, 1, 1) or hw.shape[2] % 8 or hw.shape[2] > limits["conv111_max_cin"]:
            return False
        for m in self.modules():
            if m is self:
                continue
            if m._forward_hooks or m._forward_pre_hooks or m._backward_hooks:
                return False
            if getattr(m, "increment_level_deltas", True) is not True or getattr(m, "decrement_level_deltas", True) is not True:
                return False
        return grouped.supported(aprs, [])

    def prepare_inference(self, aprs=None, levels=None):
        """Builds the restricted stencils (restrict_kernel) of every stencil convolution once and keeps them on the
        convolution modules, so that the grouped inference path does not recompute them in every forward pass.
        ``levels``: number of APR levels the stencils are expanded to (default: taken from ``aprs``).  The kept
        stencils are dropped by ``train()``, ``load_state_dict()``, ``.to()`` / ``.float()`` ... and
        ``invalidate_inference_cache()``; call the latter after writing weights in a way autograd does not see
        (``weight.data.copy_()``, EMA swaps).  Without this call every forward pass restricts its stencils anew."""
        from pyapr.aprnet import _ops
        if levels is None:
            if aprs is None:
                raise ValueError("prepare_inference needs the APRs or the number of levels")
            levels = max(a.level_max() - a.level_min() + 1 for a in aprs)
        self.invalidate_inference_cache()
        with torch.no_grad():
            for m in self.modules():
                if isinstance(m, aprnet.APRConv) and tuple(m.weight.shape[3:]) != (1, 1, 1) and m.weight.is_cuda:
                    m._inference_stencils = (int(levels), _ops.restrict_kernel_forward(m.weight.detach().float().contiguous(), int(levels)))
        return self

    def invalidate_inference_cache(self):
        for m in self.modules():
            if hasattr(m, "_inference_stencils"):
                del m._inference_stencils
        return self

    def train(self, mode=True):
        if mode:
            self.invalidate_inference_cache()
        return super().train(mode)

    def load_state_dict(self, *args, **kwargs):
        self.invalidate_inference_cache()
        return super().load_state_dict(*args, **kwargs)

    def _apply(self, fn, *args, **kwargs):
        self.invalidate_inference_cache()
        return super()._apply(fn, *args, **kwargs)

    def _forward_grouped(self, x, aprs, level_deltas):
        from pyapr.aprnet import grouped as g8
        from pyapr.aprnet import _ops
        levels = max(a.level_max() - a.level_min() + 1 for a in aprs)

        def restricted(conv_module):
            # stencils of the coarser levels: taken from prepare_inference() when it ran for this number of levels,
            # otherwise computed here (never cached implicitly: a write through weight.data would go unnoticed)
            kept = getattr(conv_module, "_inference_stencils", None)
            if kept is not None and kept[0] == levels:
                return kept[1]
            return _ops.restrict_kernel_forward(conv_module.weight.detach().float().contiguous(), levels)

        def conv(bb, inp, second=None, coarse=None):
            w = bb.conv.weight.detach().float()
            bias = None if bb.conv.bias is None else bb.conv.bias.detach()
            if tuple(w.shape[3:]) == (1, 1, 1):
                return g8.conv111_forward(aprs, inp, w, level_deltas, bias, relu=True)
            return g8.conv_forward(aprs, inp, restricted(bb.conv), level_deltas, bias, relu=True, x2=second, x2_coarse=coarse)

        def block(cb, inp, second=None):
            for i, bb in enumerate(cb.blocks):
                inp = conv(bb, inp, second if i == 0 else None)
            return inp

        skips = [block(self.encoder[0], x.contiguous())]
        for stage in self.encoder[1:]:
            pooled = g8.maxpool_forward(aprs, skips[-1], level_deltas)
            level_deltas += 1
            skips.append(block(stage.conv, pooled))
            del pooled
        hw = self.head.weight.detach().float()
        hb = None if self.head.bias is None else self.head.bias.detach()

        def last_conv_with_head(bb, inp, second=None, coarse=None):
            # the network's last stencil convolution and the 1x1x1 head in one kernel: its 16 channels at full
            # resolution are neither written nor read back
            bias = None if bb.conv.bias is None else bb.conv.bias.detach()
            return g8.conv_head_forward(aprs, inp, restricted(bb.conv), level_deltas, bias, hw, hb, relu=True, x2=second,
                                        x2_coarse=coarse)

        y = skips.pop()
        for si, stage in enumerate(self.decoder):
            skip = skips.pop()
            z = conv(stage.reduce_ch, y)
            y = g8.upsample_const_forward(aprs, z, level_deltas)
            level_deltas -= 1
            # (the mean tree of the upsampled tensor is read off z: it holds what its nodes were upsampled from)
            blocks = stage.conv.blocks
            last = blocks[-1]
            fuse_head = si == len(self.decoder) - 1 and tuple(last.conv.weight.shape[3:]) != (1, 1, 1) \
                and g8.head_limits_ok(last.conv.weight.shape[1], hw)
            if fuse_head and len(blocks) == 1:
                return last_conv_with_head(last, skip, y, z)
            out = conv(blocks[0], skip, y, z)
            y = skip = z = None
            for bb in blocks[1:-1] if fuse_head else blocks[1:]:
                out = conv(bb, out)
            if fuse_head:
                return last_conv_with_head(last, out)
            y = out
            del out
        return g8.conv111_forward(aprs, y, hw, level_deltas, hb, relu=False, grouped_output=False)

    def forward(self, x, aprs, level_deltas=None):
        if level_deltas is None:
            level_deltas = torch.zeros(len(aprs), dtype=torch.int32, device=torch.device("cpu"))
        if self._grouped_ok(x, aprs):
            from pyapr.aprnet._ops import UnsupportedError
            saved = level_deltas.clone()
            try:
                return self._forward_grouped(x, aprs, level_deltas)
            except UnsupportedError:
                # a limit of the grouped kernels that _grouped_ok cannot see (the plan's window lists could not be
                # built, or were switched off): the plane operators compute the same network
                level_deltas.copy_(saved)
        skips = [self.encoder[0](x, aprs, level_deltas)]
        for stage in self.encoder[1:]:
            skips.append(stage(skips[-1], aprs, level_deltas))
        # every skip tensor is dropped as soon as its decoder stage has read it: at inference the peak working set is
        # then one stage's inputs and output, not the whole encoder
        y = skips.pop()
        for stage in self.decoder:
            skip = skips.pop()
            if torch.is_grad_enabled():
                y = stage(y, skip, aprs, level_deltas)
            else:
                # UpConv.forward (unet_parts.py:78-83) unrolled here, so that the skip tensor and the upsampled tensor
                # are released as soon as the first convolution of the stage has read them (inside stage.forward the
                # caller's references would keep both alive until the whole stage returns)
                y = stage.upsample(stage.reduce_ch(y, aprs, level_deltas), aprs, level_deltas)
                blocks = stage.conv.blocks
                out = blocks[0](skip, aprs, level_deltas, y)
                y = None
                skip = None
                for block in blocks[1:]:
                    out = block(out, aprs, level_deltas)
                y = out
                del out
            del skip
        return self.head(y, aprs, level_deltas)


@torch.no_grad()
def fold_norms(model):
    """Inference-time folding of BatchNorm1d (running statistics) into the preceding bias-free APRConv:
    w' = w * gamma / sqrt(var + eps) per output channel, bias' = beta - mean * gamma / sqrt(var + eps).
    The conv gains a bias parameter and the norm becomes nn.Identity.  GroupNorm depends on the input
    and cannot be folded; models meant for folded inference are built with norm='batch'."""
    from .hybrid_unet_parts import PixelBasicBlock
    for m in model.modules():
        if isinstance(m, PixelBasicBlock) and isinstance(m.norm, nn.BatchNorm3d):      # dense stages of the hybrid net
            bn, conv = m.norm, m.conv
            scale = bn.weight / torch.sqrt(bn.running_var + bn.eps)
            conv.weight.mul_(scale.view(-1, 1, 1, 1, 1))                               # [Cout, Cin, kz, kx, ky]
            conv.bias = nn.Parameter((bn.bias - bn.running_mean * scale).clone())
            m.norm = nn.Identity()
        if isinstance(m, BasicBlock) and isinstance(m.norm, nn.BatchNorm1d):
            bn, conv = m.norm, m.conv
            scale = bn.weight / torch.sqrt(bn.running_var + bn.eps)
            conv.weight.mul_(scale.view(1, -1, 1, 1, 1, 1))        # device layout [S, Cout, Cin, kz, kx, ky]
            conv.bias = nn.Parameter((bn.bias - bn.running_mean * scale).clone())
            m.norm = nn.Identity()
    return model
