"""torch.nn.BatchNorm1d and torch.nn.GroupNorm for [batch, channels, particles] GPU tensors, computed by the
library's streaming kernels, optionally with the ReLU that follows them in BasicBlock
(apr_models/unet/unet_parts.py:17-26).

Subclasses of the torch modules the reference uses: same constructor arguments, parameters, buffers and
state_dict keys, same running-statistics bookkeeping.  Tensors the kernels do not take (CPU tensors, 2-D inputs,
element types other than float32 / bfloat16) go through the torch implementation, which is what the reference
calls."""
import torch
import torch.nn as nn
import torch.nn.functional as F

from pyapr.aprnet.functional import NormFunction


def _native(x):
    return x.is_cuda and x.dim() == 3 and x.dtype in (torch.float32, torch.bfloat16) and x.numel() > 0 and x.shape[0] * x.shape[1] <= 65535


class ParticleBatchNorm(nn.BatchNorm1d):
    def forward(self, x, relu=False):
        if not _native(x):
            y = super().forward(x)
            return F.relu(y) if relu else y
        self._check_input_dim(x)
        # bookkeeping of torch.nn.modules.batchnorm._BatchNorm.forward
        factor = 0.0 if self.momentum is None else self.momentum
        if self.training and self.track_running_stats and self.num_batches_tracked is not None:
            self.num_batches_tracked.add_(1)
            factor = 1.0 / float(self.num_batches_tracked) if self.momentum is None else self.momentum
        use_batch_stats = self.training or (self.running_mean is None and self.running_var is None)
        stats = None if use_batch_stats else (self.running_mean, self.running_var)
        y, mean, var = NormFunction.apply(x, self.weight, self.bias, "batch", 1, self.eps, relu, stats)
        if self.training and self.track_running_stats and self.running_mean is not None:
            n = x.shape[0] * x.shape[2]
            with torch.no_grad():
                self.running_mean.lerp_(mean.to(self.running_mean.dtype), factor)
                self.running_var.lerp_((var * (n / max(n - 1, 1))).to(self.running_var.dtype), factor)
        return y


class ParticleGroupNorm(nn.GroupNorm):
    def forward(self, x, relu=False):
        if not _native(x):
            y = super().forward(x)
            return F.relu(y) if relu else y
        return NormFunction.apply(x, self.weight, self.bias, "group", self.num_groups, self.eps, relu, None)[0]
