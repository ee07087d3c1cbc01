"""``pyapr.aprnet.cuda`` (pyapr/aprnet/cuda/__init__.py:1-5): the flavour `apr_models` imports.
Weights are stored as [S, Cout, Cin, kz, kx, ky]; MaxPool leaves zeros behind the last particle of a
batch item (wrap_maxpool_gpu.hpp:42).  Unlike the reference's CUDA flavour, every stencil of the CPU
flavour (1x3x3, 1x5x5, 5x5x5) is available here too."""
from ..functional import CUDA_LAYOUT
from ..modules import APRConv as _APRConv, MaxPool as _MaxPool, UpSampleConst, Reconstruct, SampleParticles


class APRConv(_APRConv):
    weight_layout = CUDA_LAYOUT


class MaxPool(_MaxPool):
    pad_value = 0.0


__all__ = ["APRConv", "MaxPool", "UpSampleConst", "Reconstruct", "SampleParticles"]
