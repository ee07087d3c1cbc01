"""``pyapr.aprnet``: APRConv, MaxPool, UpSampleConst with the CPU-flavour parameter layout, ``utils``,
and the ``cuda`` sub-package with the device-flavour layout plus Reconstruct / SampleParticles
(pyapr/aprnet/__init__.py:1-7).  Both flavours run the same HIP kernels on GPU tensors."""
from . import utils
from .modules import APRConv, MaxPool, UpSampleConst
from . import cuda
from . import stardist_utils
from .stardist_utils import labels_to_dist, get_prob_apr, get_particle_coordinates

__all__ = ["APRConv", "MaxPool", "UpSampleConst", "utils", "cuda", "stardist_utils", "labels_to_dist", "get_prob_apr",
           "get_particle_coordinates"]
