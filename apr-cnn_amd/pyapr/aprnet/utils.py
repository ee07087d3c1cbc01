"""``aprnet.utils``: particle-count helpers (pyapr/aprnet/src/utils.hpp:336-384)."""
from ._ops import (number_particles, number_parts, number_particles_after_pooling,
                   number_particles_after_upsampling)

__all__ = ["number_particles", "number_parts", "number_particles_after_pooling",
           "number_particles_after_upsampling"]
