"""Particle-space models built on ``pyapr.aprnet.cuda`` (apr_models/apr_models/__init__.py)."""
from . import unet
from . import utils

__all__ = ["unet", "utils"]
