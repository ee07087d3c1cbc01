"""MI355X-native counterpart of the ``pyapr`` modules that APR-CNN's network operators need:
``pyapr.aprnet`` (+ ``pyapr.aprnet.cuda``), the ``APR`` container and an image -> APR converter."""
from .data_containers import APR, APRParameters, LinearIterator, APRPtrVector
from . import converter
from . import synthetic
from . import io

__all__ = ["APR", "APRParameters", "LinearIterator", "APRPtrVector", "converter", "synthetic", "io", "aprnet"]


def __getattr__(name):
    if name == "aprnet":
        import importlib
        return importlib.import_module(".aprnet", __name__)
    raise AttributeError(name)
