from .unet_model import APRUNet, fold_norms
from .unet_parts import BasicBlock, ConvBlock, DownConv, UpConv

__all__ = ["APRUNet", "fold_norms", "BasicBlock", "ConvBlock", "DownConv", "UpConv"]
