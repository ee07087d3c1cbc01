from .unet_model import APRUNet, fold_norms
from .unet_parts import BasicBlock, ConvBlock, DownConv, UpConv
from .hybrid_model import HybridAPRUNet
from .stardist_model import APRStardistUNet, HybridStardistUNet, OutBlock
from .hybrid_unet_parts import (PixelBasicBlock, PixelConvBlock, PixelDownConv, PixelUpConv, TransitionDownConv,
                                TransitionUpConv)

__all__ = ["APRUNet", "HybridAPRUNet", "APRStardistUNet", "HybridStardistUNet", "OutBlock", "fold_norms", "BasicBlock", "ConvBlock", "DownConv", "UpConv", "PixelBasicBlock",
           "PixelConvBlock", "PixelDownConv", "PixelUpConv", "TransitionDownConv", "TransitionUpConv"]
