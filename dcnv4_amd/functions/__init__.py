from .dcnv4_func import DCNv4Function
from .depthwise_conv_func import DepthwiseConvNHWCFunction
from .flash_deform_attn_func import FlashDeformAttnFunction

__all__ = ["DCNv4Function", "DepthwiseConvNHWCFunction", "FlashDeformAttnFunction"]
