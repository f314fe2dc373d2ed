from .center_feature_func import CenterFeatureBlendFunction
from .dcnv4_func import DCNv4Function
from .depthwise_conv_func import DepthwiseConvNHWCFunction
from .flash_deform_attn_func import FlashDeformAttnFunction, FlashDeformAttnSplitFunction
from .layer_norm_func import LayerNormResidualFunction, layer_norm_residual

__all__ = ["CenterFeatureBlendFunction", "DCNv4Function", "DepthwiseConvNHWCFunction", "FlashDeformAttnFunction", "FlashDeformAttnSplitFunction", "LayerNormResidualFunction",
           "layer_norm_residual"]
