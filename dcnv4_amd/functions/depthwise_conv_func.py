"""``DepthwiseConvNHWCFunction``: autograd wrapper of the channels-last depthwise convolution that a
DCNv4 block applies before its offset/mask projection (``offset_mask_dw``,
DCNv4_op/DCNv4/modules/dcnv4.py:67-75,121-123).  The reference permutes NHWC -> NCHW, calls
nn.Conv2d and permutes back; this operator reads and writes NHWC.
"""
import torch
from torch.amp import custom_bwd, custom_fwd
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import ext


class DepthwiseConvNHWCFunction(Function):
    """forward(input (N,H,W,C), weight (C,1,k,k), bias (C,) or None, pad) -> (N,Ho,Wo,C)."""

    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, input, weight, bias, pad):
        # under autocast the convolution runs in the autocast dtype, like nn.Conv2d; otherwise in the
        # dtype of the activations
        if torch.is_autocast_enabled():
            dtype = torch.get_autocast_dtype("cuda")
            input = input.to(dtype)
        else:
            dtype = input.dtype
        w = weight.to(dtype).contiguous()
        b = bias.to(dtype).contiguous() if bias is not None else None
        input = input.contiguous()
        ctx.pad = pad
        ctx.has_bias = bias is not None
        ctx.param_dtypes = (weight.dtype, bias.dtype if bias is not None else None)
        ctx.save_for_backward(input, w)
        return ext.depthwise_conv_forward(input, w, b, pad)

    @staticmethod
    @once_differentiable
    @custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        input, w = ctx.saved_tensors
        need_in, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1] or (ctx.has_bias and ctx.needs_input_grad[2])
        gi, gw, gb = ext.depthwise_conv_backward(input, w, grad_output.contiguous().to(input.dtype), ctx.pad,
                                                 ctx.has_bias, need_in, need_w)
        wdt, bdt = ctx.param_dtypes
        if gw is not None:
            gw = gw.to(wdt)
        if gb is not None:
            gb = gb.to(bdt)
        return gi, gw, gb, None
