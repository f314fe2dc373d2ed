"""Centre-feature blend of a DCNv4 layer (DCNv4_op/DCNv4/modules/dcnv4.py:17-26,142-147): a per-(pixel, group) gate
``s = sigmoid(W y + b)`` computed from the sampled features ``y`` mixes them with the un-sampled projection ``x``:
``out = y * (1 - s) + x * s``, every channel using its group's gate.  Forward and backward each run as one kernel of
libdcnv4_gfx950.so; the two parameter gradients are a matrix product of the kernel's logit gradients with ``y``.
"""
import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import ext


class CenterFeatureBlendFunction(Function):
    """apply(y (..., C), x (..., C), weight (G, C), bias (G,)) -> (..., C)."""

    @staticmethod
    def forward(ctx, y, x, weight, bias):
        y, x, weight, bias = y.contiguous(), x.contiguous(), weight.contiguous(), bias.contiguous()
        dtype = y.dtype
        x, weight, bias = x.to(dtype), weight.to(dtype), bias.to(dtype)
        ctx.save_for_backward(y, x, weight, bias)
        return ext.center_feature_blend_forward(y, x, weight, bias)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        y, x, weight, bias = ctx.saved_tensors
        grad_y, grad_x, grad_logits = ext.center_feature_blend_backward(grad_out.contiguous().to(y.dtype), y, x, weight, bias)
        grad_weight = grad_bias = None
        if ctx.needs_input_grad[2]:
            grad_weight = (grad_logits.t() @ y.reshape(-1, y.shape[-1]).float()).to(weight.dtype)
        if ctx.needs_input_grad[3]:
            grad_bias = grad_logits.sum(0).to(bias.dtype)
        return grad_y, grad_x, grad_weight, grad_bias
