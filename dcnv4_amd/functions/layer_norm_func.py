"""``layer_norm_residual``: the tail of a FlashInternImage block, ``residual + gamma * LayerNorm(y)``
(classification/models/flash_intern_image.py:425-440), as one kernel instead of the framework's three.

Forward and backward run on the library's kernels whenever the tensors allow it (one floating dtype for activations
and parameters, contiguous, channel count a whole number of 16-byte vectors, no autocast in force); otherwise the
expression is left to torch's own operators and autograd.
"""
import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import ext

_MAX_VECTORS = 512


class LayerNormResidualFunction(Function):
    @staticmethod
    def forward(ctx, y, residual, weight, bias, gamma, eps):
        ctx.eps = eps
        ctx.has = (residual is not None, gamma is not None)
        ctx.save_for_backward(y, weight, bias, gamma if gamma is not None else weight)
        return ext.layer_norm_residual_forward(y, residual, weight, bias, gamma, eps)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        y, weight, bias, gamma = ctx.saved_tensors
        has_residual, has_gamma = ctx.has
        need_params = any(ctx.needs_input_grad[2:5])
        grad_y, grad_weight, grad_bias, grad_gamma = ext.layer_norm_residual_backward(
            grad_out.contiguous(), y, weight, bias, gamma if has_gamma else None, ctx.eps, need_params)
        return (grad_y, grad_out if has_residual else None, grad_weight, grad_bias, grad_gamma if has_gamma else None, None)


def _fusable(y, residual, weight, bias, gamma):
    if not y.is_cuda or y.dtype not in (torch.float32, torch.float16, torch.bfloat16) or torch.is_autocast_enabled():
        return False
    tensors = [t for t in (residual, weight, bias, gamma) if t is not None]
    if any(t.dtype != y.dtype or not t.is_contiguous() for t in tensors) or not y.is_contiguous():
        return False
    if residual is not None and residual.shape != y.shape:
        return False
    vec = 16 // y.element_size()
    return y.shape[-1] % vec == 0 and y.shape[-1] // vec <= _MAX_VECTORS


def layer_norm_residual(y, norm, gamma=None, residual=None):
    """``residual + gamma * norm(y)`` for an ``nn.LayerNorm`` over the last axis; ``gamma`` a per-channel tensor or None."""
    if norm.weight is None or norm.bias is None or tuple(norm.normalized_shape) != (y.shape[-1],) or \
            not _fusable(y, residual, norm.weight, norm.bias, gamma):
        out = norm(y)
        if gamma is not None:
            out = gamma * out
        return out if residual is None else residual + out
    return LayerNormResidualFunction.apply(y, residual, norm.weight, norm.bias, gamma, norm.eps)
