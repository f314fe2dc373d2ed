"""TEST INFRASTRUCTURE ONLY: CPU statement of ``residual + gamma * LayerNorm(y)`` over the last axis, the tail of
a FlashInternImage block (classification/models/flash_intern_image.py:425-440 with nn.LayerNorm(eps=1e-6) from
build_norm_layer :34-55): biased variance, affine weight and bias, in float64 numpy.  Pinned in
tests/test_oracle_pins.py against torch's layer_norm and against the properties that define it (zero mean and unit
variance of the normalised rows before the affine map, invariance to a shift of the row).
"""
import numpy as np


def layer_norm_residual(y, weight, bias, eps, gamma=None, residual=None):
    y = np.asarray(y, dtype=np.float64)
    mean = y.mean(axis=-1, keepdims=True)
    var = ((y - mean) ** 2).mean(axis=-1, keepdims=True)
    out = (y - mean) / np.sqrt(var + eps) * np.asarray(weight, dtype=np.float64) + np.asarray(bias, dtype=np.float64)
    if gamma is not None:
        out = out * np.asarray(gamma, dtype=np.float64)
    if residual is not None:
        out = out + np.asarray(residual, dtype=np.float64)
    return out


def layer_norm_residual_backward(grad_out, y, weight, bias, eps, gamma=None):
    """Gradients of ``layer_norm_residual`` for ``grad_out``: (grad_y, grad_weight, grad_bias, grad_gamma or None); the
    gradient of the residual is ``grad_out`` itself.  Chain rule through out = residual + gamma * (xhat * weight + bias),
    xhat = (y - mean) / sqrt(var + eps): what autograd derives for flash_intern_image.py:425-440.  Pinned against
    torch autograd and finite differences in tests/test_oracle_pins.py."""
    g = np.asarray(grad_out, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    w = np.asarray(weight, dtype=np.float64)
    b = np.asarray(bias, dtype=np.float64)
    mean = y.mean(axis=-1, keepdims=True)
    rstd = 1.0 / np.sqrt(((y - mean) ** 2).mean(axis=-1, keepdims=True) + eps)
    xhat = (y - mean) * rstd
    gg = g if gamma is None else g * np.asarray(gamma, dtype=np.float64)       # gradient of the normalisation's output
    a = gg * w
    grad_y = rstd * (a - a.mean(axis=-1, keepdims=True) - xhat * (a * xhat).mean(axis=-1, keepdims=True))
    flat = lambda t: t.reshape(-1, t.shape[-1]).sum(axis=0)
    grad_gamma = None if gamma is None else flat(g * (xhat * w + b))
    return grad_y, flat(gg * xhat), flat(gg), grad_gamma
