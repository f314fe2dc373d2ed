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
