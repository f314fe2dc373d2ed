"""TEST INFRASTRUCTURE ONLY: CPU statement, in float64 numpy, of the centre-feature blend of a DCNv4 layer
(DCNv4_op/DCNv4/modules/dcnv4.py:17-26 CenterFeatureScaleModule, :142-147): ``gate = sigmoid(y W^T + b)`` per
(pixel, group), ``out = y * (1 - gate) + x * gate`` with every channel using its group's gate.  Pinned in
tests/test_oracle_pins.py against the reference's own torch expression (linear, sigmoid, repeat, blend), torch autograd
through it, and finite differences.
"""
import numpy as np


def _gates(y, weight, bias):
    z = y @ np.asarray(weight, dtype=np.float64).T + np.asarray(bias, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-z))


def blend_forward(y, x, weight, bias):
    """y, x (..., C); weight (G, C); bias (G,) -> (..., C)."""
    y, x = np.asarray(y, dtype=np.float64), np.asarray(x, dtype=np.float64)
    groups = np.asarray(bias).shape[0]
    s = np.repeat(_gates(y, weight, bias), y.shape[-1] // groups, axis=-1)       # dcnv4.py:145-146
    return y * (1 - s) + x * s


def blend_backward(grad_out, y, x, weight, bias):
    """(grad_y, grad_x, grad_weight, grad_bias, grad_gate_logits) for ``grad_out``."""
    q, y, x = (np.asarray(t, dtype=np.float64) for t in (grad_out, y, x))
    w = np.asarray(weight, dtype=np.float64)
    groups, channels = w.shape
    width = channels // groups
    s = _gates(y, w, bias)
    s_full = np.repeat(s, width, axis=-1)
    d_gate = (q * (x - y)).reshape(*y.shape[:-1], groups, width).sum(axis=-1)
    d_logit = d_gate * s * (1 - s)
    grad_y = q * (1 - s_full) + d_logit @ w
    grad_x = q * s_full
    dl2, y2 = d_logit.reshape(-1, groups), y.reshape(-1, channels)
    return grad_y, grad_x, dl2.T @ y2, dl2.sum(axis=0), d_logit
