"""TEST INFRASTRUCTURE ONLY: CPU statement of the channels-last depthwise convolution that a DCNv4
block applies before its offset/mask projection, and of its gradients.

The reference builds the layer as ``nn.Conv2d(C, C, k, stride=1, padding=(k-1)//2, groups=C)``
(DCNv4_op/DCNv4/modules/dcnv4.py:67-75) and calls it between two permutes (dcnv4.py:121-123), so the
mathematics is PyTorch's cross-correlation:

    out[b,y,x,c] = bias[c] + sum_{i,j} weight[c,i,j] * input[b, y+i-pad, x+j-pad, c]   (zero outside)

Written here as k*k shifted slices of the zero-padded input in float64 numpy.  Pinned in
tests/test_oracle_pins.py against torch's own conv2d and autograd and against closed forms (a one-hot
kernel is a shifted copy, an all-ones kernel a box sum).
"""
import numpy as np


def _f64(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float64))


def depthwise_forward(inp, weight, bias, pad):
    """inp (N,H,W,C), weight (C,k,k) or (C,1,k,k), bias (C,) or None -> (N,Ho,Wo,C) float64."""
    x, w = _f64(inp), _f64(weight)
    N, H, W, C = x.shape
    k = w.shape[-1]
    w = w.reshape(C, k, k)
    Ho, Wo = H + 2 * pad - k + 1, W + 2 * pad - k + 1
    xp = np.pad(x, ((0, 0), (pad, pad), (pad, pad), (0, 0)))
    out = np.zeros((N, Ho, Wo, C))
    for i in range(k):
        for j in range(k):
            out += xp[:, i:i + Ho, j:j + Wo, :] * w[:, i, j]
    if bias is not None:
        out += _f64(bias)
    return out


def depthwise_backward(inp, weight, grad_out, pad):
    """-> grad_input (N,H,W,C), grad_weight (C,k,k), grad_bias (C,), all float64."""
    x, w, go = _f64(inp), _f64(weight), _f64(grad_out)
    N, H, W, C = x.shape
    k = w.shape[-1]
    w = w.reshape(C, k, k)
    Ho, Wo = go.shape[1], go.shape[2]
    xp = np.pad(x, ((0, 0), (pad, pad), (pad, pad), (0, 0)))
    gxp = np.zeros_like(xp)
    gw = np.zeros((C, k, k))
    for i in range(k):
        for j in range(k):
            gxp[:, i:i + Ho, j:j + Wo, :] += go * w[:, i, j]
            gw[:, i, j] = (go * xp[:, i:i + Ho, j:j + Wo, :]).sum(axis=(0, 1, 2))
    gx = gxp[:, pad:pad + H, pad:pad + W, :]
    return np.ascontiguousarray(gx), gw, go.sum(axis=(0, 1, 2))
