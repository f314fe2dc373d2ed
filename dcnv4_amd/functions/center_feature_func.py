"""Centre-feature blend of a DCNv4 layer (DCNv4_op/DCNv4/modules/dcnv4.py:17-26,142-147): a per-(pixel, group) gate
``s = sigmoid(W y + b)`` computed from the sampled features ``y`` mixes them with the un-sampled projection ``x``:
``out = y * (1 - s) + x * s``, every channel using its group's gate.
"""
import torch
import torch.nn.functional as F


def blend_reference(y, x, weight, bias):
    """The blend composed from torch operators."""
    groups = weight.shape[0]
    gate = torch.sigmoid(F.linear(y, weight, bias))                       # (N,H,W,G)
    gate = gate.unsqueeze(-1).expand(*gate.shape, y.shape[-1] // groups).reshape(y.shape)
    return y * (1 - gate) + x * gate


class CenterFeatureBlendFunction:
    """apply(y (N,H,W,C), x (N,H,W,C), weight (G,C), bias (G,)) -> (N,H,W,C)."""

    @staticmethod
    def apply(y, x, weight, bias):
        return blend_reference(y, x, weight, bias)
