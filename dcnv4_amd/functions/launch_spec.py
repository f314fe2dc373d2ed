"""Launch hints for gfx950, the counterpart of the reference's ``findspec`` / ``find_spec_bwd``
(DCNv4_op/DCNv4/functions/dcnv4_func.py:21-60, flash_deform_attn_func.py:38-67) and of its
NVIDIA-tuned ``table.py``.

A spec is ``(d_stride, n_thread)``: channels per lane and lanes per workgroup.  On gfx950 a lane
always moves 16 bytes when the group width allows it, and a workgroup is sized to roughly 256
lanes made of whole pixels; both follow in O(1) from (G, C, element size), so there is no factor
scan over B*H*W and nothing to memoise.  ``GFX950_TABLE`` holds measured overrides keyed like the
reference's table (``"BxHxWxGxC"``); entries are optional.
"""

GFX950_TABLE = {}
GFX950_BWD_TABLE = {}

_TARGET_LANES = 256


def _vector_channels(group_channels, elem_bytes):
    cpt = 1
    while cpt * 2 * elem_bytes <= 16 and group_channels % (cpt * 2) == 0:
        cpt *= 2
    return cpt


def _spec(group, group_channels, elem_bytes, scatter=False):
    # backward scatters with one channel per lane (contiguous dwords per atomic instruction)
    d_stride = 1 if scatter and group_channels <= 64 else _vector_channels(group_channels, elem_bytes)
    lanes_per_group = 1
    while lanes_per_group < group_channels // d_stride:
        lanes_per_group *= 2
    lanes_per_pixel = group * lanes_per_group
    pixels = max(1, _TARGET_LANES // lanes_per_pixel)
    return d_stride, pixels * lanes_per_pixel


def findspec(B, H, W, G, C, elem_bytes=2):
    key = f"{B}x{H}x{W}x{G}x{C}"
    if key in GFX950_TABLE:
        return GFX950_TABLE[key][0], GFX950_TABLE[key][1]
    return _spec(G, C, elem_bytes)


def find_spec_bwd(B, H, W, G, C, elem_bytes=2):
    key = f"{B}x{H}x{W}x{G}x{C}"
    if key in GFX950_BWD_TABLE:
        return GFX950_BWD_TABLE[key][0], GFX950_BWD_TABLE[key][1]
    return _spec(G, C, elem_bytes, scatter=True)


def findspec_attn(B, Q, G, C, elem_bytes=2):
    return _spec(G, C, elem_bytes)


def findspec_attn_bwd(B, Q, G, C, elem_bytes=2):
    return _spec(G, C, elem_bytes, scatter=True)
