"""Launch specs for gfx950, the counterpart of the reference's ``findspec`` / ``find_spec_bwd``
(DCNv4_op/DCNv4/functions/dcnv4_func.py:21-60, flash_deform_attn_func.py:38-67) and of its
NVIDIA-tuned ``table.py``.

A spec is ``(d_stride, n_thread)``: channels per lane and lanes per workgroup.  On gfx950 a lane
always moves 16 bytes when the group width allows it, and a workgroup is sized to roughly 256
lanes made of whole pixels; both follow in O(1) from (G, C, element size), and the answer is
memoised per shape, so a call costs one dictionary look-up (the reference scans the factors of
B*H*W on every call).

Measured overrides live in ``gfx950_table.json`` next to this file, written by ``python -m dcnv4_amd.tune``
(the counterpart of DCNv4_op/scripts/search_dcnv4.py, search_dcnv4_bwd.py and find_best.py).  Its keys are the
reference's ``"BxHxWxGxC"`` plus the element size and the direction; an entry holds the two hints and, optionally,
launch options (``gather`` = tiled / direct, ``tile`` = 8 / 16 / 32, ``reach`` = pixels, ``gather_tile`` = 4 / 8 / 16;
for the attention operator ``fda_order`` = rows / heads and ``scatter`` = tiled / atomic), which
:func:`launch_options_for` hands to the library as thread-local launch options around the call.  Attention keys are
``"attn:BxQxGxC:LxK"`` plus element size and direction.
"""
import functools
import json
import os

TABLE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gfx950_table.json")

_TARGET_LANES = 256


def _load_table(path=TABLE_PATH):
    if not os.path.exists(path):
        return {}
    with open(path) as f:
        return json.load(f).get("entries", {})


# key -> {"d_stride": int, "n_thread": int, and optionally "gather": str, "tile": int, "reach": int}
OPTION_KEYS = ("gather", "scatter", "tile", "reach", "gather_tile", "gv_threads", "dual", "fda_order", "fda_stage")
GFX950_TABLE = _load_table()


def table_key(B, H, W, G, C, elem_bytes, direction):
    """``C`` is the number of channels per group, as in the reference's table keys ("64x56x56x4x16")."""
    return f"{B}x{H}x{W}x{G}x{C}:{elem_bytes}:{direction}"


def _vector_channels(group_channels, elem_bytes):
    cpt = 1
    while cpt * 2 * elem_bytes <= 16 and group_channels % (cpt * 2) == 0:
        cpt *= 2
    return cpt


def _spec(group, group_channels, elem_bytes, scatter=False):
    # forward and backward gather with 16-byte lanes (grad_value is a gather too); `scatter` is kept for callers that
    # name the direction
    d_stride = _vector_channels(group_channels, elem_bytes)
    lanes_per_group = 1
    while lanes_per_group < group_channels // d_stride:
        lanes_per_group *= 2
    lanes_per_pixel = group * lanes_per_group
    pixels = max(1, _TARGET_LANES // lanes_per_pixel)
    return d_stride, pixels * lanes_per_pixel


@functools.lru_cache(maxsize=None)
def _lookup(B, H, W, G, C, elem_bytes, direction):
    entry = GFX950_TABLE.get(table_key(B, H, W, G, C, elem_bytes, direction))
    if entry is not None:
        options = {k: entry[k] for k in OPTION_KEYS if entry.get(k, "auto") not in ("auto", None)}
        return (int(entry["d_stride"]), int(entry["n_thread"])), options
    return _spec(G, C, elem_bytes, scatter=direction == "bwd"), {}


def findspec(B, H, W, G, C, elem_bytes=2):
    return _lookup(B, H, W, G, C, elem_bytes, "fwd")[0]


def find_spec_bwd(B, H, W, G, C, elem_bytes=2):
    return _lookup(B, H, W, G, C, elem_bytes, "bwd")[0]


def launch_options_for(B, H, W, G, C, elem_bytes, direction):
    """Kernel-family options a table entry asks for ({} for shapes without an entry: the library chooses)."""
    return _lookup(B, H, W, G, C, elem_bytes, direction)[1]


def findspec_attn(B, Q, G, C, elem_bytes=2):
    return _spec(G, C, elem_bytes)


def findspec_attn_bwd(B, Q, G, C, elem_bytes=2):
    return _spec(G, C, elem_bytes, scatter=True)


def attn_table_key(B, Q, G, C, L, K, elem_bytes, direction):
    return f"attn:{B}x{Q}x{G}x{C}:{L}x{K}:{elem_bytes}:{direction}"


@functools.lru_cache(maxsize=None)
def attn_launch_options_for(B, Q, G, C, L, K, elem_bytes, direction):
    """Options a table entry asks for around a flash-deformable-attention call ({}: the library chooses)."""
    entry = GFX950_TABLE.get(attn_table_key(B, Q, G, C, L, K, elem_bytes, direction))
    if entry is None:
        return {}
    return {k: entry[k] for k in OPTION_KEYS if entry.get(k, "auto") not in ("auto", None)}
