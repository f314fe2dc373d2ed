"""ctypes binding of libdcnv4_gfx950.so (C ABI declared in include/dcnv4_gfx950.h).

The library is the only compute path: if it is missing the import of :mod:`dcnv4_amd.ext`
fails, there is no CPU or pure-PyTorch fallback (the reference behaves the same way:
DCNv4_op/src/dcnv4.h:35,61,82,106 raise "Not implemented on the CPU").
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libdcnv4_gfx950.so")

ABI_VERSION = 6
OK, ERR_INVALID_ARGUMENT, ERR_RUNTIME = 0, 1, 2
DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2

_vp, _i, _f, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/dcnv4_gfx950.h declaration by declaration
SIGNATURES = {
    "dcnv4_gfx950_abi_version": (_i, []),
    "dcnv4_gfx950_last_error": (ctypes.c_char_p, []),
    "dcnv4_gfx950_set_launch_option": (_i, [ctypes.c_char_p, _i]),
    "dcnv4_gfx950_get_launch_option": (_i, [ctypes.c_char_p, ctypes.POINTER(_i)]),
    "dcnv4_gfx950_forward": (_i, [_vp, _vp, _vp, _i] + [_i] * 13 + [_f] + [_i] * 6 + [_vp]),
    "dcnv4_gfx950_backward_workspace_bytes": (_sz, [_i] * 6),
    "dcnv4_gfx950_backward": (_i, [_vp] * 6 + [_sz, _i] + [_i] * 13 + [_f] + [_i] * 6 + [_vp]),
    "dcnv4_gfx950_backward_static_scratch": (_i, [_vp] * 5 + [_i] + [_i] * 13 + [_f] + [_i] * 6 + [_vp]),
    "flash_deform_attn_gfx950_forward": (_i, [_vp] * 5 + [_i] * 11 + [_vp]),
    "flash_deform_attn_gfx950_backward_workspace_bytes": (_sz, [_i] * 8),
    "flash_deform_attn_gfx950_backward": (_i, [_vp] * 8 + [_sz] + [_i] * 11 + [_vp]),
    "dcnv4_gfx950_depthwise_conv_forward": (_i, [_vp] * 4 + [_i] * 7 + [_vp]),
    "dcnv4_gfx950_depthwise_conv_backward_workspace_bytes": (_sz, [_i] * 7),
    "dcnv4_gfx950_depthwise_conv_backward": (_i, [_vp] * 7 + [_sz] + [_i] * 7 + [_vp]),
    "dcnv4_gfx950_layer_norm_residual_forward": (_i, [_vp] * 6 + [_i, ctypes.c_longlong, _i, _f, _vp]),
    "flash_deform_attn_gfx950_forward_split": (_i, [_vp] * 6 + [_i] * 12 + [_vp]),
    "flash_deform_attn_gfx950_backward_split": (_i, [_vp] * 10 + [_sz] + [_i] * 12 + [_vp]),
    "dcnv4_gfx950_layer_norm_residual_backward_workspace_bytes": (_sz, [_i, ctypes.c_longlong, _i]),
    "dcnv4_gfx950_layer_norm_residual_backward": (_i, [_vp] * 10 + [_sz, _i, ctypes.c_longlong, _i, _f, _vp]),
    "dcnv4_gfx950_center_feature_blend_forward": (_i, [_vp] * 5 + [_i, ctypes.c_longlong, _i, _i, _vp]),
    "dcnv4_gfx950_stream_copy": (_i, [_vp, _vp, _sz, _vp]),
    "dcnv4_gfx950_lds_read_probe": (_i, [_i, _i, _vp, _vp]),
    "dcnv4_gfx950_center_feature_blend_backward": (_i, [_vp] * 8 + [_i, ctypes.c_longlong, _i, _i, _vp]),
}

_lib = None


def load():
    """Loads the shared library once; raises ImportError with build instructions if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python dcnv4_amd/build.py` (or `python setup.py build_ext`) (needs hipcc, targets gfx950). "
            "dcnv4_amd has no CPU or pure-PyTorch fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = restype, argtypes
    got = lib.dcnv4_gfx950_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI version {got}, this package expects {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def check(rc):
    """Maps a status code to the exception class the reference's pybind layer would raise."""
    if rc == OK:
        return
    msg = load().dcnv4_gfx950_last_error().decode("utf-8", "replace")
    if rc == ERR_INVALID_ARGUMENT:
        raise ValueError(msg)
    raise RuntimeError(msg)
