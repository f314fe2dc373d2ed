"""TEST INFRASTRUCTURE ONLY: numpy/ctypes front end of oracle/sampling_oracle.c.

``coord_f32=True`` rounds the sampling-coordinate arithmetic to fp32 the way the reference's
kernels do for fp32/fp16/bf16 tensors (the mode GPU parity tests use); the default keeps
everything in float64 (the mode the mathematical pins use).

Every function takes and returns float64 numpy arrays in the operators' own
layouts (NHWC value, packed offset_mask, packed sampling_loc_attn) and follows the
reference's host wrappers for shapes: DCNv4_op/src/cuda/dcnv4_cuda.cu:26-175,
DCNv4_op/src/cuda/flash_deform_attn_cuda.cu:26-163.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libsampling_oracle.so")
_lib = None

_dp = ctypes.POINTER(ctypes.c_double)
_ip = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    src = os.path.join(_HERE, "sampling_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libsampling_oracle.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        i, d = ctypes.c_int, ctypes.c_double
        dcn_tail = [i] * 13 + [d, i, i, i, i]
        _lib.oracle_dcnv4_forward.argtypes = [_dp, _dp, _dp] + dcn_tail
        _lib.oracle_dcnv4_backward.argtypes = [_dp, _dp, _dp, _dp, _dp] + dcn_tail
        _lib.oracle_flash_deform_attn_forward.argtypes = [_dp, _ip, _ip, _dp, _dp] + [i] * 8
        _lib.oracle_flash_deform_attn_backward.argtypes = [_dp, _ip, _ip, _dp, _dp, _dp, _dp] + [i] * 8
        _lib.oracle_out_extent.argtypes = [i] * 5
        _lib.oracle_out_extent.restype = i
        for f in (_lib.oracle_dcnv4_forward, _lib.oracle_dcnv4_backward,
                  _lib.oracle_flash_deform_attn_forward, _lib.oracle_flash_deform_attn_backward):
            f.restype = None
    return _lib


def _f64(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.float64))


def _i64(a):
    return np.ascontiguousarray(np.asarray(a, dtype=np.int64))


def _p(a):
    return a.ctypes.data_as(_dp if a.dtype == np.float64 else _ip)


def out_hw(H, W, kh, kw, sh, sw, ph, pw, dh, dw):
    L = lib()
    return L.oracle_out_extent(H, ph, dh, kh, sh), L.oracle_out_extent(W, pw, dw, kw, sw)


def _dcn_check(value, offset_mask, kh, kw, sh, sw, ph, pw, dh, dw, group, group_channels, remove_center):
    B, H, W, C = value.shape
    if C != group * group_channels:
        raise ValueError("channels != group * group_channels")
    Ho, Wo = out_hw(H, W, kh, kw, sh, sw, ph, pw, dh, dw)
    Kp = kh * kw - int(bool(remove_center))
    P_pad = offset_mask.shape[-1]
    if offset_mask.shape[:3] != (B, Ho, Wo) or P_pad < group * 3 * Kp or Kp > 64:
        raise ValueError(f"offset_mask shape {offset_mask.shape} does not fit (B,Ho,Wo,>=G*3K)=({B},{Ho},{Wo},{group*3*Kp})")
    return B, H, W, Ho, Wo, P_pad


def dcnv4_forward(value, offset_mask, kh, kw, sh, sw, ph, pw, dh, dw, group, group_channels,
                  offset_scale, remove_center=0, softmax=False, coord_f32=False):
    value, offset_mask = _f64(value), _f64(offset_mask)
    B, H, W, Ho, Wo, P_pad = _dcn_check(value, offset_mask, kh, kw, sh, sw, ph, pw, dh, dw, group,
                                        group_channels, remove_center)
    out = np.empty((B, Ho, Wo, group * group_channels), dtype=np.float64)
    lib().oracle_dcnv4_forward(_p(value), _p(offset_mask), _p(out), B, H, W, group, group_channels,
                               kh, kw, sh, sw, ph, pw, dh, dw, float(offset_scale),
                               int(bool(remove_center)), int(bool(softmax)), P_pad, int(bool(coord_f32)))
    return out


def dcnv4_backward(value, offset_mask, grad_out, kh, kw, sh, sw, ph, pw, dh, dw, group,
                   group_channels, offset_scale, remove_center=0, softmax=False, coord_f32=False):
    value, offset_mask, grad_out = _f64(value), _f64(offset_mask), _f64(grad_out)
    B, H, W, Ho, Wo, P_pad = _dcn_check(value, offset_mask, kh, kw, sh, sw, ph, pw, dh, dw, group,
                                        group_channels, remove_center)
    if grad_out.shape != (B, Ho, Wo, group * group_channels):
        raise ValueError("grad_out shape")
    gv, gom = np.empty_like(value), np.empty_like(offset_mask)
    lib().oracle_dcnv4_backward(_p(value), _p(offset_mask), _p(grad_out), _p(gv), _p(gom), B, H, W,
                                group, group_channels, kh, kw, sh, sw, ph, pw, dh, dw,
                                float(offset_scale), int(bool(remove_center)), int(bool(softmax)), P_pad, int(bool(coord_f32)))
    return gv, gom


def _fda_check(value, shapes, level_start, sla, K):
    B, N, G, D = value.shape
    L = shapes.shape[0]
    Q = sla.shape[1]
    if sla.shape != (B, Q, G, L * K * 3) or L * K > 64:
        raise ValueError(f"sampling_loc_attn shape {sla.shape} != {(B, Q, G, L * K * 3)}")
    if int((shapes[:, 0] * shapes[:, 1]).sum()) != N or level_start.shape != (L,):
        raise ValueError("spatial_shapes / level_start_index do not cover value")
    return B, N, G, D, L, Q


def flash_deform_attn_forward(value, shapes, level_start, sla, K, coord_f32=False):
    value, sla, shapes, level_start = _f64(value), _f64(sla), _i64(shapes), _i64(level_start)
    B, N, G, D, L, Q = _fda_check(value, shapes, level_start, sla, K)
    out = np.empty((B, Q, G * D), dtype=np.float64)
    lib().oracle_flash_deform_attn_forward(_p(value), _p(shapes), _p(level_start), _p(sla), _p(out),
                                           B, N, G, D, L, K, Q, int(bool(coord_f32)))
    return out


def flash_deform_attn_backward(value, shapes, level_start, sla, grad_out, K, coord_f32=False):
    value, sla, grad_out = _f64(value), _f64(sla), _f64(grad_out)
    shapes, level_start = _i64(shapes), _i64(level_start)
    B, N, G, D, L, Q = _fda_check(value, shapes, level_start, sla, K)
    if grad_out.size != B * Q * G * D:
        raise ValueError("grad_out shape")
    gv, gs = np.empty_like(value), np.empty_like(sla)
    lib().oracle_flash_deform_attn_backward(_p(value), _p(shapes), _p(level_start), _p(sla),
                                            _p(grad_out), _p(gv), _p(gs), B, N, G, D, L, K, Q, int(bool(coord_f32)))
    return gv, gs
