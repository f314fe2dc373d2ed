"""Test-side helpers that call libdcnv4_gfx950.so through its C ABI with torch tensors as device memory,
and run the CPU oracle on the same bits."""
import numpy as np
import torch

from dcnv4_amd import _lib

CODES = {torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def dcn_out_hw(H, W, kh, kw, sh, sw, ph, pw, dh, dw):
    return ((H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1, (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1)


def dcnv4_forward(value, om, geom, G, D, scale, rc=0, softmax=0, im2col_step=256, d_stride=0, block_thread=0):
    L = _lib.load()
    B, H, W, _ = value.shape
    Ho, Wo = dcn_out_hw(H, W, *geom)
    out = torch.full((B, Ho, Wo, G * D), float("nan"), dtype=value.dtype, device=value.device)
    rc_ = L.dcnv4_gfx950_forward(value.data_ptr(), om.data_ptr(), out.data_ptr(), CODES[value.dtype], B, H, W, G, D,
                                 *geom, float(scale), im2col_step, rc, om.shape[-1], softmax, d_stride, block_thread,
                                 _stream())
    _lib.check(rc_)
    return out


def dcnv4_backward(value, om, go, geom, G, D, scale, rc=0, softmax=0, im2col_step=256, d_stride=0, block_thread=0):
    L = _lib.load()
    B, H, W, _ = value.shape
    gv = torch.full_like(value, float("nan"))
    gom = torch.full_like(om, float("nan"))
    nbytes = L.dcnv4_gfx950_backward_workspace_bytes(CODES[value.dtype], B, H, W, G, D)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=value.device)
    rc_ = L.dcnv4_gfx950_backward(value.data_ptr(), om.data_ptr(), go.data_ptr(), gv.data_ptr(), gom.data_ptr(),
                                  ws.data_ptr(), nbytes, CODES[value.dtype], B, H, W, G, D, *geom, float(scale),
                                  im2col_step, rc, om.shape[-1], softmax, d_stride, block_thread, _stream())
    _lib.check(rc_)
    return gv, gom


def fda_forward(value, shapes, starts, sla, K, im2col_step=64, d_stride=0, block_thread=0):
    L = _lib.load()
    B, N, G, D = value.shape
    Q = sla.shape[1]
    out = torch.full((B, Q, G * D), float("nan"), dtype=value.dtype, device=value.device)
    rc_ = L.flash_deform_attn_gfx950_forward(value.data_ptr(), shapes.data_ptr(), starts.data_ptr(), sla.data_ptr(),
                                             out.data_ptr(), CODES[value.dtype], B, N, G, D, shapes.shape[0], Q, K,
                                             im2col_step, d_stride, block_thread, _stream())
    _lib.check(rc_)
    return out


def fda_backward(value, shapes, starts, sla, go, K, im2col_step=64, d_stride=0, block_thread=0):
    L = _lib.load()
    B, N, G, D = value.shape
    Q = sla.shape[1]
    gv = torch.full_like(value, float("nan"))
    gs = torch.full_like(sla, float("nan"))
    nbytes = L.flash_deform_attn_gfx950_backward_workspace_bytes(CODES[value.dtype], B, N, G, D, shapes.shape[0], Q, K)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=value.device)
    rc_ = L.flash_deform_attn_gfx950_backward(value.data_ptr(), shapes.data_ptr(), starts.data_ptr(), sla.data_ptr(),
                                              go.data_ptr(), gv.data_ptr(), gs.data_ptr(), ws.data_ptr(), nbytes,
                                              CODES[value.dtype], B, N, G, D, shapes.shape[0], Q, K, im2col_step,
                                              d_stride, block_thread, _stream())
    _lib.check(rc_)
    return gv, gs


def f64(t):
    """Exact widening of a (possibly half-precision) tensor to a float64 numpy array."""
    return t.detach().cpu().to(torch.float64).numpy()


def assert_close(got, want, rtol, atol, what=""):
    got = f64(got) if isinstance(got, torch.Tensor) else got
    assert np.isfinite(got).all(), f"{what}: non-finite values (unwritten output?)"
    err = np.abs(got - want)
    tol = atol + rtol * np.abs(want)
    bad = err > tol
    if bad.any():
        i = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} / {bad.size} elements off; worst at {i}: got {got[i]!r} want {want[i]!r} "
                             f"(rtol {rtol}, atol {atol})")


def depthwise_forward(inp, weight, bias, pad):
    """inp (N,H,W,C), weight (C,k,k), bias (C,) or None, all on the GPU in one dtype."""
    L = _lib.load()
    B, H, W, C = inp.shape
    k = weight.shape[-1]
    out = torch.full((B, H + 2 * pad - k + 1, W + 2 * pad - k + 1, C), float("nan"), dtype=inp.dtype, device=inp.device)
    _lib.check(L.dcnv4_gfx950_depthwise_conv_forward(inp.data_ptr(), weight.data_ptr(),
                                                      bias.data_ptr() if bias is not None else None, out.data_ptr(),
                                                      CODES[inp.dtype], B, H, W, C, k, pad, _stream()))
    return out


def depthwise_backward(inp, weight, go, pad, with_bias=True):
    L = _lib.load()
    B, H, W, C = inp.shape
    k = weight.shape[-1]
    gi = torch.full_like(inp, float("nan"))
    gw = torch.full_like(weight, float("nan"))
    gb = torch.full((C,), float("nan"), dtype=inp.dtype, device=inp.device) if with_bias else None
    nbytes = L.dcnv4_gfx950_depthwise_conv_backward_workspace_bytes(CODES[inp.dtype], B, H, W, C, k, pad)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=inp.device)
    _lib.check(L.dcnv4_gfx950_depthwise_conv_backward(inp.data_ptr(), weight.data_ptr(), go.data_ptr(), gi.data_ptr(),
                                                       gw.data_ptr(), gb.data_ptr() if gb is not None else None,
                                                       ws.data_ptr(), nbytes, CODES[inp.dtype], B, H, W, C, k, pad,
                                                       _stream()))
    return gi, gw, gb


def layer_norm_residual(y, residual, weight, bias, gamma, eps):
    L = _lib.load()
    out = torch.full_like(y, float("nan"))
    C = y.shape[-1]
    _lib.check(L.dcnv4_gfx950_layer_norm_residual_forward(
        y.data_ptr(), residual.data_ptr() if residual is not None else None, weight.data_ptr(), bias.data_ptr(),
        gamma.data_ptr() if gamma is not None else None, out.data_ptr(), CODES[y.dtype], y.numel() // C, C, float(eps), _stream()))
    return out


def dcnv4_backward_static_scratch(value, om, go, geom, G, D, scale, rc=0, softmax=0, im2col_step=256, out=None):
    """The allocation-free entry point: no workspace argument, scratch inside the library.  `out` = (grad_value,
    grad_offset_mask) tensors that exist already; without it they are created here."""
    L = _lib.load()
    B, H, W, _ = value.shape
    gv, gom = out if out is not None else (torch.full_like(value, float("nan")), torch.full_like(om, float("nan")))
    rc_ = L.dcnv4_gfx950_backward_static_scratch(value.data_ptr(), om.data_ptr(), go.data_ptr(), gv.data_ptr(), gom.data_ptr(),
                                                 CODES[value.dtype], B, H, W, G, D, *geom, float(scale), im2col_step, rc,
                                                 om.shape[-1], softmax, 0, 0, _stream())
    _lib.check(rc_)
    return gv, gom


def layer_norm_residual_backward(go, y, weight, bias, gamma, eps, want_params=True):
    L = _lib.load()
    C = y.shape[-1]
    rows = y.numel() // C
    gy = torch.full_like(y, float("nan"))
    new = lambda: torch.full((C,), float("nan"), dtype=y.dtype, device=y.device)
    gw, gb = (new(), new()) if want_params else (None, None)
    gg = new() if (want_params and gamma is not None) else None
    nbytes = L.dcnv4_gfx950_layer_norm_residual_backward_workspace_bytes(CODES[y.dtype], rows, C)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=y.device)
    ptr = lambda t: t.data_ptr() if t is not None else None
    _lib.check(L.dcnv4_gfx950_layer_norm_residual_backward(go.data_ptr(), y.data_ptr(), weight.data_ptr(), ptr(bias), ptr(gamma),
                                                            gy.data_ptr(), ptr(gw), ptr(gb), ptr(gg), ws.data_ptr(), nbytes,
                                                            CODES[y.dtype], rows, C, float(eps), _stream()))
    return gy, gw, gb, gg


def center_feature_blend_forward(y, x, weight, bias):
    L = _lib.load()
    C = y.shape[-1]
    out = torch.full_like(y, float("nan"))
    _lib.check(L.dcnv4_gfx950_center_feature_blend_forward(y.data_ptr(), x.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                                            out.data_ptr(), CODES[y.dtype], y.numel() // C, C, bias.numel(), _stream()))
    return out


def center_feature_blend_backward(go, y, x, weight, bias):
    L = _lib.load()
    C = y.shape[-1]
    rows = y.numel() // C
    gy, gx = torch.full_like(y, float("nan")), torch.full_like(y, float("nan"))
    gl = torch.full((rows, bias.numel()), float("nan"), dtype=torch.float32, device=y.device)
    _lib.check(L.dcnv4_gfx950_center_feature_blend_backward(go.data_ptr(), y.data_ptr(), x.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                                                             gy.data_ptr(), gx.data_ptr(), gl.data_ptr(), CODES[y.dtype], rows, C,
                                                             bias.numel(), _stream()))
    return gy, gx, gl


def fda_forward_split(value, shapes, starts, loc, logits, K, im2col_step=64):
    L = _lib.load()
    B, N, G, D = value.shape
    Q = logits.shape[1]
    out = torch.full((B, Q, G * D), float("nan"), dtype=value.dtype, device=value.device)
    _lib.check(L.flash_deform_attn_gfx950_forward_split(value.data_ptr(), shapes.data_ptr(), starts.data_ptr(), loc.data_ptr(),
                                                         logits.data_ptr(), out.data_ptr(), CODES[value.dtype], CODES[loc.dtype], B, N,
                                                         G, D, shapes.shape[0], Q, K, im2col_step, 0, 0, _stream()))
    return out


def fda_backward_split(value, shapes, starts, loc, logits, go, K, im2col_step=64):
    L = _lib.load()
    B, N, G, D = value.shape
    Q = logits.shape[1]
    gv = torch.full_like(value, float("nan"))
    gloc = torch.full_like(loc, float("nan"))
    glog = torch.full_like(logits, float("nan"))
    nbytes = L.flash_deform_attn_gfx950_backward_workspace_bytes(CODES[value.dtype], B, N, G, D, shapes.shape[0], Q, K)
    ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=value.device)
    _lib.check(L.flash_deform_attn_gfx950_backward_split(value.data_ptr(), shapes.data_ptr(), starts.data_ptr(), loc.data_ptr(),
                                                          logits.data_ptr(), go.data_ptr(), gv.data_ptr(), gloc.data_ptr(),
                                                          glog.data_ptr(), ws.data_ptr(), nbytes, CODES[value.dtype], CODES[loc.dtype],
                                                          B, N, G, D, shapes.shape[0], Q, K, im2col_step, 0, 0, _stream()))
    return gv, gloc, glog
