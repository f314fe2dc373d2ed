"""Drop-in for the reference's ``DCNv4.ext`` pybind module (DCNv4_op/src/vision.cpp:14-21).

Four functions with the reference's positional signatures (DCNv4_op/src/dcnv4.h:19-107).  Each
checks its tensors the way the reference's host wrappers do (DCNv4_op/src/cuda/dcnv4_cuda.cu:34-60,
flash_deform_attn_cuda.cu:31-62), allocates the results with torch, and hands raw device pointers
plus torch's current HIP stream to the C ABI.  ``d_stride`` / ``block_thread`` are launch hints:
any value the reference accepts is accepted; results never depend on them.
"""
import torch

from . import _lib

_L = _lib.load()

_DTYPES = {torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16, torch.bfloat16: _lib.DTYPE_BF16}


def _dtype_code(t, name):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"{name}: dtype {t.dtype} is not supported on gfx950 (float32, float16, bfloat16)") from None


def _check(t, name, dtype=None):
    if not t.is_contiguous():
        raise RuntimeError(f"{name} tensor has to be contiguous")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor (Not implemented on the CPU)")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} has dtype {t.dtype}, expected {dtype}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    # the raw handle of torch's current stream on the current device (the direct binding costs a tenth of a
    # microsecond, going through the Stream object three: the small stages' calls are bound by host time)
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


class _on_device:
    """`with torch.cuda.device(d)` for the common case that d is the current device already: nothing to switch."""

    def __init__(self, device):
        self.ctx = None if device.index is None or device.index == torch.cuda.current_device() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


def _hint(v):
    # the C ABI treats 0 as "choose for me"; the reference's tables only ever pass positive values
    return int(v) if v is not None else 0


_FAMILY = {"auto": 0, "tiled": 1, "direct": 2, "atomic": 2}
_ORDER = {"auto": 0, "rows": 1, "heads": 2}


class launch_options:
    """Context manager over the calling thread's launch options (include/dcnv4_gfx950.h,
    ``dcnv4_gfx950_set_launch_option``): ``gather`` in auto / tiled / direct, ``scatter`` in auto / tiled / atomic,
    ``reach`` an int or None, ``tile`` 8 / 16 / 32 or None, ``gather_tile`` 4 / 8 / 16 or None, ``gv_threads`` 512 / 1024 or None, ``dual`` in auto / on / off, ``fda_order`` in auto / rows / heads, ``fda_stage`` in auto / on / off.  Used by the tuner,
    by dispatch-table entries that carry options and by tests that force a kernel family; on exit every option is
    back at the value it had on entry, so contexts nest.  Results do not depend on the options beyond the rounding
    of sums."""

    def __init__(self, gather=None, scatter=None, reach=None, tile=None, fda_order=None, gather_tile=None, gv_threads=None,
                 fda_stage=None, dual=None):
        self.values = {}
        if gather is not None:
            self.values["gather"] = _FAMILY[gather]
        if scatter is not None:
            self.values["scatter"] = _FAMILY[scatter]
        if reach is not None:
            self.values["reach"] = int(reach)
        if tile is not None:
            self.values["tile"] = int(tile)
        if gather_tile is not None:
            self.values["gather_tile"] = int(gather_tile)
        if gv_threads is not None:
            self.values["gv_threads"] = int(gv_threads)
        if dual is not None:
            self.values["dual"] = {"auto": 0, "on": 1, "off": 2}[dual]
        if fda_order is not None:
            self.values["fda_order"] = _ORDER[fda_order]
        if fda_stage is not None:
            self.values["fda_stage"] = {"auto": 0, "on": 1, "off": 2}[fda_stage]
        self.saved = {}

    def __enter__(self):
        import ctypes
        for name, value in self.values.items():
            old = ctypes.c_int(0)
            _lib.check(_L.dcnv4_gfx950_get_launch_option(name.encode(), ctypes.byref(old)))
            self.saved[name] = old.value
            _lib.check(_L.dcnv4_gfx950_set_launch_option(name.encode(), value))
        return self

    def __exit__(self, *exc):
        for name, value in self.saved.items():
            _L.dcnv4_gfx950_set_launch_option(name.encode(), value)
        self.saved = {}
        return False


def _out_hw(h, w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w):
    return ((h + 2 * pad_h - (dilation_h * (kernel_h - 1) + 1)) // stride_h + 1,
            (w + 2 * pad_w - (dilation_w * (kernel_w - 1) + 1)) // stride_w + 1)


def dcnv4_forward(value, p_offset, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h,
                  dilation_w, group, group_channels, offset_scale, im2col_step, remove_center, d_stride,
                  block_thread, softmax):
    _check(value, "input")
    _check(p_offset, "offset", value.dtype)
    if value.dim() != 4 or p_offset.dim() != 4:
        raise RuntimeError("input and offset_mask must be 4-d (N, H, W, C)")
    code = _dtype_code(value, "input")
    batch, h, w, channels = value.shape
    if channels != group * group_channels:
        raise RuntimeError(f"Input channels and group times group channels wont match: ({channels} vs {group * group_channels}).")
    ho, wo = _out_hw(h, w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w)
    if tuple(p_offset.shape[:3]) != (batch, ho, wo):
        raise RuntimeError(f"offset_mask shape {tuple(p_offset.shape)} does not match output ({batch}, {ho}, {wo}, *)")
    with _on_device(value.device):
        output = torch.empty((batch, ho, wo, channels), dtype=value.dtype, device=value.device)
        _lib.check(_L.dcnv4_gfx950_forward(
            value.data_ptr(), p_offset.data_ptr(), output.data_ptr(), code, batch, h, w, group, group_channels,
            kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, float(offset_scale),
            int(im2col_step), int(remove_center), p_offset.shape[3], int(bool(softmax)), _hint(d_stride),
            _hint(block_thread), _stream()))
    return output


def dcnv4_backward(value, p_offset, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h,
                   dilation_w, group, group_channels, offset_scale, im2col_step, grad_output, remove_center,
                   d_stride, block_thread, softmax):
    _check(value, "input")
    _check(p_offset, "offset", value.dtype)
    _check(grad_output, "grad_output", value.dtype)
    if value.dim() != 4 or p_offset.dim() != 4:
        raise RuntimeError("input and offset_mask must be 4-d (N, H, W, C)")
    code = _dtype_code(value, "input")
    batch, h, w, channels = value.shape
    if channels != group * group_channels:
        raise RuntimeError(f"Input channels and group times group channels wont match: ({channels} vs {group * group_channels}).")
    ho, wo = _out_hw(h, w, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w)
    if tuple(p_offset.shape[:3]) != (batch, ho, wo) or grad_output.numel() != batch * ho * wo * channels:
        raise RuntimeError("offset_mask / grad_output shapes do not match the output extent")
    with _on_device(value.device):
        grad_input = torch.empty_like(value)
        grad_offset = torch.empty_like(p_offset)
        ws_bytes = _L.dcnv4_gfx950_backward_workspace_bytes(code, batch, h, w, group, group_channels)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=value.device) if ws_bytes else None
        _lib.check(_L.dcnv4_gfx950_backward(
            value.data_ptr(), p_offset.data_ptr(), grad_output.data_ptr(), grad_input.data_ptr(),
            grad_offset.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes, code, batch, h, w, group,
            group_channels, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w,
            float(offset_scale), int(im2col_step), int(remove_center), p_offset.shape[3], int(bool(softmax)),
            _hint(d_stride), _hint(block_thread), _stream()))
    return [grad_input, grad_offset]


def _fda_common(value, spatial_shapes, level_start_index, sampling_loc_attn, K):
    _check(value, "value")
    _check(spatial_shapes, "spatial_shapes", torch.int64)
    _check(level_start_index, "level_start_index", torch.int64)
    _check(sampling_loc_attn, "sampling_loc_attn", value.dtype)
    if value.dim() != 4 or sampling_loc_attn.dim() != 4:
        raise RuntimeError("value must be (N, S, M, D) and sampling_loc_attn (N, Lq, M, L*K*3)")
    batch, spatial_size, num_heads, channels = value.shape
    num_levels = spatial_shapes.shape[0]
    num_query = sampling_loc_attn.shape[1]
    if level_start_index.numel() != num_levels:
        raise RuntimeError("level_start_index must have one entry per level")
    if tuple(sampling_loc_attn.shape) != (batch, num_query, num_heads, num_levels * K * 3):
        raise RuntimeError(f"sampling_loc_attn shape {tuple(sampling_loc_attn.shape)} != "
                           f"{(batch, num_query, num_heads, num_levels * K * 3)}")
    return batch, spatial_size, num_heads, channels, num_levels, num_query


def flash_deform_attn_forward(value, spatial_shapes, level_start_index, sampling_loc_attn, im2col_step=64, K=8,
                              d_stride=8, block_thread=0):
    batch, spatial_size, num_heads, channels, num_levels, num_query = _fda_common(
        value, spatial_shapes, level_start_index, sampling_loc_attn, K)
    code = _dtype_code(value, "value")
    with _on_device(value.device):
        output = torch.empty((batch, num_query, num_heads * channels), dtype=value.dtype, device=value.device)
        _lib.check(_L.flash_deform_attn_gfx950_forward(
            value.data_ptr(), spatial_shapes.data_ptr(), level_start_index.data_ptr(), sampling_loc_attn.data_ptr(),
            output.data_ptr(), code, batch, spatial_size, num_heads, channels, num_levels, num_query, int(K),
            int(im2col_step), _hint(d_stride), _hint(block_thread), _stream()))
    return output


def flash_deform_attn_backward(value, spatial_shapes, level_start_index, sampling_loc_attn, grad_output,
                               im2col_step=64, K=8, d_stride=2, block_thread=0):
    batch, spatial_size, num_heads, channels, num_levels, num_query = _fda_common(
        value, spatial_shapes, level_start_index, sampling_loc_attn, K)
    _check(grad_output, "grad_output", value.dtype)
    if grad_output.numel() != batch * num_query * num_heads * channels:
        raise RuntimeError("grad_output shape does not match the output")
    code = _dtype_code(value, "value")
    with _on_device(value.device):
        grad_value = torch.empty_like(value)
        grad_sla = torch.empty_like(sampling_loc_attn)
        ws_bytes = _L.flash_deform_attn_gfx950_backward_workspace_bytes(code, batch, spatial_size, num_heads, channels,
                                                                        num_levels, num_query, int(K))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=value.device) if ws_bytes else None
        _lib.check(_L.flash_deform_attn_gfx950_backward(
            value.data_ptr(), spatial_shapes.data_ptr(), level_start_index.data_ptr(), sampling_loc_attn.data_ptr(),
            grad_output.data_ptr(), grad_value.data_ptr(), grad_sla.data_ptr(),
            ws.data_ptr() if ws is not None else None, ws_bytes, code, batch, spatial_size, num_heads, channels,
            num_levels, num_query, int(K), int(im2col_step), _hint(d_stride), _hint(block_thread), _stream()))
    return [grad_value, grad_sla]


def depthwise_conv_forward(input, weight, bias, pad):
    """Depthwise convolution of an NHWC tensor, stride 1, dilation 1: the ``offset_mask_dw`` layer of a
    DCNv4 block (DCNv4_op/DCNv4/modules/dcnv4.py:67-75,121-123) without the permutes around it.
    ``weight`` is nn.Conv2d's (C, 1, k, k) or (C, k, k); ``bias`` (C,) or None.  Returns (N, Ho, Wo, C)."""
    _check(input, "input")
    _check(weight, "weight", input.dtype)
    if bias is not None:
        _check(bias, "bias", input.dtype)
    if input.dim() != 4:
        raise RuntimeError("input must be 4-d (N, H, W, C)")
    code = _dtype_code(input, "input")
    batch, h, w, channels = input.shape
    k = weight.shape[-1]
    if weight.numel() != channels * k * k or weight.shape[0] != channels or weight.shape[-2] != k:
        raise RuntimeError(f"weight shape {tuple(weight.shape)} is not a depthwise kernel for {channels} channels")
    if bias is not None and bias.numel() != channels:
        raise RuntimeError(f"bias has {bias.numel()} elements for {channels} channels")
    ho, wo = h + 2 * pad - k + 1, w + 2 * pad - k + 1
    with _on_device(input.device):
        output = torch.empty((batch, max(ho, 0), max(wo, 0), channels), dtype=input.dtype, device=input.device)
        _lib.check(_L.dcnv4_gfx950_depthwise_conv_forward(
            input.data_ptr(), weight.data_ptr(), bias.data_ptr() if bias is not None else None, output.data_ptr(),
            code, batch, h, w, channels, k, int(pad), _stream()))
    return output


def depthwise_conv_backward(input, weight, grad_output, pad, has_bias=True, need_input_grad=True,
                            need_weight_grad=True):
    """Gradients of :func:`depthwise_conv_forward`: ``[grad_input, grad_weight, grad_bias]`` (None for
    the ones not asked for); grad_weight has the shape of ``weight``."""
    _check(input, "input")
    _check(weight, "weight", input.dtype)
    _check(grad_output, "grad_output", input.dtype)
    code = _dtype_code(input, "input")
    batch, h, w, channels = input.shape
    k = weight.shape[-1]
    ho, wo = h + 2 * pad - k + 1, w + 2 * pad - k + 1
    if tuple(grad_output.shape) != (batch, ho, wo, channels):
        raise RuntimeError(f"grad_output shape {tuple(grad_output.shape)} does not match the output {(batch, ho, wo, channels)}")
    with _on_device(input.device):
        grad_input = torch.empty_like(input) if need_input_grad else None
        grad_weight = torch.empty_like(weight) if need_weight_grad else None
        grad_bias = torch.empty(channels, dtype=input.dtype, device=input.device) if (need_weight_grad and has_bias) else None
        ws_bytes = _L.dcnv4_gfx950_depthwise_conv_backward_workspace_bytes(code, batch, h, w, channels, k, int(pad)) \
            if need_weight_grad else 0
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=input.device) if ws_bytes else None
        ptr = lambda t: t.data_ptr() if t is not None else None
        _lib.check(_L.dcnv4_gfx950_depthwise_conv_backward(
            input.data_ptr(), weight.data_ptr(), grad_output.data_ptr(), ptr(grad_input), ptr(grad_weight),
            ptr(grad_bias), ptr(ws), ws_bytes, code, batch, h, w, channels, k, int(pad), _stream()))
    return [grad_input, grad_weight, grad_bias]


def layer_norm_residual_forward(input, residual, weight, bias, gamma, eps):
    """``residual + gamma * layer_norm(input)`` over the last axis in one kernel; ``residual`` and ``gamma`` may be
    None.  All tensors share one dtype; the channel count must be a whole number of 16-byte vectors."""
    _check(input, "input")
    _check(weight, "weight", input.dtype)
    _check(bias, "bias", input.dtype)
    if residual is not None:
        _check(residual, "residual", input.dtype)
        if residual.shape != input.shape:
            raise RuntimeError("residual must have the shape of the input")
    if gamma is not None:
        _check(gamma, "gamma", input.dtype)
    code = _dtype_code(input, "input")
    channels = input.shape[-1]
    if weight.numel() != channels or bias.numel() != channels or (gamma is not None and gamma.numel() != channels):
        raise RuntimeError(f"weight, bias and gamma must have {channels} elements")
    with _on_device(input.device):
        output = torch.empty_like(input)
        if input.numel():
            _lib.check(_L.dcnv4_gfx950_layer_norm_residual_forward(
                input.data_ptr(), residual.data_ptr() if residual is not None else None, weight.data_ptr(), bias.data_ptr(),
                gamma.data_ptr() if gamma is not None else None, output.data_ptr(), code, input.numel() // channels,
                channels, float(eps), _stream()))
    return output


def layer_norm_residual_backward(grad_output, input, weight, bias, gamma, eps, need_param_grads=True):
    """Gradients of :func:`layer_norm_residual_forward` with respect to ``input``, ``weight``, ``bias`` and ``gamma``
    (the gradient of the residual is ``grad_output`` itself): ``[grad_input, grad_weight, grad_bias, grad_gamma]``,
    None for what is absent or not asked for."""
    _check(grad_output, "grad_output", input.dtype)
    _check(input, "input")
    _check(weight, "weight", input.dtype)
    if bias is not None:
        _check(bias, "bias", input.dtype)
    if gamma is not None:
        _check(gamma, "gamma", input.dtype)
        if bias is None:
            raise RuntimeError("the gradient of gamma needs the bias of the normalisation")
    if grad_output.shape != input.shape:
        raise RuntimeError("grad_output must have the shape of the input")
    code = _dtype_code(input, "input")
    channels = input.shape[-1]
    rows = input.numel() // max(channels, 1)
    with _on_device(input.device):
        grad_input = torch.empty_like(input)
        new = lambda: torch.empty(channels, dtype=input.dtype, device=input.device)
        grad_weight = new() if need_param_grads else None
        grad_bias = new() if need_param_grads else None
        grad_gamma = new() if (need_param_grads and gamma is not None) else None
        if input.numel():
            ws_bytes = _L.dcnv4_gfx950_layer_norm_residual_backward_workspace_bytes(code, rows, channels)
            ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=input.device)
            ptr = lambda t: t.data_ptr() if t is not None else None
            _lib.check(_L.dcnv4_gfx950_layer_norm_residual_backward(
                grad_output.data_ptr(), input.data_ptr(), weight.data_ptr(), ptr(bias), ptr(gamma), grad_input.data_ptr(),
                ptr(grad_weight), ptr(grad_bias), ptr(grad_gamma), ws.data_ptr(), ws_bytes, code, rows, channels,
                float(eps), _stream()))
    return [grad_input, grad_weight, grad_bias, grad_gamma]


def _aligned16(t):
    """`t`, or a copy of it when its storage does not start on a 16-byte boundary (a view into a flat parameter
    buffer): the kernels read this tensor in 16-byte vectors."""
    return t if t.data_ptr() % 16 == 0 else t.clone(memory_format=torch.contiguous_format)


def _blend_common(sampled, projected, weight, bias):
    _check(sampled, "sampled")
    _check(projected, "projected", sampled.dtype)
    _check(weight, "weight", sampled.dtype)
    _check(bias, "bias", sampled.dtype)
    channels = sampled.shape[-1]
    groups = bias.numel()
    if projected.shape != sampled.shape or tuple(weight.shape) != (groups, channels):
        raise RuntimeError(f"projected must have the shape of sampled and weight be ({groups}, {channels})")
    return _dtype_code(sampled, "sampled"), sampled.numel() // max(channels, 1), channels, groups


def center_feature_blend_forward(sampled, projected, weight, bias):
    """``sampled * (1 - gate) + projected * gate`` with ``gate = sigmoid(sampled @ weight.T + bias)`` per (pixel,
    group), every channel using its group's gate (DCNv4_op/DCNv4/modules/dcnv4.py:142-147) in one kernel."""
    code, rows, channels, groups = _blend_common(sampled, projected, weight, bias)
    weight = _aligned16(weight)
    with _on_device(sampled.device):
        output = torch.empty_like(sampled)
        if sampled.numel():
            _lib.check(_L.dcnv4_gfx950_center_feature_blend_forward(
                sampled.data_ptr(), projected.data_ptr(), weight.data_ptr(), bias.data_ptr(), output.data_ptr(), code,
                rows, channels, groups, _stream()))
    return output


def center_feature_blend_backward(grad_output, sampled, projected, weight, bias):
    """``[grad_sampled, grad_projected, grad_gate_logits]``; the last is fp32 (rows, groups): ``grad_weight`` is
    ``grad_gate_logits.T @ sampled`` and ``grad_bias`` its column sums."""
    code, rows, channels, groups = _blend_common(sampled, projected, weight, bias)
    weight = _aligned16(weight)
    _check(grad_output, "grad_output", sampled.dtype)
    if grad_output.shape != sampled.shape:
        raise RuntimeError("grad_output must have the shape of sampled")
    with _on_device(sampled.device):
        grad_sampled, grad_projected = torch.empty_like(sampled), torch.empty_like(sampled)
        grad_logits = torch.empty((rows, groups), dtype=torch.float32, device=sampled.device)
        if sampled.numel():
            _lib.check(_L.dcnv4_gfx950_center_feature_blend_backward(
                grad_output.data_ptr(), sampled.data_ptr(), projected.data_ptr(), weight.data_ptr(), bias.data_ptr(),
                grad_sampled.data_ptr(), grad_projected.data_ptr(), grad_logits.data_ptr(), code, rows, channels,
                groups, _stream()))
    return [grad_sampled, grad_projected, grad_logits]


def _fda_split_common(value, spatial_shapes, level_start_index, locations, logits, K):
    _check(value, "value")
    _check(spatial_shapes, "spatial_shapes", torch.int64)
    _check(level_start_index, "level_start_index", torch.int64)
    _check(locations, "sampling_locations")
    _check(logits, "attention_logits", value.dtype)
    if locations.dtype not in (torch.float32, value.dtype):
        raise RuntimeError(f"sampling_locations must be float32 or {value.dtype}, got {locations.dtype}")
    if value.dim() != 4:
        raise RuntimeError("value must be (N, S, M, D)")
    batch, spatial_size, num_heads, channels = value.shape
    num_levels = spatial_shapes.shape[0]
    num_query = logits.shape[1]
    if level_start_index.numel() != num_levels:
        raise RuntimeError("level_start_index must have one entry per level")
    if tuple(logits.shape) != (batch, num_query, num_heads, num_levels * K) or \
            locations.numel() != batch * num_query * num_heads * num_levels * K * 2:
        raise RuntimeError(f"sampling_locations {tuple(locations.shape)} / attention_logits {tuple(logits.shape)} do not "
                           f"match {(batch, num_query, num_heads, num_levels * K)}")
    return batch, spatial_size, num_heads, channels, num_levels, num_query


def flash_deform_attn_forward_split(value, spatial_shapes, level_start_index, sampling_locations, attention_logits,
                                    im2col_step=64, K=8, d_stride=8, block_thread=0):
    """:func:`flash_deform_attn_forward` on un-packed rows: ``sampling_locations`` (N, Lq, M, L*K*2) or (N, Lq, M, L,
    K, 2) in float32 or the value's dtype, rounded through fp16 inside the kernel as the reference's module rounds
    them before packing (DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133); ``attention_logits`` (N, Lq, M, L*K)."""
    batch, spatial_size, num_heads, channels, num_levels, num_query = _fda_split_common(
        value, spatial_shapes, level_start_index, sampling_locations, attention_logits, K)
    code = _dtype_code(value, "value")
    with _on_device(value.device):
        output = torch.empty((batch, num_query, num_heads * channels), dtype=value.dtype, device=value.device)
        _lib.check(_L.flash_deform_attn_gfx950_forward_split(
            value.data_ptr(), spatial_shapes.data_ptr(), level_start_index.data_ptr(), sampling_locations.data_ptr(),
            attention_logits.data_ptr(), output.data_ptr(), code, _DTYPES[sampling_locations.dtype], batch, spatial_size,
            num_heads, channels, num_levels, num_query, int(K), int(im2col_step), _hint(d_stride), _hint(block_thread),
            _stream()))
    return output


def flash_deform_attn_backward_split(value, spatial_shapes, level_start_index, sampling_locations, attention_logits,
                                     grad_output, im2col_step=64, K=8, d_stride=2, block_thread=0):
    """``[grad_value, grad_sampling_locations, grad_attention_logits]`` of :func:`flash_deform_attn_forward_split`."""
    batch, spatial_size, num_heads, channels, num_levels, num_query = _fda_split_common(
        value, spatial_shapes, level_start_index, sampling_locations, attention_logits, K)
    _check(grad_output, "grad_output", value.dtype)
    if grad_output.numel() != batch * num_query * num_heads * channels:
        raise RuntimeError("grad_output shape does not match the output")
    code = _dtype_code(value, "value")
    with _on_device(value.device):
        grad_value = torch.empty_like(value)
        grad_loc = torch.empty_like(sampling_locations)
        grad_logits = torch.empty_like(attention_logits)
        ws_bytes = _L.flash_deform_attn_gfx950_backward_workspace_bytes(code, batch, spatial_size, num_heads, channels,
                                                                        num_levels, num_query, int(K))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=value.device) if ws_bytes else None
        _lib.check(_L.flash_deform_attn_gfx950_backward_split(
            value.data_ptr(), spatial_shapes.data_ptr(), level_start_index.data_ptr(), sampling_locations.data_ptr(),
            attention_logits.data_ptr(), grad_output.data_ptr(), grad_value.data_ptr(), grad_loc.data_ptr(),
            grad_logits.data_ptr(), ws.data_ptr() if ws is not None else None, ws_bytes, code,
            _DTYPES[sampling_locations.dtype], batch, spatial_size, num_heads, channels, num_levels, num_query, int(K),
            int(im2col_step), _hint(d_stride), _hint(block_thread), _stream()))
    return [grad_value, grad_loc, grad_logits]


def stream_copy(src, dst):
    """Copies ``src`` into ``dst`` (same byte size, a multiple of 16) with the library's streaming kernel: the measured
    memory ceiling of the benchmark and the known-size workload that calibrates byte counters."""
    _check(src, "src")
    _check(dst, "dst")
    nbytes = src.numel() * src.element_size()
    if nbytes != dst.numel() * dst.element_size():
        raise RuntimeError("src and dst differ in size")
    with _on_device(src.device):
        _lib.check(_L.dcnv4_gfx950_stream_copy(src.data_ptr(), dst.data_ptr(), nbytes, _stream()))
    return dst


def lds_read_probe(pattern, iters=4000, device=None):
    """Ticks of the cycle counter per wave-level 16-byte LDS read for one of the probe's address patterns (0 consecutive,
    1 random cells with slot = lane & 15, 2 slot = lane & 7, 3 random cells and slots, 4 all lanes on one slot)."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else device
    with _on_device(device):
        out = torch.zeros(1, dtype=torch.int32, device=device)
        _lib.check(_L.dcnv4_gfx950_lds_read_probe(int(pattern), int(iters), out.data_ptr(), _stream()))
        return out.item() / 1000.0
