"""``FlashDeformAttnFunction``: autograd wrapper of flash deformable attention with the
reference's signature (DCNv4_op/DCNv4/functions/flash_deform_attn_func.py:69-114).

The reference gates its import on a table of CUDA compute capabilities (:21-36); there is no
such gate here - the library is built for gfx950 and checks its own LDS budget per call.
"""
import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import ext
from .launch_spec import attn_launch_options_for, findspec_attn, findspec_attn_bwd


class FlashDeformAttnFunction(Function):
    @staticmethod
    @torch.autocast("cuda", enabled=True, dtype=torch.float16)
    def forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_loc_attn, im2col_step, K=8):
        ctx.im2col_step = im2col_step
        ctx.K = K
        B, _, G, C = value.shape
        Q = sampling_loc_attn.shape[1]
        es = value.element_size()
        d_stride, block_thread = findspec_attn(B, Q, G, C, es)
        ctx.d_stride_backward, ctx.blockthread_backward = findspec_attn_bwd(B, Q, G, C, es)
        L = value_spatial_shapes.shape[0]
        ctx.backward_options = attn_launch_options_for(B, Q, G, C, L, K, es, "bwd")
        with ext.launch_options(**attn_launch_options_for(B, Q, G, C, L, K, es, "fwd")):
            output = ext.flash_deform_attn_forward(value, value_spatial_shapes, value_level_start_index,
                                                   sampling_loc_attn, im2col_step, K, d_stride, block_thread)
        ctx.save_for_backward(value, value_spatial_shapes, value_level_start_index, sampling_loc_attn)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        value, value_spatial_shapes, value_level_start_index, sampling_loc_attn = ctx.saved_tensors
        with ext.launch_options(**ctx.backward_options):
            grad_value, grad_sampling_loc_attn = ext.flash_deform_attn_backward(
                value, value_spatial_shapes, value_level_start_index, sampling_loc_attn, grad_output.contiguous(),
                ctx.im2col_step, ctx.K, ctx.d_stride_backward, ctx.blockthread_backward)
        return grad_value, None, None, grad_sampling_loc_attn, None, None


class FlashDeformAttnSplitFunction(Function):
    """The same operator on un-packed rows: ``apply(value, spatial_shapes, level_start_index, sampling_locations,
    attention_logits, im2col_step, K)``.  The reference's module rounds the locations to fp16 and concatenates them
    with the logits in front of the operator (DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133); here both steps
    happen while the kernels stage their rows, and the backward returns the two gradients autograd would derive
    through the ``cat`` and the cast."""

    @staticmethod
    @torch.autocast("cuda", enabled=True, dtype=torch.float16)
    def forward(ctx, value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_logits,
                im2col_step, K=8):
        ctx.im2col_step = im2col_step
        ctx.K = K
        B, _, G, C = value.shape
        Q = attention_logits.shape[1]
        es = value.element_size()
        d_stride, block_thread = findspec_attn(B, Q, G, C, es)
        ctx.d_stride_backward, ctx.blockthread_backward = findspec_attn_bwd(B, Q, G, C, es)
        L = value_spatial_shapes.shape[0]
        ctx.backward_options = attn_launch_options_for(B, Q, G, C, L, K, es, "bwd")
        with ext.launch_options(**attn_launch_options_for(B, Q, G, C, L, K, es, "fwd")):
            output = ext.flash_deform_attn_forward_split(value, value_spatial_shapes, value_level_start_index,
                                                         sampling_locations, attention_logits, im2col_step, K, d_stride,
                                                         block_thread)
        ctx.save_for_backward(value, value_spatial_shapes, value_level_start_index, sampling_locations, attention_logits)
        return output

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_output):
        value, shapes, starts, locations, logits = ctx.saved_tensors
        with ext.launch_options(**ctx.backward_options):
            grad_value, grad_locations, grad_logits = ext.flash_deform_attn_backward_split(
                value, shapes, starts, locations, logits, grad_output.contiguous(), ctx.im2col_step, ctx.K,
                ctx.d_stride_backward, ctx.blockthread_backward)
        return grad_value, None, None, grad_locations, grad_logits, None, None
