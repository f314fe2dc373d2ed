"""``DCNv4Function``: autograd wrapper of the DCNv4 operator with the reference's signature
(DCNv4_op/DCNv4/functions/dcnv4_func.py:62-129): 15 positional arguments in, one tensor out,
``(grad_input, grad_offset_mask, None x 13)`` back.
"""
import torch
from torch.amp import custom_bwd, custom_fwd
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from .. import ext
from .launch_spec import find_spec_bwd, findspec, launch_options_for


class DCNv4Function(Function):
    @staticmethod
    @custom_fwd(device_type="cuda")
    def forward(ctx, input, offset_mask, kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w,
                dilation_h, dilation_w, group, group_channels, offset_scale, im2col_step, remove_center):
        B, H, W, _ = input.shape
        es = input.element_size()
        fwd_d_stride, fwd_threads = findspec(B, H, W, group, group_channels, es)
        bwd_d_stride, bwd_threads = find_spec_bwd(B, H, W, group, group_channels, es)
        ctx.geometry = (kernel_h, kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w,
                        group, group_channels, offset_scale, im2col_step)
        ctx.remove_center = remove_center
        ctx.backward_d_stride = bwd_d_stride
        ctx.backward_block_thread = bwd_threads
        ctx.backward_options = launch_options_for(B, H, W, group, group_channels, es, "bwd")
        options = launch_options_for(B, H, W, group, group_channels, es, "fwd")
        if options:        # a tuned table entry that names kernel families
            with ext.launch_options(**options):
                output = ext.dcnv4_forward(input, offset_mask, *ctx.geometry, remove_center, fwd_d_stride, fwd_threads, False)
        else:
            output = ext.dcnv4_forward(input, offset_mask, *ctx.geometry, remove_center, fwd_d_stride, fwd_threads, False)
        ctx.save_for_backward(input, offset_mask)
        return output

    @staticmethod
    @once_differentiable
    @custom_bwd(device_type="cuda")
    def backward(ctx, grad_output):
        input, offset_mask = ctx.saved_tensors
        args = (input, offset_mask, *ctx.geometry, grad_output.contiguous(), ctx.remove_center,
                ctx.backward_d_stride, ctx.backward_block_thread, False)
        if ctx.backward_options:
            with ext.launch_options(**ctx.backward_options):
                grad_input, grad_offset_mask = ext.dcnv4_backward(*args)
        else:
            grad_input, grad_offset_mask = ext.dcnv4_backward(*args)
        return (grad_input, grad_offset_mask) + (None,) * 13
