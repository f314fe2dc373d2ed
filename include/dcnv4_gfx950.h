/*
 * C ABI of libdcnv4_gfx950.so: the DCNv4 deformable convolution and flash deformable
 * attention operators for AMD MI355X (gfx950).
 *
 * These four operators are what the reference exposes to Python as the pybind11 module
 * `DCNv4.ext` (DCNv4_op/src/vision.cpp:14-21, prototypes DCNv4_op/src/dcnv4.h:19-107).  Here
 * they are plain C functions over raw device pointers so that any host language can bind
 * them; tensor allocation, dtype discovery and stream lookup stay with the caller.
 *
 * Conventions
 *   - every data pointer is device memory, dense row-major, 16-byte aligned;
 *   - `dtype` is one of DCNV4_DTYPE_*; all tensors of a call share it; arithmetic is fp32;
 *   - `stream` is a hipStream_t (NULL = the default stream); calls only enqueue work, they
 *     never synchronise, allocate or free;
 *   - the return value is DCNV4_OK or an error code; dcnv4_gfx950_last_error() then holds a
 *     message for the calling thread.  DCNV4_ERR_INVALID_ARGUMENT corresponds to the
 *     reference's std::invalid_argument (ValueError in Python: unsupported kernel shape, level
 *     count, channel stride); DCNV4_ERR_RUNTIME to its AT_ASSERTM / launch failures
 *     (RuntimeError in Python);
 *   - `d_stride` (channels per lane) and `block_thread` (lanes per workgroup) are the
 *     reference's launch hints; 0 lets the library choose.  Results do not depend on them.
 */
#ifndef DCNV4_GFX950_H
#define DCNV4_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DCNV4_GFX950_ABI_VERSION 6

#define DCNV4_DTYPE_F32 0
#define DCNV4_DTYPE_F16 1
#define DCNV4_DTYPE_BF16 2

#define DCNV4_OK 0
#define DCNV4_ERR_INVALID_ARGUMENT 1
#define DCNV4_ERR_RUNTIME 2

/* ABI version of the loaded library (DCNV4_GFX950_ABI_VERSION it was built with). */
int dcnv4_gfx950_abi_version(void);

/* Message of the last failed call on this thread ("" if none). The pointer stays valid until
 * the next failing call on the same thread. */
const char *dcnv4_gfx950_last_error(void);

/*
 * Launch options of the calling thread, for tuners and for dispatch tables made by them; they play the
 * part of the reference's per-shape launch table (DCNv4_op/DCNv4/functions/table.py, filled by
 * DCNv4_op/scripts/search_dcnv4.py, search_dcnv4_bwd.py and find_best.py).  They choose between kernels that
 * compute the same result (up to the rounding of sums); workspace sizes never depend on them, and the library
 * reads no environment variables.
 *   "gather"     0 library's choice, 1 LDS-tiled gathers where the shape allows, 2 direct gathers
 *                (DCNv4 forward and grad_offset_mask kernels)
 *   "scatter"    0 library's choice, 1 binned LDS accumulation where the shape allows, 2 global atomics
 *                (grad_value of flash deformable attention)
 *   "reach"      -1 library's choice (5), else 0..64: input pixels around an output pixel's reference point that
 *                the LDS-tiled DCNv4 gathers stage; sampling points beyond it are fetched from memory
 *   "tile"       0 library's choice (32), else 8, 16 or 32: largest side of the input tile a workgroup of the
 *                DCNv4 grad_value kernel owns
 *   "gather_tile" 0 library's choice (16), else 4, 8 or 16: largest side of the output tile a workgroup of the
 *                LDS-tiled DCNv4 gathers owns
 *   "fda_order"  0 library's choice, 1 whole query rows per workgroup, 2 one head per workgroup
 *                (flash deformable attention forward and grad_sampling_loc_attn kernels)
 *   "fda_stage"  0 library's choice, 1 stage the smallest levels of one head's value slice in LDS whenever the
 *                one-head-per-workgroup order is used, 2 never (flash deformable attention forward)
 *   "gv_threads" 0 library's choice, else 512 or 1024: lanes per workgroup of the DCNv4 grad_value kernel
 *   "dual"       DCNv4 backward on images small enough to be one grad_value tile: 0 / 1 both kernels as one launch with
 *                two workgroup roles when the shape suits it, 2 always two launches
 * dcnv4_gfx950_get_launch_option reads a value back, so that a caller can restore what it found.
 */
int dcnv4_gfx950_set_launch_option(const char *name, int value);
int dcnv4_gfx950_get_launch_option(const char *name, int *value);

/*
 * DCNv4 forward.  Replaces dcnv4_forward / dcnv4_cuda_forward
 * (DCNv4_op/src/dcnv4.h:64-83, DCNv4_op/src/cuda/dcnv4_cuda.cu:26-90).
 *   value        [batch, height_in, width_in, group*group_channels]
 *   offset_mask  [batch, height_out, width_out, padded_offset_dim]; per group 2K offsets
 *                (x,y interleaved, kernel-tap order x-major) then K modulation scalars,
 *                K = kernel_h*kernel_w - remove_center; tail up to padded_offset_dim unused
 *   output       [batch, height_out, width_out, group*group_channels]  (fully overwritten)
 *   height_out = (height_in + 2*pad_h - (dilation_h*(kernel_h-1)+1)) / stride_h + 1, same for w
 *   softmax != 0 normalises the K modulation scalars of a group with a softmax
 */
int dcnv4_gfx950_forward(const void *value, const void *offset_mask, void *output, int dtype,
                         int batch, int height_in, int width_in, int group, int group_channels,
                         int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h,
                         int pad_w, int dilation_h, int dilation_w, float offset_scale,
                         int im2col_step, int remove_center, int padded_offset_dim, int softmax,
                         int d_stride, int block_thread, void *stream);

/* Scratch bytes dcnv4_gfx950_backward needs: 256 (a few words of state shared by its kernels), whatever the sizes. */
size_t dcnv4_gfx950_backward_workspace_bytes(int dtype, int batch, int height_in, int width_in,
                                             int group, int group_channels);

/*
 * DCNv4 backward.  Replaces dcnv4_backward / dcnv4_cuda_backward
 * (DCNv4_op/src/dcnv4.h:85-107, DCNv4_op/src/cuda/dcnv4_cuda.cu:92-175).
 *   grad_output       like output
 *   grad_value        like value        (fully overwritten; need not be cleared)
 *   grad_offset_mask  like offset_mask  (fully overwritten, tail = 0)
 *   workspace         device scratch of at least ..._workspace_bytes(), 16-byte aligned;
 *                     contents are destroyed; may be NULL when the size is 0
 */
int dcnv4_gfx950_backward(const void *value, const void *offset_mask, const void *grad_output,
                          void *grad_value, void *grad_offset_mask, void *workspace,
                          size_t workspace_bytes, int dtype, int batch, int height_in,
                          int width_in, int group, int group_channels, int kernel_h, int kernel_w,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h,
                          int dilation_w, float offset_scale, int im2col_step, int remove_center,
                          int padded_offset_dim, int softmax, int d_stride, int block_thread,
                          void *stream);

/*
 * DCNv4 backward for callers that cannot allocate device memory (code running under HIP graph capture, serving
 * loops, harnesses that forbid hipMalloc): dcnv4_gfx950_backward without the workspace arguments.  It has no
 * counterpart in the reference.  The scratch lives in a device array inside the library, DCNV4_GFX950_STATIC_SCRATCH_BYTES
 * per GPU, held until the process ends; the call fails with DCNV4_ERR_RUNTIME when
 * dcnv4_gfx950_backward_workspace_bytes() for these sizes is larger.  The call allocates and frees nothing.  All
 * calls on one GPU share the array: two such calls that overlap in time on the same GPU (different streams or
 * threads) race; calls on one stream are ordered and safe.
 */
#define DCNV4_GFX950_STATIC_SCRATCH_BYTES 4096u
int dcnv4_gfx950_backward_static_scratch(const void *value, const void *offset_mask, const void *grad_output,
                                         void *grad_value, void *grad_offset_mask, int dtype, int batch,
                                         int height_in, int width_in, int group, int group_channels,
                                         int kernel_h, int kernel_w, int stride_h, int stride_w, int pad_h,
                                         int pad_w, int dilation_h, int dilation_w, float offset_scale,
                                         int im2col_step, int remove_center, int padded_offset_dim, int softmax,
                                         int d_stride, int block_thread, void *stream);

/*
 * Flash deformable attention forward.  Replaces flash_deform_attn_forward /
 * flash_deform_attn_cuda_forward (DCNv4_op/src/dcnv4.h:19-36,
 * DCNv4_op/src/cuda/flash_deform_attn_cuda.cu:26-84).
 *   value              [batch, spatial_size, num_heads, head_channels]
 *   spatial_shapes     [num_levels, 2] int64 (H_l, W_l), device memory
 *   level_start_index  [num_levels] int64, device memory
 *   sampling_loc_attn  [batch, num_query, num_heads, num_levels*num_points*3]: 2*L*K
 *                      normalised (x,y) locations then L*K attention logits
 *   output             [batch, num_query, num_heads*head_channels]  (fully overwritten)
 */
int flash_deform_attn_gfx950_forward(const void *value, const int64_t *spatial_shapes,
                                     const int64_t *level_start_index,
                                     const void *sampling_loc_attn, void *output, int dtype,
                                     int batch, int spatial_size, int num_heads,
                                     int head_channels, int num_levels, int num_query,
                                     int num_points, int im2col_step, int d_stride,
                                     int block_thread, void *stream);

/*
 * Bytes of device scratch flash_deform_attn_gfx950_backward needs for this problem (16-byte aligned;
 * contents need no initialisation).  Head widths that are multiples of 8 up to 128 take about 34 bytes
 * per sampling point (a key, a position-and-probability record, and list space for binning the points by
 * tile) plus grad_output once more and a tile table; other widths take an fp32 image of value for 16-bit
 * tensors.  The reference allocates its fp32 gradient buffers itself
 * (DCNv4_op/src/cuda/flash_deform_attn_cuda.cu:127-133).
 */
size_t flash_deform_attn_gfx950_backward_workspace_bytes(int dtype, int batch, int spatial_size,
                                                         int num_heads, int head_channels,
                                                         int num_levels, int num_query,
                                                         int num_points);

/*
 * Flash deformable attention backward.  Replaces flash_deform_attn_backward /
 * flash_deform_attn_cuda_backward (DCNv4_op/src/dcnv4.h:38-62,
 * DCNv4_op/src/cuda/flash_deform_attn_cuda.cu:86-163).
 *   grad_value like value, grad_sampling_loc_attn like sampling_loc_attn; both fully
 *   overwritten.  A tap outside its level contributes zero to the softmax Jacobian.
 */
int flash_deform_attn_gfx950_backward(const void *value, const int64_t *spatial_shapes,
                                      const int64_t *level_start_index,
                                      const void *sampling_loc_attn, const void *grad_output,
                                      void *grad_value, void *grad_sampling_loc_attn,
                                      void *workspace, size_t workspace_bytes, int dtype,
                                      int batch, int spatial_size, int num_heads,
                                      int head_channels, int num_levels, int num_query,
                                      int num_points, int im2col_step, int d_stride,
                                      int block_thread, void *stream);

/*
 * Flash deformable attention with the rows of a (query, head) given as two tensors instead of one packed row.
 * Replaces, together with the operator itself, the packing the reference's module does in front of it
 * (DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133: `sampling_locations.flatten(-3).half()` followed by
 * `torch.cat([sampling_locations, attention_weights], dim=-1)`, two passes over the largest tensor of the layer):
 * every location passes through fp16 while it is staged, exactly as `.half()` rounds it, and is then used as the
 * packed operator uses it.
 *   sampling_locations  [batch, num_query, num_heads, num_levels*num_points*2] normalised (x,y); dtype
 *                       `location_dtype`: DCNV4_DTYPE_F32 or the same as `dtype`
 *   attention_logits    [batch, num_query, num_heads, num_levels*num_points], dtype `dtype`
 *   other arguments and the result as flash_deform_attn_gfx950_forward
 */
int flash_deform_attn_gfx950_forward_split(const void *value, const int64_t *spatial_shapes,
                                           const int64_t *level_start_index,
                                           const void *sampling_locations, const void *attention_logits,
                                           void *output, int dtype, int location_dtype, int batch,
                                           int spatial_size, int num_heads, int head_channels,
                                           int num_levels, int num_query, int num_points,
                                           int im2col_step, int d_stride, int block_thread, void *stream);

/*
 * Backward of flash_deform_attn_gfx950_forward_split: flash_deform_attn_gfx950_backward with the row gradient
 * written as two tensors (the split that autograd derives from the reference's `cat` and `.half()`,
 * DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133; the cast passes the gradient through unchanged).
 *   grad_sampling_locations like sampling_locations (dtype `location_dtype`), grad_attention_logits like
 *   attention_logits; both fully overwritten.  Workspace as flash_deform_attn_gfx950_backward_workspace_bytes.
 */
int flash_deform_attn_gfx950_backward_split(const void *value, const int64_t *spatial_shapes,
                                            const int64_t *level_start_index,
                                            const void *sampling_locations, const void *attention_logits,
                                            const void *grad_output, void *grad_value,
                                            void *grad_sampling_locations, void *grad_attention_logits,
                                            void *workspace, size_t workspace_bytes, int dtype,
                                            int location_dtype, int batch, int spatial_size, int num_heads,
                                            int head_channels, int num_levels, int num_query,
                                            int num_points, int im2col_step, int d_stride,
                                            int block_thread, void *stream);

/*
 * Depthwise convolution over channels-last tensors, stride 1, dilation 1, square kernel of size
 * 1, 3, 5 or 7: the `offset_mask_dw` layer of a DCNv4 block.  Replaces the nn.Conv2d call and the
 * NHWC -> NCHW -> NHWC permutes around it (DCNv4_op/DCNv4/modules/dcnv4.py:67-75 and :121-123).
 *   input    [batch, height, width, channels]
 *   weight   [channels, kernel_size, kernel_size]   (nn.Conv2d's [channels, 1, k, k])
 *   bias     [channels] or NULL
 *   output   [batch, height_out, width_out, channels], height_out = height + 2*pad - kernel_size + 1
 *            (fully overwritten)
 *   out[b,y,x,c] = bias[c] + sum_{i,j} weight[c,i,j] * input[b, y+i-pad, x+j-pad, c], zero outside
 */
int dcnv4_gfx950_depthwise_conv_forward(const void *input, const void *weight, const void *bias,
                                        void *output, int dtype, int batch, int height, int width,
                                        int channels, int kernel_size, int pad, void *stream);

/* Scratch bytes dcnv4_gfx950_depthwise_conv_backward needs for grad_weight at these sizes. */
size_t dcnv4_gfx950_depthwise_conv_backward_workspace_bytes(int dtype, int batch, int height,
                                                            int width, int channels,
                                                            int kernel_size, int pad);

/*
 * Gradients of the depthwise convolution above (what autograd derives for the nn.Conv2d of
 * DCNv4_op/DCNv4/modules/dcnv4.py:121).
 *   grad_output  like output
 *   grad_input   like input, or NULL to skip it           (fully overwritten)
 *   grad_weight  like weight, or NULL to skip it and grad_bias   (fully overwritten)
 *   grad_bias    like bias, or NULL
 *   workspace    device scratch of at least ..._workspace_bytes(), 16-byte aligned; only used for
 *                grad_weight / grad_bias; contents are destroyed
 * Sums are formed in fp32 in a fixed order: results are bit-reproducible.
 */
int dcnv4_gfx950_depthwise_conv_backward(const void *input, const void *weight,
                                         const void *grad_output, void *grad_input,
                                         void *grad_weight, void *grad_bias, void *workspace,
                                         size_t workspace_bytes, int dtype, int batch, int height,
                                         int width, int channels, int kernel_size, int pad,
                                         void *stream);

/*
 * output = residual + gamma * LayerNorm(input) over rows of `channels` elements (biased variance, affine
 * weight and bias, fp32 arithmetic, one rounding): the tail of a FlashInternImage block,
 * `x + drop_path(gamma1 * norm1(dcn(x)))` (classification/models/flash_intern_image.py:425-440), which the
 * framework runs as three kernels.  `residual` and `gamma` may be NULL (plain layer normalisation when both
 * are).  channels must be a multiple of 16 bytes' worth of elements and at most 512 such vectors.
 *   input, residual, output  [rows, channels];  weight, bias, gamma  [channels]
 */
int dcnv4_gfx950_layer_norm_residual_forward(const void *input, const void *residual, const void *weight,
                                             const void *bias, const void *gamma, void *output,
                                             int dtype, long long rows, int channels, float eps,
                                             void *stream);

/*
 * Bytes of device scratch dcnv4_gfx950_layer_norm_residual_backward needs (partial column sums of the parameter
 * gradients, one row per workgroup; no initialisation needed).
 */
size_t dcnv4_gfx950_layer_norm_residual_backward_workspace_bytes(int dtype, long long rows, int channels);

/*
 * Backward of dcnv4_gfx950_layer_norm_residual_forward: what autograd derives for the block tail
 * `x + drop_path(gamma1 * norm1(dcn(x)))` (classification/models/flash_intern_image.py:425-440) through
 * layer_norm, the broadcast multiply and the add, in two kernels.  The row statistics are recomputed from
 * `input`; the parameter gradients are column sums added in a fixed order (no atomics).
 *   grad_output, input, grad_input  [rows, channels];  weight, bias, gamma  [channels]
 *   grad_weight, grad_bias, grad_gamma  [channels], each may be NULL (not wanted)
 *   bias is needed only with gamma (it enters grad_gamma); gamma may be NULL.
 *   The gradient of the residual is grad_output itself and is not written.
 */
int dcnv4_gfx950_layer_norm_residual_backward(const void *grad_output, const void *input, const void *weight,
                                              const void *bias, const void *gamma, void *grad_input,
                                              void *grad_weight, void *grad_bias, void *grad_gamma,
                                              void *workspace, size_t workspace_bytes, int dtype,
                                              long long rows, int channels, float eps, void *stream);

/*
 * Centre-feature blend of a DCNv4 layer (DCNv4_op/DCNv4/modules/dcnv4.py:17-26 CenterFeatureScaleModule and
 * :142-147): gate = sigmoid(sampled . weight^T + bias) per (row, group), then
 * output = sampled * (1 - gate) + projected * gate with every channel using its group's gate - the reference's
 * linear, sigmoid, `repeat`, and three element-wise kernels in one pass.
 *   sampled, projected, output  [rows, channels];  weight [groups, channels];  bias [groups]
 *   channels / groups must be a whole number of 16-byte vectors.
 */
int dcnv4_gfx950_center_feature_blend_forward(const void *sampled, const void *projected, const void *weight,
                                              const void *bias, void *output, int dtype, long long rows,
                                              int channels, int groups, void *stream);

/*
 * Backward of the centre-feature blend (autograd through DCNv4_op/DCNv4/modules/dcnv4.py:142-147).
 *   grad_sampled, grad_projected  [rows, channels], fully overwritten
 *   grad_gate_logits  [rows, groups] fp32: the gradient of the gates' pre-sigmoid values; the parameter
 *   gradients are grad_weight = grad_gate_logits^T . sampled and grad_bias = its column sums, a plain matrix
 *   product left to the caller's GEMM library.
 */
int dcnv4_gfx950_center_feature_blend_backward(const void *grad_output, const void *sampled,
                                               const void *projected, const void *weight, const void *bias,
                                               void *grad_sampled, void *grad_projected,
                                               float *grad_gate_logits, int dtype, long long rows,
                                               int channels, int groups, void *stream);

/*
 * Measurement aid without a counterpart in the reference: copies `bytes` (a multiple of 16) from src to dst with
 * the library's own streaming kernel (16-byte non-temporal loads and stores).  Its rate is the ceiling the
 * benchmark quotes beside the nominal HBM peak, and its known traffic calibrates hardware byte counters.
 */
int dcnv4_gfx950_stream_copy(const void *src, void *dst, size_t bytes, void *stream);

/*
 * Measurement aid without a counterpart in the reference: one 1024-lane workgroup reads 16-byte vectors from LDS at
 * addresses cell * 1024 + slot * 16 (a new cell of 64 for every read) for `iters` rounds of eight reads per lane and
 * writes the cycle counter's ticks per 1000 wave-level read instructions to the device word `ticks_per_1000_reads`.
 *   pattern 0  one cell per wave, slot = lane (consecutive addresses)
 *           1  a random cell per lane, slot = lane & 15 (16 consecutive lanes cover 16 different slots of 256 bytes)
 *           2  a random cell per lane, slot = lane & 7
 *           3  a random cell and a random slot per lane (a gather of rows at data-dependent cells)
 *           4  a random cell per lane, slot 0 for all (worst case)
 * The ratios between the patterns say which address patterns the sampling kernels' LDS reads can hope for.
 */
int dcnv4_gfx950_lds_read_probe(int pattern, int iters, unsigned int *ticks_per_1000_reads, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DCNV4_GFX950_H */
