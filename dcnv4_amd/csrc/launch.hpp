// Host-visible launch descriptors: the C-ABI entry points (capi.hip) fill these and call the
// launchers defined next to the kernels.  Everything is plain data passed by value to kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <unordered_set>

namespace dcn {

// Largest span (bytes) one launch may address through a 32-bit buffer offset.  Value tensors
// larger than this are cut into batch chunks by the entry points.
constexpr uint64_t kMaxSpanBytes = 0x7fff0000ull;
constexpr int kMaxTaps = 64;       // DCNv4: kh*kw - remove_center; attention: L*K
constexpr int kMaxLevels = 16;
constexpr int kBlockThreads = 256;
constexpr size_t kMaxDynamicLds = 64 * 1024;      // without raising the per-kernel limit
constexpr size_t kMaxLdsPerWorkgroup = 160 * 1024;  // gfx950

// Device-side scratch word block shared by the kernels of one backward call (256 bytes).
constexpr int kFarSlots = 56;
struct GradState {
  uint32_t unused0;
  uint32_t unused1;
  uint32_t reach_needed;   // DCNv4: ceiling of the largest Chebyshev distance (pixels) of an in-range sampling point from its output pixel's reference point, over the points within the reach cap
  uint32_t reserved;       // attention backward: set when a level has more tiles than the binning kernel can count
  uint32_t pad[4];
  // DCNv4: for the sampling points beyond the reach cap, per workgroup of the grad_value kernel (tile and chunk of
  // groups; they share the slots round-robin): how far from the tile the output pixels lie whose points land in it; 0: none.
  // Only the workgroups an outlier lands in pay for it.
  uint32_t far_reach[kFarSlots];
};
static_assert(sizeof(GradState) == 256, "GradState fills the state block");

// Dynamic LDS above 64 KB needs hipFuncAttributeMaxDynamicSharedMemorySize on the kernel, on every device that runs
// it (the reference sets it on every launch, DCNv4_op/src/cuda/dcnv4_col2im_cuda.cuh:454).  Set once per (kernel,
// device); safe from concurrent host threads.
inline hipError_t ensure_dynamic_lds_limit(const void *kernel, size_t bytes) {
  static std::mutex mu;
  static std::unordered_set<uint64_t> done;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev)) return e;
  const uint64_t key = (uint64_t)reinterpret_cast<uintptr_t>(kernel) * 64u + (uint64_t)(dev & 63);
  {
    std::lock_guard<std::mutex> lock(mu);
    if (done.count(key)) return hipSuccess;
  }
  if (hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes)) return e;
  std::lock_guard<std::mutex> lock(mu);
  done.insert(key);
  return hipSuccess;
}

struct LaneMap {
  int cpt;          // channels per lane (power of two, cpt * elem_bytes <= 16)
  int tpg;          // lanes that hold one (pixel, group): D / cpt
  int tpgp_log2;    // log2 of tpg rounded up to a power of two (cluster width for reductions)
};

// DCNv4 (reference: DCNv4_op/src/cuda/dcnv4_im2col_cuda.cuh:246-325 launcher arguments)
struct DcnLaunch {
  const void *value;        // [n_img, H, W, G*D]
  const void *offset_mask;  // [n_pix, P_pad]
  const void *grad_out;     // [n_pix, G*D]            (backward)
  void *out;                // [n_pix, G*D]            (forward)
  void *grad_offset_mask;   // [n_pix, P_pad]          (backward)
  uint32_t value_bytes;
  int n_pix;                // images in this launch * Ho * Wo
  int Q, Wo, H, W, G, D;
  int kh, kw, sh, sw, ph, pw, dh, dw;
  int Kp, P_pad, remove_center, softmax;
  float offset_scale;
  int npix_block;           // output pixels per workgroup
  LaneMap lanes;
  // tiled grad_value path
  void *grad_value;         // [n_img, H, W, G*D] in the tensor dtype
  GradState *state;
  int n_img;
  int tile_h, tile_w;       // input-space tile one workgroup owns (an even split of the image, at most 32 x 32)
  int tile_h_log2, tile_w_log2;   // log2 of the tile extents rounded up to powers of two: the stride of the cell index
  int ng_chunk;             // groups per workgroup (channel chunk = ng_chunk * D)
  int strip_pix;            // output pixels staged per strip
  int gv_threads;           // lanes per workgroup of the grad_value kernel: 512 or 1024
  int gv_cw;                // channels a lane accumulates per corner: 8 or 16
  int gv_lps_log2;          // log2 of the lanes that share one (cell, group): group width / gv_cw, rounded up to a power of two
  int gv_whole;             // 1: a tile is a whole image, so every output pixel is visited and the reach statistic is not read
  int gv_go_stride;         // bytes between the parked grad_out rows of consecutive pixels (an odd number of 16-byte units)
  // LDS-tiled gather path (forward and grad_offset_mask); gt_h == 0: not planned
  int gt_h, gt_w;           // output tile one workgroup owns
  int gt_ng;                // groups per workgroup
  int gt_lpg;               // lanes per (pixel, group): 1, or 2 when a group is 64 bytes or wider
  int gt_pad;               // bytes between the cells of the staged window (16: fewer LDS bank conflicts; 0: a larger window fits)
  int gt_wh, gt_ww;         // largest input window (rows, columns of cells) a tile stages
  int gt_reach;             // input pixels around an output pixel's reference point that the window covers
  int dual_interleave;      // two-role backward: workgroups of the two roles alternate in eights (else one role after the other)
  float gv_reach_cap;       // sampling points farther than this from their reference point stay out of reach_needed and are folded into GradState::far_reach
};

// Slot of GradState::far_reach that the workgroup of the grad_value kernel for (image within its launch, tile, chunk of
// groups) uses.
__host__ __device__ inline uint32_t dcnv4_far_slot(int img, int ty, int tx, int nty, int ntx, int chunk, int n_chunks) {
  return (uint32_t)(((img * nty + ty) * ntx + tx) * n_chunks + chunk) % (uint32_t)kFarSlots;
}
// A sampling point beyond the reach cap, of group g, with first corner (y0, x0), of an output pixel of image `img` whose
// reference point is (p0y, p0x): for every grad_value tile one of its in-image corners lands in, records how far outside
// the tile the pixel lies (the condition under which the tile's workgroup for that group visits a pixel,
// dcnv4_grad_value.hip).  Rare path: straight to memory.
__device__ inline void dcnv4_fold_far_point(const DcnLaunch &p, int img, int g, int y0, int x0, int p0y, int p0x) {
  const int nty = (p.H + p.tile_h - 1) / p.tile_h, ntx = (p.W + p.tile_w - 1) / p.tile_w;
  const int n_chunks = (p.G + p.ng_chunk - 1) / p.ng_chunk, chunk = g / p.ng_chunk;
  for (int c = 0; c < 4; ++c) {
    const int cy = y0 + (c >> 1), cx = x0 + (c & 1);
    if ((unsigned)cy >= (unsigned)p.H || (unsigned)cx >= (unsigned)p.W) continue;
    const int ty = cy / p.tile_h, tx = cx / p.tile_w;
    const int ty0 = ty * p.tile_h, tx0 = tx * p.tile_w;
    const int b = max(max(ty0 - p0y, p0y - (ty0 + p.tile_h - 1)), max(tx0 - p0x, p0x - (tx0 + p.tile_w - 1)));
    if (b > 0) atomicMax(&p.state->far_reach[dcnv4_far_slot(img, ty, tx, nty, ntx, chunk, n_chunks)], (uint32_t)min(b, 1 << 20));
  }
}

// Lower bound of the reach cap: the statistic in reach_needed then stays at what the bulk of the sampling points needs
// when a few offsets are outliers.
constexpr int kReachCap = 16;

// Work items a lane of the tiled grad_value kernel handles per strip, at most.  An item is one sampling point, or -
// for a 3x3 kernel - a column of the kernel: three points of one (pixel, group), the removed centre included.
constexpr int kGradValueRounds = 5;            // items of one point
constexpr int kGradValueColumnRounds = 2;      // items of three points
// floats between the cells of the fp32 tile image in which the corner sums meet: the cell's channels rounded up to an odd
// number of 16-byte units, so that the lanes of one LDS instruction (consecutive cells) fall into different banks
__host__ __device__ inline int dcnv4_grad_value_image_stride(int channels) { return ((((channels + 3) / 4) | 1) * 4); }

// Flash deformable attention (reference: DCNv4_op/src/cuda/flash_deform_im2col_cuda.cuh:211-272)
typedef float f32x4_t __attribute__((ext_vector_type(4)));

struct FdaLaunch {
  const void *value;        // [n_img, N, G, D]
  const void *sla;          // [n_row, G, 3*L*K]       n_row = images * Q (null when the rows come split)
  // split rows: locations and logits as two tensors, the locations rounded through fp16 on their way in
  const void *loc;          // [n_row, G, L*K*2], fp32 (loc_f32) or the tensor dtype; null when the rows come packed
  const void *logits;       // [n_row, G, L*K], tensor dtype
  void *grad_loc;           // like loc
  void *grad_logits;        // like logits
  int loc_f32;
  const void *grad_out;     // [n_row, G*D]
  void *out;                // [n_row, G*D]
  float *grad_value_acc;    // [n_img, N, G, D] fp32, zeroed
  void *grad_sla;           // [n_row, G, 3*L*K]
  const int64_t *shapes;    // [L, 2] (H_l, W_l), device memory
  const int64_t *level_start;  // [L], device memory
  uint32_t value_bytes;
  int n_row;
  int Q, N, G, D, L, K;
  int nq_block;             // queries per workgroup
  int head_major;           // forward: a workgroup takes nq_block queries of ONE head, workgroups ordered [image][head][block]
  // forward with the smallest levels of one head's value slice staged in LDS (stage_budget > 0; implies head_major)
  int stage_budget;         // bytes of LDS for staged levels, behind the rows; the kernel stages the last levels that fit
  int stage_blocks;         // workgroups per (image, head); each walks its share of the queries in passes of as many
                            // queries as its lanes hold
  LaneMap lanes;
  // tiled grad_value path
  void *grad_value;         // [n_img, N, G, D] in the tensor dtype
  GradState *state;         // `reserved` only
  int clear_state;          // first kernel of the tiled backward: clear the state block
  uint16_t *keys;           // [n_img, G, L, QKp] one key per sampling point (QKp = Q*K rounded up to even)
  f32x4_t *recs;            // same layout: (x, y, softmax probability, 0) of the point, x and y in cells of its level
  void *go_rows;            // [n_img, G, Q, D] grad_out regrouped by head, tensor dtype: a head's rows lie densely
  uint32_t *table;          // [n_img * G * L * n_chunks][tile_stride] (offset | count << 16) of every tile in every chunk's sorted list
  uint32_t *regions;        // [n_img * G * L * n_chunks][4 * kFdaChunkPoints] point ids of a chunk, sorted by tile
  int n_chunks;             // chunks of kFdaChunkPoints points per (image, head, level)
  int tile_stride;          // table row length: an upper bound of the tiles of one level
  int n_img;
  int gv_c0, gv_dc;         // tiled grad_value kernel: the window [gv_c0, gv_c0 + gv_dc) of a head's channels this launch accumulates (at most 32)
};

// Key of a sampling point: (y0 + 1) << 8 | (x0 + 1) for the integer position (y0, x0) of its first
// corner, y0 in [-1, H-1]; two reserved values for a point outside its level and for a position that
// does not fit the 8-bit fields (the consumer then recomputes it from sampling_loc_attn).
constexpr uint32_t kFdaKeyOutside = 0xfeffu;
constexpr uint32_t kFdaKeySaturated = 0xffffu;
constexpr int kFdaKeyFieldMax = 0xfe;
constexpr int kFdaChunkPoints = 8192;          // points one binning workgroup sorts
constexpr int kFdaMaxTilesPerLevel = 8192;     // LDS histogram of the binning kernel
__host__ __device__ inline size_t fda_key_stride(int Q, int K) { return ((size_t)Q * K + 1) & ~size_t(1); }

enum FdaBackwardMode {
  kFdaFull = 0,        // grad_sampling_loc_attn + fp32 atomic scatter of grad_value (any head width)
  kFdaNoScatter = 1,   // grad_sampling_loc_attn + keys + probabilities, no scatter
  kFdaFallback = 2,    // scatter with fp32 atomics into an fp32 image, only when the binning kernel gave up on a level
};

// Accumulator channels per cell of the tiled flash-attention grad_value kernel (head width rounded up to
// 8, 16, 32 or 64).
__host__ __device__ inline int fda_padded_channels(int D) {
  const int c = (D + 7) / 8;
  return (c <= 2 ? c : (c <= 4 ? 4 : 8)) * 8;
}

// Depthwise convolution over NHWC tensors (stride 1, dilation 1); one launch covers tensors below 2 GiB.
struct DwLaunch {
  const void *in;          // [B, H, W, C]
  const void *weight;      // [C, kh, kw]
  const void *bias;        // [C] or null
  void *out;               // [B, Ho, Wo, C]   (forward / grad_input)
  const void *grad_out;    // [B, Ho, Wo, C]   (grad_weight)
  float *partial;          // [n_part][kh*kw + 1][C] partial sums of grad_weight and grad_bias
  void *grad_weight;       // [C, kh, kw]
  void *grad_bias;         // [C] or null
  int B, H, W, C, Ho, Wo;
  int kh, kw, ph, pw;
  int seg, n_seg;          // output columns per lane visit, segments per row
  int flip;                // forward: read the kernel back to front (grad_input)
  int slab, n_part;        // grad_weight: row segments (seg columns each) per workgroup, workgroups
};

// out = residual + gamma * LayerNorm(y) over rows of C channels (residual and gamma may be null).
struct LnLaunch {
  const void *y, *residual, *weight, *bias, *gamma;
  void *out;
  long long rows;
  int C;
  float eps;
  int team;      // lanes per row: a power of two, <= 64
  int vpl;       // 16-byte vectors per lane: 1, 2, 4 or 8 (team * vpl * 16 bytes cover a row)
  // backward
  const void *grad_out;
  void *grad_y, *grad_weight, *grad_bias, *grad_gamma;     // the three parameter gradients may be null
  float *partial;   // [n_part][3][C] column sums of one workgroup each: grad_weight, grad_bias, grad_gamma
  long long slab;   // consecutive rows per workgroup (a multiple of the rows one pass of the workgroup takes)
  int n_part;       // workgroups of the backward
};
// Centre-feature blend: out = y * (1 - gate) + x * gate, gate[g] = sigmoid(<W[g,:], y> + b[g]) per (row, group).
struct CfLaunch {
  const void *y, *x, *weight, *bias;      // y, x [rows, C]; weight [G, C]; bias [G]
  void *out;                              // forward
  const void *grad_out;                   // backward
  void *grad_y, *grad_x;
  float *grad_logits;                     // [rows, G] fp32
  long long rows;
  int C, G, D;                            // D = C / G channels per group, a whole number of 16-byte vectors
  int team, vpl;                          // as in LnLaunch
};
hipError_t launch_center_feature_blend(int dtype, const CfLaunch &p, bool backward, hipStream_t stream);
hipError_t launch_layer_norm_residual(int dtype, const LnLaunch &p, hipStream_t stream);
hipError_t launch_layer_norm_residual_backward(int dtype, const LnLaunch &p, hipStream_t stream);

// Each returns hipSuccess or the launch error.  dtype: 0 fp32, 1 fp16, 2 bf16.
hipError_t launch_depthwise_forward(int dtype, const DwLaunch &p, hipStream_t stream);
// channels per lane of the grad_weight kernel, and lanes of a workgroup that share a channel vector
int depthwise_grad_weight_vector(int elem_bytes, int C, int k);
int depthwise_grad_weight_pixel_lanes(int elem_bytes, int C, int k);
hipError_t launch_depthwise_grad_weight_partials(int dtype, const DwLaunch &p, hipStream_t stream);
hipError_t launch_depthwise_grad_weight_reduce(int dtype, const DwLaunch &p, hipStream_t stream);
hipError_t launch_dcnv4_forward(int dtype, const DcnLaunch &p, hipStream_t stream);
hipError_t launch_dcnv4_offset_mask_grad(int dtype, const DcnLaunch &p, hipStream_t stream);
hipError_t launch_dcnv4_grad_value(int dtype, const DcnLaunch &p, hipStream_t stream);
// Both kernels of the backward as one launch with two workgroup roles, for shapes whose grad_value tiles are whole images
// (dcnv4_backward_dual.hip).
bool dcnv4_backward_dual_fits(const DcnLaunch &p, int elem_bytes);
uint32_t dcnv4_backward_dual_workgroups(const DcnLaunch &p, int n_img);
hipError_t launch_dcnv4_backward_dual(int dtype, const DcnLaunch &p, hipStream_t stream);
// Entry slots of the tiled grad_value kernel per (pixel, group) of a strip, and at most per strip: three-point items
// for a 3x3 kernel (nine slots, also when the centre is removed), else an item per sampling point.
inline bool dcnv4_grad_value_columns(const DcnLaunch &p) { return p.kh == 3 && p.kw == 3; }
inline int dcnv4_grad_value_slots(const DcnLaunch &p) { return dcnv4_grad_value_columns(p) ? 9 : p.Kp; }
inline int dcnv4_grad_value_max_slots(const DcnLaunch &p, int threads) {
  return dcnv4_grad_value_columns(p) ? kGradValueColumnRounds * threads * 3 : kGradValueRounds * threads;
}
size_t dcnv4_grad_value_lds_bytes(const DcnLaunch &p);
hipError_t launch_dcnv4_forward_tiled(int dtype, const DcnLaunch &p, hipStream_t stream);
hipError_t launch_dcnv4_offset_mask_grad_tiled(int dtype, const DcnLaunch &p, hipStream_t stream);
size_t dcnv4_tiled_gather_lds_bytes(const DcnLaunch &p, int elem_bytes);
hipError_t launch_fda_forward(int dtype, const FdaLaunch &p, hipStream_t stream);
// Lanes of a workgroup that takes one head (measured on the 128x128 pyramid against 256: the first backward pass is
// 2 % faster with 512 and slower with 1024; the forward 6 % faster with 1024 on 128-byte heads, unchanged on 64-byte ones)
constexpr int kFdaBackwardThreads = 512;
constexpr int kFdaForwardThreads = 1024;
constexpr int kFdaStagedThreads = 1024;      // lanes of a workgroup of the staged forward
hipError_t launch_fda_backward(int dtype, const FdaLaunch &p, int mode, hipStream_t stream);
hipError_t launch_fda_grad_value(int dtype, const FdaLaunch &p, hipStream_t stream);
size_t fda_grad_value_lds_bytes(const FdaLaunch &p, int elem_bytes);

size_t dcnv4_forward_lds_bytes(const DcnLaunch &p);
size_t dcnv4_backward_lds_bytes(const DcnLaunch &p);
size_t fda_forward_lds_bytes(const FdaLaunch &p);
size_t fda_backward_lds_bytes(const FdaLaunch &p);
// Zero bytes at the start of the staged forward's level area, read by corners that fall outside their level: one
// head's width, so that any lane's channel offset stays inside them.
__host__ __device__ inline int fda_staged_zero_bytes(int head_bytes) { return head_bytes < 64 ? 64 : (head_bytes + 15) & ~15; }

}  // namespace dcn
