// C-ABI entry points of libdcnv4_gfx950.so (declared in include/dcnv4_gfx950.h): argument
// checks, launch geometry for wave64, batch chunking for 32-bit buffer addressing, and the
// small utility kernels (clear, fp32 -> half cast) around the sampling kernels.
// Host-side counterpart of the reference's DCNv4_op/src/cuda/dcnv4_cuda.cu:26-175 and
// DCNv4_op/src/cuda/flash_deform_attn_cuda.cu:26-163, minus tensor allocation, which the
// caller owns.
#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/dcnv4_gfx950.h"
#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

int elem_bytes(int dtype) {
  switch (dtype) {
    case DCNV4_DTYPE_F32: return 4;
    case DCNV4_DTYPE_F16:
    case DCNV4_DTYPE_BF16: return 2;
  }
  return 0;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int ceil_log2(int v) {
  int l = 0;
  while ((1 << l) < v) ++l;
  return l;
}

// Channels per lane: the widest power-of-two vector (<= 16 bytes) that divides D, unless a
// valid d_stride hint asks for a narrower one.  Reference table: dcnv4_im2col_cuda.cuh:342-415.
int choose_lanes(int D, int s, int d_stride, bool scatter, LaneMap *lm) {
  if (d_stride != 0 && d_stride != 1 && d_stride != 2 && d_stride != 4 && d_stride != 8 && d_stride != 16)
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "invalid d_stride %d", d_stride);
  int cpt = 1;
  while (cpt * 2 * s <= 16 && D % (cpt * 2) == 0) cpt *= 2;
  if (d_stride > 0 && d_stride < cpt && D % d_stride == 0) cpt = d_stride;
  // Kernels that scatter with fp32 atomics want one channel per lane: the lanes of a group then
  // cover one contiguous run of dwords per atomic instruction, and the L2 atomic units retire
  // about one dword per clock per channel however the dwords are spread over lanes.
  else if (scatter && d_stride == 0 && D <= kWave) cpt = 1;
  lm->cpt = cpt;
  lm->tpg = D / cpt;
  lm->tpgp_log2 = ceil_log2(lm->tpg);
  return DCNV4_OK;
}

// ---------------------------------------------------------------- utility kernels
__global__ void __launch_bounds__(256) clear_kernel(uint32_t *dst, size_t n16, size_t n_words) {
  // n16 aligned 16-byte groups, then the (< 4) trailing 32-bit words
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (size_t i = tid; i < n16; i += stride) reinterpret_cast<u32x4 *>(dst)[i] = u32x4{0, 0, 0, 0};
  for (size_t i = n16 * 4 + tid; i < n_words; i += stride) dst[i] = 0u;
}

template <typename Tag>
__global__ void __launch_bounds__(256) narrow_kernel(const float *src, void *dst, size_t n8, size_t n) {
  // n8 groups of 8 elements, then a scalar tail
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (size_t i = tid; i < n8; i += stride) {
    const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + 2 * i);
    const f32x4 b = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + 2 * i + 1);
    const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    reinterpret_cast<u32x4 *>(dst)[i] = Pack<Tag, 8>::encode(f);
  }
  for (size_t i = n8 * 8 + tid; i < n; i += stride) {
    const float f[1] = {src[i]};
    reinterpret_cast<uint16_t *>(dst)[i] = Pack<Tag, 1>::encode(f);
  }
}

// Plain streaming copy, four 16-byte vectors per lane: the yardstick for what the memory system sustains.
__global__ void __launch_bounds__(256) stream_copy_kernel(const u32x4 *src, u32x4 *dst, size_t n16) {
  const size_t base = (size_t)blockIdx.x * (256 * 4) + threadIdx.x;
  u32x4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (base + u * 256 < n16) v[u] = __builtin_nontemporal_load(src + base + u * 256);
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (base + u * 256 < n16) __builtin_nontemporal_store(v[u], dst + base + u * 256);
}

// LDS read probe: a 1024-lane workgroup issues `iters` rounds of eight 16-byte LDS reads per lane whose addresses follow
// one of a few patterns, and reports the cycle counter's ticks per wave instruction.  Every lane reads at
// cell * 1024 + slot * 16 with a cell (of 64) that changes per read.
//   0  all lanes of a wave in one cell, slot = lane (1 KB of consecutive addresses)
//   1  a random cell per lane, slot = lane & 15: any 16 consecutive lanes cover 16 different slots of 256 bytes
//   2  a random cell per lane, slot = lane & 7: 8 consecutive lanes cover the 8 slots of 128 bytes
//   3  a random cell and a random slot per lane (what a gather from rows at data-dependent cells looks like)
//   4  a random cell per lane, slot 0 for every lane (the worst case)
__global__ void __launch_bounds__(1024) lds_read_probe_kernel(int pattern, int iters, uint32_t *ticks_per_1000) {
  __shared__ u32x4 cells[4096];                   // 64 KB
  for (int i = threadIdx.x; i < 4096; i += 1024) cells[i] = u32x4{(uint32_t)i, 0u, 0u, 0u};
  __syncthreads();
  const int lane = threadIdx.x & 63;
  uint32_t seed = threadIdx.x * 131u + 7u;
  u32x4 acc = {0u, 0u, 0u, 0u};
  const int fixed_slot = pattern == 0 ? lane : (pattern == 1 ? (lane & 15) : (pattern == 2 ? (lane & 7) : 0));
  __syncthreads();
  const long long t0 = clock64();
  for (int i = 0; i < iters; ++i) {
    seed = seed * 1664525u + 1013904223u;
    const uint32_t r = seed >> 8;
    u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int cell = pattern == 0 ? ((i + u) & 63) : (int)((r >> (3 * u)) & 63u);
      const int slot = pattern == 3 ? (int)((r >> (2 * u + 1)) & 63u) : fixed_slot;
      v[u] = cells[cell * 64 + slot];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  const long long t1 = clock64();
  if (threadIdx.x == 0) *ticks_per_1000 = (uint32_t)((t1 - t0) * 1000 / ((long long)iters * 8 * 16));      // 16 waves, 8 reads a round
  if (acc.x == 0xdeadbeefu) *ticks_per_1000 = acc.y;      // keeps the reads alive
}

int grid_for(size_t work_items) {
  const size_t blocks = (work_items + 255) / 256;
  return (int)std::min<size_t>(std::max<size_t>(blocks, 1), 256 * 32);
}

// Clears n_words 32-bit words at a 16-byte aligned address with a kernel rather than a memset
// node, so the call stays safe under HIP-graph capture.
hipError_t clear_async(void *dst, size_t n_words, hipStream_t stream) {
  if (n_words == 0) return hipSuccess;
  const size_t n16 = n_words / 4;
  hipLaunchKernelGGL(clear_kernel, dim3(grid_for(std::max<size_t>(n16, 1))), dim3(256), 0, stream,
                     reinterpret_cast<uint32_t *>(dst), n16, n_words);
  return hipGetLastError();
}

// The same two, run only when the attention backward's binning kernel has raised its flag (GradState::reserved): the
// fallback kernel then sums in an fp32 image that is cleared before it and narrowed after it.
__global__ void __launch_bounds__(256) clear_if_flagged_kernel(const GradState *state, uint32_t *dst, size_t n16) {
  if (state->reserved == 0u) return;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride)
    reinterpret_cast<u32x4 *>(dst)[i] = u32x4{0, 0, 0, 0};
}

template <typename Tag>
__global__ void __launch_bounds__(256) narrow_if_flagged_kernel(const GradState *state, const float *src, void *dst, size_t n8) {
  if (state->reserved == 0u) return;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8; i += stride) {
    const f32x4 a = reinterpret_cast<const f32x4 *>(src)[2 * i], b = reinterpret_cast<const f32x4 *>(src)[2 * i + 1];
    const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    reinterpret_cast<u32x4 *>(dst)[i] = Pack<Tag, 8>::encode(f);
  }
}

hipError_t narrow_async(int dtype, const float *src, void *dst, size_t n, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  const size_t n8 = n / 8;
  const dim3 grid(grid_for(std::max<size_t>(n8, 1))), block(256);
  if (dtype == DCNV4_DTYPE_F16) hipLaunchKernelGGL(narrow_kernel<F16>, grid, block, 0, stream, src, dst, n8, n);
  else hipLaunchKernelGGL(narrow_kernel<BF16>, grid, block, 0, stream, src, dst, n8, n);
  return hipGetLastError();
}

size_t round16(size_t v) { return (v + 15) & ~size_t(15); }

__global__ void init_state_kernel(GradState *st) {
  if (threadIdx.x < sizeof(GradState) / sizeof(uint32_t)) reinterpret_cast<uint32_t *>(st)[threadIdx.x] = 0u;
}
static_assert(sizeof(GradState) / sizeof(uint32_t) <= 64, "init_state_kernel runs one wave");

constexpr size_t kStateBytes = 256;     // GradState, padded
constexpr int kMaxBackwardGroupChannels = 512;    // widest group of the backward: 64 lanes of 16 bytes in the gather, 16 lanes of 32 channels per slot

// Per-thread launch options (dcnv4_gfx950_set_launch_option).  They choose between kernels that compute the same
// result; nothing else in the library reads the environment or any other hidden state.
enum { kOptAuto = 0, kOptTiled = 1, kOptPlain = 2 };
struct LaunchOptions {
  int gather = kOptAuto;       // LDS-tiled / direct gathers (DCNv4 forward, grad_offset_mask)
  int scatter = kOptAuto;      // attention grad_value: binned LDS accumulation / global atomics
  int reach = -1;              // input pixels around a reference point that the tiled gathers stage; -1: default
  int tile = 0;                // largest side of a grad_value tile (8, 16, 32); 0: default
  int gather_tile = 0;         // largest side of an output tile of the tiled gathers (4, 8, 16); 0: default (16)
  int gv_threads = 0;          // lanes per workgroup of the grad_value kernel (512, 1024); 0: default
  int dual = kOptAuto;         // DCNv4 backward whose grad_value tiles are whole images: 1 / auto one launch with two workgroup roles, 2 two launches
  int fda_order = kOptAuto;    // attention forward: 1 whole query rows per workgroup, 2 one head per workgroup
  int fda_stage = kOptAuto;    // attention forward: 1 stage the smallest levels of a head in LDS, 2 never
};
thread_local LaunchOptions g_opt;

constexpr int kDefaultReach = 5;

int reach_setting() { return g_opt.reach < 0 ? kDefaultReach : std::min(g_opt.reach, 64); }

// Flash attention backward: head widths the tiled grad_value kernel handles (whole 8-channel blocks; a launch
// accumulates up to 32 channels - 8 lanes x 4 - and wider heads take a launch per window of 32 over the same point
// records and lists), with point counts that fit its 32-bit point ids.
constexpr int kFdaWindowChannels = 32;
bool fda_tiled_shape(int D, int L, int Q, int K) {
  return D % 8 == 0 && D <= 4 * kFdaWindowChannels && L >= 1 && K >= 1 && (long long)Q * K < (1ll << 31);
}

constexpr size_t kL2BytesPerXcd = 4u << 20;
constexpr int kCusPerDevice = 256;      // MI355X: 8 XCDs of 32 CUs

bool fda_tiled_enabled() { return g_opt.scatter != kOptPlain; }

// Tile, group chunk, lanes per slot and strip of the tiled grad_value kernel such that a workgroup has at most one
// (anchor, group, channel part) per lane and its LDS footprint fits.
static bool plan_grad_value_for(DcnLaunch *L, int threads, int park_bytes) {
  auto even_split = [](int extent, int c) { const int n = (extent + c - 1) / c; return (extent + n - 1) / n; };
  L->gv_threads = threads;
  const size_t budget = kMaxLdsPerWorkgroup / (1024 / threads) - 512;
  const int max_lists = threads >> L->gv_lps_log2;      // a lane per (anchor, group, channel part)
  if (max_lists < 4) return false;
  const int cap = g_opt.tile == 8 ? 8 : (g_opt.tile == 16 ? 16 : 31);
  // the image is split evenly into tiles of at most cap x cap cells (all workgroups then carry the same load); the
  // anchors of a tile, one row and one column more than its cells, must fit the workgroup
  int cap_h = cap, cap_w = cap;
  for (;;) {
    L->tile_h = even_split(L->H, cap_h);
    L->tile_w = even_split(L->W, cap_w);
    if ((L->tile_h + 1) * (L->tile_w + 1) <= max_lists) break;
    if (cap_h >= cap_w) cap_h = std::max(1, cap_h - 1); else cap_w = std::max(1, cap_w - 1);
  }
  L->tile_h_log2 = ceil_log2(L->tile_h);
  L->tile_w_log2 = ceil_log2(L->tile_w);
  const int anchors = (L->tile_h + 1) * (L->tile_w + 1);
  const int max_items = dcnv4_grad_value_max_slots(*L, threads), slots = dcnv4_grad_value_slots(*L);
  for (int ng = std::min({L->G, max_lists / anchors, 63, max_items / slots}); ng >= 1; --ng) {
    L->ng_chunk = ng;
    int units = (ng * (L->gv_cw << L->gv_lps_log2) * park_bytes + 15) / 16;
    units |= 1;                                     // an odd number of 16-byte units spreads the rows over the LDS banks
    L->gv_go_stride = units * 16;
    for (int s = std::min(1023, max_items / (slots * ng)); s >= 1; s = s > 64 ? s - 16 : s - 1) {
      L->strip_pix = s;
      if (dcnv4_grad_value_lds_bytes(*L) <= budget) return true;
    }
  }
  return false;
}

int plan_grad_value_tiles(DcnLaunch *L, int dtype, int batch) {
  const int D = L->D;
  L->gv_cw = D <= 8 ? 8 : 16;
  L->gv_lps_log2 = 0;
  while ((L->gv_cw << L->gv_lps_log2) < D) ++L->gv_lps_log2;
  const int park_bytes = 4;      // grad_out rows are parked as fp32 for every tensor dtype
  if (g_opt.gv_threads != 0) {
    if (plan_grad_value_for(L, g_opt.gv_threads, park_bytes) || plan_grad_value_for(L, 1024, park_bytes)) return DCNV4_OK;
    return fail(DCNV4_ERR_RUNTIME, "kernel with %d taps and %d group channels does not fit the tiled backward", L->Kp, D);
  }
  // Workgroups of 1024 lanes (one per CU, the whole LDS) or of 512 (two per CU).  A workgroup takes about the same
  // time either way - its lanes each own one anchor and walk lists of the same length - so the kernel's time goes
  // with the number of passes the workgroups make over the chip, and a pass of 512-lane workgroups is a little
  // shorter (two workgroups on a CU fill each other's barrier waits).  With few passes a partly filled last one
  // counts in full.  Measured at batch 64: 56x56 with 4 groups, 1024 lanes: 4 passes, 96 us; 512 lanes: 4.5 passes,
  // 102 us; 28x28 with 8 groups: 2 passes either way, 512 lanes 4 % faster; 256x256 with 10 groups, batch 2: 10 %.
  double best_cost = 0.;
  int best = 0;
  for (int threads = 1024; threads >= 512; threads /= 2) {
    DcnLaunch trial = *L;
    if (!plan_grad_value_for(&trial, threads, park_bytes)) continue;
    const double wgs = (double)batch * ((L->H + trial.tile_h - 1) / trial.tile_h) * ((L->W + trial.tile_w - 1) / trial.tile_w) *
                       ((L->G + trial.ng_chunk - 1) / trial.ng_chunk);
    const double passes = wgs / (double)(kCusPerDevice * (1024 / threads));
    // a tile that is a whole image revisits nothing and needs no reach statistic (28x28 with 8 groups at batch 64:
    // 1024 lanes and whole images 2-3 % faster than 512 lanes and half images)
    const bool whole = trial.tile_h >= L->H && trial.tile_w >= L->W;
    const double cost = (passes < 6. ? std::ceil(passes) : passes) * (threads == 512 ? 0.92 : 1.0) * (whole ? 0.9 : 1.0);
    if (best == 0 || cost < best_cost) { best = threads; best_cost = cost; }
  }
  if (best != 0 && plan_grad_value_for(L, best, park_bytes)) return DCNV4_OK;
  return fail(DCNV4_ERR_RUNTIME, "kernel with %d taps and %d group channels does not fit the tiled backward", L->Kp, D);
}

bool tiled_gather_enabled() { return g_opt.gather != kOptPlain; }

// Output tile, group chunk and input window of the LDS-tiled gather kernels.  Returns false (and
// leaves gt_h = 0) when the shape does not suit them: group width not a power-of-two number of
// 16-byte vectors or above 128 bytes, or no tile whose window fits in LDS.
constexpr int kTiledGatherThreads = 512;     // launch bound of the tiled gather kernels

bool plan_gather_tiles(DcnLaunch *L, int s, bool backward) {
  L->gt_h = L->gt_w = L->gt_ng = L->gt_wh = L->gt_ww = 0;
  L->gt_lpg = 1;
  L->gt_pad = 16;
  L->gt_reach = reach_setting();
  if (!tiled_gather_enabled()) return false;
  const int lane_bytes = L->D * s;
  if (lane_bytes % 16 != 0) return false;
  const int nv = lane_bytes / 16;
  if (nv != 1 && nv != 2 && nv != 4 && nv != 8) return false;      // up to 128 bytes per group: 64 16-bit or 32 fp32 channels
  // Groups of 64 channels (16-bit tensors): a corner is a whole 128-byte line, which the direct gathers fetch well.
  // Measured at 64x56x56, 4 groups of 64, fp16: forward 149 us direct against 173 us tiled, grad_offset_mask 10 % faster tiled.
  if (!backward && L->D > 32) return false;
  if (L->Kp > 64) return false;
  L->gt_lpg = nv >= 4 ? 2 : 1;      // wide groups: two lanes each, for twice the waves per workgroup
  const int Ho = L->Q / L->Wo, Wo = L->Wo;
  auto even_split = [](int extent, int cap) { const int n = (extent + cap - 1) / cap; return (extent + n - 1) / n; };
  const int cap0 = g_opt.gather_tile > 0 ? g_opt.gather_tile : 16;
  // The largest tile and group chunk that fit `budget` bytes of LDS with `reach`, with at least `min_lanes` lanes.
  auto fit = [&](size_t budget, int reach, int min_lanes) {
    for (int cap_h = cap0, cap_w = cap0; cap_h >= 4 && cap_w >= 4;) {
      L->gt_reach = reach;
      L->gt_h = even_split(Ho, cap_h);
      L->gt_w = even_split(Wo, cap_w);
      L->gt_wh = std::min((L->gt_h - 1) * L->sh + 2 * reach + 1, L->H + 2);
      L->gt_ww = std::min((L->gt_w - 1) * L->sw + 2 * reach + 1, L->W + 2);
      const int px = L->gt_h * L->gt_w;
      for (int ng = std::min(L->G, kTiledGatherThreads / (px * L->gt_lpg)); ng >= 1; --ng) {
        // 16-bit tensors: keep the offset_mask slices dword-aligned when the tap count is odd
        if (s == 2 && ((ng * 3 * L->Kp) & 1) && ng > 1) continue;
        if (px * ng * L->gt_lpg < min_lanes) break;
        L->gt_ng = ng;
        if (dcnv4_tiled_gather_lds_bytes(*L, s) <= budget) return true;
      }
      if (cap_h >= cap_w) cap_h /= 2; else cap_w /= 2;
    }
    return false;
  };
  // Two workgroups per CU when the window allows it, so that one stages while the other computes, and workgroups of
  // 384 lanes or more (a small workgroup stages its window in short pieces and leaves the CU short of waves).  A
  // shape too wide for that with the full reach stages a window one or two pixels shorter - the sampling points
  // beyond it are served from memory - before it settles for a small workgroup or a whole CU's LDS.
  const size_t half = kMaxLdsPerWorkgroup / 2 - 512, whole = kMaxLdsPerWorkgroup - 1024;
  const int R = L->gt_reach;
  const int want_lanes = std::min(384, Ho * Wo * L->G * L->gt_lpg);
  const int shorter = g_opt.reach < 0 ? 2 : 0;        // an explicit reach is kept
  for (int d = 0; d <= shorter && d <= R - 2; ++d)
    for (int pad = 16; pad >= (d == 0 ? 0 : 16); pad -= 16) {       // the full reach is worth more than the padding between the cells
      L->gt_pad = pad;
      if (fit(half, R - d, want_lanes)) return true;
    }
  L->gt_pad = 16;
  if (fit(half, R, 1) || fit(whole, R, 1)) return true;
  L->gt_h = L->gt_w = L->gt_ng = L->gt_wh = L->gt_ww = 0;
  L->gt_reach = R;
  return false;
}

// ---------------------------------------------------------------- DCNv4
// Output pixels per workgroup: about block_thread (default 256) lanes of whole pixels, capped by
// the LDS that the staged offset_mask rows (and, backward, their gradients) take.
int choose_block_pixels(DcnLaunch *L, int block_thread, bool backward) {
  const int lanes_per_pix = L->G << L->lanes.tpgp_log2;
  const int want = block_thread > 0 ? block_thread : kBlockThreads;
  int npix = std::max(1, want / lanes_per_pix);
  const size_t lds_per_pix = (size_t)L->P_pad * sizeof(float) * (backward ? 2 : 1);
  while (npix > 1 && npix * lds_per_pix > kMaxDynamicLds) --npix;
  if (npix * lds_per_pix > kMaxDynamicLds)
    return fail(DCNV4_ERR_RUNTIME, "offset_mask row of %d elements does not fit in LDS", L->P_pad);
  L->npix_block = npix;
  return DCNV4_OK;
}

struct DcnProblem {
  DcnLaunch launch;      // geometry common to every chunk
  int batch, Ho, Wo, s;
  size_t img_elems, img_out_elems, img_om_elems;
};

int out_extent(int in, int pad, int dil, int k, int stride) {     // dcnv4_cuda.cu:48-52
  return (in + 2 * pad - (dil * (k - 1) + 1)) / stride + 1;
}

int dcn_prepare(DcnProblem *pr, bool backward, int dtype, int batch, int H, int W, int G, int D, int kh,
                int kw, int sh, int sw, int ph, int pw, int dh, int dw, float offset_scale, int im2col_step,
                int remove_center, int P_pad, int softmax, int d_stride, int block_thread) {
  const int s = elem_bytes(dtype);
  if (s == 0) return fail(DCNV4_ERR_RUNTIME, "unsupported dtype code %d (fp32, fp16, bf16 only)", dtype);
  if (batch <= 0 || H <= 0 || W <= 0 || G <= 0 || D <= 0)
    return fail(DCNV4_ERR_RUNTIME, "empty or negative tensor extent (batch %d, H %d, W %d, group %d, group_channels %d)",
                batch, H, W, G, D);
  if (kh <= 0 || kw <= 0 || sh <= 0 || sw <= 0 || dh <= 0 || dw <= 0 || ph < 0 || pw < 0)
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "invalid kernel shape");
  remove_center = remove_center ? 1 : 0;
  if (remove_center && (kh % 2 == 0 || kw % 2 == 0))
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "remove_center needs an odd kernel, got %dx%d", kh, kw);
  const int Kp = kh * kw - remove_center;
  if (Kp < 1 || Kp > kMaxTaps) return fail(DCNV4_ERR_INVALID_ARGUMENT, "invalid kernel shape: %d taps (1..%d)", Kp, kMaxTaps);
  if (im2col_step <= 0) return fail(DCNV4_ERR_RUNTIME, "im2col_step must be positive");
  const int step = std::min(batch, im2col_step);
  if (batch % step != 0) return fail(DCNV4_ERR_RUNTIME, "batch(%d) must divide im2col_step(%d)", batch, step);
  const int Ho = out_extent(H, ph, dh, kh, sh), Wo = out_extent(W, pw, dw, kw, sw);
  if (Ho <= 0 || Wo <= 0) return fail(DCNV4_ERR_RUNTIME, "kernel does not fit the padded input (output %dx%d)", Ho, Wo);
  if (P_pad < G * Kp * 3)
    return fail(DCNV4_ERR_RUNTIME, "offset_mask last dim %d is smaller than group*K*3 = %d", P_pad, G * Kp * 3);

  DcnLaunch &L = pr->launch;
  L = DcnLaunch{};
  if (int rc = choose_lanes(D, s, d_stride, false, &L.lanes)) return rc;
  const int width = 1 << L.lanes.tpgp_log2;
  if (backward && (width > kWave || D > kMaxBackwardGroupChannels))
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "backward takes groups of up to %d channels in at most 64 lanes of 16 bytes, got %d channels",
                kMaxBackwardGroupChannels, D);
  L.Q = Ho * Wo; L.Wo = Wo; L.H = H; L.W = W; L.G = G; L.D = D;
  L.kh = kh; L.kw = kw; L.sh = sh; L.sw = sw; L.ph = ph; L.pw = pw; L.dh = dh; L.dw = dw;
  L.Kp = Kp; L.P_pad = P_pad; L.remove_center = remove_center; L.softmax = softmax ? 1 : 0;
  L.offset_scale = offset_scale;

  if (int rc = choose_block_pixels(&L, block_thread, backward)) return rc;

  pr->batch = batch; pr->Ho = Ho; pr->Wo = Wo; pr->s = s;
  pr->img_elems = (size_t)H * W * G * D;
  pr->img_out_elems = (size_t)Ho * Wo * G * D;
  pr->img_om_elems = (size_t)Ho * Wo * P_pad;
  if ((uint64_t)pr->img_elems * (backward ? 4 : s) > kMaxSpanBytes)
    return fail(DCNV4_ERR_RUNTIME, "one image of %zu elements exceeds the 2 GiB addressing span of a launch", pr->img_elems);
  return DCNV4_OK;
}

int images_per_launch(const DcnProblem &pr, bool backward) {
  const uint64_t per_img = (uint64_t)pr.img_elems * (backward ? 4 : pr.s);
  uint64_t n = std::max<uint64_t>(1, kMaxSpanBytes / per_img);
  n = std::min<uint64_t>(n, 0x7fffffffull / (uint64_t)pr.launch.Q);   // n_pix stays an int
  return (int)std::min<uint64_t>(n, (uint64_t)pr.batch);
}

// ---------------------------------------------------------------- flash deformable attention
struct FdaProblem {
  FdaLaunch launch;
  int batch, s;
  size_t img_elems, img_row_elems, img_out_elems;
};

int fda_prepare(FdaProblem *pr, bool backward, bool scatter, int dtype, int batch, int N, int G, int D, int L, int Q, int K,
                int im2col_step, int d_stride, int block_thread) {
  const int s = elem_bytes(dtype);
  if (s == 0) return fail(DCNV4_ERR_RUNTIME, "unsupported dtype code %d (fp32, fp16, bf16 only)", dtype);
  if (batch <= 0 || N <= 0 || G <= 0 || D <= 0 || Q <= 0)
    return fail(DCNV4_ERR_RUNTIME, "empty or negative tensor extent (batch %d, spatial %d, heads %d, channels %d, queries %d)",
                batch, N, G, D, Q);
  if (L < 1 || L > kMaxLevels) return fail(DCNV4_ERR_INVALID_ARGUMENT, "invalid number of scales: %d (1..%d)", L, kMaxLevels);
  if (K < 1 || L * K > kMaxTaps)
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "invalid number of points: K=%d with %d levels (L*K <= %d)", K, L, kMaxTaps);
  if (im2col_step <= 0) return fail(DCNV4_ERR_RUNTIME, "im2col_step must be positive");
  const int step = std::min(batch, im2col_step);
  if (batch % step != 0) return fail(DCNV4_ERR_RUNTIME, "batch(%d) must divide im2col_step(%d)", batch, step);

  FdaLaunch &F = pr->launch;
  F = FdaLaunch{};
  // The gather kernels (forward, and the backward in front of the tiled grad_value kernel) take 16-byte lanes whatever
  // the hint: a reference-style d_stride of 1 or 2 would cost them 25-180 % (cfg 4, fp16: forward 0.146 -> 0.233 / 0.407
  // ms, backward 0.584 -> 0.728 / 1.039 ms).  The hint is still checked, and narrows the lanes of the atomic scatter.
  LaneMap hinted;
  if (int rc = choose_lanes(D, s, d_stride, scatter, &hinted)) return rc;
  if (scatter) F.lanes = hinted;
  else if (int rc = choose_lanes(D, s, 0, false, &F.lanes)) return rc;
  const int width = 1 << F.lanes.tpgp_log2;
  if (backward && width > kWave)
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "backward needs head_channels/%d <= 64 lanes per head, got %d",
                F.lanes.cpt, F.lanes.tpg);
  F.Q = Q; F.N = N; F.G = G; F.D = D; F.L = L; F.K = K;
  const int lanes_per_row = G * width;
  const int want = block_thread > 0 ? block_thread : kBlockThreads;
  int nq = std::max(1, want / lanes_per_row);
  const size_t lds_per_row = (size_t)G * 3 * L * K * sizeof(float) * (backward ? 2 : 1);
  while (nq > 1 && nq * lds_per_row > kMaxDynamicLds) --nq;
  if (nq * lds_per_row > kMaxDynamicLds)
    return fail(DCNV4_ERR_RUNTIME, "sampling_loc_attn row of %d x %d elements does not fit in LDS", G, 3 * L * K);
  F.nq_block = nq;

  pr->batch = batch; pr->s = s;
  pr->img_elems = (size_t)N * G * D;
  pr->img_row_elems = (size_t)Q * G * 3 * L * K;
  pr->img_out_elems = (size_t)Q * G * D;
  if ((uint64_t)pr->img_elems * (backward ? 4 : s) > kMaxSpanBytes)
    return fail(DCNV4_ERR_RUNTIME, "one value image of %zu elements exceeds the 2 GiB addressing span of a launch", pr->img_elems);
  return DCNV4_OK;
}

// One head per workgroup, workgroups ordered [image][head][block of queries], when the whole value image does not fit
// an XCD's L2 with room to spare: an XCD then gathers from one head's slice of it at a time.  In the forward also when
// that slice alone exceeds the L2 - it is still an n-th of what the query-row order gathers from (4 images of
// 128x128.., 8 heads of 64 fp32 channels: 0.895 -> 0.453 ms; 100x152.., 2 images: 0.401 -> 0.218 ms).  A workgroup
// takes as many queries as fill it with one head's lanes (and fit the LDS).
void fda_choose_order(FdaLaunch *F, const FdaProblem &pr, int N, int G, int D, int L, int K, bool backward) {
  const size_t line = 128, head_bytes = (size_t)D * pr.s;
  const size_t lines_per_pixel = (std::max(head_bytes, line) + line - 1) / line;      // cache lines a head touches per pixel
  const size_t head_footprint = (size_t)N * lines_per_pixel * line;
  F->head_major = 0;
  if (g_opt.fda_order == 1 || G <= 1) return;
  if (g_opt.fda_order != 2 && (pr.img_elems * pr.s <= kL2BytesPerXcd / 2 || (backward && head_footprint > kL2BytesPerXcd))) return;
  // a decoder's few hundred queries gather too little for the L2 to matter, and one head per workgroup only makes the
  // workgroups small (8 images of 128x128.., 300 queries: 0.024 -> 0.019 ms by query rows)
  if (g_opt.fda_order != 2 && !backward && F->Q < 512) return;
  F->head_major = 1;
  const int width = 1 << F->lanes.tpgp_log2;
  const size_t lds_per_row = (size_t)3 * L * K * sizeof(float) * (backward ? 2 : 1);
  F->nq_block = std::max(1, std::min((backward ? kFdaBackwardThreads : kFdaForwardThreads) / width, (int)(kMaxDynamicLds / lds_per_row)));
  // Forward: the smallest levels of the head's value slice in LDS.  The level shapes live in device memory, so the
  // choice goes by what a pyramid with a factor of two between levels would need: its last level holds about 1.2 %
  // of the pixels (1.5 % asked for).  The kernel stages whatever really fits; with nothing staged it only runs at
  // lower occupancy.
  F->stage_budget = 0;
  if (backward || g_opt.fda_stage == kOptPlain || (head_bytes % 16) != 0 || width > 64) return;
  const size_t rows_bytes = (size_t)(kFdaStagedThreads / width) * lds_per_row;
  if (rows_bytes + 4096 > kMaxLdsPerWorkgroup - 2048) return;
  const size_t budget = std::min<size_t>(kMaxLdsPerWorkgroup - 2048 - rows_bytes, 112 * 1024);
  const bool level_fits = L >= 2 && (size_t)N * head_bytes * 3 / 200 + fda_staged_zero_bytes((int)head_bytes) <= budget;
  // The workgroups of a launch - one per CU, 1024 lanes and most of the LDS each - pass over the chip in two even
  // rounds (other counts leave a partial last round, or stage the levels more often).  Measured forward times,
  // staged against one head per workgroup without staging, 8 heads of 32 channels, fp16 / fp32:
  //   128x128.. 4 levels x 4 points, 4 images  0.142 / 0.294 against 0.172 / 0.215 ms
  //   128x128.. 4 x 8, 4 images                0.309 / 0.519 against 0.327 / 0.393
  //   100x152.. 4 x 8, 2 images                0.141 / 0.169 against 0.158 / 0.185;  8 images 0.678 / 1.09 against 0.573 / 0.694
  //   64x64.. 4 x 8, 8 images                  0.124 / 0.158 against 0.139 / 0.193;  80x80.. 3 x 8, 4 images 0.095 / 0.119 against 0.105 / 0.127
  //   one image (64 workgroups per head, 1.2 rounds of queries each): 2-5 % slower staged
  //   heads of 128 bytes and more with 4 x 4 points: 3-27 % slower staged (100x152.., 2 images, 64 fp16 channels: 0.110
  //   against 0.099 ms); heads of 16 fp32 channels: 15-27 % faster staged on four shapes, 9 % slower on 128x128.. 4 x 8
  // What decides is the L2: the 32 workgroups that an XCD runs at a time belong to 32 / (workgroups per head)
  // consecutive heads, whose slices of the value image (heads of one pixel share 128-byte lines) must stay in its
  // 4 MB together - and every workgroup needs at least two rounds of queries, or the rounds do not divide evenly.
  // Wide heads gain only with long rows (24 points and more per query and head: 80x80.. 3 x 8, 32 fp32 channels
  // 0.119 against 0.128 ms).
  const int pairs = (int)(F->n_row / F->Q) * G;
  const int sub_q = kFdaStagedThreads / width;
  const int cus_per_xcd = kCusPerDevice / 8;
  // Two rounds when the L2 then holds the heads an XCD works on; else twice, four or eight times as many workgroups (more
  // rounds, each workgroup staging again, but fewer heads at a time: 8 images of 100x152.., 4 x 4 points, fp16: 0.302 ms
  // plain, 0.306 ms staged in two rounds, 0.268 ms in four; 16 images of 128x128..: 0.644 / 0.936 / 0.605 ms in eight).
  int blocks = 0;
  bool l2_holds = false, rounds_even = false;
  // (heads of 128 bytes lose 12-13 % when staged in more than two rounds; so do small pyramids, whose head slices the
  // plain kernel's L2 holds several of anyway: 16 images of 80x80.., 0.193 ms plain against 0.232 ms staged in four rounds)
  const int max_mul = head_bytes <= 64 && (size_t)N * line >= kL2BytesPerXcd / 2 ? 8 : 1;
  for (int mul = 1; mul <= max_mul && !(l2_holds && rounds_even); mul *= 2) {
    blocks = std::max(1, 2 * kCusPerDevice / std::max(1, pairs)) * mul;
    const size_t heads_at_once = (size_t)std::max(1, (cus_per_xcd + blocks - 1) / blocks);
    const size_t lines_at_once = (heads_at_once * head_bytes + line - 1) / line;
    l2_holds = (size_t)N * lines_at_once * line <= kL2BytesPerXcd * 3 / 4;
    rounds_even = (long long)(F->Q + sub_q - 1) / sub_q >= 2LL * blocks;
    if (!rounds_even) break;      // more workgroups only shorten the rounds further
  }
  if (!(l2_holds && rounds_even)) blocks = std::max(1, 2 * kCusPerDevice / std::max(1, pairs));      // what a forced staging launches
  const bool width_pays = head_bytes <= 64 || L * K >= 24;
  if (g_opt.fda_stage != kOptTiled && !(level_fits && l2_holds && rounds_even && width_pays)) return;
  F->stage_budget = (int)(budget & ~size_t(15));
  F->stage_blocks = std::max(1, std::min(blocks, (F->Q + sub_q - 1) / sub_q));
}

int images_per_launch(const FdaProblem &pr, bool backward) {
  const uint64_t per_img = (uint64_t)pr.img_elems * (backward ? 4 : pr.s);
  uint64_t n = std::max<uint64_t>(1, kMaxSpanBytes / per_img);
  n = std::min<uint64_t>(n, 0x7fffffffull / (uint64_t)pr.launch.Q);
  return (int)std::min<uint64_t>(n, (uint64_t)pr.batch);
}

int check_ptrs(std::initializer_list<const void *> ptrs) {
  for (const void *p : ptrs) {
    if (p == nullptr) return fail(DCNV4_ERR_RUNTIME, "null tensor pointer");
    if (!aligned16(p)) return fail(DCNV4_ERR_RUNTIME, "tensor pointer %p is not 16-byte aligned", p);
  }
  return DCNV4_OK;
}

// A small parameter vector that the kernels read element by element (a view into a flat parameter buffer need not
// start on a 16-byte boundary).
int check_elem_ptr(const void *p, int elem_bytes_of_ptr) {
  if (p == nullptr) return fail(DCNV4_ERR_RUNTIME, "null tensor pointer");
  if ((reinterpret_cast<uintptr_t>(p) & (uintptr_t)(elem_bytes_of_ptr - 1)) != 0)
    return fail(DCNV4_ERR_RUNTIME, "tensor pointer %p is not aligned to its %d-byte elements", p, elem_bytes_of_ptr);
  return DCNV4_OK;
}

int hip_fail(const char *what, hipError_t e) {
  return fail(DCNV4_ERR_RUNTIME, "%s: %s", what, hipGetErrorString(e));
}


// ---------------------------------------------------------------- depthwise convolution (NHWC)
struct DwProblem {
  DwLaunch launch;         // geometry of one image; B, pointers and partial-sum fields set per launch
  int s;                   // bytes per element
  size_t in_img, out_img;  // elements per image
  int per;                 // images per launch (tensors of a launch stay below 2 GiB)
  int slab;                // row segments per grad_weight workgroup
  size_t total_parts;
};

constexpr int kDwPartTarget = 2048;      // grad_weight partial sums per call, about
constexpr int kDwGradSeg = 8;            // output columns a grad_weight lane walks per visit

int dw_prepare(DwProblem *pr, int dtype, int batch, int H, int W, int C, int k, int pad) {
  const int s = elem_bytes(dtype);
  if (s == 0) return fail(DCNV4_ERR_RUNTIME, "unsupported dtype code %d (fp32, fp16, bf16 only)", dtype);
  if (batch <= 0 || H <= 0 || W <= 0 || C <= 0)
    return fail(DCNV4_ERR_RUNTIME, "empty or negative tensor extent (batch %d, H %d, W %d, channels %d)", batch, H, W, C);
  if (k != 1 && k != 3 && k != 5 && k != 7)
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "depthwise kernel size %d is not supported (1, 3, 5 or 7)", k);
  if (pad < 0 || pad > k - 1) return fail(DCNV4_ERR_INVALID_ARGUMENT, "padding %d does not suit a %dx%d kernel (0..%d)", pad, k, k, k - 1);
  const int Ho = H + 2 * pad - k + 1, Wo = W + 2 * pad - k + 1;
  if (Ho <= 0 || Wo <= 0) return fail(DCNV4_ERR_RUNTIME, "kernel does not fit the padded input (output %dx%d)", Ho, Wo);
  DwLaunch &L = pr->launch;
  L = DwLaunch{};
  L.H = H; L.W = W; L.C = C; L.Ho = Ho; L.Wo = Wo; L.kh = L.kw = k; L.ph = L.pw = pad;
  pr->s = s;
  pr->in_img = (size_t)H * W * C;
  pr->out_img = (size_t)Ho * Wo * C;
  const size_t img_bytes = std::max(pr->in_img, pr->out_img) * s;
  if (img_bytes >= (size_t(1) << 31))
    return fail(DCNV4_ERR_RUNTIME, "one image of %zu bytes exceeds the 2 GiB addressing span of a launch", img_bytes);
  pr->per = (int)std::min<size_t>((size_t)batch, ((size_t(1) << 31) - 1) / img_bytes);
  // grad_weight: a workgroup takes `slab` row segments of kDwGradSeg columns, a whole number of rounds of
  // its pixel lanes, sized for about kDwPartTarget workgroups per call
  L.seg = std::min(kDwGradSeg, Wo);
  L.n_seg = (Wo + L.seg - 1) / L.seg;
  const int lanes = depthwise_grad_weight_pixel_lanes(s, C, k);
  const size_t n_rowseg = (size_t)batch * Ho * L.n_seg;
  const size_t rounds = std::max<size_t>(1, (n_rowseg + (size_t)kDwPartTarget * lanes - 1) / ((size_t)kDwPartTarget * lanes));
  pr->slab = (int)std::min<size_t>(rounds * lanes, 1u << 30);
  pr->total_parts = 0;
  for (int b0 = 0; b0 < batch; b0 += pr->per)
    pr->total_parts += ((size_t)std::min(pr->per, batch - b0) * Ho * L.n_seg + pr->slab - 1) / pr->slab;
  return DCNV4_OK;
}

// output columns per lane: long enough to reuse the sliding window, short enough to fill the GPU
void dw_segments(DwLaunch *L, int elem_bytes_of_launch) {
  const int vec = 16 / elem_bytes_of_launch;
  const size_t lanes_per_col = (size_t)L->B * L->Ho * std::max(1, L->C / vec);
  int seg = 8;
  while (seg > 2 && lanes_per_col * ((L->Wo + seg - 1) / seg) < 256u * 1024u) seg /= 2;
  L->seg = std::min(seg, L->Wo);
  L->n_seg = (L->Wo + L->seg - 1) / L->seg;
}

// ---------------------------------------------------------------- static scratch
// Scratch of dcnv4_gfx950_backward_static_scratch, for callers that cannot allocate: one array per GPU, held from
// the moment the library's code is loaded on that GPU until the process ends.  The name of a __device__ array is
// only a host-side handle; the array's device address is looked up once per device and kept.
constexpr size_t kStaticScratchBytes = DCNV4_GFX950_STATIC_SCRATCH_BYTES;
__device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch_of_current_device(void **out) {
  int dev = -1;
  if (hipError_t e = hipGetDevice(&dev)) return fail(DCNV4_ERR_RUNTIME, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(DCNV4_ERR_RUNTIME, "device ordinal %d is out of range (0..%d)", dev, kMaxDevices - 1);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void *ptr = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch)))
      return fail(DCNV4_ERR_RUNTIME, "hipGetSymbolAddress(static scratch) on device %d: %s", dev, hipGetErrorString(e));
    if (ptr == nullptr || !aligned16(ptr)) return fail(DCNV4_ERR_RUNTIME, "static scratch of device %d has address %p", dev, ptr);
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return DCNV4_OK;
}

const char *at(const void *base, size_t elems, int s) { return static_cast<const char *>(base) + elems * s; }
char *at(void *base, size_t elems, int s) { return static_cast<char *>(base) + elems * s; }

}  // namespace
}  // namespace dcn

using namespace dcn;

extern "C" {

int dcnv4_gfx950_abi_version(void) { return DCNV4_GFX950_ABI_VERSION; }

const char *dcnv4_gfx950_last_error(void) { return g_error; }

static int *launch_option_slot(const char *name) {
  if (name == nullptr) return nullptr;
  if (std::strcmp(name, "gather") == 0) return &g_opt.gather;
  if (std::strcmp(name, "scatter") == 0) return &g_opt.scatter;
  if (std::strcmp(name, "reach") == 0) return &g_opt.reach;
  if (std::strcmp(name, "tile") == 0) return &g_opt.tile;
  if (std::strcmp(name, "gather_tile") == 0) return &g_opt.gather_tile;
  if (std::strcmp(name, "gv_threads") == 0) return &g_opt.gv_threads;
  if (std::strcmp(name, "dual") == 0) return &g_opt.dual;
  if (std::strcmp(name, "fda_order") == 0) return &g_opt.fda_order;
  if (std::strcmp(name, "fda_stage") == 0) return &g_opt.fda_stage;
  return nullptr;
}

int dcnv4_gfx950_set_launch_option(const char *name, int value) {
  int *slot = launch_option_slot(name);
  if (slot == nullptr) return fail(DCNV4_ERR_INVALID_ARGUMENT, "unknown launch option %s", name ? name : "(null)");
  const bool family = value == kOptAuto || value == kOptTiled || value == kOptPlain;
  const bool ok = slot == &g_opt.reach ? (value >= -1 && value <= 64)
                  : slot == &g_opt.tile ? (value == 0 || value == 8 || value == 16 || value == 32)
                  : slot == &g_opt.gather_tile ? (value == 0 || value == 4 || value == 8 || value == 16)
                  : slot == &g_opt.gv_threads ? (value == 0 || value == 512 || value == 1024)
                                        : family;
  if (!ok) return fail(DCNV4_ERR_INVALID_ARGUMENT, "launch option %s does not take the value %d", name, value);
  *slot = value;
  return DCNV4_OK;
}

int dcnv4_gfx950_get_launch_option(const char *name, int *value) {
  const int *slot = launch_option_slot(name);
  if (slot == nullptr || value == nullptr) return fail(DCNV4_ERR_INVALID_ARGUMENT, "unknown launch option %s", name ? name : "(null)");
  *value = *slot;
  return DCNV4_OK;
}

int dcnv4_gfx950_forward(const void *value, const void *offset_mask, void *output, int dtype, int batch,
                         int height_in, int width_in, int group, int group_channels, int kernel_h,
                         int kernel_w, int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h,
                         int dilation_w, float offset_scale, int im2col_step, int remove_center,
                         int padded_offset_dim, int softmax, int d_stride, int block_thread, void *stream) {
  DcnProblem pr;
  if (int rc = dcn_prepare(&pr, false, dtype, batch, height_in, width_in, group, group_channels, kernel_h,
                           kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, offset_scale,
                           im2col_step, remove_center, padded_offset_dim, softmax, d_stride, block_thread))
    return rc;
  if (int rc = check_ptrs({value, offset_mask, output})) return rc;
  const int per = images_per_launch(pr, false);
  const bool tiled = plan_gather_tiles(&pr.launch, pr.s, false);
  for (int b0 = 0; b0 < batch; b0 += per) {
    const int nb = std::min(per, batch - b0);
    DcnLaunch L = pr.launch;
    L.value = at(value, b0 * pr.img_elems, pr.s);
    L.offset_mask = at(offset_mask, b0 * pr.img_om_elems, pr.s);
    L.out = at(output, b0 * pr.img_out_elems, pr.s);
    L.value_bytes = (uint32_t)(nb * pr.img_elems * pr.s);
    L.n_pix = nb * L.Q;
    const hipError_t e = tiled ? launch_dcnv4_forward_tiled(dtype, L, static_cast<hipStream_t>(stream))
                               : launch_dcnv4_forward(dtype, L, static_cast<hipStream_t>(stream));
    if (e) return hip_fail("dcnv4 forward launch", e);
  }
  return DCNV4_OK;
}

size_t dcnv4_gfx950_backward_workspace_bytes(int dtype, int batch, int height_in, int width_in, int group,
                                             int group_channels) {
  if (elem_bytes(dtype) == 0 || batch <= 0 || height_in <= 0 || width_in <= 0 || group <= 0 || group_channels <= 0)
    return 0;
  return kStateBytes;      // a function of nothing: in particular not of the launch options
}

static int dcn_backward_impl(const void *value, const void *offset_mask, const void *grad_output, void *grad_value,
                             void *grad_offset_mask, void *workspace, size_t workspace_bytes, int dtype, int batch,
                             int height_in, int width_in, int group, int group_channels, int kernel_h, int kernel_w,
                             int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w,
                             float offset_scale, int im2col_step, int remove_center, int padded_offset_dim,
                             int softmax, int d_stride, int block_thread, void *stream) {
  DcnProblem pr;
  if (int rc = dcn_prepare(&pr, true, dtype, batch, height_in, width_in, group, group_channels, kernel_h,
                           kernel_w, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w, offset_scale,
                           im2col_step, remove_center, padded_offset_dim, softmax, d_stride, block_thread))
    return rc;
  if (int rc = check_ptrs({value, offset_mask, grad_output, grad_value, grad_offset_mask})) return rc;
  const size_t need = dcnv4_gfx950_backward_workspace_bytes(dtype, batch, height_in, width_in, group, group_channels);
  if (need > 0) {
    if (workspace == nullptr || !aligned16(workspace) || workspace_bytes < need)
      return fail(DCNV4_ERR_RUNTIME, "workspace of %zu bytes needed, got %zu at %p", need, workspace_bytes, workspace);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);

  // state reset, then 1. grad_offset_mask + the reach the sampling points need  2. tiled grad_value (plain stores)
  DcnLaunch base = pr.launch;
  if (int rc = plan_grad_value_tiles(&base, dtype, batch)) return rc;
  // the grad_value kernel addresses one image's offset_mask and grad_out with 32-bit element offsets
  if (base.Q >= (1 << 24) || (uint64_t)base.Q * (uint64_t)base.P_pad >= (1ull << 31) ||
      (uint64_t)base.Q * (uint64_t)(base.G * base.D) >= (1ull << 31))
    return fail(DCNV4_ERR_RUNTIME, "one image of %d output pixels is too large for the backward", base.Q);
  const bool gather_tiled = plan_gather_tiles(&base, pr.s, true);
  base.state = static_cast<GradState *>(workspace);
  // When a grad_value tile is a whole image its workgroups visit every output pixel whatever the reach: nobody reads
  // the statistic that the first kernel folds into the state, and the launch that resets it is left out.
  base.gv_whole = (base.tile_h >= base.H && base.tile_w >= base.W) ? 1 : 0;
  // Otherwise a workgroup of the grad_value kernel visits the output pixels within reach_needed of its tile, one
  // number for the whole call - and one outlier among the offsets must not make every tile scan its surroundings that
  // far.  Points farther than the cap from their reference point stay out of that number; the tiles they land in
  // learn how far to look for them (GradState::far_reach) and only their workgroups visit the pixels in between.
  // The cap exceeds what a staged window of the first kernel spans, so that a point beyond it is always one of the
  // points that kernel serves from memory - where it is folded.
  base.gv_reach_cap = 3.0e38f;
  if (!base.gv_whole) {
    int cap = kReachCap;
    if (gather_tiled) cap = std::max(cap, std::max((base.gt_h - 1) * base.sh, (base.gt_w - 1) * base.sw) + base.gt_reach + 1);
    base.gv_reach_cap = (float)cap;
  }
  if (!base.gv_whole) {
    hipLaunchKernelGGL(init_state_kernel, dim3(1), dim3(64), 0, st, base.state);
    if (hipError_t e = hipGetLastError()) return hip_fail("state init launch", e);
  }
  const int per = images_per_launch(pr, false);
  // both kernels in one launch when they do not depend on each other and the shape suits the two-role kernel
  const bool dual = g_opt.dual != kOptPlain && dcnv4_backward_dual_fits(base, pr.s);
  if (dual) base.dual_interleave = dcnv4_backward_dual_workgroups(base, std::min(per, batch)) <= 3u * kCusPerDevice ? 1 : 0;
  for (int pass = 0; pass < (dual ? 1 : 2); ++pass) {
    for (int b0 = 0; b0 < batch; b0 += per) {
      const int nb = std::min(per, batch - b0);
      DcnLaunch L = base;
      L.value = at(value, b0 * pr.img_elems, pr.s);
      L.offset_mask = at(offset_mask, b0 * pr.img_om_elems, pr.s);
      L.grad_out = at(grad_output, b0 * pr.img_out_elems, pr.s);
      L.grad_value = at(grad_value, b0 * pr.img_elems, pr.s);
      L.grad_offset_mask = at(grad_offset_mask, b0 * pr.img_om_elems, pr.s);
      L.value_bytes = (uint32_t)(nb * pr.img_elems * pr.s);
      L.n_pix = nb * L.Q;
      L.n_img = nb;
      hipError_t e = hipSuccess;
      if (dual) e = launch_dcnv4_backward_dual(dtype, L, st);
      else if (pass == 0 && gather_tiled) e = launch_dcnv4_offset_mask_grad_tiled(dtype, L, st);
      else if (pass == 0) e = launch_dcnv4_offset_mask_grad(dtype, L, st);
      else e = launch_dcnv4_grad_value(dtype, L, st);
      if (e) return hip_fail("dcnv4 backward launch", e);
    }
  }
  return DCNV4_OK;
}

int dcnv4_gfx950_backward(const void *value, const void *offset_mask, const void *grad_output, void *grad_value,
                          void *grad_offset_mask, void *workspace, size_t workspace_bytes, int dtype, int batch,
                          int height_in, int width_in, int group, int group_channels, int kernel_h, int kernel_w,
                          int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w,
                          float offset_scale, int im2col_step, int remove_center, int padded_offset_dim,
                          int softmax, int d_stride, int block_thread, void *stream) {
  return dcn_backward_impl(value, offset_mask, grad_output, grad_value, grad_offset_mask, workspace, workspace_bytes, dtype,
                           batch, height_in, width_in, group, group_channels, kernel_h, kernel_w, stride_h, stride_w, pad_h,
                           pad_w, dilation_h, dilation_w, offset_scale, im2col_step, remove_center, padded_offset_dim,
                           softmax, d_stride, block_thread, stream);
}

int dcnv4_gfx950_backward_static_scratch(const void *value, const void *offset_mask, const void *grad_output,
                                         void *grad_value, void *grad_offset_mask, int dtype, int batch, int height_in,
                                         int width_in, int group, int group_channels, int kernel_h, int kernel_w,
                                         int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h,
                                         int dilation_w, float offset_scale, int im2col_step, int remove_center,
                                         int padded_offset_dim, int softmax, int d_stride, int block_thread,
                                         void *stream) {
  const size_t need = dcnv4_gfx950_backward_workspace_bytes(dtype, batch, height_in, width_in, group, group_channels);
  if (need > kStaticScratchBytes)
    return fail(DCNV4_ERR_RUNTIME,
                "this backward needs %zu bytes of scratch; the library's static scratch holds %zu "
                "(use dcnv4_gfx950_backward with a caller-provided workspace)", need, kStaticScratchBytes);
  void *scratch = nullptr;
  if (int rc = static_scratch_of_current_device(&scratch)) return rc;
  return dcn_backward_impl(value, offset_mask, grad_output, grad_value, grad_offset_mask, scratch, kStaticScratchBytes, dtype,
                           batch, height_in, width_in, group, group_channels, kernel_h, kernel_w, stride_h, stride_w, pad_h,
                           pad_w, dilation_h, dilation_w, offset_scale, im2col_step, remove_center, padded_offset_dim,
                           softmax, d_stride, block_thread, stream);
}

// Rows of a (query, head): either one packed tensor (sla) or locations + logits (loc, logits; the locations in fp32
// or in the tensor dtype).
struct FdaRows {
  const void *sla, *loc, *logits;
  void *grad_sla, *grad_loc, *grad_logits;
  int loc_bytes;      // 0: packed rows
};

static void fda_set_rows(FdaLaunch *F, const FdaRows &r, const FdaProblem &pr, int b0, int LK) {
  const size_t pairs = (size_t)b0 * F->Q * F->G;
  F->sla = r.sla ? at(r.sla, b0 * pr.img_row_elems, pr.s) : nullptr;
  F->grad_sla = r.grad_sla ? at(r.grad_sla, b0 * pr.img_row_elems, pr.s) : nullptr;
  F->loc = r.loc ? at(r.loc, pairs * 2 * LK, r.loc_bytes) : nullptr;
  F->grad_loc = r.grad_loc ? at(r.grad_loc, pairs * 2 * LK, r.loc_bytes) : nullptr;
  F->logits = r.logits ? at(r.logits, pairs * LK, pr.s) : nullptr;
  F->grad_logits = r.grad_logits ? at(r.grad_logits, pairs * LK, pr.s) : nullptr;
  F->loc_f32 = r.loc_bytes == 4 ? 1 : 0;
}

static int fda_check_split(int dtype, int location_dtype, int *loc_bytes) {
  if (elem_bytes(dtype) == 0) return fail(DCNV4_ERR_RUNTIME, "unsupported dtype code %d (fp32, fp16, bf16 only)", dtype);
  if (location_dtype != DCNV4_DTYPE_F32 && location_dtype != dtype)
    return fail(DCNV4_ERR_RUNTIME, "sampling locations must be fp32 or of the value's dtype (codes %d, %d)", location_dtype, dtype);
  *loc_bytes = elem_bytes(location_dtype);
  return DCNV4_OK;
}

static int fda_forward_impl(const void *value, const int64_t *spatial_shapes, const int64_t *level_start_index,
                            const FdaRows &rows, void *output, int dtype, int batch, int spatial_size, int num_heads,
                            int head_channels, int num_levels, int num_query, int num_points, int im2col_step,
                            int d_stride, int block_thread, void *stream) {
  FdaProblem pr;
  if (int rc = fda_prepare(&pr, false, false, dtype, batch, spatial_size, num_heads, head_channels, num_levels, num_query,
                           num_points, im2col_step, d_stride, block_thread))
    return rc;
  if (int rc = rows.loc_bytes == 0 ? check_ptrs({value, rows.sla, output}) : check_ptrs({value, rows.loc, rows.logits, output})) return rc;
  if (spatial_shapes == nullptr || level_start_index == nullptr) return fail(DCNV4_ERR_RUNTIME, "null level tensors");
  const int per = images_per_launch(pr, false);
  for (int b0 = 0; b0 < batch; b0 += per) {
    const int nb = std::min(per, batch - b0);
    FdaLaunch F = pr.launch;
    F.value = at(value, b0 * pr.img_elems, pr.s);
    fda_set_rows(&F, rows, pr, b0, num_levels * num_points);
    F.out = at(output, b0 * pr.img_out_elems, pr.s);
    F.shapes = spatial_shapes;
    F.level_start = level_start_index;
    F.value_bytes = (uint32_t)(nb * pr.img_elems * pr.s);
    F.n_row = nb * F.Q;
    fda_choose_order(&F, pr, spatial_size, num_heads, head_channels, num_levels, num_points, false);
    if (hipError_t e = launch_fda_forward(dtype, F, static_cast<hipStream_t>(stream)))
      return hip_fail("flash_deform_attn forward launch", e);
  }
  return DCNV4_OK;
}

int flash_deform_attn_gfx950_forward(const void *value, const int64_t *spatial_shapes,
                                     const int64_t *level_start_index, const void *sampling_loc_attn,
                                     void *output, int dtype, int batch, int spatial_size, int num_heads,
                                     int head_channels, int num_levels, int num_query, int num_points,
                                     int im2col_step, int d_stride, int block_thread, void *stream) {
  const FdaRows rows{sampling_loc_attn, nullptr, nullptr, nullptr, nullptr, nullptr, 0};
  return fda_forward_impl(value, spatial_shapes, level_start_index, rows, output, dtype, batch, spatial_size, num_heads,
                          head_channels, num_levels, num_query, num_points, im2col_step, d_stride, block_thread, stream);
}

int flash_deform_attn_gfx950_forward_split(const void *value, const int64_t *spatial_shapes,
                                           const int64_t *level_start_index, const void *sampling_locations,
                                           const void *attention_logits, void *output, int dtype, int location_dtype,
                                           int batch, int spatial_size, int num_heads, int head_channels,
                                           int num_levels, int num_query, int num_points, int im2col_step,
                                           int d_stride, int block_thread, void *stream) {
  int loc_bytes = 0;
  if (int rc = fda_check_split(dtype, location_dtype, &loc_bytes)) return rc;
  const FdaRows rows{nullptr, sampling_locations, attention_logits, nullptr, nullptr, nullptr, loc_bytes};
  return fda_forward_impl(value, spatial_shapes, level_start_index, rows, output, dtype, batch, spatial_size, num_heads,
                          head_channels, num_levels, num_query, num_points, im2col_step, d_stride, block_thread, stream);
}

// Scratch of the tiled attention backward, in this order: GradState, keys, point records, grad_out regrouped by head,
// tile table, sorted point lists.  The last two are sized for the images of one launch and reused by the next.
struct FdaScratch {
  size_t keys, recs, go_rows, table, regions, total;     // byte offsets, total bytes
  int n_chunks, tile_stride, per;
};

FdaScratch fda_scratch(int s, int batch, int N, int G, int D, int L, int Q, int K) {
  FdaScratch sc;
  const uint64_t per_img = (uint64_t)N * G * D * 4;
  uint64_t per = std::max<uint64_t>(1, kMaxSpanBytes / per_img);
  per = std::min<uint64_t>(per, 0x7fffffffull / (uint64_t)Q);
  sc.per = (int)std::min<uint64_t>(per, (uint64_t)batch);
  const size_t points = (size_t)G * L * fda_key_stride(Q, K);          // per image
  sc.n_chunks = (int)(((size_t)Q * K + kFdaChunkPoints - 1) / kFdaChunkPoints);
  // a level of H x W cells is cut into tiles of min(8, ceil(dim / 4)) cells per side: at most N/8 + 64 tiles
  sc.tile_stride = (int)std::min<size_t>(kFdaMaxTilesPerLevel, (size_t)N / 8 + 64);
  const size_t segs = (size_t)sc.per * G * L * sc.n_chunks;
  sc.keys = kStateBytes;
  sc.recs = sc.keys + round16((size_t)batch * points * sizeof(uint16_t));
  sc.go_rows = sc.recs + round16((size_t)batch * points * 16);
  sc.table = sc.go_rows + round16((size_t)batch * G * Q * D * s);
  sc.regions = sc.table + round16(segs * sc.tile_stride * sizeof(uint32_t));
  sc.total = sc.regions + round16(segs * 4 * kFdaChunkPoints * sizeof(uint32_t));
  return sc;
}

size_t flash_deform_attn_gfx950_backward_workspace_bytes(int dtype, int batch, int spatial_size, int num_heads,
                                                         int head_channels, int num_levels, int num_query,
                                                         int num_points) {
  if (elem_bytes(dtype) == 0 || batch <= 0 || spatial_size <= 0 || num_heads <= 0 || head_channels <= 0) return 0;
  size_t need = 0;
  // 16-bit tensors: an fp32 image of grad_value behind the state block (the atomic paths sum in fp32 and narrow once)
  if (elem_bytes(dtype) == 2) need = kStateBytes + round16((size_t)batch * spatial_size * num_heads * head_channels * sizeof(float));
  if (fda_tiled_shape(head_channels, num_levels, num_query, num_points))
    need = std::max(need, fda_scratch(elem_bytes(dtype), batch, spatial_size, num_heads, head_channels, num_levels, num_query, num_points).total);
  return need;
}

static int fda_backward_impl(const void *value, const int64_t *spatial_shapes, const int64_t *level_start_index,
                             const FdaRows &rows, const void *grad_output, void *grad_value, void *workspace,
                             size_t workspace_bytes, int dtype, int batch, int spatial_size, int num_heads,
                             int head_channels, int num_levels, int num_query, int num_points, int im2col_step,
                             int d_stride, int block_thread, void *stream) {
  FdaProblem pr;
  // the tiled grad_value kernel addresses one image's sampling_loc_attn and grad_out with 32-bit byte offsets
  const unsigned long long row_bytes = (unsigned long long)std::max(num_heads, 1) *
                                       std::max(3 * num_levels * num_points, head_channels) * 4ull;
  // fp32 tensors with few sampling points per image (a decoder's few hundred queries against an encoder's pyramid):
  // the atomic scatter adds straight into grad_value and is done before the binned kernels have walked the pyramid's
  // tiles (2 images of 100x152.., 100 queries: 0.028 against 0.057 ms; 900 queries: 0.107 against 0.067 ms)
  const bool sparse = g_opt.scatter == kOptAuto && elem_bytes(dtype) == 4 &&
                      3ll * num_query * num_levels * num_points < (long long)spatial_size;
  const bool tiled = fda_tiled_shape(head_channels, num_levels, num_query, num_points) && fda_tiled_enabled() && !sparse &&
                     (unsigned long long)num_query * row_bytes < (1ull << 31);
  // the tiled path gathers only: 16-byte lanes; the atomic path wants one channel per lane
  if (int rc = fda_prepare(&pr, true, !tiled, dtype, batch, spatial_size, num_heads, head_channels, num_levels, num_query,
                           num_points, im2col_step, d_stride, block_thread))
    return rc;
  if (int rc = rows.loc_bytes == 0 ? check_ptrs({value, rows.sla, grad_output, grad_value, rows.grad_sla})
                        : check_ptrs({value, rows.loc, rows.logits, grad_output, grad_value, rows.grad_loc, rows.grad_logits}))
    return rc;
  if (spatial_shapes == nullptr || level_start_index == nullptr) return fail(DCNV4_ERR_RUNTIME, "null level tensors");
  const size_t need = flash_deform_attn_gfx950_backward_workspace_bytes(dtype, batch, spatial_size, num_heads, head_channels,
                                                                        num_levels, num_query, num_points);
  if (need > 0) {
    if (workspace == nullptr || !aligned16(workspace) || workspace_bytes < need)
      return fail(DCNV4_ERR_RUNTIME, "workspace of %zu bytes needed, got %zu at %p", need, workspace_bytes, workspace);
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t total = (size_t)batch * pr.img_elems;
  const int per = images_per_launch(pr, true);      // equals FdaScratch::per

  if (tiled) {
    // pass 0: grad_sampling_loc_attn, keys, point records, regrouped grad_out; pass 1: tiled grad_value; pass 2: fallback
    FdaLaunch base = pr.launch;
    base.state = static_cast<GradState *>(workspace);
    const FdaScratch sc = fda_scratch(pr.s, batch, spatial_size, num_heads, head_channels, num_levels, num_query, num_points);
    const size_t img_keys = (size_t)num_heads * num_levels * fda_key_stride(num_query, num_points);
    char *ws = static_cast<char *>(workspace);
    uint16_t *keys = reinterpret_cast<uint16_t *>(ws + sc.keys);
    f32x4_t *recs = reinterpret_cast<f32x4_t *>(ws + sc.recs);
    char *go_rows = ws + sc.go_rows;
    base.table = reinterpret_cast<uint32_t *>(ws + sc.table);
    base.regions = reinterpret_cast<uint32_t *>(ws + sc.regions);
    base.n_chunks = sc.n_chunks;
    base.tile_stride = sc.tile_stride;
    // The state block (the binning kernel's flag) is cleared by the first kernel itself, which runs to its end
    // before the binning kernel starts.  The fallback - three launches that return at once without the flag - can
    // only be needed when a level has more tiles than the binning kernel counts (kFdaMaxTilesPerLevel); tiles have
    // at least 8 cells (a level of up to four rows is cut into 1 x 8 pieces), so a tensor of fewer cells than that
    // many tiles' worth cannot raise the flag and the launches are left out.
    const bool fallback_possible = (size_t)spatial_size / 8 + 64 > (size_t)kFdaMaxTilesPerLevel;
    for (int pass = 0; pass < (fallback_possible ? 3 : 2); ++pass) {
      for (int b0 = 0; b0 < batch; b0 += per) {
        const int nb = std::min(per, batch - b0);
        FdaLaunch F = base;
        F.value = at(value, b0 * pr.img_elems, pr.s);
        fda_set_rows(&F, rows, pr, b0, num_levels * num_points);
        F.grad_out = at(grad_output, b0 * pr.img_out_elems, pr.s);
        F.grad_value = at(grad_value, b0 * pr.img_elems, pr.s);
        F.keys = keys + b0 * img_keys;
        F.recs = recs + b0 * img_keys;
        F.go_rows = go_rows + (size_t)b0 * pr.img_out_elems * pr.s;
        F.shapes = spatial_shapes;
        F.level_start = level_start_index;
        F.value_bytes = (uint32_t)(nb * pr.img_elems * pr.s);
        F.n_row = nb * F.Q;
        F.n_img = nb;
        hipError_t e = hipSuccess;
        if (pass == 0) fda_choose_order(&F, pr, spatial_size, num_heads, head_channels, num_levels, num_points, true);
        F.clear_state = (pass == 0 && b0 == 0) ? 1 : 0;
        if (pass == 0) e = launch_fda_backward(dtype, F, kFdaNoScatter, st);
        else if (pass == 1) {
          for (int c0 = 0; c0 < head_channels && e == hipSuccess; c0 += kFdaWindowChannels) {
            F.gv_c0 = c0;
            F.gv_dc = std::min(kFdaWindowChannels, head_channels - c0);
            e = launch_fda_grad_value(dtype, F, st);
          }
        } else {
          // The fallback sums with fp32 atomics: straight into grad_value for fp32 tensors (the tiled kernel has left
          // it zeroed), for 16-bit tensors into an fp32 image that takes the place of the - by now dead - keys and
          // records, is cleared first and narrowed afterwards; all three launches return at once without the flag.
          const size_t n = (size_t)nb * pr.img_elems;      // a multiple of 8: heads of whole 8-channel blocks
          float *acc = pr.s == 2 ? reinterpret_cast<float *>(ws + kStateBytes) + (size_t)b0 * pr.img_elems : static_cast<float *>(F.grad_value);
          F.grad_value_acc = acc;
          const dim3 grid((unsigned)std::min<size_t>((n / 8 + 255) / 256, 4096)), block(256);
          if (pr.s == 2) hipLaunchKernelGGL(clear_if_flagged_kernel, grid, block, 0, st, base.state, reinterpret_cast<uint32_t *>(acc), n / 4);
          e = launch_fda_backward(dtype, F, kFdaFallback, st);
          if (e == hipSuccess && dtype == DCNV4_DTYPE_F16)
            hipLaunchKernelGGL(narrow_if_flagged_kernel<F16>, grid, block, 0, st, base.state, acc, F.grad_value, n / 8);
          if (e == hipSuccess && dtype == DCNV4_DTYPE_BF16)
            hipLaunchKernelGGL(narrow_if_flagged_kernel<BF16>, grid, block, 0, st, base.state, acc, F.grad_value, n / 8);
          if (e == hipSuccess) e = hipGetLastError();
        }
        if (e) return hip_fail("flash_deform_attn backward launch", e);
      }
    }
    return DCNV4_OK;
  }

  const bool widen = pr.s == 2;
  float *acc = widen ? static_cast<float *>(workspace) : static_cast<float *>(grad_value);
  if (hipError_t e = clear_async(acc, total, st)) return hip_fail("clear launch", e);
  for (int b0 = 0; b0 < batch; b0 += per) {
    const int nb = std::min(per, batch - b0);
    FdaLaunch F = pr.launch;
    F.value = at(value, b0 * pr.img_elems, pr.s);
    fda_set_rows(&F, rows, pr, b0, num_levels * num_points);
    F.grad_out = at(grad_output, b0 * pr.img_out_elems, pr.s);
    F.grad_value_acc = acc + b0 * pr.img_elems;
    F.shapes = spatial_shapes;
    F.level_start = level_start_index;
    F.value_bytes = (uint32_t)(nb * pr.img_elems * pr.s);
    F.n_row = nb * F.Q;
    if (hipError_t e = launch_fda_backward(dtype, F, kFdaFull, st)) return hip_fail("flash_deform_attn backward launch", e);
  }
  if (widen)
    if (hipError_t e = narrow_async(dtype, acc, grad_value, total, st)) return hip_fail("cast launch", e);
  return DCNV4_OK;
}

int flash_deform_attn_gfx950_backward(const void *value, const int64_t *spatial_shapes,
                                      const int64_t *level_start_index, const void *sampling_loc_attn,
                                      const void *grad_output, void *grad_value, void *grad_sampling_loc_attn,
                                      void *workspace, size_t workspace_bytes, int dtype, int batch,
                                      int spatial_size, int num_heads, int head_channels, int num_levels,
                                      int num_query, int num_points, int im2col_step, int d_stride,
                                      int block_thread, void *stream) {
  const FdaRows rows{sampling_loc_attn, nullptr, nullptr, grad_sampling_loc_attn, nullptr, nullptr, 0};
  return fda_backward_impl(value, spatial_shapes, level_start_index, rows, grad_output, grad_value, workspace, workspace_bytes,
                           dtype, batch, spatial_size, num_heads, head_channels, num_levels, num_query, num_points,
                           im2col_step, d_stride, block_thread, stream);
}

int flash_deform_attn_gfx950_backward_split(const void *value, const int64_t *spatial_shapes,
                                            const int64_t *level_start_index, const void *sampling_locations,
                                            const void *attention_logits, const void *grad_output, void *grad_value,
                                            void *grad_sampling_locations, void *grad_attention_logits,
                                            void *workspace, size_t workspace_bytes, int dtype, int location_dtype,
                                            int batch, int spatial_size, int num_heads, int head_channels,
                                            int num_levels, int num_query, int num_points, int im2col_step,
                                            int d_stride, int block_thread, void *stream) {
  int loc_bytes = 0;
  if (int rc = fda_check_split(dtype, location_dtype, &loc_bytes)) return rc;
  const FdaRows rows{nullptr, sampling_locations, attention_logits, nullptr, grad_sampling_locations, grad_attention_logits, loc_bytes};
  return fda_backward_impl(value, spatial_shapes, level_start_index, rows, grad_output, grad_value, workspace, workspace_bytes,
                           dtype, batch, spatial_size, num_heads, head_channels, num_levels, num_query, num_points,
                           im2col_step, d_stride, block_thread, stream);
}

int dcnv4_gfx950_depthwise_conv_forward(const void *input, const void *weight, const void *bias, void *output,
                                        int dtype, int batch, int height, int width, int channels, int kernel_size,
                                        int pad, void *stream) {
  DwProblem pr;
  if (int rc = dw_prepare(&pr, dtype, batch, height, width, channels, kernel_size, pad)) return rc;
  if (int rc = check_ptrs({input, weight, output})) return rc;
  if (bias != nullptr && !aligned16(bias)) return fail(DCNV4_ERR_RUNTIME, "tensor pointer %p is not 16-byte aligned", bias);
  hipStream_t st = static_cast<hipStream_t>(stream);
  for (int b0 = 0; b0 < batch; b0 += pr.per) {
    DwLaunch L = pr.launch;
    L.B = std::min(pr.per, batch - b0);
    L.in = at(input, b0 * pr.in_img, pr.s);
    L.out = at(output, b0 * pr.out_img, pr.s);
    L.weight = weight;
    L.bias = bias;
    dw_segments(&L, pr.s);
    if (hipError_t e = launch_depthwise_forward(dtype, L, st)) return hip_fail("depthwise forward launch", e);
  }
  return DCNV4_OK;
}

size_t dcnv4_gfx950_depthwise_conv_backward_workspace_bytes(int dtype, int batch, int height, int width, int channels,
                                                            int kernel_size, int pad) {
  DwProblem pr;
  if (dw_prepare(&pr, dtype, batch, height, width, channels, kernel_size, pad)) return 0;
  return round16(pr.total_parts * (size_t)(kernel_size * kernel_size + 1) * channels * sizeof(float));
}

int dcnv4_gfx950_depthwise_conv_backward(const void *input, const void *weight, const void *grad_output, void *grad_input,
                                         void *grad_weight, void *grad_bias, void *workspace, size_t workspace_bytes,
                                         int dtype, int batch, int height, int width, int channels, int kernel_size,
                                         int pad, void *stream) {
  DwProblem pr;
  if (int rc = dw_prepare(&pr, dtype, batch, height, width, channels, kernel_size, pad)) return rc;
  if (int rc = check_ptrs({grad_output})) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (grad_input != nullptr) {
    // correlation of grad_output with the flipped kernel, padding k - 1 - pad: output extent = the input's
    if (int rc = check_ptrs({weight, grad_input})) return rc;
    for (int b0 = 0; b0 < batch; b0 += pr.per) {
      DwLaunch L = pr.launch;
      L.B = std::min(pr.per, batch - b0);
      L.H = pr.launch.Ho; L.W = pr.launch.Wo; L.Ho = pr.launch.H; L.Wo = pr.launch.W;
      L.ph = L.pw = kernel_size - 1 - pad;
      L.flip = 1;
      L.in = at(grad_output, b0 * pr.out_img, pr.s);
      L.out = at(grad_input, b0 * pr.in_img, pr.s);
      L.weight = weight;
      L.bias = nullptr;
      dw_segments(&L, pr.s);
      if (hipError_t e = launch_depthwise_forward(dtype, L, st)) return hip_fail("depthwise grad_input launch", e);
    }
  }
  if (grad_weight != nullptr) {
    if (int rc = check_ptrs({input, grad_weight})) return rc;
    const size_t row = (size_t)(kernel_size * kernel_size + 1) * channels;
    const size_t need = round16(pr.total_parts * row * sizeof(float));
    if (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))
      return fail(DCNV4_ERR_RUNTIME, "workspace of %zu bytes needed, got %zu at %p", need, workspace_bytes, workspace);
    size_t parts_done = 0;
    for (int b0 = 0; b0 < batch; b0 += pr.per) {
      DwLaunch L = pr.launch;
      L.B = std::min(pr.per, batch - b0);
      L.in = at(input, b0 * pr.in_img, pr.s);
      L.grad_out = at(grad_output, b0 * pr.out_img, pr.s);
      L.slab = pr.slab;
      L.n_part = (int)(((size_t)L.B * L.Ho * L.n_seg + pr.slab - 1) / pr.slab);
      L.partial = static_cast<float *>(workspace) + parts_done * row;
      if (hipError_t e = launch_depthwise_grad_weight_partials(dtype, L, st)) return hip_fail("depthwise grad_weight launch", e);
      parts_done += (size_t)L.n_part;
    }
    DwLaunch L = pr.launch;
    L.partial = static_cast<float *>(workspace);
    L.n_part = (int)parts_done;
    L.grad_weight = grad_weight;
    L.grad_bias = grad_bias;
    if (hipError_t e = launch_depthwise_grad_weight_reduce(dtype, L, st)) return hip_fail("depthwise grad_weight reduction launch", e);
  }
  return DCNV4_OK;
}

// Row geometry shared by the layer-norm forward and backward: a team of lanes per row, 16-byte vectors per lane.
static int ln_prepare(LnLaunch *L, int dtype, long long rows, int channels, float eps) {
  const int s = elem_bytes(dtype);
  if (s == 0) return fail(DCNV4_ERR_RUNTIME, "unsupported dtype code %d (fp32, fp16, bf16 only)", dtype);
  if (rows <= 0 || channels <= 0) return fail(DCNV4_ERR_RUNTIME, "empty or negative extent (rows %lld, channels %d)", rows, channels);
  const int V = 16 / s;
  if (channels % V != 0) return fail(DCNV4_ERR_INVALID_ARGUMENT, "channels (%d) must be a multiple of %d for this dtype", channels, V);
  const int nvec = channels / V;
  if (nvec > 64 * 8) return fail(DCNV4_ERR_INVALID_ARGUMENT, "rows of %d channels are too long (at most %d)", channels, 64 * 8 * V);
  *L = LnLaunch{};
  L->rows = rows; L->C = channels; L->eps = eps;
  L->team = 1;
  while (L->team < 64 && L->team < nvec) L->team *= 2;
  L->vpl = 1;
  while (L->team * L->vpl < nvec) L->vpl *= 2;
  // backward: about 2048 workgroups at most, each a slab of whole passes; partial sums stay below 32 MB
  const long long rows_per_pass = 256 / L->team;
  long long parts = std::min<long long>((rows + rows_per_pass - 1) / rows_per_pass, 2048);
  while (parts > 1 && (size_t)parts * 3 * channels * sizeof(float) > (size_t(32) << 20)) parts /= 2;
  L->slab = ((rows + parts - 1) / parts + rows_per_pass - 1) / rows_per_pass * rows_per_pass;
  L->n_part = (int)((rows + L->slab - 1) / L->slab);
  return DCNV4_OK;
}

int dcnv4_gfx950_layer_norm_residual_forward(const void *input, const void *residual, const void *weight,
                                             const void *bias, const void *gamma, void *output, int dtype,
                                             long long rows, int channels, float eps, void *stream) {
  LnLaunch L;
  if (int rc = ln_prepare(&L, dtype, rows, channels, eps)) return rc;
  if (int rc = check_ptrs({input, weight, bias, output})) return rc;
  if ((residual != nullptr && !aligned16(residual)) || (gamma != nullptr && !aligned16(gamma)))
    return fail(DCNV4_ERR_RUNTIME, "tensor pointer is not 16-byte aligned");
  L.y = input; L.residual = residual; L.weight = weight; L.bias = bias; L.gamma = gamma; L.out = output;
  if (hipError_t e = launch_layer_norm_residual(dtype, L, static_cast<hipStream_t>(stream)))
    return hip_fail("layer norm launch", e);
  return DCNV4_OK;
}

size_t dcnv4_gfx950_layer_norm_residual_backward_workspace_bytes(int dtype, long long rows, int channels) {
  LnLaunch L;
  if (ln_prepare(&L, dtype, rows, channels, 0.f)) return 0;
  return round16((size_t)L.n_part * 3 * channels * sizeof(float));
}

int dcnv4_gfx950_layer_norm_residual_backward(const void *grad_output, const void *input, const void *weight,
                                              const void *bias, const void *gamma, void *grad_input,
                                              void *grad_weight, void *grad_bias, void *grad_gamma, void *workspace,
                                              size_t workspace_bytes, int dtype, long long rows, int channels,
                                              float eps, void *stream) {
  LnLaunch L;
  if (int rc = ln_prepare(&L, dtype, rows, channels, eps)) return rc;
  if (int rc = check_ptrs({grad_output, input, weight, grad_input})) return rc;
  if (gamma != nullptr && bias == nullptr) return fail(DCNV4_ERR_RUNTIME, "the gradient of gamma needs the bias of the normalisation");
  for (const void *q : {bias, gamma, (const void *)grad_weight, (const void *)grad_bias, (const void *)grad_gamma})
    if (q != nullptr && !aligned16(q)) return fail(DCNV4_ERR_RUNTIME, "tensor pointer %p is not 16-byte aligned", q);
  if (grad_gamma != nullptr && gamma == nullptr) return fail(DCNV4_ERR_RUNTIME, "grad_gamma asked for without gamma");
  const size_t need = round16((size_t)L.n_part * 3 * channels * sizeof(float));
  if (workspace == nullptr || !aligned16(workspace) || workspace_bytes < need)
    return fail(DCNV4_ERR_RUNTIME, "workspace of %zu bytes needed, got %zu at %p", need, workspace_bytes, workspace);
  L.grad_out = grad_output; L.y = input; L.weight = weight; L.bias = bias; L.gamma = gamma;
  L.grad_y = grad_input; L.grad_weight = grad_weight; L.grad_bias = grad_bias; L.grad_gamma = grad_gamma;
  L.partial = static_cast<float *>(workspace);
  if (hipError_t e = launch_layer_norm_residual_backward(dtype, L, static_cast<hipStream_t>(stream)))
    return hip_fail("layer norm backward launch", e);
  return DCNV4_OK;
}

static int cf_prepare(CfLaunch *L, int dtype, long long rows, int channels, int groups) {
  const int s = elem_bytes(dtype);
  if (s == 0) return fail(DCNV4_ERR_RUNTIME, "unsupported dtype code %d (fp32, fp16, bf16 only)", dtype);
  if (rows <= 0 || channels <= 0 || groups <= 0)
    return fail(DCNV4_ERR_RUNTIME, "empty or negative extent (rows %lld, channels %d, groups %d)", rows, channels, groups);
  const int V = 16 / s;
  if (channels % groups != 0) return fail(DCNV4_ERR_INVALID_ARGUMENT, "%d channels cannot be split into %d equal groups", channels, groups);
  const int D = channels / groups;
  if (D % V != 0) return fail(DCNV4_ERR_INVALID_ARGUMENT, "group width (%d) must be a multiple of %d for this dtype", D, V);
  const int nvec = channels / V;
  if (nvec > 64 * 8) return fail(DCNV4_ERR_INVALID_ARGUMENT, "rows of %d channels are too long (at most %d)", channels, 64 * 8 * V);
  *L = CfLaunch{};
  L->rows = rows; L->C = channels; L->G = groups; L->D = D;
  L->team = 1;
  while (L->team < 64 && L->team < nvec) L->team *= 2;
  L->vpl = 1;
  while (L->team * L->vpl < nvec) L->vpl *= 2;
  return DCNV4_OK;
}

int dcnv4_gfx950_center_feature_blend_forward(const void *sampled, const void *projected, const void *weight,
                                              const void *bias, void *output, int dtype, long long rows,
                                              int channels, int groups, void *stream) {
  CfLaunch L;
  if (int rc = cf_prepare(&L, dtype, rows, channels, groups)) return rc;
  if (int rc = check_ptrs({sampled, projected, weight, output})) return rc;
  if (int rc = check_elem_ptr(bias, elem_bytes(dtype))) return rc;      // read with scalar loads
  L.y = sampled; L.x = projected; L.weight = weight; L.bias = bias; L.out = output;
  if (hipError_t e = launch_center_feature_blend(dtype, L, false, static_cast<hipStream_t>(stream)))
    return hip_fail("centre-feature blend launch", e);
  return DCNV4_OK;
}

int dcnv4_gfx950_center_feature_blend_backward(const void *grad_output, const void *sampled, const void *projected,
                                               const void *weight, const void *bias, void *grad_sampled,
                                               void *grad_projected, float *grad_gate_logits, int dtype,
                                               long long rows, int channels, int groups, void *stream) {
  CfLaunch L;
  if (int rc = cf_prepare(&L, dtype, rows, channels, groups)) return rc;
  if (int rc = check_ptrs({grad_output, sampled, projected, weight, grad_sampled, grad_projected, grad_gate_logits})) return rc;
  if (int rc = check_elem_ptr(bias, elem_bytes(dtype))) return rc;
  L.grad_out = grad_output; L.y = sampled; L.x = projected; L.weight = weight; L.bias = bias;
  L.grad_y = grad_sampled; L.grad_x = grad_projected; L.grad_logits = grad_gate_logits;
  if (hipError_t e = launch_center_feature_blend(dtype, L, true, static_cast<hipStream_t>(stream)))
    return hip_fail("centre-feature blend backward launch", e);
  return DCNV4_OK;
}

int dcnv4_gfx950_lds_read_probe(int pattern, int iters, unsigned int *ticks_per_1000_reads, void *stream) {
  if (pattern < 0 || pattern > 4 || iters < 1 || iters > (1 << 20))
    return fail(DCNV4_ERR_INVALID_ARGUMENT, "LDS read probe: pattern %d (0..4), %d rounds (1..2^20)", pattern, iters);
  if (ticks_per_1000_reads == nullptr) return fail(DCNV4_ERR_RUNTIME, "null tensor pointer");
  hipLaunchKernelGGL(lds_read_probe_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream), pattern, iters, ticks_per_1000_reads);
  if (hipError_t e = hipGetLastError()) return hip_fail("LDS read probe launch", e);
  return DCNV4_OK;
}

int dcnv4_gfx950_stream_copy(const void *src, void *dst, size_t bytes, void *stream) {
  if (int rc = check_ptrs({src, dst})) return rc;
  if (bytes % 16 != 0) return fail(DCNV4_ERR_INVALID_ARGUMENT, "stream copy takes a multiple of 16 bytes, got %zu", bytes);
  const size_t n16 = bytes / 16;
  if (n16 == 0) return DCNV4_OK;
  const size_t blocks = (n16 + 1023) / 1024;
  if (blocks > 0x7fffffffull) return fail(DCNV4_ERR_RUNTIME, "stream copy of %zu bytes is too large for one launch", bytes);
  hipLaunchKernelGGL(stream_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const u32x4 *>(src), static_cast<u32x4 *>(dst), n16);
  if (hipError_t e = hipGetLastError()) return hip_fail("stream copy launch", e);
  return DCNV4_OK;
}

}  // extern "C"
