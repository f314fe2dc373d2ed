// Device code of the LDS-tiled gathers (dcnv4_tiled_gather.hip holds the kernels and their launchers; the backward's
// body is also part of the two-role kernel in dcnv4_backward_dual.hip).
#pragma once
// DCNv4 forward and grad_offset_mask with the gather served from LDS.
//
// The reference's forward (DCNv4_op/src/cuda/dcnv4_im2col_cuda.cuh:142-244) fetches four vectors
// per sampling point straight from global memory: 36 scattered 32-byte segments per (pixel,
// group).  On MI355X that pattern is bound by the vector-memory address path, an order of
// magnitude below what HBM delivers.  Sampling points stay close to their output pixel, so here
//
//   * a workgroup owns a tile of gt_h x gt_w output pixels of one image for gt_ng groups and
//     copies the input window those pixels can reach (their reference points +- gt_reach input
//     pixels, clipped to the image plus a one-pixel ring of zeros) into LDS with coalesced
//     128-bit loads; cells outside the image come back as zeros from the buffer range check;
//   * the workgroup's slice of offset_mask is parked in LDS next to it, in the tensor dtype;
//   * one lane owns all D channels of one (pixel, group) - or half of them when a group is 64 bytes
//     or wider, which doubles the waves that hide LDS latency: the bilinear set-up is done once
//     (twice) per sampling point instead of once per 16-byte channel chunk, at most one DPP add
//     crosses lanes, and the four corners are read from LDS with ds_read_b128;
//   * a sampling point whose corners leave the window is remembered in a per-lane bit mask and
//     served afterwards from global memory (the range-checked gather of dcnv4_kernels.hip), so
//     any offset is handled; with offsets inside the window that code never runs.
// The softmax variant of the modulation (dcnv4_im2col_cuda.cuh:173-193, dcnv4_col2im_cuda.cuh:352-365; never
// requested by the reference's Python side) runs on the instantiations for a run-time kernel shape (KP == 0) only, so
// that the 3x3 instantiations carry nothing for it.
#include <type_traits>

#include "common.hpp"
#include "launch.hpp"


namespace dcn {
namespace {

constexpr int kTiledThreads = 512;      // lanes per workgroup at most: leaves each wave 128+ registers

// n / d for 0 <= n < 2^20 with inv = rcp(d) (one instruction, accurate to an ulp): the exact
// quotient sits at least 0.5/d away from the next integer, far more than the error of the product.
__device__ __forceinline__ float rcp(float d) { return __builtin_amdgcn_rcpf(d); }
__device__ __forceinline__ int fdiv(int n, float inv) { return (int)(((float)n + 0.5f) * inv); }

// a.lo * b.lo + a.hi * b.hi + c for two packed 16-bit elements per word, products and sum in fp32
template <typename Tag>
__device__ __forceinline__ float dot2_pair(uint32_t a, uint32_t b, float c) {
  if constexpr (Tag::kCode == F16::kCode) return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, a), __builtin_bit_cast(f16x2, b), c, false);
  else return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, a), __builtin_bit_cast(bf16x2, b), c, false);
}

template <typename Tag>
__device__ __forceinline__ float lds_elem(const typename RawWord<Tag::kBytes>::type *p, int i) {
  float f[1];
  Pack<Tag, 1>::decode(p[i], f);
  return f[0];
}

// Geometry of one workgroup: its output tile, its group chunk and the input window it stages.
struct TileGeom {
  int b, g0, ng;           // image (within the launch), first group, groups in this chunk
  int oy0, ox0, th, tw;    // output tile origin and extent inside the image
  int wy0, wx0, wh, ww;    // input window origin (may be -1) and extent in cells
};

__device__ __forceinline__ TileGeom tile_geometry(const DcnLaunch &p, uint32_t bid, uint32_t nblocks) {
  TileGeom t;
  const int Ho = p.Q / p.Wo;
  const int n_chunks = (p.G + p.gt_ng - 1) / p.gt_ng;
  const int nty = (Ho + p.gt_h - 1) / p.gt_h, ntx = (p.Wo + p.gt_w - 1) / p.gt_w;
  uint32_t id = xcd_contiguous_block(bid, nblocks);
  const int chunk = id % n_chunks; id /= n_chunks;
  const int tx = id % ntx; id /= ntx;
  const int ty = id % nty;
  t.b = id / nty;
  t.g0 = chunk * p.gt_ng;
  t.ng = min(p.gt_ng, p.G - t.g0);
  t.oy0 = ty * p.gt_h; t.ox0 = tx * p.gt_w;
  t.th = min(p.gt_h, Ho - t.oy0); t.tw = min(p.gt_w, p.Wo - t.ox0);
  // reference points (centre tap at zero offset) of the tile's first and last pixel
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
  const int yc0 = half_h - p.ph + t.oy0 * p.sh, yc1 = yc0 + (t.th - 1) * p.sh;
  const int xc0 = half_w - p.pw + t.ox0 * p.sw, xc1 = xc0 + (t.tw - 1) * p.sw;
  t.wy0 = max(yc0 - p.gt_reach, -1); t.wx0 = max(xc0 - p.gt_reach, -1);
  t.wh = max(min(yc1 + p.gt_reach, p.H) - t.wy0 + 1, 0);
  t.ww = max(min(xc1 + p.gt_reach, p.W) - t.wx0 + 1, 0);
  return t;
}

// offset_mask / grad_offset_mask slices of a tile move in whole dwords when a pixel's run starts on a dword boundary
// in memory and in LDS and either ends on one or has room for one element more: behind the last group the row is
// padded, and a chunk with fewer groups than gt_ng leaves its LDS slice partly unused.
template <typename Tag>
__device__ __forceinline__ bool tile_runs_in_dwords(const DcnLaunch &p, const TileGeom &t) {
  if constexpr (Tag::kBytes == 4) return true;
  const int run = t.ng * 3 * p.Kp, lds_row = p.gt_ng * 3 * p.Kp;
  if (((p.P_pad | (t.g0 * 3 * p.Kp) | lds_row) & 1) != 0) return false;
  return (run & 1) == 0 || (run + 1 <= lds_row && t.g0 * 3 * p.Kp + run + 1 <= p.P_pad);
}

// Fills the workgroup's LDS: the input window and this chunk's slice of offset_mask.
//
// Window: [wy0, wy0+wh) x [wx0, wx0+ww) of this chunk's channels, cell-major (cell = all channels
// of the chunk for one input pixel, cell_stride bytes apart), followed by ww + 2 cells of zeros
// that serve every corner of a sampling point that must contribute nothing.
// offset_mask: tile pixel q, group gl of the chunk -> s_om[(q * gt_ng + gl) * 3 * Kp ...], in the
// tensor dtype, untouched.
//
// The time of this phase is memory latency and address arithmetic, so: a lane keeps its place
// inside a row (window row: cell and 16-byte piece; tile row: pixel and dword) and only the row
// advances, by a uniform step; rows outside the image and idle lanes read through the dropped
// offset of the buffer descriptor; and a lane issues a batch of loads before it stores any.
template <typename Tag, int NV>
__device__ __forceinline__ void stage_tile(const DcnLaunch &p, const TileGeom &t, char *s_win,
                                           typename RawWord<Tag::kBytes>::type *s_om, int cell_stride) {
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int kBatch = 8;
  const int bd = blockDim.x, tid = threadIdx.x;

  // ---- offset_mask slices: geometry, and the first batch of loads, which is requested before the window's loads so
  // that both fly together (the phase is a chain of load latencies, not of bytes; measured the other way round,
  // window first, the phase is slower than without any overlap)
  constexpr int EPW = 4 / Tag::kBytes;
  constexpr int kOmBatch = 16;
  const int run = t.ng * 3 * p.Kp, lds_row = p.gt_ng * 3 * p.Kp;          // elements per pixel: copied / LDS stride
  const elem_t *om = reinterpret_cast<const elem_t *>(p.offset_mask) + ((size_t)t.b * p.Q + (size_t)t.oy0 * p.Wo + t.ox0) * p.P_pad +
                     t.g0 * 3 * p.Kp;                                      // first element of the tile's slice
  // whole dwords when every run starts on a dword boundary (always for fp32); a run of an odd number of 16-bit
  // elements - the last chunk of an odd number of groups - takes the element behind it along, which lies in the row's
  // padding and has room in the LDS slice
  const bool dwords = tile_runs_in_dwords<Tag>(p, t);
  const int rw = (run + EPW - 1) / EPW;                                   // dwords per pixel
  int team_log2 = 0;
  while ((1 << team_log2) < rw) ++team_log2;
  const bool teams = dwords && (1 << team_log2) <= bd;
  // a power-of-two team of lanes per tile pixel; the tile's rows are row_bytes apart in memory
  const uint32_t om_row_bytes = (uint32_t)p.Wo * p.P_pad * Tag::kBytes;
  const __amdgpu_buffer_rsrc_t om_rows = make_rsrc(om, teams ? (uint32_t)(t.th - 1) * om_row_bytes + (uint32_t)((t.tw - 1) * p.P_pad + rw * EPW) * Tag::kBytes : 0u);
  uint32_t *s_om_w = reinterpret_cast<uint32_t *>(s_om);
  const int ppp = max(bd >> team_log2, 1);                                // pixels per pass
  const int pl = tid >> team_log2, j = tid & ((1 << team_log2) - 1);
  auto om_request = [&](int px0, int py0, uint32_t (&raw)[kOmBatch]) {
    const int px = px0 + pl;
    const uint32_t g_lane = (px < t.tw && j < rw) ? (uint32_t)(px * p.P_pad) * Tag::kBytes + 4u * j : kDropOffset;
#pragma unroll
    for (int u = 0; u < kOmBatch / 2; ++u)
      raw[u] = buffer_load<4>(om_rows, (py0 + u < t.th && g_lane != kDropOffset) ? g_lane + (uint32_t)(py0 + u) * om_row_bytes : kDropOffset);
    if (t.th - py0 > kOmBatch / 2) {        // uniform: short tiles request half a batch
#pragma unroll
      for (int u = kOmBatch / 2; u < kOmBatch; ++u)
        raw[u] = buffer_load<4>(om_rows, (py0 + u < t.th && g_lane != kDropOffset) ? g_lane + (uint32_t)(py0 + u) * om_row_bytes : kDropOffset);
    }
  };
  auto om_park = [&](int px0, int py0, const uint32_t (&raw)[kOmBatch]) {
    const int px = px0 + pl;
    if (!(px < t.tw && j < rw)) return;
    const int l_lane = px * (lds_row / EPW) + j;
#pragma unroll
    for (int u = 0; u < kOmBatch; ++u)
      if (py0 + u < t.th) s_om_w[l_lane + (py0 + u) * (p.gt_w * (lds_row / EPW))] = raw[u];
  };
  uint32_t om_first[kOmBatch];
  if (teams) om_request(0, 0, om_first);

  // ---- window
  {
    const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);
    const uint32_t pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
    const uint32_t img_base = (uint32_t)t.b * (uint32_t)(p.H * p.W) * pix_bytes + (uint32_t)(t.g0 * p.D) * Tag::kBytes;
    const int ppc = t.ng * (p.D * Tag::kBytes / 16);     // 16-byte pieces per cell
    const int row_pieces = max(t.ww * ppc, 1);
    const int rpp = max(bd / row_pieces, 1);             // window rows per pass
    const int lanes_pp = min(bd, row_pieces);            // lanes of one row in one pass
    const int col_passes = (row_pieces + bd - 1) / bd;   // > 1 only when a row is longer than the workgroup
    const int r = fdiv(tid, rcp((float)row_pieces));    // row within the pass (0 when a row is longer)
    for (int cp = 0; cp < col_passes; ++cp) {
      const int rem = (col_passes == 1 ? tid - r * row_pieces : tid) + cp * lanes_pp;
      const int wx = fdiv(rem, rcp((float)ppc)), piece = rem - wx * ppc;
      const int x = t.wx0 + wx;
      const bool lane_ok = (col_passes == 1 ? r < rpp : true) && rem < row_pieces;
      const bool x_in = lane_ok && (unsigned)x < (unsigned)p.W;
      const uint32_t g_lane = img_base + (uint32_t)x * pix_bytes + (uint32_t)piece * 16u;
      const int l_lane = wx * cell_stride + piece * 16;
      const int rows_step = col_passes == 1 ? rpp : 1;
      for (int row0 = 0; row0 < t.wh; row0 += kBatch * rows_step) {
        u32x4 raw[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int wy = row0 + u * rows_step + (col_passes == 1 ? r : 0), y = t.wy0 + wy;
          const bool in = x_in && wy < t.wh && (unsigned)y < (unsigned)p.H;
          raw[u] = buffer_load<16>(value, in ? g_lane + (uint32_t)(y * p.W) * pix_bytes : kDropOffset);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int wy = row0 + u * rows_step + (col_passes == 1 ? r : 0);
          if (lane_ok && wy < t.wh) *reinterpret_cast<u32x4 *>(s_win + l_lane + wy * (t.ww * cell_stride)) = raw[u];
        }
      }
    }
    const int zero_base = t.wh * t.ww * cell_stride;
    const int n_zero = (t.ww + 2) * cell_stride / 16;
    for (int i = tid; i < n_zero; i += bd)
      *reinterpret_cast<u32x4 *>(s_win + zero_base + i * 16) = u32x4{0u, 0u, 0u, 0u};
  }

  // ---- offset_mask slices: the rest
  if (teams) {
    om_park(0, 0, om_first);
    for (int px0 = 0; px0 < t.tw; px0 += ppp)
      for (int py0 = px0 == 0 ? kOmBatch : 0; py0 < t.th; py0 += kOmBatch) {
        uint32_t raw[kOmBatch];
        om_request(px0, py0, raw);
        om_park(px0, py0, raw);
      }
  } else {            // odd alignments and very long rows: element by element
    const int npx = p.gt_h * p.gt_w;
    const float inv_run = rcp((float)run), inv_gtw = rcp((float)p.gt_w);
    for (int idx = tid; idx < npx * run; idx += bd) {
      const int q = fdiv(idx, inv_run), jj = idx - q * run;
      const int py = fdiv(q, inv_gtw), px = q - py * p.gt_w;
      if (py < t.th && px < t.tw) s_om[q * lds_row + jj] = om[((size_t)py * p.Wo + px) * p.P_pad + jj];
    }
  }
}

// Writes the gradient slices parked in LDS (layout of stage_tile) back to grad_offset_mask, and
// zeros the padding tail of the rows when this workgroup owns the last group.
template <typename Tag>
__device__ __forceinline__ void unstage_tile_grads(const DcnLaunch &p, const TileGeom &t,
                                                   const typename RawWord<Tag::kBytes>::type *s_om) {
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int EPW = 4 / Tag::kBytes;
  const int bd = blockDim.x, tid = threadIdx.x;
  const int run = t.ng * 3 * p.Kp, lds_row = p.gt_ng * 3 * p.Kp;
  elem_t *gom = reinterpret_cast<elem_t *>(p.grad_offset_mask) + ((size_t)t.b * p.Q + (size_t)t.oy0 * p.Wo + t.ox0) * p.P_pad +
                t.g0 * 3 * p.Kp;
  const bool dwords = tile_runs_in_dwords<Tag>(p, t);
  const int rw = (run + EPW - 1) / EPW;
  const bool odd_run = (run % EPW) != 0;      // the last dword's upper half lies in the padding: its gradient is zero
  int team_log2 = 0;
  while ((1 << team_log2) < rw) ++team_log2;
  if (dwords && (1 << team_log2) <= bd) {
    const uint32_t row_bytes = (uint32_t)p.Wo * p.P_pad * Tag::kBytes;
    const __amdgpu_buffer_rsrc_t rows = make_rsrc(gom, (uint32_t)(t.th - 1) * row_bytes + (uint32_t)((t.tw - 1) * p.P_pad + rw * EPW) * Tag::kBytes);
    const uint32_t *s_om_w = reinterpret_cast<const uint32_t *>(s_om);
    // fp32 gradients leave with the nontemporal hint (T stage 1 backward 0.187 -> 0.181 ms); with 16-bit tensors the
    // same hint costs 1-3 %
    constexpr int kStorePolicy = Tag::kBytes == 4 ? 2 : 0;
    const int ppp = bd >> team_log2;
    const int pl = tid >> team_log2, j = tid & ((1 << team_log2) - 1);
    for (int px0 = 0; px0 < t.tw; px0 += ppp) {
      const int px = px0 + pl;
      if (px < t.tw && j < rw) {
        const uint32_t g_lane = (uint32_t)(px * p.P_pad) * Tag::kBytes + 4u * j;
        const int l_lane = px * (lds_row / EPW) + j;
        const uint32_t keep = (odd_run && j == rw - 1) ? 0xffffu : 0xffffffffu;
        for (int py = 0; py < t.th; ++py)
          __builtin_amdgcn_raw_buffer_store_b32(s_om_w[l_lane + py * (p.gt_w * (lds_row / EPW))] & keep, rows,
                                                g_lane + (uint32_t)py * row_bytes, 0, kStorePolicy);
      }
    }
  } else {
    const int npx = p.gt_h * p.gt_w;
    const float inv_run = rcp((float)run), inv_gtw = rcp((float)p.gt_w);
    for (int idx = tid; idx < npx * run; idx += bd) {
      const int q = fdiv(idx, inv_run), jj = idx - q * run;
      const int py = fdiv(q, inv_gtw), px = q - py * p.gt_w;
      if (py < t.th && px < t.tw) gom[((size_t)py * p.Wo + px) * p.P_pad + jj] = s_om[q * lds_row + jj];
    }
  }
  const int tail = p.P_pad - p.G * 3 * p.Kp;
  if (tail > 0 && t.g0 + t.ng == p.G) {
    const float inv_tail = rcp((float)tail), inv_tw = rcp((float)t.tw);
    for (int idx = tid; idx < t.th * t.tw * tail; idx += bd) {
      const int q = fdiv(idx, inv_tail), jj = idx - q * tail;
      const int py = fdiv(q, inv_tw), px = q - py * t.tw;
      gom[((size_t)py * p.Wo + px) * p.P_pad + run + jj] = elem_t(0);
    }
  }
}

// Two adjacent lanes that share a (pixel, group) - each with half of its channels - also share the work per sampling
// point that does not depend on the channel: of every two points the even lane prepares the first and the odd lane
// the second, and both read what the other prepared with a DPP move (J = 0: the even lane's value, 1: the odd lane's).
template <int J> __device__ __forceinline__ int pair_pick(int v) {
  return __builtin_amdgcn_update_dpp(0, v, J == 0 ? 0xA0 : 0xF5, 0xf, 0xf, true);      // quad_perm [J, J, 2 + J, 2 + J]
}
template <int J> __device__ __forceinline__ float pair_pick(float v) {
  return __builtin_bit_cast(float, pair_pick<J>(__builtin_bit_cast(int, v)));
}

// One sampling point against the staged window.
struct WinTap {
  float w[4];          // bilinear weights of the four corners (without the modulation)
  float ly, lx;
  int addr;            // LDS byte address of corner 0 for this lane's channels (the zero cells when !ok)
  int ry, rx;          // corner 0 relative to the window origin
  bool inside, ok;     // passes the reference's range test / and both corner rows and columns are staged
};

__device__ __forceinline__ WinTap window_tap(float y, float x, int H, int W, const TileGeom &t, int cell_stride,
                                             int lane_bytes, int zero_base) {
  WinTap r;
  r.inside = (y > -1.f) && (x > -1.f) && (y < (float)H) && (x < (float)W);       // dcnv4_im2col_cuda.cuh:227
  y = r.inside ? y : 0.f;
  x = r.inside ? x : 0.f;
  const float fy = floorf(y), fx = floorf(x);
  const int ry = (int)fy - t.wy0, rx = (int)fx - t.wx0;
  r.ry = ry; r.rx = rx;
  r.ly = y - fy; r.lx = x - fx;
  const float hy = 1.f - r.ly, hx = 1.f - r.lx;
  r.w[0] = hy * hx; r.w[1] = hy * r.lx; r.w[2] = r.ly * hx; r.w[3] = r.ly * r.lx;
  const bool near = (unsigned)ry < (unsigned)max(t.wh - 1, 0) && (unsigned)rx < (unsigned)max(t.ww - 1, 0);
  r.ok = r.inside && near;
  r.addr = r.ok ? __mul24(ry, __mul24(t.ww, cell_stride)) + __mul24(rx, cell_stride) + lane_bytes : zero_base;      // two full-rate 24-bit multiply-adds
  return r;
}

template <typename Tag, int NV, int KP, bool PAIR>      // PAIR: gt_lpg == 2 and KP > 0
__global__ void __launch_bounds__(kTiledThreads) dcnv4_forward_tiled_kernel(const DcnLaunch p) {
  extern __shared__ u32x4 lds128[];
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int EPV = 16 / Tag::kBytes;           // elements per 16-byte vector
  typedef Pack<Tag, EPV> pack;
  const TileGeom t = tile_geometry(p, blockIdx.x, gridDim.x);
  const int Kp = p.Kp;
  const int cell_stride = p.gt_ng * p.D * Tag::kBytes + p.gt_pad;
  char *s_win = reinterpret_cast<char *>(lds128);
  elem_t *s_om = reinterpret_cast<elem_t *>(s_win + (size_t)(p.gt_wh * p.gt_ww + p.gt_ww + 2) * cell_stride);
  stage_tile<Tag, NV>(p, t, s_win, s_om, cell_stride);
  __syncthreads();

  // lane -> (tile pixel, group of the chunk, part): gt_lpg (1 or 2) adjacent lanes share one (pixel, group),
  // each with NV of its 16-byte vectors
  const int part = threadIdx.x & (p.gt_lpg - 1), unit = threadIdx.x >> (p.gt_lpg - 1);
  const int q = fdiv(unit, rcp((float)p.gt_ng)), gl = unit - q * p.gt_ng;
  const int py = fdiv(q, rcp((float)p.gt_w)), px = q - py * p.gt_w;
  if (q >= p.gt_h * p.gt_w || gl >= t.ng || py >= t.th || px >= t.tw) return;
  const int ho = t.oy0 + py, wo = t.ox0 + px;
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
  const float x_base = sub_rn((float)(half_w - p.pw + wo * p.sw), mul_rn((float)half_w, p.offset_scale));
  const float y_base = sub_rn((float)(half_h - p.ph + ho * p.sh), mul_rn((float)half_h, p.offset_scale));
  const elem_t *om = s_om + unit * 3 * Kp;
  const int zero_base = t.wh * t.ww * cell_stride, row_bytes = t.ww * cell_stride;
  const int lane_bytes = gl * p.D * Tag::kBytes + part * NV * 16;
  float acc[NV][EPV];
#pragma unroll
  for (int v = 0; v < NV; ++v)
#pragma unroll
    for (int c = 0; c < EPV; ++c) acc[v][c] = 0.f;
  typedef typename std::conditional<(KP > 0), uint32_t, uint64_t>::type mask_t;     // one bit per sampling point
  mask_t far_mask = 0;
  // softmax over the group's modulation logits: running maximum and reciprocal sum, the probabilities are recomputed per tap
  float sm_max = 0.f, sm_inv = 1.f;
  if constexpr (KP == 0) {
    if (p.softmax) {
      sm_max = lds_elem<Tag>(om, 2 * Kp);
      for (int k = 1; k < Kp; ++k) sm_max = fmaxf(sm_max, lds_elem<Tag>(om, 2 * Kp + k));
      float sum = 0.f;
      for (int k = 0; k < Kp; ++k) sum += __expf(lds_elem<Tag>(om, 2 * Kp + k) - sm_max);
      sm_inv = 1.f / sum;
    }
  }

  auto position = [&](int k, int i, int j, float &y, float &x, float &m) {
    x = add_rn(x_base, mul_rn(add_rn((float)(i * p.dw), lds_elem<Tag>(om, 2 * k)), p.offset_scale));
    y = add_rn(y_base, mul_rn(add_rn((float)(j * p.dh), lds_elem<Tag>(om, 2 * k + 1)), p.offset_scale));
    m = lds_elem<Tag>(om, 2 * Kp + k);
    if constexpr (KP == 0) {
      if (p.softmax) m = __expf(m - sm_max) * sm_inv;
    }
  };
  // A sampling point in flight: its four modulated corner weights and its LDS reads.
  struct Flight {
    float w[4];
    u32x4 raw[4][NV];
  };
  auto issue = [&](int k, int i, int j, Flight &fl) {
    float y, x, m;
    position(k, i, j, y, x, m);
    const WinTap wt = window_tap(y, x, p.H, p.W, t, cell_stride, lane_bytes, zero_base);
    far_mask |= (mask_t)(wt.inside && !wt.ok) << k;
#pragma unroll
    for (int cn = 0; cn < 4; ++cn) {
      fl.w[cn] = m * wt.w[cn];
      const char *src = s_win + wt.addr + (cn & 1) * cell_stride + (cn >> 1) * row_bytes;
#pragma unroll
      for (int v = 0; v < NV; ++v) fl.raw[cn][v] = *reinterpret_cast<const u32x4 *>(src + 16 * v);
    }
  };
  auto retire = [&](const Flight &fl) {
#pragma unroll
    for (int cn = 0; cn < 4; ++cn) {
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        float f[EPV];
        pack::decode(fl.raw[cn][v], f);
#pragma unroll
        for (int c = 0; c < EPV; ++c) acc[v][c] = fmaf(fl.w[cn], f[c], acc[v][c]);
      }
    }
  };
  // a sampling point whose corners lie outside the staged window: gather from memory instead
  const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);
  const uint32_t pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
  const uint32_t img_base = (uint32_t)t.b * (uint32_t)(p.H * p.W) * pix_bytes + (uint32_t)((t.g0 + gl) * p.D) * Tag::kBytes + (uint32_t)(part * NV * 16);
  auto far_tap = [&](int k, int i, int j) {
    float y, x, m;
    position(k, i, j, y, x, m);
    const Tap tp = make_tap(y, x, p.H, p.W, img_base, pix_bytes);
#pragma unroll
    for (int cn = 0; cn < 4; ++cn) {
      const float w = m * tp.w[cn];
#pragma unroll
      for (int v = 0; v < NV; ++v) {
        float f[EPV];
        pack::decode(buffer_load<16>(value, tp.off[cn] + 16u * v), f);      // a dropped corner stays out of range
#pragma unroll
        for (int c = 0; c < EPV; ++c) acc[v][c] = fmaf(w, f[c], acc[v][c]);
      }
    }
  };

  if constexpr (KP > 0) {
    // A real loop, one sampling point at a time: unrolled, the compiler front-loads all 72 LDS reads
    // and spills, and keeping two points in flight by hand costs more in registers (occupancy) than
    // the overlap returns; other waves cover the LDS latency.
    int k_first = 0;
    if constexpr (PAIR) {
      const int common_bytes = lane_bytes - part * NV * 16, part_bytes = part * NV * 16;
#pragma unroll 1
      for (int k0 = 0; k0 + 1 < KP; k0 += 2) {
        int i, j;
        tap_ij_3x3(KP, k0 + part, i, j);
        float y, x, m;
        position(k0 + part, i, j, y, x, m);
        const WinTap wt = window_tap(y, x, p.H, p.W, t, cell_stride, common_bytes, zero_base);
        const int far_own = wt.inside && !wt.ok;
        float wq[4];
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) wq[cn] = m * wt.w[cn];
        auto one = [&](auto jj) {
          constexpr int J = decltype(jj)::value;
          far_mask |= (mask_t)pair_pick<J>(far_own) << (k0 + J);
          const int addr = pair_pick<J>(wt.addr) + part_bytes;
          Flight fl;
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) {
            fl.w[cn] = pair_pick<J>(wq[cn]);
            const char *src = s_win + addr + (cn & 1) * cell_stride + (cn >> 1) * row_bytes;
#pragma unroll
            for (int v = 0; v < NV; ++v) fl.raw[cn][v] = *reinterpret_cast<const u32x4 *>(src + 16 * v);
          }
          retire(fl);
        };
        one(std::integral_constant<int, 0>{});
        one(std::integral_constant<int, 1>{});
      }
      k_first = KP & ~1;      // an odd last point: both lanes prepare it
    }
#pragma unroll 1
    for (int k = k_first; k < KP; ++k) {
      int i, j;
      tap_ij_3x3(KP, k, i, j);
      Flight fl;
      issue(k, i, j, fl);
      retire(fl);
    }
    if (far_mask != 0) {
      for (int k = 0; k < KP; ++k) {
        if (!((far_mask >> k) & 1)) continue;
        int i, j;
        tap_ij_3x3(KP, k, i, j);
        far_tap(k, i, j);
      }
    }
  } else {
    for (int pass = 0; pass < 2; ++pass) {
      if (pass == 1 && far_mask == 0) break;
      int k = 0;
      for (int i = 0; i < p.kw; ++i)
        for (int j = 0; j < p.kh; ++j) {
          if (p.remove_center && i == p.kw / 2 && j == p.kh / 2) continue;
          if (pass == 0) {
            Flight fl;
            issue(k, i, j, fl);
            retire(fl);
          } else if ((far_mask >> k) & 1) {
            far_tap(k, i, j);
          }
          ++k;
        }
    }
  }

  char *dst = (char *)p.out + (((size_t)t.b * p.Q + (size_t)ho * p.Wo + wo) * (p.G * p.D) + (t.g0 + gl) * p.D) * Tag::kBytes + part * NV * 16;
#pragma unroll
  for (int v = 0; v < NV; ++v) *reinterpret_cast<u32x4 *>(dst + 16 * v) = pack::encode(acc[v]);
}

// ------------------------------------------------------------------------------- backward
// grad_offset_mask from the staged window (the part of dcnv4_col2im_cuda.cuh:280-350 and
// common.h:188-211 that does not scatter): for every sampling point the four corner . grad_out
// dot products give d/dx, d/dy and d/dmask.  One lane holds all D channels of its (pixel, group),
// so nothing is reduced across lanes.  The gradients replace the lane's own offset_mask slice in
// LDS (each slot is read before it is overwritten) and the slices go back to memory as rows;
// the workgroup that owns the last groups also clears the padding tail of its rows.  The kernel
// also folds the reach the grad_value kernel has to cover into GradState.
// (the body of the kernel as a function of the workgroup's number, so that a grid can also hold workgroups of another role)
template <typename Tag, int NV, int KP, bool PAIR>      // PAIR: gt_lpg == 2 and KP > 0
__device__ __forceinline__ void dcnv4_offset_mask_grad_tiled_body(const DcnLaunch &p, uint32_t bid, uint32_t nblocks) {
  extern __shared__ u32x4 lds128[];
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int EPV = 16 / Tag::kBytes;
  typedef Pack<Tag, EPV> pack;
  const TileGeom t = tile_geometry(p, bid, nblocks);
  const int Kp = p.Kp;
  const int cell_stride = p.gt_ng * p.D * Tag::kBytes + p.gt_pad;
  char *s_win = reinterpret_cast<char *>(lds128);
  elem_t *s_om = reinterpret_cast<elem_t *>(s_win + (size_t)(p.gt_wh * p.gt_ww + p.gt_ww + 2) * cell_stride);
  __shared__ uint32_t s_reach;
  if (threadIdx.x == 0) s_reach = 0u;

  // lane -> (tile pixel, group of the chunk); its grad_out vector is requested before the staging
  const int part = threadIdx.x & (p.gt_lpg - 1), unit = threadIdx.x >> (p.gt_lpg - 1);
  const int q = fdiv(unit, rcp((float)p.gt_ng)), gl = unit - q * p.gt_ng;
  const int py = fdiv(q, rcp((float)p.gt_w)), px = q - py * p.gt_w;
  const bool active = q < p.gt_h * p.gt_w && gl < t.ng && py < t.th && px < t.tw;
  const int ho = t.oy0 + py, wo = t.ox0 + px;
  u32x4 go_raw[NV];
  {
    const char *src = (const char *)p.grad_out +
                      (((size_t)t.b * p.Q + (size_t)(active ? ho * p.Wo + wo : 0)) * (p.G * p.D) + (active ? t.g0 + gl : 0) * p.D) * Tag::kBytes +
                      part * NV * 16;
#pragma unroll
    for (int v = 0; v < NV; ++v) go_raw[v] = *reinterpret_cast<const u32x4 *>(src + 16 * v);
  }
  stage_tile<Tag, NV>(p, t, s_win, s_om, cell_stride);
  __syncthreads();

  uint32_t reach_needed = 0;
  uint32_t reach_bits = 0;      // bit pattern of the largest distance so far: non-negative floats order like their bits
  if (active) {
    float go[NV][EPV];
#pragma unroll
    for (int v = 0; v < NV; ++v) pack::decode(go_raw[v], go[v]);
    const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
    const int p0y = half_h - p.ph + ho * p.sh, p0x = half_w - p.pw + wo * p.sw;      // reference point
    const float p0xf = (float)p0x, p0yf = (float)p0y;
    const float x_base = sub_rn(p0xf, mul_rn((float)half_w, p.offset_scale));
    const float y_base = sub_rn(p0yf, mul_rn((float)half_h, p.offset_scale));
    elem_t *om = s_om + unit * 3 * Kp;
    const int zero_base = t.wh * t.ww * cell_stride, row_bytes = t.ww * cell_stride;
    const int lane_bytes = gl * p.D * Tag::kBytes + part * NV * 16;
    // the two lanes of a (pixel, group) add their halves of each dot product (known at compile time for the 3x3 instantiations)
    const bool pair = KP > 0 ? PAIR : p.gt_lpg == 2;
    typedef typename std::conditional<(KP > 0), uint32_t, uint64_t>::type mask_t;
    mask_t far_mask = 0;
    // softmax over the group's modulation logits (KP == 0 only): statistics before the slots turn into gradients;
    // sm_dot collects sum_k p_k * dL/dp_k in the lane that writes, for the Jacobian at the end
    float sm_max = 0.f, sm_inv = 1.f, sm_dot = 0.f;
    if constexpr (KP == 0) {
      if (p.softmax) {
        sm_max = lds_elem<Tag>(om, 2 * Kp);
        for (int k = 1; k < Kp; ++k) sm_max = fmaxf(sm_max, lds_elem<Tag>(om, 2 * Kp + k));
        float sum = 0.f;
        for (int k = 0; k < Kp; ++k) sum += __expf(lds_elem<Tag>(om, 2 * Kp + k) - sm_max);
        sm_inv = 1.f / sum;
      }
    }
    auto put = [&](int k, float gx, float gy, float gz, float m, bool writer) {
      if (!writer) return;
      if constexpr (KP == 0) {
        if (p.softmax) {      // the slot holds p_k * dL/dp_k until every tap is done (dcnv4_col2im_cuda.cuh:337-339)
          gz *= m;
          sm_dot += gz;
        }
      }
      const float f0[1] = {gx * p.offset_scale * m}, f1[1] = {gy * p.offset_scale * m}, f2[1] = {gz};
      om[2 * k] = Pack<Tag, 1>::encode(f0);
      om[2 * k + 1] = Pack<Tag, 1>::encode(f1);
      om[2 * Kp + k] = Pack<Tag, 1>::encode(f2);
    };
    auto combine = [&](int k, const float (&d)[4], float ly, float lx, const float (&w)[4], float m, bool writer) {
      const float hy = 1.f - ly, hx = 1.f - lx;
      const float gx = hy * (d[1] - d[0]) + ly * (d[3] - d[2]);      // common.h:188-201
      const float gy = hx * (d[2] - d[0]) + lx * (d[3] - d[1]);
      const float gz = w[0] * d[0] + w[1] * d[1] + w[2] * d[2] + w[3] * d[3];
      put(k, gx, gy, gz, m, writer);
    };
    auto one_tap = [&](int k, int i, int j) {
      const float x = add_rn(x_base, mul_rn(add_rn((float)(i * p.dw), lds_elem<Tag>(om, 2 * k)), p.offset_scale));
      const float y = add_rn(y_base, mul_rn(add_rn((float)(j * p.dh), lds_elem<Tag>(om, 2 * k + 1)), p.offset_scale));
      float m = lds_elem<Tag>(om, 2 * Kp + k);
      if constexpr (KP == 0) {
        if (p.softmax) m = __expf(m - sm_max) * sm_inv;
      }
      const WinTap wt = window_tap(y, x, p.H, p.W, t, cell_stride, lane_bytes, zero_base);
      far_mask |= (mask_t)(wt.inside && !wt.ok) << k;
      // Chebyshev distance of the point from the reference point; its ceiling is how far the weighted corners of
      // the 2x2 block lie from it at most (a point at an integer distance k has its far corners at weight 0)
      // (points beyond the cap are not `ok` - the cap exceeds what any window covers - and are folded where they are served)
      const float dist = fmaxf(fabsf(x - p0xf), fabsf(y - p0yf));
      reach_bits = max(reach_bits, (wt.inside && dist <= p.gv_reach_cap) ? __builtin_bit_cast(uint32_t, dist) : 0u);
      u32x4 raw[4][NV];
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        const char *src = s_win + wt.addr + (cn & 1) * cell_stride + (cn >> 1) * row_bytes;
#pragma unroll
        for (int v = 0; v < NV; ++v) raw[cn][v] = *reinterpret_cast<const u32x4 *>(src + 16 * v);
      }
      float d[4];
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        float acc = 0.f;
        if constexpr (Tag::kBytes == 2) {
          // 16-bit tensors: two channels per instruction straight from the raw words, products and sums in fp32;
          // two running sums, so that consecutive instructions do not wait for each other
          float acc1 = 0.f;
#pragma unroll
          for (int v = 0; v < NV; ++v) {
            const u32x4 a = raw[cn][v], g = go_raw[v];
            const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, gw[4] = {g.x, g.y, g.z, g.w};
            acc = dot2_pair<Tag>(aw[0], gw[0], acc);
            acc1 = dot2_pair<Tag>(aw[1], gw[1], acc1);
            acc = dot2_pair<Tag>(aw[2], gw[2], acc);
            acc1 = dot2_pair<Tag>(aw[3], gw[3], acc1);
          }
          acc += acc1;
        } else {
#pragma unroll
          for (int v = 0; v < NV; ++v) {
            float f[EPV];
            pack::decode(raw[cn][v], f);
#pragma unroll
            for (int c = 0; c < EPV; ++c) acc = fmaf(f[c], go[v][c], acc);
          }
        }
        d[cn] = pair ? acc + dpp_quad_xor1(acc) : acc;
      }
      combine(k, d, wt.ly, wt.lx, wt.w, m, part == 0);      // all zeros for a point outside the image or the window
    };
    // The corner . grad_out sums of one point from the window, over all channels of the group.
    auto window_dots = [&](int addr, float (&d)[4]) {
      u32x4 raw[4][NV];
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        const char *src = s_win + addr + (cn & 1) * cell_stride + (cn >> 1) * row_bytes;
#pragma unroll
        for (int v = 0; v < NV; ++v) raw[cn][v] = *reinterpret_cast<const u32x4 *>(src + 16 * v);
      }
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        float acc = 0.f;
        if constexpr (Tag::kBytes == 2) {
          float acc1 = 0.f;
#pragma unroll
          for (int v = 0; v < NV; ++v) {
            const u32x4 a = raw[cn][v], g = go_raw[v];
            const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, gw[4] = {g.x, g.y, g.z, g.w};
            acc = dot2_pair<Tag>(aw[0], gw[0], acc);
            acc1 = dot2_pair<Tag>(aw[1], gw[1], acc1);
            acc = dot2_pair<Tag>(aw[2], gw[2], acc);
            acc1 = dot2_pair<Tag>(aw[3], gw[3], acc1);
          }
          acc += acc1;
        } else {
#pragma unroll
          for (int v = 0; v < NV; ++v) {
            float f[EPV];
            pack::decode(raw[cn][v], f);
#pragma unroll
            for (int c = 0; c < EPV; ++c) acc = fmaf(f[c], go[v][c], acc);
          }
        }
        d[cn] = acc + dpp_quad_xor1(acc);
      }
    };
    // Two points at a time for a pair of lanes: each prepares one of them, both gather and multiply for both, and
    // the lane that prepared a point forms its gradients and writes them.
    auto two_taps = [&](int k0) {
      const int k = k0 + part;
      int i, j;
      tap_ij_3x3(KP, k, i, j);
      const float x = add_rn(x_base, mul_rn(add_rn((float)(i * p.dw), lds_elem<Tag>(om, 2 * k)), p.offset_scale));
      const float y = add_rn(y_base, mul_rn(add_rn((float)(j * p.dh), lds_elem<Tag>(om, 2 * k + 1)), p.offset_scale));
      const float m = lds_elem<Tag>(om, 2 * Kp + k);
      const int part_bytes = part * NV * 16;
      const WinTap wt = window_tap(y, x, p.H, p.W, t, cell_stride, lane_bytes - part_bytes, zero_base);
      const int far_own = wt.inside && !wt.ok;
      const float dist = fmaxf(fabsf(x - p0xf), fabsf(y - p0yf));
      reach_bits = max(reach_bits, (wt.inside && dist <= p.gv_reach_cap) ? __builtin_bit_cast(uint32_t, dist) : 0u);
      far_mask |= ((mask_t)pair_pick<0>(far_own) << k0) | ((mask_t)pair_pick<1>(far_own) << (k0 + 1));
      float d0[4], d1[4], d[4];
      window_dots(pair_pick<0>(wt.addr) + part_bytes, d0);
      window_dots(pair_pick<1>(wt.addr) + part_bytes, d1);
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) d[cn] = part ? d1[cn] : d0[cn];
      combine(k, d, wt.ly, wt.lx, wt.w, m, true);
    };
    // a sampling point whose corners lie outside the staged window: gather from memory; its
    // offsets are re-read from memory because the LDS slots already hold gradients
    const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);
    const uint32_t pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
    const uint32_t img_base = (uint32_t)t.b * (uint32_t)(p.H * p.W) * pix_bytes + (uint32_t)((t.g0 + gl) * p.D) * Tag::kBytes + (uint32_t)(part * NV * 16);
    const elem_t *om_g = reinterpret_cast<const elem_t *>(p.offset_mask) +
                         ((size_t)t.b * p.Q + (size_t)ho * p.Wo + wo) * p.P_pad + (t.g0 + gl) * 3 * Kp;
    auto far_tap = [&](int k, int i, int j) {
      const float x = add_rn(x_base, mul_rn(add_rn((float)(i * p.dw), lds_elem<Tag>(om_g, 2 * k)), p.offset_scale));
      const float y = add_rn(y_base, mul_rn(add_rn((float)(j * p.dh), lds_elem<Tag>(om_g, 2 * k + 1)), p.offset_scale));
      float m = lds_elem<Tag>(om_g, 2 * Kp + k);
      if constexpr (KP == 0) {
        if (p.softmax) m = __expf(m - sm_max) * sm_inv;
      }
      const Tap tp = make_tap(y, x, p.H, p.W, img_base, pix_bytes);
      // beyond the reach cap: left out of the reach statistic above, folded per destination tile instead
      if (tp.valid != 0 && fmaxf(fabsf(x - p0xf), fabsf(y - p0yf)) > p.gv_reach_cap) dcnv4_fold_far_point(p, t.b, t.g0 + gl, tp.y0, tp.x0, p0y, p0x);
      float d[4];
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        float acc = 0.f;
#pragma unroll
        for (int v = 0; v < NV; ++v) {
          float f[EPV];
          pack::decode(buffer_load<16>(value, tp.off[cn] + 16u * v), f);
#pragma unroll
          for (int c = 0; c < EPV; ++c) acc = fmaf(f[c], go[v][c], acc);
        }
        d[cn] = pair ? acc + dpp_quad_xor1(acc) : acc;
      }
      combine(k, d, tp.ly, tp.lx, tp.w, m, part == 0);
    };

    if constexpr (KP > 0) {
      int k_first = 0;
      if constexpr (PAIR) {
#pragma unroll 1
        for (int k0 = 0; k0 + 1 < KP; k0 += 2) two_taps(k0);
        k_first = KP & ~1;      // an odd last point: both lanes prepare it, the even one writes
      }
#pragma unroll 1
      for (int k = k_first; k < KP; ++k) {
        int i, j;
        tap_ij_3x3(KP, k, i, j);
        one_tap(k, i, j);
      }
      if (far_mask != 0) {
        for (int k = 0; k < KP; ++k) {
          if (!((far_mask >> k) & 1)) continue;
          int i, j;
          tap_ij_3x3(KP, k, i, j);
          far_tap(k, i, j);
        }
      }
    } else {
      for (int pass = 0; pass < 2; ++pass) {
        if (pass == 1 && far_mask == 0) break;
        int k = 0;
        for (int i = 0; i < p.kw; ++i)
          for (int j = 0; j < p.kh; ++j) {
            if (p.remove_center && i == p.kw / 2 && j == p.kh / 2) continue;
            if (pass == 0) one_tap(k, i, j);
            else if ((far_mask >> k) & 1) far_tap(k, i, j);
            ++k;
          }
      }
      // softmax Jacobian: dL/dlogit_k = p_k * dL/dp_k - p_k * sum_j p_j * dL/dp_j (dcnv4_col2im_cuda.cuh:352-365); the
      // logits are read from memory again, their slots hold the first term
      if (p.softmax && part == 0) {
        for (int k = 0; k < Kp; ++k) {
          const float pk = __expf(lds_elem<Tag>(om_g, 2 * Kp + k) - sm_max) * sm_inv;
          const float f[1] = {lds_elem<Tag>(om, 2 * Kp + k) - pk * sm_dot};
          om[2 * Kp + k] = Pack<Tag, 1>::encode(f);
        }
      }
    }
  }

  // the reach the grad_value kernel has to cover: fold in LDS, then touch the global word only when it would grow
  // (same-address global atomics retire slowly)
  reach_needed = wave_max_u32((uint32_t)min(ceilf(__builtin_bit_cast(float, reach_bits)), 1048576.f));
  if ((threadIdx.x & (kWave - 1)) == 0 && reach_needed != 0) atomicMax(&s_reach, reach_needed);
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t *dst = &p.state->reach_needed;
    const uint32_t mine = s_reach;
    if (mine > __hip_atomic_load(dst, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(dst, mine);
  }
  unstage_tile_grads<Tag>(p, t, s_om);
}


}  // namespace
}  // namespace dcn
