// Flash deformable attention backward, gradient of value, without global atomics.
//
// The reference scatters 4 * L * K * D fp32 atomicAdds per (query, head)
// (DCNv4_op/src/cuda/flash_deform_col2im_cuda.cuh:240-270 through common.h:153-184).  Sampling
// locations are free to land anywhere in their level, so unlike the DCNv4 operator there is no
// window around the query to exploit.  Instead the sampling points are first BINNED by the tile
// of their level they touch, and then a workgroup that OWNS a tile adds them up in LDS:
//
//   * the grad_sampling_loc_attn kernel, which runs first, leaves one 16-bit key (integer position of
//     the first corner, or "outside") and the softmax probability per sampling point, both laid out
//     [image][head][level][query][point], and the maximum of |grad_out| in GradState;
//   * fda_bin_points_kernel: one workgroup per chunk of 8192 points of one (image, head, level)
//     counting-sorts the chunk by tile in LDS (a point whose 2x2 corner block straddles tiles is
//     listed under each of them) and writes the sorted point ids to the chunk's region of the
//     workspace plus one (offset, count) word per tile to a table - no global atomics, no host
//     round trip, every chunk independent;
//   * fda_grad_value_kernel: persistent workgroups walk (tile, image, head) items, smallest level
//     first.  An item collects its tile's slices of all chunk lists into LDS and applies them in
//     batches: one lane per point rebuilds the position from sampling_loc_attn and, with the stored
//     probability, the four corner weights, while the previous batch is being applied (two record
//     buffers, one barrier per batch; all loads are requested one batch ahead); then a row of 8 lanes
//     per point, each holding its own channels of the point's grad_out row in registers, adds the
//     contributions to the tile's accumulators with 64-bit integer
//     LDS atomics on fixed-point values (normalised by max |grad_out|; probability * bilinear weight
//     <= 1), so the result does not depend on the order of arrival and is bit-reproducible;
//   * the finished tile is written to grad_value with plain stores in the tensor dtype.
//
// Tiles are at most 8x8 cells and every level is cut into 16 of them or more, so items stay
// small (several workgroups share a CU and hide each other's latencies) and comparable in size.
// Levels and tile shapes are derived on the device from the spatial_shapes tensor; the host never
// reads it.  A level with more tiles than the binning kernel's LDS histogram holds raises a flag in
// GradState: grad_value is then left zeroed for the atomic fallback kernel, like for non-finite
// statistics.
#include <algorithm>

#include "common.hpp"
#include "launch.hpp"

namespace dcn {

namespace {

constexpr int kBinThreads = 1024;
constexpr int kBinWordsPerLane = kFdaChunkPoints / 2 / kBinThreads;      // dwords of two keys per lane: 4
constexpr int kApplyThreads = 512;
constexpr int kRowLanes = 8;                 // lanes that apply one listed point
constexpr int kBatch = 128;                  // listed points applied between two barriers
constexpr int kListCap = 1024;               // listed points held in LDS at a time
constexpr int kTabCap = 256;                 // chunk table entries held in LDS at a time
constexpr int kCellBitsF = 7;                // tiles have at most 64 cells; cell 64.. = trash
constexpr int kTileCells = 64;

struct LevelPlan {
  int H, W, start;
  int th, tw, nty, ntx;      // tile shape (1..8 each) and tile grid
};

__device__ __forceinline__ LevelPlan level_plan(const FdaLaunch &p, int l) {
  LevelPlan lp;
  lp.H = (int)p.shapes[2 * l]; lp.W = (int)p.shapes[2 * l + 1]; lp.start = (int)p.level_start[l];
  lp.th = max(1, min(8, (lp.H + 3) / 4));
  lp.tw = max(1, min(8, (lp.W + 3) / 4));
  lp.nty = lp.H > 0 ? (lp.H + lp.th - 1) / lp.th : 0;
  lp.ntx = lp.W > 0 ? (lp.W + lp.tw - 1) / lp.tw : 0;
  return lp;
}

template <typename Tag>
__device__ __forceinline__ float elem_at(const void *base, size_t i) {
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  float f[1];
  Pack<Tag, 1>::decode(reinterpret_cast<const elem_t *>(base)[i], f);
  return f[0];
}

// n / d for small non-negative n and 1 <= d <= 8
__device__ __forceinline__ int div_small(int n, float inv) { return (int)(((float)n + 0.5f) * inv); }

// ------------------------------------------------------------------------------- binning
// The tiles a sampling point touches: the tile of the first in-level row and column of its corner
// block, and whether the block continues into the next tile column / row.
struct Touch {
  uint32_t t00;        // 0xffffffff = none
  uint32_t dx, dy;
};

template <typename Tag>
__global__ void __launch_bounds__(kBinThreads) fda_bin_points_kernel(const FdaLaunch p) {
  __shared__ uint32_t s_hist[kFdaMaxTilesPerLevel];       // counts, then running cursors
  __shared__ uint32_t s_wave_sum[kBinThreads / kWave];
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int QK = p.Q * p.K, LK = p.L * p.K;
  const int chunk = blockIdx.x % p.n_chunks, seg = blockIdx.x / p.n_chunks;       // seg = (image * G + head) * L + level
  const int l = seg % p.L, bg = seg / p.L;
  const int b = bg / p.G, g = bg - b * p.G;
  const LevelPlan lp = level_plan(p, l);
  const int n_tiles = lp.nty * lp.ntx;
  if (n_tiles > p.tile_stride || n_tiles > kFdaMaxTilesPerLevel) {
    if (tid == 0) atomicOr(&p.state->reserved, 1u);       // the fallback kernel takes over
    return;
  }
  for (int i = tid; i < n_tiles; i += kBinThreads) s_hist[i] = 0u;
  __syncthreads();

  const size_t QKp = fda_key_stride(p.Q, p.K);
  const uint32_t *keys = reinterpret_cast<const uint32_t *>(p.keys + (size_t)seg * QKp);
  const int n_words = (int)(QKp / 2);
  const float inv_th = 1.f / (float)lp.th, inv_tw = 1.f / (float)lp.tw;
  const size_t sla_bg = ((size_t)b * p.Q * p.G + g) * 3 * LK;

  auto touch_of = [&](uint32_t k16, uint32_t pt) {
    Touch t;
    t.t00 = 0xffffffffu; t.dx = t.dy = 0u;
    if (pt >= (uint32_t)QK || k16 == kFdaKeyOutside) return t;
    int y1 = (int)(k16 >> 8), x1 = (int)(k16 & 0xffu);             // y0 + 1, x0 + 1
    if (k16 == kFdaKeySaturated) {                                // position beyond the key's fields: recompute it
      const uint32_t q = pt / (uint32_t)p.K;
      const int tt = l * p.K + (int)(pt - q * p.K);
      const size_t row = sla_bg + (size_t)q * p.G * 3 * LK;
      const float x = sub_rn(mul_rn(elem_at<Tag>(p.sla, row + 2 * tt), (float)lp.W), 0.5f);
      const float y = sub_rn(mul_rn(elem_at<Tag>(p.sla, row + 2 * tt + 1), (float)lp.H), 0.5f);
      const Tap tp = make_tap(y, x, lp.H, lp.W, 0u, 0u);
      if (tp.valid == 0) return t;
      y1 = tp.y0 + 1; x1 = tp.x0 + 1;
    }
    // rows y1 - 1 and y1 of the block, where they exist
    const int ty_lo = div_small(y1 >= 1 ? y1 - 1 : y1, inv_th), ty_hi = y1 <= lp.H - 1 ? div_small(y1, inv_th) : ty_lo;
    const int tx_lo = div_small(x1 >= 1 ? x1 - 1 : x1, inv_tw), tx_hi = x1 <= lp.W - 1 ? div_small(x1, inv_tw) : tx_lo;
    t.t00 = (uint32_t)(ty_lo * lp.ntx + tx_lo);
    t.dx = (uint32_t)(tx_hi != tx_lo);
    t.dy = (uint32_t)(ty_hi != ty_lo);
    return t;
  };

  // ---- pass 1: count
  Touch touch[2 * kBinWordsPerLane];
#pragma unroll
  for (int u = 0; u < kBinWordsPerLane; ++u) {
    const int w = chunk * (kFdaChunkPoints / 2) + u * kBinThreads + tid;
    const uint32_t word = keys[min(w, n_words - 1)];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const Touch t = touch_of((word >> (16 * h)) & 0xffffu, w < n_words ? 2u * (uint32_t)w + h : 0xffffffffu);
      touch[2 * u + h] = t;
      if (t.t00 != 0xffffffffu) {
        atomicAdd(&s_hist[t.t00], 1u);
        if (t.dx) atomicAdd(&s_hist[t.t00 + 1], 1u);
        if (t.dy) atomicAdd(&s_hist[t.t00 + lp.ntx], 1u);
        if (t.dx && t.dy) atomicAdd(&s_hist[t.t00 + lp.ntx + 1], 1u);
      }
    }
  }
  __syncthreads();

  // ---- exclusive prefix over the tiles (8 consecutive tiles per lane), table row out
  constexpr int kPer = kFdaMaxTilesPerLevel / kBinThreads;      // 8
  uint32_t cnt[kPer], sum = 0;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int i = tid * kPer + j;
    cnt[j] = i < n_tiles ? s_hist[i] : 0u;
    sum += cnt[j];
  }
  uint32_t incl = sum;
  for (int o = 1; o < kWave; o <<= 1) {
    const uint32_t v = (uint32_t)__shfl_up((int)incl, o, kWave);
    if (lane >= o) incl += v;
  }
  if (lane == kWave - 1) s_wave_sum[wave] = incl;
  __syncthreads();
  uint32_t before = incl - sum;
  for (int w = 0; w < wave; ++w) before += s_wave_sum[w];
  uint32_t *table = p.table + (size_t)blockIdx.x * p.tile_stride;
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int i = tid * kPer + j;
    if (i < n_tiles) {
      table[i] = before | (cnt[j] << 16);                 // offset <= 32767 and count <= 32768 for 8192 points
      s_hist[i] = before;                                 // now the running cursor of the tile
    }
    before += cnt[j];
  }
  __syncthreads();

  // ---- pass 2: place
  uint32_t *region = p.regions + (size_t)blockIdx.x * (4 * kFdaChunkPoints);
#pragma unroll
  for (int u = 0; u < kBinWordsPerLane; ++u) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const Touch t = touch[2 * u + h];
      if (t.t00 == 0xffffffffu) continue;
      const uint32_t pt = 2u * (uint32_t)(chunk * (kFdaChunkPoints / 2) + u * kBinThreads + tid) + h;
      region[atomicAdd(&s_hist[t.t00], 1u)] = pt;
      if (t.dx) region[atomicAdd(&s_hist[t.t00 + 1], 1u)] = pt;
      if (t.dy) region[atomicAdd(&s_hist[t.t00 + lp.ntx], 1u)] = pt;
      if (t.dx && t.dy) region[atomicAdd(&s_hist[t.t00 + lp.ntx + 1], 1u)] = pt;
    }
  }
}

// ------------------------------------------------------------------------------- accumulation
template <typename Tag, int CPL>
__global__ void __launch_bounds__(kApplyThreads) fda_grad_value_kernel(const FdaLaunch p) {
  extern __shared__ unsigned long long lds64[];
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int DP = CPL * kRowLanes;                         // accumulator channels per cell (D rounded up)
  const int D = p.D, LK = p.L * p.K, QK = p.Q * p.K;
  unsigned long long *acc = lds64;                            // [(kTileCells + 1) * DP], last cell = trash
  constexpr int n_acc = (kTileCells + 1) * DP;
  f32x4 *rec_w = reinterpret_cast<f32x4 *>(lds64 + n_acc);    // [2][kBatch]: one batch is applied while the next is prepared
  uint32_t *rec_meta = reinterpret_cast<uint32_t *>(rec_w + 2 * kBatch);   // [2][kBatch] four 7-bit cells
  uint32_t *s_list = rec_meta + 2 * kBatch;                   // [kListCap]
  uint32_t *s_tab = s_list + kListCap;                        // [kTabCap] (offset | count << 16) of the item's tile per chunk
  uint32_t *s_pre = s_tab + kTabCap;                          // [kTabCap + 1] exclusive prefix of the counts
  __shared__ LevelPlan s_plan[kMaxLevels];
  __shared__ int s_first[kMaxLevels + 1];                     // rank of each level's first tile in the walk

  const int tid = threadIdx.x;
  if (tid == 0) {
    int rank = 0;                                             // walk order: last level first
    for (int l = p.L - 1; l >= 0; --l) {
      s_plan[l] = level_plan(p, l);
      s_first[l] = rank;
      rank += s_plan[l].nty * s_plan[l].ntx;
    }
    s_first[p.L] = rank;                                      // total
  }
  __syncthreads();
  const int n_tiles = s_first[p.L];
  const int BG = p.n_img * p.G;

  // value rows that no level covers (spatial_size beyond the levels, gaps between them) get zeros, like the
  // reference's zeros_like(value) (flash_deform_attn_cuda.cu:118)
  {
    typedef typename RawWord<Tag::kBytes>::type elem0_t;
    const long long rows = (long long)p.n_img * p.N;
    const int row_elems = p.G * p.D;
    for (long long r = (long long)blockIdx.x * kApplyThreads + tid; r < rows; r += (long long)gridDim.x * kApplyThreads) {
      const int n = (int)(r % p.N);
      bool covered = false;
      for (int l = 0; l < p.L; ++l) covered |= n >= s_plan[l].start && n < s_plan[l].start + s_plan[l].H * s_plan[l].W;
      if (!covered) {
        elem0_t *row = reinterpret_cast<elem0_t *>(p.grad_value) + (size_t)r * row_elems;
        for (int i = 0; i < row_elems; ++i) row[i] = elem0_t(0);
      }
    }
  }

  const uint32_t gmax = p.state->go_max_bits;
  const bool usable = gmax < 0x7f800000u && gmax != 0u && p.state->reserved == 0u;
  const int e_go = (int)(gmax >> 23) - 126;                  // 2^e_go > max |grad_out|
  const int e_out = e_go - p.fix_bits;
  const size_t QKp = fda_key_stride(p.Q, p.K);

  for (int item = blockIdx.x; item < n_tiles * BG; item += gridDim.x) {
    const int rank = item / BG, bg = item - rank * BG;
    const int b = bg / p.G, g = bg - b * p.G;
    int l = 0;
    for (int i = 0; i < p.L; ++i)       // first ranks fall with the level index: the first level whose rank fits
      if (s_first[i] <= rank && s_plan[i].nty * s_plan[i].ntx > 0) { l = i; break; }
    const LevelPlan lp = s_plan[l];
    const int t_in = rank - s_first[l];
    const int ty = t_in / lp.ntx, tx = t_in - ty * lp.ntx;
    const int ty0 = ty * lp.th, tx0 = tx * lp.tw;
    const int th = min(lp.th, lp.H - ty0), tw = min(lp.tw, lp.W - tx0);
    const int n_cells = th * tw;                             // <= 64; cell n_cells.. = trash
    const int seg = bg * p.L + l;

    for (int i = tid; i < n_acc; i += kApplyThreads) acc[i] = 0ull;

    const float *probs = p.probs + (size_t)seg * QKp;
    const size_t sla_bg = ((size_t)b * p.Q * p.G + g) * 3 * LK;       // + q * G * 3LK
    const size_t go_bg = ((size_t)b * p.Q * p.G + g) * D;             // + q * G * D

    // Everything a batch needs is requested through range-checked buffer loads of raw words: no branches
    // around the loads, so they all fly together, and nothing is converted before it is needed.
    typedef typename RawWord<2 * Tag::kBytes>::type xy_t;      // (x, y) of a point are adjacent
    const __amdgpu_buffer_rsrc_t sla_rs = make_rsrc(reinterpret_cast<const elem_t *>(p.sla) + sla_bg,
                                                    (uint32_t)((size_t)p.Q * p.G * 3 * LK * Tag::kBytes));
    const __amdgpu_buffer_rsrc_t go_rs = make_rsrc(reinterpret_cast<const elem_t *>(p.grad_out) + go_bg,
                                                   (uint32_t)((size_t)p.Q * p.G * D * Tag::kBytes));
    const __amdgpu_buffer_rsrc_t pr_rs = make_rsrc(probs, (uint32_t)QK * 4u);
    // A row of 8 lanes owns a listed point; lane c of the row owns the CPL consecutive channels from c * CPL, loads
    // them itself and keeps them in registers until the point is applied.
    typedef typename RawWord<CPL * Tag::kBytes>::type goN_t;
    constexpr int kRowsPerLane = kBatch * kRowLanes / kApplyThreads;      // rows a lane serves per batch: 2
    constexpr int kRowStep = kApplyThreads / kRowLanes;
    const int row_in_block = tid / kRowLanes, c = tid & (kRowLanes - 1);
    struct Ahead {
      xy_t xy;                         // lanes < batch size: their point
      uint32_t pr;
      goN_t go[kRowsPerLane];
    };
    auto fetch = [&](uint32_t b0, int nb) {
      Ahead a;
      {
        const uint32_t pt = s_list[b0 + min(tid, max(nb - 1, 0))];
        const uint32_t q = pt / (uint32_t)p.K;
        const int t = l * p.K + (int)(pt - q * p.K);
        const bool live = tid < nb;
        a.xy = buffer_load<2 * Tag::kBytes>(sla_rs, live ? (q * (uint32_t)(p.G * 3 * LK) + 2u * t) * Tag::kBytes : kDropOffset);
        a.pr = buffer_load<4>(pr_rs, live ? pt * 4u : kDropOffset);
      }
#pragma unroll
      for (int u = 0; u < kRowsPerLane; ++u) {
        const int h = row_in_block + u * kRowStep;
        const bool live = h < nb && c * CPL < D;
        const uint32_t q = s_list[b0 + min(h, max(nb - 1, 0))] / (uint32_t)p.K;
        a.go[u] = buffer_load<CPL * Tag::kBytes>(go_rs, live ? (q * (uint32_t)(p.G * D) + (uint32_t)(c * CPL)) * Tag::kBytes : kDropOffset);
      }
      return a;
    };
    // one lane per point: corner weights and accumulator cells, into record buffer `buf`
    auto park = [&](const Ahead &a, int nb, int buf) {
      if (tid < nb) {
        float xy[2];
        Pack<Tag, 2>::decode(a.xy, xy);
        const float x = sub_rn(mul_rn(xy[0], (float)lp.W), 0.5f);       // flash_deform_im2col_cuda.cuh:188-189
        const float y = sub_rn(mul_rn(xy[1], (float)lp.H), 0.5f);
        const Tap tp = make_tap(y, x, lp.H, lp.W, 0u, 0u);
        const float ps = ldexpf(__builtin_bit_cast(float, a.pr), p.fix_bits);
        const int ly = tp.y0 - ty0, lx = tp.x0 - tx0;
        uint32_t cells[4];
        float w[4];
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          const int cy = ly + (cn >> 1), cx = lx + (cn & 1);
          const bool ok = (tp.valid & (1u << cn)) && cy >= 0 && cy < th && cx >= 0 && cx < tw;
          cells[cn] = ok ? (uint32_t)(cy * tw + cx) : (uint32_t)n_cells;
          w[cn] = ok ? ps * tp.w[cn] : 0.f;
        }
        rec_w[buf * kBatch + tid] = f32x4{w[0], w[1], w[2], w[3]};
        rec_meta[buf * kBatch + tid] = cells[0] | (cells[1] << kCellBitsF) | (cells[2] << (2 * kCellBitsF)) | (cells[3] << (3 * kCellBitsF));
      }
    };
    // Accumulator word of (lane c, slot j) is c + 8 j: the lanes of a row touch consecutive words.  The LDS serves a
    // wave's 64-bit atomics 16 lanes per pass over its 32 banks, two rows of eight lanes: row r visits its slots
    // starting from slot r mod CPL, so neighbouring rows are on slots of different parity and the two rows of a pass
    // fill the banks exactly once whatever their cells are.  The lane's channel values are rotated to that order
    // once per point.
    const int rot = row_in_block & (CPL - 1);
    int slot_off[CPL];
#pragma unroll
    for (int j = 0; j < CPL; ++j) slot_off[j] = kRowLanes * ((j + rot) & (CPL - 1));
    // applies the first n entries of s_list; called by every lane, ends past a barrier
    auto apply_list = [&](uint32_t n) {
      if (n == 0) return;
      int nb = (int)min((uint32_t)kBatch, n);
      Ahead cur = fetch(0, nb);
      park(cur, nb, 0);
      __syncthreads();
      int buf = 0;
      for (uint32_t b0 = 0; b0 < n; b0 += kBatch) {
        const int nb_next = b0 + kBatch < n ? (int)min((uint32_t)kBatch, n - b0 - kBatch) : 0;
        Ahead nxt = cur;
        if (nb_next > 0) nxt = fetch(b0 + kBatch, nb_next);      // flies while this batch is applied
#pragma unroll
        for (int u = 0; u < kRowsPerLane; ++u) {
          const int h = row_in_block + u * kRowStep;
          if (h >= nb) break;
          const f32x4 w = rec_w[buf * kBatch + h];
          const uint32_t meta = rec_meta[buf * kBatch + h];
          const uint32_t cells[4] = {meta & 127u, (meta >> kCellBitsF) & 127u, (meta >> (2 * kCellBitsF)) & 127u,
                                     (meta >> (3 * kCellBitsF)) & 127u};
          const float wv[4] = {w.x, w.y, w.z, w.w};
          float g[CPL], gn[CPL];
          Pack<Tag, CPL>::decode(cur.go[u], g);
#pragma unroll
          for (int j = 0; j < CPL; ++j) g[j] = ldexpf(g[j], -e_go);      // normalised to [-1, 1]
          if constexpr (CPL == 4) {          // gn[j] = g[(j + rot) & 3]
            const bool r1 = rot & 1, r2 = rot & 2;
            const float a0 = r1 ? g[1] : g[0], a1 = r1 ? g[2] : g[1], a2 = r1 ? g[3] : g[2], a3 = r1 ? g[0] : g[3];
            gn[0] = r2 ? a2 : a0; gn[1] = r2 ? a3 : a1; gn[2] = r2 ? a0 : a2; gn[3] = r2 ? a1 : a3;
          } else if constexpr (CPL == 2) {
            gn[0] = rot ? g[1] : g[0]; gn[1] = rot ? g[0] : g[1];
          } else {
            gn[0] = g[0];
          }
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) {
            unsigned long long *dst = acc + __umul24(cells[cn], (uint32_t)DP) + c;
            // the same resolution for every tensor dtype: small gradients next to large ones (loss scaling) keep
            // their bits, as they do when the reference sums in fp32
            const double wd = (double)wv[cn];
#pragma unroll
            for (int j = 0; j < CPL; ++j)
              __hip_atomic_fetch_add(dst + slot_off[j], fixed_product((double)gn[j], wd), __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_WORKGROUP);
          }
        }
        if (nb_next > 0) park(nxt, nb_next, buf ^ 1);
        __syncthreads();
        cur = nxt;
        nb = nb_next;
        buf ^= 1;
      }
    };

    // ---- collect this tile's slices of the chunk lists (a group of chunks at a time) and apply them
    if (usable) {
      for (int c0 = 0; c0 < p.n_chunks; c0 += kTabCap) {
        const int nc = min(kTabCap, p.n_chunks - c0);
        __syncthreads();
        for (int c = tid; c < nc; c += kApplyThreads)
          s_tab[c] = p.table[((size_t)seg * p.n_chunks + c0 + c) * p.tile_stride + t_in];
        __syncthreads();
        if (tid < kWave) {            // exclusive prefix of the counts, one wave
          uint32_t run = 0;
          for (int base = 0; base < nc; base += kWave) {
            const int c = base + tid;
            const uint32_t v = c < nc ? s_tab[c] >> 16 : 0u;
            uint32_t incl = v;
            for (int o = 1; o < kWave; o <<= 1) {
              const uint32_t up = (uint32_t)__shfl_up((int)incl, o, kWave);
              if (tid >= o) incl += up;
            }
            if (c < nc) s_pre[c] = run + incl - v;
            run += (uint32_t)__shfl((int)incl, kWave - 1, kWave);
          }
          if (tid == 0) s_pre[nc] = run;
        }
        __syncthreads();
        const uint32_t total = s_pre[nc];
        // copy the slices into s_list, kListCap entries at a time; lane -> entry -> chunk by bisection
        for (uint32_t e0 = 0; e0 < total; e0 += kListCap) {
          const uint32_t ne = min((uint32_t)kListCap, total - e0);
          for (uint32_t i = tid; i < ne; i += kApplyThreads) {
            const uint32_t e = e0 + i;
            int lo = 0, hi = nc;                       // largest c with s_pre[c] <= e
            while (hi - lo > 1) {
              const int mid = (lo + hi) >> 1;
              if (s_pre[mid] <= e) lo = mid; else hi = mid;
            }
            const uint32_t *region = p.regions + ((size_t)seg * p.n_chunks + c0 + lo) * (4 * kFdaChunkPoints);
            s_list[i] = region[(s_tab[lo] & 0xffffu) + (e - s_pre[lo])];
          }
          __syncthreads();
          apply_list(ne);
        }
      }
    }
    __syncthreads();

    // ---- the tile is complete (zeros when the statistics are unusable: the fallback kernel then adds everything)
    elem_t *gv = reinterpret_cast<elem_t *>(p.grad_value);
    for (int i = tid; i < n_cells * D; i += kApplyThreads) {
      const int cell = i / D, ch = i - cell * D;
      const int cy = cell / tw, cx = cell - cy * tw;
      const unsigned long long a = acc[cell * DP + ch / CPL + kRowLanes * (ch % CPL)];
      const double v = ldexp((double)(int)(a >> 32) * 4294967296.0 + (double)(uint32_t)a, e_out);
      const float f[1] = {(float)v};
      const long long n = (long long)lp.start + (long long)(ty0 + cy) * lp.W + tx0 + cx;      // level tables are not validated
      if (n >= 0 && n < p.N) gv[(((size_t)b * p.N + (size_t)n) * p.G + g) * D + ch] = Pack<Tag, 1>::encode(f);
    }
    __syncthreads();
  }
}

template <typename Tag>
hipError_t launch_t(const FdaLaunch &p, hipStream_t stream) {
  // binning: one workgroup per chunk of every (image, head, level)
  hipLaunchKernelGGL(fda_bin_points_kernel<Tag>, dim3((unsigned)(p.n_img * p.G * p.L * p.n_chunks)), dim3(kBinThreads), 0, stream, p);
  if (hipError_t e = hipGetLastError()) return e;

  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  const size_t lds = fda_grad_value_lds_bytes(p);
  const int per_cu = (int)std::max<size_t>(1, std::min<size_t>(4, (kMaxLdsPerWorkgroup - 4096) / (lds + 1024)));
  const dim3 grid((unsigned)(cus * per_cu)), block(kApplyThreads);
  auto go = [&](auto kernel) -> hipError_t {
    if (hipError_t e = ensure_dynamic_lds_limit(reinterpret_cast<const void *>(kernel), kMaxLdsPerWorkgroup - 2048)) return e;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return hipGetLastError();
  };
  switch (fda_padded_channels(p.D) / kRowLanes) {
    case 1: return go(fda_grad_value_kernel<Tag, 1>);
    case 2: return go(fda_grad_value_kernel<Tag, 2>);
    case 4: return go(fda_grad_value_kernel<Tag, 4>);
  }
  return hipErrorInvalidValue;      // wider heads take the atomic path (the entry point checks)
}

}  // namespace

size_t fda_grad_value_lds_bytes(const FdaLaunch &p) {
  const size_t dp = (size_t)fda_padded_channels(p.D);
  return ((size_t)kTileCells + 1) * dp * sizeof(unsigned long long) + 2 * kBatch * (sizeof(f32x4) + sizeof(uint32_t)) +
         ((size_t)kListCap + 2 * kTabCap + 4) * sizeof(uint32_t);
}

hipError_t launch_fda_grad_value(int dtype, const FdaLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_t<F32>(p, stream);
    case F16::kCode: return launch_t<F16>(p, stream);
    case BF16::kCode: return launch_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
