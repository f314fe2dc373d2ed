// Flash deformable attention backward, gradient of value, without global atomics.
//
// The reference scatters 4 * L * K * D fp32 atomicAdds per (query, head)
// (DCNv4_op/src/cuda/flash_deform_col2im_cuda.cuh:240-270 through common.h:153-184).  Sampling
// locations are free to land anywhere in their level, so unlike the DCNv4 operator there is no
// window around the query to exploit.  Instead the sampling points are first BINNED by the tile
// of their level they touch, and then a workgroup that OWNS a tile adds them up in LDS:
//
//   * the grad_sampling_loc_attn kernel, which runs first, leaves per sampling point a 16-bit key (integer position
//     of the first corner, or "outside") and a 16-byte record (position, softmax probability), both laid out
//     [image][head][level][query][point], and grad_out regrouped by head;
//   * fda_bin_points_kernel: one workgroup per chunk of 8192 points of one (image, head, level)
//     counting-sorts the chunk by tile in LDS (a point whose 2x2 corner block straddles tiles is
//     listed under each of them) and writes the sorted point ids to the chunk's region of the
//     workspace plus one (offset, count) word per tile to a table - no global atomics, no host
//     round trip, every chunk independent;
//   * fda_grad_value_kernel: persistent workgroups walk (tile, image, head) items, an XCD staying with one
//     (image, head) pair and going through its levels coarsest first.  An item collects its tile's slices of all
//     chunk lists into LDS and applies them in batches of 256 points: records and grad_out rows are requested one
//     batch ahead; per batch every corner inside the tile draws a rank in its cell's list with an integer LDS
//     atomic, a 64-entry scan gives every cell a segment, the (weight, parked row) entries are placed, and the
//     lanes of a cell walk the cell's entries with fp32 sums in registers.  The arithmetic is the reference's
//     (every term rounded to fp32, summed in fp32, rounded once to the tensor dtype); the order of the terms of a
//     cell follows the ranks, which the atomics fix per run, like the reference's atomics do;
//   * the finished tile is written to grad_value with plain stores in the tensor dtype.
//
// Tiles are at most 8x8 cells and every level is cut into 16 of them or more, so items stay
// small (several workgroups share a CU and hide each other's latencies) and comparable in size.
// Levels and tile shapes are derived on the device from the spatial_shapes tensor; the host never
// reads it.  A level with more tiles than the binning kernel's LDS histogram holds raises a flag in
// GradState: this kernel then writes zeros and the atomic fallback kernel adds everything (in fp32).
#include <algorithm>

#include "common.hpp"
#include "launch.hpp"

namespace dcn {

namespace {

constexpr int kBinThreads = 1024;
constexpr int kBinWordsPerLane = kFdaChunkPoints / 2 / kBinThreads;      // dwords of two keys per lane: 4
constexpr int kBinSortedCap = 2 * kFdaChunkPoints;                       // list entries of a chunk put together in LDS
constexpr int kBatch = 256;                  // listed points per batch: one per lane of the first four waves
constexpr int kListCap = 1024;               // listed point ids held in LDS at a time
constexpr int kTabCap = 256;                 // chunk table entries held in LDS at a time
constexpr int kTileCells = 64;               // tiles have at most 8 x 8 cells
constexpr int kSubLists = 1;                 // sub-lists (groups of lanes) every cell has at least; small tiles get more

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
  __shared__ __align__(16) uint16_t s_sorted[kBinSortedCap];      // the sorted list's first entries, as point numbers inside the chunk
  const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid / kWave;
  const int QK = p.Q * p.K;
  const int chunk = blockIdx.x % p.n_chunks, seg = blockIdx.x / p.n_chunks;       // seg = (image * G + head) * L + level
  const int l = seg % p.L;
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

  auto touch_of = [&](uint32_t k16, uint32_t pt) {
    Touch t;
    t.t00 = 0xffffffffu; t.dx = t.dy = 0u;
    if (pt >= (uint32_t)QK || k16 == kFdaKeyOutside) return t;
    int y1 = (int)(k16 >> 8), x1 = (int)(k16 & 0xffu);             // y0 + 1, x0 + 1
    if (k16 == kFdaKeySaturated) {                                // position beyond the key's fields: recompute it
      const f32x4_t rec = p.recs[(size_t)seg * QKp + pt];          // the position the first backward kernel formed
      const Tap tp = make_tap(rec.y, rec.x, lp.H, lp.W, 0u, 0u);
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
    const uint32_t word = __builtin_nontemporal_load(keys + min(w, n_words - 1));
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

  // ---- pass 2: place.  The list is put together in LDS and leaves in whole 16-byte pieces (scattered 4-byte stores
  // cost the L2 a request each); entries beyond what the LDS array holds - a chunk whose points mostly straddle
  // tiles - go to memory directly.
  uint32_t total = 0;
  for (int w = 0; w < kBinThreads / kWave; ++w) total += s_wave_sum[w];
  uint32_t *region = p.regions + (size_t)blockIdx.x * (4 * kFdaChunkPoints);
  const uint32_t pt0 = (uint32_t)chunk * kFdaChunkPoints;
  auto place = [&](uint32_t tile, uint32_t local) {
    const uint32_t at = atomicAdd(&s_hist[tile], 1u);
    if (at < (uint32_t)kBinSortedCap) s_sorted[at] = (uint16_t)local;
    else region[at] = pt0 + local;
  };
#pragma unroll
  for (int u = 0; u < kBinWordsPerLane; ++u) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const Touch t = touch[2 * u + h];
      if (t.t00 == 0xffffffffu) continue;
      const uint32_t local = 2u * (uint32_t)(u * kBinThreads + tid) + h;
      place(t.t00, local);
      if (t.dx) place(t.t00 + 1, local);
      if (t.dy) place(t.t00 + lp.ntx, local);
      if (t.dx && t.dy) place(t.t00 + lp.ntx + 1, local);
    }
  }
  __syncthreads();
  const uint32_t n_lds = min(total, (uint32_t)kBinSortedCap);
  for (uint32_t i = 4u * tid; i < n_lds; i += 4u * kBinThreads) {      // the last piece may run past the list, inside the region
    const u32x2 w = *reinterpret_cast<const u32x2 *>(s_sorted + i);
    __builtin_nontemporal_store(u32x4{pt0 + (w.x & 0xffffu), pt0 + (w.x >> 16), pt0 + (w.y & 0xffffu), pt0 + (w.y >> 16)},
                                reinterpret_cast<u32x4 *>(region + i));
  }
}

// ------------------------------------------------------------------------------- accumulation
// Inclusive prefix sum over a wave with DPP moves (rows of 16 lanes by shifts, then row broadcasts).
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_add(uint32_t v) {
  return v + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, ROW_MASK, 0xf, false);
}
__device__ __forceinline__ uint32_t wave_inclusive_scan(uint32_t v) {
  v = dpp_add<0x111, 0xf>(v);      // row_shr:1
  v = dpp_add<0x112, 0xf>(v);      // row_shr:2
  v = dpp_add<0x114, 0xf>(v);      // row_shr:4
  v = dpp_add<0x118, 0xf>(v);      // row_shr:8
  v = dpp_add<0x142, 0xa>(v);      // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xc>(v);      // row_bcast:31 into rows 2 and 3
  return v;
}

// CW: channels a lane accumulates (at most 16 bytes of the tensor dtype); LPC lanes (4 or 8) share a cell, so a cell
// holds DP = LPC * CW channels (the head width rounded up to 8, 16 or 32).  A workgroup has one lane per (cell, part):
// 64 * LPC lanes.  grad_out rows are parked in LDS in the tensor dtype.
template <typename Tag, int CW, int LPC, int SUBS>
__global__ void __launch_bounds__(kTileCells * LPC * SUBS) fda_grad_value_kernel(const FdaLaunch p) {
  extern __shared__ __align__(16) uint32_t lds32[];      // 16-byte aligned behind the static arrays: LDS stalls on 8- and 16-byte accesses that are not
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int kSlots = kTileCells * SUBS;                   // every cell has at least SUBS sub-lists
  constexpr int kApplyThreads = kSlots * LPC;
  static_assert(kBatch <= kApplyThreads && (kBatch * LPC) % kApplyThreads == 0, "a lane per point, whole rows per lane");
  constexpr int kCellLanes = LPC;
  constexpr int kCellLanesLog2 = LPC == 8 ? 3 : 2;
  constexpr int DP = CW * kCellLanes;
  constexpr int kParkBytes = Tag::kBytes;
  constexpr int kGoStride = (((DP * kParkBytes + 15) / 16) | 1) * 16;     // an odd number of 16-byte units per parked row
  // D: the head's channels in memory; this launch accumulates the window [c0, c0 + Dc) of them (heads wider than 32
  // channels take several launches over the same records and lists)
  const int D = p.D, c0 = p.gv_c0, Dc = p.gv_dc, QK = p.Q * p.K;
  uint32_t *s_count = lds32;                                  // [kTileCells] entries per cell in this batch
  uint32_t *s_offs = s_count + kTileCells;                    // [kTileCells + 4] first entry of every cell, then the total
  uint32_t *s_list = s_offs + kTileCells + 4;                 // [kListCap] listed point ids
  uint32_t *s_tab = s_list + kListCap;                        // [kTabCap] (offset | count << 16) of the item's tile per chunk
  uint32_t *s_pre = s_tab + kTabCap;                          // [kTabCap + 4] exclusive prefix of the counts
  u32x2 *s_entry = reinterpret_cast<u32x2 *>(s_pre + kTabCap + 4);      // [4 * kBatch + 2] (weight, parked row), sorted by cell
  char *s_go = reinterpret_cast<char *>(s_entry + 4 * kBatch + 2);      // [kBatch + 1] parked grad_out rows of the batch, then a row of zeros
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
  if (tid < kTileCells) s_count[tid] = 0u;
  if (tid < kGoStride / 4) reinterpret_cast<uint32_t *>(s_go + kBatch * kGoStride)[tid] = 0u;      // the row of zeros
  __syncthreads();
  const int n_tiles = s_first[p.L];
  const int BG = p.n_img * p.G;

  // value rows that no level covers (spatial_size beyond the levels, gaps between them) get zeros, like the
  // reference's zeros_like(value) (flash_deform_attn_cuda.cu:118); whole rows, by the launch of the first window
  if (c0 == 0) {
    const long long rows = (long long)p.n_img * p.N;
    const int row_elems = p.G * p.D;
    for (long long r = (long long)blockIdx.x * kApplyThreads + tid; r < rows; r += (long long)gridDim.x * kApplyThreads) {
      const int n = (int)(r % p.N);
      bool covered = false;
      for (int l = 0; l < p.L; ++l) covered |= n >= s_plan[l].start && n < s_plan[l].start + s_plan[l].H * s_plan[l].W;
      if (!covered) {
        elem_t *row = reinterpret_cast<elem_t *>(p.grad_value) + (size_t)r * row_elems;
        for (int i = 0; i < row_elems; ++i) row[i] = elem_t(0);
      }
    }
  }

  const bool usable = p.state->reserved == 0u;               // else the atomic fallback kernel adds everything
  const size_t QKp = fda_key_stride(p.Q, p.K);
  const int my_slot = tid >> kCellLanesLog2, my_part = tid & (kCellLanes - 1);      // slot: (cell, sub-list), 64 of them

  // Item order.  The hardware deals consecutive workgroup ids to the 8 XCDs in turn.  When the (image, head) pairs
  // divide evenly among them, an XCD works through its pairs one after the other, and through a pair level by level
  // (coarsest first): the pair's regrouped grad_out rows and the level's point records and lists - a few MB - then
  // stay in that XCD's L2 while its points are gathered.  Otherwise tiles are dealt over everything, in the same
  // level order.
  const bool by_pair = BG % kXcds == 0 && (int)gridDim.x % kXcds == 0;
  const int n_items = n_tiles * BG;
  const int xcd = blockIdx.x % kXcds, wg_in_xcd = blockIdx.x / kXcds, wgs_per_xcd = gridDim.x / kXcds;
  const int items_per_xcd = n_items / kXcds;
  for (int it = by_pair ? wg_in_xcd : (int)blockIdx.x; it < (by_pair ? items_per_xcd : n_items); it += by_pair ? wgs_per_xcd : (int)gridDim.x) {
    int rank, bg;
    if (by_pair) {
      const int j = it / n_tiles;                             // the XCD's j-th pair
      rank = it - j * n_tiles;
      bg = j * kXcds + xcd;
    } else {
      rank = it / BG;
      bg = it - rank * BG;
    }
    const int b = bg / p.G, g = bg - b * p.G;
    int l = 0;
    for (int i = 0; i < p.L; ++i)       // first ranks fall with the level index: the first level whose rank fits
      if (s_first[i] <= rank && s_plan[i].nty * s_plan[i].ntx > 0) { l = i; break; }
    const LevelPlan lp = s_plan[l];
    const int t_in = rank - s_first[l];
    const int ty = t_in / lp.ntx, tx = t_in - ty * lp.ntx;
    const int ty0 = ty * lp.th, tx0 = tx * lp.tw;
    const int th = min(lp.th, lp.H - ty0), tw = min(lp.tw, lp.W - tx0);
    const int n_cells = th * tw;                             // <= 64
    // A tile of few cells gives every cell several lanes: cells rounded up to a power of two, 64 / that many sub-lists
    // per cell; lane (cell, sub) takes the cell's entries sub, sub + n_sub, ...; the partial sums meet at the end.
    int cells_log2 = 0;
    while ((1 << cells_log2) < n_cells) ++cells_log2;
    const int n_sub = kSlots >> cells_log2;
    const int my_cell = my_slot & ((1 << cells_log2) - 1), my_sub = my_slot >> cells_log2;
    const int seg = bg * p.L + l;
    const float Hf = (float)lp.H, Wf = (float)lp.W;

    float acc[CW];
#pragma unroll
    for (int c = 0; c < CW; ++c) acc[c] = 0.f;

    // Everything a batch needs is requested through range-checked buffer loads of raw words: no branches
    // around the loads, so they all fly together, and nothing is converted before it is needed.
    const __amdgpu_buffer_rsrc_t rec_rs = make_rsrc(p.recs + (size_t)seg * QKp, (uint32_t)QK * 16u);
    const __amdgpu_buffer_rsrc_t go_rs = make_rsrc(reinterpret_cast<const elem_t *>(p.go_rows) + (size_t)bg * p.Q * D,
                                                   (uint32_t)((size_t)p.Q * D * Tag::kBytes));
    // kCellLanes lanes fetch a listed point's grad_out row, CW channels each; a lane serves kRowsPerLane rows of a batch.
    typedef typename RawWord<CW * Tag::kBytes>::type goN_t;
    constexpr int kRowsPerLane = kBatch * kCellLanes / kApplyThreads;
    constexpr int kRowStep = kApplyThreads / kCellLanes;
    struct Ahead {
      u32x4 rec;                       // this lane's point of the batch: x, y, probability
      goN_t go[kRowsPerLane];
    };
    auto fetch = [&](uint32_t b0, int nb) {
      Ahead a;
      {
        const uint32_t pt = s_list[min((int)b0 + min(tid, max(nb - 1, 0)), kListCap - 1)];
        a.rec = buffer_load<16>(rec_rs, tid < nb ? pt * 16u : kDropOffset);
      }
#pragma unroll
      for (int u = 0; u < kRowsPerLane; ++u) {
        const int h = my_slot + u * kRowStep;
        const bool live = h < nb && my_part * CW < Dc;
        const uint32_t q = s_list[min((int)b0 + min(h, max(nb - 1, 0)), kListCap - 1)] / (uint32_t)p.K;
        a.go[u] = buffer_load<CW * Tag::kBytes>(go_rs, live ? (q * (uint32_t)D + (uint32_t)(c0 + my_part * CW)) * Tag::kBytes : kDropOffset);
      }
      return a;
    };

    // Applies the first n entries of s_list in batches of kBatch points, one lane per point:
    //   A      the lane rebuilds its point's position; each corner inside the tile draws a rank in its cell
    //          (integer LDS atomic) - barrier
    //   scan   exclusive prefix sum of the 64 cell counts (one wave); all lanes park the batch's grad_out rows - barrier
    //   place  (weight, parked row) entries go to cell start + rank; the next batch's loads are requested - barrier
    //   B      four lanes per cell walk the cell's entries: sum += weight * grad_out row, fp32, in registers.
    // No barrier after B: the next batch's phase A only touches the counters, and everything B reads is rewritten
    // after that batch's first barrier.
    auto apply_list = [&](uint32_t n) {
      if (n == 0) return;
      int nb = (int)min((uint32_t)kBatch, n);
      Ahead cur = fetch(0, nb);
      for (uint32_t b0 = 0; b0 < n; b0 += kBatch) {
        // ---- phase A
        float rec_w[4] = {0.f, 0.f, 0.f, 0.f};
        uint32_t rec_cr[4] = {~0u, ~0u, ~0u, ~0u};            // cell << 16 | rank
        if (tid < nb) {
          // the position the first backward kernel formed (flash_deform_im2col_cuda.cuh:188-189), and the probability
          // (a vector element is copied to a scalar first: a bit cast of the element expression itself reads element 0)
          const uint32_t rx = cur.rec.x, ry = cur.rec.y, rz = cur.rec.z;
          const float x = __builtin_bit_cast(float, rx), y = __builtin_bit_cast(float, ry);
          if ((y > -1.f) && (x > -1.f) && (y < Hf) && (x < Wf)) {
            const float fy = floorf(y), fx = floorf(x);
            const float ly = y - fy, lx = x - fx, hy = 1.f - ly, hx = 1.f - lx;
            const float pr = __builtin_bit_cast(float, rz);
            const float w4[4] = {hy * hx, hy * lx, ly * hx, ly * lx};
            // corner 0 relative to the tile; a corner inside the tile is inside the level (tiles are clipped to it)
            const int cy0 = (int)fy - ty0, cx0 = (int)fx - tx0;
#pragma unroll
            for (int cn = 0; cn < 4; ++cn) {
              const int cy = cy0 + (cn >> 1), cx = cx0 + (cn & 1);
              if ((unsigned)cy < (unsigned)th && (unsigned)cx < (unsigned)tw) {
                const uint32_t cell = (uint32_t)(cy * tw + cx);
                rec_w[cn] = pr * w4[cn];
                rec_cr[cn] = (cell << 16) | __hip_atomic_fetch_add(&s_count[cell], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
              }
            }
          }
        }
        __syncthreads();

        // ---- scan (first wave) and park (everyone)
        if (tid < kWave) {
          const uint32_t c = s_count[tid];
          const uint32_t incl = wave_inclusive_scan(c);
          s_offs[tid] = incl - c;
          if (tid == kWave - 1) s_offs[kWave] = incl;
        }
#pragma unroll
        for (int u = 0; u < kRowsPerLane; ++u) {
          const int h = my_slot + u * kRowStep;
          if (h >= nb) break;
          *reinterpret_cast<goN_t *>(s_go + h * kGoStride + my_part * (CW * kParkBytes)) = cur.go[u];
        }
        __syncthreads();

        // ---- place
        if (tid < kTileCells) s_count[tid] = 0u;              // for the next batch; the scan has read them
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          const uint32_t cr = rec_cr[cn];
          if (cr == ~0u) continue;
          s_entry[s_offs[cr >> 16] + (cr & 0xffffu)] = u32x2{__builtin_bit_cast(uint32_t, rec_w[cn]), (uint32_t)(tid * kGoStride)};
        }
        const int nb_next = b0 + kBatch < n ? (int)min((uint32_t)kBatch, n - b0 - kBatch) : 0;
        cur = fetch(b0 + kBatch, nb_next);      // flies while this batch is applied (after the last batch: nothing is read)
        __syncthreads();

        // ---- phase B: a lane walks every n_sub-th entry of its cell, two at a time and without branches inside
        // (past the end of the list: weight 0 times the row of zeros), so that all LDS reads of a step are in
        // flight together
        if (my_cell < n_cells) {
          const uint32_t beg = s_offs[my_cell], end = s_offs[my_cell + 1];
          const char *go_lane = s_go + my_part * (CW * kParkBytes);
          const uint32_t step = (uint32_t)n_sub;
          for (uint32_t e = beg + (uint32_t)my_sub; e < end; e += 2u * step) {
            const bool two = e + step < end;
            const u32x2 ent0 = s_entry[e];
            u32x2 ent1 = s_entry[two ? e + step : e];
            ent1.x = two ? ent1.x : 0u;
            ent1.y = two ? ent1.y : (uint32_t)(kBatch * kGoStride);
            const goN_t row0 = *reinterpret_cast<const goN_t *>(go_lane + ent0.y);
            const goN_t row1 = *reinterpret_cast<const goN_t *>(go_lane + ent1.y);
            const uint32_t w0_bits = ent0.x, w1_bits = ent1.x;
            const float w0 = __builtin_bit_cast(float, w0_bits), w1 = __builtin_bit_cast(float, w1_bits);
            float g0[CW], g1[CW];
            Pack<Tag, CW>::decode(row0, g0);
            Pack<Tag, CW>::decode(row1, g1);
#pragma unroll
            for (int c = 0; c < CW; ++c) acc[c] = fmaf(w1, g1[c], fmaf(w0, g0[c], acc[c]));
          }
        }
        nb = nb_next;
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
            const uint32_t incl = wave_inclusive_scan(v);
            if (c < nc) s_pre[c] = run + incl - v;
            run += (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
          }
          if (tid == 0) s_pre[nc] = run;
        }
        __syncthreads();
        const uint32_t total = s_pre[nc];
        // copy the slices into s_list, kListCap entries at a time; lane -> entry -> chunk by bisection
        for (uint32_t e0 = 0; e0 < total; e0 += kListCap) {
          const uint32_t ne = min((uint32_t)kListCap, total - e0);
          __syncthreads();                                     // the previous list has been fetched from
          for (uint32_t i = tid; i < ne; i += kApplyThreads) {
            const uint32_t e = e0 + i;
            int lo = 0, hi = nc;                       // largest c with s_pre[c] <= e
            while (hi - lo > 1) {
              const int mid = (lo + hi) >> 1;
              if (s_pre[mid] <= e) lo = mid; else hi = mid;
            }
            const uint32_t *region = p.regions + ((size_t)seg * p.n_chunks + c0 + lo) * (4 * kFdaChunkPoints);
            s_list[i] = __builtin_nontemporal_load(region + (s_tab[lo] & 0xffffu) + (e - s_pre[lo]));      // read once
          }
          __syncthreads();
          apply_list(ne);
        }
      }
    }

    // ---- the tile is complete: the sub-lists' partial sums meet in LDS, then registers -> memory (zeros when the
    // binning gave up: the fallback kernel then adds everything).  The lanes of a cell write DP contiguous channels.
    if (n_sub > 1) {
      __syncthreads();                                       // the last phase B is over: lists, entries and rows are free
      float *s_part = reinterpret_cast<float *>(s_list);     // [kSlots][kCellLanes][CW]
#pragma unroll
      for (int c = 0; c < CW; ++c) s_part[(tid * CW) + c] = acc[c];
      __syncthreads();
      if (my_sub == 0) {
        for (int j = 1; j < n_sub; ++j) {
          const float *o = s_part + ((((j << cells_log2) + my_cell) << kCellLanesLog2) + my_part) * CW;
#pragma unroll
          for (int c = 0; c < CW; ++c) acc[c] += o[c];
        }
      }
      __syncthreads();                                       // read before the row of zeros is restored
      if (tid < kGoStride / 4) reinterpret_cast<uint32_t *>(s_go + kBatch * kGoStride)[tid] = 0u;
    }
    if (my_cell < n_cells && my_sub == 0) {
      const int cy = my_cell / tw, cx = my_cell - cy * tw;
      const long long n = (long long)lp.start + (long long)(ty0 + cy) * lp.W + tx0 + cx;      // level tables are not validated
      if (n >= 0 && n < p.N) {
        elem_t *dst = reinterpret_cast<elem_t *>(p.grad_value) + (((size_t)b * p.N + (size_t)n) * p.G + g) * D + c0 + my_part * CW;
        if ((D % CW) == 0 && (Dc % CW) == 0 && (CW * Tag::kBytes) % 4 == 0) {
          if (my_part * CW < Dc) __builtin_nontemporal_store(Pack<Tag, CW>::encode(acc), reinterpret_cast<goN_t *>(dst));
        } else {
#pragma unroll
          for (int c = 0; c < CW; ++c)
            if (my_part * CW + c < Dc) { const float f[1] = {acc[c]}; dst[c] = Pack<Tag, 1>::encode(f); }
        }
      }
    }
  }
}

// lanes per cell: four, or eight when four lanes of 16 bytes do not cover the (padded) head width
int fda_cell_lanes(int D, int elem_bytes) { return fda_padded_channels(D) * elem_bytes > 64 ? 8 : 4; }
int fda_sub_lists_for(int) { return kSubLists; }

template <typename Tag>
hipError_t launch_t(const FdaLaunch &p, hipStream_t stream) {
  // binning: one workgroup per chunk of every (image, head, level); once, in front of the first channel window
  if (p.gv_c0 == 0) {
    hipLaunchKernelGGL(fda_bin_points_kernel<Tag>, dim3((unsigned)(p.n_img * p.G * p.L * p.n_chunks)), dim3(kBinThreads), 0, stream, p);
    if (hipError_t e = hipGetLastError()) return e;
  }

  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  const size_t lds = fda_grad_value_lds_bytes(p, Tag::kBytes);
  const int lpc = fda_cell_lanes(p.gv_dc, Tag::kBytes), cw = fda_padded_channels(p.gv_dc) / lpc;
  const int subs = fda_sub_lists_for(lpc);
  const int threads = kTileCells * lpc * subs;
  // persistent workgroups: as many per CU as LDS and wave slots (32 per CU) allow
  // persistent workgroups: as many as are resident at once (registers, LDS and wave slots decide)
  const dim3 block((unsigned)threads);
  auto go = [&](auto kernel) -> hipError_t {
    if (hipError_t e = ensure_dynamic_lds_limit(reinterpret_cast<const void *>(kernel), kMaxLdsPerWorkgroup - 2048)) return e;
    int per_cu = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, lds) != hipSuccess || per_cu < 1) per_cu = 1;
    hipLaunchKernelGGL(kernel, dim3((unsigned)(cus * per_cu)), block, lds, stream, p);
    return hipGetLastError();
  };
  if (lpc == 8) {
    if constexpr (Tag::kBytes == 4) {
      if (cw == 4) return go(fda_grad_value_kernel<Tag, 4, 8, kSubLists>);      // fp32 heads of 17 .. 32 channels
    }
    return hipErrorInvalidValue;
  }
  switch (cw) {
    case 2: return go(fda_grad_value_kernel<Tag, 2, 4, kSubLists>);
    case 4: return go(fda_grad_value_kernel<Tag, 4, 4, kSubLists>);
    case 8:
      if constexpr (Tag::kBytes == 2) return go(fda_grad_value_kernel<Tag, 8, 4, kSubLists>);
      break;
  }
  return hipErrorInvalidValue;      // wider heads take the atomic path (the entry point checks)
}

}  // namespace

size_t fda_grad_value_lds_bytes(const FdaLaunch &p, int elem_bytes) {
  const size_t go_stride = ((((size_t)fda_padded_channels(p.gv_dc) * elem_bytes + 15) / 16) | 1) * 16;
  const size_t head = ((size_t)2 * kTileCells + 4) * sizeof(uint32_t);
  const size_t batch = head + ((size_t)kListCap + 2 * kTabCap + 4) * sizeof(uint32_t) + ((size_t)4 * kBatch + 2) * sizeof(u32x2) +
                       (size_t)(kBatch + 1) * go_stride;
  // the sub-lists' partial sums meet in LDS behind the counters: a float per lane and channel it holds
  const size_t meet = head + (size_t)kTileCells * kSubLists * fda_padded_channels(p.gv_dc) * sizeof(float);
  return std::max(batch, meet);
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
