// DCNv4 backward, gradient of the input (grad_value): no atomics on data, fp32 sums in registers.
//
// The reference scatters 36*C fp32 atomicAdds per output pixel into memory
// (DCNv4_op/src/cuda/common.h:153-184 called from dcnv4_col2im_cuda.cuh:280-350).  On MI355X the
// memory-side atomic units retire about one dword per clock per channel, which caps that scheme
// two orders of magnitude below the HBM roofline, and LDS floating-point atomics are serialised
// per lane.  This kernel turns the scatter into a gather:
//
//   * a workgroup OWNS a tile_h x tile_w tile of the input image for a chunk of groups, and is
//     the only writer of that part of grad_value: plain stores, no clearing pass, no cast pass;
//   * a (cell, group) of the tile is a SLOT; a lane owns one slot (or one part of it when a group
//     is wider than 32 channels) and keeps the slot's sums in fp32 registers for the whole
//     kernel - the arithmetic is the reference's: every term rounded to fp32, summed in fp32,
//     the result rounded once to the tensor dtype;
//   * the workgroup visits every output pixel whose reference point lies within the reach the
//     data needs (GradState::reach_needed, written by the grad_offset_mask kernel that runs
//     first; any value up to the whole image), in strips of interleaved rows, so that every
//     strip spreads its terms evenly over the tile.  Per strip:
//       park   the strip's grad_out rows are copied to LDS;
//       A      one lane per (group, pixel, kernel tap) recomputes the sampling position; for each
//              of its corners inside the tile it draws a rank in the corner's slot with an
//              integer LDS atomic (ds_add_rtn_u32) and keeps (weight, slot, rank) in registers;
//       scan   an exclusive prefix sum of the slot counts gives every slot a segment of the
//              entry array;
//       place  the lanes write their (weight, address of the pixel's parked grad_out) entries
//              to segment start + rank: the entries are now sorted by slot;
//       B      every lane walks its own slot's entries: sum += weight * grad_out row.
// Integer atomics only order the entries inside a slot; sums depend on that order at the level
// of fp32 rounding, like the reference's atomics do.
#include <algorithm>

#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

constexpr int kValThreads = 1024;

// grad_out is parked in LDS as it is for fp32 and fp16 tensors (fp16 feeds mixed-precision FMAs directly)
// and widened to fp32 for bf16.
template <typename Tag> struct ParkType { typedef float type; };
template <> struct ParkType<F16> { typedef _Float16 type; };

__device__ __forceinline__ int fdiv_small(int n, float inv) { return (int)(((float)n + 0.5f) * inv); }   // exact for n < 2^20

// Inclusive prefix sum over the 64 lanes of a wave with DPP moves: within rows of 16 lanes by shifts, then the last
// lane of a row is broadcast into the rows after it.  Lanes without a source add 0.
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
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_readlane((int)wave_inclusive_scan(v), kWave - 1);
}

// CW: channels a lane accumulates (8, 16 or 32): the group width rounded up, or 32 with several lanes per slot.
template <typename Tag, int KP, int CW, int ROUNDS>
__global__ void __launch_bounds__(kValThreads) dcnv4_grad_value_kernel(const DcnLaunch p) {
  extern __shared__ __align__(16) uint32_t lds32[];
  typedef typename ParkType<Tag>::type park_t;
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int kParkBytes = sizeof(park_t);
  constexpr int kLaneBytes = CW * kParkBytes;                 // bytes of a parked row a lane reads per entry
  const int Kp = p.Kp, D = p.D, C = p.G * p.D;
  const int n_chunks = (p.G + p.ng_chunk - 1) / p.ng_chunk;
  const int nty = (p.H + p.tile_h - 1) >> p.tile_h_log2, ntx = (p.W + p.tile_w - 1) >> p.tile_w_log2;
  uint32_t id = xcd_contiguous_block(blockIdx.x, gridDim.x);
  const int chunk = id % n_chunks; id /= n_chunks;
  const int tx = id % ntx; id /= ntx;
  const int ty = id % nty;
  const int b = id / nty;
  const int g0 = chunk * p.ng_chunk, ng = min(p.ng_chunk, p.G - g0);
  const int ty0 = ty << p.tile_h_log2, tx0 = tx << p.tile_w_log2;
  const int th = min(p.tile_h, p.H - ty0), tw = min(p.tile_w, p.W - tx0);
  const int lps_log2 = p.gv_lps_log2;
  const int Dp = CW << lps_log2;                              // parked channels per group
  const int go_stride = p.gv_go_stride;                       // bytes between parked pixels (an odd number of 16-byte units)
  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);

  uint32_t *s_count = lds32;                                  // [kValThreads] entries per slot in this strip
  uint32_t *s_offs = lds32 + kValThreads;                     // [kValThreads + 4] first entry of every slot, then the total
  char *s_go = reinterpret_cast<char *>(lds32 + 2 * kValThreads + 4);
  u32x2 *s_entry = reinterpret_cast<u32x2 *>(s_go + (size_t)p.strip_pix * go_stride);

  // output pixels this tile visits: reference point (centre tap at zero offset) within `reach` of the tile
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
  const int cy0 = half_h - p.ph, cx0 = half_w - p.pw, Ho = p.Q / p.Wo;
  const int reach = (int)min(p.state->reach_needed, 1u << 20);
  const int ho_lo = max(0, ceil_div_signed(ty0 - reach - cy0, p.sh));
  const int ho_hi = min(Ho, ceil_div_signed(ty0 + p.tile_h + reach - cy0, p.sh));
  const int wo_lo_all = max(0, ceil_div_signed(tx0 - reach - cx0, p.sw));
  const int wo_hi_all = min(p.Wo, ceil_div_signed(tx0 + p.tile_w + reach - cx0, p.sw));
  const int n_rows = ho_hi - ho_lo;
  // a window wider than a strip holds is walked in blocks of columns
  const int cols_cap = max(1, min(wo_hi_all - wo_lo_all, p.strip_pix));

  // this lane's slot: (cell, group of the chunk), and its part of the group's channels
  const float inv_ng = 1.f / (float)p.ng_chunk;
  const int my_slot = tid >> lps_log2, my_part = tid & ((1 << lps_log2) - 1);
  const int my_cell = fdiv_small(my_slot, inv_ng), my_gl = my_slot - my_cell * p.ng_chunk;
  const int my_ly = my_cell >> p.tile_w_log2, my_lx = my_cell & (p.tile_w - 1);
  const bool slot_live = my_ly < th && my_lx < tw && my_gl < ng;
  float acc[CW];
#pragma unroll
  for (int c = 0; c < CW; ++c) acc[c] = 0.f;

  s_count[tid] = 0u;
  __syncthreads();

  const float x_sub = mul_rn((float)half_w, p.offset_scale), y_sub = mul_rn((float)half_h, p.offset_scale);
  const float Hf = (float)p.H, Wf = (float)p.W;
  const elem_t *om_img = reinterpret_cast<const elem_t *>(p.offset_mask) + (size_t)b * p.Q * p.P_pad;
  const elem_t *go_img = reinterpret_cast<const elem_t *>(p.grad_out) + (size_t)b * p.Q * C;
  auto load_f = [](const elem_t *ptr) { float f[1]; Pack<Tag, 1>::decode(*ptr, f); return f[0]; };
  auto to_f = [](elem_t raw) { float f[1]; Pack<Tag, 1>::decode(raw, f); return f[0]; };

  for (int wo_lo = wo_lo_all; wo_lo < wo_hi_all && n_rows > 0; wo_lo += cols_cap) {
    const int nwx = min(cols_cap, wo_hi_all - wo_lo);

    // strips of interleaved rows: strip s takes rows ho_lo + s, ho_lo + s + n_strips, ...
    const int rows_cap = max(1, p.strip_pix / nwx);
    const int n_strips = (n_rows + rows_cap - 1) / rows_cap;
    const int rows_full = (n_rows + n_strips - 1) / n_strips;           // rows of the first strips (the last ones may have one fewer)
    const int per_group = rows_full * nwx * Kp;                         // items of a group in a full strip
    const int n_items = ng * per_group;
    const float inv_per_group = 1.f / (float)per_group, inv_nwx = 1.f / (float)nwx, inv_kp = 1.f / (float)Kp;

    // Phase A work items of this lane, one per round: row of the strip | column << 10 | group << 20 | tap << 26,
    // all ones for a lane without an item.  The decode does not depend on the strip.
    uint32_t item[ROUNDS];
#pragma unroll
    for (int v = 0; v < ROUNDS; ++v) {
      const int j = v * kValThreads + tid;
      const bool in_range = j < n_items;
      const int gl = in_range ? fdiv_small(j, inv_per_group) : 0;
      const int rem = in_range ? j - gl * per_group : 0;
      const int px = KP > 0 ? rem / (KP > 0 ? KP : 1) : fdiv_small(rem, inv_kp);
      const int t = rem - px * Kp;
      const int r = fdiv_small(px, inv_nwx), col = px - r * nwx;
      item[v] = in_range ? (uint32_t)r | ((uint32_t)col << 10) | ((uint32_t)gl << 20) | ((uint32_t)t << 26) : ~0u;
    }

    // parking: 16-byte vectors when a group's channels are whole vectors and fill their parked width
    constexpr int kVec = 16 / Tag::kBytes;
    typedef typename Pack<Tag, kVec>::raw_t vec_t;
    const bool vec_park = D == Dp && D % kVec == 0;
    const int vpp = vec_park ? ng * D / kVec : ng * Dp;                 // vectors (elements) per parked pixel
    const float inv_vpp = 1.f / (float)vpp;

    // a lane's offsets and modulation scalars of a strip, requested one strip ahead (before the previous strip's
    // phase B) so that their latency hides there
    elem_t pf_x[ROUNDS], pf_y[ROUNDS], pf_m[ROUNDS];
    auto prefetch = [&](int s) {
      const int rows_s = (n_rows - s + n_strips - 1) / n_strips;
#pragma unroll
      for (int v = 0; v < ROUNDS; ++v) {
        pf_x[v] = pf_y[v] = pf_m[v] = elem_t(0);
        const uint32_t it = item[v];
        const int r = (int)(it & 0x3ffu), col = (int)((it >> 10) & 0x3ffu), gl = (int)((it >> 20) & 0x3fu), t = (int)(it >> 26);
        if (it == ~0u || r >= rows_s) continue;
        const int ho = ho_lo + s + r * n_strips, wo = wo_lo + col;
        const elem_t *om = om_img + ((uint32_t)(ho * p.Wo + wo) * (uint32_t)p.P_pad + (uint32_t)((g0 + gl) * 3 * Kp));
        pf_x[v] = om[2 * t]; pf_y[v] = om[2 * t + 1]; pf_m[v] = om[2 * Kp + t];
      }
    };
    prefetch(0);

    // Barriers of a strip: after phase A (counts complete), after scan + park (offsets and grad_out in place), after
    // place (entries in place).  None after phase B: the next strip's phase A only touches the counters, which phase B
    // does not read, and everything phase B reads is rewritten only after the next strip's first barrier.
    for (int s = 0; s < n_strips; ++s) {
      const int rows_s = (n_rows - s + n_strips - 1) / n_strips;
      const int npx = rows_s * nwx;

      // ---- phase A: one lane per (group, pixel, tap): corners inside the tile draw a rank in their slot.  A record
      // (what the lane keeps until the entries are placed): modulation and the two fractions, the slot of the first
      // corner with the corners that count, and the four ranks.
      float rec_m[ROUNDS], rec_ly[ROUNDS], rec_lx[ROUNDS];
      uint32_t rec_slot[ROUNDS], rec_rank[ROUNDS][2];       // first slot (signed, 24 bits) | corners << 24; ranks, 16 bits each
#pragma unroll
      for (int v = 0; v < ROUNDS; ++v) {
        rec_m[v] = rec_ly[v] = rec_lx[v] = 0.f;
        rec_slot[v] = rec_rank[v][0] = rec_rank[v][1] = 0u;
        if (v * kValThreads >= n_items) continue;               // uniform
        const uint32_t it = item[v];
        const int r = (int)(it & 0x3ffu), col = (int)((it >> 10) & 0x3ffu), gl = (int)((it >> 20) & 0x3fu), t = (int)(it >> 26);
        if (it == ~0u || r >= rows_s) continue;
        int ti, tj;
        if constexpr (KP > 0) {
          tap_ij_3x3(KP, t, ti, tj);
        } else {      // x index outer, y index inner, centre skipped when remove_center
          int tt = t;
          if (p.remove_center && tt >= (p.kw / 2) * p.kh + p.kh / 2) ++tt;
          ti = tt / p.kh; tj = tt - ti * p.kh;
        }
        const int ho = ho_lo + s + r * n_strips, wo = wo_lo + col;
        const float off_x = to_f(pf_x[v]), off_y = to_f(pf_y[v]);
        const float x_base = sub_rn((float)(cx0 + wo * p.sw), x_sub), y_base = sub_rn((float)(cy0 + ho * p.sh), y_sub);
        const float x = add_rn(x_base, mul_rn(add_rn((float)(ti * p.dw), off_x), p.offset_scale));
        const float y = add_rn(y_base, mul_rn(add_rn((float)(tj * p.dh), off_y), p.offset_scale));
        // the reference's range test (dcnv4_col2im_cuda.cuh:317); NaN and huge coordinates fail it
        if (!((y > -1.f) && (x > -1.f) && (y < Hf) && (x < Wf))) continue;
        const float fy = floorf(y), fx = floorf(x);
        // corner 0 relative to the tile; a corner inside the tile is inside the image (the tile is clipped to it)
        const int ly = (int)fy - ty0, lx = (int)fx - tx0;
        const bool r0 = (unsigned)ly < (unsigned)th, r1 = (unsigned)(ly + 1) < (unsigned)th;
        const bool c0 = (unsigned)lx < (unsigned)tw, c1 = (unsigned)(lx + 1) < (unsigned)tw;
        const uint32_t valid = (uint32_t)(r0 && c0) | ((uint32_t)(r0 && c1) << 1) | ((uint32_t)(r1 && c0) << 2) | ((uint32_t)(r1 && c1) << 3);
        if (valid == 0) continue;
        float m = to_f(pf_m[v]);
        if (p.softmax) {          // rare: normalise over this group's taps
          const elem_t *om = om_img + ((uint32_t)(ho * p.Wo + wo) * (uint32_t)p.P_pad + (uint32_t)((g0 + gl) * 3 * Kp));
          float mx = load_f(om + 2 * Kp), sum = 0.f;
          for (int k = 1; k < Kp; ++k) mx = fmaxf(mx, load_f(om + 2 * Kp + k));
          for (int k = 0; k < Kp; ++k) sum += __expf(load_f(om + 2 * Kp + k) - mx);
          m = __expf(m - mx) / sum;
        }
        rec_m[v] = m; rec_ly[v] = y - fy; rec_lx[v] = x - fx;
        const int slot0 = ((ly << p.tile_w_log2) + lx) * p.ng_chunk + gl;      // may be negative: corner block starts outside
        rec_slot[v] = ((uint32_t)slot0 & 0xffffffu) | (valid << 24);
        uint32_t ranks[4] = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          if (!(valid & (1u << cn))) continue;
          const int slot = slot0 + (((cn >> 1) << p.tile_w_log2) + (cn & 1)) * p.ng_chunk;
          ranks[cn] = __hip_atomic_fetch_add(&s_count[slot], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        rec_rank[v][0] = ranks[0] | (ranks[1] << 16);
        rec_rank[v][1] = ranks[2] | (ranks[3] << 16);
        __builtin_amdgcn_sched_barrier(0);      // one round at a time: interleaved, the rounds' temporaries spill
      }
      __syncthreads();

      // ---- scan: exclusive prefix sum of the slot counts (a wave adds up the counts of the waves before it itself)
      {
        const uint32_t c = s_count[tid];
        const uint32_t incl = wave_inclusive_scan(c);
        uint32_t before = 0;
        for (int w = 0; w < wave; ++w) before += s_count[w * kWave + lane];
        before = wave_sum(before);
        s_offs[tid] = before + incl - c;
        if (tid == kValThreads - 1) s_offs[kValThreads] = before + incl;
      }

      // ---- park the strip's grad_out (this chunk's channels)
      for (int idx = tid; idx < npx * vpp; idx += kValThreads) {
        const int px = fdiv_small(idx, inv_vpp), u = idx - px * vpp;
        const int r = fdiv_small(px, inv_nwx), col = px - r * nwx;
        const elem_t *src = go_img + ((size_t)((ho_lo + s + r * n_strips) * p.Wo + wo_lo + col) * C + g0 * D);
        char *dst = s_go + px * go_stride;
        if (vec_park) {
          const vec_t raw = *reinterpret_cast<const vec_t *>(src + u * kVec);
          if constexpr (Tag::kCode == BF16::kCode) {
            float f[kVec];
            Pack<Tag, kVec>::decode(raw, f);
            f32x4 *d4 = reinterpret_cast<f32x4 *>(dst + u * kVec * 4);
            d4[0] = f32x4{f[0], f[1], f[2], f[3]};
            d4[1] = f32x4{f[4], f[5], f[6], f[7]};
          } else {
            *reinterpret_cast<vec_t *>(dst + u * 16) = raw;
          }
        } else {
          const int gl = u / Dp, ch = u - gl * Dp;
          const float f = ch < D ? load_f(src + gl * D + ch) : 0.f;
          reinterpret_cast<park_t *>(dst)[u] = (park_t)f;
        }
      }
      __syncthreads();

      // ---- place: the entries, sorted by slot
      s_count[tid] = 0u;                                         // for the next strip; nobody reads the counts any more
#pragma unroll
      for (int v = 0; v < ROUNDS; ++v) {
        if (v * kValThreads >= n_items) continue;
        const uint32_t valid = rec_slot[v] >> 24;
        if (valid == 0) continue;
        const int slot0 = (int)(rec_slot[v] << 8) >> 8;          // sign-extend 24 bits
        const uint32_t it = item[v];
        const int px = (int)(it & 0x3ffu) * nwx + (int)((it >> 10) & 0x3ffu), gl = (int)((it >> 20) & 0x3fu);
        const uint32_t go_addr = (uint32_t)(px * go_stride + gl * Dp * kParkBytes);
        const float m = rec_m[v], ly = rec_ly[v], lx = rec_lx[v], hy = 1.f - ly, hx = 1.f - lx;
        const float wv[4] = {m * (hy * hx), m * (hy * lx), m * (ly * hx), m * (ly * lx)};     // common.h:48-58, 153-184
        const uint32_t ranks[4] = {rec_rank[v][0] & 0xffffu, rec_rank[v][0] >> 16, rec_rank[v][1] & 0xffffu, rec_rank[v][1] >> 16};
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          if (!(valid & (1u << cn))) continue;
          const int slot = slot0 + (((cn >> 1) << p.tile_w_log2) + (cn & 1)) * p.ng_chunk;
          s_entry[s_offs[slot] + ranks[cn]] = u32x2{__builtin_bit_cast(uint32_t, wv[cn]), go_addr};
        }
      }
      if (s + 1 < n_strips) prefetch(s + 1);
      __syncthreads();

      // ---- phase B: every lane sums its slot's entries; the next entry is read while the current one is applied
      if (slot_live) {
        uint32_t e = s_offs[my_slot];
        const uint32_t end = s_offs[my_slot + 1];
        const char *go_lane = s_go + my_part * kLaneBytes;
        u32x2 ent = s_entry[e];                                  // (one entry past the last is inside the allocation)
        while (e < end) {
          const u32x2 next = s_entry[++e];
          const uint32_t w_bits = ent.x;
          const float w = __builtin_bit_cast(float, w_bits);
          const char *g = go_lane + ent.y;
          park_t gv[CW];
#pragma unroll
          for (int q = 0; q < kLaneBytes / 16; ++q)
            *reinterpret_cast<u32x4 *>(reinterpret_cast<char *>(gv) + 16 * q) = *reinterpret_cast<const u32x4 *>(g + 16 * q);
#pragma unroll
          for (int c = 0; c < CW; ++c) acc[c] = fmaf(w, (float)gv[c], acc[c]);
          ent = next;
        }
      }
    }
  }
  __syncthreads();      // the last phase B is over: LDS is free

  // The tile is complete: registers -> tensor dtype -> memory.  Whole 16-byte pieces go through LDS so that the lanes
  // of a store instruction cover consecutive pieces of a (cell, group) instead of one piece of 64 different ones.
  constexpr int kVecOut = 16 / Tag::kBytes;
  if (D % kVecOut == 0) {
    constexpr int kPieces = CW / kVecOut;                       // 16-byte pieces a lane holds
    u32x4 *s_out = reinterpret_cast<u32x4 *>(lds32);
#pragma unroll
    for (int q = 0; q < kPieces; ++q) {
      float f[kVecOut];
#pragma unroll
      for (int i = 0; i < kVecOut; ++i) f[i] = acc[q * kVecOut + i];
      s_out[tid * kPieces + q] = Pack<Tag, kVecOut>::encode(f);
    }
    __syncthreads();
    elem_t *gv_img = reinterpret_cast<elem_t *>(p.grad_value) + (size_t)b * p.H * p.W * C;
#pragma unroll
    for (int k = 0; k < kPieces; ++k) {
      const int idx = k * kValThreads + tid;
      const int src = idx / kPieces, q = idx - src * kPieces;   // the lane that held this piece, and which of its pieces
      const int slot = src >> lps_log2, part = src & ((1 << lps_log2) - 1);
      const int cell = fdiv_small(slot, inv_ng), gl = slot - cell * p.ng_chunk;
      const int cy = cell >> p.tile_w_log2, cx = cell & (p.tile_w - 1);
      const int ch = part * CW + q * kVecOut;                   // first channel of the piece within its group
      if (cy < th && cx < tw && gl < ng && ch < D)
        *reinterpret_cast<u32x4 *>(gv_img + ((size_t)((ty0 + cy) * p.W + tx0 + cx) * C + (g0 + gl) * D + ch)) = s_out[idx];
    }
  } else if (slot_live) {
    const int ch0 = my_part * CW;
    elem_t *dst = reinterpret_cast<elem_t *>(p.grad_value) +
                  ((((size_t)b * p.H + ty0 + my_ly) * p.W + tx0 + my_lx) * C + (g0 + my_gl) * D + ch0);
#pragma unroll
    for (int c = 0; c < CW; ++c) {
      if (ch0 + c < D) {
        const float f[1] = {acc[c]};
        dst[c] = Pack<Tag, 1>::encode(f);
      }
    }
  }
}

template <typename Tag>
hipError_t launch_t(const DcnLaunch &p, hipStream_t stream) {
  const int n_chunks = (p.G + p.ng_chunk - 1) / p.ng_chunk;
  const int nty = (p.H + p.tile_h - 1) >> p.tile_h_log2, ntx = (p.W + p.tile_w - 1) >> p.tile_w_log2;
  const dim3 grid((unsigned)(p.n_img * nty * ntx * n_chunks)), block(kValThreads);
  const size_t lds = dcnv4_grad_value_lds_bytes(p);
  const bool k3 = p.kh == 3 && p.kw == 3;
  auto go = [&](auto kernel) -> hipError_t {
    if (hipError_t e = ensure_dynamic_lds_limit(reinterpret_cast<const void *>(kernel), kMaxLdsPerWorkgroup)) return e;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return hipGetLastError();
  };
#define GV_CASE(KPV)                                                                \
  do {                                                                              \
    if (p.gv_cw == 8) return go(dcnv4_grad_value_kernel<Tag, KPV, 8, dcnv4_grad_value_rounds(8)>);      \
    if (p.gv_cw == 16) return go(dcnv4_grad_value_kernel<Tag, KPV, 16, dcnv4_grad_value_rounds(16)>);   \
    return go(dcnv4_grad_value_kernel<Tag, KPV, 32, dcnv4_grad_value_rounds(32)>);                      \
  } while (0)
  if (k3 && !p.remove_center) GV_CASE(9);
  if (k3 && p.remove_center) GV_CASE(8);
  GV_CASE(0);
#undef GV_CASE
}

}  // namespace

size_t dcnv4_grad_value_lds_bytes(const DcnLaunch &p) {
  const size_t items = (size_t)p.strip_pix * p.Kp * p.ng_chunk;
  // counters and offsets, parked grad_out, entries (+ the one the read-ahead of phase B touches); at the end the
  // finished tile is staged over all of it: at most 4 bytes per channel and lane
  const size_t strip = (2 * kValThreads + 4) * sizeof(uint32_t) + (size_t)p.strip_pix * p.gv_go_stride + (items * 4 + 2) * sizeof(u32x2);
  return std::max(strip, (size_t)kValThreads * p.gv_cw * 4);
}

hipError_t launch_dcnv4_grad_value(int dtype, const DcnLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_t<F32>(p, stream);
    case F16::kCode: return launch_t<F16>(p, stream);
    case BF16::kCode: return launch_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
