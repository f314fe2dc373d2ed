// DCNv4 backward, gradient of the input (grad_value), without global atomics.
//
// The reference scatters 36*C fp32 atomicAdds per output pixel into memory
// (DCNv4_op/src/cuda/common.h:153-184 called from dcnv4_col2im_cuda.cuh:280-350).  On MI355X the
// memory-side atomic units retire about one dword per clock per channel, which caps that scheme
// two orders of magnitude below the HBM roofline, and LDS floating-point atomics are serialised
// per lane.  LDS *integer* atomics run at full rate, so this kernel turns the scatter around:
//
//   * a workgroup OWNS a tile_h x tile_w tile of the input image for a chunk of groups, and is
//     the only writer of that part of grad_value: plain stores, no clearing pass, no cast pass;
//   * it visits every output pixel whose reference point lies within the reach the data needs
//     (GradState::reach_needed, capped by the planned `reach`), strip by strip, in two phases:
//       A  tap-parallel: one lane per (pixel, group, kernel tap) recomputes the sampling position
//          and, when a corner lands inside the tile, appends a hit record (four accumulator cells,
//          four weights, pixel) to a per-group list in LDS; the strip's grad_out is parked in LDS;
//       B  channel-parallel: a row of R lanes (2 for groups of up to 16 channels, 4 up to 32, 8 up to
//          64) takes one hit record, lane c owns the CPL consecutive channels from c * CPL and adds
//          its four corner contributions with 64-bit integer LDS atomics on fixed-point values.  Few
//          lanes per record keep the per-record work (reading and unpacking it) small next to the
//          adds.  The 64 / R rows of a wave are dealt evenly to the groups of the chunk, and the n-th
//          row of a group starts its walk over the lane's channels at the n-th, so the rows of one
//          ds_add_u64 instruction spread evenly over the banks (32 banks of 4 bytes; a 64-bit operation is
//          served 16 lanes per pass): four passes, the least 64 lanes of 8 bytes can take;
//   * fixed point: contributions are normalised by the global maxima of |grad_out| and
//     |modulation| (GradState, produced by the grad_offset_mask kernel that runs first) and carry
//     `fix_bits` fractional bits (up to 50; each product is exact in double precision and rounded
//     once), i.e. an absolute resolution of 2^-fix_bits of the largest possible contribution - finer
//     than fp32 accumulation unless a sum is > 2^25 times smaller than that.
//     Integer sums make the result bit-reproducible, independent of scheduling;
//   * corners farther than `reach` from their output pixel's tile, and the case of non-finite
//     statistics, are left to the fallback scatter kernel (dcnv4_kernels.hip, kBwdFallback),
//     which runs afterwards and does nothing in the common case.
#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

constexpr int kValThreads = 1024;
constexpr int kWaves = kValThreads / kWave;
constexpr int kTrashPad = 64;
constexpr int kMaxChunkGroups = 4;      // rows of a wave <-> groups of the chunk
constexpr int kMetaPosBits = 6;         // row + 1 and column + 1 of a record's first corner inside the tile: 0..32

// A hit record's second word: (row + 1) | (column + 1) << 6 of the first corner relative to the tile (-1 when the
// corner block starts one row or column before it), the corners inside the tile (4 bits) << 12, and the strip-local
// output pixel << 16.
typedef uint32_t HitMeta;

// lanes that apply one hit record, and channels per lane (1, 2, 4 or 8; odd counts round up)
__host__ __device__ inline int lanes_per_record(int D) { return D <= 16 ? 2 : (D <= 32 ? 4 : 8); }
__host__ __device__ inline int channels_per_lane(int D) {
  const int r = lanes_per_record(D), c = (D + r - 1) / r;
  return c <= 2 ? c : (c <= 4 ? 4 : 8);
}

// Accumulator words per cell, channels in their natural order.  PACK (16-bit tensors): one 64-bit word
// holds two 32-bit fixed-point sums, channels 2w (low half) and 2w + 1 (high half).  Otherwise one word
// per channel.
__host__ __device__ inline int acc_words_per_group(int D, bool pack) { return pack ? (D + 1) / 2 : D; }
__host__ __device__ inline int acc_words_per_cell(int ng_chunk, int D, bool pack) {
  return ng_chunk * acc_words_per_group(D, pack);
}

// FAST (0 = off, else log2 of the tile width): groups of 16 channels in 32-wide tiles with one group per workgroup, or
// 16- and 8-wide tiles with four.  The four corners of a hit record then lie at compile-time distances from the
// first one, so their addresses are immediates of one base register; a corner outside
// the tile carries weight zero and its add lands, harmlessly, on whatever the LDS holds there - another cell, or the
// hit weights in front of the accumulators or the parked grad_out behind them (adding the integer 0 changes nothing).
template <typename Tag, int KP, int R, int CPL, bool PACK, int FAST>
__global__ void __launch_bounds__(kValThreads) dcnv4_grad_value_kernel(const DcnLaunch p) {
  extern __shared__ unsigned long long lds64[];
  // Packed sums, one group per workgroup: a cell is 64 bytes, half of what the LDS takes in one pass of eight
  // records (16 lanes x 8 bytes over 32 banks), so two records on the same unit collide when their cells' columns
  // have the same parity.  The hit list is therefore kept in two parts - even first columns from the front, odd
  // ones from the back - and the rows of a wave draw from them alternately: every pass then holds four records of
  // each parity on four different units, for all four corners (the other corners shift every record alike).
  constexpr bool kTwoEnded = PACK && FAST == 5;
  const int Kp = p.Kp, D = p.D, C = p.G * p.D;
  const int n_chunks = (p.G + p.ng_chunk - 1) / p.ng_chunk;
  const int nty = (p.H + p.tile_h - 1) >> p.tile_h_log2, ntx = (p.W + p.tile_w - 1) >> p.tile_w_log2;
  uint32_t id = xcd_contiguous_block(blockIdx.x, gridDim.x);
  const int chunk = id % n_chunks; id /= n_chunks;
  const int tx = id % ntx; id /= ntx;
  const int ty = id % nty;
  const int b = id / nty;
  const int g0 = chunk * p.ng_chunk, ng = min(p.ng_chunk, p.G - g0);
  const int ch_stride = p.ng_chunk * D;                 // channels of the chunk
  const int group_words = acc_words_per_group(D, PACK);                 // accumulator words of a group within a cell
  const int acc_stride = p.ng_chunk * group_words;                      // ... of a cell
  const int ty0 = ty << p.tile_h_log2, tx0 = tx << p.tile_w_log2;
  const int th = min(p.tile_h, p.H - ty0), tw = min(p.tile_w, p.W - tx0);
  const int n_cells = p.tile_h * p.tile_w;
  // the slots past the tile absorb the zero-valued adds of corners outside the tile, and of lanes
  // whose channel index runs past D (group widths that are not multiples of 16)
  const int n_acc = ((n_cells + 1) * acc_stride + kTrashPad + 1) & ~1;     // even: keeps the lists 16-byte aligned
  const int list_cap = p.strip_pix * Kp;                // hit records per group list
  // FAST keeps the hit weights in front of the accumulators: they are the landing zone of corners above the tile
  unsigned long long *acc = FAST != 0 ? lds64 + 2 * (size_t)p.ng_chunk * list_cap : lds64;
  f32x4 *hit_w = reinterpret_cast<f32x4 *>(FAST != 0 ? lds64 : lds64 + n_acc);         // [ng_chunk][list_cap]
  float *s_go = reinterpret_cast<float *>(FAST != 0 ? reinterpret_cast<f32x4 *>(acc + n_acc) : hit_w + p.ng_chunk * list_cap);   // [strip_pix][ch_stride], 16-byte aligned
  HitMeta *hit_meta = reinterpret_cast<HitMeta *>(s_go + p.strip_pix * ch_stride);  // [ng_chunk][list_cap]
  uint32_t *s_count = reinterpret_cast<uint32_t *>(hit_meta + p.ng_chunk * list_cap);  // two sets of [kMaxChunkGroups]

  const uint32_t gmax = p.state->go_max_bits, mmax = p.state->mask_max_bits;
  const bool finite = gmax < 0x7f800000u && mmax < 0x7f800000u;
  // 2^e > max >= 2^(e-1); zero maxima mean an all-zero gradient and any exponent works
  const int e_go = (int)(gmax >> 23) - 126, e_m = (int)(mmax >> 23) - 126;

  for (int i = threadIdx.x; i < n_acc; i += kValThreads) acc[i] = 0ull;

  // output pixels this tile visits: reference point within `reach` of the tile (near_box)
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
  const int cy0 = half_h - p.ph, cx0 = half_w - p.pw, Ho = p.Q / p.Wo;
  // every in-image corner that carries weight lies within reach_needed of its reference point, so a smaller window than the
  // planned cap loses nothing; beyond the cap the fallback kernel takes over
  const int reach = min(p.reach, (int)p.state->reach_needed);
  const int ho_lo = max(0, ceil_div_signed(ty0 - reach - cy0, p.sh));
  const int ho_hi = min(Ho, ceil_div_signed(ty0 + p.tile_h + reach - cy0, p.sh));
  const int wo_lo = max(0, ceil_div_signed(tx0 - reach - cx0, p.sw));
  const int wo_hi = min(p.Wo, ceil_div_signed(tx0 + p.tile_w + reach - cx0, p.sw));
  const int nwx = wo_hi - wo_lo;
  const int lane = threadIdx.x & (kWave - 1), c = lane & (R - 1);
  static_assert(kWave / R >= kMaxChunkGroups, "a wave holds at least one row per group of a full chunk");
  static_assert(!PACK || CPL % 2 == 0, "packed sums pair the channels of one lane");
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int row_in_wave = lane / R;
  const float x_sub = mul_rn((float)half_w, p.offset_scale), y_sub = mul_rn((float)half_h, p.offset_scale);
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  const elem_t *om_g = reinterpret_cast<const elem_t *>(p.offset_mask);
  const elem_t *go_g = reinterpret_cast<const elem_t *>(p.grad_out);
  auto load_f = [](const elem_t *ptr) { float f[1]; Pack<Tag, 1>::decode(*ptr, f); return f[0]; };

  if (finite && nwx > 0 && ho_hi > ho_lo && (gmax | mmax) != 0) {
    const int rows_per_strip = max(1, p.strip_pix / nwx);
    const int npx_full = rows_per_strip * nwx;
    const float inv_nwx = 1.f / (float)nwx;
    // this image's tensors, addressed with 32-bit element offsets (the entry point checks they fit)
    const elem_t *om_img = om_g + (size_t)b * p.Q * p.P_pad;
    const elem_t *go_img = go_g + (size_t)b * p.Q * C;
    constexpr int kStageRounds = 2;     // staging rounds whose grad_out is prefetched (a round: 16 waves x ppw pixels)

    // Phase A work item of a (wave slot, lane): group, strip-local pixel, tap.  The decode depends only
    // on the strip geometry, not on the strip, so the first round's item is decoded once per lane.
    struct Item {
      bool in_range;
      int gl, px, r, t, ti, tj;
      uint32_t om_off;       // element offset of this (pixel, group)'s offset_mask slice for the first strip
      float x_base;
    };
    const int per_group_full = npx_full * Kp, waves_per_group = (per_group_full + kWave - 1) / kWave;
    const int n_wk = ng * waves_per_group;
    auto item_of = [&](int wk) {
      Item it;
      it.gl = wk / waves_per_group;                                          // scalar: same for the wave
      const int j = (wk - it.gl * waves_per_group) * kWave + lane;
      it.in_range = wk < n_wk && j < per_group_full;
      it.px = KP > 0 ? j / KP : j / Kp;
      it.t = j - it.px * Kp;
      if (!it.in_range) { it.gl = 0; it.px = 0; it.t = 0; }
      it.r = (int)(((float)it.px + 0.5f) * inv_nwx);                         // exact: px < 1024
      const int wo = wo_lo + (it.px - it.r * nwx);
      if constexpr (KP > 0) {
        tap_ij_3x3(KP, it.t, it.ti, it.tj);
      } else {      // x index outer, y index inner, centre skipped when remove_center
        int tt = it.t;
        if (p.remove_center && tt >= (p.kw / 2) * p.kh + p.kh / 2) ++tt;
        it.ti = tt / p.kh; it.tj = tt - it.ti * p.kh;
      }
      it.om_off = __umul24((uint32_t)((ho_lo + it.r) * p.Wo + wo), (uint32_t)p.P_pad) + (uint32_t)((g0 + it.gl) * 3 * Kp);
      it.x_base = sub_rn((float)(cx0 + wo * p.sw), x_sub);
      return it;
    };
    constexpr int kItemRounds = 2;      // phase A rounds whose items are decoded once and whose taps are prefetched
    Item my_item[kItemRounds];
#pragma unroll
    for (int v = 0; v < kItemRounds; ++v) my_item[v] = item_of(wave + v * kWaves);
    // staging: a lane parks one 16-byte vector of grad_out (kVec channels of a pixel), a wave ppw whole pixels per
    // round; the first kStageRounds rounds are prefetched.  Group widths that are not whole vectors, and chunks
    // whose vector count is not a power of two, park element by element without prefetch.
    constexpr int kVec = 16 / Tag::kBytes;
    typedef typename Pack<Tag, kVec>::raw_t vec_t;
    const int px_lanes = ch_stride / kVec;
    const bool vec_park = D % kVec == 0 && px_lanes <= kWave && (px_lanes & (px_lanes - 1)) == 0;
    const int px_lanes_log2 = vec_park ? 31 - __builtin_clz(px_lanes) : 0;
    const int ppw = kWave >> px_lanes_log2;
    const int lane_px = lane >> px_lanes_log2, lane_ch = (lane & (px_lanes - 1)) * kVec;
    uint32_t go_off[kStageRounds];
#pragma unroll
    for (int u = 0; u < kStageRounds; ++u) {
      const int px = (wave + u * kWaves) * ppw + lane_px, r = px / nwx;
      go_off[u] = (uint32_t)(((ho_lo + r) * p.Wo + wo_lo + (px - r * nwx)) * C + g0 * D + lane_ch);
    }
    const uint32_t om_strip = (uint32_t)(rows_per_strip * p.Wo) * (uint32_t)p.P_pad;   // offset step per strip
    const uint32_t go_strip = (uint32_t)(rows_per_strip * p.Wo * C);

    struct Prefetch {
      elem_t ox[kItemRounds], oy[kItemRounds], m[kItemRounds];      // phase A, first rounds: this lane's tap
      vec_t go[kStageRounds];           // staging: this lane's vector of its pixel in the first rounds
    };
    // loads of the next strip, issued before the current strip's phase B so their latency hides there
    auto prefetch = [&](int s_idx, int npx) {
      Prefetch pf;
#pragma unroll
      for (int v = 0; v < kItemRounds; ++v) {
        pf.ox[v] = pf.oy[v] = pf.m[v] = elem_t(0);
        if (my_item[v].in_range && my_item[v].px < npx) {
          const elem_t *om = om_img + (my_item[v].om_off + (uint32_t)s_idx * om_strip);
          pf.ox[v] = om[2 * my_item[v].t]; pf.oy[v] = om[2 * my_item[v].t + 1]; pf.m[v] = om[2 * Kp + my_item[v].t];
        }
      }
#pragma unroll
      for (int u = 0; u < kStageRounds; ++u) {
        pf.go[u] = vec_t{};
        if (vec_park && (wave + u * kWaves) * ppw + lane_px < npx && lane_ch < ng * D)
          pf.go[u] = *reinterpret_cast<const vec_t *>(go_img + (go_off[u] + (uint32_t)s_idx * go_strip));
      }
      return pf;
    };
    auto to_f = [](elem_t raw) { float f[1]; Pack<Tag, 1>::decode(raw, f); return f[0]; };

    int hs = ho_lo;
    int npx = min(rows_per_strip, ho_hi - hs) * nwx;
    Prefetch pf = prefetch(0, npx);
    if (threadIdx.x < 2 * kMaxChunkGroups) s_count[threadIdx.x] = 0u;

    for (int s_idx = 0; hs < ho_hi; ++s_idx) {
      uint32_t *count = s_count + (s_idx & 1) * kMaxChunkGroups;
      __syncthreads();      // previous strip's phase B is done (first time: acc and counters are clear)

      // ---- park the strip's grad_out (this chunk's channels), normalised to [-1, 1]
      if (vec_park) {
        for (int base = wave * ppw, u = 0; base < npx; base += kWaves * ppw, ++u) {
          const int px = base + lane_px;
          if (px >= npx) continue;
          float f[kVec];
#pragma unroll
          for (int i = 0; i < kVec; ++i) f[i] = 0.f;
          if (lane_ch < ng * D) {
            vec_t raw = pf.go[0];
            if (u < kStageRounds) {
#pragma unroll
              for (int v = 1; v < kStageRounds; ++v) raw = u == v ? pf.go[v] : raw;
            } else {
              const int r = px / nwx;
              raw = *reinterpret_cast<const vec_t *>(go_img + ((uint32_t)(((hs + r) * p.Wo + wo_lo + (px - r * nwx)) * C) + g0 * D + lane_ch));
            }
            Pack<Tag, kVec>::decode(raw, f);
          }
          f32x4 *dst = reinterpret_cast<f32x4 *>(s_go + px * ch_stride + lane_ch);
#pragma unroll
          for (int i = 0; i < kVec / 4; ++i)
            dst[i] = f32x4{ldexpf(f[4 * i], -e_go), ldexpf(f[4 * i + 1], -e_go), ldexpf(f[4 * i + 2], -e_go), ldexpf(f[4 * i + 3], -e_go)};
        }
      } else {
        for (int px = wave; px < npx; px += kWaves) {
          const int r = px / nwx;
          const elem_t *src = go_img + ((uint32_t)(((hs + r) * p.Wo + wo_lo + (px - r * nwx)) * C) + g0 * D);
          for (int ch = lane; ch < ch_stride; ch += kWave) s_go[px * ch_stride + ch] = ch < ng * D ? ldexpf(load_f(src + ch), -e_go) : 0.f;
        }
      }

      // ---- phase A: one lane per (group, pixel, tap); a wave never mixes groups
      for (int wk = wave, round = 0; wk < n_wk; wk += kWaves, ++round) {
        Item it;
        elem_t pf_ox = elem_t(0), pf_oy = elem_t(0), pf_m = elem_t(0);
        if (round < kItemRounds) {
          it = my_item[0]; pf_ox = pf.ox[0]; pf_oy = pf.oy[0]; pf_m = pf.m[0];
#pragma unroll
          for (int v = 1; v < kItemRounds; ++v)
            if (round == v) { it = my_item[v]; pf_ox = pf.ox[v]; pf_oy = pf.oy[v]; pf_m = pf.m[v]; }
        } else {
          it = item_of(wk);
        }
        const bool valid_item = it.in_range && it.px < npx;
        bool hit = false;
        f32x4 w = {0.f, 0.f, 0.f, 0.f};
        HitMeta meta = 0u;
        if (valid_item) {
          const elem_t *om = om_img + (it.om_off + (uint32_t)s_idx * om_strip);
          const float off_x = round < kItemRounds ? to_f(pf_ox) : load_f(om + 2 * it.t);
          const float off_y = round < kItemRounds ? to_f(pf_oy) : load_f(om + 2 * it.t + 1);
          const float y_base = sub_rn((float)(cy0 + (hs + it.r) * p.sh), y_sub);
          const float x = add_rn(it.x_base, mul_rn(add_rn((float)(it.ti * p.dw), off_x), p.offset_scale));
          const float y = add_rn(y_base, mul_rn(add_rn((float)(it.tj * p.dh), off_y), p.offset_scale));
          const Tap tp = make_tap(y, x, p.H, p.W, 0u, 0u);
          const int ly = tp.y0 - ty0, lx = tp.x0 - tx0;
          const bool r0 = ly >= 0 && ly < th, r1 = ly + 1 >= 0 && ly + 1 < th;
          const bool c0 = lx >= 0 && lx < tw, c1 = lx + 1 >= 0 && lx + 1 < tw;
          const uint32_t valid = tp.valid & ((uint32_t)(r0 && c0) | ((uint32_t)(r0 && c1) << 1) |
                                             ((uint32_t)(r1 && c0) << 2) | ((uint32_t)(r1 && c1) << 3));
          hit = valid != 0;
          if (hit) {
            float m = round < kItemRounds ? to_f(pf_m) : load_f(om + 2 * Kp + it.t);
            if (p.softmax) {          // rare: normalise over this group's taps
              float mx = load_f(om + 2 * Kp), sum = 0.f;
              for (int k = 1; k < Kp; ++k) mx = fmaxf(mx, load_f(om + 2 * Kp + k));
              for (int k = 0; k < Kp; ++k) sum += __expf(load_f(om + 2 * Kp + k) - mx);
              m = __expf(m - mx) / sum;
            }
            const float ms = ldexpf(m, p.fix_bits - e_m);
#pragma unroll
            for (int cn = 0; cn < 4; ++cn) w[cn] = (valid & (1u << cn)) ? ms * tp.w[cn] : 0.f;
            meta = (uint32_t)(ly + 1) | ((uint32_t)(lx + 1) << kMetaPosBits) | (valid << (2 * kMetaPosBits)) | ((uint32_t)it.px << 16);
          }
        }
        if constexpr (kTwoEnded) {
          // records whose first cell has an even column grow the list from its front, the others from its back
          const bool odd = (meta >> kMetaPosBits) & 1u ? false : true;      // the field holds column + 1
          const uint64_t mask_e = __builtin_amdgcn_ballot_w64(hit && !odd), mask_o = __builtin_amdgcn_ballot_w64(hit && odd);
          if ((mask_e | mask_o) != 0) {
            uint32_t base = 0;
            if (lane < 2) base = atomicAdd(&count[lane], (uint32_t)__builtin_popcountll(lane == 0 ? mask_e : mask_o));
            const uint32_t base_e = (uint32_t)__builtin_amdgcn_readlane((int)base, 0), base_o = (uint32_t)__builtin_amdgcn_readlane((int)base, 1);
            if (hit) {
              const uint64_t mine = odd ? mask_o : mask_e;
              const uint32_t rank = __builtin_amdgcn_mbcnt_hi((uint32_t)(mine >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mine, 0u));
              const uint32_t slot = odd ? (uint32_t)list_cap - 1u - (base_o + rank) : base_e + rank;
              hit_w[slot] = w;
              hit_meta[slot] = meta;
            }
          }
          continue;
        }
      // append the wave's hits to its group's list: one LDS counter bump per wave
        const uint64_t mask = __builtin_amdgcn_ballot_w64(hit);
        if (mask != 0) {
          uint32_t base = 0;
          if (lane == 0) base = atomicAdd(&count[it.gl], (uint32_t)__builtin_popcountll(mask));
          base = __builtin_amdgcn_readfirstlane(base);
          if (hit) {
            const uint32_t slot = it.gl * list_cap + base +
                                  __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
            hit_w[slot] = w;
            hit_meta[slot] = meta;
          }
        }
      }
      __syncthreads();

      // next strip's loads fly while this strip's hits are applied; the other counter set is idle
      const int hs_next = hs + rows_per_strip;
      const int npx_next = hs_next < ho_hi ? min(rows_per_strip, ho_hi - hs_next) * nwx : 0;
      if (npx_next > 0) pf = prefetch(s_idx + 1, npx_next);
      if (threadIdx.x < kMaxChunkGroups) s_count[((s_idx + 1) & 1) * kMaxChunkGroups + threadIdx.x] = 0u;

      // ---- phase B: a row of R lanes applies one hit record; lane c owns channels c * CPL .. c * CPL + CPL - 1.
      // The rows of a wave are split evenly over the chunk's groups; row n of a group visits its lane's
      // channels (channel pairs when packed) starting from the n-th, so the rows that work for one group
      // touch different words in every instruction.
      constexpr int kUnits = PACK ? CPL / 2 : CPL;                       // accumulator words per lane
      const int rows_per_group = (kWave / R) / p.ng_chunk;
      int my_group = row_in_wave / rows_per_group, my_slot = row_in_wave - my_group * rows_per_group;
      int first_unit = my_slot;
      if (PACK && R == 2 && p.ng_chunk == 4 && group_words == 8) {
        // A cell of packed sums is 32 words, 8 per group, and the LDS serves a wave's 64-bit atomics 16 lanes (8 rows)
        // per pass over 16 word slots: deal each run of 8 rows as 2 groups x 4 starting units (16 rows: 4 groups), so
        // that the rows of a pass touch different slots whatever their cells are (groups in consecutive rows would
        // put rows of groups g and g + 2 on the same slots).
        const int half = row_in_wave >> 4, i = row_in_wave & 15;
        my_group = i >> 2;
        first_unit = i & 3;
        my_slot = half * 4 + first_unit;
      }
      const bool group_live = my_group < ng;
      const uint32_t n_mine = group_live ? count[my_group] : 0u;
      uint32_t n_max = count[0];
      for (int g = 1; g < ng; ++g) n_max = max(n_max, count[g]);
      const int lane_group = group_live ? my_group : 0;                  // idle rows only ever add zeros to the trash slots
      unsigned long long *acc_lane = acc + lane_group * group_words + c * kUnits;
      const float *go_lane = s_go + lane_group * D + c * CPL;
      int unit_of[kUnits];                                               // this row's visiting order
#pragma unroll
      for (int u = 0; u < kUnits; ++u) unit_of[u] = (u + first_unit) & (kUnits - 1);
      if constexpr (FAST != 0) {
        static_assert(R == 2 && CPL == 8, "groups of 16 channels");
        constexpr int kGroups = FAST == 5 ? 1 : 4, kTileW = 1 << FAST;            // groups per workgroup, cells per tile row
        constexpr int kGroupWords = PACK ? 8 : 16, kCellWords = kGroups * kGroupWords;
        constexpr int kCorner[4] = {0, kCellWords, kTileW * kCellWords, (kTileW + 1) * kCellWords};
        unsigned long long *acc_row = acc + lane_group * kGroupWords + c * kUnits;
        const float *go_row = s_go + lane_group * 16 + c * CPL;
        const f32x4 *w_list = hit_w + lane_group * list_cap;
        const HitMeta *meta_list = hit_meta + lane_group * list_cap;
        // two-ended list: rows 2j and 2j + 1 of a wave take the j-th even and the j-th odd record of the pass
        const uint32_t n_two = kTwoEnded ? ((my_slot & 1) ? count[1] : count[0]) : 0u;
        const uint32_t bound = kTwoEnded ? max(count[0], count[1]) : n_max;
        const uint32_t lane_step = kTwoEnded ? (uint32_t)(my_slot >> 1) : (uint32_t)my_slot;
        const uint32_t wave_rows = kTwoEnded ? (uint32_t)(kWave / R / 2) : (uint32_t)rows_per_group;
        if constexpr (kTwoEnded) {
#pragma unroll
          for (int u = 0; u < kUnits; ++u) unit_of[u] = (u + (my_slot >> 1)) & (kUnits - 1);
        }
        for (uint32_t i0 = wave * wave_rows; i0 < bound; i0 += kWaves * wave_rows) {
          uint32_t i = i0 + lane_step;
          if (i >= (kTwoEnded ? n_two : n_mine)) continue;
          if (kTwoEnded && (my_slot & 1)) i = (uint32_t)list_cap - 1u - i;
          const f32x4 w = w_list[i];
          const HitMeta meta = meta_list[i];
          const float *go_px = go_row + (meta >> 16) * (kGroups * 16);
          const int first_cell = ((int)(meta & 63u) - 1) * kTileW + (int)((meta >> kMetaPosBits) & 63u) - 1;
          unsigned long long *base = acc_row + first_cell * kCellWords;
          const float wv[4] = {w.x, w.y, w.z, w.w};
          if constexpr (PACK) {
            f32x2 g[kUnits];
#pragma unroll
            for (int u = 0; u < kUnits; ++u) g[u] = *reinterpret_cast<const f32x2 *>(go_px + 2 * unit_of[u]);
#pragma unroll
            for (int u = 0; u < kUnits; ++u) {
              const float g_lo = g[u].x, g_hi = g[u].y;
              unsigned long long *dst = base + unit_of[u];
#pragma unroll
              for (int cn = 0; cn < 4; ++cn)
                __hip_atomic_fetch_add(dst + kCorner[cn], pack_fixed32(to_fixed32(g_lo, wv[cn]), to_fixed32(g_hi, wv[cn])),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          } else {
            const double wd[4] = {(double)wv[0], (double)wv[1], (double)wv[2], (double)wv[3]};
            float g[kUnits];
#pragma unroll
            for (int u = 0; u < kUnits; ++u) g[u] = go_px[unit_of[u]];
#pragma unroll
            for (int u = 0; u < kUnits; ++u) {
              const double gd = (double)g[u];
              unsigned long long *dst = base + unit_of[u];
#pragma unroll
              for (int cn = 0; cn < 4; ++cn)
                __hip_atomic_fetch_add(dst + kCorner[cn], fixed_product(gd, wd[cn]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          }
        }
      } else {
        for (uint32_t i0 = wave * rows_per_group; i0 < n_max; i0 += kWaves * rows_per_group) {
          const uint32_t i = i0 + my_slot;
          if (i >= n_mine) continue;        // rows past the end of their group's list sit this pass out
          const f32x4 w = hit_w[lane_group * list_cap + i];
          const HitMeta meta = hit_meta[lane_group * list_cap + i];
          const float *go_px = go_lane + (meta >> 16) * ch_stride;
          const int first_cell = ((int)(meta & 63u) - 1) * p.tile_w + (int)((meta >> kMetaPosBits) & 63u) - 1;
          uint32_t cells[4];
  #pragma unroll
          for (int cn = 0; cn < 4; ++cn)      // corners outside the tile carry weight 0: send them to the trash cell
            cells[cn] = (meta & (1u << (2 * kMetaPosBits + cn))) ? (uint32_t)(first_cell + (cn >> 1) * p.tile_w + (cn & 1)) : (uint32_t)n_cells;
          const float wv[4] = {w.x, w.y, w.z, w.w};
          unsigned long long *dst[4];
  #pragma unroll
          for (int cn = 0; cn < 4; ++cn) dst[cn] = acc_lane + __umul24(cells[cn], (uint32_t)acc_stride);
          if constexpr (PACK) {
            // two channels per atomic: sum = hi * 2^32 + lo with both halves signed, so the low term is
            // sign-extended into the high word before the add
  #pragma unroll
            for (int u = 0; u < kUnits; ++u) {
              const int ch = 2 * unit_of[u];
              const float g_lo = (c * CPL + ch < D) ? go_px[ch] : 0.f;
              const float g_hi = (c * CPL + ch + 1 < D) ? go_px[ch + 1] : 0.f;
  #pragma unroll
              for (int cn = 0; cn < 4; ++cn) {
                __hip_atomic_fetch_add(dst[cn] + unit_of[u], pack_fixed32(to_fixed32(g_lo, wv[cn]), to_fixed32(g_hi, wv[cn])),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
              }
            }
          } else {
            const double wd[4] = {(double)wv[0], (double)wv[1], (double)wv[2], (double)wv[3]};
  #pragma unroll
            for (int u = 0; u < kUnits; ++u) {
              const int ch = unit_of[u];
              const double gd = (c * CPL + ch < D) ? (double)go_px[ch] : 0.0;
  #pragma unroll
              for (int cn = 0; cn < 4; ++cn)
                __hip_atomic_fetch_add(dst[cn] + ch, fixed_product(gd, wd[cn]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          }
        }
      }
      hs = hs_next;
      npx = npx_next;
    }
  }
  __syncthreads();

  // the tile is complete: fixed point -> tensor dtype, plain stores (zeros when not finite: the
  // fallback kernel then adds every corner)
  const int e_out = e_go + e_m - p.fix_bits;
  const int n_ch = ng * D;
  // A lane converts four consecutive channels of a cell and stores them as one vector, a wave whole cells (64 / lanes
  // per cell of them per step).  Group widths that are not multiples of four, and chunks whose lane count per cell is
  // not a power of two, go element by element, one cell per wave and step.
  const int cell_lanes = n_ch >> 2;
  if ((D & 3) == 0 && cell_lanes <= kWave && (cell_lanes & (cell_lanes - 1)) == 0) {
    const int cl_log2 = 31 - __builtin_clz(cell_lanes);
    const int sub = lane >> cl_log2, ch = (lane & (cell_lanes - 1)) * 4;
    const int g = ch / D, cg = ch - g * D;
    const int word = PACK ? g * group_words + (cg >> 1) : ch;
    typedef typename Pack<Tag, 4>::raw_t out_t;
    for (int cell0 = wave << (6 - cl_log2); cell0 < n_cells; cell0 += kValThreads >> cl_log2) {
      const int cell = cell0 + sub;
      const int ly = cell >> p.tile_w_log2, lx = cell & (p.tile_w - 1);
      if (ly >= th || lx >= tw) continue;
      const u64x2 *src = reinterpret_cast<const u64x2 *>(acc + cell * acc_stride + word);
      float f[4];
      if constexpr (PACK) {
        const u64x2 a = src[0];
        const unsigned long long a0 = a.x, a1 = a.y;
        f[0] = ldexpf((float)packed_field(a0, 0), e_out); f[1] = ldexpf((float)packed_field(a0, 1), e_out);
        f[2] = ldexpf((float)packed_field(a1, 0), e_out); f[3] = ldexpf((float)packed_field(a1, 1), e_out);
      } else {
        const u64x2 a = src[0], b2 = src[1];
        const unsigned long long w4[4] = {a.x, a.y, b2.x, b2.y};
#pragma unroll
        for (int i = 0; i < 4; ++i)
          f[i] = (float)ldexp((double)(int)(w4[i] >> 32) * 4294967296.0 + (double)(uint32_t)w4[i], e_out);
      }
      out_t *dst = reinterpret_cast<out_t *>(reinterpret_cast<elem_t *>(p.grad_value) +
                                             ((((size_t)b * p.H + ty0 + ly) * p.W + tx0 + lx) * C + g0 * D + ch));
      *dst = Pack<Tag, 4>::encode(f);
    }
  } else {
    for (int cell = wave; cell < th * tw; cell += kWaves) {
      const int ly = cell / tw, lx = cell - ly * tw;
      const unsigned long long *src = acc + ((ly << p.tile_w_log2) + lx) * acc_stride;
      elem_t *dst = reinterpret_cast<elem_t *>(p.grad_value) + (((size_t)b * p.H + ty0 + ly) * p.W + tx0 + lx) * C + g0 * D;
      for (int ch = lane; ch < n_ch; ch += kWave) {
        float f[1];
        if constexpr (PACK) {
          const int g = ch / D, cg = ch - g * D;
          f[0] = ldexpf((float)packed_field(src[g * group_words + (cg >> 1)], cg & 1), e_out);
        } else {
          const unsigned long long a = src[ch];
          f[0] = (float)ldexp((double)(int)(a >> 32) * 4294967296.0 + (double)(uint32_t)a, e_out);
        }
        dst[ch] = Pack<Tag, 1>::encode(f);
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
    // the limit is a per-function attribute: raise it once per process and kernel
    static bool raised = false;
    if (!raised) {
      if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLdsPerWorkgroup))
        return e;
      raised = true;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return hipGetLastError();
  };
  const int r = lanes_per_record(p.D), cpl = channels_per_lane(p.D);
  constexpr bool kCanPack = Tag::kBytes == 2;
  // the immediate-offset variants: their stray zero adds reach tile_w + 1 cells before and after the accumulators,
  // which must stay inside the hit weights in front and the trash slots plus the parked grad_out behind
  int fast = 0;
  if (p.D == 16 && p.tile_w_log2 >= 3 && p.tile_w_log2 <= 5 && p.ng_chunk == (p.tile_w_log2 == 5 ? 1 : 4)) {
    const size_t cell_bytes = (size_t)acc_words_per_cell(p.ng_chunk, 16, p.pack32 != 0) * sizeof(unsigned long long);
    const size_t guard = (size_t)(p.tile_w + 1) * cell_bytes;
    if ((size_t)p.ng_chunk * p.strip_pix * p.Kp * sizeof(f32x4) >= guard &&
        cell_bytes + (size_t)p.strip_pix * p.ng_chunk * 16 * sizeof(float) >= guard)
      fast = p.tile_w_log2;
  }
#define GV_CASE(KPV)                                                                        \
  do {                                                                                      \
    if constexpr (kCanPack) {                                                               \
      if (p.pack32 && fast == 5) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, true, 5>);  \
      if (p.pack32 && fast == 4) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, true, 4>);  \
      if (p.pack32 && fast == 3) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, true, 3>);  \
      if (p.pack32 && r == 2 && cpl == 8) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, true, 0>);   \
      if (p.pack32 && r == 4) return go(dcnv4_grad_value_kernel<Tag, KPV, 4, 8, true, 0>);     \
      if (p.pack32 && r == 8) return go(dcnv4_grad_value_kernel<Tag, KPV, 8, 8, true, 0>);     \
    }                                                                                       \
    if (!p.pack32 && fast == 5) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, false, 5>); \
    if (!p.pack32 && fast == 4) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, false, 4>); \
    if (!p.pack32 && fast == 3) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, false, 3>); \
    if (r == 4) return go(dcnv4_grad_value_kernel<Tag, KPV, 4, 8, false, 0>);                  \
    if (r == 8) return go(dcnv4_grad_value_kernel<Tag, KPV, 8, 8, false, 0>);                  \
    if (cpl == 1) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 1, false, 0>);                \
    if (cpl == 2) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 2, false, 0>);                \
    if (cpl == 4) return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 4, false, 0>);                \
    return go(dcnv4_grad_value_kernel<Tag, KPV, 2, 8, false, 0>);                              \
  } while (0)
  if (k3 && !p.remove_center) GV_CASE(9);
  if (k3 && p.remove_center) GV_CASE(8);
  GV_CASE(0);
#undef GV_CASE
}

}  // namespace

size_t dcnv4_grad_value_lds_bytes(const DcnLaunch &p) {
  const size_t ch_stride = (size_t)p.ng_chunk * p.D, list = (size_t)p.ng_chunk * p.strip_pix * p.Kp;
  const size_t acc_stride = acc_words_per_cell(p.ng_chunk, p.D, p.pack32 != 0);
  return ((((size_t)(p.tile_h * p.tile_w + 1) * acc_stride + kTrashPad + 1) & ~size_t(1)) * sizeof(unsigned long long)) +  // accumulators
         list * sizeof(f32x4) + (size_t)p.strip_pix * ch_stride * sizeof(float) +                      // hit weights, grad_out
         list * sizeof(HitMeta) + 2 * kMaxChunkGroups * sizeof(uint32_t);                              // hit cells, two counter sets
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
