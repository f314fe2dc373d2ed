// Device code of the tiled grad_value kernel (dcnv4_grad_value.hip holds the kernel and its launcher; the body is also
// part of the two-role kernel in dcnv4_backward_dual.hip).
#pragma once
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
//   * a sampling point's 2x2 corner block is named by its first corner, the ANCHOR.  The anchors
//     whose block touches the tile form a grid one row and one column larger than the tile
//     (the first row and column lie just outside it).  A lane owns one (anchor, group) - or one
//     part of it when a group is wider than 16 channels - and keeps FOUR sets of fp32 sums in
//     registers for the whole kernel, one per corner of the block: a point's grad_out row is
//     read once and feeds all four corners.  The arithmetic is the reference's: every term
//     rounded to fp32, summed in fp32, the result rounded once to the tensor dtype;
//   * the workgroup visits every output pixel whose reference point lies within the reach the
//     data needs (GradState::reach_needed, written by the grad_offset_mask kernel that runs
//     first: what the sampling points within the reach cap need; a tile that points beyond the
//     cap land in reads its own, larger number from GradState::far_reach), in strips of
//     interleaved rows, so that every strip spreads its points evenly over the tile.  Per strip:
//       park   the strip's grad_out rows are copied to LDS;
//       A      one lane per (group, pixel, kernel tap) recomputes the sampling position and links
//              a 16-byte entry (m * hy, m * ly, lx, address of the pixel's parked grad_out | next)
//              into its anchor's list with ONE integer LDS exchange on the list head
//              (ds_wrxchg_rtn_b32): no counting, no prefix sum, no second pass;
//       B      every lane walks its own anchor's list: four corner weights from the entry,
//              sums[corner] += weight * grad_out row;
//   * at the end the four corner sums of every anchor meet in an fp32 image of the tile in LDS,
//     one corner at a time (within one corner every cell has exactly one writer), and the tile
//     goes to memory in 16-byte pieces.
// The exchanges only order the entries inside a list; sums depend on that order at the level
// of fp32 rounding, like the reference's atomics do.
#include <algorithm>

#include "common.hpp"
#include "launch.hpp"


namespace dcn {
namespace {


// grad_out is parked in LDS as fp32, also for 16-bit tensors: parked as fp16 and fed to mixed-precision FMAs it
// takes half the LDS, but the kernel measured 5-8 % slower (T stage 1 fp16 backward 0.169 -> 0.156 ms with fp32 rows).
template <typename Tag> struct ParkType { typedef float type; };

__device__ __forceinline__ int fdiv_small(int n, float inv) { return (int)(((float)n + 0.5f) * inv); }   // exact for n < 2^20


// CW: channels a lane accumulates for each of the four corners (8 or 16): the group width rounded up, or 16 with
// several lanes per (anchor, group).
// NT: lanes per workgroup (512: two workgroups share a CU and overlap each other's phases; 1024: one workgroup with
// the whole LDS); one (anchor, group) list per lane at most.
// (the body of the kernel as a function of the workgroup's number, so that a grid can also hold workgroups of another role)
template <typename Tag, int KP, int CW, int ROUNDS, int NT>
__device__ __forceinline__ void dcnv4_grad_value_body(const DcnLaunch &p, uint32_t bid, uint32_t nblocks) {
  constexpr int kValThreads = NT, kMaxAnchorSlots = NT;
  extern __shared__ __align__(16) uint32_t lds32[];
  typedef typename ParkType<Tag>::type park_t;
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int kParkBytes = sizeof(park_t);
  constexpr int kLaneBytes = CW * kParkBytes;                 // bytes of a parked row a lane reads per entry
  const int Kp = p.Kp, D = p.D, C = p.G * p.D;
  const int n_chunks = (p.G + p.ng_chunk - 1) / p.ng_chunk;
  const int eh = p.tile_h, ew = p.tile_w;                     // tile extent; cells are indexed with the power-of-two stride
  const int nty = (p.H + eh - 1) / eh, ntx = (p.W + ew - 1) / ew;
  uint32_t id = xcd_contiguous_block(bid, nblocks);
  const int chunk = id % n_chunks; id /= n_chunks;
  const int tx = id % ntx; id /= ntx;
  const int ty = id % nty;
  const int b = id / nty;
  const int g0 = chunk * p.ng_chunk, ng = min(p.ng_chunk, p.G - g0);
  const int ty0 = ty * eh, tx0 = tx * ew;
  const int th = min(eh, p.H - ty0), tw = min(ew, p.W - tx0);
  const int aw = ew + 1;                                      // anchors per row of the anchor grid
  const int lps_log2 = p.gv_lps_log2;
  const int Dp = CW << lps_log2;                              // parked channels per group
  const int go_stride = p.gv_go_stride;                       // bytes between parked pixels (an odd number of 16-byte units)
  const int tid = threadIdx.x;

  uint32_t *s_head = lds32;                                   // [2][kMaxAnchorSlots] first entry of every list; strips alternate between the halves
  char *s_go = reinterpret_cast<char *>(lds32 + 2 * kMaxAnchorSlots);
  u32x4 *s_entry = reinterpret_cast<u32x4 *>(s_go + (size_t)p.strip_pix * go_stride);
  // an entry's last word: parked grad_out address / 16 (14 bits) | index of the next entry << 14; the list ends at
  // the dummy entry behind the strip's items, which points at itself
  // Phase A's work items: for a 3x3 kernel a column of the kernel - three sampling points of one (pixel, group), with
  // consecutive offsets in memory - so that what they share (the item's decode, the pixel's address and reference
  // point) is done once; otherwise one sampling point.  Every item has kTaps entry slots.
  constexpr int kTaps = KP > 0 ? 3 : 1;
  const int upp = KP > 0 ? 3 : Kp;                            // items per (pixel, group)
  const uint32_t end_idx = (uint32_t)(p.strip_pix * upp * kTaps * p.ng_chunk);

  // output pixels this tile visits: reference point (centre tap at zero offset) within `reach` of the tile
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
  const int cy0 = half_h - p.ph, cx0 = half_w - p.pw, Ho = p.Q / p.Wo;
  // the reach that the bulk of the sampling points needs, or - for a tile that points beyond the reach cap land in -
  // how far away the output pixels of those points lie (GradState::far_reach): only such tiles pay for outliers
  const int reach = p.gv_whole ? (1 << 20)
                               : (int)min(max(p.state->reach_needed, p.state->far_reach[dcnv4_far_slot(b, ty, tx, nty, ntx, chunk, n_chunks)]), 1u << 20);
  const int ho_lo = max(0, ceil_div_signed(ty0 - reach - cy0, p.sh));
  const int ho_hi = min(Ho, ceil_div_signed(ty0 + eh + reach - cy0, p.sh));
  const int wo_lo_all = max(0, ceil_div_signed(tx0 - reach - cx0, p.sw));
  const int wo_hi_all = min(p.Wo, ceil_div_signed(tx0 + ew + reach - cx0, p.sw));
  const int n_rows = ho_hi - ho_lo;
  // a window wider than a strip holds is walked in blocks of columns
  const int cols_cap = max(1, min(wo_hi_all - wo_lo_all, p.strip_pix));

  // this lane's list: (anchor row, group of the chunk, anchor column), and its part of the group's channels
  const int n_lists = (eh + 1) * p.ng_chunk * aw;
  const int my_list = tid >> lps_log2, my_part = tid & ((1 << lps_log2) - 1);
  bool list_live;
  {
    const int row = fdiv_small(my_list, 1.f / (float)aw), ax = my_list - row * aw;      // row = anchor row * ng + group
    const int ay = fdiv_small(row, 1.f / (float)p.ng_chunk), gl = row - ay * p.ng_chunk;
    list_live = my_list < n_lists && ay <= th && ax <= tw && gl < ng;
  }
  float acc[4][CW];
#pragma unroll
  for (int k = 0; k < 4; ++k)
#pragma unroll
    for (int c = 0; c < CW; ++c) acc[k][c] = 0.f;

  s_head[tid] = end_idx;
  s_head[kMaxAnchorSlots + tid] = end_idx;
  if (tid == 0) s_entry[end_idx] = u32x4{0u, 0u, 0u, end_idx << 14};
  __syncthreads();

  const float x_sub = mul_rn((float)half_w, p.offset_scale), y_sub = mul_rn((float)half_h, p.offset_scale);
  const float Hf = (float)p.H, Wf = (float)p.W;
  const elem_t *om_img = reinterpret_cast<const elem_t *>(p.offset_mask) + (size_t)b * p.Q * p.P_pad;
  const elem_t *go_img = reinterpret_cast<const elem_t *>(p.grad_out) + (size_t)b * p.Q * C;
  auto load_f = [](const elem_t *ptr) { float f[1]; Pack<Tag, 1>::decode(*ptr, f); return f[0]; };
  auto to_f = [](elem_t raw) { float f[1]; Pack<Tag, 1>::decode(raw, f); return f[0]; };

  int parity = 0;                                             // which half of s_head the current strip uses
  for (int wo_lo = wo_lo_all; wo_lo < wo_hi_all && n_rows > 0; wo_lo += cols_cap) {
    const int nwx = min(cols_cap, wo_hi_all - wo_lo);

    // strips of interleaved rows: strip s takes rows ho_lo + s, ho_lo + s + n_strips, ...
    const int rows_cap = max(1, p.strip_pix / nwx);
    const int n_strips = (n_rows + rows_cap - 1) / rows_cap;
    const int rows_full = (n_rows + n_strips - 1) / n_strips;           // rows of the first strips (the last ones may have one fewer)
    const int per_group = rows_full * nwx * upp;                        // items of a group in a full strip
    const int n_items = ng * per_group;
    const float inv_per_group = 1.f / (float)per_group, inv_nwx = 1.f / (float)nwx, inv_upp = 1.f / (float)upp;

    // Phase A work items of this lane, one per round: row of the strip | column << 10 | group << 20 | item of the
    // (pixel, group) << 26, all ones for a lane without an item.  The decode does not depend on the strip.
    uint32_t item[ROUNDS];
#pragma unroll
    for (int v = 0; v < ROUNDS; ++v) {
      const int j = v * kValThreads + tid;
      const bool in_range = j < n_items;
      const int gl = in_range ? fdiv_small(j, inv_per_group) : 0;
      const int rem = in_range ? j - gl * per_group : 0;
      const int px = KP > 0 ? rem / 3 : fdiv_small(rem, inv_upp);
      const int t = rem - px * upp;
      const int r = fdiv_small(px, inv_nwx), col = px - r * nwx;
      item[v] = in_range ? (uint32_t)r | ((uint32_t)col << 10) | ((uint32_t)gl << 20) | ((uint32_t)t << 26) : ~0u;
    }
    // sampling point tj of item u: its index k among the group's points and its kernel position (x index outer,
    // y index inner, dcnv4_im2col_cuda.cuh:216-236); false for the removed centre
    auto tap_of = [&](int u, int tj, int &k, int &ti, int &tjj) -> bool {
      if constexpr (KP == 9) {
        k = 3 * u + tj; ti = u; tjj = tj;
        return true;
      } else if constexpr (KP == 8) {
        const int kk = 3 * u + tj;
        k = kk > 4 ? kk - 1 : kk; ti = u; tjj = tj;
        return kk != 4;
      } else {
        k = u;
        int tt = u;
        if (p.remove_center && tt >= (p.kw / 2) * p.kh + p.kh / 2) ++tt;
        ti = tt / p.kh; tjj = tt - ti * p.kh;
        return true;
      }
    };

    // parking: 16-byte vectors when a group's channels are whole vectors and fill their parked width
    constexpr int kVec = 16 / Tag::kBytes;
    typedef typename Pack<Tag, kVec>::raw_t vec_t;
    const bool vec_park = D == Dp && D % kVec == 0;
    const int vpp = vec_park ? ng * D / kVec : ng * Dp;                 // vectors (elements) per parked pixel
    const float inv_vpp = 1.f / (float)vpp;

    // a lane's offsets of a strip, requested one strip ahead (before the previous strip's phase B) so that their
    // latency hides there; the modulation scalar lies in the same row and is read when it is needed
    elem_t pf_x[ROUNDS][kTaps], pf_y[ROUNDS][kTaps];
    auto prefetch = [&](int s) {
      const int rows_s = (n_rows - s + n_strips - 1) / n_strips;
#pragma unroll
      for (int v = 0; v < ROUNDS; ++v) {
#pragma unroll
        for (int tj = 0; tj < kTaps; ++tj) pf_x[v][tj] = pf_y[v][tj] = elem_t(0);
        uint32_t it = item[v];
        asm volatile("" : "+v"(it));        // decoded afresh every strip: hoisted out of the loop, the fields of all rounds stay in registers
        const int r = (int)(it & 0x3ffu), col = (int)((it >> 10) & 0x3ffu), gl = (int)((it >> 20) & 0x3fu), u = (int)(it >> 26);
        if (it == ~0u || r >= rows_s) continue;
        const int ho = ho_lo + s + r * n_strips, wo = wo_lo + col;
        const elem_t *om = om_img + ((uint32_t)(ho * p.Wo + wo) * (uint32_t)p.P_pad + (uint32_t)((g0 + gl) * 3 * Kp));
#pragma unroll
        for (int tj = 0; tj < kTaps; ++tj) {
          int k, ti, tjj;
          if (!tap_of(u, tj, k, ti, tjj)) continue;
          pf_x[v][tj] = om[2 * k]; pf_y[v][tj] = om[2 * k + 1];
        }
      }
    };
    prefetch(0);

    // Barriers of a strip: after park + phase A (rows and lists in place), after phase B (rows, entries and list heads
    // may be rewritten).  A strip's list heads live in one half of s_head; every lane resets its list's head in the
    // other half during phase B, for the next strip.
    for (int s = 0; s < n_strips; ++s) {
      const int rows_s = (n_rows - s + n_strips - 1) / n_strips;
      const int npx = rows_s * nwx;
      uint32_t *head = s_head + parity * kMaxAnchorSlots;
      parity ^= 1;

      // ---- park the strip's grad_out (this chunk's channels)
      for (int idx = tid; idx < npx * vpp; idx += kValThreads) {
        const int px = fdiv_small(idx, inv_vpp), u = idx - px * vpp;
        const int r = fdiv_small(px, inv_nwx), col = px - r * nwx;
        const elem_t *src = go_img + ((size_t)((ho_lo + s + r * n_strips) * p.Wo + wo_lo + col) * C + g0 * D);
        char *dst = s_go + px * go_stride;
        if (vec_park) {
          const vec_t raw = *reinterpret_cast<const vec_t *>(src + u * kVec);
          if constexpr (Tag::kBytes == 2) {
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

      // ---- phase A: one lane per item.  A sampling point whose 2x2 corner block touches the tile is
      // linked into the list of its ANCHOR - the block's first corner, which may lie one row above or one column left
      // of the tile: the lane swaps its entry's index into the list head and stores the old head as its successor.
#pragma unroll
      for (int v = 0; v < ROUNDS; ++v) {
        if (v * kValThreads >= n_items) continue;               // uniform
        uint32_t it = item[v];
        asm volatile("" : "+v"(it));
        const int r = (int)(it & 0x3ffu), col = (int)((it >> 10) & 0x3ffu), gl = (int)((it >> 20) & 0x3fu), u = (int)(it >> 26);
        if (it == ~0u || r >= rows_s) continue;
        const int ho = ho_lo + s + r * n_strips, wo = wo_lo + col;
        const elem_t *om = om_img + ((uint32_t)(ho * p.Wo + wo) * (uint32_t)p.P_pad + (uint32_t)((g0 + gl) * 3 * Kp));
        const float x_base = sub_rn((float)(cx0 + wo * p.sw), x_sub), y_base = sub_rn((float)(cy0 + ho * p.sh), y_sub);
        const int px = r * nwx + col;
        const uint32_t go_addr16 = (uint32_t)(px * go_stride + gl * Dp * kParkBytes) >> 4;
        const int list_row = gl * aw;
        // the item's modulation scalars, requested together before any position is formed: one latency per item
        elem_t m_raws[kTaps];
#pragma unroll
        for (int tj = 0; tj < kTaps; ++tj) {
          int k, ti, tjj;
          m_raws[tj] = tap_of(u, tj, k, ti, tjj) ? om[2 * Kp + k] : elem_t(0);
        }
#pragma unroll
        for (int tj = 0; tj < kTaps; ++tj) {
          int k, ti, tjj;
          if (!tap_of(u, tj, k, ti, tjj)) continue;
          const elem_t m_raw = m_raws[tj];
          const float off_x = to_f(pf_x[v][tj]), off_y = to_f(pf_y[v][tj]);
          const float x = add_rn(x_base, mul_rn(add_rn((float)(ti * p.dw), off_x), p.offset_scale));
          const float y = add_rn(y_base, mul_rn(add_rn((float)(tjj * p.dh), off_y), p.offset_scale));
          // the reference's range test (dcnv4_col2im_cuda.cuh:317); NaN and huge coordinates fail it
          if (!((y > -1.f) && (x > -1.f) && (y < Hf) && (x < Wf))) continue;
          const float fy = floorf(y), fx = floorf(x);
          // anchor relative to the anchor grid, whose first row and column lie one cell outside the tile
          const int ay = (int)fy - ty0 + 1, ax = (int)fx - tx0 + 1;
          if ((unsigned)ay > (unsigned)th || (unsigned)ax > (unsigned)tw) continue;
          float m = to_f(m_raw);
          if (p.softmax) {          // rare: normalise over this group's taps
            float mx = load_f(om + 2 * Kp), sum = 0.f;
            for (int kk = 1; kk < Kp; ++kk) mx = fmaxf(mx, load_f(om + 2 * Kp + kk));
            for (int kk = 0; kk < Kp; ++kk) sum += __expf(load_f(om + 2 * Kp + kk) - mx);
            m = __expf(m - mx) / sum;
          }
          const float ly = y - fy, lx = x - fx;
          const int list = ay * (p.ng_chunk * aw) + list_row + ax;
          const uint32_t mine = (uint32_t)((v * kValThreads + tid) * kTaps + tj);
          const uint32_t succ = __hip_atomic_exchange(&head[list], mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
          s_entry[mine] = u32x4{__builtin_bit_cast(uint32_t, m * (1.f - ly)), __builtin_bit_cast(uint32_t, m * ly),
                                __builtin_bit_cast(uint32_t, lx), go_addr16 | (succ << 14)};
        }
        __builtin_amdgcn_sched_barrier(0);      // one round at a time: interleaved, the rounds' temporaries spill
      }
      if (s + 1 < n_strips) prefetch(s + 1);
      __syncthreads();

      // ---- phase B: every lane walks its own anchor's list; the next entry is read while the current one is applied.
      // Corner weights (common.h:48-58, 153-184): modulation * row weight * column weight.
      if (list_live) {
        uint32_t e = head[my_list];
        s_head[parity * kMaxAnchorSlots + my_list] = end_idx;    // the next strip's head of this list
        const char *go_lane = s_go + my_part * kLaneBytes;
        u32x4 ent = s_entry[e];
        while (e != end_idx) {
          e = ent.w >> 14;
          const u32x4 next = s_entry[e];
          const uint32_t a_bits = ent.x, b_bits = ent.y, fx_bits = ent.z;
          const float wa = __builtin_bit_cast(float, a_bits), wb = __builtin_bit_cast(float, b_bits);
          const float fxv = __builtin_bit_cast(float, fx_bits), hxv = 1.f - fxv;
          const float w4[4] = {wa * hxv, wa * fxv, wb * hxv, wb * fxv};
          const char *g = go_lane + ((ent.w & 0x3fffu) << 4);
          // the row in pieces of at most 32 bytes, one piece in registers at a time
          constexpr int kPieceBytes = kLaneBytes < 32 ? kLaneBytes : 32;
          constexpr int kPiece = kPieceBytes / kParkBytes;       // channels per piece
#pragma unroll
          for (int h = 0; h < CW / kPiece; ++h) {
            park_t gv[kPiece];
#pragma unroll
            for (int q = 0; q < kPieceBytes / 16; ++q)
              *reinterpret_cast<u32x4 *>(reinterpret_cast<char *>(gv) + 16 * q) = *reinterpret_cast<const u32x4 *>(g + kPieceBytes * h + 16 * q);
#pragma unroll
            for (int k = 0; k < 4; ++k)
#pragma unroll
              for (int c = 0; c < kPiece; ++c) acc[k][h * kPiece + c] = fmaf(w4[k], (float)gv[c], acc[k][h * kPiece + c]);
            if (h + 1 < CW / kPiece) __builtin_amdgcn_sched_barrier(0);
          }
          ent = next;
        }
      }
      __syncthreads();
    }
  }

  // The four corner sums of every anchor meet in an fp32 image of the tile, [cell][group][Dp], one corner at a time:
  // anchor (ay, ax) holds the sums of cells (ay - 1 + dy, ax - 1 + dx); for a given corner no two anchors name the
  // same cell, so plain LDS stores and read-modify-writes suffice.  Corner 0 reaches every cell of the tile and so
  // initialises the image.
  float *s_sum = reinterpret_cast<float *>(lds32);
  int list_now = my_list;
  asm volatile("" : "+v"(list_now));      // the list's coordinates are decoded here, not kept in registers from the start
  const int my_row = fdiv_small(list_now, 1.f / (float)aw), my_ax = list_now - my_row * aw;
  const int my_ay = fdiv_small(my_row, 1.f / (float)p.ng_chunk), my_gl = my_row - my_ay * p.ng_chunk;
  const int row_floats = dcnv4_grad_value_image_stride(p.ng_chunk * Dp);      // floats between cells (an odd number of 16-byte units)
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int cy = my_ay - 1 + (k >> 1), cx = my_ax - 1 + (k & 1);
    if (list_live && (unsigned)cy < (unsigned)th && (unsigned)cx < (unsigned)tw) {
      float *dst = s_sum + (cy * ew + cx) * row_floats + my_gl * Dp + my_part * CW;
#pragma unroll
      for (int q = 0; q < CW / 4; ++q) {
        f32x4 v = f32x4{acc[k][4 * q], acc[k][4 * q + 1], acc[k][4 * q + 2], acc[k][4 * q + 3]};
        if (k > 0) v += *reinterpret_cast<const f32x4 *>(dst + 4 * q);
        *reinterpret_cast<f32x4 *>(dst + 4 * q) = v;
      }
    }
    __syncthreads();
  }

  // fp32 image -> tensor dtype -> memory, a lane per 16-byte piece (whole groups of channels) or per element
  elem_t *gv_img = reinterpret_cast<elem_t *>(p.grad_value) + (size_t)b * p.H * p.W * C;
  constexpr int kVecOut = 16 / Tag::kBytes;
  if (D % kVecOut == 0) {
    const int ppc = ng * (D / kVecOut);                          // pieces per cell
    const float inv_ppc = 1.f / (float)ppc, inv_tw = 1.f / (float)tw, inv_dv = 1.f / (float)(D / kVecOut);
    for (int idx = tid; idx < th * tw * ppc; idx += kValThreads) {
      const int cell = fdiv_small(idx, inv_ppc), piece = idx - cell * ppc;
      const int cy = fdiv_small(cell, inv_tw), cx = cell - cy * tw;
      const int gl = fdiv_small(piece, inv_dv), ch = (piece - gl * (D / kVecOut)) * kVecOut;
      const float *src = s_sum + (cy * ew + cx) * row_floats + gl * Dp + ch;
      float f[kVecOut];
#pragma unroll
      for (int i = 0; i < kVecOut; i += 4) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(src + i);
        f[i] = v.x; f[i + 1] = v.y; f[i + 2] = v.z; f[i + 3] = v.w;
      }
      u32x4 *dst = reinterpret_cast<u32x4 *>(gv_img + ((size_t)((ty0 + cy) * p.W + tx0 + cx) * C + (g0 + gl) * D + ch));
      // fp32 tensors: with the nontemporal hint (T stage 1 backward 0.187 -> 0.180 ms); 16-bit ones lose 1-3 % to it
      if constexpr (Tag::kBytes == 4) __builtin_nontemporal_store(Pack<Tag, kVecOut>::encode(f), dst);
      else *dst = Pack<Tag, kVecOut>::encode(f);
    }
  } else {
    const int epc = ng * D;                                      // elements per cell
    const float inv_epc = 1.f / (float)epc, inv_tw = 1.f / (float)tw, inv_d = 1.f / (float)D;
    for (int idx = tid; idx < th * tw * epc; idx += kValThreads) {
      const int cell = fdiv_small(idx, inv_epc), el = idx - cell * epc;
      const int cy = fdiv_small(cell, inv_tw), cx = cell - cy * tw;
      const int gl = fdiv_small(el, inv_d), ch = el - gl * D;
      const float f[1] = {s_sum[(cy * ew + cx) * row_floats + gl * Dp + ch]};
      gv_img[(size_t)((ty0 + cy) * p.W + tx0 + cx) * C + (g0 + gl) * D + ch] = Pack<Tag, 1>::encode(f);
    }
  }
}


}  // namespace
}  // namespace dcn
