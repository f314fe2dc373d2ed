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
//   * it visits every output pixel whose reference point lies within `reach` pixels of the tile
//     (strip by strip, offset_mask slices staged in LDS), recomputes the bilinear corners, and
//     accumulates the corners that land inside its tile into LDS with 64-bit integer atomics on
//     fixed-point values: results are bit-reproducible, independent of scheduling;
//   * fixed point: contributions are normalised by the global maxima of |grad_out| and
//     |modulation| (GradState, produced by the grad_offset_mask kernel that runs first) and carry
//     `fix_bits` fractional bits, i.e. an absolute resolution of 2^-fix_bits of the largest possible
//     contribution - finer than fp32 accumulation unless a sum is > 2^25 times smaller than that;
//   * corners farther than `reach` from their output pixel's tile, and the case of non-finite
//     statistics, are left to the fallback scatter kernel (dcnv4_kernels.hip, kBwdFallback),
//     which runs afterwards and does nothing in the common case.
//
// Lane layout: a row of 16 lanes owns one (output pixel, group); lane c owns channels c, c+16, ...
// A wave is four rows - the four groups of one pixel when ng_chunk = 4, D = 16 - so one
// ds_add_u64 instruction covers 64 distinct channels of 4 cells: exactly two conflict-free
// sweeps of the 64 LDS banks.  The 16 lanes of a row first work tap-parallel (lane t computes
// tap t: position, weights, cell index, validity), then each tap's results are broadcast along
// the row with DPP row_newbcast and every lane adds its own channel.
#include <utility>

#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

constexpr int kValThreads = 1024;
constexpr int kRow = 16;
constexpr int kTrashPad = 64;
constexpr int kStageBatch = 8;     // independent staging loads in flight per thread
constexpr int kPassBatch = 4;      // row passes whose grad_out loads are issued together

template <int K> __device__ __forceinline__ float row_bcast_f(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x150 + K, 0xf, 0xf, false));
}
template <int K> __device__ __forceinline__ int row_bcast_i(int v) {
  return __builtin_amdgcn_update_dpp(0, v, 0x150 + K, 0xf, 0xf, false);
}
__device__ __forceinline__ int row_bcast_dyn(int v, int k) {   // k < 16, same for the whole wave
  const int lane = threadIdx.x & (kWave - 1);
  return __builtin_amdgcn_ds_bpermute(((lane & ~(kRow - 1)) + k) << 2, v);
}

// float (|t| < 2^62) -> two's-complement 64-bit integer, exact (t carries 24 significant bits).
__device__ __forceinline__ unsigned long long to_fixed(float t) {
  const float th = floorf(t * 0x1p-32f);
  const int hi = (int)th;
  const uint32_t lo = (uint32_t)fmaf(th, -0x1p32f, t);
  return ((unsigned long long)(uint32_t)hi << 32) | lo;
}

struct RowTap {       // what lane t of a row holds for tap t
  int cell_off;       // ((y0 - tile_y0) * tile_w + (x0 - tile_x0)) * ch_stride; corners add 0, 1, tile_w, tile_w+1 cells
  int valid;          // bit c: corner c is inside the image and inside this tile
  float w[4];         // modulation * bilinear weight on the fixed-point grid, 0 for corners that are not valid
};

template <typename Tag, int KP, int CPL>
__global__ void __launch_bounds__(kValThreads) dcnv4_grad_value_kernel(const DcnLaunch p) {
  extern __shared__ unsigned long long lds64[];
  const int Kp = p.Kp, D = p.D, C = p.G * p.D;
  const int n_chunks = (p.G + p.ng_chunk - 1) / p.ng_chunk;
  const int nty = (p.H + p.tile_h - 1) >> p.tile_h_log2, ntx = (p.W + p.tile_w - 1) >> p.tile_w_log2;
  uint32_t id = xcd_contiguous_block(blockIdx.x, gridDim.x);
  const int chunk = id % n_chunks; id /= n_chunks;
  const int tx = id % ntx; id /= ntx;
  const int ty = id % nty;
  const int b = id / nty;
  const int g0 = chunk * p.ng_chunk, ng = min(p.ng_chunk, p.G - g0);
  const int ch_stride = p.ng_chunk * D;                 // accumulator channels per cell
  const int ty0 = ty << p.tile_h_log2, tx0 = tx << p.tile_w_log2;
  const int th = min(p.tile_h, p.H - ty0), tw = min(p.tile_w, p.W - tx0);
  const int n_cells = p.tile_h * p.tile_w;
  // the slots past the tile absorb the zero-valued adds of lanes whose corner is not in the tile,
  // and of lanes whose channel index runs past D (group widths that are not multiples of 16)
  const int trash_off = n_cells * ch_stride;
  const int n_acc = trash_off + ch_stride + kTrashPad;
  unsigned long long *acc = lds64;
  float *s_om = reinterpret_cast<float *>(lds64 + n_acc);
  const int slice = ng * 3 * Kp;                        // staged offset_mask elements per pixel

  const uint32_t gmax = p.state->go_max_bits, mmax = p.state->mask_max_bits;
  const bool finite = gmax < 0x7f800000u && mmax < 0x7f800000u;
  // 2^e > max >= 2^(e-1); zero maxima mean an all-zero gradient and any exponent works
  const int e_go = (int)(gmax >> 23) - 126, e_m = (int)(mmax >> 23) - 126;

  for (int i = threadIdx.x; i < n_acc; i += kValThreads) acc[i] = 0ull;

  // output pixels this tile visits: reference point within `reach` of the tile (near_box)
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
  const int cy0 = half_h - p.ph, cx0 = half_w - p.pw, Ho = p.Q / p.Wo;
  const int ho_lo = max(0, ceil_div_signed(ty0 - p.reach - cy0, p.sh));
  const int ho_hi = min(Ho, ceil_div_signed(ty0 + p.tile_h + p.reach - cy0, p.sh));
  const int wo_lo = max(0, ceil_div_signed(tx0 - p.reach - cx0, p.sw));
  const int wo_hi = min(p.Wo, ceil_div_signed(tx0 + p.tile_w + p.reach - cx0, p.sw));
  const int nwx = wo_hi - wo_lo;
  const int lane = threadIdx.x & (kWave - 1), c = lane & (kRow - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int row_in_wave = lane / kRow;
  const float x_sub = mul_rn((float)half_w, p.offset_scale), y_sub = mul_rn((float)half_h, p.offset_scale);
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  const elem_t *om_g = reinterpret_cast<const elem_t *>(p.offset_mask);
  const elem_t *go_g = reinterpret_cast<const elem_t *>(p.grad_out);

  if (finite && nwx > 0 && ho_hi > ho_lo && (gmax | mmax) != 0) {
    const int rows_per_strip = max(1, p.strip_pix / nwx);
    for (int hs = ho_lo; hs < ho_hi; hs += rows_per_strip) {
      const int nrows = min(rows_per_strip, ho_hi - hs);
      const int npx = nrows * nwx;
      __syncthreads();      // previous strip fully consumed (and acc cleared, first time round)
      // stage the strip's offset_mask slices: thread -> (pixel, element), all loads of a thread
      // issued back to back before the first LDS write so their latencies overlap
      {
        const int e_lanes = slice <= 128 ? 128 : (slice <= 256 ? 256 : 1024);
        const int e0 = threadIdx.x & (e_lanes - 1), px_step = kValThreads / e_lanes;
        for (int e = e0; e < slice; e += e_lanes) {
          for (int pxb = threadIdx.x / e_lanes; pxb < npx; pxb += kStageBatch * px_step) {
            elem_t raw[kStageBatch];
#pragma unroll
            for (int u = 0; u < kStageBatch; ++u) {
              const int px = pxb + u * px_step;
              raw[u] = elem_t(0);
              if (px < npx) {
                const int r = px / nwx, wx = px - r * nwx;
                raw[u] = om_g[((size_t)b * p.Q + (size_t)(hs + r) * p.Wo + wo_lo + wx) * p.P_pad + g0 * 3 * Kp + e];
              }
            }
#pragma unroll
            for (int u = 0; u < kStageBatch; ++u) {
              const int px = pxb + u * px_step;
              if (px < npx) {
                float f[1];
                Pack<Tag, 1>::decode(raw[u], f);
                s_om[px * slice + e] = f[0];
              }
            }
          }
        }
      }
      __syncthreads();

      const int n_items = npx * ng;
      constexpr int kItemStep = kValThreads / kRow;       // rows of 16 lanes per workgroup pass
      for (int itemb = wave * 4; itemb < n_items; itemb += kPassBatch * kItemStep) {
       // grad_out of the next kPassBatch passes: loads issued together, latencies overlap
       elem_t go_raw[kPassBatch][CPL];
#pragma unroll
       for (int u = 0; u < kPassBatch; ++u) {
         const int item = itemb + u * kItemStep + row_in_wave;
         const int px = item < n_items ? item / ng : 0, gl = item < n_items ? item - px * ng : 0;
         const int r = px / nwx, wx = px - r * nwx;
         const elem_t *gsrc = go_g + ((size_t)b * p.Q + (size_t)(hs + r) * p.Wo + wo_lo + wx) * C + (g0 + gl) * D;
#pragma unroll
         for (int j = 0; j < CPL; ++j) {
           go_raw[u][j] = elem_t(0);
           if (item < n_items && c + kRow * j < D) go_raw[u][j] = gsrc[c + kRow * j];
         }
       }
#pragma unroll
       for (int u = 0; u < kPassBatch; ++u) {
        const int item0 = itemb + u * kItemStep;
        if (item0 >= n_items) break;
        const int item = item0 + row_in_wave;
        const bool live = item < n_items;
        const int px = live ? item / ng : 0, gl = live ? item - px * ng : 0;
        const int r = px / nwx, wx = px - r * nwx;
        const int ho = hs + r, wo = wo_lo + wx;
        const float *om = s_om + px * slice + gl * 3 * Kp;
        // this lane's channels of grad_out, normalised to [-1, 1]; channels past D stay 0
        float gn[CPL];
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
          float f[1];
          Pack<Tag, 1>::decode(go_raw[u][j], f);
          gn[j] = ldexpf(f[0], -e_go);
        }
        float mx = 0.f, inv = 1.f;
        if (p.softmax && live) softmax_stats(om + 2 * Kp, Kp, mx, inv);
        const float x_base = sub_rn((float)(cx0 + wo * p.sw), x_sub), y_base = sub_rn((float)(cy0 + ho * p.sh), y_sub);
        unsigned long long *acc_lane = acc + gl * D + c;

        for (int t0 = 0; t0 < Kp; t0 += kRow) {           // 16 taps at a time, one per lane
          RowTap rt;
          rt.cell_off = trash_off; rt.valid = 0;
          rt.w[0] = rt.w[1] = rt.w[2] = rt.w[3] = 0.f;
          const int t = t0 + c;
          if (live && t < Kp) {
            int i, j;
            if constexpr (KP > 0) {
              tap_ij_3x3(KP, t, i, j);
            } else {
              // x index outer, y index inner, centre skipped when remove_center
              int tt = t;
              if (p.remove_center && tt >= (p.kw / 2) * p.kh + p.kh / 2) ++tt;
              i = tt / p.kh; j = tt - i * p.kh;
            }
            const float x = add_rn(x_base, mul_rn(add_rn((float)(i * p.dw), om[2 * t]), p.offset_scale));
            const float y = add_rn(y_base, mul_rn(add_rn((float)(j * p.dh), om[2 * t + 1]), p.offset_scale));
            float m = om[2 * Kp + t];
            if (p.softmax) m = __expf(m - mx) * inv;
            const Tap tp = make_tap(y, x, p.H, p.W, 0u, 0u);
            const int ly = tp.y0 - ty0, lx = tp.x0 - tx0;
            const bool r0 = ly >= 0 && ly < th, r1 = ly + 1 >= 0 && ly + 1 < th;
            const bool c0 = lx >= 0 && lx < tw, c1 = lx + 1 >= 0 && lx + 1 < tw;
            rt.valid = (int)(tp.valid & ((uint32_t)(r0 && c0) | ((uint32_t)(r0 && c1) << 1) | ((uint32_t)(r1 && c0) << 2) |
                                         ((uint32_t)(r1 && c1) << 3)));
            rt.cell_off = ((ly << p.tile_w_log2) + lx) * ch_stride;
            const float ms = ldexpf(m, p.fix_bits - e_m);
#pragma unroll
            for (int cn = 0; cn < 4; ++cn) rt.w[cn] = (rt.valid & (1 << cn)) ? ms * tp.w[cn] : 0.f;
          }
          auto scatter_tap = [&](int cell_off, int valid, float w0, float w1, float w2, float w3) {
            if (__builtin_amdgcn_ballot_w64(valid != 0) == 0) return;       // nobody in the wave hits the tile
            const float w[4] = {w0, w1, w2, w3};
#pragma unroll
            for (int cn = 0; cn < 4; ++cn) {
              const bool ok = valid & (1 << cn);
              if (__builtin_amdgcn_ballot_w64(ok) == 0) continue;
              const int off = ok ? cell_off + ((cn >> 1) * p.tile_w + (cn & 1)) * ch_stride : trash_off;
#pragma unroll
              for (int j = 0; j < CPL; ++j)
                __hip_atomic_fetch_add(acc_lane + off + kRow * j, to_fixed(gn[j] * w[cn]), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_WORKGROUP);
            }
          };
          if constexpr (KP > 0) {
            auto unrolled = [&]<int... Ks>(std::integer_sequence<int, Ks...>) {
              (scatter_tap(row_bcast_i<Ks>(rt.cell_off), row_bcast_i<Ks>(rt.valid), row_bcast_f<Ks>(rt.w[0]),
                           row_bcast_f<Ks>(rt.w[1]), row_bcast_f<Ks>(rt.w[2]), row_bcast_f<Ks>(rt.w[3])), ...);
            };
            unrolled(std::make_integer_sequence<int, KP>{});
          } else {
            const int nt = min(kRow, Kp - t0);
            for (int k = 0; k < nt; ++k)
              scatter_tap(row_bcast_dyn(rt.cell_off, k), row_bcast_dyn(rt.valid, k),
                          __builtin_bit_cast(float, row_bcast_dyn(__builtin_bit_cast(int, rt.w[0]), k)),
                          __builtin_bit_cast(float, row_bcast_dyn(__builtin_bit_cast(int, rt.w[1]), k)),
                          __builtin_bit_cast(float, row_bcast_dyn(__builtin_bit_cast(int, rt.w[2]), k)),
                          __builtin_bit_cast(float, row_bcast_dyn(__builtin_bit_cast(int, rt.w[3]), k)));
          }
        }
       }
      }
    }
  }
  __syncthreads();

  // the tile is complete: fixed point -> tensor dtype, plain stores (zeros when not finite: the
  // fallback kernel then adds every corner)
  const int e_out = e_go + e_m - p.fix_bits;
  const int n_ch = ng * D;
  for (int cell = wave; cell < th * tw; cell += kValThreads / kWave) {     // one cell per wave: contiguous channels
    const int ly = cell / tw, lx = cell - ly * tw;
    const unsigned long long *src = acc + ((ly << p.tile_w_log2) + lx) * ch_stride;
    elem_t *dst = reinterpret_cast<elem_t *>(p.grad_value) + (((size_t)b * p.H + ty0 + ly) * p.W + tx0 + lx) * C + g0 * D;
    for (int ch = lane; ch < n_ch; ch += kWave) {
      const unsigned long long a = src[ch];
      const double v = ldexp((double)(int)(a >> 32) * 4294967296.0 + (double)(uint32_t)a, e_out);
      const float f[1] = {(float)v};
      dst[ch] = Pack<Tag, 1>::encode(f);
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
  const int cpl = (p.D + kRow - 1) / kRow;      // channels per lane: 1, 2 or 4 (3 rounds up to 4)
#define GV_CASE(KPV)                                                        \
  do {                                                                      \
    if (cpl == 1) return go(dcnv4_grad_value_kernel<Tag, KPV, 1>);          \
    if (cpl == 2) return go(dcnv4_grad_value_kernel<Tag, KPV, 2>);          \
    return go(dcnv4_grad_value_kernel<Tag, KPV, 4>);                        \
  } while (0)
  if (k3 && !p.remove_center) GV_CASE(9);
  if (k3 && p.remove_center) GV_CASE(8);
  GV_CASE(0);
#undef GV_CASE
}

}  // namespace

size_t dcnv4_grad_value_lds_bytes(const DcnLaunch &p) {
  return ((size_t)(p.tile_h * p.tile_w + 1) * p.ng_chunk * p.D + kTrashPad) * sizeof(unsigned long long) +
         (size_t)p.strip_pix * p.ng_chunk * 3 * p.Kp * sizeof(float);
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
