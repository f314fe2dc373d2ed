// Flash deformable attention kernels for gfx950 (wave64): multi-level bilinear sampling with
// the softmax over all L*K taps fused in.
//
// Replaces the reference's forward_kernel_reg (DCNv4_op/src/cuda/flash_deform_im2col_cuda.cuh:129-209)
// and backward_kernel_warp_primitive (DCNv4_op/src/cuda/flash_deform_col2im_cuda.cuh:171-318).
//
// A workgroup owns `nq_block` consecutive queries (all heads).  Their sampling_loc_attn rows
// are one contiguous span: streamed once into LDS as fp32 and shared by the channel lanes of a
// (query, head).  One lane owns `cpt` contiguous channels (16 bytes).  The softmax needs only a
// running max and sum per (query, head); each tap's probability is recomputed from its logit,
// so L and K stay run-time values.  Backward applies the Jacobian in closed form,
// p_i (a_i - sum_j p_j a_j), where the reference loops over all (L*K)^2 pairs
// (flash_deform_col2im_cuda.cuh:301-316); a tap outside its level contributes a_i = 0.
#include "common.hpp"
#include "launch.hpp"

#include <algorithm>
#include <utility>

namespace dcn {
namespace {

struct Level { int H, W, start; };

__device__ __forceinline__ Level load_level(const FdaLaunch &p, int l) {
  Level lv;
  lv.H = (int)p.shapes[2 * l];
  lv.W = (int)p.shapes[2 * l + 1];
  lv.start = (int)p.level_start[l];
  return lv;
}

// n / d for 0 <= n < 2^20 with inv = 1 / d
__device__ __forceinline__ int fdiv20(int n, float inv) { return (int)(((float)n + 0.5f) * inv); }

template <typename Tag>
__device__ __forceinline__ float elem_f32(const void *base, size_t i) {
  float f[1];
  Pack<Tag, 1>::decode(reinterpret_cast<const typename RawWord<Tag::kBytes>::type *>(base)[i], f);
  return f[0];
}

// Rows of the workgroup's (query, head) pairs into LDS as fp32, [pair][3 * L * K]: 2 L K locations, then L K logits.
// Pair j is query row0 + j / heads_here, head g0 + j % heads_here.  Packed input: one tensor in the tensor dtype.
// Split input (p.loc set): locations and logits are separate tensors, and every location passes through fp16 on its
// way in, which is what the reference's module does before it packs them
// (DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133: `.half()`, then `cat` with the logits).
template <typename Tag>
__device__ __forceinline__ void fda_stage_rows(float *lds, const FdaLaunch &p, int row0, int nrow, int g0, int heads_here) {
  const int LK = p.L * p.K, row_len = 3 * LK, pairs = nrow * heads_here;
  const float inv_h = 1.f / (float)heads_here;
  if (p.loc == nullptr) {
    if (heads_here == p.G) {
      const bool vec16 = ((size_t)p.G * row_len * Tag::kBytes) % 16 == 0;
      stage_rows_to_lds<Tag>(lds, (const char *)p.sla + (size_t)row0 * p.G * row_len * Tag::kBytes, pairs * row_len, vec16);
    } else if (constexpr int EPV = 16 / Tag::kBytes; row_len % EPV == 0) {      // rows of some heads: 16-byte pieces of a row
      const int vpr = row_len / EPV;
      const float inv_vpr = 1.f / (float)vpr;
      const u32x4 *src = reinterpret_cast<const u32x4 *>(p.sla);
      for (int i = threadIdx.x; i < pairs * vpr; i += blockDim.x) {
        const int j = fdiv20(i, inv_vpr), v = i - j * vpr;
        const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
        float f[EPV];
        Pack<Tag, EPV>::decode(__builtin_nontemporal_load(src + ((size_t)(row0 + r) * p.G + g0 + gh) * vpr + v), f);
#pragma unroll
        for (int e = 0; e < EPV; e += 4)
          *reinterpret_cast<f32x4 *>(lds + i * EPV + e) = f32x4{f[e], f[e + 1], f[e + 2], f[e + 3]};
      }
    } else {
      const float inv_len = 1.f / (float)row_len;
      for (int i = threadIdx.x; i < pairs * row_len; i += blockDim.x) {
        const int j = fdiv20(i, inv_len), e = i - j * row_len;
        const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
        lds[i] = elem_f32<Tag>(p.sla, ((size_t)(row0 + r) * p.G + g0 + gh) * row_len + e);
      }
    }
    return;
  }
  const float inv_2lk = 1.f / (float)(2 * LK), inv_lk = 1.f / (float)LK;
  for (int i = threadIdx.x; i < pairs * 2 * LK; i += blockDim.x) {
    const int j = fdiv20(i, inv_2lk), e = i - j * 2 * LK;
    const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
    const size_t src = ((size_t)(row0 + r) * p.G + g0 + gh) * (2 * LK) + e;
    const float v = p.loc_f32 ? reinterpret_cast<const float *>(p.loc)[src] : elem_f32<Tag>(p.loc, src);
    lds[j * row_len + e] = (float)(_Float16)v;
  }
  for (int i = threadIdx.x; i < pairs * LK; i += blockDim.x) {
    const int j = fdiv20(i, inv_lk), e = i - j * LK;
    const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
    lds[j * row_len + 2 * LK + e] = elem_f32<Tag>(p.logits, ((size_t)(row0 + r) * p.G + g0 + gh) * LK + e);
  }
}

// The gradient rows back to memory, same layouts.  The gradient of a location is written in the locations' dtype;
// for fp32 locations it is rounded through fp16 first (values beyond the fp16 range become infinities), as autograd
// does in the reference's module: the gradient of `sampling_locations.half()` arrives as an fp16 tensor and is then
// widened (DCNv4_op/DCNv4/modules/flash_deform_attn.py:132-133).
template <typename Tag>
__device__ __forceinline__ void fda_unstage_grads(const float *lds, const FdaLaunch &p, int row0, int nrow, int g0, int heads_here) {
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  const int LK = p.L * p.K, row_len = 3 * LK, pairs = nrow * heads_here;
  const float inv_h = 1.f / (float)heads_here;
  if (p.loc == nullptr) {
    if (heads_here == p.G) {
      const bool vec16 = ((size_t)p.G * row_len * Tag::kBytes) % 16 == 0;
      unstage_rows_from_lds<Tag>((char *)p.grad_sla + (size_t)row0 * p.G * row_len * Tag::kBytes, lds, pairs * row_len, vec16);
    } else if (constexpr int EPV = 16 / Tag::kBytes; row_len % EPV == 0) {
      const int vpr = row_len / EPV;
      const float inv_vpr = 1.f / (float)vpr;
      u32x4 *dst = reinterpret_cast<u32x4 *>(p.grad_sla);
      for (int i = threadIdx.x; i < pairs * vpr; i += blockDim.x) {
        const int j = fdiv20(i, inv_vpr), v = i - j * vpr;
        const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
        float f[EPV];
#pragma unroll
        for (int e = 0; e < EPV; e += 4) {
          const f32x4 q = *reinterpret_cast<const f32x4 *>(lds + i * EPV + e);
          f[e] = q.x; f[e + 1] = q.y; f[e + 2] = q.z; f[e + 3] = q.w;
        }
        __builtin_nontemporal_store(Pack<Tag, EPV>::encode(f), dst + ((size_t)(row0 + r) * p.G + g0 + gh) * vpr + v);
      }
    } else {
      const float inv_len = 1.f / (float)row_len;
      for (int i = threadIdx.x; i < pairs * row_len; i += blockDim.x) {
        const int j = fdiv20(i, inv_len), e = i - j * row_len;
        const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
        const float f[1] = {lds[i]};
        reinterpret_cast<elem_t *>(p.grad_sla)[((size_t)(row0 + r) * p.G + g0 + gh) * row_len + e] = Pack<Tag, 1>::encode(f);
      }
    }
    return;
  }
  const float inv_2lk = 1.f / (float)(2 * LK), inv_lk = 1.f / (float)LK;
  for (int i = threadIdx.x; i < pairs * 2 * LK; i += blockDim.x) {
    const int j = fdiv20(i, inv_2lk), e = i - j * 2 * LK;
    const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
    const size_t dst = ((size_t)(row0 + r) * p.G + g0 + gh) * (2 * LK) + e;
    const float f[1] = {lds[j * row_len + e]};
    if (p.loc_f32) reinterpret_cast<float *>(p.grad_loc)[dst] = (float)(_Float16)f[0];
    else reinterpret_cast<elem_t *>(p.grad_loc)[dst] = Pack<Tag, 1>::encode(f);
  }
  for (int i = threadIdx.x; i < pairs * LK; i += blockDim.x) {
    const int j = fdiv20(i, inv_lk), e = i - j * LK;
    const int r = fdiv20(j, inv_h), gh = j - r * heads_here;
    const float f[1] = {lds[j * row_len + 2 * LK + e]};
    reinterpret_cast<elem_t *>(p.grad_logits)[((size_t)(row0 + r) * p.G + g0 + gh) * LK + e] = Pack<Tag, 1>::encode(f);
  }
}

// ------------------------------------------------------------------------------- forward, shared set-up inside a quad
// When four or more lanes share a (query, head) - aligned quads of the wave - and K is a multiple of four, the lanes of
// a quad split the per-point work that does not depend on the channel: lane j of the quad takes every fourth logit for
// the softmax statistics and prepares sampling point k0 + j of each group of four (position, probability, the four
// corner weights times the probability, the four corner offsets); the other three read what it prepared with DPP
// quad broadcasts and add their own channel offset.  Per point and lane that leaves the gathers and the multiply-adds.
template <int J> __device__ __forceinline__ int quad_pick(int v) {
  return __builtin_amdgcn_update_dpp(0, v, J * 0x55, 0xf, 0xf, true);
}
template <int... Js, typename F>
__device__ __forceinline__ void static_for(std::integer_sequence<int, Js...>, F &&f) {
  (f(std::integral_constant<int, Js>{}), ...);
}

__device__ __forceinline__ void quad_softmax_stats(const float *m, int n, int my_k, float &mx, float &inv) {
  mx = m[my_k];
  for (int k = my_k + 4; k < n; k += 4) mx = fmaxf(mx, m[k]);
  mx = fmaxf(mx, dpp_quad_xor1(mx));
  mx = fmaxf(mx, dpp_quad_xor2(mx));
  float sum = 0.f;
  for (int k = my_k; k < n; k += 4) sum += __expf(m[k] - mx);
  sum += dpp_quad_xor1(sum);
  sum += dpp_quad_xor2(sum);
  inv = 1.f / sum;
}

// The K points of level l for one lane.  base: byte offset of the level's pixel 0 for this (image, head), without
// the lane's channels; staged: the level lies in LDS at s_stage + base, with one head's width of zero bytes at s_stage
// for corners outside the level (a lane's channel offset stays inside them).
template <typename Tag, int CPT>
__device__ __forceinline__ void fda_quad_level(float (&acc)[CPT], const float *s, int LK, int K, int l, const Level &lv,
                                               float mx, float inv, uint32_t base, uint32_t step, uint32_t lane_off,
                                               int my_k, bool staged, const char *s_stage,
                                               const __amdgpu_buffer_rsrc_t &value) {
  typedef Pack<Tag, CPT> pack;
  typedef typename pack::raw_t raw_t;
  for (int k0 = 0; k0 < K; k0 += 4) {
    const int t = l * K + k0 + my_k;
    const float x = sub_rn(mul_rn(s[2 * t], (float)lv.W), 0.5f);       // flash_deform_im2col_cuda.cuh:188-189
    const float y = sub_rn(mul_rn(s[2 * t + 1], (float)lv.H), 0.5f);
    const float pr = __expf(s[2 * LK + t] - mx) * inv;
    const Tap tp = make_tap(y, x, lv.H, lv.W, base, step);
    int wq[4], oq[4];
#pragma unroll
    for (int cn = 0; cn < 4; ++cn) {
      wq[cn] = __builtin_bit_cast(int, pr * tp.w[cn]);
      oq[cn] = (int)((staged && !((tp.valid >> cn) & 1u)) ? 0u : tp.off[cn]);
    }
    raw_t raw[4][4];
    float w[4][4];
    if (staged) {
      static_for(std::make_integer_sequence<int, 4>{}, [&](auto j) {
        constexpr int J = decltype(j)::value;
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          w[J][cn] = __builtin_bit_cast(float, quad_pick<J>(wq[cn]));
          raw[J][cn] = *reinterpret_cast<const raw_t *>(s_stage + ((uint32_t)quad_pick<J>(oq[cn]) + lane_off));
        }
      });
    } else {
      static_for(std::make_integer_sequence<int, 4>{}, [&](auto j) {
        constexpr int J = decltype(j)::value;
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          w[J][cn] = __builtin_bit_cast(float, quad_pick<J>(wq[cn]));
          raw[J][cn] = buffer_load<pack::kBytes>(value, (uint32_t)quad_pick<J>(oq[cn]) + lane_off);
        }
      });
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        float v[CPT];
        pack::decode(raw[j][cn], v);
#pragma unroll
        for (int c = 0; c < CPT; ++c) acc[c] = fmaf(w[j][cn], v[c], acc[c]);
      }
  }
}

// Backward counterpart: the lanes of a quad gather the corners of four points prepared one by each of them, form their
// channels' share of the sixteen corner dot products, and add them up across the quad so that each sum ends in the
// lane that prepared its point (a transpose-reduce: after the exchange with the lane one away a lane holds the points
// of its own parity, after the exchange with the lane two away its own point).  That lane applies the bilinear
// derivatives and writes the point's three gradient slots, and its key and record (keys, recs: those of the query's
// first point of this level).  Returns the lane's sum of probability x d(out)/d(prob).
template <typename Tag, int CPT>
__device__ __forceinline__ float fda_quad_level_backward(const float (&go)[CPT], const float *s, float *gs, int LK, int K, int l,
                                                        const Level &lv, float mx, float inv, uint32_t base, uint32_t step,
                                                        uint32_t lane_off, int my_k, int width, bool writer,
                                                        const __amdgpu_buffer_rsrc_t &value, uint16_t *keys, f32x4_t *recs) {
  typedef Pack<Tag, CPT> pack;
  typedef typename pack::raw_t raw_t;
  const bool odd = (my_k & 1) != 0, high = (my_k & 2) != 0;
  float dot_mine = 0.f;
  for (int k0 = 0; k0 < K; k0 += 4) {
    const int t = l * K + k0 + my_k;
    const float x = sub_rn(mul_rn(s[2 * t], (float)lv.W), 0.5f);
    const float y = sub_rn(mul_rn(s[2 * t + 1], (float)lv.H), 0.5f);
    const float pr = __expf(s[2 * LK + t] - mx) * inv;
    const Tap tp = make_tap(y, x, lv.H, lv.W, base, step);
    raw_t raw[4][4];
    static_for(std::make_integer_sequence<int, 4>{}, [&](auto j) {
      constexpr int J = decltype(j)::value;
#pragma unroll
      for (int cn = 0; cn < 4; ++cn)
        raw[J][cn] = buffer_load<pack::kBytes>(value, (uint32_t)quad_pick<J>((int)tp.off[cn]) + lane_off);
    });
    float d[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        float v[CPT];
        pack::decode(raw[j][cn], v);
        float a = 0.f;
#pragma unroll
        for (int c = 0; c < CPT; ++c) a = fmaf(v[c], go[c], a);
        d[j][cn] = a;
      }
    float r[4];
#pragma unroll
    for (int cn = 0; cn < 4; ++cn) {
      float pair[2];
#pragma unroll
      for (int jh = 0; jh < 2; ++jh) {
        const float give = odd ? d[2 * jh][cn] : d[2 * jh + 1][cn], keep = odd ? d[2 * jh + 1][cn] : d[2 * jh][cn];
        pair[jh] = keep + dpp_quad_xor1(give);
      }
      const float give = high ? pair[0] : pair[1], keep = high ? pair[1] : pair[0];
      r[cn] = keep + dpp_quad_xor2(give);
      for (int o = 4; o < width; o <<= 1) r[cn] += __shfl_xor(r[cn], o, kWave);      // the other quads' channels
    }
    const float hy = 1.f - tp.ly, hx = 1.f - tp.lx;
    const float gx = hy * (r[1] - r[0]) + tp.ly * (r[3] - r[2]);
    const float gy = hx * (r[2] - r[0]) + tp.lx * (r[3] - r[1]);
    const float gz = tp.w[0] * r[0] + tp.w[1] * r[1] + tp.w[2] * r[2] + tp.w[3] * r[3];
    if (writer) {
      gs[2 * t] = gx * (float)lv.W * pr;          // flash_deform_col2im_cuda.cuh:273-276
      gs[2 * t + 1] = gy * (float)lv.H * pr;
      gs[2 * LK + t] = gz;
      // key and record of the point for the tiled grad_value kernel: the writers of a wave hold consecutive points
      // of consecutive queries, whole 16-byte records side by side
      uint32_t key = kFdaKeyOutside;
      if (tp.valid != 0)
        key = (tp.y0 + 1 >= kFdaKeyFieldMax || tp.x0 + 1 >= kFdaKeyFieldMax) ? kFdaKeySaturated
                                                                            : ((uint32_t)(tp.y0 + 1) << 8) | (uint32_t)(tp.x0 + 1);
      __builtin_nontemporal_store((uint16_t)key, keys + k0 + my_k);
      __builtin_nontemporal_store(f32x4_t{x, y, pr, 0.f}, recs + k0 + my_k);
    }
    dot_mine = fmaf(pr, gz, dot_mine);
  }
  return dot_mine;
}

// ------------------------------------------------------------------------------- forward
template <typename Tag, int CPT, int KT, bool QUAD>
__global__ void __launch_bounds__(kFdaForwardThreads) fda_forward_kernel(const FdaLaunch p) {
  extern __shared__ float lds[];
  typedef Pack<Tag, CPT> pack;
  const int LK = p.L * p.K, row_len = 3 * LK;
  const uint32_t blk = xcd_contiguous_block(blockIdx.x, gridDim.x);
  int row0, nrow, heads_here = p.G, g_fixed = 0;
  if (p.head_major) {
    // Workgroups ordered [image][head][block of queries], each for ONE head: an XCD then works through one head of one
    // image at a time, whose slice of `value` (N x D elements, one or two heads per cache line) fits its L2, where the
    // whole image does not.
    const int blocks_per_image = (p.Q + p.nq_block - 1) / p.nq_block;
    const int rb = (int)(blk % (uint32_t)blocks_per_image), bg = (int)(blk / (uint32_t)blocks_per_image);
    const int b = bg / p.G;
    g_fixed = bg - b * p.G;
    heads_here = 1;
    const int q0 = rb * p.nq_block;
    nrow = min(p.nq_block, p.Q - q0);
    row0 = b * p.Q + q0;
  } else {
    row0 = (int)blk * p.nq_block;
    nrow = min(p.nq_block, p.n_row - row0);
  }
  fda_stage_rows<Tag>(lds, p, row0, nrow, g_fixed, heads_here);
  __syncthreads();

  const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);
  const int tpgp_log2 = p.lanes.tpgp_log2;
  const int items = (nrow * heads_here) << tpgp_log2;
  const uint32_t pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
  const int K = KT > 0 ? KT : p.K;

  for (int it = threadIdx.x; it < items; it += blockDim.x) {
    const int chunk = it & ((1 << tpgp_log2) - 1);
    if (chunk >= p.lanes.tpg) continue;
    const int rg = it >> tpgp_log2;                 // (row, head) index inside the workgroup
    const int lr = rg / heads_here, g = g_fixed + rg - lr * heads_here;
    const int b = (row0 + lr) / p.Q;
    const float *s = lds + rg * row_len;
    float acc[CPT];
#pragma unroll
    for (int c = 0; c < CPT; ++c) acc[c] = 0.f;
    float mx, inv;
    if constexpr (QUAD) {
      const int my_k = chunk & 3;
      quad_softmax_stats(s + 2 * LK, LK, my_k, mx, inv);
      const uint32_t lane_off = (uint32_t)(chunk * CPT) * Tag::kBytes;
      for (int l = 0; l < p.L; ++l) {
        const Level lv = load_level(p, l);
        const uint32_t base = (uint32_t)(b * p.N + lv.start) * pix_bytes + (uint32_t)(g * p.D) * Tag::kBytes;
        fda_quad_level<Tag, CPT>(acc, s, LK, K, l, lv, mx, inv, base, pix_bytes, lane_off, my_k, false, nullptr, value);
      }
    } else {
      softmax_stats(s + 2 * LK, LK, mx, inv);
      const uint32_t lane_base = (uint32_t)(g * p.D + chunk * CPT) * Tag::kBytes;
      for (int l = 0; l < p.L; ++l) {
        const Level lv = load_level(p, l);
        const uint32_t base = (uint32_t)(b * p.N + lv.start) * pix_bytes + lane_base;
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const int t = l * K + k;
          const float x = sub_rn(mul_rn(s[2 * t], (float)lv.W), 0.5f);       // flash_deform_im2col_cuda.cuh:188-189
          const float y = sub_rn(mul_rn(s[2 * t + 1], (float)lv.H), 0.5f);
          const float pr = __expf(s[2 * LK + t] - mx) * inv;
          const Tap tp = make_tap(y, x, lv.H, lv.W, base, pix_bytes);
          typename pack::raw_t raw[4];
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) raw[cn] = buffer_load<pack::kBytes>(value, tp.off[cn]);
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) {
            float v[CPT];
            pack::decode(raw[cn], v);
            const float w = pr * tp.w[cn];
#pragma unroll
            for (int c = 0; c < CPT; ++c) acc[c] = fmaf(w, v[c], acc[c]);
          }
        }
      }
    }
    char *dst = (char *)p.out + ((size_t)(row0 + lr) * (p.G * p.D) + g * p.D + chunk * CPT) * Tag::kBytes;
    __builtin_nontemporal_store(pack::encode(acc), reinterpret_cast<typename pack::raw_t *>(dst));
  }
}

// ------------------------------------------------------------------------------- forward, small levels in LDS
// The gathers of the forward are bound by the rate at which the L2 answers 64- or 128-byte requests at random
// addresses.  In a feature pyramid half of the sampling points fall on the two smallest levels, whose slice for one
// head is a few tens of KB: a workgroup of 1024 lanes that works on ONE (image, head) copies the last levels that fit
// its LDS budget into LDS once; then its waves walk the workgroup's queries independently, each staging the rows of its
// own 64 lanes' queries (no workgroup barriers); sampling points on a staged level are served from LDS, the others from
// memory as in fda_forward_kernel.  Same arithmetic in the same order per
// (query, head): identical results.  Which levels fit is decided on the device from spatial_shapes.
template <typename Tag, int CPT, int KT, bool QUAD>
__global__ void __launch_bounds__(kFdaStagedThreads) fda_forward_staged_kernel(const FdaLaunch p) {
  extern __shared__ float lds[];
  __shared__ int s_level_off[kMaxLevels];       // byte offset of a staged level in the stage area, -1: not staged
  typedef Pack<Tag, CPT> pack;
  const int LK = p.L * p.K, row_len = 3 * LK;
  const int tpgp_log2 = p.lanes.tpgp_log2;
  const int sub_q = kFdaStagedThreads >> tpgp_log2;       // queries per pass
  const uint32_t blk = xcd_contiguous_block(blockIdx.x, gridDim.x);
  const int rb = (int)(blk % (uint32_t)p.stage_blocks), bg = (int)(blk / (uint32_t)p.stage_blocks);
  const int b = bg / p.G, g = bg - b * p.G;
  // The queries of an (image, head) in passes of sub_q; its workgroups take whole passes, the first ones one more
  // than the others when the passes do not divide evenly.
  const int passes = (p.Q + sub_q - 1) / sub_q, base_passes = passes / p.stage_blocks, extra = passes - base_passes * p.stage_blocks;
  const int q_begin = (rb * base_passes + min(rb, extra)) * sub_q;
  const int q_end = min(p.Q, q_begin + (base_passes + (rb < extra ? 1 : 0)) * sub_q);
  const uint32_t head_bytes = (uint32_t)p.D * Tag::kBytes, pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
  char *s_stage = reinterpret_cast<char *>(lds + (size_t)sub_q * row_len);      // zero bytes, then the staged levels
  const int zero_bytes = fda_staged_zero_bytes((int)head_bytes);
  const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);

  if (threadIdx.x == 0) {
    int used = zero_bytes;
    bool open = true;
    for (int l = p.L - 1; l >= 0; --l) {
      const Level lv = load_level(p, l);
      const long long bytes = (long long)lv.H * lv.W * head_bytes;
      open = open && lv.H > 0 && lv.W > 0 && used + bytes <= p.stage_budget;
      s_level_off[l] = open ? used : -1;
      if (open) used += (int)bytes;
    }
  }
  if ((int)threadIdx.x < zero_bytes / 16) reinterpret_cast<u32x4 *>(s_stage)[threadIdx.x] = u32x4{0u, 0u, 0u, 0u};
  __syncthreads();
  for (int l = 0; l < p.L; ++l) {
    const int off = s_level_off[l];
    if (off < 0) continue;
    const Level lv = load_level(p, l);
    const int vpr = (int)head_bytes / 16, n_vec = lv.H * lv.W * vpr;
    const float inv_vpr = 1.f / (float)vpr;
    const uint32_t base = (uint32_t)(b * p.N + lv.start) * pix_bytes + (uint32_t)g * head_bytes;
    for (int i = threadIdx.x; i < n_vec; i += kFdaStagedThreads) {
      const int n = fdiv20(i, inv_vpr), v = i - n * vpr;
      *reinterpret_cast<u32x4 *>(s_stage + off + i * 16) = buffer_load<16>(value, base + (uint32_t)n * pix_bytes + 16u * v);
    }
  }

  __syncthreads();                        // the levels are in place; from here on the waves go their own ways

  // Every wave walks its own passes of 64 / lanes-per-(query, head) queries: it stages their rows in its own slice of
  // the row area and works on them, with no workgroup barrier (a wave's LDS operations complete in program order).
  const int K = KT > 0 ? KT : p.K;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int qpw = kWave >> tpgp_log2;
  const int chunk = lane & ((1 << tpgp_log2) - 1), lr = lane >> tpgp_log2;
  const uint32_t lane_off = (uint32_t)(chunk * CPT) * Tag::kBytes;
  float *rows = lds + (size_t)wave * qpw * row_len;
  constexpr int EPV = 16 / Tag::kBytes;
  const bool vec_rows = p.loc == nullptr && (row_len % EPV) == 0;
  const int vpr = row_len / EPV;                                     // 16-byte vectors per row (vec_rows)
  const float inv_vpr = 1.f / (float)max(vpr, 1), inv_len = 1.f / (float)row_len;
  const float inv_2lk = 1.f / (float)(2 * LK), inv_lk = 1.f / (float)LK;
  for (int q0 = q_begin + wave * qpw; q0 < q_end; q0 += (kFdaStagedThreads / kWave) * qpw) {
    const int nrow = min(qpw, q_end - q0), row0 = b * p.Q + q0;
    __builtin_amdgcn_wave_barrier();      // the previous pass has read its rows
    if (vec_rows) {
      const u32x4 *src = reinterpret_cast<const u32x4 *>(p.sla);
      for (int i = lane; i < nrow * vpr; i += kWave) {
        const int r = fdiv20(i, inv_vpr), v = i - r * vpr;
        float f[EPV];
        Pack<Tag, EPV>::decode(src[((size_t)(row0 + r) * p.G + g) * vpr + v], f);
#pragma unroll
        for (int j = 0; j < EPV; j += 4)
          *reinterpret_cast<f32x4 *>(rows + r * row_len + v * EPV + j) = f32x4{f[j], f[j + 1], f[j + 2], f[j + 3]};
      }
    } else if (p.loc == nullptr) {
      for (int i = lane; i < nrow * row_len; i += kWave) {
        const int r = fdiv20(i, inv_len), e = i - r * row_len;
        rows[i] = elem_f32<Tag>(p.sla, ((size_t)(row0 + r) * p.G + g) * row_len + e);
      }
    } else {      // locations (rounded through fp16) and logits from their own tensors
      for (int i = lane; i < nrow * 2 * LK; i += kWave) {
        const int r = fdiv20(i, inv_2lk), e = i - r * 2 * LK;
        const size_t at = ((size_t)(row0 + r) * p.G + g) * (2 * LK) + e;
        const float v = p.loc_f32 ? reinterpret_cast<const float *>(p.loc)[at] : elem_f32<Tag>(p.loc, at);
        rows[r * row_len + e] = (float)(_Float16)v;
      }
      for (int i = lane; i < nrow * LK; i += kWave) {
        const int r = fdiv20(i, inv_lk), e = i - r * LK;
        rows[r * row_len + 2 * LK + e] = elem_f32<Tag>(p.logits, ((size_t)(row0 + r) * p.G + g) * LK + e);
      }
    }
    __builtin_amdgcn_wave_barrier();
    if (lr >= nrow || chunk >= p.lanes.tpg) continue;
    const float *s = rows + lr * row_len;
    float mx, inv;
    float acc[CPT];
#pragma unroll
    for (int c = 0; c < CPT; ++c) acc[c] = 0.f;
    if constexpr (QUAD) {
      const int my_k = chunk & 3;
      quad_softmax_stats(s + 2 * LK, LK, my_k, mx, inv);
      for (int l = 0; l < p.L; ++l) {
        const Level lv = load_level(p, l);
        const int off = s_level_off[l];
        const bool staged = off >= 0;
        const uint32_t base = staged ? (uint32_t)off : (uint32_t)(b * p.N + lv.start) * pix_bytes + (uint32_t)g * head_bytes;
        fda_quad_level<Tag, CPT>(acc, s, LK, K, l, lv, mx, inv, base, staged ? head_bytes : pix_bytes, lane_off, my_k, staged,
                                 s_stage, value);
      }
    } else {
      softmax_stats(s + 2 * LK, LK, mx, inv);
      for (int l = 0; l < p.L; ++l) {
        const Level lv = load_level(p, l);
        const int off = s_level_off[l];
        const bool staged = off >= 0;
        // staged: byte offsets into the stage area, a corner outside the level reads the zero bytes at its start
        const uint32_t base =
            (staged ? (uint32_t)off : (uint32_t)(b * p.N + lv.start) * pix_bytes + (uint32_t)g * head_bytes) + lane_off;
        const uint32_t step = staged ? head_bytes : pix_bytes;
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const int t = l * K + k;
          const float x = sub_rn(mul_rn(s[2 * t], (float)lv.W), 0.5f);       // flash_deform_im2col_cuda.cuh:188-189
          const float y = sub_rn(mul_rn(s[2 * t + 1], (float)lv.H), 0.5f);
          const float pr = __expf(s[2 * LK + t] - mx) * inv;
          const Tap tp = make_tap(y, x, lv.H, lv.W, base, step);
          typename pack::raw_t raw[4];
          if (staged) {
#pragma unroll
            for (int cn = 0; cn < 4; ++cn)
              raw[cn] = *reinterpret_cast<const typename pack::raw_t *>(s_stage + ((tp.valid >> cn) & 1u ? tp.off[cn] : 0u));
          } else {
#pragma unroll
            for (int cn = 0; cn < 4; ++cn) raw[cn] = buffer_load<pack::kBytes>(value, tp.off[cn]);
          }
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) {
            float v[CPT];
            pack::decode(raw[cn], v);
            const float w = pr * tp.w[cn];
#pragma unroll
            for (int c = 0; c < CPT; ++c) acc[c] = fmaf(w, v[c], acc[c]);
          }
        }
      }
    }
    char *dst = (char *)p.out + ((size_t)(row0 + lr) * (p.G * p.D) + g * p.D + chunk * CPT) * Tag::kBytes;
    *reinterpret_cast<typename pack::raw_t *>(dst) = pack::encode(acc);
  }
}

// ------------------------------------------------------------------------------- backward
// One kernel body, three roles (FdaBackwardMode):
//   kFdaFull       grad_sampling_loc_attn, and grad_value scattered with fp32 buffer atomics into a
//                  cleared fp32 image (any head width)
//   kFdaNoScatter  grad_sampling_loc_attn, plus what the tiled grad_value kernel needs: per sampling point a key
//                  and a (position, softmax probability) record, and grad_out regrouped by head
//   kFdaFallback   exits at once unless the binning kernel flagged a level it cannot hold; then it scatters
//                  with fp32 atomics into an fp32 image (grad_value itself for fp32 tensors, left zeroed by the tiled kernel)
template <typename Tag, int CPT, int KT, int MODE, bool QUAD>      // QUAD: only with kFdaNoScatter
__global__ void __launch_bounds__(kFdaBackwardThreads) fda_backward_kernel(const FdaLaunch p) {
  extern __shared__ float lds[];
  typedef Pack<Tag, CPT> pack;
  if constexpr (MODE == kFdaFallback) {
    if (p.state->reserved == 0u) return;
  }
  if constexpr (MODE == kFdaNoScatter) {
    // the first kernel of the tiled backward clears the state block for the kernels behind it (nobody reads it before
    // this kernel has ended); with several launches per call only the first one does
    if (p.clear_state && blockIdx.x == 0 && threadIdx.x < sizeof(GradState) / sizeof(uint32_t))
      reinterpret_cast<uint32_t *>(p.state)[threadIdx.x] = 0u;
  }
  const int LK = p.L * p.K, row_len = 3 * LK;
  const uint32_t blk = xcd_contiguous_block(blockIdx.x, gridDim.x);
  int row0, nrow, heads_here = p.G, g_fixed = 0;
  if (p.head_major) {       // one head per workgroup, workgroups ordered [image][head][block of queries] (see the forward kernel)
    const int blocks_per_image = (p.Q + p.nq_block - 1) / p.nq_block;
    const int rb = (int)(blk % (uint32_t)blocks_per_image), bg = (int)(blk / (uint32_t)blocks_per_image);
    const int b = bg / p.G;
    g_fixed = bg - b * p.G;
    heads_here = 1;
    const int q0 = rb * p.nq_block;
    nrow = min(p.nq_block, p.Q - q0);
    row0 = b * p.Q + q0;
  } else {
    row0 = (int)blk * p.nq_block;
    nrow = min(p.nq_block, p.n_row - row0);
  }
  float *s_in = lds, *s_grad = lds + p.nq_block * heads_here * row_len;
  fda_stage_rows<Tag>(s_in, p, row0, nrow, g_fixed, heads_here);
  __syncthreads();      // every slot of s_grad is written below: no clearing needed

  const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);
  const __amdgpu_buffer_rsrc_t gacc = make_rsrc(p.grad_value_acc, p.value_bytes / Tag::kBytes * 4);
  const int tpgp_log2 = p.lanes.tpgp_log2, width = 1 << tpgp_log2;
  const int items = (nrow * heads_here) << tpgp_log2;
  const uint32_t pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
  const int K = KT > 0 ? KT : p.K;
  const size_t key_stride = fda_key_stride(p.Q, K);

  for (int it = threadIdx.x; it < items; it += blockDim.x) {
    const int chunk = it & (width - 1);
    const bool active = chunk < p.lanes.tpg;
    const int rg = it >> tpgp_log2;
    const int lr = rg / heads_here, g = g_fixed + rg - lr * heads_here;
    const int b = (row0 + lr) / p.Q;
    const float *s = s_in + rg * row_len;
    float *gs = s_grad + rg * row_len;
    float mx, inv;
    if constexpr (QUAD) quad_softmax_stats(s + 2 * LK, LK, chunk & 3, mx, inv);
    else softmax_stats(s + 2 * LK, LK, mx, inv);
    const uint32_t lane_base = (uint32_t)(g * p.D + (active ? chunk : 0) * CPT) * Tag::kBytes;

    float go[CPT];
    {
      const char *src = (const char *)p.grad_out + ((size_t)(row0 + lr) * (p.G * p.D)) * Tag::kBytes + lane_base;
      pack::decode(__builtin_nontemporal_load(reinterpret_cast<const typename pack::raw_t *>(src)), go);
      if (!active) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) go[c] = 0.f;
      }
    }
    float dot_rg = 0.f;
    const int b_local = (row0 + lr) / p.Q, q = (row0 + lr) - b_local * p.Q;
    if constexpr (MODE == kFdaNoScatter) {      // grad_out regrouped by head: the grad_value kernel gathers rows of one head at a time
      if (active) {
        char *dst = (char *)p.go_rows + ((((size_t)b_local * p.G + g) * p.Q + q) * p.D + chunk * CPT) * Tag::kBytes;
        __builtin_nontemporal_store(pack::encode(go), reinterpret_cast<typename pack::raw_t *>(dst));
      }
    }

    if constexpr (QUAD) {      // every lane of the cluster is active; the first quad writes the gradient slots
      const int my_k = chunk & 3;
      const uint32_t lane_off = (uint32_t)(chunk * CPT) * Tag::kBytes;
      for (int l = 0; l < p.L; ++l) {
        const Level lv = load_level(p, l);
        const uint32_t base = (uint32_t)(b * p.N + lv.start) * pix_bytes + (uint32_t)(g * p.D) * Tag::kBytes;
        const size_t slot = (((size_t)b_local * p.G + g) * p.L + l) * key_stride + (size_t)q * K;
        dot_rg += fda_quad_level_backward<Tag, CPT>(go, s, gs, LK, K, l, lv, mx, inv, base, pix_bytes, lane_off, my_k, width,
                                                    chunk < 4, value, p.keys + slot, p.recs + slot);
      }
      dot_rg += dpp_quad_xor1(dot_rg);
      dot_rg += dpp_quad_xor2(dot_rg);
      if (chunk < 4) {
        for (int t = my_k; t < LK; t += 4) {      // the lane's own points
          const float pr = __expf(s[2 * LK + t] - mx) * inv;
          gs[2 * LK + t] = pr * (gs[2 * LK + t] - dot_rg);
        }
      }
      continue;
    }
    for (int l = 0; l < p.L; ++l) {
      const Level lv = load_level(p, l);
      const uint32_t base = (uint32_t)(b * p.N + lv.start) * pix_bytes + lane_base;
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const int t = l * K + k;
        const float x = sub_rn(mul_rn(s[2 * t], (float)lv.W), 0.5f);
        const float y = sub_rn(mul_rn(s[2 * t + 1], (float)lv.H), 0.5f);
        const float pr = __expf(s[2 * LK + t] - mx) * inv;
        Tap tp = make_tap(y, x, lv.H, lv.W, base, pix_bytes);
        if (!active) {
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) tp.off[cn] = kDropOffset;
        }
        if constexpr (MODE == kFdaFallback) {      // fp32 atomics into the fp32 image (the tensor itself for fp32 tensors)
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) {
            const float w = pr * tp.w[cn];
            const uint32_t aoff = (tp.off[cn] == kDropOffset) ? kDropOffset : tp.off[cn] * (4 / Tag::kBytes);
#pragma unroll
            for (int c = 0; c < CPT; ++c)
              __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(go[c] * w, gacc, aoff + 4 * c, 0, 0);
          }
          continue;
        }
        typename pack::raw_t raw[4];
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) raw[cn] = buffer_load<pack::kBytes>(value, tp.off[cn]);
        float dots[4];
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          float v[CPT];
          pack::decode(raw[cn], v);
          float d = 0.f;
#pragma unroll
          for (int c = 0; c < CPT; ++c) d = fmaf(v[c], go[c], d);
          dots[cn] = d;
          if constexpr (MODE == kFdaFull) {
            const float w = pr * tp.w[cn];
            const uint32_t aoff = (tp.off[cn] == kDropOffset) ? kDropOffset : tp.off[cn] * (4 / Tag::kBytes);
#pragma unroll
            for (int c = 0; c < CPT; ++c)
              __builtin_amdgcn_raw_ptr_buffer_atomic_fadd_f32(go[c] * w, gacc, aoff + 4 * c, 0, 0);
          }
        }
        const float hy = 1.f - tp.ly, hx = 1.f - tp.lx;
        float gx = hy * (dots[1] - dots[0]) + tp.ly * (dots[3] - dots[2]);
        float gy = hx * (dots[2] - dots[0]) + tp.lx * (dots[3] - dots[1]);
        float gz = tp.w[0] * dots[0] + tp.w[1] * dots[1] + tp.w[2] * dots[2] + tp.w[3] * dots[3];
        gx = cluster_sum(gx, width);
        gy = cluster_sum(gy, width);
        gz = cluster_sum(gz, width);
        if (chunk == 0) {
          gs[2 * t] = gx * (float)lv.W * pr;          // flash_deform_col2im_cuda.cuh:273-276
          gs[2 * t + 1] = gy * (float)lv.H * pr;
          gs[2 * LK + t] = gz;
        }
        dot_rg = fmaf(pr, gz, dot_rg);
      }
    }
    if (MODE != kFdaFallback && chunk == 0) {
      for (int t = 0; t < LK; ++t) {
        const float pr = __expf(s[2 * LK + t] - mx) * inv;
        gs[2 * LK + t] = pr * (gs[2 * LK + t] - dot_rg);
        // the probability takes the logit's place for the record pass below (only this wave reads the row, and its
        // lanes are past the tap loop)
        if constexpr (MODE == kFdaNoScatter) const_cast<float *>(s)[2 * LK + t] = pr;
      }
    }
  }
  if constexpr (MODE == kFdaFallback) return;
  __syncthreads();
  if constexpr (MODE == kFdaNoScatter && !QUAD) {
    // Keys and records of the workgroup's sampling points, one lane per point in the order they lie in memory
    // ([head][level][query][point]: whole 16-byte records side by side), from the staged rows.
    for (int hl = 0; hl < heads_here * p.L; ++hl) {
      const int gh = hl / p.L, l = hl - gh * p.L, g = g_fixed + gh;
      const Level lv = load_level(p, l);
      for (int i = threadIdx.x; i < nrow * K; i += blockDim.x) {
        const int lr = i / K, k = i - lr * K, t = l * K + k;
        const float *s = s_in + (lr * heads_here + gh) * row_len;
        const float x = sub_rn(mul_rn(s[2 * t], (float)lv.W), 0.5f);
        const float y = sub_rn(mul_rn(s[2 * t + 1], (float)lv.H), 0.5f);
        const Tap tp = make_tap(y, x, lv.H, lv.W, 0u, 0u);
        uint32_t key = kFdaKeyOutside;
        if (tp.valid != 0)
          key = (tp.y0 + 1 >= kFdaKeyFieldMax || tp.x0 + 1 >= kFdaKeyFieldMax) ? kFdaKeySaturated
                                                                              : ((uint32_t)(tp.y0 + 1) << 8) | (uint32_t)(tp.x0 + 1);
        const int b_local = (row0 + lr) / p.Q, q = (row0 + lr) - b_local * p.Q;
        const size_t slot = (((size_t)b_local * p.G + g) * p.L + l) * key_stride + (size_t)q * K + k;
        p.keys[slot] = (uint16_t)key;
        p.recs[slot] = f32x4_t{x, y, s[2 * LK + t], 0.f};
      }
    }
  }
  fda_unstage_grads<Tag>(s_grad, p, row0, nrow, g_fixed, heads_here);
}

// Lanes of a (query, head) fill whole quads and the points come in fours: the lanes of a quad share the set-up.
bool fda_quad_setup(const FdaLaunch &p) {
  return (p.K % 4) == 0 && p.lanes.tpg >= 4 && p.lanes.tpg == (1 << p.lanes.tpgp_log2);
}

template <typename Tag, int CPT>
hipError_t launch_staged(const FdaLaunch &p, hipStream_t stream) {
  const dim3 grid((unsigned)((p.n_row / p.Q) * p.G * p.stage_blocks)), block(kFdaStagedThreads);
  const size_t lds = (size_t)(kFdaStagedThreads >> p.lanes.tpgp_log2) * 3 * p.L * p.K * sizeof(float) + (size_t)p.stage_budget;
  auto go = [&](auto kernel) -> hipError_t {
    if (hipError_t e = ensure_dynamic_lds_limit(reinterpret_cast<const void *>(kernel), kMaxLdsPerWorkgroup - 1024)) return e;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return hipGetLastError();
  };
  if (fda_quad_setup(p)) return go(fda_forward_staged_kernel<Tag, CPT, 0, true>);
  if (p.K == 4) return go(fda_forward_staged_kernel<Tag, CPT, 4, false>);
  return go(fda_forward_staged_kernel<Tag, CPT, 0, false>);      // (unrolled for 8 points the kernel spills a hundred registers)
}

template <typename Tag, int CPT, int MODE>      // MODE -1: forward
hipError_t launch_k(const FdaLaunch &p, hipStream_t stream, dim3 grid, dim3 block, size_t lds) {
  if constexpr (MODE < 0) {
    if (p.stage_budget > 0) return launch_staged<Tag, CPT>(p, stream);
  }
#define FDA_LAUNCH(KT)                                                                                     \
  do {                                                                                                     \
    if constexpr (MODE >= 0) hipLaunchKernelGGL((fda_backward_kernel<Tag, CPT, KT, MODE, false>), grid, block, lds, stream, p); \
    else hipLaunchKernelGGL((fda_forward_kernel<Tag, CPT, KT, false>), grid, block, lds, stream, p);       \
  } while (0)
  if constexpr (MODE < 0) {
    if (fda_quad_setup(p)) {
      hipLaunchKernelGGL((fda_forward_kernel<Tag, CPT, 0, true>), grid, block, lds, stream, p);
      return hipGetLastError();
    }
  }
  if constexpr (MODE == kFdaNoScatter) {
    if (fda_quad_setup(p)) {
      hipLaunchKernelGGL((fda_backward_kernel<Tag, CPT, 0, MODE, true>), grid, block, lds, stream, p);
      return hipGetLastError();
    }
  }
  if (p.K == 4) FDA_LAUNCH(4);
  else if (p.K == 8) FDA_LAUNCH(8);
  else FDA_LAUNCH(0);
#undef FDA_LAUNCH
  return hipGetLastError();
}

template <typename Tag, int MODE>
hipError_t launch_by_cpt(const FdaLaunch &p, hipStream_t stream) {
  const bool head_major = p.head_major != 0;
  const dim3 grid(head_major ? (unsigned)((p.n_row / p.Q) * p.G * ((p.Q + p.nq_block - 1) / p.nq_block))
                             : (unsigned)((p.n_row + p.nq_block - 1) / p.nq_block)),
      // one head per workgroup: as many lanes as its queries fill (long rows leave the LDS room for fewer queries)
      block(head_major && (MODE == kFdaNoScatter || MODE < 0)
                ? (unsigned)std::min(MODE < 0 ? kFdaForwardThreads : kFdaBackwardThreads,
                                     ((p.nq_block << p.lanes.tpgp_log2) + kWave - 1) / kWave * kWave)
                : (unsigned)kBlockThreads);
  const size_t lds = MODE >= 0 ? fda_backward_lds_bytes(p) : fda_forward_lds_bytes(p);
#define FDA_CASE(N)                                                                       \
  case N:                                                                                 \
    if constexpr (N * Tag::kBytes <= 16) return launch_k<Tag, N, MODE>(p, stream, grid, block, lds); \
    break;
  switch (p.lanes.cpt) {
    FDA_CASE(1) FDA_CASE(2) FDA_CASE(4) FDA_CASE(8)
  }
#undef FDA_CASE
  return hipErrorInvalidValue;
}

template <int MODE> hipError_t launch_by_dtype(int dtype, const FdaLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_by_cpt<F32, MODE>(p, stream);
    case F16::kCode: return launch_by_cpt<F16, MODE>(p, stream);
    case BF16::kCode: return launch_by_cpt<BF16, MODE>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

size_t fda_forward_lds_bytes(const FdaLaunch &p) {
  return (size_t)p.nq_block * (p.head_major ? 1 : p.G) * 3 * p.L * p.K * sizeof(float);
}
size_t fda_backward_lds_bytes(const FdaLaunch &p) { return 2 * fda_forward_lds_bytes(p); }

hipError_t launch_fda_forward(int dtype, const FdaLaunch &p, hipStream_t stream) {
  return launch_by_dtype<-1>(dtype, p, stream);
}
hipError_t launch_fda_backward(int dtype, const FdaLaunch &p, int mode, hipStream_t stream) {
  switch (mode) {
    case kFdaFull: return launch_by_dtype<kFdaFull>(dtype, p, stream);
    case kFdaNoScatter: return launch_by_dtype<kFdaNoScatter>(dtype, p, stream);
    case kFdaFallback: return launch_by_dtype<kFdaFallback>(dtype, p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
