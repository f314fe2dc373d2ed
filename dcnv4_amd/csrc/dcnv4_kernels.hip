// DCNv4 deformable-convolution kernels for gfx950 (wave64).
//
// Replaces the reference's forward_kernel_dcn_reg (DCNv4_op/src/cuda/dcnv4_im2col_cuda.cuh:142-244)
// and backward_kernel_dcn_warp_primitive (DCNv4_op/src/cuda/dcnv4_col2im_cuda.cuh:196-366).
//
// Work decomposition: a workgroup owns `npix_block` consecutive output pixels (all groups).
// Its offset_mask rows are one contiguous span of memory: they are streamed once with 128-bit
// loads into LDS (as fp32) and shared by every channel lane.  One lane owns `cpt` contiguous
// channels of one (pixel, group) - 16 bytes - so the lanes of a (pixel, group) form one
// contiguous D*s-byte segment per gathered corner and the output store of a wave is one
// contiguous kilobyte.  Corners outside the image are range-dropped by the buffer descriptor.
// Backward: coordinate / modulation partials are summed over the lanes of a (pixel, group) with
// DPP, parked in LDS and written back as whole rows (padding tail included, so the gradient
// tensor needs no separate clearing); the value gradient is the tiled gather of dcnv4_grad_value.hip.
#include <algorithm>

#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

struct PixelGeom {
  float x_base, y_base;   // tap (0,0) position before the learned offset, dcnv4_im2col_cuda.cuh:203-210
  uint32_t img_base;      // byte offset of this image + this lane's channels
};

template <typename Tag>
__device__ __forceinline__ PixelGeom pixel_geometry(const DcnLaunch &p, int pix, int g, int chunk) {
  const int b = pix / p.Q, q = pix - b * p.Q;
  const int ho = q / p.Wo, wo = q - ho * p.Wo;
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;
  PixelGeom geo;
  geo.x_base = sub_rn((float)(half_w - p.pw + wo * p.sw), mul_rn((float)half_w, p.offset_scale));
  geo.y_base = sub_rn((float)(half_h - p.ph + ho * p.sh), mul_rn((float)half_h, p.offset_scale));
  geo.img_base = ((uint32_t)b * (uint32_t)(p.H * p.W) * (uint32_t)(p.G * p.D) +
                  (uint32_t)(g * p.D + chunk * p.lanes.cpt)) * Tag::kBytes;
  return geo;
}

// ------------------------------------------------------------------------------- forward
template <typename Tag, int CPT, int KP>
__global__ void __launch_bounds__(kBlockThreads) dcnv4_forward_kernel(const DcnLaunch p) {
  extern __shared__ float lds[];
  typedef Pack<Tag, CPT> pack;
  const uint32_t blk = xcd_contiguous_block(blockIdx.x, gridDim.x);
  const int pix0 = (int)blk * p.npix_block;
  const int npix = min(p.npix_block, p.n_pix - pix0);
  const bool vec16 = (p.P_pad * Tag::kBytes) % 16 == 0;
  stage_rows_to_lds<Tag>(lds, (const char *)p.offset_mask + (size_t)pix0 * p.P_pad * Tag::kBytes,
                         npix * p.P_pad, vec16);
  __syncthreads();

  const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);
  const int tpgp_log2 = p.lanes.tpgp_log2;
  const int items = (npix * p.G) << tpgp_log2;
  const uint32_t pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
  const int Kp = p.Kp;

  for (int it = threadIdx.x; it < items; it += blockDim.x) {
    const int chunk = it & ((1 << tpgp_log2) - 1);
    if (chunk >= p.lanes.tpg) continue;
    const int pg = it >> tpgp_log2;
    const int lp = pg / p.G, g = pg - lp * p.G;
    const PixelGeom geo = pixel_geometry<Tag>(p, pix0 + lp, g, chunk);
    const float *om = lds + lp * p.P_pad + g * 3 * Kp;
    float mx = 0.f, inv = 1.f;
    if (p.softmax) softmax_stats(om + 2 * Kp, Kp, mx, inv);

    float acc[CPT];
#pragma unroll
    for (int c = 0; c < CPT; ++c) acc[c] = 0.f;

    auto one_tap = [&](int k, int i, int j) {
      const float x = add_rn(geo.x_base, mul_rn(add_rn((float)(i * p.dw), om[2 * k]), p.offset_scale));
      const float y = add_rn(geo.y_base, mul_rn(add_rn((float)(j * p.dh), om[2 * k + 1]), p.offset_scale));
      float m = om[2 * Kp + k];
      if (p.softmax) m = __expf(m - mx) * inv;
      const Tap t = make_tap(y, x, p.H, p.W, geo.img_base, pix_bytes);
      typename pack::raw_t raw[4];
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) raw[cn] = buffer_load<pack::kBytes>(value, t.off[cn]);
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        float v[CPT];
        pack::decode(raw[cn], v);
        const float w = m * t.w[cn];
#pragma unroll
        for (int c = 0; c < CPT; ++c) acc[c] = fmaf(w, v[c], acc[c]);
      }
    };

    if constexpr (KP > 0) {
#pragma unroll
      for (int k = 0; k < KP; ++k) {
        int i, j;
        tap_ij_3x3(KP, k, i, j);
        one_tap(k, i, j);
      }
    } else {
      int k = 0;
      for (int i = 0; i < p.kw; ++i)
        for (int j = 0; j < p.kh; ++j) {
          if (p.remove_center && i == p.kw / 2 && j == p.kh / 2) continue;
          one_tap(k, i, j);
          ++k;
        }
    }

    char *dst = (char *)p.out + ((size_t)(pix0 + lp) * (p.G * p.D) + g * p.D + chunk * CPT) * Tag::kBytes;
    *reinterpret_cast<typename pack::raw_t *>(dst) = pack::encode(acc);
  }
}

// ------------------------------------------------------------------------------- backward
// grad_offset_mask for any group width (the part of dcnv4_col2im_cuda.cuh:280-350 and common.h:188-211 that does not
// scatter), plus the reach the grad_value kernel has to cover.
template <typename Tag, int CPT, int KP>
__global__ void __launch_bounds__(kBlockThreads) dcnv4_offset_mask_grad_kernel(const DcnLaunch p) {
  extern __shared__ float lds[];
  typedef Pack<Tag, CPT> pack;
  const bool vec16 = (p.P_pad * Tag::kBytes) % 16 == 0;
  float *s_om = lds, *s_grad = lds + p.npix_block * p.P_pad;
  uint32_t reach_needed = 0;
  const uint32_t blk = xcd_contiguous_block(blockIdx.x, gridDim.x);
  const int pix0 = (int)blk * p.npix_block;
  const int npix = min(p.npix_block, p.n_pix - pix0);
  stage_rows_to_lds<Tag>(s_om, (const char *)p.offset_mask + (size_t)pix0 * p.P_pad * Tag::kBytes,
                         npix * p.P_pad, vec16);
  for (int i = threadIdx.x; i < npix * p.P_pad; i += blockDim.x) s_grad[i] = 0.f;
  __syncthreads();

  const __amdgpu_buffer_rsrc_t value = make_rsrc(p.value, p.value_bytes);
  const int tpgp_log2 = p.lanes.tpgp_log2, width = 1 << tpgp_log2;
  const int items = (npix * p.G) << tpgp_log2;
  const uint32_t pix_bytes = (uint32_t)(p.G * p.D) * Tag::kBytes;
  const int Kp = p.Kp;
  const int half_w = (p.dw * (p.kw - 1)) >> 1, half_h = (p.dh * (p.kh - 1)) >> 1;

  for (int it = threadIdx.x; it < items; it += blockDim.x) {
    const int chunk = it & (width - 1);
    const bool active = chunk < p.lanes.tpg;       // false only on padding lanes of a non-2^n cluster
    const int pg = it >> tpgp_log2;
    const int lp = pg / p.G, g = pg - lp * p.G;
    const int pix = pix0 + lp;
    const PixelGeom geo = pixel_geometry<Tag>(p, pix, g, active ? chunk : 0);
    const float *om = s_om + lp * p.P_pad + g * 3 * Kp;
    float *gom = s_grad + lp * p.P_pad + g * 3 * Kp;
    float mx = 0.f, inv = 1.f;
    if (p.softmax) softmax_stats(om + 2 * Kp, Kp, mx, inv);
    // reference point of this output pixel (centre tap at zero offset)
    const int q = pix % p.Q;
    const int p0y = half_h - p.ph + (q / p.Wo) * p.sh, p0x = half_w - p.pw + (q % p.Wo) * p.sw;

    float go[CPT];
    {
      const char *src = (const char *)p.grad_out +
                        ((size_t)pix * (p.G * p.D) + g * p.D + (active ? chunk : 0) * CPT) * Tag::kBytes;
      pack::decode(*reinterpret_cast<const typename pack::raw_t *>(src), go);
      if (!active) {
#pragma unroll
        for (int c = 0; c < CPT; ++c) go[c] = 0.f;
      }
    }
    float dot_pg = 0.f;     // sum_k p_k * gz_k, softmax Jacobian only

    auto one_tap = [&](int k, int i, int j) {
      const float x = add_rn(geo.x_base, mul_rn(add_rn((float)(i * p.dw), om[2 * k]), p.offset_scale));
      const float y = add_rn(geo.y_base, mul_rn(add_rn((float)(j * p.dh), om[2 * k + 1]), p.offset_scale));
      float m = om[2 * Kp + k];
      if (p.softmax) m = __expf(m - mx) * inv;
      Tap t = make_tap(y, x, p.H, p.W, geo.img_base, pix_bytes);
      if (!active) {
        t.valid = 0;
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) t.off[cn] = kDropOffset;
      }
      {
        if (t.valid != 0) {     // distance of the in-image part of the 2x2 corner block from the reference point;
          // a far row or column whose bilinear weight is exactly zero (integer coordinate) adds nothing and is left out
          const int y1 = t.y0 + (t.ly > 0.f ? 1 : 0), x1 = t.x0 + (t.lx > 0.f ? 1 : 0);
          const int d = max(max(p0y - max(t.y0, 0), min(y1, p.H - 1) - p0y),
                            max(p0x - max(t.x0, 0), min(x1, p.W - 1) - p0x));
          if ((float)d > p.gv_reach_cap) { if (chunk == 0) dcnv4_fold_far_point(p, pix / p.Q, g, t.y0, t.x0, p0y, p0x); }
          else reach_needed = max(reach_needed, (uint32_t)max(d, 0));
        }
      }
      typename pack::raw_t raw[4];
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) raw[cn] = buffer_load<pack::kBytes>(value, t.off[cn]);
      float dots[4];
#pragma unroll
      for (int cn = 0; cn < 4; ++cn) {
        float v[CPT];
        pack::decode(raw[cn], v);
        float d = 0.f;
#pragma unroll
        for (int c = 0; c < CPT; ++c) d = fmaf(v[c], go[c], d);
        dots[cn] = d;
      }
      const float hy = 1.f - t.ly, hx = 1.f - t.lx;
      float gx = hy * (dots[1] - dots[0]) + t.ly * (dots[3] - dots[2]);   // common.h:188-201
      float gy = hx * (dots[2] - dots[0]) + t.lx * (dots[3] - dots[1]);
      float gz = t.w[0] * dots[0] + t.w[1] * dots[1] + t.w[2] * dots[2] + t.w[3] * dots[3];
      gx = cluster_sum(gx, width);
      gy = cluster_sum(gy, width);
      gz = cluster_sum(gz, width);
      if (chunk == 0) {
        gom[2 * k] = gx * p.offset_scale * m;
        gom[2 * k + 1] = gy * p.offset_scale * m;
        gom[2 * Kp + k] = gz;
      }
      dot_pg = fmaf(m, gz, dot_pg);
    };

    if constexpr (KP > 0) {
#pragma unroll
      for (int k = 0; k < KP; ++k) {
        int i, j;
        tap_ij_3x3(KP, k, i, j);
        one_tap(k, i, j);
      }
    } else {
      int k = 0;
      for (int i = 0; i < p.kw; ++i)
        for (int j = 0; j < p.kh; ++j) {
          if (p.remove_center && i == p.kw / 2 && j == p.kh / 2) continue;
          one_tap(k, i, j);
          ++k;
        }
    }
    if (p.softmax && chunk == 0) {      // p_k (g_k - sum_j p_j g_j), dcnv4_col2im_cuda.cuh:352-365
      for (int k = 0; k < Kp; ++k) {
        const float pk = __expf(om[2 * Kp + k] - mx) * inv;
        gom[2 * Kp + k] = pk * (gom[2 * Kp + k] - dot_pg);
      }
    }
  }
  {
    // Same-address atomics retire slowly at the memory side: fold the workgroup's value in LDS first and only
    // touch the global word when it would actually grow.
    __shared__ uint32_t s_reach;
    if (threadIdx.x == 0) s_reach = 0u;
    __syncthreads();
    reach_needed = wave_max_u32(reach_needed);
    if ((threadIdx.x & (kWave - 1)) == 0 && reach_needed != 0) atomicMax(&s_reach, reach_needed);
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t *dst = &p.state->reach_needed;
      const uint32_t mine = s_reach;
      if (mine > __hip_atomic_load(dst, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(dst, mine);
    }
  }
  __syncthreads();
  unstage_rows_from_lds<Tag>((char *)p.grad_offset_mask + (size_t)pix0 * p.P_pad * Tag::kBytes, s_grad,
                             npix * p.P_pad, vec16);
}

template <typename Tag, int CPT>
hipError_t launch_fwd_k(const DcnLaunch &p, hipStream_t stream, dim3 grid, dim3 block, size_t lds) {
  const bool k3 = p.kh == 3 && p.kw == 3;
  if (k3 && !p.remove_center) hipLaunchKernelGGL((dcnv4_forward_kernel<Tag, CPT, 9>), grid, block, lds, stream, p);
  else if (k3 && p.remove_center) hipLaunchKernelGGL((dcnv4_forward_kernel<Tag, CPT, 8>), grid, block, lds, stream, p);
  else hipLaunchKernelGGL((dcnv4_forward_kernel<Tag, CPT, 0>), grid, block, lds, stream, p);
  return hipGetLastError();
}

template <typename Tag, int CPT>
hipError_t launch_bwd_k(const DcnLaunch &p, hipStream_t stream, dim3 grid, dim3 block, size_t lds) {
  const bool k3 = p.kh == 3 && p.kw == 3;
  if (k3 && !p.remove_center) hipLaunchKernelGGL((dcnv4_offset_mask_grad_kernel<Tag, CPT, 9>), grid, block, lds, stream, p);
  else if (k3 && p.remove_center) hipLaunchKernelGGL((dcnv4_offset_mask_grad_kernel<Tag, CPT, 8>), grid, block, lds, stream, p);
  else hipLaunchKernelGGL((dcnv4_offset_mask_grad_kernel<Tag, CPT, 0>), grid, block, lds, stream, p);
  return hipGetLastError();
}

template <typename Tag, bool BWD>
hipError_t launch_by_cpt(const DcnLaunch &p, hipStream_t stream) {
  const unsigned n_blocks = (unsigned)((p.n_pix + p.npix_block - 1) / p.npix_block);
  const dim3 grid(n_blocks), block(kBlockThreads);
  const size_t lds = BWD ? dcnv4_backward_lds_bytes(p) : dcnv4_forward_lds_bytes(p);
#define DCN_CASE(N)                                                              \
  case N:                                                                        \
    if constexpr (N * Tag::kBytes <= 16) {                                       \
      if constexpr (BWD) return launch_bwd_k<Tag, N>(p, stream, grid, block, lds); \
      else return launch_fwd_k<Tag, N>(p, stream, grid, block, lds);             \
    }                                                                            \
    break;
  switch (p.lanes.cpt) {
    DCN_CASE(1) DCN_CASE(2) DCN_CASE(4) DCN_CASE(8)
  }
#undef DCN_CASE
  return hipErrorInvalidValue;
}

template <bool BWD> hipError_t launch_by_dtype(int dtype, const DcnLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_by_cpt<F32, BWD>(p, stream);
    case F16::kCode: return launch_by_cpt<F16, BWD>(p, stream);
    case BF16::kCode: return launch_by_cpt<BF16, BWD>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

size_t dcnv4_forward_lds_bytes(const DcnLaunch &p) { return (size_t)p.npix_block * p.P_pad * sizeof(float); }
size_t dcnv4_backward_lds_bytes(const DcnLaunch &p) { return 2 * dcnv4_forward_lds_bytes(p); }

hipError_t launch_dcnv4_forward(int dtype, const DcnLaunch &p, hipStream_t stream) {
  return launch_by_dtype<false>(dtype, p, stream);
}
hipError_t launch_dcnv4_offset_mask_grad(int dtype, const DcnLaunch &p, hipStream_t stream) {
  return launch_by_dtype<true>(dtype, p, stream);
}

}  // namespace dcn
