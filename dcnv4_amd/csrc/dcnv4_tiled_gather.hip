// Kernels and launchers of the LDS-tiled gathers: DCNv4 forward and grad_offset_mask with the gather served from LDS
// (device code and its description: dcnv4_tiled_gather.hpp).
#include "dcnv4_tiled_gather.hpp"

namespace dcn {
namespace {

template <typename Tag, int NV, int KP, bool PAIR>
__global__ void __launch_bounds__(kTiledThreads) dcnv4_offset_mask_grad_tiled_kernel(const DcnLaunch p) {
  dcnv4_offset_mask_grad_tiled_body<Tag, NV, KP, PAIR>(p, blockIdx.x, gridDim.x);
}

template <typename Tag, int NV, bool BWD, bool PAIR>
hipError_t launch_nv(const DcnLaunch &p, hipStream_t stream, dim3 grid, dim3 block, size_t lds) {
  // the 3x3 instantiations know their lanes per (pixel, group) at compile time; the softmax variant lives in the
  // run-time-shape ones
  const bool k3 = p.kh == 3 && p.kw == 3 && !p.softmax && (PAIR || p.gt_lpg == 1);
  auto go = [&](auto kernel) -> hipError_t {
    // leaves room for the kernels' static LDS
    if (hipError_t e = ensure_dynamic_lds_limit(reinterpret_cast<const void *>(kernel), kMaxLdsPerWorkgroup - 1024)) return e;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return hipGetLastError();
  };
  if constexpr (BWD) {
    if (k3 && !p.remove_center) return go(dcnv4_offset_mask_grad_tiled_kernel<Tag, NV, 9, PAIR>);
    if (k3 && p.remove_center) return go(dcnv4_offset_mask_grad_tiled_kernel<Tag, NV, 8, PAIR>);
    return go(dcnv4_offset_mask_grad_tiled_kernel<Tag, NV, 0, false>);
  } else {
    if (k3 && !p.remove_center) return go(dcnv4_forward_tiled_kernel<Tag, NV, 9, PAIR>);
    if (k3 && p.remove_center) return go(dcnv4_forward_tiled_kernel<Tag, NV, 8, PAIR>);
    return go(dcnv4_forward_tiled_kernel<Tag, NV, 0, false>);
  }
}

template <typename Tag, bool BWD>
hipError_t launch_t(const DcnLaunch &p, hipStream_t stream) {
  const int Ho = p.Q / p.Wo;
  const int n_chunks = (p.G + p.gt_ng - 1) / p.gt_ng;
  const int nty = (Ho + p.gt_h - 1) / p.gt_h, ntx = (p.Wo + p.gt_w - 1) / p.gt_w;
  const int n_img = p.n_pix / p.Q;
  const dim3 grid((unsigned)(n_img * nty * ntx * n_chunks));
  const dim3 block((unsigned)((p.gt_h * p.gt_w * p.gt_ng * p.gt_lpg + kWave - 1) / kWave * kWave));
  const size_t lds = dcnv4_tiled_gather_lds_bytes(p, Tag::kBytes);
  const bool pair = p.gt_lpg == 2;      // two lanes per (pixel, group): they share the set-up of the sampling points
  switch (p.D * Tag::kBytes / 16 / p.gt_lpg) {      // 16-byte vectors per lane
    case 1: return launch_nv<Tag, 1, BWD, false>(p, stream, grid, block, lds);
    case 2: return pair ? launch_nv<Tag, 2, BWD, true>(p, stream, grid, block, lds) : launch_nv<Tag, 2, BWD, false>(p, stream, grid, block, lds);
    case 4: return pair ? launch_nv<Tag, 4, BWD, true>(p, stream, grid, block, lds) : launch_nv<Tag, 4, BWD, false>(p, stream, grid, block, lds);
    case 8: return launch_nv<Tag, 8, BWD, false>(p, stream, grid, block, lds);
  }
  return hipErrorInvalidValue;
}

template <bool BWD>
hipError_t launch_any(int dtype, const DcnLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_t<F32, BWD>(p, stream);
    case F16::kCode: return launch_t<F16, BWD>(p, stream);
    case BF16::kCode: return launch_t<BF16, BWD>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace

size_t dcnv4_tiled_gather_lds_bytes(const DcnLaunch &p, int elem_bytes) {
  const size_t cell = (size_t)p.gt_ng * p.D * elem_bytes + p.gt_pad;
  return (size_t)(p.gt_wh * p.gt_ww + p.gt_ww + 2) * cell +                     // window + zero cells
         (((size_t)p.gt_h * p.gt_w * p.gt_ng * 3 * p.Kp * elem_bytes + 15) & ~size_t(15));   // offset_mask slices
}

hipError_t launch_dcnv4_forward_tiled(int dtype, const DcnLaunch &p, hipStream_t stream) {
  return launch_any<false>(dtype, p, stream);
}

hipError_t launch_dcnv4_offset_mask_grad_tiled(int dtype, const DcnLaunch &p, hipStream_t stream) {
  return launch_any<true>(dtype, p, stream);
}

}  // namespace dcn
