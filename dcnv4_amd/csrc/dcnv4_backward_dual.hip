// DCNv4 backward as ONE launch with two workgroup roles.
//
// When a grad_value tile is a whole image, the two kernels of the backward - grad_offset_mask from the staged window
// (dcnv4_tiled_gather.hpp) and grad_value as an anchor-owned gather (dcnv4_grad_value.hpp) - do not depend on each
// other: the grad_value workgroups visit every output pixel whatever the reach the first kernel measures.  On the
// small stages (14x14, 7x7 images: a few hundred workgroups, 15-20 us per kernel of which a quarter is the fixed cost
// of a dispatch) the two launches run back to back with the chip half empty.  Here both kinds of workgroup share one
// grid: when it is small enough to be resident at once, every 16 consecutive workgroup ids hold 8 workgroups of each
// role, so that both roles are on every CU together and a role's k-th workgroup still runs on XCD k % 8 (the order
// both bodies assume for their L2 locality); a larger grid holds one role after the other, which still saves a
// dispatch and lets the second role start while the first one's last workgroups finish.  The bodies are the kernels'
// own, unchanged: identical bits.
// Reference for the two roles: DCNv4_op/src/cuda/dcnv4_col2im_cuda.cuh:196-366 (one kernel there, with atomics).
#include "dcnv4_grad_value.hpp"
#include "dcnv4_tiled_gather.hpp"

namespace dcn {
namespace {

constexpr int kDualThreads = 512;

// Role and number within its role of workgroup `bid`: n1 workgroups of the first role, n2 of the second.
__device__ __forceinline__ bool dual_first_role(uint32_t bid, uint32_t n1, uint32_t n2, uint32_t &local, bool interleave) {
  const uint32_t m = interleave ? min(n1, n2) & ~7u : 0u;           // interleaved in eights while both roles last
  if (bid < 2u * m) {
    const uint32_t r = bid & 15u;
    local = (bid >> 4) * 8u + (r & 7u);
    return r < 8u;
  }
  const uint32_t e = bid - 2u * m, rest1 = n1 - m;
  const bool first = e < rest1;
  local = m + (first ? e : e - rest1);
  return first;
}

template <typename Tag, int NV, bool PAIR>
__global__ void __launch_bounds__(kDualThreads, 4) dcnv4_backward_dual_kernel(const DcnLaunch p, uint32_t n1, uint32_t n2, int interleave) {
  uint32_t local;
  if (dual_first_role(blockIdx.x, n1, n2, local, interleave != 0)) dcnv4_offset_mask_grad_tiled_body<Tag, NV, 9, PAIR>(p, local, n1);
  else dcnv4_grad_value_body<Tag, 9, 16, kGradValueColumnRounds, kDualThreads>(p, local, n2);
}

// workgroups of the two roles for n_img images
void role_counts(const DcnLaunch &p, int n_img, uint32_t *n1, uint32_t *n2) {
  const int Ho = p.Q / p.Wo;
  *n1 = (uint32_t)(n_img * ((Ho + p.gt_h - 1) / p.gt_h) * ((p.Wo + p.gt_w - 1) / p.gt_w) * ((p.G + p.gt_ng - 1) / p.gt_ng));
  *n2 = (uint32_t)(n_img * ((p.H + p.tile_h - 1) / p.tile_h) * ((p.W + p.tile_w - 1) / p.tile_w) * ((p.G + p.ng_chunk - 1) / p.ng_chunk));
}

template <typename Tag>
hipError_t launch_t(const DcnLaunch &p, hipStream_t stream) {
  uint32_t n1, n2;
  role_counts(p, p.n_img, &n1, &n2);
  const size_t lds = std::max(dcnv4_tiled_gather_lds_bytes(p, Tag::kBytes), dcnv4_grad_value_lds_bytes(p));
  auto go = [&](auto kernel) -> hipError_t {
    if (hipError_t e = ensure_dynamic_lds_limit(reinterpret_cast<const void *>(kernel), kMaxLdsPerWorkgroup - 1024)) return e;
    hipLaunchKernelGGL(kernel, dim3(n1 + n2), dim3(kDualThreads), lds, stream, p, n1, n2, p.dual_interleave);
    return hipGetLastError();
  };
  const bool pair = p.gt_lpg == 2;
  switch (p.D * Tag::kBytes / 16 / p.gt_lpg) {      // 16-byte vectors per lane of the first role
    case 1: return go(dcnv4_backward_dual_kernel<Tag, 1, false>);
    case 2: return pair ? go(dcnv4_backward_dual_kernel<Tag, 2, true>) : go(dcnv4_backward_dual_kernel<Tag, 2, false>);
    case 4: return pair ? go(dcnv4_backward_dual_kernel<Tag, 4, true>) : go(dcnv4_backward_dual_kernel<Tag, 4, false>);
  }
  return hipErrorInvalidValue;
}

}  // namespace

// The launch plans (tiled gather and grad_value, both in p) suit the two-role kernel: a 3x3 kernel with its centre, whole
// images as grad_value tiles in 512-lane workgroups, at most 64 channels a lane pair in the first role, 512 lanes there too.
bool dcnv4_backward_dual_fits(const DcnLaunch &p, int elem_bytes) {
  if (!p.gv_whole || p.gt_h == 0 || p.softmax || p.kh != 3 || p.kw != 3 || p.remove_center) return false;
  if (p.gv_threads != kDualThreads || p.gv_cw != 16) return false;
  if (p.gt_h * p.gt_w * p.gt_ng * p.gt_lpg > kDualThreads) return false;
  const int nv = p.D * elem_bytes / 16 / p.gt_lpg;
  if (p.D * elem_bytes % (16 * p.gt_lpg) != 0 || !(nv == 1 || nv == 2 || nv == 4)) return false;
  if (nv == 1 && p.gt_lpg != 1) return false;      // the one-vector instantiation is built for one lane per (pixel, group)
  return std::max(dcnv4_tiled_gather_lds_bytes(p, elem_bytes), dcnv4_grad_value_lds_bytes(p)) <= kMaxLdsPerWorkgroup / 2 - 512;
}

// Workgroups of both roles together, for n_img images.  Few enough to be resident (nearly) all at once, two per CU, and
// the roles are interleaved and overlap (batch 64, 7x7 images of 32 groups, 512 / 704 workgroups: 30.8 -> 21.7 us fp16,
// 32.3 -> 27.5 us fp32); more, and interleaving only slows both roles down (14x14 images of 16 groups, 1024 / 1536
// workgroups: 41.4 -> 41.4 us, 46.1 -> 50.0 us), while one role after the other in the same grid still saves a dispatch
// and the first role's tail (38.2 us, 45.4 us).
uint32_t dcnv4_backward_dual_workgroups(const DcnLaunch &p, int n_img) {
  uint32_t n1, n2;
  role_counts(p, n_img, &n1, &n2);
  return n1 + n2;
}

hipError_t launch_dcnv4_backward_dual(int dtype, const DcnLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_t<F32>(p, stream);
    case F16::kCode: return launch_t<F16>(p, stream);
    case BF16::kCode: return launch_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
