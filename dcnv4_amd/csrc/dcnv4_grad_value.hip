// Kernel and launcher of the tiled grad_value pass of the DCNv4 backward (device code and its description:
// dcnv4_grad_value.hpp).
#include "dcnv4_grad_value.hpp"

namespace dcn {
namespace {

template <typename Tag, int KP, int CW, int ROUNDS, int NT>
__global__ void __launch_bounds__(NT) dcnv4_grad_value_kernel(const DcnLaunch p) {
  dcnv4_grad_value_body<Tag, KP, CW, ROUNDS, NT>(p, blockIdx.x, gridDim.x);
}

constexpr int gv_rounds(int kp) { return kp > 0 ? kGradValueColumnRounds : kGradValueRounds; }

template <typename Tag>
hipError_t launch_t(const DcnLaunch &p, hipStream_t stream) {
  const int n_chunks = (p.G + p.ng_chunk - 1) / p.ng_chunk;
  const int nty = (p.H + p.tile_h - 1) / p.tile_h, ntx = (p.W + p.tile_w - 1) / p.tile_w;
  const dim3 grid((unsigned)(p.n_img * nty * ntx * n_chunks)), block((unsigned)p.gv_threads);
  const size_t lds = dcnv4_grad_value_lds_bytes(p);
  const bool k3 = p.kh == 3 && p.kw == 3;
  auto go = [&](auto kernel) -> hipError_t {
    if (hipError_t e = ensure_dynamic_lds_limit(reinterpret_cast<const void *>(kernel), kMaxLdsPerWorkgroup)) return e;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return hipGetLastError();
  };
#define GV_CASE(KPV)                                                                \
  do {                                                                              \
    if (p.gv_threads == 512) {                                                      \
      if (p.gv_cw == 8) return go(dcnv4_grad_value_kernel<Tag, KPV, 8, gv_rounds(KPV), 512>);      \
      return go(dcnv4_grad_value_kernel<Tag, KPV, 16, gv_rounds(KPV), 512>);      \
    }                                                                               \
    if (p.gv_cw == 8) return go(dcnv4_grad_value_kernel<Tag, KPV, 8, gv_rounds(KPV), 1024>);       \
    return go(dcnv4_grad_value_kernel<Tag, KPV, 16, gv_rounds(KPV), 1024>);       \
  } while (0)
  if (k3 && !p.remove_center) GV_CASE(9);
  if (k3 && p.remove_center) GV_CASE(8);
  GV_CASE(0);
#undef GV_CASE
}

}  // namespace

size_t dcnv4_grad_value_lds_bytes(const DcnLaunch &p) {
  const size_t items = (size_t)p.strip_pix * dcnv4_grad_value_slots(p) * p.ng_chunk;
  // list heads (two sets), parked grad_out, entries + the dummy entry that ends every list; at the end the fp32 image
  // of the tile takes the place of all of it
  const size_t strip = 2 * (size_t)p.gv_threads * sizeof(uint32_t) + (size_t)p.strip_pix * p.gv_go_stride + (items + 1) * sizeof(u32x4);
  const size_t image = (size_t)p.tile_h * p.tile_w * dcnv4_grad_value_image_stride(p.ng_chunk * (p.gv_cw << p.gv_lps_log2)) * sizeof(float);
  return std::max(strip, image);
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
