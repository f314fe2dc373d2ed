// Layer normalisation over the channel axis of an NHWC tensor, fused with what follows it in a
// FlashInternImage block: out = residual + gamma * LayerNorm(y) (post-norm blocks with layer scale,
// classification/models/flash_intern_image.py:425-440: `x + drop_path(gamma1 * norm1(dcn(x)))`), or any
// prefix of that (no residual, no gamma).  The framework runs this as three kernels (normalise, broadcast
// multiply, add) that move seven tensors' worth of bytes at about 1 TB/s; here a row is read once, kept in
// registers, and written once: three tensors' worth.
//
// A team of T lanes (a power of two up to 64, so a team never leaves its wave) owns one row of C channels;
// a lane holds VPL 16-byte vectors of it.  Mean and variance are two passes over the registers (sum, then
// sum of squared deviations), each closed by an xor-shuffle reduction inside the team; all arithmetic is fp32
// and the result is rounded once.  HBM-bound.
#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

constexpr int kLnThreads = 256;

template <typename Tag, int VPL>
__global__ void __launch_bounds__(kLnThreads) layer_norm_residual_kernel(const LnLaunch p) {
  constexpr int V = 16 / Tag::kBytes;
  typedef Pack<Tag, V> pack;
  typedef typename pack::raw_t raw_t;
  const int team = p.team, nvec = p.C / V;
  const int teams_per_block = kLnThreads / team;
  const int lane_in_team = threadIdx.x & (team - 1);
  const size_t row = (size_t)blockIdx.x * teams_per_block + threadIdx.x / team;
  const bool row_live = row < (size_t)p.rows;
  const raw_t *y = reinterpret_cast<const raw_t *>(p.y) + row * nvec;
  const raw_t *res = reinterpret_cast<const raw_t *>(p.residual) + row * nvec;
  raw_t *out = reinterpret_cast<raw_t *>(p.out) + row * nvec;

  float v[VPL][V];
  bool live[VPL];
  float sum = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const int i = lane_in_team + u * team;
    live[u] = row_live && i < nvec;
    if (live[u]) {
      pack::decode(y[i], v[u]);
#pragma unroll
      for (int c = 0; c < V; ++c) sum += v[u][c];
    } else {
#pragma unroll
      for (int c = 0; c < V; ++c) v[u][c] = 0.f;
    }
  }
  for (int o = team >> 1; o > 0; o >>= 1) sum += __shfl_xor(sum, o, kWave);
  const float mean = sum / (float)p.C;
  float sq = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u)
    if (live[u])
#pragma unroll
      for (int c = 0; c < V; ++c) sq = fmaf(v[u][c] - mean, v[u][c] - mean, sq);
  for (int o = team >> 1; o > 0; o >>= 1) sq += __shfl_xor(sq, o, kWave);
  const float rstd = rsqrtf(sq / (float)p.C + p.eps);

#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    if (!live[u]) continue;
    const int i = lane_in_team + u * team;
    float w[V], b[V], r[V];
    pack::decode(reinterpret_cast<const raw_t *>(p.weight)[i], w);
    pack::decode(reinterpret_cast<const raw_t *>(p.bias)[i], b);
#pragma unroll
    for (int c = 0; c < V; ++c) r[c] = fmaf((v[u][c] - mean) * rstd, w[c], b[c]);
    if (p.gamma != nullptr) {
      float g[V];
      pack::decode(reinterpret_cast<const raw_t *>(p.gamma)[i], g);
#pragma unroll
      for (int c = 0; c < V; ++c) r[c] *= g[c];
    }
    if (p.residual != nullptr) {
      float x[V];
      pack::decode(res[i], x);
#pragma unroll
      for (int c = 0; c < V; ++c) r[c] += x[c];
    }
    out[i] = pack::encode(r);
  }
}

template <typename Tag>
hipError_t launch_t(const LnLaunch &p, hipStream_t stream) {
  const int teams_per_block = kLnThreads / p.team;
  const dim3 grid((unsigned)((p.rows + teams_per_block - 1) / teams_per_block)), block(kLnThreads);
  switch (p.vpl) {
    case 1: hipLaunchKernelGGL((layer_norm_residual_kernel<Tag, 1>), grid, block, 0, stream, p); break;
    case 2: hipLaunchKernelGGL((layer_norm_residual_kernel<Tag, 2>), grid, block, 0, stream, p); break;
    case 4: hipLaunchKernelGGL((layer_norm_residual_kernel<Tag, 4>), grid, block, 0, stream, p); break;
    case 8: hipLaunchKernelGGL((layer_norm_residual_kernel<Tag, 8>), grid, block, 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_layer_norm_residual(int dtype, const LnLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_t<F32>(p, stream);
    case F16::kCode: return launch_t<F16>(p, stream);
    case BF16::kCode: return launch_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
