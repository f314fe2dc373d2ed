// Centre-feature blend of a DCNv4 layer (DCNv4_op/DCNv4/modules/dcnv4.py:17-26,142-147):
//   gate[g] = sigmoid(<W[g, :], y> + b[g])            one gate per (pixel, group), from ALL channels of the pixel
//   out[c]  = y[c] * (1 - gate[g(c)]) + x[c] * gate[g(c)]
// with y the sampled features (the DCNv4 operator's output) and x the un-sampled projection.  The reference
// composes it from a linear layer, a sigmoid, a `repeat` that materialises the gates per channel and three
// element-wise kernels; here a row is read once, kept in registers and written once.
//
// Same lane layout as the layer-norm kernels: a team of T lanes (a power of two up to 64) owns a row of C
// channels, a lane holds VPL 16-byte vectors of it; a vector lies inside one group (the entry point checks that
// the group width is a whole number of vectors).  The G dot products are formed one group at a time: every
// lane multiplies its channels with the matching piece of W[g, :] (the teams of a wave read the same addresses),
// a butterfly of DPP moves (and shuffles beyond 16 lanes) closes the sum inside the team, and the lanes whose vectors belong to group g keep the gate.
// fp32 arithmetic, one rounding.
//
// Backward, for grad_out q:  grad_x = q * gate;  d gate[g] = sum over the group's channels of q * (x - y);
// d logit[g] = d gate[g] * gate[g] * (1 - gate[g]);  grad_y = q * (1 - gate) + sum_g d logit[g] * W[g, :].
// The kernel writes grad_x, grad_y and the logit gradients [rows, G] in fp32; the parameter gradients are
// grad_W = d logit^T . y and grad_b = column sums of d logit, a plain matrix product the caller owns.
#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

constexpr int kCfThreads = 256;

__device__ __forceinline__ float sigmoid(float z) { return 1.f / (1.f + __expf(-z)); }

template <typename Tag, int VPL, bool BWD>
__global__ void __launch_bounds__(kCfThreads) center_feature_blend_kernel(const CfLaunch p) {
  constexpr int V = 16 / Tag::kBytes;
  typedef Pack<Tag, V> pack;
  typedef typename pack::raw_t raw_t;
  const int team = p.team, nvec = p.C / V;
  const int teams_per_block = kCfThreads / team;
  const int lane_in_team = threadIdx.x & (team - 1);
  const long long row = (long long)blockIdx.x * teams_per_block + threadIdx.x / team;
  const bool row_live = row < p.rows;
  const raw_t *y_row = reinterpret_cast<const raw_t *>(p.y) + row * nvec;
  const raw_t *x_row = reinterpret_cast<const raw_t *>(p.x) + row * nvec;
  const raw_t *wt = reinterpret_cast<const raw_t *>(p.weight);
  const int vec_per_group = p.D / V;

  float y[VPL][V], x[VPL][V], q[VPL][V], gy[VPL][V], gate[VPL];
  int grp[VPL];
  bool live[VPL];
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const int i = lane_in_team + u * team;
    live[u] = row_live && i < nvec;
    grp[u] = i / vec_per_group;
    gate[u] = 0.f;
#pragma unroll
    for (int c = 0; c < V; ++c) y[u][c] = x[u][c] = q[u][c] = gy[u][c] = 0.f;
    if (live[u]) {
      pack::decode(y_row[i], y[u]);
      pack::decode(x_row[i], x[u]);
      if constexpr (BWD) pack::decode(reinterpret_cast<const raw_t *>(p.grad_out)[row * nvec + i], q[u]);
    }
  }

  for (int g = 0; g < p.G; ++g) {
    float wv[VPL][V];
    float z = 0.f, dgate = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const int i = lane_in_team + u * team;
      if (i < nvec) pack::decode(wt[(size_t)g * nvec + i], wv[u]);
      else {
#pragma unroll
        for (int c = 0; c < V; ++c) wv[u][c] = 0.f;
      }
#pragma unroll
      for (int c = 0; c < V; ++c) z = fmaf(wv[u][c], y[u][c], z);
      if constexpr (BWD) {
        if (grp[u] == g) {
#pragma unroll
          for (int c = 0; c < V; ++c) dgate = fmaf(q[u][c], x[u][c] - y[u][c], dgate);
        }
      }
    }
    z = cluster_sum(z, team);
    if constexpr (BWD) dgate = cluster_sum(dgate, team);
    if constexpr (!BWD) {        // forward: a lane keeps the logit of its own group(s) and takes one sigmoid at the end
#pragma unroll
      for (int u = 0; u < VPL; ++u) gate[u] = grp[u] == g ? z : gate[u];
      continue;
    }
    float bias_g[1];
    Pack<Tag, 1>::decode(reinterpret_cast<const typename RawWord<Tag::kBytes>::type *>(p.bias)[g], bias_g);
    const float s = sigmoid(z + bias_g[0]);
#pragma unroll
    for (int u = 0; u < VPL; ++u) gate[u] = grp[u] == g ? s : gate[u];
    if constexpr (BWD) {
      const float dlogit = dgate * s * (1.f - s);
      if (row_live && lane_in_team == 0) p.grad_logits[row * p.G + g] = dlogit;
#pragma unroll
      for (int u = 0; u < VPL; ++u)
#pragma unroll
        for (int c = 0; c < V; ++c) gy[u][c] = fmaf(dlogit, wv[u][c], gy[u][c]);
    }
  }

  if constexpr (!BWD) {
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      float bias_g[1];
      Pack<Tag, 1>::decode(reinterpret_cast<const typename RawWord<Tag::kBytes>::type *>(p.bias)[min(grp[u], p.G - 1)], bias_g);
      gate[u] = sigmoid(gate[u] + bias_g[0]);
    }
  }
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    if (!live[u]) continue;
    const int i = lane_in_team + u * team;
    float r[V];
    if constexpr (BWD) {
      float rx[V];
#pragma unroll
      for (int c = 0; c < V; ++c) {
        r[c] = fmaf(q[u][c], 1.f - gate[u], gy[u][c]);
        rx[c] = q[u][c] * gate[u];
      }
      reinterpret_cast<raw_t *>(p.grad_y)[row * nvec + i] = pack::encode(r);
      reinterpret_cast<raw_t *>(p.grad_x)[row * nvec + i] = pack::encode(rx);
    } else {
#pragma unroll
      for (int c = 0; c < V; ++c) r[c] = y[u][c] * (1.f - gate[u]) + x[u][c] * gate[u];
      reinterpret_cast<raw_t *>(p.out)[row * nvec + i] = pack::encode(r);
    }
  }
}

template <typename Tag, bool BWD>
hipError_t launch_t(const CfLaunch &p, hipStream_t stream) {
  const int teams_per_block = kCfThreads / p.team;
  const dim3 grid((unsigned)((p.rows + teams_per_block - 1) / teams_per_block)), block(kCfThreads);
  switch (p.vpl) {
    case 1: hipLaunchKernelGGL((center_feature_blend_kernel<Tag, 1, BWD>), grid, block, 0, stream, p); break;
    case 2: hipLaunchKernelGGL((center_feature_blend_kernel<Tag, 2, BWD>), grid, block, 0, stream, p); break;
    case 4: hipLaunchKernelGGL((center_feature_blend_kernel<Tag, 4, BWD>), grid, block, 0, stream, p); break;
    case 8: hipLaunchKernelGGL((center_feature_blend_kernel<Tag, 8, BWD>), grid, block, 0, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_center_feature_blend(int dtype, const CfLaunch &p, bool backward, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return backward ? launch_t<F32, true>(p, stream) : launch_t<F32, false>(p, stream);
    case F16::kCode: return backward ? launch_t<F16, true>(p, stream) : launch_t<F16, false>(p, stream);
    case BF16::kCode: return backward ? launch_t<BF16, true>(p, stream) : launch_t<BF16, false>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
