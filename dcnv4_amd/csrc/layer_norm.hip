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
  sum = cluster_sum(sum, team);
  const float mean = sum / (float)p.C;
  float sq = 0.f;
#pragma unroll
  for (int u = 0; u < VPL; ++u)
    if (live[u])
#pragma unroll
      for (int c = 0; c < V; ++c) sq = fmaf(v[u][c] - mean, v[u][c] - mean, sq);
  sq = cluster_sum(sq, team);
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


// ------------------------------------------------------------------------------- backward
// Gradients of out = residual + gamma * (xhat * weight + bias), xhat = (y - mean) * rstd, for grad_out g:
//   grad_y      = rstd * (a - mean(a) - xhat * mean(a * xhat)),  a = g * gamma * weight      (row-wise)
//   grad_weight = sum over rows of g * gamma * xhat
//   grad_bias   = sum over rows of g * gamma
//   grad_gamma  = sum over rows of g * (xhat * weight + bias)
// (grad_residual is g itself.)  Same lane layout as the forward: a team owns a row and recomputes its
// statistics from y in registers, so nothing is saved by the forward.  A workgroup walks a slab of
// consecutive rows and keeps the three column sums of its lanes' channels in registers; at the end the teams
// of the workgroup are added through LDS in a fixed order and the workgroup writes one row of partial sums;
// a second kernel adds the partial rows in order.  No atomics: the result does not depend on scheduling.
template <typename Tag, int VPL>
__global__ void __launch_bounds__(kLnThreads) layer_norm_residual_backward_kernel(const LnLaunch p) {
  extern __shared__ float s_cols[];                     // [teams][C]
  constexpr int V = 16 / Tag::kBytes;
  typedef Pack<Tag, V> pack;
  typedef typename pack::raw_t raw_t;
  const int team = p.team, nvec = p.C / V;
  const int teams_per_block = kLnThreads / team;
  const int lane_in_team = threadIdx.x & (team - 1), team_id = threadIdx.x / team;
  const float inv_c = 1.f / (float)p.C;

  float w[VPL][V], gam[VPL][V], b[VPL][V];
  float dw[VPL][V], db[VPL][V], dg[VPL][V];
  bool col_live[VPL];
#pragma unroll
  for (int u = 0; u < VPL; ++u) {
    const int i = lane_in_team + u * team;
    col_live[u] = i < nvec;
#pragma unroll
    for (int c = 0; c < V; ++c) { w[u][c] = 0.f; gam[u][c] = 1.f; b[u][c] = 0.f; dw[u][c] = db[u][c] = dg[u][c] = 0.f; }
    if (col_live[u]) {
      pack::decode(reinterpret_cast<const raw_t *>(p.weight)[i], w[u]);
      if (p.gamma != nullptr) {
        pack::decode(reinterpret_cast<const raw_t *>(p.gamma)[i], gam[u]);
        pack::decode(reinterpret_cast<const raw_t *>(p.bias)[i], b[u]);
      }
    }
  }

  const long long row_begin = (long long)blockIdx.x * p.slab;
  const long long row_end = row_begin + p.slab < p.rows ? row_begin + p.slab : p.rows;
  // the rows of the next pass are requested before the current pass is worked on
  raw_t next_y[VPL], next_g[VPL];
  auto request = [&](long long row0) {
    const long long row = row0 + team_id;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      const int i = lane_in_team + u * team;
      if (row < row_end && col_live[u]) {
        next_y[u] = reinterpret_cast<const raw_t *>(p.y)[row * nvec + i];
        next_g[u] = reinterpret_cast<const raw_t *>(p.grad_out)[row * nvec + i];
      } else {
        next_y[u] = raw_t{};
        next_g[u] = raw_t{};
      }
    }
  };
  request(row_begin);
  for (long long row0 = row_begin; row0 < row_end; row0 += teams_per_block) {
    const long long row = row0 + team_id;
    const bool row_live = row < row_end;
    float v[VPL][V], g[VPL][V];
    float sum = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      pack::decode(next_y[u], v[u]);
      pack::decode(next_g[u], g[u]);
#pragma unroll
      for (int c = 0; c < V; ++c) sum += v[u][c];
    }
    request(row0 + teams_per_block);
    sum = cluster_sum(sum, team);
    const float mean = sum * inv_c;
    float sq = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u)
      if (col_live[u])
#pragma unroll
        for (int c = 0; c < V; ++c) sq = fmaf(v[u][c] - mean, v[u][c] - mean, sq);
    sq = cluster_sum(sq, team);
    const float rstd = rsqrtf(sq * inv_c + p.eps);

    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
#pragma unroll
      for (int c = 0; c < V; ++c) {
        const float xh = (row_live && col_live[u]) ? (v[u][c] - mean) * rstd : 0.f;
        const float gg = g[u][c] * gam[u][c];               // g * gamma
        const float a = gg * w[u][c];
        s1 += a;
        s2 = fmaf(a, xh, s2);
        dw[u][c] = fmaf(gg, xh, dw[u][c]);
        db[u][c] += gg;
        dg[u][c] = fmaf(g[u][c], fmaf(xh, w[u][c], b[u][c]), dg[u][c]);
        v[u][c] = xh;
        g[u][c] = a;
      }
    }
    s1 = cluster_sum(s1, team);
    s2 = cluster_sum(s2, team);
    const float m1 = s1 * inv_c, m2 = s2 * inv_c;
    if (row_live) {
      raw_t *gy = reinterpret_cast<raw_t *>(p.grad_y) + row * nvec;
#pragma unroll
      for (int u = 0; u < VPL; ++u) {
        if (!col_live[u]) continue;
        float r[V];
#pragma unroll
        for (int c = 0; c < V; ++c) r[c] = rstd * (g[u][c] - m1 - v[u][c] * m2);
        gy[lane_in_team + u * team] = pack::encode(r);
      }
    }
  }

  // teams of the workgroup, one quantity at a time, added in team order
  float *part = p.partial + (size_t)blockIdx.x * 3 * p.C;
#pragma unroll
  for (int q = 0; q < 3; ++q) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < VPL; ++u) {
      if (!col_live[u]) continue;
      float *dst = s_cols + (size_t)team_id * p.C + (size_t)(lane_in_team + u * team) * V;
#pragma unroll
      for (int c = 0; c < V; ++c) dst[c] = q == 0 ? dw[u][c] : (q == 1 ? db[u][c] : dg[u][c]);
    }
    __syncthreads();
    for (int c = threadIdx.x; c < p.C; c += kLnThreads) {
      float acc = 0.f;
      for (int t = 0; t < teams_per_block; ++t) acc += s_cols[(size_t)t * p.C + c];
      part[(size_t)q * p.C + c] = acc;
    }
  }
}

// partial [n_part][3][C] -> grad_weight, grad_bias, grad_gamma.  A workgroup takes 8 columns; its 128 row lanes each add
// every 128th partial row (independent loads, many in flight), then the row lanes meet through LDS in lane order: a fixed
// summation tree, so the result does not depend on scheduling.
constexpr int kPgCols = 8, kPgRows = 128;
template <typename Tag>
__global__ void __launch_bounds__(kPgCols * kPgRows) layer_norm_param_grad_kernel(const LnLaunch p) {
  __shared__ float s_part[kPgRows][kPgCols + 1];
  const int col = threadIdx.x % kPgCols, rl = threadIdx.x / kPgCols;
  const int idx = blockIdx.x * kPgCols + col;                   // column of the [3][C] row
  float acc = 0.f;
  if (idx < 3 * p.C)
    for (int w = rl; w < p.n_part; w += kPgRows) acc += p.partial[(size_t)w * 3 * p.C + idx];
  s_part[rl][col] = acc;
  __syncthreads();
  if (rl != 0 || idx >= 3 * p.C) return;
  float total = 0.f;
#pragma unroll
  for (int r = 0; r < kPgRows; ++r) total += s_part[r][col];
  const int q = idx / p.C, c = idx - q * p.C;
  void *dst = q == 0 ? p.grad_weight : (q == 1 ? p.grad_bias : p.grad_gamma);
  if (dst == nullptr) return;
  const float f[1] = {total};
  reinterpret_cast<typename RawWord<Tag::kBytes>::type *>(dst)[c] = Pack<Tag, 1>::encode(f);
}

template <typename Tag>
hipError_t launch_bwd_t(const LnLaunch &p, hipStream_t stream) {
  const int teams_per_block = kLnThreads / p.team;
  const dim3 grid((unsigned)p.n_part), block(kLnThreads);
  const size_t lds = (size_t)teams_per_block * p.C * sizeof(float);
  switch (p.vpl) {
    case 1: hipLaunchKernelGGL((layer_norm_residual_backward_kernel<Tag, 1>), grid, block, lds, stream, p); break;
    case 2: hipLaunchKernelGGL((layer_norm_residual_backward_kernel<Tag, 2>), grid, block, lds, stream, p); break;
    case 4: hipLaunchKernelGGL((layer_norm_residual_backward_kernel<Tag, 4>), grid, block, lds, stream, p); break;
    case 8: hipLaunchKernelGGL((layer_norm_residual_backward_kernel<Tag, 8>), grid, block, lds, stream, p); break;
    default: return hipErrorInvalidValue;
  }
  if (hipError_t e = hipGetLastError()) return e;
  hipLaunchKernelGGL((layer_norm_param_grad_kernel<Tag>), dim3((unsigned)((3 * p.C + kPgCols - 1) / kPgCols)), dim3(kPgCols * kPgRows), 0, stream, p);
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

hipError_t launch_layer_norm_residual_backward(int dtype, const LnLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_bwd_t<F32>(p, stream);
    case F16::kCode: return launch_bwd_t<F16>(p, stream);
    case BF16::kCode: return launch_bwd_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
