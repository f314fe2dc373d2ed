// Depthwise convolution over NHWC tensors: the `offset_mask_dw` layer that feeds the offset/mask
// projection of a DCNv4 block (DCNv4_op/DCNv4/modules/dcnv4.py:67-75, applied at dcnv4.py:121-123
// between two NHWC <-> NCHW permutes).  The tensors of a DCNv4 block are channels-last, a layout for
// which the vendor convolution library only has its generic one-thread-per-output kernel when the
// convolution is depthwise; these kernels work on NHWC directly, so the permutes disappear as well.
//
//   forward      out[b,y,x,c] = bias[c] + sum_{i,j} w[c,i,j] * in[b, y+i-ph, x+j-pw, c]
//                one lane per (image row, segment of output columns, 16-byte channel vector); the
//                lanes of a wave are neighbouring channel vectors and segments, so every load
//                instruction reads runs of whole pixels; the kh x kw window of a lane slides along the
//                row in registers (kh new vectors per output); fp32 accumulation
//   grad_input   the same kernel with the kernel flipped and padding k-1-p
//   grad_weight  grad_w[c,i,j] = sum_{b,y,x} go[b,y,x,c] * in[b, y+i-ph, x+j-pw, c], grad_bias[c] = sum go:
//                a workgroup takes a slab of output pixels, a lane a channel vector and every n-th pixel
//                of the slab; lanes add up in registers, the lanes of a workgroup in LDS in a fixed order,
//                workgroups through a partial-sum table that a second kernel adds up in a fixed order:
//                no atomics, bit-reproducible.
// Stride and dilation are 1 (the layer is built that way).  HBM-bound: one read of the input and one
// write of the output when the row above and below stay in cache.
#include "common.hpp"
#include "launch.hpp"

namespace dcn {
namespace {

constexpr int kDwThreads = 256;

template <typename Tag, int V>
__device__ __forceinline__ void load_vec(__amdgpu_buffer_rsrc_t rs, uint32_t off, float (&f)[V]) {
  Pack<Tag, V>::decode(buffer_load<V * Tag::kBytes>(rs, off), f);
}

// KH == 0: kernel size taken from the launch record (any size up to 7x7), weights re-read per tap.
template <typename Tag, int V, int KH, int KW>
__global__ void __launch_bounds__(kDwThreads) dwconv_forward_kernel(const DwLaunch p) {
  constexpr int kVecBytes = V * Tag::kBytes;
  const int kh = KH > 0 ? KH : p.kh, kw = KH > 0 ? KW : p.kw;
  const int nvec = p.C / V;
  // consecutive workgroups share input rows: keep them on one XCD (one L2)
  uint32_t t = xcd_contiguous_block(blockIdx.x, gridDim.x) * kDwThreads + threadIdx.x;
  const int cvec = t % nvec; t /= nvec;
  const int xs = t % p.n_seg; t /= p.n_seg;
  const int y = t % p.Ho;
  const uint32_t b = t / p.Ho;
  if (b >= (uint32_t)p.B) return;
  const __amdgpu_buffer_rsrc_t in_rs = make_rsrc(p.in, (uint32_t)((size_t)p.B * p.H * p.W * p.C * Tag::kBytes));
  const __amdgpu_buffer_rsrc_t w_rs = make_rsrc(p.weight, (uint32_t)((size_t)p.C * kh * kw * Tag::kBytes));
  const uint32_t pix_bytes = (uint32_t)p.C * Tag::kBytes, row_bytes = (uint32_t)p.W * pix_bytes;
  const uint32_t img = b * (uint32_t)p.H * row_bytes + (uint32_t)cvec * kVecBytes;
  const int x_begin = xs * p.seg, x_end = min(p.Wo, x_begin + p.seg);

  float bias[V];
#pragma unroll
  for (int v = 0; v < V; ++v) bias[v] = 0.f;
  if (p.bias != nullptr) {
    const __amdgpu_buffer_rsrc_t b_rs = make_rsrc(p.bias, (uint32_t)((size_t)p.C * Tag::kBytes));
    load_vec<Tag, V>(b_rs, (uint32_t)cvec * kVecBytes, bias);
  }
  typedef typename RawWord<kVecBytes>::type raw_t;
  raw_t *out = reinterpret_cast<raw_t *>(p.out) + ((size_t)b * p.Ho + y) * p.Wo * nvec + cvec;

  if constexpr (KH > 0) {
    // weights [C][KH][KW]: this lane's V channels are V * KH * KW contiguous elements, read as KH * KW
    // vectors and regrouped into w[tap][v]; `flip` reads the kernel back to front
    float w[KH * KW][V];
    {
      float flat[KH * KW * V];
#pragma unroll
      for (int k = 0; k < KH * KW; ++k) {
        float f[V];
        load_vec<Tag, V>(w_rs, (uint32_t)(cvec * KH * KW + k) * kVecBytes, f);
#pragma unroll
        for (int v = 0; v < V; ++v) flat[k * V + v] = f[v];
      }
#pragma unroll
      for (int k = 0; k < KH * KW; ++k)
#pragma unroll
        for (int v = 0; v < V; ++v) w[k][v] = p.flip ? flat[v * KH * KW + KH * KW - 1 - k] : flat[v * KH * KW + k];
    }
    // byte offsets of the window's rows (dropped when the row is outside the image)
    uint32_t row_off[KH];
#pragma unroll
    for (int i = 0; i < KH; ++i) {
      const int yy = y + i - p.ph;
      row_off[i] = (yy >= 0 && yy < p.H) ? img + (uint32_t)yy * row_bytes : kDropOffset;
    }
    auto column = [&](int xx, raw_t (&col)[KH]) {
      const bool ok = xx >= 0 && xx < p.W;
#pragma unroll
      for (int i = 0; i < KH; ++i)
        col[i] = buffer_load<kVecBytes>(in_rs, (ok && row_off[i] != kDropOffset) ? row_off[i] + (uint32_t)xx * pix_bytes : kDropOffset);
    };
    raw_t win[KW][KH];                  // win[j] = input column x + j - pw
#pragma unroll
    for (int j = 0; j < KW - 1; ++j) column(x_begin + j - p.pw, win[j]);
    for (int x = x_begin; x < x_end; ++x) {
      column(x + KW - 1 - p.pw, win[KW - 1]);
      float acc[V];
#pragma unroll
      for (int v = 0; v < V; ++v) acc[v] = bias[v];
#pragma unroll
      for (int j = 0; j < KW; ++j)
#pragma unroll
        for (int i = 0; i < KH; ++i) {
          float f[V];
          Pack<Tag, V>::decode(win[j][i], f);
#pragma unroll
          for (int v = 0; v < V; ++v) acc[v] = fmaf(f[v], w[i * KW + j][v], acc[v]);
        }
      out[(size_t)x * nvec] = Pack<Tag, V>::encode(acc);
#pragma unroll
      for (int j = 0; j < KW - 1; ++j)
#pragma unroll
        for (int i = 0; i < KH; ++i) win[j][i] = win[j + 1][i];
    }
  } else {
    for (int x = x_begin; x < x_end; ++x) {
      float acc[V];
#pragma unroll
      for (int v = 0; v < V; ++v) acc[v] = bias[v];
      for (int i = 0; i < kh; ++i) {
        const int yy = y + i - p.ph;
        for (int j = 0; j < kw; ++j) {
          const int xx = x + j - p.pw;
          const bool ok = yy >= 0 && yy < p.H && xx >= 0 && xx < p.W;
          float f[V];
          load_vec<Tag, V>(in_rs, ok ? img + (uint32_t)yy * row_bytes + (uint32_t)xx * pix_bytes : kDropOffset, f);
          const int k = i * kw + j, src = p.flip ? kh * kw - 1 - k : k;
#pragma unroll
          for (int v = 0; v < V; ++v) {
            float wv[1];
            load_vec<Tag, 1>(w_rs, (uint32_t)((cvec * V + v) * kh * kw + src) * Tag::kBytes, wv);
            acc[v] = fmaf(f[v], wv[0], acc[v]);
          }
        }
      }
      out[(size_t)x * nvec] = Pack<Tag, V>::encode(acc);
    }
  }
}

// Partial sums of grad_weight and grad_bias: partial[workgroup][tap (kh*kw, then the bias)][C], fp32.
// blockIdx.y selects a run of kDwThreads channel vectors when C / V exceeds the workgroup.
template <typename Tag, int V, int KH, int KW>
__global__ void __launch_bounds__(kDwThreads) dwconv_grad_weight_kernel(const DwLaunch p) {
  constexpr int kVecBytes = V * Tag::kBytes;
  constexpr int kTaps = KH * KW;
  __shared__ float s_part[kDwThreads * V];
  const int nvec = p.C / V;
  const int vec0 = blockIdx.y * kDwThreads, nv_here = min(kDwThreads, nvec - vec0);
  const int px_lanes = kDwThreads / nv_here;                 // lanes that share a channel vector
  const int pl = threadIdx.x / nv_here, cv = threadIdx.x - pl * nv_here;
  const bool live = pl < px_lanes;
  const int cvec = vec0 + cv;
  const __amdgpu_buffer_rsrc_t in_rs = make_rsrc(p.in, (uint32_t)((size_t)p.B * p.H * p.W * p.C * Tag::kBytes));
  const __amdgpu_buffer_rsrc_t go_rs = make_rsrc(p.grad_out, (uint32_t)((size_t)p.B * p.Ho * p.Wo * p.C * Tag::kBytes));
  const uint32_t pix_bytes = (uint32_t)p.C * Tag::kBytes, row_bytes = (uint32_t)p.W * pix_bytes;

  float acc[kTaps + 1][V];
#pragma unroll
  for (int k = 0; k <= kTaps; ++k)
#pragma unroll
    for (int v = 0; v < V; ++v) acc[k][v] = 0.f;

  // the slab is a run of row segments (seg output columns each); a lane walks its segments with the
  // KH x KW input window sliding in registers: KH new input vectors and one grad_out vector per pixel
  typedef typename RawWord<kVecBytes>::type raw_t;
  const uint32_t n_rowseg = (uint32_t)p.B * p.Ho * p.n_seg;
  const uint32_t slab_id = xcd_contiguous_block(blockIdx.x, gridDim.x);      // neighbouring slabs share rows: same XCD
  const uint32_t first = slab_id * (uint32_t)p.slab, last = min(n_rowseg, first + (uint32_t)p.slab);
  if (live)
    for (uint32_t q = first + pl; q < last; q += px_lanes) {
      const uint32_t row = q / (uint32_t)p.n_seg;                       // b * Ho + y
      const int xs = q - row * p.n_seg;
      const uint32_t b = row / (uint32_t)p.Ho;
      const int y = row - b * p.Ho;
      const int x_begin = xs * p.seg, x_end = min(p.Wo, x_begin + p.seg);
      const uint32_t img = b * (uint32_t)p.H * row_bytes + (uint32_t)cvec * kVecBytes;
      const uint32_t go_row = row * (uint32_t)p.Wo * pix_bytes + (uint32_t)cvec * kVecBytes;
      uint32_t row_off[KH];
#pragma unroll
      for (int i = 0; i < KH; ++i) {
        const int yy = y + i - p.ph;
        row_off[i] = (yy >= 0 && yy < p.H) ? img + (uint32_t)yy * row_bytes : kDropOffset;
      }
      auto column = [&](int xx, raw_t (&col)[KH]) {
        const bool ok = xx >= 0 && xx < p.W;
#pragma unroll
        for (int i = 0; i < KH; ++i)
          col[i] = buffer_load<kVecBytes>(in_rs, (ok && row_off[i] != kDropOffset) ? row_off[i] + (uint32_t)xx * pix_bytes : kDropOffset);
      };
      raw_t win[KW][KH];
#pragma unroll
      for (int j = 0; j < KW - 1; ++j) column(x_begin + j - p.pw, win[j]);
      // the next pixel's input column and grad_out vector are requested before this pixel's sums
      raw_t col_next[KH], go_next;
      column(x_begin + KW - 1 - p.pw, col_next);
      go_next = buffer_load<kVecBytes>(go_rs, go_row + (uint32_t)x_begin * pix_bytes);
      for (int x = x_begin; x < x_end; ++x) {
#pragma unroll
        for (int i = 0; i < KH; ++i) win[KW - 1][i] = col_next[i];
        float g[V];
        Pack<Tag, V>::decode(go_next, g);
        if (x + 1 < x_end) {
          column(x + KW - p.pw, col_next);
          go_next = buffer_load<kVecBytes>(go_rs, go_row + (uint32_t)(x + 1) * pix_bytes);
        }
#pragma unroll
        for (int j = 0; j < KW; ++j)
#pragma unroll
          for (int i = 0; i < KH; ++i) {
            float f[V];
            Pack<Tag, V>::decode(win[j][i], f);
#pragma unroll
            for (int v = 0; v < V; ++v) acc[i * KW + j][v] = fmaf(g[v], f[v], acc[i * KW + j][v]);
          }
#pragma unroll
        for (int v = 0; v < V; ++v) acc[kTaps][v] += g[v];
#pragma unroll
        for (int j = 0; j < KW - 1; ++j)
#pragma unroll
          for (int i = 0; i < KH; ++i) win[j][i] = win[j + 1][i];
      }
    }

  // lanes of the workgroup, one tap at a time: the first lane of each channel vector adds the others in order
  float *part = p.partial + ((size_t)slab_id * (kTaps + 1)) * p.C + (size_t)cvec * V;
#pragma unroll
  for (int k = 0; k <= kTaps; ++k) {
    __syncthreads();
#pragma unroll
    for (int v = 0; v < V; ++v) s_part[threadIdx.x * V + v] = acc[k][v];
    __syncthreads();
    if (live && pl == 0) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        float s = acc[k][v];
        for (int o = 1; o < px_lanes; ++o) s += s_part[(o * nv_here + cv) * V + v];
        part[(size_t)k * p.C + v] = s;
      }
    }
  }
}

// grad_weight[c][tap] and grad_bias[c] from the partial sums.  A workgroup takes 16 consecutive
// (tap, channel) entries; THREADS / 16 lanes per entry each add every so-manieth partial sum, then the first lane
// adds the lane sums in index order: a fixed order whatever the schedule.  64 lanes per entry when there are few
// entries (112 channels: 0.110 -> 0.103 ms for the whole backward), 16 otherwise.
constexpr int kReduceEntries = 16;

template <typename Tag, int THREADS>
__global__ void __launch_bounds__(THREADS) dwconv_reduce_kernel(const DwLaunch p, int taps, int n_part) {
  constexpr int kReduceLanes = THREADS / kReduceEntries;
  __shared__ float s_sum[kReduceLanes][kReduceEntries];
  const int e = threadIdx.x % kReduceEntries, g = threadIdx.x / kReduceEntries;
  const int i = blockIdx.x * kReduceEntries + e;              // tap * C + c
  const int n = (taps + 1) * p.C;
  float s[4] = {0.f, 0.f, 0.f, 0.f};
  if (i < n) {
    const float *src = p.partial + i;
    const size_t step = (size_t)n;
    int w = g;
    for (; w + 3 * kReduceLanes < n_part; w += 4 * kReduceLanes)
#pragma unroll
      for (int u = 0; u < 4; ++u) s[u] += src[(size_t)(w + u * kReduceLanes) * step];
    for (; w < n_part; w += kReduceLanes) s[0] += src[(size_t)w * step];
  }
  s_sum[g][e] = (s[0] + s[1]) + (s[2] + s[3]);
  __syncthreads();
  if (g != 0 || i >= n) return;
  float total[1] = {0.f};
  for (int o = 0; o < kReduceLanes; ++o) total[0] += s_sum[o][e];
  const int k = i / p.C, c = i - k * p.C;
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  if (k < taps) reinterpret_cast<elem_t *>(p.grad_weight)[(size_t)c * taps + k] = Pack<Tag, 1>::encode(total);
  else if (p.grad_bias != nullptr) reinterpret_cast<elem_t *>(p.grad_bias)[c] = Pack<Tag, 1>::encode(total);
}

template <typename Tag, int V>
hipError_t forward_v(const DwLaunch &p, hipStream_t stream) {
  const size_t lanes = (size_t)p.B * p.Ho * p.n_seg * (p.C / V);
  const dim3 grid((unsigned)((lanes + kDwThreads - 1) / kDwThreads)), block(kDwThreads);
  if (p.kh == 3 && p.kw == 3) hipLaunchKernelGGL((dwconv_forward_kernel<Tag, V, 3, 3>), grid, block, 0, stream, p);
  else hipLaunchKernelGGL((dwconv_forward_kernel<Tag, V, 0, 0>), grid, block, 0, stream, p);
  return hipGetLastError();
}

template <typename Tag>
hipError_t forward_t(const DwLaunch &p, hipStream_t stream) {
  constexpr int kFull = 16 / Tag::kBytes;
  if (p.C % kFull == 0) return forward_v<Tag, kFull>(p, stream);
  if (p.C % 2 == 0) return forward_v<Tag, 2>(p, stream);
  return forward_v<Tag, 1>(p, stream);
}

template <typename Tag, int V>
hipError_t grad_weight_v(const DwLaunch &p, hipStream_t stream) {
  const int nvec = p.C / V;
  const dim3 grid((unsigned)p.n_part, (unsigned)((nvec + kDwThreads - 1) / kDwThreads)), block(kDwThreads);
#define DW_CASE(K)                                                                                        \
  if (p.kh == K && p.kw == K) {                                                                           \
    hipLaunchKernelGGL((dwconv_grad_weight_kernel<Tag, V, K, K>), grid, block, 0, stream, p);             \
    return hipGetLastError();                                                                             \
  }
  DW_CASE(1) DW_CASE(3)
  if constexpr (V <= 2) { DW_CASE(5) DW_CASE(7) }     // (taps + 1) * V sums must fit the register file
#undef DW_CASE
  return hipErrorInvalidValue;
}

template <typename Tag>
hipError_t grad_weight_t(const DwLaunch &p, hipStream_t stream) {
  constexpr int kFull = 16 / Tag::kBytes;
  const int v = depthwise_grad_weight_vector(Tag::kBytes, p.C, p.kh);
  if (v == kFull) return grad_weight_v<Tag, kFull>(p, stream);
  if (v == 2) return grad_weight_v<Tag, 2>(p, stream);
  return grad_weight_v<Tag, 1>(p, stream);
}

template <typename Tag>
hipError_t reduce_t(const DwLaunch &p, hipStream_t stream) {
  const int taps = p.kh * p.kw, n = (taps + 1) * p.C;
  const dim3 grid((unsigned)((n + kReduceEntries - 1) / kReduceEntries));
  if (n <= 3072) hipLaunchKernelGGL((dwconv_reduce_kernel<Tag, 1024>), grid, dim3(1024), 0, stream, p, taps, p.n_part);
  else hipLaunchKernelGGL((dwconv_reduce_kernel<Tag, 256>), grid, dim3(256), 0, stream, p, taps, p.n_part);
  return hipGetLastError();
}

}  // namespace

// Narrow vectors keep the register footprint of (taps + 1) * V sums in bounds: the kernel waits on its loads every
// pixel, so waves per SIMD count for more than bytes per load.  16-bit tensors: two channels per lane (measured
// 128x56x56x112 fp16: 103 us with 8 channels per lane, 68 us with 2); fp32: no difference between 4, 2 and 1.
int depthwise_grad_weight_vector(int elem_bytes, int C, int k) {
  const int full = 16 / elem_bytes;
  if (k <= 3 && elem_bytes == 2 && C % 2 == 0) return 2;
  if (k <= 3 && C % full == 0) return full;
  return C % 2 == 0 ? 2 : 1;
}

int depthwise_grad_weight_pixel_lanes(int elem_bytes, int C, int k) {
  const int nvec = C / depthwise_grad_weight_vector(elem_bytes, C, k);
  return kDwThreads / (nvec < kDwThreads ? nvec : kDwThreads);
}

hipError_t launch_depthwise_forward(int dtype, const DwLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return forward_t<F32>(p, stream);
    case F16::kCode: return forward_t<F16>(p, stream);
    case BF16::kCode: return forward_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_depthwise_grad_weight_partials(int dtype, const DwLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return grad_weight_t<F32>(p, stream);
    case F16::kCode: return grad_weight_t<F16>(p, stream);
    case BF16::kCode: return grad_weight_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

hipError_t launch_depthwise_grad_weight_reduce(int dtype, const DwLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return reduce_t<F32>(p, stream);
    case F16::kCode: return reduce_t<F16>(p, stream);
    case BF16::kCode: return reduce_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
