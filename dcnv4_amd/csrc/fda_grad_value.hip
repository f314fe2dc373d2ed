// Flash deformable attention backward, gradient of value, without global atomics.
//
// The reference scatters 4 * L * K * D fp32 atomicAdds per (query, head)
// (DCNv4_op/src/cuda/flash_deform_col2im_cuda.cuh:240-270 through common.h:153-184).  Sampling
// locations are free to land anywhere in their level, so unlike the DCNv4 operator there is no
// window around the query to exploit; instead a workgroup OWNS a tile of one level of one
// (image, head) and finds its contributions by scanning:
//
//   * the grad_sampling_loc_attn kernel, which runs first, leaves one 16-bit key (integer position of
//     the first corner, or "outside") and the softmax probability per sampling point, both laid out
//     [image][head][level][query][point], and the maximum of |grad_out| in GradState;
//   * scan: the workgroup streams the keys of its (image, head, level) - coalesced dwords of two keys, a handful
//     of instructions per point - and appends the points whose 2x2 corner block touches its tile
//     to a list in LDS;
//   * apply, in batches of 256 listed points: one lane per point recomputes the position from
//     sampling_loc_attn and, with the softmax probability the first kernel left beside the key,
//     the four corner weights; grad_out rows of the batch are parked in LDS (both requested one
//     batch ahead, so the loads fly while the previous batch is applied); a row of 8 lanes per point adds the
//     contributions to the tile's accumulators with 64-bit integer LDS atomics on fixed-point
//     values (normalised by max |grad_out|; probability * bilinear weight <= 1), so the result
//     does not depend on the order of arrival and is bit-reproducible;
//   * the finished tile is written to grad_value with plain stores in the tensor dtype.
//
// Workgroups are persistent and walk the (tile, image, head) items with a stride, smallest levels
// first: those tiles collect the most points each.  Levels, tile shapes and the item count are
// derived on the device from the spatial_shapes tensor; the host never reads it.
#include "common.hpp"
#include "launch.hpp"

namespace dcn {

namespace {

constexpr int kThreads = 1024;
constexpr int kRowLanes = 8;                 // lanes that apply one listed point
constexpr int kBatch = 256;                  // listed points applied between two barriers
constexpr int kScanPerLane = 16;             // dwords (two keys each) per lane and scan step: one memory latency per step
constexpr int kRoundKeys = 4;                // dwords per lane tested between two looks at the list's fill
constexpr int kScanStep = kThreads * kScanPerLane;
constexpr int kListCap = 3 * kRoundKeys * kThreads;      // flushed when another round (2 * kRoundKeys points per lane) might not fit
constexpr int kCellBitsF = 9;

struct LevelPlan {
  int H, W, start;
  int th, tw, nty, ntx;      // tile shape and tile grid
  int first_item_rank;       // rank of this level's first tile in the walk (smallest level first)
};

// float -> two's-complement 64-bit integer, see dcnv4_grad_value.hip
template <bool WIDE> __device__ __forceinline__ unsigned long long to_fixed64(float t) {
  if constexpr (WIDE) {
    const float th = floorf(t * 0x1p-32f);
    const int hi = (int)th;
    const uint32_t lo = (uint32_t)fmaf(th, -0x1p32f, t);
    return ((unsigned long long)(uint32_t)hi << 32) | lo;
  } else {
    const int v = (int)t;
    return ((unsigned long long)(uint32_t)(v >> 31) << 32) | (uint32_t)v;
  }
}

template <typename Tag>
__device__ __forceinline__ float elem_at(const void *base, size_t i) {
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  float f[1];
  Pack<Tag, 1>::decode(reinterpret_cast<const elem_t *>(base)[i], f);
  return f[0];
}

template <typename Tag, int CPL>
__global__ void __launch_bounds__(kThreads) fda_grad_value_kernel(const FdaLaunch p) {
  extern __shared__ unsigned long long lds64[];
  typedef typename RawWord<Tag::kBytes>::type elem_t;
  constexpr int DP = CPL * kRowLanes;                         // accumulator channels per cell (D rounded up)
  const int D = p.D, LK = p.L * p.K, QK = p.Q * p.K;
  const int cells_max = fda_tile_cells(D);
  unsigned long long *acc = lds64;                            // [(cells_max + 1) * DP], last cell = trash
  const int n_acc = (cells_max + 1) * DP;
  f32x4 *rec_w = reinterpret_cast<f32x4 *>(lds64 + n_acc);    // [kBatch]
  u32x2 *rec_meta = reinterpret_cast<u32x2 *>(rec_w + kBatch);   // [kBatch] cells 0,1,2 | cell 3
  float *s_go = reinterpret_cast<float *>(rec_meta + kBatch); // [kBatch][DP]
  uint32_t *s_list = reinterpret_cast<uint32_t *>(s_go + kBatch * DP);   // [kListCap]
  __shared__ LevelPlan s_plan[kMaxLevels];
  __shared__ int s_items;
  __shared__ uint32_t s_count;

  const int tid = threadIdx.x, lane = tid & (kWave - 1);
  if (tid == 0) {
    // walk order: last level first
    int rank = 0;
    for (int l = p.L - 1; l >= 0; --l) {
      LevelPlan lp;
      lp.H = (int)p.shapes[2 * l]; lp.W = (int)p.shapes[2 * l + 1]; lp.start = (int)p.level_start[l];
      lp.tw = max(1, min(lp.W, 16));
      lp.th = max(1, min(lp.H, cells_max / lp.tw));
      auto tiles = [&]() { return ((lp.H + lp.th - 1) / lp.th) * ((lp.W + lp.tw - 1) / lp.tw); };
      while (tiles() < 16 && lp.th * lp.tw > 16) {           // small levels: more, smaller tiles
        if (lp.th >= lp.tw) lp.th = (lp.th + 1) / 2; else lp.tw = (lp.tw + 1) / 2;
      }
      lp.nty = (lp.H + lp.th - 1) / lp.th; lp.ntx = (lp.W + lp.tw - 1) / lp.tw;
      lp.first_item_rank = rank;
      rank += (lp.H > 0 && lp.W > 0) ? lp.nty * lp.ntx : 0;
      s_plan[l] = lp;
    }
    s_items = rank;
    s_count = 0u;
  }
  __syncthreads();
  const int n_tiles = s_items;
  const int BG = p.n_img * p.G;

  const uint32_t gmax = p.state->go_max_bits;
  const bool finite = gmax < 0x7f800000u;
  const int e_go = (int)(gmax >> 23) - 126;                  // 2^e_go > max |grad_out|
  const int e_out = e_go - p.fix_bits;

  for (int item = blockIdx.x; item < n_tiles * BG; item += gridDim.x) {
    const int rank = item / BG, bg = item - rank * BG;
    const int b = bg / p.G, g = bg - b * p.G;
    int l = 0;
    for (int i = 0; i < p.L; ++i)
      if (s_plan[i].first_item_rank <= rank && (s_plan[i].H > 0 && s_plan[i].W > 0)) {
        // levels were ranked from the last one down: the matching level is the smallest index whose first rank <= rank
        l = i;
        break;
      }
    const LevelPlan lp = s_plan[l];
    const int t_in = rank - lp.first_item_rank;
    const int ty = t_in / lp.ntx, tx = t_in - ty * lp.ntx;
    const int ty0 = ty * lp.th, tx0 = tx * lp.tw;
    const int th = min(lp.th, lp.H - ty0), tw = min(lp.tw, lp.W - tx0);
    const int n_cells = th * tw;                             // <= cells_max; cell n_cells.. = trash

    for (int i = tid; i < n_acc; i += kThreads) acc[i] = 0ull;
    __syncthreads();

    const size_t QKp = fda_key_stride(p.Q, p.K);
    const uint32_t *keys = reinterpret_cast<const uint32_t *>(p.keys + ((size_t)(b * p.G + g) * p.L + l) * QKp);      // two keys per dword
    const int n_words = (int)(QKp / 2);
    const size_t sla_bg = ((size_t)b * p.Q * p.G + g) * 3 * LK;       // + q * G * 3LK
    const size_t go_bg = ((size_t)b * p.Q * p.G + g) * D;             // + q * G * D

    // exact position of point `pt` of this level, from sampling_loc_attn (dcnv4 convention: x first)
    auto position = [&](uint32_t pt, float &y, float &x, uint32_t &q) {
      q = pt / (uint32_t)p.K;
      const int k = (int)(pt - q * p.K);
      const size_t row = sla_bg + (size_t)q * p.G * 3 * LK;
      const int t = l * p.K + k;
      x = sub_rn(mul_rn(elem_at<Tag>(p.sla, row + 2 * t), (float)lp.W), 0.5f);       // flash_deform_im2col_cuda.cuh:188-189
      y = sub_rn(mul_rn(elem_at<Tag>(p.sla, row + 2 * t + 1), (float)lp.H), 0.5f);
    };

    // ---- apply the first `n` listed points, in batches.  What a batch needs from memory (position,
    // probability, grad_out rows) is requested one batch ahead, so the loads fly while the previous
    // batch is applied.
    const float *probs = p.probs + ((size_t)(b * p.G + g) * p.L + l) * QKp;
    constexpr int kParts = DP / 4;                           // 4-channel pieces of a grad_out row
    constexpr int kGoLoads = kBatch * kParts / kThreads;     // pieces per lane and batch (DP = 32: 2)
    static_assert(kBatch * kParts % kThreads == 0 || kBatch * kParts < kThreads, "grad_out pieces divide over the lanes");
    constexpr int kGoPerLane = kGoLoads > 0 ? kGoLoads : 1;
    // Everything is requested through range-checked buffer loads of raw words: no branches around
    // the loads, so they all fly together, and nothing is converted before it is needed.
    typedef typename RawWord<2 * Tag::kBytes>::type xy_t;      // (x, y) of a point are adjacent
    typedef typename RawWord<4 * Tag::kBytes>::type go4_t;     // 4 channels of grad_out
    const __amdgpu_buffer_rsrc_t sla_rs = make_rsrc(reinterpret_cast<const elem_t *>(p.sla) + sla_bg,
                                                    (uint32_t)((size_t)p.Q * p.G * 3 * LK * Tag::kBytes));
    const __amdgpu_buffer_rsrc_t go_rs = make_rsrc(reinterpret_cast<const elem_t *>(p.grad_out) + go_bg,
                                                   (uint32_t)((size_t)p.Q * p.G * D * Tag::kBytes));
    const __amdgpu_buffer_rsrc_t pr_rs = make_rsrc(probs, (uint32_t)QK * 4u);
    struct Ahead {
      xy_t xy;                         // lanes < batch size: their point
      uint32_t pr;
      go4_t go[kGoPerLane];
    };
    auto fetch = [&](uint32_t b0, int nb) {
      Ahead a;
      {
        const uint32_t pt = s_list[b0 + min(tid, max(nb - 1, 0))];
        const uint32_t q = pt / (uint32_t)p.K;
        const int t = l * p.K + (int)(pt - q * p.K);
        const bool live = tid < nb;
        a.xy = buffer_load<2 * Tag::kBytes>(sla_rs, live ? (q * (uint32_t)(p.G * 3 * LK) + 2u * t) * Tag::kBytes : kDropOffset);
        a.pr = buffer_load<4>(pr_rs, live ? pt * 4u : kDropOffset);
      }
#pragma unroll
      for (int u = 0; u < kGoPerLane; ++u) {
        const int i = tid + u * kThreads, h = i / kParts, part = i - h * kParts;
        const bool live = h < nb && i < kBatch * kParts && 4 * part < D;
        const uint32_t q = s_list[b0 + min(h, max(nb - 1, 0))] / (uint32_t)p.K;
        a.go[u] = buffer_load<4 * Tag::kBytes>(go_rs, live ? (q * (uint32_t)(p.G * D) + 4u * part) * Tag::kBytes : kDropOffset);
      }
      return a;
    };
    auto park = [&](const Ahead &a, int nb) {
      if (tid < nb) {          // one lane per point: corner weights and accumulator cells
        float xy[2];
        Pack<Tag, 2>::decode(a.xy, xy);
        const float x = sub_rn(mul_rn(xy[0], (float)lp.W), 0.5f);       // flash_deform_im2col_cuda.cuh:188-189
        const float y = sub_rn(mul_rn(xy[1], (float)lp.H), 0.5f);
        const Tap tp = make_tap(y, x, lp.H, lp.W, 0u, 0u);
        const float ps = ldexpf(__builtin_bit_cast(float, a.pr), p.fix_bits);
        const int ly = tp.y0 - ty0, lx = tp.x0 - tx0;
        uint32_t cells[4];
        float w[4];
#pragma unroll
        for (int cn = 0; cn < 4; ++cn) {
          const int cy = ly + (cn >> 1), cx = lx + (cn & 1);
          const bool ok = (tp.valid & (1u << cn)) && cy >= 0 && cy < th && cx >= 0 && cx < tw;
          cells[cn] = ok ? (uint32_t)(cy * tw + cx) : (uint32_t)n_cells;
          w[cn] = ok ? ps * tp.w[cn] : 0.f;
        }
        rec_w[tid] = f32x4{w[0], w[1], w[2], w[3]};
        rec_meta[tid] = u32x2{cells[0] | (cells[1] << kCellBitsF) | (cells[2] << (2 * kCellBitsF)), cells[3]};
      }
#pragma unroll
      for (int u = 0; u < kGoPerLane; ++u) {      // grad_out rows, normalised to [-1, 1] (zeros past the head width)
        const int i = tid + u * kThreads, h = i / kParts, part = i - h * kParts;
        if (h < nb && i < kBatch * kParts) {
          float g4[4];
          Pack<Tag, 4>::decode(a.go[u], g4);
          *reinterpret_cast<f32x4 *>(s_go + h * DP + 4 * part) =
              f32x4{ldexpf(g4[0], -e_go), ldexpf(g4[1], -e_go), ldexpf(g4[2], -e_go), ldexpf(g4[3], -e_go)};
        }
      }
    };
    auto apply_list = [&](uint32_t n) {
      if (n == 0) return;
      Ahead ahead = fetch(0, (int)min((uint32_t)kBatch, n));
      for (uint32_t b0 = 0; b0 < n; b0 += kBatch) {
        const int nb = (int)min((uint32_t)kBatch, n - b0);
        park(ahead, nb);
        __syncthreads();
        if (b0 + kBatch < n) ahead = fetch(b0 + kBatch, (int)min((uint32_t)kBatch, n - b0 - kBatch));
        // a row of 8 lanes per point; row r starts its channel blocks at (r mod CPL), so the rows of one
        // instruction spread over the banks
        const int row_in_block = tid / kRowLanes, c = tid & (kRowLanes - 1);
        for (int h = row_in_block; h < nb; h += kThreads / kRowLanes) {
          const f32x4 w = rec_w[h];
          const u32x2 meta = rec_meta[h];
          const uint32_t cells[4] = {meta.x & 511u, (meta.x >> kCellBitsF) & 511u, (meta.x >> (2 * kCellBitsF)) & 511u, meta.y & 511u};
          const float wv[4] = {w.x, w.y, w.z, w.w};
          float gn[CPL];
          int ch_off[CPL];
#pragma unroll
          for (int j = 0; j < CPL; ++j) {
            ch_off[j] = kRowLanes * ((j + row_in_block) & (CPL - 1));
            gn[j] = s_go[h * DP + c + ch_off[j]];
          }
#pragma unroll
          for (int cn = 0; cn < 4; ++cn) {
            unsigned long long *dst = acc + __umul24(cells[cn], (uint32_t)DP) + c;
#pragma unroll
            for (int j = 0; j < CPL; ++j)
              __hip_atomic_fetch_add(dst + ch_off[j], to_fixed64<Tag::kBytes == 4>(gn[j] * wv[cn]), __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_WORKGROUP);
          }
        }
        __syncthreads();
      }
    };

    // ---- scan the keys of (image, head, level); flush the list whenever another step might overflow it
    if (finite && gmax != 0u) {
      // A step = kScanPerLane dwords (two keys each) per lane, loaded in one go (and one step ahead) so that
      // the memory latency is paid once per step; the step is then tested in rounds of kRoundKeys dwords per
      // lane, few enough that the list can always take a whole round.
      auto load_keys = [&](int base, uint32_t (&key)[kScanPerLane]) {
#pragma unroll
        for (int u = 0; u < kScanPerLane; ++u) {
          const int i = base + u * kThreads + tid;
          key[u] = keys[min(i, n_words - 1)];             // points past the end are masked when tested
        }
      };
      uint32_t key[kScanPerLane], key_next[kScanPerLane];
      load_keys(0, key_next);
      for (int base = 0; base < n_words; base += kScanStep) {
#pragma unroll
        for (int u = 0; u < kScanPerLane; ++u) key[u] = key_next[u];
        if (base + kScanStep < n_words) load_keys(base + kScanStep, key_next);      // in flight while this step is tested
        // a real loop (the flush below must not be replicated per round): each round tests key[0..kRoundKeys)
        // and then shifts the rest of the step's keys down
#pragma unroll 1
        for (int r = 0; r < kScanPerLane / kRoundKeys; ++r) {
          // test the round's points first, then reserve list slots for all of them with one LDS atomic per wave
          uint64_t masks[2 * kRoundKeys];
          uint32_t total = 0;
#pragma unroll
          for (int uu = 0; uu < 2 * kRoundKeys; ++uu) {
            const uint32_t k16 = (key[uu >> 1] >> (16 * (uu & 1))) & 0xffffu;
            const uint32_t pt = 2u * (uint32_t)(base + (r * kRoundKeys + (uu >> 1)) * kThreads + tid) + (uu & 1);
            bool hit = false;
            if (pt >= (uint32_t)QK) {
            } else if (k16 == kFdaKeySaturated) {                   // position beyond the key's fields: exact test
              float y, x;
              uint32_t q;
              position(pt, y, x, q);
              const Tap tp = make_tap(y, x, lp.H, lp.W, 0u, 0u);
              hit = tp.valid != 0 && tp.y0 + 1 >= ty0 && tp.y0 < ty0 + th && tp.x0 + 1 >= tx0 && tp.x0 < tx0 + tw;
            } else if (k16 != kFdaKeyOutside) {
              // key = (y0 + 1) << 8 | (x0 + 1); the corner block {x0, x0 + 1} meets [tx0, tx0 + tw) iff 0 <= x0 + 1 - tx0 <= tw
              hit = (uint32_t)((int)(k16 & 0xffu) - tx0) <= (uint32_t)tw && (uint32_t)((int)(k16 >> 8) - ty0) <= (uint32_t)th;
            }
            masks[uu] = __builtin_amdgcn_ballot_w64(hit);
            total += (uint32_t)__builtin_popcountll(masks[uu]);
          }
          if (total != 0) {
            uint32_t slot0 = 0;
            if (lane == 0) slot0 = atomicAdd(&s_count, total);
            slot0 = __builtin_amdgcn_readfirstlane(slot0);
#pragma unroll
            for (int uu = 0; uu < 2 * kRoundKeys; ++uu) {
              const uint64_t mask = masks[uu];
              if ((mask >> lane) & 1) {
                const uint32_t pt = 2u * (uint32_t)(base + (r * kRoundKeys + (uu >> 1)) * kThreads + tid) + (uu & 1);
                s_list[slot0 + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u))] = pt;
              }
              slot0 += (uint32_t)__builtin_popcountll(mask);
            }
          }
          __syncthreads();
          const uint32_t n = s_count;
          const bool last = base + kScanStep >= n_words && r == kScanPerLane / kRoundKeys - 1;
          if (n > (uint32_t)(kListCap - 2 * kRoundKeys * kThreads) || last) {
            __syncthreads();                // everyone has read the count
            if (tid == 0) s_count = 0u;
            apply_list(n);                  // ends with a barrier
          }
#pragma unroll
          for (int u = 0; u + kRoundKeys < kScanPerLane; ++u) key[u] = key[u + kRoundKeys];
        }
      }
    }
    __syncthreads();

    // ---- the tile is complete (zeros when the statistics are unusable: the caller then runs the atomic path)
    elem_t *gv = reinterpret_cast<elem_t *>(p.grad_value);
    for (int i = tid; i < n_cells * D; i += kThreads) {
      const int cell = i / D, ch = i - cell * D;
      const int cy = cell / tw, cx = cell - cy * tw;
      const unsigned long long a = acc[cell * DP + ch];
      const double v = ldexp((double)(int)(a >> 32) * 4294967296.0 + (double)(uint32_t)a, e_out);
      const float f[1] = {(float)v};
      gv[(((size_t)b * p.N + lp.start + (size_t)(ty0 + cy) * lp.W + tx0 + cx) * p.G + g) * D + ch] = Pack<Tag, 1>::encode(f);
    }
    __syncthreads();
  }
}

template <typename Tag>
hipError_t launch_t(const FdaLaunch &p, hipStream_t stream) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) {
    int v = 0;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && v > 0) cus = v;
  }
  const dim3 grid((unsigned)cus), block(kThreads);
  const size_t lds = fda_grad_value_lds_bytes(p);
  auto go = [&](auto kernel) -> hipError_t {
    static bool raised = false;
    if (!raised) {
      if (hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLdsPerWorkgroup - 2048))
        return e;
      raised = true;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return hipGetLastError();
  };
  switch (fda_padded_channels(p.D) / kRowLanes) {
    case 1: return go(fda_grad_value_kernel<Tag, 1>);
    case 2: return go(fda_grad_value_kernel<Tag, 2>);
    case 4: return go(fda_grad_value_kernel<Tag, 4>);
  }
  return hipErrorInvalidValue;      // wider heads take the atomic path (the entry point checks)
}

}  // namespace

size_t fda_grad_value_lds_bytes(const FdaLaunch &p) {
  const size_t dp = (size_t)fda_padded_channels(p.D);
  return ((size_t)fda_tile_cells(p.D) + 1) * dp * sizeof(unsigned long long) + kBatch * (sizeof(f32x4) + sizeof(u32x2)) +
         kBatch * dp * sizeof(float) + (size_t)kListCap * sizeof(uint32_t);
}

hipError_t launch_fda_grad_value(int dtype, const FdaLaunch &p, hipStream_t stream) {
  switch (dtype) {
    case F32::kCode: return launch_t<F32>(p, stream);
    case F16::kCode: return launch_t<F16>(p, stream);
    case BF16::kCode: return launch_t<BF16>(p, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace dcn
