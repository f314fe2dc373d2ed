// Device-side building blocks shared by the DCNv4 and flash-deformable-attention kernels
// (gfx950 / CDNA4, wave64).  Counterpart of the reference's DCNv4_op/src/cuda/common.h:41-212
// (bilinear gather, bilinear scatter + coordinate partials), rebuilt around CDNA buffer
// addressing: every gather and scatter goes through a raw buffer descriptor whose range check
// turns an out-of-image corner into a zero load / dropped atomic, so the hot loop has no
// divergent branches and no clamped addresses.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dcn {

typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// dtype tags; the numeric values are the dtype codes of the C ABI
struct F32 { static constexpr int kBytes = 4; static constexpr int kCode = 0; };
struct F16 { static constexpr int kBytes = 2; static constexpr int kCode = 1; };
struct BF16 { static constexpr int kBytes = 2; static constexpr int kCode = 2; };

constexpr int kWave = 64;
constexpr int kXcds = 8;                      // MI355X: 8 accelerator dies, one L2 each
constexpr uint32_t kDropOffset = 0x80000000u; // >= num_records of every descriptor we build

// ---------------------------------------------------------------- raw words of N bytes
template <int BYTES> struct RawWord;
template <> struct RawWord<2> { typedef uint16_t type; };
template <> struct RawWord<4> { typedef uint32_t type; };
template <> struct RawWord<8> { typedef u32x2 type; };
template <> struct RawWord<16> { typedef u32x4 type; };

// Raw buffer descriptor over [base, base+bytes): untyped, no swizzle, range-checked.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

template <int BYTES>
__device__ __forceinline__ typename RawWord<BYTES>::type buffer_load(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  if constexpr (BYTES == 2) return __builtin_amdgcn_raw_buffer_load_b16(r, off, 0, 0);
  else if constexpr (BYTES == 4) return __builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0);
  else if constexpr (BYTES == 8) return __builtin_amdgcn_raw_buffer_load_b64(r, off, 0, 0);
  else return __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
}

// ---------------------------------------------------------------- element <-> fp32 conversion
// N contiguous elements of dtype Tag, held as one raw word, to / from N floats.
template <typename Tag, int N> struct Pack {
  static constexpr int kBytes = N * Tag::kBytes;
  typedef typename RawWord<kBytes>::type raw_t;

  static __device__ __forceinline__ void decode(raw_t raw, float (&out)[N]) {
    if constexpr (Tag::kBytes == 4) {
      // element reads go through by-value helpers: bit-casting a vector-subscript lvalue
      // directly was observed to read lane 0 of the vector for every index
      if constexpr (N == 1) out[0] = word_to_float(raw);
      else {
#pragma unroll
        for (int i = 0; i < N; ++i) out[i] = word_to_float(raw[i]);
      }
    } else if constexpr (N == 1) {
      out[0] = half_bits_to_float((uint32_t)raw);
    } else if constexpr (N == 2) {
      pair_to_float(raw, out[0], out[1]);
    } else {
#pragma unroll
      for (int i = 0; i < N / 2; ++i) pair_to_float(raw[i], out[2 * i], out[2 * i + 1]);
    }
  }

  static __device__ __forceinline__ raw_t encode(const float (&in)[N]) {
    raw_t raw;
    if constexpr (Tag::kBytes == 4) {
      if constexpr (N == 1) raw = float_to_word(in[0]);
      else {
#pragma unroll
        for (int i = 0; i < N; ++i) raw[i] = float_to_word(in[i]);
      }
    } else if constexpr (N == 1) {
      raw = (uint16_t)(float_pair_to_bits(in[0], 0.f) & 0xffffu);
    } else if constexpr (N == 2) {
      raw = float_pair_to_bits(in[0], in[1]);
    } else {
#pragma unroll
      for (int i = 0; i < N / 2; ++i) raw[i] = float_pair_to_bits(in[2 * i], in[2 * i + 1]);
    }
    return raw;
  }

 private:
  static __device__ __forceinline__ float word_to_float(uint32_t w) { return __builtin_bit_cast(float, w); }
  static __device__ __forceinline__ uint32_t float_to_word(float f) { return __builtin_bit_cast(uint32_t, f); }
  static __device__ __forceinline__ float half_bits_to_float(uint32_t bits) {
    if constexpr (Tag::kCode == F16::kCode) return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
    else return __builtin_bit_cast(float, bits << 16);
  }
  static __device__ __forceinline__ void pair_to_float(uint32_t bits, float &lo, float &hi) {
    if constexpr (Tag::kCode == F16::kCode) {
      f16x2 h = __builtin_bit_cast(f16x2, bits);
      lo = (float)h.x; hi = (float)h.y;
    } else {
      lo = __builtin_bit_cast(float, bits << 16);
      hi = __builtin_bit_cast(float, bits & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ uint32_t float_pair_to_bits(float lo, float hi) {
    f32x2 f = {lo, hi};
    if constexpr (Tag::kCode == F16::kCode) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
    else return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
  }
};

// ---------------------------------------------------------------- coordinate arithmetic
// Sampling coordinates are formed in fp32 one rounded operation at a time, in the reference's
// source order (dcnv4_im2col_cuda.cuh:203-224, flash_deform_im2col_cuda.cuh:188-189), never
// fused: a coordinate that differs by one ulp moves every bilinear weight of the tap, which
// is visible at the fp32 forward tolerance.
// (the pragma keeps the compiler from contracting a product with a later sum into one fma)
__device__ __forceinline__ float mul_rn(float a, float b) {
#pragma clang fp contract(off)
  return a * b;
}
__device__ __forceinline__ float add_rn(float a, float b) {
#pragma clang fp contract(off)
  return a + b;
}
__device__ __forceinline__ float sub_rn(float a, float b) {
#pragma clang fp contract(off)
  return a - b;
}

// ---------------------------------------------------------------- bilinear tap
// Corner order: (y0,x0) (y0,x0+1) (y0+1,x0) (y0+1,x0+1), as common.h:48-58.
// `off` are byte offsets into the descriptor, kDropOffset for a corner outside the image
// (and for all four when the tap fails the range test of dcnv4_im2col_cuda.cuh:227).
struct Tap {
  uint32_t off[4];
  float w[4];
  float ly, lx;     // fractional parts; d w / d y = (-hx,-lx,hx,lx), d w / d x = (-hy,hy,-ly,ly)
  int y0, x0;       // integer position of corner 0 (-1 .. H-1 / W-1 when the tap is inside)
  uint32_t valid;   // bit c set when corner c lies inside the image
};

// base = byte offset of (image, row 0, col 0, this lane's channels); pix_bytes = bytes per pixel.
__device__ __forceinline__ Tap make_tap(float y, float x, int H, int W, uint32_t base, uint32_t pix_bytes) {
  Tap t;
  const bool inside = (y > -1.f) && (x > -1.f) && (y < (float)H) && (x < (float)W);
  y = inside ? y : 0.f;            // also scrubs NaN / huge coordinates before the int conversion
  x = inside ? x : 0.f;
  const float fy = floorf(y), fx = floorf(x);
  const int y0 = (int)fy, x0 = (int)fx;
  const float ly = y - fy, lx = x - fx, hy = 1.f - ly, hx = 1.f - lx;
  t.ly = ly; t.lx = lx;
  t.w[0] = hy * hx; t.w[1] = hy * lx; t.w[2] = ly * hx; t.w[3] = ly * lx;
  const bool top = inside && y0 >= 0, bot = inside && (y0 + 1 < H);
  const bool lef = x0 >= 0, rig = x0 + 1 < W;
  const uint32_t o00 = base + (uint32_t)(y0 * W + x0) * pix_bytes;   // wraps harmlessly when dropped
  const uint32_t row = (uint32_t)W * pix_bytes;
  t.off[0] = (top && lef) ? o00 : kDropOffset;
  t.off[1] = (top && rig) ? o00 + pix_bytes : kDropOffset;
  t.off[2] = (bot && lef) ? o00 + row : kDropOffset;
  t.off[3] = (bot && rig) ? o00 + row + pix_bytes : kDropOffset;
  t.y0 = y0; t.x0 = x0;
  t.valid = (uint32_t)(top && lef) | ((uint32_t)(top && rig) << 1) | ((uint32_t)(bot && lef) << 2) |
            ((uint32_t)(bot && rig) << 3);
  return t;
}

__device__ __forceinline__ int ceil_div_signed(int a, int b) {    // b > 0
  return a >= 0 ? (a + b - 1) / b : -((-a) / b);
}

// ---------------------------------------------------------------- small shared helpers
// Running max and reciprocal sum for a softmax over n logits held in LDS.
__device__ __forceinline__ void softmax_stats(const float *m, int n, float &mx, float &inv) {
  mx = m[0];
  for (int k = 1; k < n; ++k) mx = fmaxf(mx, m[k]);
  float s = 0.f;
  for (int k = 0; k < n; ++k) s += __expf(m[k] - mx);
  inv = 1.f / s;
}

// Kernel-tap decode for a 3x3 kernel with (kp == 8) or without (kp == 9) the centre removed:
// x index i outer, y index j inner (dcnv4_im2col_cuda.cuh:216-236).
__device__ __forceinline__ void tap_ij_3x3(int kp, int k, int &i, int &j) {
  const int kk = (kp == 8 && k >= 4) ? k + 1 : k;
  i = kk / 3; j = kk - 3 * i;
}

// ---------------------------------------------------------------- cross-lane sums
// Sum over an aligned cluster of `width` (power of two) adjacent lanes; every lane of the
// cluster ends with the total.  xor-1 / xor-2 stay inside a quad and use DPP quad_perm.
__device__ __forceinline__ float dpp_quad_xor1(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, true));
}
// Inside a row of 16 lanes the two further steps are DPP mirrors: once every lane holds its quad's sum, the lane
// mirrored within 8 (then within 16) lies in the other quad (the other half), so adding it doubles the span just as
// xor-4 (xor-8) would, without the LDS crossbar.
__device__ __forceinline__ float dpp_row_half_mirror(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, true));
}
__device__ __forceinline__ float dpp_row_mirror(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, true));
}
__device__ __forceinline__ float cluster_sum(float v, int width) {
  if (width >= 2) v += dpp_quad_xor1(v);
  if (width >= 4) v += dpp_quad_xor2(v);
  if (width >= 8) v += dpp_row_half_mirror(v);
  if (width >= 16) v += dpp_row_mirror(v);
  for (int o = 16; o < width; o <<= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// ---------------------------------------------------------------- wave reductions
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
  for (int o = 32; o > 0; o >>= 1) v = max(v, (uint32_t)__shfl_xor((int)v, o, kWave));
  return v;
}

// ---------------------------------------------------------------- workgroup -> tile order
// Hardware hands consecutive workgroup ids to the 8 XCDs round-robin.  Remap so that each XCD
// walks one contiguous eighth of the tile sequence: neighbouring tiles then share that XCD's L2.
__device__ __forceinline__ uint32_t xcd_contiguous_block(uint32_t bid, uint32_t nblocks) {
  const uint32_t per = nblocks / kXcds, rem = nblocks % kXcds;
  const uint32_t xcd = bid % kXcds, idx = bid / kXcds;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

// ---------------------------------------------------------------- LDS staging of packed rows
// Per-query parameter rows (offset_mask / sampling_loc_attn) are contiguous in memory for the
// consecutive queries one workgroup owns: stream them once with 128-bit coalesced loads,
// widen to fp32 and park them in LDS, where all channel lanes of a (query, group) share them.
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <typename Tag>
__device__ __forceinline__ void stage_rows_to_lds(float *dst, const void *src, int n_elem, bool vec16) {
  constexpr int EPV = 16 / Tag::kBytes;
  if (vec16) {
    const u32x4 *s = reinterpret_cast<const u32x4 *>(src);
    for (int i = threadIdx.x; i < n_elem / EPV; i += blockDim.x) {
      float f[EPV];
      Pack<Tag, EPV>::decode(__builtin_nontemporal_load(s + i), f);
#pragma unroll
      for (int j = 0; j < EPV; j += 4)
        *reinterpret_cast<f32x4 *>(dst + i * EPV + j) = f32x4{f[j], f[j + 1], f[j + 2], f[j + 3]};
    }
  } else {
    typedef typename RawWord<Tag::kBytes>::type elem_t;
    const elem_t *s = reinterpret_cast<const elem_t *>(src);
    for (int i = threadIdx.x; i < n_elem; i += blockDim.x) {
      float f[1];
      Pack<Tag, 1>::decode(s[i], f);
      dst[i] = f[0];
    }
  }
}

template <typename Tag>
__device__ __forceinline__ void unstage_rows_from_lds(void *dst, const float *src, int n_elem, bool vec16) {
  constexpr int EPV = 16 / Tag::kBytes;
  if (vec16) {
    u32x4 *d = reinterpret_cast<u32x4 *>(dst);
    for (int i = threadIdx.x; i < n_elem / EPV; i += blockDim.x) {
      float f[EPV];
#pragma unroll
      for (int j = 0; j < EPV; j += 4) {
        const f32x4 v = *reinterpret_cast<const f32x4 *>(src + i * EPV + j);
        f[j] = v.x; f[j + 1] = v.y; f[j + 2] = v.z; f[j + 3] = v.w;
      }
      d[i] = Pack<Tag, EPV>::encode(f);
    }
  } else {
    typedef typename RawWord<Tag::kBytes>::type elem_t;
    elem_t *d = reinterpret_cast<elem_t *>(dst);
    for (int i = threadIdx.x; i < n_elem; i += blockDim.x) {
      const float f[1] = {src[i]};
      d[i] = Pack<Tag, 1>::encode(f);
    }
  }
}

}  // namespace dcn
