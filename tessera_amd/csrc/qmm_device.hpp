// Device-side helpers shared by the gfx950 quantized-matmul kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace qmm {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef int int8v_t __attribute__((ext_vector_type(8)));
typedef int int4v_t __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
constexpr uint32_t kQ4KBlockBytes = 144;
constexpr uint32_t kQ4KBlockElems = 256;

template <class To, class From>
__device__ __forceinline__ To bit_cast(const From& v) {
  static_assert(sizeof(To) == sizeof(From), "size mismatch");
  return __builtin_bit_cast(To, v);
}

// binary16 bits -> fp32; exact for every input (hardware v_cvt_f32_f16).
__device__ __forceinline__ float half_bits_to_float(uint32_t bits16) {
  return static_cast<float>(bit_cast<_Float16>(static_cast<uint16_t>(bits16)));
}

// E8M0 shared exponent -> 2^(s-127).  s = 0 is the fp32 subnormal 2^-127; s = 255
// yields +inf like ldexp would overflow to (it does not occur in real weights).
__device__ __forceinline__ float e8m0_to_float(uint32_t s) {
  return bit_cast<float>(s == 0u ? 0x00400000u : (s << 23));
}

// OCP FP8 E4M3 byte -> fp32 (bias 7, subnormals m*2^-9, 0x7F/0xFF NaN).
__device__ __forceinline__ float e4m3_to_float(uint32_t c) {
  const uint32_t e = (c >> 3) & 15u, m = c & 7u;
  float v;
  if (e == 0u) {
    v = static_cast<float>(m) * 0x1p-9f;
  } else if (e == 15u && m == 7u) {
    v = bit_cast<float>(0x7FC00000u);
  } else {
    v = bit_cast<float>(((e + 120u) << 23) | (m << 20));
  }
  return (c & 0x80u) ? -v : v;
}

// OCP E2M1 nibble -> fp32: {0, .5, 1, 1.5, 2, 3, 4, 6}, bit 3 = sign.
__device__ __forceinline__ float e2m1_to_float(uint32_t nib) {
  const uint32_t e = (nib >> 1) & 3u, m = nib & 1u;
  float v = e == 0u ? 0.5f * static_cast<float>(m)
                    : bit_cast<float>(((e + 126u) << 23) | (m << 22));
  return (nib & 8u) ? -v : v;
}

// fp32 -> OCP FP8 E4M3 byte, round to nearest even; NaN and |x| > 448 -> 0x7F|sign.
// Integer-only restatement of the reference encoder
// (src/core/numerics/quant.cpp:299-342): a value below 2^-6 rounds on the
// subnormal grid of 2^-9, anything else on a 3-bit mantissa, a mantissa carry bumps
// the exponent.  Like the reference, the subnormal branch caps at mantissa 7, so
// [7.5 * 2^-9, 2^-6) encodes as 0x07 rather than rounding up to the normal 0x08.
__device__ __forceinline__ uint32_t float_to_e4m3(float v) {
  const uint32_t b = bit_cast<uint32_t>(v);
  const uint32_t sign = (b >> 24) & 0x80u;
  const uint32_t mag = b & 0x7FFFFFFFu;
  if (mag > 0x43E00000u) {  // above 448, inf or NaN
    return sign | 0x7Fu;
  }
  if (mag < 0x3C800000u) {  // below 2^-6: subnormal grid, RNE via the fp32 adder
    const float a = bit_cast<float>(mag);
    const uint32_t m = static_cast<uint32_t>(__builtin_rintf(a * 512.0f));
    return sign | (m > 7u ? 7u : m);
  }
  // Normal: keep 3 mantissa bits with RNE; the carry propagates into the exponent.
  const uint32_t r = mag + 0x7FFFFu + ((mag >> 20) & 1u);
  const uint32_t code = (r >> 20) - (120u << 3);
  return sign | (code > 0x7Eu ? 0x7Eu : code);
}

// Sum over the 64 lanes of a wavefront; every lane returns the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    v += __shfl_xor(v, off, kWave);
  }
  return v;
}

// DPP add: v + (v moved across lanes by `ctrl`); lanes the move does not reach add 0.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, bit_cast<int>(v), kCtrl, kRowMask, 0xF, false);
  return v + bit_cast<float>(moved);
}

// Sum over the 64 lanes using DPP only (no LDS crossbar): xor-butterflies inside each
// row of 16 lanes, then row broadcasts.  The total is valid in lane 63.
__device__ __forceinline__ float wave_sum_last(float v) {
  v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
  v = dpp_add<0x140, 0xF>(v);  // row_mirror: every lane holds its row's sum
  v = dpp_add<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Sum over each aligned run of 16 lanes (a DPP row); every lane of the run returns its total.
// A run must be active or idle as a whole.
__device__ __forceinline__ float row16_sum(float v) {
  v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
  v = dpp_add<0x140, 0xF>(v);  // row_mirror
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    v = fmaxf(v, __shfl_xor(v, off, kWave));
  }
  return v;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every
// outstanding global load (its fence covers all address spaces), which would drain a
// register prefetch pipeline at every barrier.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ uint4 load_u4(const void* p) {
  return *reinterpret_cast<const uint4*>(p);
}

}  // namespace qmm
