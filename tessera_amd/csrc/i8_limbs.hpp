// Activations as signed 8-bit limbs for the int8 matrix cores: the pieces shared by the kernels that
// multiply Q4_K / Q5_K / Q6_K quants with fp32 activations on v_mfma_i32_16x16x64_i8.
#pragma once

#include "qmm_device.hpp"

namespace qmm {
namespace i8limbs {

constexpr uint32_t kSlot = 1024u + 32u + 16u;   // limbs of a block, eight sub-block sums, the shift

template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_move(float v) {
  return bit_cast<float>(__builtin_amdgcn_update_dpp(0, bit_cast<int>(v), kCtrl, kRowMask, 0xF, false));
}

// 24-bit multiply-add (v_mad_i32_i24); written in C so that the compiler keeps track of the wait
// states between a matrix instruction and the first read of its result.
__device__ __forceinline__ int mad24(int a, int b, int c) { return ((a << 8) >> 8) * ((b << 8) >> 8) + c; }

// 256 activations (four per lane) -> a private LDS slot: for sub-block s, lane half h, limb m the 16
// bytes at s*128 + h*64 + m*16 (the A operand of one matrix row), then the sums of the even and of
// the odd sub-blocks, then the shift: limbs = round(x * 2^sh), sh = 29 - exponent of the block's
// largest magnitude, as sum_m L_m 256^m with every L_m a signed byte.
__device__ __forceinline__ void convert_block(const float4 v, uint32_t lane, uint8_t* slot) {
  float m = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
  m = fmaxf(m, dpp_move<0xB1, 0xF>(m));
  m = fmaxf(m, dpp_move<0x4E, 0xF>(m));
  m = fmaxf(m, dpp_move<0x141, 0xF>(m));
  m = fmaxf(m, dpp_move<0x140, 0xF>(m));
  m = fmaxf(m, dpp_move<0x142, 0xA>(m));
  m = fmaxf(m, dpp_move<0x143, 0xC>(m));
  const uint32_t mb = __builtin_amdgcn_readlane(bit_cast<int>(m), 63);
  const int sh = 156 - static_cast<int>((mb >> 23) & 0xFFu);
  const float xv[4] = {v.x, v.y, v.z, v.w};
  uint32_t L[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int X = static_cast<int>(__builtin_rintf(__builtin_ldexpf(xv[i], sh)));
    // bytes of X as signed digits: add 128 to every byte, then flip the top bits back
    L[i] = (static_cast<uint32_t>(X) + 0x80808080u) ^ 0x80808080u;
  }
  // 4 x 4 byte transpose: limb m of the lane's four values into one register
  const uint32_t t0 = __builtin_amdgcn_perm(L[1], L[0], 0x05010400u);
  const uint32_t t1 = __builtin_amdgcn_perm(L[1], L[0], 0x07030602u);
  const uint32_t t2 = __builtin_amdgcn_perm(L[3], L[2], 0x05010400u);
  const uint32_t t3 = __builtin_amdgcn_perm(L[3], L[2], 0x07030602u);
  const uint32_t s = lane >> 3;
  uint32_t* dst = reinterpret_cast<uint32_t*>(slot + s * 128u + ((lane >> 2) & 1u) * 64u + (lane & 3u) * 4u);
  dst[0] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
  dst[4] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
  dst[8] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
  dst[12] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
  float sum = (v.x + v.y) + (v.z + v.w);
  sum += dpp_move<0xB1, 0xF>(sum);
  sum += dpp_move<0x4E, 0xF>(sum);
  sum += dpp_move<0x141, 0xF>(sum);
  if ((lane & 7u) == 0u) reinterpret_cast<float*>(slot + 1024u)[(s & 1u) * 4u + (s >> 1)] = sum;
  if (lane == 0u) reinterpret_cast<int*>(slot + 1056u)[0] = sh;
}

}  // namespace i8limbs
}  // namespace qmm
