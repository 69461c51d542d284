// Pieces shared by the Q4_K matrix-core kernels (the prefill GEMM and the routed-expert kernels):
// direct HBM -> LDS loads, the power-of-two row scale of the fp16 activation copies, the
// in-register super-block decode (src/core/numerics/quant.cpp:58-70,656-675) and the tile loop.
#pragma once

#include <type_traits>

#include "qmm_device.hpp"

namespace qmm {
namespace {

__device__ __forceinline__ void direct_load16(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// Largest |v| over a 256-thread workgroup (every thread returns it).
__device__ __forceinline__ float block_amax(float v, float* red) {
  v = wave_max(v);
  if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  const float r = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  return r;
}

// Power-of-two scale that brings a row with largest magnitude `amax` to [1024, 2048): the
// fp16 copy then neither overflows nor loses small values to subnormals, and the scaling itself
// is exact.  Zero rows (and non-finite ones) get scale 1.
__device__ __forceinline__ float row_scale_for(float amax) {
  const uint32_t e = (bit_cast<uint32_t>(amax) >> 23) & 0xFFu;
  if (e == 0u || e == 0xFFu) return 1.0f;
  const int se = static_cast<int>(e) - 10;
  return bit_cast<float>(static_cast<uint32_t>(se < 1 ? 1 : se) << 23);
}

__device__ __forceinline__ half8_t to_f16_group(const float4& lo, const float4& hi, float inv) {
  // the order 0,2,1,3,4,6,5,7 inside each group of 8 (what the in-register weight decode yields)
  half8_t v;
  v[0] = static_cast<_Float16>(lo.x * inv), v[1] = static_cast<_Float16>(lo.z * inv);
  v[2] = static_cast<_Float16>(lo.y * inv), v[3] = static_cast<_Float16>(lo.w * inv);
  v[4] = static_cast<_Float16>(hi.x * inv), v[5] = static_cast<_Float16>(hi.z * inv);
  v[6] = static_cast<_Float16>(hi.y * inv), v[7] = static_cast<_Float16>(hi.w * inv);
  return v;
}

// body(integral_constant<int, 0>) ... body(integral_constant<int, N - 1>), in order.
template <int N, int I = 0, typename F>
__device__ __forceinline__ void unrolled(F&& body) {
  if constexpr (I < N) {
    body(std::integral_constant<int, I>{});
    unrolled<N, I + 1>(body);
  }
}

// Two packed fp16 weights RN16(fma(q, dsc, ndmm)) from the nibbles (low: HI = 0, high: HI = 1) of
// bytes 0 and 2 of `x`.  A nibble masked in place inside a 16-bit half is the fp16 subnormal
// q * 2^-24 (16 q * 2^-24 for a high nibble), which the mixed-precision multiply-add reads as it
// is: `dsc24` is d*sc * 2^24 (d*sc * 2^20 for high nibbles), so the fp32 result is exactly
// DequantizeQ4K's and one instruction per weight forms it and rounds it to fp16.
template <int HI>
__device__ __forceinline__ half2_t decode_pair(uint32_t x, float dsc24, float ndmm) {
  const half2_t q = bit_cast<half2_t>(x & (HI ? 0x00F000F0u : 0x000F000Fu));
  return half2_t{static_cast<_Float16>(fmaf(static_cast<float>(q[0]), dsc24, ndmm)),
                 static_cast<_Float16>(fmaf(static_cast<float>(q[1]), dsc24, ndmm))};
}

// The 6-bit scales and mins of a super-block, one byte each (src/core/numerics/quant.cpp:58-70):
// sc[0], mn[0] hold sub-blocks 0..3, sc[1], mn[1] sub-blocks 4..7.
struct ScaleBytes {
  uint32_t sc[2], mn[2];
};
__device__ __forceinline__ ScaleBytes unpack_scales(uint32_t s0, uint32_t s1, uint32_t s2) {
  ScaleBytes r;
  r.sc[0] = s0 & 0x3F3F3F3Fu;
  r.mn[0] = s1 & 0x3F3F3F3Fu;
  r.sc[1] = (s2 & 0x0F0F0F0Fu) | ((s0 >> 2) & 0x30303030u);
  r.mn[1] = ((s2 >> 4) & 0x0F0F0F0Fu) | ((s1 >> 2) & 0x30303030u);
  return r;
}

// (d * sc * 2^24, -(dmin * mn)) of sub-block SB in fp32, both exact (11-bit header times 6-bit
// integer; the 2^24 undoes the subnormal reading of the nibbles in decode_pair).  Odd sub-blocks
// live in the high nibbles, which read as 16 q: their factor is 2^20.
struct ScaleMin {
  float dsc, ndmm;
};
template <int SB>
__device__ __forceinline__ ScaleMin scale_min_f32(const ScaleBytes& sbytes, float d, float ndmin) {
  const float sc = static_cast<float>((sbytes.sc[SB >> 2] >> (8 * (SB & 3))) & 0xFFu);
  const float mn = static_cast<float>((sbytes.mn[SB >> 2] >> (8 * (SB & 3))) & 0xFFu);
  return ScaleMin{d * sc * ((SB & 1) ? 0x1p20f : 0x1p24f), ndmin * mn};
}

// Header of the super-block at `raw` (a lane's weight row inside a raw LDS stage): d, -dmin and
// the unpacked 6-bit scales and mins.
struct BlockHead {
  float d, ndmin;
  ScaleBytes sbytes;
};
__device__ __forceinline__ BlockHead load_block_head(const uint8_t* raw) {
  const uint4 head = *reinterpret_cast<const uint4*>(raw);
  return BlockHead{half_bits_to_float(head.x & 0xFFFFu), -half_bits_to_float(head.x >> 16),
                   unpack_scales(head.y, head.z, head.w)};
}

// The B operands of sub-block SB (32 weights of one row) for a lane of K half `kg`: b[t] holds
// the weights 16kg + 8t + [0,8) in the order 0,2,1,3,4,6,5,7 (any assignment of the sub-block's K
// positions to matrix steps and lane halves will do as long as the activation fragments follow it;
// this one lets a lane take its sixteen bytes with ONE 16-byte LDS read, which sixteen lanes 144
// bytes apart make without a bank conflict, where two 8-byte reads a lane put lanes l and l + 16 on
// the same banks).  Sub-block SB lives in the low (even SB) or high nibbles of bytes
// (SB/2)*32 + [0,32) (src/core/numerics/quant.cpp:656-675); an odd SB decodes the bytes its even
// predecessor loaded, so `qw` (the words) and `qs8` (the same shifted down one byte, for bytes 1
// and 3) are carried from that call.
template <int SB>
__device__ __forceinline__ void decode_subblock(const uint8_t* raw, uint32_t kg, const BlockHead& h, uint32_t (&qw)[4],
                                                uint32_t (&qs8)[4], half8_t (&b)[2]) {
  constexpr int kHi = SB & 1;
  const ScaleMin sm = scale_min_f32<SB>(h.sbytes, h.d, h.ndmin);
  if (kHi == 0) {
    const uint4 q = *reinterpret_cast<const uint4*>(raw + 16 + (SB >> 1) * 32 + kg * 16u);
    qw[0] = q.x, qw[1] = q.y, qw[2] = q.z, qw[3] = q.w;
#pragma unroll
    for (int x = 0; x < 4; ++x) qs8[x] = qw[x] >> 8;
  }
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) {
    const half2_t p0 = decode_pair<kHi>(qw[2 * tt], sm.dsc, sm.ndmm), p1 = decode_pair<kHi>(qs8[2 * tt], sm.dsc, sm.ndmm);
    const half2_t p2 = decode_pair<kHi>(qw[2 * tt + 1], sm.dsc, sm.ndmm), p3 = decode_pair<kHi>(qs8[2 * tt + 1], sm.dsc, sm.ndmm);
    b[tt] = half8_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  }
}

// Wavefronts of a BM x BN tile whose wavefronts each own WM rows x WN columns.
template <int BM, int BN, int WM, int WN>
constexpr int tile_waves() { return (BM / WM) * (BN / WN); }

// One BM x BN tile of C at (m0, n0); columns at and past n_end are not stored.  A wavefront owns
// WM rows x WN columns of it.  Every MFMA takes its activation fragment from LDS (1 KB a
// wavefront, against 128 bytes a clock for the whole CU, which four SIMDs running 32-clock MFMAs
// would need in full); with WN = 64 a fragment read feeds two MFMAs.  The price is that the
// BM / WM wavefronts that share a column range each decode its weights.
template <int BM, int BN, int WM, int WN>
__device__ __forceinline__ void q4k_gemm_tile(
    const _Float16* __restrict__ a16, const float* __restrict__ a_scale, const uint8_t* __restrict__ w,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k, uint32_t m0, uint32_t n0, uint32_t n_end) {
  constexpr int kWaves = tile_waves<BM, BN, WM, WN>();
  constexpr int kWavesN = BN / WN;
  constexpr int kTI = WM / 32, kTJ = WN / 32;      // MFMA tiles per wavefront: rows x columns
  constexpr int kABlk = BM / 16 / kWaves;          // 1 KB activation blocks a wavefront loads per step
  constexpr int kWL = (BN * 9 + 64 * kWaves - 1) / (64 * kWaves);  // 1 KB weight blocks per super-block
  constexpr uint32_t kAStage = BM * 64, kWStage = kWL * kWaves * 1024;
  static_assert(BM % WM == 0 && BN % WN == 0 && WM % 32 == 0 && WN % 32 == 0 && BM % (16 * kWaves) == 0, "tile shape");
  __shared__ __attribute__((aligned(16))) uint8_t lds[4 * kAStage + 2 * kWStage];

  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t wave_m = wave / kWavesN, wave_n = wave % kWavesN;
  const uint32_t l32 = lane & 31u, kg = lane >> 5;
  const uint32_t row_blocks = k / 256;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)lds));
  const uint8_t* a_tile = reinterpret_cast<const uint8_t*>(a16) + static_cast<size_t>(m0) * k * 2;
  const uint8_t* w_tile = w + static_cast<size_t>(n0) * row_blocks * 144;

  // Direct loads.  Activation block L of a step (1 KB, rows 16L..16L+15, four 16-byte chunks
  // a row): lane p fetches row 16L + p/4, chunk (p%4) ^ ((row>>2)&3).  Weight chunk q of a
  // super-block column (q = 9*row + part, 144 bytes a row): the tile's blocks are copied as
  // they lie, 64 chunks a load; chunks past the tile repeat its last chunk into spare LDS.
  // Rows past the matrix edge are clamped to the last row (never stored).
  uint32_t a_src[kABlk], w_src[kWL];
#pragma unroll
  for (int i = 0; i < kABlk; ++i) {
    const uint32_t row = 16u * (wave * kABlk + i) + lane / 4u;
    const uint32_t chunk = (lane % 4u) ^ ((row >> 2) & 3u);
    a_src[i] = (m0 + row < m ? row : m - 1u - m0) * (k * 2u) + chunk * 16u;
  }
#pragma unroll
  for (int i = 0; i < kWL; ++i) {
    uint32_t q = (wave * kWL + i) * 64u + lane;
    q = q < BN * 9u ? q : BN * 9u - 1u;
    const uint32_t row = q / 9u, part = q % 9u;
    w_src[i] = (n0 + row < n ? row : n - 1u - n0) * (row_blocks * 144u) + part * 16u;
  }
  auto issue_a = [&](uint32_t stage, uint32_t slice) {      // slice = 32 K values = 64 bytes a row
    const uint8_t* g = a_tile + slice * 64u;
#pragma unroll
    for (int i = 0; i < kABlk; ++i) direct_load16(g, a_src[i], lds_base + stage * kAStage + (wave * kABlk + i) * 1024u);
  };
  auto issue_w = [&](uint32_t stage, uint32_t block) {
    const uint8_t* g = w_tile + block * 144u;
#pragma unroll
    for (int i = 0; i < kWL; ++i) direct_load16(g, w_src[i], lds_base + 4 * kAStage + stage * kWStage + (wave * kWL + i) * 1024u);
  };

  float16_t acc[kTI][kTJ];
#pragma unroll
  for (int i = 0; i < kTI; ++i)
#pragma unroll
    for (int j = 0; j < kTJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // This lane's first weight row inside a raw stage (column tile j is 32 rows further), and its
  // activation fragment offsets: MFMA step t of a slice takes chunk 2kg + t of the row
  // (k = 16kg + 8t + [0,8), the positions decode_subblock gives the step).
  const uint32_t w_row = (wave_n * WN + l32) * 144u;
  uint32_t a_fr[2];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) a_fr[tt] = (wave_m * WM + l32) * 64u + (((kg * 2u + tt) ^ ((l32 >> 2) & 3u)) * 16u);

  const uint32_t slices = k / 32;

  // Prologue: first super-block and three activation slices in flight, then the first of each
  // is waited for.
  issue_w(0, 0);
  issue_a(0, 0);
  issue_a(1, slices > 1 ? 1 : 0);
  issue_a(2, slices > 2 ? 2 : slices - 1);
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * kABlk) : "memory");

  for (uint32_t blk = 0; blk < row_blocks; ++blk) {
    const uint8_t* raw = lds + 4 * kAStage + (blk & 1u) * kWStage + w_row;
    const bool more = blk + 1 < row_blocks;        // uniform
    BlockHead head[kTJ];
#pragma unroll
    for (int j = 0; j < kTJ; ++j) head[j] = load_block_head(raw + j * 32 * 144);
    uint32_t qw[kTJ][4], qs8[kTJ][4];
    unrolled<8>([&](auto step) {
      constexpr int sb = decltype(step)::value;
      const uint32_t slice = blk * 8u + sb;
      if (sb == 0 && more) issue_w((blk + 1u) & 1u, blk + 1u);
      issue_a((slice + 3u) & 3u, slice + 3u < slices ? slice + 3u : slices - 1u);

      half8_t b[kTJ][2];
#pragma unroll
      for (int j = 0; j < kTJ; ++j) decode_subblock<sb>(raw + j * 32 * 144, kg, head[j], qw[j], qs8[j], b[j]);

      const uint8_t* a_stage = lds + (slice & 3u) * kAStage;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
        for (int i = 0; i < kTI; ++i) {
          const half8_t af = *reinterpret_cast<const half8_t*>(a_stage + a_fr[tt] + i * 32 * 64);
#pragma unroll
          for (int j = 0; j < kTJ; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, b[j][tt], acc[i][j], 0, 0, 0);
        }
      }

      // Publish slice + 1: every direct load older than the two youngest activation slices
      // (and, in the two steps after a weight refill was issued, older than that refill)
      // has landed; this wavefront's LDS reads of the stage about to be refilled are done.
      if (sb <= 1 && more) {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * kABlk + kWL) : "memory");
      } else {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * kABlk) : "memory");
      }
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive the workgroup

  // Epilogue: lane holds column l32 and rows (e/4)*8 + kg*4 + e%4 of each 32 x 32 tile; the
  // four row scales of each e/4 group are one 16-byte load (the scale array is padded, so rows
  // past m read something harmless).
#pragma unroll
  for (int i = 0; i < kTI; ++i) {
    const uint32_t row0 = m0 + wave_m * WM + i * 32u + kg * 4u;
    float4 sc[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) sc[q] = *reinterpret_cast<const float4*>(a_scale + row0 + q * 8u);
#pragma unroll
    for (int j = 0; j < kTJ; ++j) {
      const uint32_t col = n0 + wave_n * WN + j * 32u + l32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = row0 + (e >> 2) * 8u + (e & 3u);
        const float4 s4 = sc[e >> 2];
        const float rs = (e & 3) == 0 ? s4.x : (e & 3) == 1 ? s4.y : (e & 3) == 2 ? s4.z : s4.w;
        if (row < m && col < n_end) c[static_cast<size_t>(row) * n + col] = acc[i][j][e] * rs;
      }
    }
  }
}

}  // namespace
}  // namespace qmm
