// Q4_K prefill GEMM on MFMA: C (m x n fp32) = A (m x k) . deq(W)^T, W = n rows of k/256
// Q4_K super-blocks (src/core/numerics/quant.hpp:11-15; reference kernel
// src/backends/rocm/rocm_kernels_wmma.cpp:30-80,334-431, which stages A and the decoded
// weights in LDS as fp16 and accumulates in fp32).
//
// Two launches.  (1) The activations are converted once to fp16 in a workspace, each row divided
// by a power-of-two scale that the epilogue multiplies back, so the fp16 range is no limit (the
// reference converts them again in every workgroup; done once, the GEMM reads 2 bytes per
// activation instead of 4 and the conversion costs one pass over A).  (2) The GEMM proper:
// v_mfma_f32_32x32x16_f16, fp32 accumulate.
//
// Weights never exist dequantized in memory: the raw 144-byte super-blocks travel
// HBM -> LDS by direct loads, and each wavefront decodes the eight weights a lane owes the
// B operand of one MFMA straight from those bytes into registers.  The decode is the reference's:
// the fp32 value fma(q, d*sc, -(dmin*mn)) -- d*sc, dmin*mn and q*(d*sc) are exact in fp32, so this
// is DequantizeQ4K's value bit for bit -- rounded ONCE to fp16 (round to nearest even), which is
// what the reference's tensor-core tile stages (rocm_kernels_wmma.cpp:73-77).  A masked nibble
// pair masked in place is a pair of fp16 subnormals (q * 2^-24) that the mixed-precision
// multiply-add consumes directly, so two weights cost one mask and two multiply-adds that also
// round to fp16.  The nibble pairs come out of a dword in the order
// (k0,k2),(k1,k3); instead of un-shuffling them, the fp16 copy of A is written with the same
// order inside every group of 8, which a dot product cannot see.
//
// A wavefront owns WM rows x WN columns of the workgroup's tile.  Small tiles (a short stack of
// rows) use WN = 32 and all rows, so no two wavefronts decode the same weight; the 256 x 256
// prefill tile uses 128 x 64, where each activation fragment read from LDS feeds two MFMAs.
//
// K advances one 32-wide sub-block per step: activation slices (BM x 64 bytes) run through
// a four-stage XOR-swizzled LDS ring, raw weight super-blocks through a two-stage ring that
// is refilled once per eight steps; waits are counted by hand as in gemm_mxfp4.hip.

#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

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

// One workgroup per destination row: fp32 row -> fp16 (round to nearest even) divided by the
// row's power-of-two scale, which goes to scale[row] and is multiplied back in the GEMM's
// epilogue.  With `pos` the rows are gathered: destination row pos[p] takes source row p / top_k.
__global__ __launch_bounds__(256) void rows_to_f16_kernel(const float* __restrict__ src, _Float16* __restrict__ dst,
                                                          float* __restrict__ scale, uint32_t cols,
                                                          const uint32_t* __restrict__ pos, uint32_t top_k) {
  __shared__ float red[4];
  const uint32_t p = blockIdx.x;
  const uint32_t drow = pos != nullptr ? pos[p] : p, srow = pos != nullptr ? p / top_k : p;
  const float4* in = reinterpret_cast<const float4*>(src + static_cast<size_t>(srow) * cols);
  float amax = 0.0f;
  for (uint32_t g = threadIdx.x; g < cols / 4u; g += 256u) {
    const float4 v = in[g];
    amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fmaxf(fabsf(v.z), fabsf(v.w)), amax));
  }
  const float s = row_scale_for(block_amax(amax, red)), inv = 1.0f / s;
  half8_t* out = reinterpret_cast<half8_t*>(dst + static_cast<size_t>(drow) * cols);
  for (uint32_t g = threadIdx.x; g < cols / 8u; g += 256u) out[g] = to_f16_group(in[2 * g], in[2 * g + 1], inv);
  if (threadIdx.x == 0) scale[drow] = s;
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
  // activation fragment offsets: MFMA step t of a slice takes chunk 2t + kg of the row
  // (k = 16t + 8kg + [0,8)).
  const uint32_t w_row = (wave_n * WN + l32) * 144u;
  uint32_t a_fr[2];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) a_fr[tt] = (wave_m * WM + l32) * 64u + (((tt * 2u + kg) ^ ((l32 >> 2) & 3u)) * 16u);

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
    float hd[kTJ], hndmin[kTJ];                    // block header: d and -dmin
    ScaleBytes sbytes[kTJ];
#pragma unroll
    for (int j = 0; j < kTJ; ++j) {
      const uint4 head = *reinterpret_cast<const uint4*>(raw + j * 32 * 144);
      hd[j] = half_bits_to_float(head.x & 0xFFFFu);
      hndmin[j] = -half_bits_to_float(head.x >> 16);
      sbytes[j] = unpack_scales(head.y, head.z, head.w);
    }
    uint32_t qw[kTJ][4], qs8[kTJ][4];
    unrolled<8>([&](auto step) {
      constexpr int sb = decltype(step)::value;
      constexpr int kHi = sb & 1;
      const uint32_t slice = blk * 8u + sb;
      if (sb == 0 && more) issue_w((blk + 1u) & 1u, blk + 1u);
      issue_a((slice + 3u) & 3u, slice + 3u < slices ? slice + 3u : slices - 1u);

      // Quant bytes of this lane's 16 weights a column: sub-block sb lives in the low (even sb)
      // or high nibbles of bytes (sb/2)*32 + [0,32) (src/core/numerics/quant.cpp:656-675).  An
      // odd step decodes the same bytes as the even step before it: the words shifted down by
      // one byte (for bytes 1 and 3) are kept from there.
      half8_t b[kTJ][2];
#pragma unroll
      for (int j = 0; j < kTJ; ++j) {
        const ScaleMin sm = scale_min_f32<sb>(sbytes[j], hd[j], hndmin[j]);
        if (kHi == 0) {
          const uint8_t* qp = raw + j * 32 * 144 + 16 + (sb >> 1) * 32 + kg * 8u;
          const uint2 q0 = *reinterpret_cast<const uint2*>(qp);
          const uint2 q1 = *reinterpret_cast<const uint2*>(qp + 16);
          qw[j][0] = q0.x, qw[j][1] = q0.y, qw[j][2] = q1.x, qw[j][3] = q1.y;
#pragma unroll
          for (int x = 0; x < 4; ++x) qs8[j][x] = qw[j][x] >> 8;
        }
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          const half2_t p0 = decode_pair<kHi>(qw[j][2 * tt], sm.dsc, sm.ndmm), p1 = decode_pair<kHi>(qs8[j][2 * tt], sm.dsc, sm.ndmm);
          const half2_t p2 = decode_pair<kHi>(qw[j][2 * tt + 1], sm.dsc, sm.ndmm), p3 = decode_pair<kHi>(qs8[j][2 * tt + 1], sm.dsc, sm.ndmm);
          b[j][tt] = half8_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
        }
      }

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

template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void q4k_gemm_kernel(
    const _Float16* __restrict__ a16, const float* __restrict__ a_scale, const uint8_t* __restrict__ w,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k, uint32_t n_begin, uint32_t n_end) {
  const uint32_t tiles_n = (n_end - n_begin + BN - 1) / BN;
  q4k_gemm_tile<BM, BN, WM, WN>(a16, a_scale, w, c, m, n, k, (blockIdx.x / tiles_n) * BM, n_begin + (blockIdx.x % tiles_n) * BN,
                        n_end);
}

// Grouped form for routed experts: segment e multiplies rows seg[e]..seg[e+1] of a16
// by expert e's weights (w + e * w_stride) into the same rows of c.  Segment bounds live in
// device memory (the routing is computed on the device); an empty segment leaves at once.
template <int BM, int BN>
__global__ __launch_bounds__(BN * 2) void q4k_gemm_grouped_kernel(
    const _Float16* __restrict__ a16, const float* __restrict__ a_scale, const uint8_t* __restrict__ w,
    float* __restrict__ c, const uint32_t* __restrict__ seg, uint64_t w_stride, uint32_t n, uint32_t k,
    uint32_t experts, uint32_t tensors, const uint8_t* __restrict__ w2, float* __restrict__ c2, uint64_t w2_stride) {
  // One-dimensional grid, decoded so that an expert's activation rows are fetched from HBM once:
  // workgroups are dealt to the eight XCDs (one L2 each) by linear index, so the expert's low three
  // bits are the index's low three bits (all its tiles on one XCD), and its column tiles of both
  // tensors follow each other in dispatch order (its rows are still in that L2 when the next tile
  // asks for them).  `tensors` = 2 runs a second expert tensor of the same shape against the same
  // rows (gate and up in one launch).
  const uint32_t tiles = (n + BN - 1) / BN;
  const uint32_t slot = blockIdx.x / 8u, per_expert = tiles * tensors;
  const uint32_t e = (slot / per_expert) * 8u + blockIdx.x % 8u;
  const uint32_t tz = slot % per_expert, tile = tz % tiles;
  if (e >= experts) return;
  if (tz >= tiles) w = w2, c = c2, w_stride = w2_stride;
  const uint32_t r0 = seg[e], r1 = seg[e + 1];
  if (r1 <= r0) return;
  const _Float16* a_e = a16 + static_cast<size_t>(r0) * k;
  const uint8_t* w_e = w + e * w_stride;
  float* c_e = c + static_cast<size_t>(r0) * n;
  for (uint32_t m0 = 0; m0 < r1 - r0; m0 += BM) {
    q4k_gemm_tile<BM, BN, BM, 32>(a_e, a_scale + r0, w_e, c_e, r1 - r0, n, k, m0, tile * BN, n);
  }
}

template <int BM, int BN, int WM = BM, int WN = 32>
void launch_range(const _Float16* a16, const float* a_scale, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                  uint32_t k, uint32_t n_begin, uint32_t n_end, hipStream_t stream) {
  const uint32_t tiles = ((m + BM - 1) / BM) * ((n_end - n_begin + BN - 1) / BN);
  hipLaunchKernelGGL((q4k_gemm_kernel<BM, BN, WM, WN>), dim3(tiles), dim3(tile_waves<BM, BN, WM, WN>() * 64), 0, stream,
                     a16, a_scale, w, c, m, n, k, n_begin, n_end);
}

}  // namespace

bool gemm_q4k_supported(uint64_t m, uint64_t k) { return k % 256 == 0 && k <= (1u << 20) && m * k < (1ull << 31); }

// fp16 copy of A, then one scale per row padded by a tile of rows (the epilogue reads scales in fours).
size_t gemm_q4k_workspace_bytes(uint64_t m, uint64_t k) { return static_cast<size_t>(m) * k * 2 + (static_cast<size_t>(m) + 256) * 4; }

// The bulk of C goes to 256 x 256 tiles, whole rounds of one tile per CU; columns left over
// when the tile count is not a multiple of the CU count are cut into 128 x 64 tiles that
// spread over every CU instead of keeping a few CUs busy for a whole extra round.
hipError_t launch_q4k_gemm(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m,
                           uint32_t n, uint32_t k, hipStream_t stream) {
  _Float16* a16 = static_cast<_Float16*>(workspace);
  float* a_scale = reinterpret_cast<float*>(a16 + static_cast<size_t>(m) * k);
  hipLaunchKernelGGL(rows_to_f16_kernel, dim3(m), dim3(256), 0, stream, a, a16, a_scale, k, nullptr, 1u);
  const uint32_t cus = static_cast<uint32_t>(num_cus());
  const uint32_t tiles_m = (m + 255u) / 256u, tiles_n = (n + 255u) / 256u;
  const uint32_t tiles = tiles_m * tiles_n;
  uint32_t main_tn = tiles_n;
  if (tiles > cus && tiles % cus != 0 && tiles % cus <= cus / 2) {
    main_tn = (tiles / cus) * cus / tiles_m;
  } else if (tiles < cus / 2) {
    main_tn = 0;
  }
  if (m <= 64) {
    // A short stack of rows is bound by the weight stream: narrow tiles (one wavefront, 32
    // columns) give every CU several workgroups' worth of super-blocks in flight.
    if (m <= 32) {
      launch_range<32, 32>(a16, a_scale, w, c, m, n, k, 0u, n, stream);
    } else {
      launch_range<64, 32>(a16, a_scale, w, c, m, n, k, 0u, n, stream);
    }
    return hipGetLastError();
  }
  const uint32_t n_split = main_tn * 256u < n ? main_tn * 256u : n;
  if (n_split > 0) launch_range<256, 256, 128, 64>(a16, a_scale, w, c, m, n, k, 0u, n_split, stream);
  if (n_split < n) launch_range<128, 64, 64, 32>(a16, a_scale, w, c, m, n, k, n_split, n, stream);
  return hipGetLastError();
}

// ---- Q5_K / Q6_K prefill: weights decoded once to fp16, then a dense fp16 MFMA GEMM ----------
// Their blocks (176 and 210 bytes, the latter only 2-byte aligned) do not suit the in-register
// decode above, and they are the minority of a K-quant file's tensors, so the weights take a
// pre-pass: every value is formed exactly in fp32 as the reference decodes it and rounded once
// to fp16 (the same operand precision as the Q4_K path), in the 0,2,1,3,4,6,5,7 order that the
// activation copy uses.  The GEMM then streams both operands as 32-K slices through four-stage
// swizzled LDS rings.
namespace {

// Eight consecutive values of a group in the stored order 0,2,1,3,4,6,5,7.
__device__ __forceinline__ void store_perm8(_Float16* dst, const float (&v)[8]) {
  half8_t h;
  h[0] = static_cast<_Float16>(v[0]), h[1] = static_cast<_Float16>(v[2]);
  h[2] = static_cast<_Float16>(v[1]), h[3] = static_cast<_Float16>(v[3]);
  h[4] = static_cast<_Float16>(v[4]), h[5] = static_cast<_Float16>(v[6]);
  h[6] = static_cast<_Float16>(v[5]), h[7] = static_cast<_Float16>(v[7]);
  *reinterpret_cast<half8_t*>(dst) = h;
}

__device__ __forceinline__ uint64_t load8_a2(const uint8_t* p) {   // eight bytes from a 2-byte aligned address
  const uint16_t* q = reinterpret_cast<const uint16_t*>(p);
  return static_cast<uint64_t>(q[0]) | (static_cast<uint64_t>(q[1]) << 16) | (static_cast<uint64_t>(q[2]) << 32) |
         (static_cast<uint64_t>(q[3]) << 48);
}

// One thread per (block, half n, eight lanes l = 8o..8o+7): 32 values, four 16-byte stores
// (src/core/numerics/quant.cpp:421-450).
__global__ __launch_bounds__(256) void q6k_to_f16_kernel(const uint8_t* __restrict__ w, _Float16* __restrict__ out,
                                                         uint64_t nitems) {
  const uint64_t t = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= nitems) return;
  const uint64_t blk = t >> 3;
  const uint32_t n = static_cast<uint32_t>(t >> 2) & 1u, o = static_cast<uint32_t>(t) & 3u, is = o >> 1;
  const uint8_t* base = w + blk * 210u;
  const uint64_t a = load8_a2(base + n * 64 + o * 8), b = load8_a2(base + n * 64 + 32 + o * 8);
  const uint64_t h = load8_a2(base + 128 + n * 32 + o * 8);
  const float d = half_bits_to_float(*reinterpret_cast<const uint16_t*>(base + 208));
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float ds = d * static_cast<float>(static_cast<int8_t>(base[192 + n * 8 + is + 2 * j]));
    const uint64_t lo = (j & 1) ? b : a;
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t nib = static_cast<uint32_t>(lo >> (8 * i + 4 * (j >> 1))) & 15u;
      const uint32_t top = static_cast<uint32_t>(h >> (8 * i + 2 * j)) & 3u;
      v[i] = ds * static_cast<float>(static_cast<int>(nib | (top << 4)) - 32);
    }
    store_perm8(out + blk * 256 + n * 128 + 32 * j + o * 8, v);
  }
}

// One thread per (block, group g, eight lanes): 16 values, two 16-byte stores
// (src/core/numerics/quant.cpp:388-419).
__global__ __launch_bounds__(256) void q5k_to_f16_kernel(const uint8_t* __restrict__ w, _Float16* __restrict__ out,
                                                         uint64_t nitems) {
  const uint64_t t = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= nitems) return;
  const uint64_t blk = t >> 4;
  const uint32_t g = static_cast<uint32_t>(t >> 2) & 3u, o = static_cast<uint32_t>(t) & 3u;
  const uint8_t* base = w + blk * 176u;
  const uint8_t* p = base + 4;
  auto scale_min = [&](uint32_t sb, uint32_t& sc, uint32_t& mn) {
    if (sb < 4) {
      sc = p[sb] & 63u;
      mn = p[sb + 4] & 63u;
    } else {
      sc = (p[sb + 4] & 15u) | ((p[sb - 4] >> 6) << 4);
      mn = (p[sb + 4] >> 4) | ((p[sb] >> 6) << 4);
    }
  };
  uint32_t sca, mna, scb, mnb;
  scale_min(2 * g, sca, mna);
  scale_min(2 * g + 1, scb, mnb);
  const uint32_t dd = *reinterpret_cast<const uint32_t*>(base);
  const float d = half_bits_to_float(dd & 0xFFFFu), dmin = half_bits_to_float(dd >> 16);
  const float d1 = d * static_cast<float>(sca), m1 = dmin * static_cast<float>(mna);
  const float d2 = d * static_cast<float>(scb), m2 = dmin * static_cast<float>(mnb);
  const uint64_t low = *reinterpret_cast<const uint64_t*>(base + 48 + g * 32 + o * 8);
  const uint64_t high = *reinterpret_cast<const uint64_t*>(base + 16 + o * 8);
  float v0[8], v1[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t lb = static_cast<uint32_t>(low >> (8 * i)) & 0xFFu, hb = static_cast<uint32_t>(high >> (8 * i)) & 0xFFu;
    v0[i] = d1 * static_cast<float>((lb & 15u) + (((hb >> (2 * g)) & 1u) << 4)) - m1;
    v1[i] = d2 * static_cast<float>((lb >> 4) + (((hb >> (2 * g + 1)) & 1u) << 4)) - m2;
  }
  store_perm8(out + blk * 256 + g * 64 + o * 8, v0);
  store_perm8(out + blk * 256 + g * 64 + 32 + o * 8, v1);
}

// C tile = A16 (rows scaled by a_scale) . W16^T, both operands fp16 row-major with row length k.
template <int BM, int BN>
__global__ __launch_bounds__(BN * 2) void f16w_gemm_kernel(
    const _Float16* __restrict__ a16, const float* __restrict__ a_scale, const _Float16* __restrict__ w16,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k, uint32_t n_begin, uint32_t n_end) {
  constexpr int kWaves = BN / 32, kTI = BM / 32;
  constexpr int kABlk = BM / 16 / kWaves, kWBlk = BN / 16 / kWaves;   // 1 KB blocks per wavefront and slice
  constexpr int kDma = kABlk + kWBlk;
  constexpr uint32_t kAStage = BM * 64, kWStage = BN * 64, kStage = kAStage + kWStage;
  static_assert(BM % (16 * kWaves) == 0 && BN % (16 * kWaves) == 0, "tile shape");
  __shared__ __attribute__((aligned(16))) uint8_t lds[4 * kStage];

  const uint32_t tiles_n = (n_end - n_begin + BN - 1) / BN;
  const uint32_t m0 = (blockIdx.x / tiles_n) * BM, n0 = n_begin + (blockIdx.x % tiles_n) * BN;
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t l32 = lane & 31u, kg = lane >> 5;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)lds));
  const uint8_t* a_tile = reinterpret_cast<const uint8_t*>(a16) + static_cast<size_t>(m0) * k * 2;
  const uint8_t* w_tile = reinterpret_cast<const uint8_t*>(w16) + static_cast<size_t>(n0) * k * 2;

  // Block L of a slice = rows 16L..16L+15, four 16-byte chunks a row: lane p fetches row
  // 16L + p/4, chunk (p%4) ^ ((row>>2)&3).  Rows past the matrix edge are clamped (never stored).
  uint32_t a_src[kABlk], w_src[kWBlk];
#pragma unroll
  for (int i = 0; i < kABlk; ++i) {
    const uint32_t row = 16u * (wave * kABlk + i) + lane / 4u;
    a_src[i] = (m0 + row < m ? row : m - 1u - m0) * (k * 2u) + (((lane % 4u) ^ ((row >> 2) & 3u)) * 16u);
  }
#pragma unroll
  for (int i = 0; i < kWBlk; ++i) {
    const uint32_t row = 16u * (wave * kWBlk + i) + lane / 4u;
    w_src[i] = (n0 + row < n ? row : n - 1u - n0) * (k * 2u) + (((lane % 4u) ^ ((row >> 2) & 3u)) * 16u);
  }
  auto issue = [&](uint32_t stage, uint32_t slice_any) {
    const uint32_t slice = __builtin_amdgcn_readfirstlane(slice_any);
#pragma unroll
    for (int i = 0; i < kABlk; ++i)
      direct_load16(a_tile + slice * 64u, a_src[i], lds_base + stage * kStage + (wave * kABlk + i) * 1024u);
#pragma unroll
    for (int i = 0; i < kWBlk; ++i)
      direct_load16(w_tile + slice * 64u, w_src[i], lds_base + stage * kStage + kAStage + (wave * kWBlk + i) * 1024u);
  };

  float16_t acc[kTI];
#pragma unroll
  for (int i = 0; i < kTI; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;
  uint32_t fr[2];   // fragment offset inside a 32-row group: MFMA step tt takes chunk 2tt + kg
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) fr[tt] = l32 * 64u + (((tt * 2u + kg) ^ ((l32 >> 2) & 3u)) * 16u);

  const uint32_t slices = k / 32;
  issue(0, 0);
  issue(1, slices > 1 ? 1 : 0);
  issue(2, slices > 2 ? 2 : slices - 1);
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * kDma) : "memory");
  for (uint32_t slice = 0; slice < slices; ++slice) {
    issue((slice + 3u) & 3u, slice + 3u < slices ? slice + 3u : slices - 1u);
    const uint8_t* stage = lds + (slice & 3u) * kStage;
    half8_t b[2];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) b[tt] = *reinterpret_cast<const half8_t*>(stage + kAStage + wave * 32 * 64 + fr[tt]);
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
      for (int i = 0; i < kTI; ++i) {
        const half8_t af = *reinterpret_cast<const half8_t*>(stage + fr[tt] + i * 32 * 64);
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, b[tt], acc[i], 0, 0, 0);
      }
    }
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(2 * kDma) : "memory");
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive the workgroup

  const uint32_t col = n0 + wave * 32u + l32;
#pragma unroll
  for (int i = 0; i < kTI; ++i) {
    float4 sc[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) sc[q] = *reinterpret_cast<const float4*>(a_scale + m0 + i * 32u + q * 8u + kg * 4u);
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const uint32_t row = m0 + i * 32u + (e >> 2) * 8u + kg * 4u + (e & 3u);
      const float4 s4 = sc[e >> 2];
      const float rs = (e & 3) == 0 ? s4.x : (e & 3) == 1 ? s4.y : (e & 3) == 2 ? s4.z : s4.w;
      if (row < m && col < n_end) c[static_cast<size_t>(row) * n + col] = acc[i][e] * rs;
    }
  }
}

}  // namespace

bool gemm_kquant_f16_supported(uint64_t m, uint64_t n, uint64_t k) {
  return k % 256 == 0 && k <= (1u << 20) && m * k < (1ull << 31) && n * k < (1ull << 31);
}

// fp16 copy of A, its row scales (padded by a tile of rows), then the fp16 copy of W.
size_t gemm_kquant_f16_workspace_bytes(uint64_t m, uint64_t n, uint64_t k) {
  return static_cast<size_t>(m) * k * 2 + (static_cast<size_t>(m) + 256) * 4 + static_cast<size_t>(n) * k * 2;
}

// block_bytes selects the format: 176 = Q5_K, 210 = Q6_K.
hipError_t launch_kquant_f16_gemm(const float* a, const uint8_t* w, uint32_t block_bytes, float* c, void* workspace,
                                  uint32_t m, uint32_t n, uint32_t k, hipStream_t stream) {
  _Float16* a16 = static_cast<_Float16*>(workspace);
  float* a_scale = reinterpret_cast<float*>(a16 + static_cast<size_t>(m) * k);
  _Float16* w16 = reinterpret_cast<_Float16*>(a_scale + m + 256);
  const uint64_t blocks = static_cast<uint64_t>(n) * (k / 256);
  if (block_bytes == 210) {
    hipLaunchKernelGGL(q6k_to_f16_kernel, dim3(static_cast<uint32_t>((blocks * 8 + 255) / 256)), dim3(256), 0, stream,
                       w, w16, blocks * 8);
  } else if (block_bytes == 176) {
    hipLaunchKernelGGL(q5k_to_f16_kernel, dim3(static_cast<uint32_t>((blocks * 16 + 255) / 256)), dim3(256), 0, stream,
                       w, w16, blocks * 16);
  } else {
    return hipErrorInvalidValue;
  }
  hipLaunchKernelGGL(rows_to_f16_kernel, dim3(m), dim3(256), 0, stream, a, a16, a_scale, k, nullptr, 1u);
  // whole rounds of 256 x 256 tiles, leftover columns as 128 x 64 tiles (as launch_q4k_gemm)
  const uint32_t cus = static_cast<uint32_t>(num_cus());
  const uint32_t tiles_m = (m + 255u) / 256u, tiles_n = (n + 255u) / 256u, tiles = tiles_m * tiles_n;
  uint32_t main_tn = tiles_n;
  if (tiles > cus && tiles % cus != 0 && tiles % cus <= cus / 2) {
    main_tn = (tiles / cus) * cus / tiles_m;
  } else if (tiles < cus / 2) {
    main_tn = 0;
  }
  const uint32_t n_split = main_tn * 256u < n ? main_tn * 256u : n;
  if (n_split > 0) {
    hipLaunchKernelGGL((f16w_gemm_kernel<256, 256>), dim3(tiles_m * main_tn), dim3(512), 0, stream, a16, a_scale, w16,
                       c, m, n, k, 0u, n_split);
  }
  if (n_split < n) {
    const uint32_t t2 = ((m + 127u) / 128u) * ((n - n_split + 63u) / 64u);
    hipLaunchKernelGGL((f16w_gemm_kernel<128, 64>), dim3(t2), dim3(128), 0, stream, a16, a_scale, w16, c, m, n, k,
                       n_split, n);
  }
  return hipGetLastError();
}

// ---- routed experts, a whole chunk of tokens grouped by expert -----------------------------
// (token, slot) pairs are sorted by expert so that each expert's weights are streamed once for
// all the tokens routed to it, and the three projections run as grouped MFMA GEMMs.
namespace {

// seg[e] = first sorted position of expert e (seg[experts] = pairs); pos[p] = sorted position
// of pair p.  Counting sort with LDS atomics: which position inside its expert's segment a pair
// gets depends on the order the atomics land in, but a row's result does not depend on where the
// row sits, so the outputs are the same on every run.
__global__ __launch_bounds__(1024) void moe_sort_kernel(const uint32_t* __restrict__ ids, uint32_t pairs,
                                                        uint32_t experts, uint32_t* __restrict__ seg,
                                                        uint32_t* __restrict__ pos) {
  __shared__ uint32_t cursor[1024];
  const uint32_t t = threadIdx.x;
  cursor[t] = 0;
  __syncthreads();
  for (uint32_t p = t; p < pairs; p += 1024u) {
    const uint32_t id = ids[p] < experts ? ids[p] : experts - 1u;   // a bad id cannot leave the tensor
    atomicAdd(&cursor[id], 1u);
  }
  __syncthreads();
  if (t == 0) {
    uint32_t run = 0;
    for (uint32_t i = 0; i < experts; ++i) {
      const uint32_t c = cursor[i];
      cursor[i] = run;
      seg[i] = run;
      run += c;
    }
    seg[experts] = run;
  }
  __syncthreads();
  for (uint32_t p = t; p < pairs; p += 1024u) {
    const uint32_t id = ids[p] < experts ? ids[p] : experts - 1u;
    pos[p] = atomicAdd(&cursor[id], 1u);
  }
}

// phi = silu(g) * u for one sorted row, written as the fp16 operand of the down GEMM with its
// own power-of-two row scale (phi can exceed the fp16 range).
__global__ __launch_bounds__(256) void moe_silu_mul_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                           _Float16* __restrict__ phi16, float* __restrict__ scale,
                                                           uint32_t inter) {
  __shared__ float red[4];
  const size_t base = static_cast<size_t>(blockIdx.x) * inter;
  const float4* gp = reinterpret_cast<const float4*>(g + base);
  const float4* up = reinterpret_cast<const float4*>(u + base);
  auto f = [](float gv, float uv) { return (gv / (1.0f + expf(-gv))) * uv; };
  auto phi4 = [&](uint32_t q) {
    const float4 a = gp[q], b = up[q];
    return make_float4(f(a.x, b.x), f(a.y, b.y), f(a.z, b.z), f(a.w, b.w));
  };
  float amax = 0.0f;
  for (uint32_t q = threadIdx.x; q < inter / 4u; q += 256u) {
    const float4 v = phi4(q);
    amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fmaxf(fabsf(v.z), fabsf(v.w)), amax));
  }
  const float s = row_scale_for(block_amax(amax, red)), inv = 1.0f / s;
  half8_t* out = reinterpret_cast<half8_t*>(phi16 + base);
  for (uint32_t q = threadIdx.x; q < inter / 8u; q += 256u) out[q] = to_f16_group(phi4(2 * q), phi4(2 * q + 1), inv);
  if (threadIdx.x == 0) scale[blockIdx.x] = s;
}

// phi[p][j] = silu(g[pos[p]][j]) * u[pos[p]][j]: the grouped gate and up products of (token,
// slot) pair p, which sit at sorted row pos[p], back in the caller's pair order as fp32.
__global__ __launch_bounds__(256) void moe_silu_scatter_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                               const uint32_t* __restrict__ pos,
                                                               float* __restrict__ phi, uint32_t inter) {
  const size_t src = static_cast<size_t>(pos[blockIdx.x]) * inter, dst = static_cast<size_t>(blockIdx.x) * inter;
  const float4* gp = reinterpret_cast<const float4*>(g + src);
  const float4* up = reinterpret_cast<const float4*>(u + src);
  float4* out = reinterpret_cast<float4*>(phi + dst);
  auto f = [](float gv, float uv) { return (gv / (1.0f + expf(-gv))) * uv; };
  for (uint32_t q = threadIdx.x; q < inter / 4u; q += 256u) {
    const float4 a = gp[q], b = up[q];
    out[q] = make_float4(f(a.x, b.x), f(a.y, b.y), f(a.z, b.z), f(a.w, b.w));
  }
}

// out[t][j] (+)= sum_slot wts[t][slot] * rows[pos[t*top_k + slot]][j], slots in order.
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ rows, const uint32_t* __restrict__ pos,
                                                          const float* __restrict__ wts, float* __restrict__ out,
                                                          uint32_t tokens, uint32_t top_k, uint32_t hidden,
                                                          bool accumulate) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (i >= static_cast<uint64_t>(tokens) * hidden) return;
  const uint32_t t = static_cast<uint32_t>(i / hidden), j = static_cast<uint32_t>(i % hidden);
  float acc = 0.0f;
  for (uint32_t s = 0; s < top_k; ++s) {
    acc += wts[t * top_k + s] * rows[static_cast<size_t>(pos[t * top_k + s]) * hidden + j];
  }
  out[i] = accumulate ? out[i] + acc : acc;
}

size_t align256(size_t v) { return (v + 255) & ~size_t{255}; }

}  // namespace

bool moe_ffn_q4k_supported(uint64_t hidden, uint64_t inter, uint64_t experts) {
  return hidden % 256 == 0 && inter % 256 == 0 && hidden <= (1u << 16) && inter <= (1u << 16) && experts >= 1 &&
         experts <= 1024;
}

size_t moe_ffn_q4k_workspace_bytes(uint64_t pairs, uint64_t hidden, uint64_t inter, uint64_t experts) {
  return align256((experts + 1) * 4) + align256(pairs * 4) + 2 * align256((pairs + 256) * 4) + align256(pairs * hidden * 2) +
         2 * align256(pairs * inter * 4) + align256(pairs * inter * 2) + align256(pairs * hidden * 4);
}

hipError_t launch_moe_ffn_q4k(const float* x, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                              const uint32_t* ids, const float* wts, float* out, void* workspace,
                              uint32_t hidden, uint32_t inter, uint32_t top_k, uint64_t gate_stride,
                              uint64_t up_stride, uint64_t down_stride, uint32_t experts, uint32_t tokens,
                              bool accumulate, hipStream_t stream) {
  const uint32_t pairs = tokens * top_k;
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  uint32_t* seg = reinterpret_cast<uint32_t*>(ws);
  ws += align256((static_cast<size_t>(experts) + 1) * 4);
  uint32_t* pos = reinterpret_cast<uint32_t*>(ws);
  ws += align256(static_cast<size_t>(pairs) * 4);
  float* x_scale = reinterpret_cast<float*>(ws);
  ws += align256((static_cast<size_t>(pairs) + 256) * 4);
  float* phi_scale = reinterpret_cast<float*>(ws);
  ws += align256((static_cast<size_t>(pairs) + 256) * 4);
  _Float16* a16 = reinterpret_cast<_Float16*>(ws);
  ws += align256(static_cast<size_t>(pairs) * hidden * 2);
  float* g = reinterpret_cast<float*>(ws);
  ws += align256(static_cast<size_t>(pairs) * inter * 4);
  float* u = reinterpret_cast<float*>(ws);
  ws += align256(static_cast<size_t>(pairs) * inter * 4);
  _Float16* phi16 = reinterpret_cast<_Float16*>(ws);
  ws += align256(static_cast<size_t>(pairs) * inter * 2);
  float* rows = reinterpret_cast<float*>(ws);

  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, seg, pos);
  hipLaunchKernelGGL(rows_to_f16_kernel, dim3(pairs), dim3(256), 0, stream, x, a16, x_scale, hidden, pos, top_k);
  constexpr int BM = 32, BN = 64;
  const uint32_t expert_groups = (experts + 7u) / 8u * 8u;
  hipLaunchKernelGGL((q4k_gemm_grouped_kernel<BM, BN>), dim3(expert_groups * ((inter + BN - 1) / BN) * 2u), dim3(BN * 2), 0,
                     stream, a16, x_scale, gate, g, seg, gate_stride, inter, hidden, experts, 2u, up, u, up_stride);
  hipLaunchKernelGGL(moe_silu_mul_kernel, dim3(pairs), dim3(256), 0, stream, g, u, phi16, phi_scale, inter);
  hipLaunchKernelGGL((q4k_gemm_grouped_kernel<BM, BN>), dim3(expert_groups * ((hidden + BN - 1) / BN)), dim3(BN * 2), 0,
                     stream, phi16, phi_scale, down, rows, seg, down_stride, hidden, inter, experts, 1u, nullptr, nullptr,
                     uint64_t{0});
  const uint64_t outs = static_cast<uint64_t>(tokens) * hidden;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(static_cast<uint32_t>((outs + 255) / 256)), dim3(256), 0, stream, rows, pos,
                     wts, out, tokens, top_k, hidden, accumulate);
  return hipGetLastError();
}

// The two halves of launch_moe_ffn_q4k behind the reference's own pair of ids
// ("moe_experts_gate_up_q4k_rows" then "moe_experts_down_q4k_rows",
// src/backends/rocm/rocm_kernels_moe.cpp:15-79) for a chunk of tokens: each sorts the pairs by
// expert, gathers its operand as fp16 rows and runs the grouped GEMM, so an expert's weights are
// read once per launch instead of once per token that chose it.  phi keeps the caller's layout
// (tokens x top_k x inter, fp32) between the two.  Workspace as for launch_moe_ffn_q4k.
hipError_t launch_moe_gate_up_q4k_grouped(const float* x, const uint8_t* gate, const uint8_t* up, const uint32_t* ids,
                                          float* phi, void* workspace, uint32_t hidden, uint32_t inter, uint32_t top_k,
                                          uint64_t gate_stride, uint64_t up_stride, uint32_t experts, uint32_t tokens,
                                          hipStream_t stream) {
  const uint32_t pairs = tokens * top_k;
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  uint32_t* seg = reinterpret_cast<uint32_t*>(ws);
  ws += align256((static_cast<size_t>(experts) + 1) * 4);
  uint32_t* pos = reinterpret_cast<uint32_t*>(ws);
  ws += align256(static_cast<size_t>(pairs) * 4);
  float* x_scale = reinterpret_cast<float*>(ws);
  ws += align256((static_cast<size_t>(pairs) + 256) * 4);
  _Float16* a16 = reinterpret_cast<_Float16*>(ws);
  ws += align256(static_cast<size_t>(pairs) * hidden * 2);
  float* g = reinterpret_cast<float*>(ws);
  ws += align256(static_cast<size_t>(pairs) * inter * 4);
  float* u = reinterpret_cast<float*>(ws);

  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, seg, pos);
  hipLaunchKernelGGL(rows_to_f16_kernel, dim3(pairs), dim3(256), 0, stream, x, a16, x_scale, hidden, pos, top_k);
  constexpr int BM = 32, BN = 64;
  const uint32_t expert_groups = (experts + 7u) / 8u * 8u;
  hipLaunchKernelGGL((q4k_gemm_grouped_kernel<BM, BN>), dim3(expert_groups * ((inter + BN - 1) / BN) * 2u), dim3(BN * 2), 0,
                     stream, a16, x_scale, gate, g, seg, gate_stride, inter, hidden, experts, 2u, up, u, up_stride);
  hipLaunchKernelGGL(moe_silu_scatter_kernel, dim3(pairs), dim3(256), 0, stream, g, u, pos, phi, inter);
  return hipGetLastError();
}

hipError_t launch_moe_down_q4k_grouped(const float* phi, const uint8_t* down, const uint32_t* ids, const float* wts,
                                       float* out, void* workspace, uint32_t hidden, uint32_t inter, uint32_t top_k,
                                       uint64_t down_stride, uint32_t experts, uint32_t tokens, bool accumulate,
                                       hipStream_t stream) {
  const uint32_t pairs = tokens * top_k;
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  uint32_t* seg = reinterpret_cast<uint32_t*>(ws);
  ws += align256((static_cast<size_t>(experts) + 1) * 4);
  uint32_t* pos = reinterpret_cast<uint32_t*>(ws);
  ws += align256(static_cast<size_t>(pairs) * 4);
  float* phi_scale = reinterpret_cast<float*>(ws);
  ws += align256((static_cast<size_t>(pairs) + 256) * 4);
  _Float16* phi16 = reinterpret_cast<_Float16*>(ws);
  ws += align256(static_cast<size_t>(pairs) * inter * 2);
  float* rows = reinterpret_cast<float*>(ws);

  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, seg, pos);
  // source row of pair p is p itself (phi is pair-major): top_k = 1 in the gather
  hipLaunchKernelGGL(rows_to_f16_kernel, dim3(pairs), dim3(256), 0, stream, phi, phi16, phi_scale, inter, pos, 1u);
  constexpr int BM = 32, BN = 64;
  const uint32_t expert_groups = (experts + 7u) / 8u * 8u;
  hipLaunchKernelGGL((q4k_gemm_grouped_kernel<BM, BN>), dim3(expert_groups * ((hidden + BN - 1) / BN)), dim3(BN * 2), 0,
                     stream, phi16, phi_scale, down, rows, seg, down_stride, hidden, inter, experts, 1u, nullptr, nullptr,
                     uint64_t{0});
  const uint64_t outs = static_cast<uint64_t>(tokens) * hidden;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(static_cast<uint32_t>((outs + 255) / 256)), dim3(256), 0, stream, rows, pos,
                     wts, out, tokens, top_k, hidden, accumulate);
  return hipGetLastError();
}

}  // namespace qmm
