// Q4_K prefill GEMM on MFMA: C (m x n fp32) = A (m x k) . deq(W)^T, W = n rows of k/256
// Q4_K super-blocks (src/core/numerics/quant.hpp:11-15; reference kernel
// src/backends/rocm/rocm_kernels_wmma.cpp:30-80,334-431, which stages A and the decoded
// weights in LDS as fp16 and accumulates in fp32).
//
// Two launches.  (1) The activations are converted once to fp16 in a workspace (the
// reference converts them again in every workgroup; done once, the GEMM reads 2 bytes per
// activation instead of 4 and the conversion costs one pass over A).  (2) The GEMM proper:
// v_mfma_f32_32x32x16_f16, fp32 accumulate.
//
// Weights never exist dequantized in memory: the raw 144-byte super-blocks travel
// HBM -> LDS by direct loads, and each wavefront decodes the eight weights a lane owes the
// B operand of one MFMA straight from those bytes into registers -- nibbles to fp16 with
// the 0x6400 exponent trick, then one packed fma with the sub-block's (d*sc, dmin*mn) pair,
// i.e. w16 = fma(q, RN16(d*sc), -RN16(dmin*mn)).  A wavefront owns 32 output columns and all
// of the tile's rows, so no two wavefronts decode the same weight.  The nibble pairs come out
// of a dword in the order (k0,k2),(k1,k3); instead of un-shuffling them, the fp16 copy of A
// is written with the same order inside every group of 8, which a dot product cannot see.
//
// K advances one 32-wide sub-block per step: activation slices (BM x 64 bytes) run through
// a four-stage XOR-swizzled LDS ring, raw weight super-blocks through a two-stage ring that
// is refilled once per eight steps; waits are counted by hand as in gemm_mxfp4.hip.

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

__device__ __forceinline__ void direct_load16(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// fp32 -> fp16 (round to nearest even) with the order 0,2,1,3,4,6,5,7 inside each group of 8.
__global__ __launch_bounds__(256) void a_to_f16_kernel(const float* __restrict__ a, _Float16* __restrict__ out,
                                                       uint64_t groups) {
  const uint64_t g = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (g >= groups) return;
  const float4 lo = reinterpret_cast<const float4*>(a)[2 * g];
  const float4 hi = reinterpret_cast<const float4*>(a)[2 * g + 1];
  half8_t v;
  v[0] = static_cast<_Float16>(lo.x);
  v[1] = static_cast<_Float16>(lo.z);
  v[2] = static_cast<_Float16>(lo.y);
  v[3] = static_cast<_Float16>(lo.w);
  v[4] = static_cast<_Float16>(hi.x);
  v[5] = static_cast<_Float16>(hi.z);
  v[6] = static_cast<_Float16>(hi.y);
  v[7] = static_cast<_Float16>(hi.w);
  reinterpret_cast<half8_t*>(out)[g] = v;
}

// Two packed fp16 weights from the nibbles at bits [3:0] and [19:16] of `x`.
__device__ __forceinline__ half2_t decode_pair(uint32_t x, half2_t scale, half2_t neg_min) {
  const half2_t q = bit_cast<half2_t>((x & 0x000F000Fu) | 0x64006400u) - half2_t{1024, 1024};  // exact 0..15
  return __builtin_elementwise_fma(q, scale, neg_min);
}

template <int BM, int BN>
__global__ __launch_bounds__(BN * 2) void q4k_gemm_kernel(
    const _Float16* __restrict__ a16, const uint8_t* __restrict__ w, float* __restrict__ c,
    uint32_t m, uint32_t n, uint32_t k, uint32_t n_begin, uint32_t n_end) {
  constexpr int kWaves = BN / 32;                  // one wavefront per 32 output columns
  constexpr int kTI = BM / 32;                     // MFMA tiles per wavefront (all rows of the tile)
  constexpr int kABlk = BM / 16 / kWaves;          // 1 KB activation blocks a wavefront loads per step
  constexpr int kWL = (BN * 9 + 64 * kWaves - 1) / (64 * kWaves);  // 1 KB weight blocks per super-block
  constexpr uint32_t kAStage = BM * 64, kWStage = kWL * kWaves * 1024;
  static_assert(BM % (16 * kWaves) == 0 && BN % 32 == 0, "tile shape");
  __shared__ __attribute__((aligned(16))) uint8_t lds[4 * kAStage + 2 * kWStage];

  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t l32 = lane & 31u, kg = lane >> 5;
  const uint32_t tiles_n = (n_end - n_begin + BN - 1) / BN;
  const uint32_t m0 = (blockIdx.x / tiles_n) * BM, n0 = n_begin + (blockIdx.x % tiles_n) * BN;
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

  float16_t acc[kTI];
#pragma unroll
  for (int i = 0; i < kTI; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;

  // This lane's weight row inside a raw stage, and its activation fragment offsets: MFMA
  // step t of a slice takes chunk 2t + kg of the row (k = 16t + 8kg + [0,8)).
  const uint32_t w_row = (wave * 32u + l32) * 144u;
  uint32_t a_fr[2];
#pragma unroll
  for (int tt = 0; tt < 2; ++tt) a_fr[tt] = l32 * 64u + (((tt * 2u + kg) ^ ((l32 >> 2) & 3u)) * 16u);

  const uint32_t slices = k / 32;
  uint32_t d_bits = 0, sc0 = 0, sc1 = 0, sc2 = 0;   // header and packed scales of the current super-block

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
    d_bits = *reinterpret_cast<const uint32_t*>(raw);
    sc0 = *reinterpret_cast<const uint32_t*>(raw + 4);
    sc1 = *reinterpret_cast<const uint32_t*>(raw + 8);
    sc2 = *reinterpret_cast<const uint32_t*>(raw + 12);
    const float d = half_bits_to_float(d_bits & 0xFFFFu), dmin = half_bits_to_float(d_bits >> 16);
#pragma unroll
    for (int sb = 0; sb < 8; ++sb) {
      const uint32_t slice = blk * 8u + sb;
      if (sb == 0 && more) issue_w((blk + 1u) & 1u, blk + 1u);
      issue_a((slice + 3u) & 3u, slice + 3u < slices ? slice + 3u : slices - 1u);

      // 6-bit scale and min of sub-block sb (src/core/numerics/quant.cpp:58-70).
      uint32_t sc, mn;
      if (sb < 4) {
        sc = (sc0 >> (8 * sb)) & 63u;
        mn = (sc1 >> (8 * sb)) & 63u;
      } else {
        const uint32_t hi = (sc2 >> (8 * (sb - 4))) & 0xFFu;
        sc = (hi & 15u) | (((sc0 >> (8 * (sb - 4) + 6)) & 3u) << 4);
        mn = (hi >> 4) | (((sc1 >> (8 * (sb - 4) + 6)) & 3u) << 4);
      }
      const _Float16 s16 = static_cast<_Float16>(d * static_cast<float>(sc));
      const _Float16 m16 = static_cast<_Float16>(-(dmin * static_cast<float>(mn)));
      const half2_t scale = {s16, s16}, neg_min = {m16, m16};

      // Quant bytes of this lane's 16 weights: sub-block sb lives in the low (even sb) or high
      // nibbles of bytes (sb/2)*32 + [0,32) (src/core/numerics/quant.cpp:656-675).
      const uint8_t* qp = raw + 16 + (sb >> 1) * 32 + kg * 8u;
      const uint2 q0 = *reinterpret_cast<const uint2*>(qp);
      const uint2 q1 = *reinterpret_cast<const uint2*>(qp + 16);
      constexpr int kNoShift = 0;
      const int sh = (sb & 1) ? 4 : kNoShift;
      half8_t b[2];
      {
        const half2_t p0 = decode_pair(q0.x >> sh, scale, neg_min), p1 = decode_pair(q0.x >> (sh + 8), scale, neg_min);
        const half2_t p2 = decode_pair(q0.y >> sh, scale, neg_min), p3 = decode_pair(q0.y >> (sh + 8), scale, neg_min);
        b[0] = half8_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
      }
      {
        const half2_t p0 = decode_pair(q1.x >> sh, scale, neg_min), p1 = decode_pair(q1.x >> (sh + 8), scale, neg_min);
        const half2_t p2 = decode_pair(q1.y >> sh, scale, neg_min), p3 = decode_pair(q1.y >> (sh + 8), scale, neg_min);
        b[1] = half8_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
      }

      const uint8_t* a_stage = lds + (slice & 3u) * kAStage;
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
        for (int i = 0; i < kTI; ++i) {
          const half8_t af = *reinterpret_cast<const half8_t*>(a_stage + a_fr[tt] + i * 32 * 64);
          acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, b[tt], acc[i], 0, 0, 0);
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
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive the workgroup

  // Epilogue: lane holds column l32 and rows (e/4)*8 + kg*4 + e%4 of each 32 x 32 tile.
  const uint32_t col = n0 + wave * 32u + l32;
#pragma unroll
  for (int i = 0; i < kTI; ++i) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const uint32_t row = m0 + i * 32u + (e >> 2) * 8u + kg * 4u + (e & 3u);
      if (row < m && col < n_end) c[static_cast<size_t>(row) * n + col] = acc[i][e];
    }
  }
}

template <int BM, int BN>
void launch_range(const _Float16* a16, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                  uint32_t n_begin, uint32_t n_end, hipStream_t stream) {
  const uint32_t tiles = ((m + BM - 1) / BM) * ((n_end - n_begin + BN - 1) / BN);
  hipLaunchKernelGGL((q4k_gemm_kernel<BM, BN>), dim3(tiles), dim3(BN * 2), 0, stream, a16, w, c, m, n, k, n_begin, n_end);
}

}  // namespace

bool gemm_q4k_supported(uint64_t m, uint64_t k) { return k % 256 == 0 && k <= (1u << 20) && m * k < (1ull << 31); }

size_t gemm_q4k_workspace_bytes(uint64_t m, uint64_t k) { return static_cast<size_t>(m) * k * 2; }

// The bulk of C goes to 256 x 256 tiles, whole rounds of one tile per CU; columns left over
// when the tile count is not a multiple of the CU count are cut into 128 x 64 tiles that
// spread over every CU instead of keeping a few CUs busy for a whole extra round.
hipError_t launch_q4k_gemm(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m,
                           uint32_t n, uint32_t k, hipStream_t stream) {
  _Float16* a16 = static_cast<_Float16*>(workspace);
  const uint64_t groups = static_cast<uint64_t>(m) * k / 8;
  hipLaunchKernelGGL(a_to_f16_kernel, dim3(static_cast<uint32_t>((groups + 255) / 256)), dim3(256), 0, stream, a, a16, groups);
  const uint32_t cus = static_cast<uint32_t>(num_cus());
  const uint32_t tiles_m = (m + 255u) / 256u, tiles_n = (n + 255u) / 256u;
  const uint32_t tiles = tiles_m * tiles_n;
  uint32_t main_tn = tiles_n;
  if (tiles > cus && tiles % cus != 0 && tiles % cus <= cus / 2) {
    main_tn = (tiles / cus) * cus / tiles_m;
  } else if (tiles < cus / 2) {
    main_tn = 0;
  }
  const uint32_t n_split = main_tn * 256u < n ? main_tn * 256u : n;
  if (n_split > 0) launch_range<256, 256>(a16, w, c, m, n, k, 0u, n_split, stream);
  if (n_split < n) launch_range<128, 64>(a16, w, c, m, n, k, n_split, n, stream);
  return hipGetLastError();
}

}  // namespace qmm
