// W4A8 GEMM on the CDNA4 scaled MFMA: C = diag(As) . A8 . deq(W)^T.
//
// A8 is the activation already quantized per token to OCP E4M3 codes (m x k bytes)
// with one fp32 scale per row; W is packed MXFP4 (n*k/2 nibble bytes, then n*k/32
// E8M0 bytes; include/tessera/backend.hpp:195-201).  v_mfma_scale_f32_32x32x64_f8f6f4
// multiplies E4M3 by E2M1 natively and applies one E8M0 scale per lane to the 32
// consecutive K values that lane supplies -- exactly one MX block -- so the weights go
// from memory into the matrix core as they are: no dequantization, no folding to
// E4M3 (the reference's gfx12 path folds and loses the small exponents,
// src/core/numerics/quant.cpp:842-898).  Products are exact; the only rounding is the
// fp32 accumulation, so the result equals the reference's QuantizeFp8Ref + GemmMxFp4Ref
// up to summation order.
//
// Tiling: a 256-thread workgroup owns a 128 x 128 tile of C; each of its four
// wavefronts a 64 x 64 quadrant (2 x 2 MFMA tiles of 32 x 32, 64 accumulator
// registers).  K advances 256 per step: the activation tile (128 x 256 bytes) goes
// through LDS, padded so the 16-byte fragment reads spread over all banks; the weight
// fragments are 16-byte loads straight from global memory into the B operand, one
// MX block per lane, with the next step's loads issued before the current step's
// MFMAs.

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

constexpr int kBM = 128, kBN = 128, kKS = 256;      // workgroup tile, K per step
constexpr int kARow = kKS + 16;                      // padded LDS row of the A tile, bytes
constexpr int kSteps = kKS / 64;                     // MFMA K-steps per K step

struct BFrag {
  uint4 q[kSteps][2];   // [k-step][n-subtile]: 32 E2M1 values of one MX block
  uint2 s[2];           // 8 E8M0 bytes per n-subtile: the row's blocks of this K step
};

__global__ __launch_bounds__(256) void mxfp4_a8_gemm_kernel(
    const uint8_t* __restrict__ a8, const float* __restrict__ as, const uint8_t* __restrict__ w,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k) {
  __shared__ __attribute__((aligned(16))) uint8_t lds_a[kBM * kARow];

  const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
  const uint32_t wm = wave >> 1, wn = wave & 1u;          // quadrant of the tile
  const uint32_t m0 = blockIdx.y * kBM, n0 = blockIdx.x * kBN;
  const uint32_t l32 = lane & 31u, kg = lane >> 5;        // MFMA row/column and K half
  const uint8_t* scales = w + static_cast<size_t>(n) * k / 2;
  const uint32_t row_bytes = k / 2, row_blocks = k / 32;

  // Weight rows of this lane's two n-subtiles (clamped at the matrix edge; the stores
  // are masked instead).
  uint32_t wrow[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint32_t r = n0 + wn * 64u + j * 32u + l32;
    wrow[j] = r < n ? r : n - 1u;
  }

  auto load_b = [&](uint32_t k0, BFrag& f) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint8_t* row = w + static_cast<size_t>(wrow[j]) * row_bytes + k0 / 2;
#pragma unroll
      for (int ks = 0; ks < kSteps; ++ks) {
        f.q[ks][j] = load_u4(row + ks * 32 + kg * 16);   // block 2*ks + kg of this step
      }
      f.s[j] = *reinterpret_cast<const uint2*>(scales + static_cast<size_t>(wrow[j]) * row_blocks + k0 / 32);
    }
  };

  // Activation tile staging: thread t moves 16 bytes of row (t / 16) + 16 * i, i = 0..7.
  const uint32_t a_col = (t & 15u) * 16u, a_row = t >> 4;
  auto load_a = [&](uint32_t k0, uint4 (&r)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t row = m0 + a_row + 16u * i;
      r[i] = row < m ? load_u4(a8 + static_cast<size_t>(row) * k + k0 + a_col) : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_a = [&](const uint4 (&r)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      *reinterpret_cast<uint4*>(&lds_a[(a_row + 16u * i) * kARow + a_col]) = r[i];
    }
  };

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  BFrag bcur, bnext;
  uint4 areg[8];
  load_a(0, areg);
  load_b(0, bcur);

  for (uint32_t k0 = 0; k0 < k; k0 += kKS) {
    __syncthreads();        // the previous step's fragment reads are done
    store_a(areg);
    __syncthreads();
    const uint32_t kn = k0 + kKS;
    if (kn < k) {           // uniform: prefetch the next step while this one computes
      load_a(kn, areg);
      load_b(kn, bnext);
    }
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) {
      int8v_t af[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        // 8-bit A operand: a lane of K half `kg` supplies k = 16*kg + [0,16) in its first
        // four registers and k = 32 + 16*kg + [0,16) in the last four (the instruction is
        // two K=32 steps back to back); the 4-bit B operand is simply k = 32*kg + [0,32).
        const uint8_t* p = &lds_a[(wm * 64u + i * 32u + l32) * kARow + ks * 64 + kg * 16u];
        const uint4 lo = *reinterpret_cast<const uint4*>(p);
        const uint4 hi = *reinterpret_cast<const uint4*>(p + 32);
        af[i] = int8v_t{static_cast<int>(lo.x), static_cast<int>(lo.y), static_cast<int>(lo.z),
                        static_cast<int>(lo.w), static_cast<int>(hi.x), static_cast<int>(hi.y),
                        static_cast<int>(hi.z), static_cast<int>(hi.w)};
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const uint4 q = bcur.q[ks][j];
        const int8v_t bf = int8v_t{static_cast<int>(q.x), static_cast<int>(q.y), static_cast<int>(q.z),
                                   static_cast<int>(q.w), 0, 0, 0, 0};
        // Scale byte of block 2*ks + kg: lanes of the upper K half shift their eight
        // bytes down by one so that every lane finds it at byte 2*ks.
        const uint64_t s64 = (static_cast<uint64_t>(bcur.s[j].y) << 32 | bcur.s[j].x) >> (kg * 8u);
        const int sreg = static_cast<int>(ks < 2 ? static_cast<uint32_t>(s64) : static_cast<uint32_t>(s64 >> 32));
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          // A: E4M3 (cbsz 0) with unit scale (E8M0 127); B: E2M1 (blgp 4) with the block scale.
          if ((ks & 1) == 0) {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf, acc[i][j], 0, 4, 0, 0x7F7F7F7F, 0, sreg);
          } else {
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf, acc[i][j], 0, 4, 0, 0x7F7F7F7F, 2, sreg);
          }
        }
      }
    }
    if (kn < k) bcur = bnext;
  }

  // Epilogue: lane holds column l32 and rows (e/4)*8 + kg*4 + e%4 of each 32 x 32 tile.
#pragma unroll
  for (int i = 0; i < 2; ++i) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const uint32_t col = n0 + wn * 64u + j * 32u + l32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = m0 + wm * 64u + i * 32u + (e >> 2) * 8u + kg * 4u + (e & 3u);
        if (row < m && col < n) c[static_cast<size_t>(row) * n + col] = acc[i][j][e] * as[row];
      }
    }
  }
}

}  // namespace

bool gemm_mxfp4_a8_supported(uint64_t k) { return k % 256 == 0; }

hipError_t launch_mxfp4_a8_gemm(const uint8_t* a8, const float* as, const uint8_t* w, float* c,
                                uint32_t m, uint32_t n, uint32_t k, hipStream_t stream) {
  const dim3 grid((n + kBN - 1) / kBN, (m + kBM - 1) / kBM);
  hipLaunchKernelGGL(mxfp4_a8_gemm_kernel, grid, dim3(256), 0, stream, a8, as, w, c, m, n, k);
  return hipGetLastError();
}

}  // namespace qmm
