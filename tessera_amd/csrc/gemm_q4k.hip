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

#include "q4k_tile.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

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


template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * 64) void q4k_gemm_kernel(
    const _Float16* __restrict__ a16, const float* __restrict__ a_scale, const uint8_t* __restrict__ w,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k, uint32_t n_begin, uint32_t n_end) {
  const uint32_t tiles_n = (n_end - n_begin + BN - 1) / BN;
  q4k_gemm_tile<BM, BN, WM, WN>(a16, a_scale, w, c, m, n, k, (blockIdx.x / tiles_n) * BM, n_begin + (blockIdx.x % tiles_n) * BN,
                        n_end);
}

template <int BM, int BN, int WM = BM, int WN = 32>
void launch_range(const _Float16* a16, const float* a_scale, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                  uint32_t k, uint32_t n_begin, uint32_t n_end, hipStream_t stream) {
  const uint32_t tiles = ((m + BM - 1) / BM) * ((n_end - n_begin + BN - 1) / BN);
  hipLaunchKernelGGL((q4k_gemm_kernel<BM, BN, WM, WN>), dim3(tiles), dim3(tile_waves<BM, BN, WM, WN>() * 64), 0, stream,
                     a16, a_scale, w, c, m, n, k, n_begin, n_end);
}

}  // namespace

void launch_rows_to_f16(const float* src, _Float16* dst, float* scale, uint32_t rows, uint32_t cols, const uint32_t* pos,
                        uint32_t top_k, hipStream_t stream) {
  hipLaunchKernelGGL(rows_to_f16_kernel, dim3(rows), dim3(256), 0, stream, src, dst, scale, cols, pos, top_k);
}

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
  launch_rows_to_f16(a, a16, a_scale, m, k, nullptr, 1u, stream);
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
  launch_rows_to_f16(a, a16, a_scale, m, k, nullptr, 1u, stream);
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

}  // namespace qmm
