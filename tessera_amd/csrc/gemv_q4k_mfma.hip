// Q4_K x a few fp32 activation rows (1..8) on the 4x4x4 fp16 MFMA, exact on the weight side.
//
//   C[r][n] = sum_k A[r][k] * deq(W)[n][k],   W = n rows of k/256 Q4_K super-blocks
//   (layout and decode: src/core/numerics/quant.cpp:57-117, GemmQ4KRef gemm.cpp:167-214).
//
// v_mfma_f32_4x4x4_16B_f16 is sixteen independent 4x4x4 products, one per quad of lanes.  Here a
// lane owns one weight row: it supplies four weights per instruction as the B operand and gets
// back, in its own four result registers, that row's partial dot products with four activation
// columns (probed on hardware: block = lane/4, A row = lane%4, B column = lane%4, D register e
// = A row e of the lane's column).  So the per-sub-block scale is applied by the lane that
// decoded it, with no transposition, and the multiply-adds leave the vector ALU:
//
//  * weights enter as the raw nibbles, masked in place, read as fp16 subnormals (n * 2^-24;
//    the matrix core honours them, probed); the high nibble stays at bit 4 (16 n) and the
//    activations of odd sub-blocks are stored divided by 16.  Five VALU operations per 8 weights.
//  * an activation row is two fp16 columns, hi = f16(x s) and lo = f16(x s - hi), s the row's
//    power of two that brings its largest magnitude to [256, 512): 22 significant bits, no
//    overflow, exact rescaling.  Products of a 4-bit integer and an 11-bit value are exact in the
//    fp32 accumulator.
//  * per sub-block the four accumulators are folded with d*sc; the -dmin*mn term is two more
//    MFMA steps of the mins (as subnormals) against the sub-block sums of the activations.
//
// A workgroup is ONE wavefront with a private ring of LDS stages filled by direct HBM->LDS
// loads (raw super-blocks, 144 bytes per lane-row, and the matching activation slices), so there
// is no barrier anywhere and wavefronts on a CU drift apart freely.  The 64 lanes are 64/KS weight
// rows x KS slices of K (more, smaller tiles for matrices with few rows); slices are summed
// through LDS at the end.

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));

constexpr uint32_t kSlots = 33;      // 32 weight dwords per lane and super-block + 1 slot of sub-block sums

__device__ __forceinline__ void dma16(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// Power of two that brings a row with largest magnitude `amax` to [256, 512).
__device__ __forceinline__ float prep_scale(float amax) {
  const uint32_t e = (bit_cast<uint32_t>(amax) >> 23) & 0xFFu;
  if (e == 0u || e == 0xFFu) return 1.0f;
  int se = 262 - static_cast<int>(e);
  se = se < 1 ? 1 : (se > 254 ? 254 : se);
  return bit_cast<float>(static_cast<uint32_t>(se) << 23);
}

struct HiLo {
  _Float16 hi, lo;
};
__device__ __forceinline__ HiLo split16(float v) {
  const _Float16 h = static_cast<_Float16>(v);
  return HiLo{h, static_cast<_Float16>(v - static_cast<float>(h))};
}

// Activation operand, one workgroup per pair of columns (row r -> columns 2r, 2r+1 = hi, lo):
//   xop[sb][slot][chain][col][8 halves],  chain = r / (XC/2), col = 2 * (r % (XC/2)) + {0,1}.
// Slot dw < 32 holds what weight dword dw of a lane's super-block multiplies: bytes 4*(dw%8)..+3
// of group g = dw/8, i.e. elements e0..e0+3 (e0 = 4*(dw%8)) of sub-block 2g in halves 0-3 and
// of sub-block 2g+1 (divided by 16) in halves 4-7, each in the order e0, e0+2, e0+1, e0+3 that
// the nibble masks produce.  Slot 32 holds the sub-block sums, order 0,2,1,3 | 4,6,5,7.
// Rows at and past m are written as zeros.
template <int XC>
__global__ __launch_bounds__(256) void q4k_rows_prep_kernel(const float* __restrict__ a, _Float16* __restrict__ xop,
                                                            float* __restrict__ inv_scale, uint32_t m,
                                                            uint32_t k, uint32_t chains) {
  __shared__ float red[4];
  const uint32_t r = blockIdx.x, t = threadIdx.x;
  const bool live = r < m;
  const float* row = a + static_cast<size_t>(live ? r : 0u) * k;
  float amax = 0.0f;
  if (live) {
    for (uint32_t i = t; i < k / 4u; i += 256u) {
      const float4 v = reinterpret_cast<const float4*>(row)[i];
      amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fmaxf(fabsf(v.z), fabsf(v.w)), amax));
    }
  }
  amax = wave_max(amax);
  if ((t & 63u) == 0) red[t >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = live ? prep_scale(amax) : 0.0f;
  if (t == 0 && live && blockIdx.y == 0) inv_scale[r] = 1.0f / s;

  constexpr uint32_t kRowsPerChain = XC / 2;
  const uint32_t chain = r / kRowsPerChain, col = 2u * (r % kRowsPerChain);
  const uint32_t sbs = k / 256u;
  auto dst = [&](uint32_t sb, uint32_t slot, uint32_t c) {
    return xop + ((((static_cast<size_t>(sb) * kSlots + slot) * chains + chain) * XC + c) * 8u);
  };
  // One item = one slot: four elements of sub-block 2g and four of 2g+1.  The eight lanes that
  // share g (consecutive, since 256 is a multiple of 8) add up the two sub-block sums of what the
  // matrix core will see (hi + lo, undivided); the sums are themselves split into hi and lo.
  constexpr uint32_t kOrder[8] = {0, 2, 1, 3, 4, 6, 5, 7};
  // grid.y workgroups share a row: each finds the row's maximum for itself (the row is a few
  // tens of KB in L2) and converts 256 slots, so the pre-pass is one short wave of work.
  {
    const uint32_t i = blockIdx.y * 256u + t;
    const bool in = i < sbs * 32u;
    const uint32_t sb = in ? i / 32u : 0u, dw = i % 32u, g = dw / 8u, e0 = 4u * (dw % 8u);
    const float4 ev = *reinterpret_cast<const float4*>(row + sb * 256u + (2u * g) * 32u + e0);
    const float4 od = *reinterpret_cast<const float4*>(row + sb * 256u + (2u * g + 1u) * 32u + e0);
    float v[8] = {ev.x * s, ev.z * s, ev.y * s, ev.w * s, od.x * s, od.z * s, od.y * s, od.w * s};
    half8_t hi, lo;
    float se = 0.0f, so = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (!live) v[j] = 0.0f;
      const HiLo p = split16(v[j]);
      const float seen = static_cast<float>(p.hi) + static_cast<float>(p.lo);
      if (j < 4) {
        se += seen, hi[j] = p.hi, lo[j] = p.lo;
      } else {                       // high nibbles stay at bit 4: their activations carry the 1/16
        so += seen;
        hi[j] = static_cast<_Float16>(static_cast<float>(p.hi) * 0.0625f);
        lo[j] = static_cast<_Float16>(static_cast<float>(p.lo) * 0.0625f);
      }
    }
#pragma unroll
    for (int off = 1; off < 8; off <<= 1) {
      se += __shfl_xor(se, off, kWave);
      so += __shfl_xor(so, off, kWave);
    }
    if (in) {
      *reinterpret_cast<half8_t*>(dst(sb, dw, col)) = hi;
      *reinterpret_cast<half8_t*>(dst(sb, dw, col + 1u)) = lo;
      if (dw % 8u == 0) {
        const HiLo pe = split16(se), po = split16(so);
        dst(sb, 32u, col)[kOrder[2u * g]] = pe.hi;
        dst(sb, 32u, col + 1u)[kOrder[2u * g]] = pe.lo;
        dst(sb, 32u, col)[kOrder[2u * g + 1u]] = po.hi;
        dst(sb, 32u, col + 1u)[kOrder[2u * g + 1u]] = po.lo;
      }
    }
  }
}

// KS: consecutive super-blocks of a row per stage, one per lane group ("slice"); KH: lanes that share one super-block (each takes 4/KH of its
// four 64-weight groups), so a wavefront covers 64/(KS*KH) weight rows; NC: chains of XC
// activation columns; XC: columns per chain that exist in memory (2: one row, lanes 2,3 of a
// quad re-read columns 0,1; 4: two rows); DEPTH: ring stages.
template <int KS, int KH, int NC, int XC, int DEPTH>
__global__ __launch_bounds__(64) void q4k_gemv_mfma_kernel(const uint8_t* __restrict__ w,
                                                           const uint8_t* __restrict__ xop,
                                                           const float* __restrict__ inv_scale,
                                                           float* __restrict__ c, uint32_t m, uint32_t n,
                                                           uint32_t k) {
  static_assert(KH == 1 || KH == 2, "a super-block is whole or split in two");
  constexpr uint32_t kRows = 64 / (KS * KH);               // weight rows of this wavefront
  constexpr uint32_t kRowQuads = kRows / 4;
  constexpr uint32_t kBlocks = kRows * KS;                 // super-blocks per stage
  constexpr uint32_t kWBytes = kBlocks * kQ4KBlockBytes;
  constexpr uint32_t kWGran = kWBytes / 16;
  constexpr int kWDma = (kWGran + 63) / 64;
  constexpr uint32_t kXsb = kSlots * NC * XC * 16;         // activation bytes per super-block
  constexpr uint32_t kXGran = KS * kXsb / 16;              // 16-byte granules of activations per stage
  constexpr int kXDma = (kXGran + 63) / 64;
  constexpr int kDma = kWDma + kXDma;
  constexpr uint32_t kStage = kWBytes + KS * kXsb;
  constexpr int kGroups = 4 / KH;                          // 64-weight groups a lane multiplies per stage
  static_assert((DEPTH - 1) * kDma <= 63, "vmcnt is a 6-bit counter");
  static_assert(kStage % 16 == 0, "stage alignment");
  static_assert(DEPTH * kStage >= NC * 4 * 64 * 4, "the final reduction reuses the ring");
  __shared__ __attribute__((aligned(16))) uint8_t lds[DEPTH * kStage];

  const uint32_t lane = threadIdx.x;
  // quad -> (row quad, slice of K, part of the super-block); the four lanes of a quad are four rows.
  const uint32_t quad = lane >> 2;
  const uint32_t rq = quad % kRowQuads, sl = (quad / kRowQuads) % KS, part = quad / (kRowQuads * KS);
  const uint32_t rl = rq * 4u + (lane & 3u);               // row inside the tile
  const uint32_t lrow = sl * kRows + rl;                   // this lane's super-block inside a stage
  const uint32_t sbs = k / 256u, sps = sbs / KS;           // super-blocks per row and per slice
  const uint32_t row_bytes = sbs * kQ4KBlockBytes;
  const uint32_t row0 = blockIdx.x * kRows;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)lds));

  // Direct loads of one stage.  Weights: granule G = i*64 + lane is 16 bytes G%9 of stage block
  // G/9 = (slice, row).  Activations: granule G of the KS slices' operand blocks.
  uint32_t w_src[kWDma], x_src[kXDma];
#pragma unroll
  for (int i = 0; i < kWDma; ++i) {
    uint32_t g = i * 64u + lane;
    g = g < kWGran ? g : kWGran - 1u;
    const uint32_t blk = g / 9u, piece = g % 9u, bs = blk / kRows, br = blk % kRows;
    const uint32_t grow = row0 + br < n ? row0 + br : n - 1u;
    w_src[i] = grow * row_bytes + bs * kQ4KBlockBytes + piece * 16u;
  }
#pragma unroll
  for (int i = 0; i < kXDma; ++i) {
    uint32_t g = i * 64u + lane;
    g = g < kXGran ? g : kXGran - 1u;
    x_src[i] = g * 16u;
  }
  auto issue = [&](uint32_t slot, uint32_t st) {
    const uint32_t stage = lds_base + slot * kStage;
    const uint8_t* wb = w + static_cast<size_t>(st) * (KS * kQ4KBlockBytes);
    const uint8_t* xb = xop + static_cast<size_t>(st) * (KS * kXsb);
    // A last, partial block is never empty: lane 0 is always in it.
#pragma unroll
    for (int i = 0; i < kWDma; ++i) {
      if (i + 1 < kWDma || kWGran % 64u == 0) {
        dma16(wb, w_src[i], stage + i * 1024u);
      } else if (lane < kWGran % 64u) {
        dma16(wb, w_src[i], stage + i * 1024u);
      }
    }
#pragma unroll
    for (int i = 0; i < kXDma; ++i) {
      if (i + 1 < kXDma || kXGran % 64u == 0) {
        dma16(xb, x_src[i], stage + kWBytes + i * 1024u);
      } else if (lane < kXGran % 64u) {
        dma16(xb, x_src[i], stage + kWBytes + i * 1024u);
      }
    }
  };

  float4_t tot[NC];
#pragma unroll
  for (int ch = 0; ch < NC; ++ch) tot[ch] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  const float4_t zero = float4_t{0.0f, 0.0f, 0.0f, 0.0f};

#pragma unroll
  for (int s = 0; s < DEPTH - 1; ++s) issue(s, static_cast<uint32_t>(s) < sps ? s : sps - 1u);

  uint32_t slot = 0;
  for (uint32_t st = 0; st < sps; ++st) {
    {
      // The slot refilled now was read in the previous iteration: its LDS reads have returned
      // (every value was consumed), and a wavefront's direct loads write LDS in issue order.
      const uint32_t nxt = st + DEPTH - 1u;
      const uint32_t fill = slot == 0 ? DEPTH - 1u : slot - 1u;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      issue(fill, nxt < sps ? nxt : sps - 1u);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * kDma) : "memory");
    const uint8_t* stage = lds + slot * kStage;
    const uint8_t* blk = stage + lrow * kQ4KBlockBytes;
    const uint8_t* xs = stage + kWBytes + sl * kXsb + (part * kGroups * 8u) * (NC * XC * 16u) + (lane & (XC - 1u)) * 16u;

    // The LDS reads are issued well ahead of their use (a wavefront is often alone on its SIMD,
    // so nothing else hides the LDS latency): the whole stage up front when its activation
    // operand fits the register file, else one 64-weight group at a time.
    constexpr bool kWholeStage = NC <= 2;
    constexpr int kXv = kWholeStage ? 8 * kGroups * NC : 8 * NC;
    uint4 hq[1 + 2 * kGroups], xv[kXv], xm[NC];
    hq[0] = *reinterpret_cast<const uint4*>(blk);
#pragma unroll
    for (int i = 0; i < 2 * kGroups; ++i) hq[1 + i] = *reinterpret_cast<const uint4*>(blk + 16 + part * kGroups * 32u + i * 16);
    if constexpr (kWholeStage) {
#pragma unroll
      for (int i = 0; i < kXv; ++i) xv[i] = *reinterpret_cast<const uint4*>(xs + i * (XC * 16));
    }
#pragma unroll
    for (int ch = 0; ch < NC; ++ch)
      xm[ch] = *reinterpret_cast<const uint4*>(stage + kWBytes + sl * kXsb + (32 * NC + ch) * (XC * 16) + (lane & (XC - 1u)) * 16u);
    asm volatile("" ::: "memory");

    const uint4 h = hq[0];
    const float d24 = half_bits_to_float(h.x & 0xFFFFu) * 0x1p24f;
    const float dmin24 = half_bits_to_float(h.x >> 16) * 0x1p24f;
    const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    // The scales of this lane's groups: bytes 0..3 = sub-blocks 2*g0 .. 2*g0+3.
    const uint32_t scw = KH == 1 ? 0u : (part == 0 ? sc_lo : sc_hi);

#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
      const uint4 qa = hq[1 + 2 * g], qb = hq[2 + 2 * g];
      const uint32_t qw[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
      if constexpr (!kWholeStage) {
#pragma unroll
        for (int i = 0; i < kXv; ++i) xv[i] = *reinterpret_cast<const uint4*>(xs + (g * kXv + i) * (XC * 16));
        asm volatile("" ::: "memory");
      }
      float4_t acc_e[NC], acc_o[NC];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t v = qw[i], v8 = v >> 8;
        const half4_t be = bit_cast<half4_t>(uint2{v & 0x000F000Fu, v8 & 0x000F000Fu});
        const half4_t bo = bit_cast<half4_t>(uint2{v & 0x00F000F0u, v8 & 0x00F000F0u});
#pragma unroll
        for (int ch = 0; ch < NC; ++ch) {
          const uint4 x4 = xv[((kWholeStage ? g * 8 : 0) + i) * NC + ch];
          const half4_t ae = bit_cast<half4_t>(uint2{x4.x, x4.y});
          const half4_t ao = bit_cast<half4_t>(uint2{x4.z, x4.w});
          acc_e[ch] = __builtin_amdgcn_mfma_f32_4x4x4f16(ae, be, i == 0 ? zero : acc_e[ch], 0, 0, 0);
          acc_o[ch] = __builtin_amdgcn_mfma_f32_4x4x4f16(ao, bo, i == 0 ? zero : acc_o[ch], 0, 0, 0);
        }
      }
      const uint32_t word = KH == 1 ? (g < 2 ? sc_lo : sc_hi) : scw;
      const float se = d24 * static_cast<float>((word >> ((2 * g) % 4 * 8)) & 0xFFu);
      const float so = d24 * static_cast<float>((word >> ((2 * g + 1) % 4 * 8)) & 0xFFu);
#pragma unroll
      for (int ch = 0; ch < NC; ++ch) tot[ch] += se * acc_e[ch] + so * acc_o[ch];
    }
    // - dmin * sum_j mn_j * Sx_j: the mins as fp16 subnormals against the sub-block sums
    // (halves 0-3 of the slot: sub-blocks 0,2,1,3; halves 4-7: 4,6,5,7).  With the super-block
    // split in two, each lane takes the step of its own four sub-blocks.
    {
      const half4_t b0 = bit_cast<half4_t>(uint2{mn_lo & 0x00FF00FFu, (mn_lo >> 8) & 0x00FF00FFu});
      const half4_t b1 = bit_cast<half4_t>(uint2{mn_hi & 0x00FF00FFu, (mn_hi >> 8) & 0x00FF00FFu});
#pragma unroll
      for (int ch = 0; ch < NC; ++ch) {
        const uint4 x4 = xm[ch];
        float4_t mm;
        if (KH == 1) {
          mm = __builtin_amdgcn_mfma_f32_4x4x4f16(bit_cast<half4_t>(uint2{x4.x, x4.y}), b0, zero, 0, 0, 0);
          mm = __builtin_amdgcn_mfma_f32_4x4x4f16(bit_cast<half4_t>(uint2{x4.z, x4.w}), b1, mm, 0, 0, 0);
        } else {
          const half4_t am = bit_cast<half4_t>(part == 0 ? uint2{x4.x, x4.y} : uint2{x4.z, x4.w});
          const half4_t bm = part == 0 ? b0 : b1;
          mm = __builtin_amdgcn_mfma_f32_4x4x4f16(am, bm, zero, 0, 0, 0);
        }
        tot[ch] -= dmin24 * mm;
      }
    }
    slot = slot + 1u == DEPTH ? 0u : slot + 1u;
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // no direct load may outlive its workgroup

  // Sum the lanes that share a weight row (stage memory is free now) and store: registers
  // e = 0,1 are the hi and lo columns of the chain's first activation row, e = 2,3 of its second.
  float* red = reinterpret_cast<float*>(lds);                   // [NC][4][64]
#pragma unroll
  for (int ch = 0; ch < NC; ++ch)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[(ch * 4 + e) * 64 + lane] = tot[ch][e];
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  if (quad < kRowQuads && row0 + rl < n) {
#pragma unroll
    for (int ch = 0; ch < NC; ++ch) {
      float4_t sum = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int s = 0; s < KS * KH; ++s)
#pragma unroll
        for (int e = 0; e < 4; ++e) sum[e] += red[(ch * 4 + e) * 64 + lane + s * kRows];
      constexpr uint32_t kRowsPerChain = XC / 2;
      const uint32_t r0 = ch * kRowsPerChain;
      if (r0 < m) c[static_cast<size_t>(r0) * n + row0 + rl] = (sum[0] + sum[1]) * inv_scale[r0];
      if (XC == 4 && r0 + 1u < m) c[static_cast<size_t>(r0 + 1u) * n + row0 + rl] = (sum[2] + sum[3]) * inv_scale[r0 + 1u];
    }
  }
}

// ---- one or two rows, activations resident in LDS --------------------------------------------
// The kernel above marches every weight row along K in 144-byte steps, which DRAM serves badly.
// Here a wavefront's stage is four weight rows x eight consecutive super-blocks: four runs of
// 1152 contiguous bytes, lane quad j = (super-block j/2, half j%2).  The quads of a wavefront then
// sit at different K, so the activation operand cannot be streamed per stage; instead the
// workgroup (eight wavefronts, one per CU) converts the whole activation rows once into LDS,
// with the per-row scale computed in place: no pre-pass, no scratch.  Work items are
// (row quad, stage) pairs dealt round-robin to the wavefronts, each with its private ring of
// direct loads; an item's four rows x m partial sums go to an LDS table, and after the last
// item a few threads add each row's stages in order and store (deterministic).
constexpr uint32_t kResWaves = 8;
constexpr uint32_t kItemBytes = 4 * 8 * kQ4KBlockBytes;        // 4608
constexpr int kItemDma = (kItemBytes / 16 + 63) / 64;          // 5, the last covers 32 lanes

template <int NC, int XC, int DEPTH, int S>
__global__ __launch_bounds__(64 * kResWaves) void q4k_rows_resident_kernel(
    const float* __restrict__ a, const uint8_t* __restrict__ w, float* __restrict__ c, uint32_t m, uint32_t n,
    uint32_t k, uint32_t quads_per_wg) {
  constexpr uint32_t kXsb = kSlots * NC * XC * 16;
  constexpr uint32_t kRows = NC * XC / 2;                      // activation rows the operand has room for
  static_assert((DEPTH - 1) * kItemDma <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const uint32_t sbs = k / 256u, stages = (sbs + 7u) / 8u;
  const uint32_t row_bytes = sbs * kQ4KBlockBytes;
  // LDS: rings | activation operand | partial table | row scales
  uint8_t* ring = lds;
  uint8_t* xop = lds + kResWaves * DEPTH * kItemBytes;
  float* partial = reinterpret_cast<float*>(xop + sbs * kXsb);
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t quads = n / 4u;
  const uint32_t q0 = blockIdx.x * quads_per_wg;
  const uint32_t q1 = q0 + quads_per_wg < quads ? q0 + quads_per_wg : quads;
  const uint32_t items = (q1 - q0) * stages;
  float* inv_s = partial + quads_per_wg * stages * 4u * kRows;
  float* wmax_all = inv_s + kRows;                             // [kRows][kResWaves]

  // ---- this wavefront's ring starts filling before the activations are touched
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)ring)) + wave * DEPTH * kItemBytes;
  uint32_t src_full[kItemDma], src_first[kItemDma], src_sbo[kItemDma];
#pragma unroll
  for (int i = 0; i < kItemDma; ++i) {
    uint32_t g = i * 64u + lane;
    g = g < kItemBytes / 16u ? g : kItemBytes / 16u - 1u;
    const uint32_t r = g / 72u, in_row = g % 72u;
    src_full[i] = r * row_bytes + in_row * 16u;
    src_first[i] = r * row_bytes + (in_row % 9u) * 16u;          // the stage's first super-block
    src_sbo[i] = in_row / 9u;
  }
  auto issue = [&](uint32_t slot, uint32_t item) {
    const uint32_t q = q0 + item / stages, st = item % stages;
    const uint32_t lim = sbs - st * 8u;                          // super-blocks this stage really has
    const uint8_t* base = w + static_cast<size_t>(q) * 4u * row_bytes + st * (8u * kQ4KBlockBytes);
    const uint32_t dst = lds_base + slot * kItemBytes;
#pragma unroll
    for (int i = 0; i < kItemDma; ++i) {
      const uint32_t off = src_sbo[i] < lim ? src_full[i] : src_first[i];
      if (i + 1 < kItemDma) {
        dma16(base, off, dst + i * 1024u);
      } else if (lane < (kItemBytes / 16u) % 64u) {
        dma16(base, off, dst + i * 1024u);
      }
    }
  };
  // ---- the activation rows are requested first (a wavefront's loads return in order, so behind
  // the ring they would wait for it): S slots of 4 + 4 elements per thread and row, slot (sb, dw)
  // = elements 4*(dw%8).. of sub-blocks 2*(dw/8) and 2*(dw/8)+1 (layout of q4k_rows_prep_kernel).
  const uint32_t nslots = sbs * 32u;
  float4 ev[kRows][S], od[kRows][S];
#pragma unroll
  for (uint32_t r = 0; r < kRows; ++r) {
    const float* row = a + static_cast<size_t>(r < m ? r : 0u) * k;
#pragma unroll
    for (int j = 0; j < S; ++j) {
      uint32_t i = t + j * (64u * kResWaves);
      i = i < nslots ? i : nslots - 1u;
      const uint32_t sb = i / 32u, dw = i % 32u;
      const float* src = row + sb * 256u + (dw / 8u) * 64u + 4u * (dw % 8u);
      ev[r][j] = *reinterpret_cast<const float4*>(src);
      od[r][j] = *reinterpret_cast<const float4*>(src + 32);
    }
  }
  const uint32_t my_items = items > wave ? (items - wave + kResWaves - 1u) / kResWaves : 0u;
  auto item_of = [&](uint32_t j) { return wave + (j < my_items ? j : my_items - 1u) * kResWaves; };
  if (my_items > 0) {
#pragma unroll
    for (int s = 0; s < DEPTH - 1; ++s) issue(s, item_of(s));
  }

  // ---- rows -> fp16 hi/lo operand in LDS; one barrier for all the row scales
#pragma unroll
  for (uint32_t r = 0; r < kRows; ++r) {
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < S; ++j) {
      amax = fmaxf(amax, fmaxf(fmaxf(fabsf(ev[r][j].x), fabsf(ev[r][j].y)), fmaxf(fabsf(ev[r][j].z), fabsf(ev[r][j].w))));
      amax = fmaxf(amax, fmaxf(fmaxf(fabsf(od[r][j].x), fabsf(od[r][j].y)), fmaxf(fabsf(od[r][j].z), fabsf(od[r][j].w))));
    }
    amax = wave_max(amax);
    if (lane == 0) wmax_all[r * kResWaves + wave] = amax;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
#pragma unroll
  for (uint32_t r = 0; r < kRows; ++r) {
    float amax = 0.0f;
#pragma unroll
    for (uint32_t wv = 0; wv < kResWaves; ++wv) amax = fmaxf(amax, wmax_all[r * kResWaves + wv]);
    const float s = r < m ? prep_scale(amax) : 0.0f;
    if (t == 0) inv_s[r] = r < m ? 1.0f / s : 0.0f;
    const uint32_t chain = r / (XC / 2), col = 2u * (r % (XC / 2));
    constexpr uint32_t kOrder[8] = {0, 2, 1, 3, 4, 6, 5, 7};
#pragma unroll
    for (int j = 0; j < S; ++j) {
      const uint32_t i = t + j * (64u * kResWaves);
      const bool in = i < nslots;
      const uint32_t sb = in ? i / 32u : 0u, dw = i % 32u, g = dw / 8u;
      float v[8] = {ev[r][j].x * s, ev[r][j].z * s, ev[r][j].y * s, ev[r][j].w * s,
                    od[r][j].x * s, od[r][j].z * s, od[r][j].y * s, od[r][j].w * s};
      half8_t hi, lo;
      float se = 0.0f, so = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (r >= m) v[e] = 0.0f;
        const HiLo p = split16(v[e]);
        const float seen = static_cast<float>(p.hi) + static_cast<float>(p.lo);
        if (e < 4) {
          se += seen, hi[e] = p.hi, lo[e] = p.lo;
        } else {
          so += seen;
          hi[e] = static_cast<_Float16>(static_cast<float>(p.hi) * 0.0625f);
          lo[e] = static_cast<_Float16>(static_cast<float>(p.lo) * 0.0625f);
        }
      }
      // the eight slots of a group sit in eight consecutive lanes
#pragma unroll
      for (int off = 1; off < 8; off <<= 1) {
        se += __shfl_xor(se, off, kWave);
        so += __shfl_xor(so, off, kWave);
      }
      if (in) {
        uint8_t* slot = xop + sb * kXsb + ((dw * NC + chain) * XC + col) * 16u;
        *reinterpret_cast<half8_t*>(slot) = hi;
        *reinterpret_cast<half8_t*>(slot + 16) = lo;
        if (dw % 8u == 0) {
          _Float16* sum = reinterpret_cast<_Float16*>(xop + sb * kXsb + ((32u * NC + chain) * XC + col) * 16u);
          const HiLo pe = split16(se), po = split16(so);
          sum[kOrder[2u * g]] = pe.hi, sum[8 + kOrder[2u * g]] = pe.lo;
          sum[kOrder[2u * g + 1u]] = po.hi, sum[8 + kOrder[2u * g + 1u]] = po.lo;
        }
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

  // ---- items
  const uint32_t quad = lane >> 2, sbo = quad >> 1, part = quad & 1u;
  const float4_t zero = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
  uint32_t slot = 0;
  for (uint32_t j = 0; j < my_items; ++j) {
    {
      const uint32_t fill = slot == 0 ? DEPTH - 1u : slot - 1u;
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      issue(fill, item_of(j + DEPTH - 1u));
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((DEPTH - 1) * kItemDma) : "memory");
    const uint32_t item = wave + j * kResWaves;
    const uint32_t st = item % stages;
    const uint32_t sb = st * 8u + sbo;
    const bool live = sb < sbs;
    const uint8_t* blk = ring + (wave * DEPTH + slot) * kItemBytes + ((lane & 3u) * 8u + sbo) * kQ4KBlockBytes;
    const uint8_t* xsb = xop + (live ? sb : 0u) * kXsb + (lane & (XC - 1u)) * 16u;
    const uint8_t* xs = xsb + (part * 16u) * (NC * XC * 16u);

    uint4 hq[5], xv[16 * NC], xm[NC];
    hq[0] = *reinterpret_cast<const uint4*>(blk);
#pragma unroll
    for (int i = 0; i < 4; ++i) hq[1 + i] = *reinterpret_cast<const uint4*>(blk + 16 + part * 64u + i * 16);
#pragma unroll
    for (int i = 0; i < 16 * NC; ++i) xv[i] = *reinterpret_cast<const uint4*>(xs + i * (XC * 16));
#pragma unroll
    for (int ch = 0; ch < NC; ++ch) xm[ch] = *reinterpret_cast<const uint4*>(xsb + (32 * NC + ch) * (XC * 16));
    asm volatile("" ::: "memory");

    const uint4 h = hq[0];
    const float d24 = live ? half_bits_to_float(h.x & 0xFFFFu) * 0x1p24f : 0.0f;
    const float dmin24 = live ? half_bits_to_float(h.x >> 16) * 0x1p24f : 0.0f;
    const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    const uint32_t scw = part == 0 ? sc_lo : sc_hi;
    float4_t tot[NC];
#pragma unroll
    for (int ch = 0; ch < NC; ++ch) tot[ch] = zero;
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      const uint4 qa = hq[1 + 2 * g], qb = hq[2 + 2 * g];
      const uint32_t qw[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
      float4_t acc_e[NC], acc_o[NC];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t v = qw[i], v8 = v >> 8;
        const half4_t be = bit_cast<half4_t>(uint2{v & 0x000F000Fu, v8 & 0x000F000Fu});
        const half4_t bo = bit_cast<half4_t>(uint2{v & 0x00F000F0u, v8 & 0x00F000F0u});
#pragma unroll
        for (int ch = 0; ch < NC; ++ch) {
          const uint4 x4 = xv[(g * 8 + i) * NC + ch];
          acc_e[ch] = __builtin_amdgcn_mfma_f32_4x4x4f16(bit_cast<half4_t>(uint2{x4.x, x4.y}), be,
                                                         i == 0 ? zero : acc_e[ch], 0, 0, 0);
          acc_o[ch] = __builtin_amdgcn_mfma_f32_4x4x4f16(bit_cast<half4_t>(uint2{x4.z, x4.w}), bo,
                                                         i == 0 ? zero : acc_o[ch], 0, 0, 0);
        }
      }
      const float se = d24 * static_cast<float>((scw >> (2 * g * 8)) & 0xFFu);
      const float so = d24 * static_cast<float>((scw >> ((2 * g + 1) * 8)) & 0xFFu);
#pragma unroll
      for (int ch = 0; ch < NC; ++ch) tot[ch] += se * acc_e[ch] + so * acc_o[ch];
    }
    {
      const half4_t b0 = bit_cast<half4_t>(uint2{mn_lo & 0x00FF00FFu, (mn_lo >> 8) & 0x00FF00FFu});
      const half4_t b1 = bit_cast<half4_t>(uint2{mn_hi & 0x00FF00FFu, (mn_hi >> 8) & 0x00FF00FFu});
#pragma unroll
      for (int ch = 0; ch < NC; ++ch) {
        const uint4 x4 = xm[ch];
        const half4_t am = bit_cast<half4_t>(part == 0 ? uint2{x4.x, x4.y} : uint2{x4.z, x4.w});
        const float4_t mm = __builtin_amdgcn_mfma_f32_4x4x4f16(am, part == 0 ? b0 : b1, zero, 0, 0, 0);
        tot[ch] -= dmin24 * mm;
      }
    }
    // Sum the sixteen quads (lane bits 2..5); lanes 0..3 then hold the item's four rows.
#pragma unroll
    for (int ch = 0; ch < NC; ++ch)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = tot[ch][e];
#pragma unroll
        for (int off = 4; off < 64; off <<= 1) v += __shfl_xor(v, off, kWave);
        tot[ch][e] = v;
      }
    if (lane < 4u) {
      float* dst = partial + (static_cast<size_t>(item) * 4u + lane) * kRows;
#pragma unroll
      for (int ch = 0; ch < NC; ++ch) {
        dst[ch * (XC / 2)] = (tot[ch][0] + tot[ch][1]) * inv_s[ch * (XC / 2)];
        if (XC == 4) dst[ch * 2 + 1] = (tot[ch][2] + tot[ch][3]) * inv_s[ch * 2 + 1];
      }
    }
    slot = slot + 1u == DEPTH ? 0u : slot + 1u;
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");   // no direct load may outlive its workgroup
  __syncthreads();
  for (uint32_t o = t; o < (q1 - q0) * 4u * m; o += 64u * kResWaves) {
    const uint32_t r = o / ((q1 - q0) * 4u), lr = o % ((q1 - q0) * 4u);   // activation row, local weight row
    const uint32_t ql = lr / 4u, rw = lr % 4u;
    float sum = 0.0f;
    for (uint32_t st = 0; st < stages; ++st) sum += partial[(static_cast<size_t>(ql * stages + st) * 4u + rw) * kRows + r];
    c[static_cast<size_t>(r) * n + (q0 + ql) * 4u + rw] = sum;
  }
}

struct MfmaPlan {
  uint32_t ks, kh, nc, xc;
};

MfmaPlan plan_for(uint32_t m, uint32_t n, uint32_t k) {
  MfmaPlan p{1, 2, 1, 4};
  if (m == 1) {
    p.xc = 2;
  } else {
    p.nc = (m + 1u) / 2u;
  }
  // More super-blocks of a row per stage (fewer rows per wavefront) until there are about two
  // wavefronts per CU; with many activation columns the operand a wavefront re-reads per stage
  // outweighs its weights, so the tiles stay larger.
  const uint32_t sbs = k / 256u, want = 2u * static_cast<uint32_t>(num_cus());
  const uint32_t ks_max = p.nc > 2 ? 2u : 4u;
  while (p.ks < ks_max && sbs % (2u * p.ks) == 0 && (n * p.ks * p.kh + 63u) / 64u < want) p.ks *= 2u;
  return p;
}

template <int KS, int KH, int NC, int XC, int DEPTH>
void launch_cfg(const uint8_t* w, const uint8_t* xop, const float* inv, float* c, uint32_t m, uint32_t n,
                uint32_t k, hipStream_t stream) {
  const uint32_t rows = 64 / (KS * KH);
  hipLaunchKernelGGL((q4k_gemv_mfma_kernel<KS, KH, NC, XC, DEPTH>), dim3((n + rows - 1) / rows), dim3(64), 0,
                     stream, w, xop, inv, c, m, n, k);
}

}  // namespace

namespace {

template <int NC, int XC, int DEPTH, int S>
hipError_t launch_resident(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                           uint32_t quads_per_wg, uint32_t grid, size_t lds_bytes, hipStream_t stream) {
  static bool raised = false;     // the default dynamic-LDS ceiling is 64 KB; raise it once per kernel
  if (!raised) {
    const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&q4k_rows_resident_kernel<NC, XC, DEPTH, S>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return e;
    raised = true;
  }
  hipLaunchKernelGGL((q4k_rows_resident_kernel<NC, XC, DEPTH, S>), dim3(grid), dim3(64 * kResWaves), lds_bytes, stream,
                     a, w, c, m, n, k, quads_per_wg);
  return hipGetLastError();
}

// LDS the resident kernel needs with `depth` ring stages; 0 if the shape is outside its range.
size_t resident_lds_bytes(uint32_t m, uint32_t n, uint32_t k, uint32_t depth, uint32_t* quads_per_wg, uint32_t* grid) {
  if (m < 1 || m > 4 || n % 4u != 0 || k % 256u != 0 || k / 8u > 5u * 64u * kResWaves) return 0;
  const uint32_t quads = n / 4u, cus = static_cast<uint32_t>(num_cus());
  const uint32_t g = quads < cus ? quads : cus;
  const uint32_t per = (quads + g - 1u) / g;
  *quads_per_wg = per;
  *grid = (quads + per - 1u) / per;
  const uint32_t sbs = k / 256u, stages = (sbs + 7u) / 8u;
  const uint32_t xc = m == 1 ? 2u : 4u, nc = m > 2 ? 2u : 1u, rows = nc * xc / 2u;
  return static_cast<size_t>(kResWaves) * depth * kItemBytes + static_cast<size_t>(sbs) * kSlots * nc * xc * 16u +
         static_cast<size_t>(per) * stages * 4u * rows * 4u + (rows + rows * kResWaves) * 4u;
}

}  // namespace

bool gemv_q4k_mfma_supported(uint64_t m, uint64_t n, uint64_t k) {
  return m >= 1 && m <= 8 && n >= 1 && k % 256 == 0 && k >= 256 && n * (k / 256) * 144 < (1ull << 32);
}

size_t gemv_q4k_mfma_workspace_bytes(uint64_t m, uint64_t k) {
  const uint64_t chains = m == 1 ? 1 : (m + 1) / 2, xc = m == 1 ? 2 : 4;
  return static_cast<size_t>((k / 256) * kSlots * chains * xc * 16 + 256);
}

hipError_t launch_q4k_gemv_mfma(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m,
                                uint32_t n, uint32_t k, hipStream_t stream) {
  {
    uint32_t per = 0, grid = 0;
    constexpr size_t kLdsMax = 160 * 1024;
    for (uint32_t depth = 3; depth >= 2; --depth) {
      const size_t need = resident_lds_bytes(m, n, k, depth, &per, &grid);
      if (need == 0 || need > kLdsMax) continue;
      const bool small = k / 8u <= 2u * 64u * kResWaves;       // activation slots per thread: 2 or 5
#define QMM_RES_CASE(NC_, XC_, D_, S_) launch_resident<NC_, XC_, D_, S_>(a, w, c, m, n, k, per, grid, need, stream)
      if (m == 1) {
        return depth == 3 ? (small ? QMM_RES_CASE(1, 2, 3, 2) : QMM_RES_CASE(1, 2, 3, 5))
                          : (small ? QMM_RES_CASE(1, 2, 2, 2) : QMM_RES_CASE(1, 2, 2, 5));
      }
      if (m == 2) {
        return depth == 3 ? (small ? QMM_RES_CASE(1, 4, 3, 2) : QMM_RES_CASE(1, 4, 3, 5))
                          : (small ? QMM_RES_CASE(1, 4, 2, 2) : QMM_RES_CASE(1, 4, 2, 5));
      }
      if (small) return depth == 3 ? QMM_RES_CASE(2, 4, 3, 2) : QMM_RES_CASE(2, 4, 2, 2);
      break;
#undef QMM_RES_CASE
    }
  }
  const MfmaPlan p = plan_for(m, n, k);
  float* inv = static_cast<float*>(workspace);
  uint8_t* xop = static_cast<uint8_t*>(workspace) + 256;
  const uint32_t prep_rows = p.nc * (p.xc / 2u);
  const dim3 prep_grid(prep_rows, (k / 256u * 32u + 255u) / 256u);
  if (p.xc == 2) {
    hipLaunchKernelGGL(q4k_rows_prep_kernel<2>, prep_grid, dim3(256), 0, stream, a,
                       reinterpret_cast<_Float16*>(xop), inv, m, k, p.nc);
  } else {
    hipLaunchKernelGGL(q4k_rows_prep_kernel<4>, prep_grid, dim3(256), 0, stream, a,
                       reinterpret_cast<_Float16*>(xop), inv, m, k, p.nc);
  }
#define QMM_MFMA_CASE(KS_, KH_, NC_, XC_, DEPTH_)                                        \
  if (p.ks == KS_ && p.kh == KH_ && p.nc == NC_ && p.xc == XC_) {                        \
    launch_cfg<KS_, KH_, NC_, XC_, DEPTH_>(w, xop, inv, c, m, n, k, stream);             \
    return hipGetLastError();                                                            \
  }
  QMM_MFMA_CASE(1, 2, 1, 2, 4) QMM_MFMA_CASE(2, 2, 1, 2, 4) QMM_MFMA_CASE(4, 2, 1, 2, 4)
  QMM_MFMA_CASE(1, 2, 1, 4, 4) QMM_MFMA_CASE(2, 2, 1, 4, 4) QMM_MFMA_CASE(4, 2, 1, 4, 3)
  QMM_MFMA_CASE(1, 2, 2, 4, 4) QMM_MFMA_CASE(2, 2, 2, 4, 3) QMM_MFMA_CASE(4, 2, 2, 4, 2)
  QMM_MFMA_CASE(1, 2, 3, 4, 4) QMM_MFMA_CASE(2, 2, 3, 4, 3)
  QMM_MFMA_CASE(1, 2, 4, 4, 4) QMM_MFMA_CASE(2, 2, 4, 4, 2)
#undef QMM_MFMA_CASE
  return hipErrorInvalidValue;
}

}  // namespace qmm
