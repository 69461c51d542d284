// Q4_K x up to 16 fp32 activation rows in ONE pass over the weights, on v_mfma_f32_16x16x32_f16,
// exact on the weight side.
//
//   C[r][n] = sum_k A[r][k] * deq(W)[n][k],   W = n rows of k/256 Q4_K super-blocks
//   (layout and decode: src/core/numerics/quant.cpp:58-70,656-675; GemmQ4KRef gemm.cpp:18-41).
//   The reference has no kernel that reads W once for 5..15 rows
//   (src/models/qwen3_5/project.cpp:294-306 falls to one GEMV pass per row).
//
// Operands of one instruction (K = 32 = one Q4_K sub-block):
//  * B = 16 weight rows.  Lane l supplies row l % 16, elements 8 * (l / 16) + [0, 8) of the
//    sub-block: eight nibbles of two dwords, masked in place two to a register and multiplied by
//    the sub-block's 6-bit scale with one 24-bit integer multiply.  An integer n < 2048 in a 16-bit
//    half is the fp16 value n * 2^-24 (subnormal below 1024, first binade above; the matrix core
//    honours both), so the operand is q * sc * 2^-24 exactly and the eight sub-blocks of a
//    super-block add up in the accumulator (2^24 is folded into d).  The four results a lane gets
//    back belong to its own weight row.
//  * A = 8 activation rows as 16 matrix rows: row r is hi = f16(x s) and lo = f16(x s - hi), s
//    the power of two that brings the largest magnitude of the row's 256-wide block to
//    [256, 512): 22 significant bits under the block's largest value, exact rescaling.  Products
//    of a 10-bit integer and an 11-bit value are exact in the fp32 accumulator.
//  * the min term is one more instruction per super-block: the mins (<= 63, integers in halves
//    again) against the sub-block sums Sx of what the matrix core sees, as fp16 hi and lo.
//  * per super-block: result += (d * (D_hi + D_lo) - dmin * Dmin) / s: for a one-hot row every
//    step is exact and the output is the reference's dequantized weight bit for bit.
//
// Work split.  A wavefront owns BW super-block columns of its workgroup's K part and keeps their
// activation operands in registers for the whole kernel (converted once in the prologue through a
// private LDS area); it walks all 16-row tiles of the workgroup's rows.  Each (tile, block) unit of
// 16 x 144 bytes comes by coalesced 16-byte loads straight into a private ring of LDS slots (no
// register in between), up to four units ahead, and is read back in matrix-core order.  No
// activation is read inside the loop and no wavefront waits for another while tiles remain: the
// wavefronts' partial tiles meet in an LDS table once (as many tiles as the table holds) and are
// added in wavefront order.  K parts (gridDim.y) write their sums to separate regions of a scratch
// buffer that a reduce launch adds in part order.  (A workgroup that arrives last adding the
// regions inside this kernel was measured four times slower: the device-scope release and acquire
// it needs write back and invalidate the L2 of its XCD under the workgroups still streaming
// weights.)  Stamps of the 100 MHz counter inside the kernel show what bounds it: a wavefront
// that has a SIMD's issue slots to itself needs 0.5 us a unit and never waits for weights; ten
// wavefronts on four SIMDs put three on two of them, and those finish last -- hence K parts of
// twelve and eight columns where the column count allows (r16_plan_unequal).

#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

constexpr uint32_t kTile = 16;            // weight rows per tile (the N of the instruction)
constexpr uint32_t kUnitBytes = kTile * 144u;
constexpr int kKL = 3;                    // 16-byte pieces a lane brings per unit: ceil(16 * 9 / 64)
constexpr uint32_t kARowBytes = 256u * 2u + 16u;   // one matrix row of a block in the conversion area
constexpr uint32_t kConvRows = 8;         // matrix rows converted at a time (four activation rows, hi and lo)

// A K part of unequal size (see r16_plan): the workgroups first_wg .. of the launch own its block
// columns b0 .. b0 + nbp - 1, one a wavefront, tiles_per_wg tiles each.
struct R16Part {
  uint32_t first_wg, tiles_per_wg, b0, nbp, tiles_per_sync;
};
constexpr uint32_t kMaxParts = 8;

struct R16Args {
  const float* a;          // m x k
  const uint8_t* w;        // n rows of k/256 blocks
  float* c;                // m x n, the result
  float* ws;               // [parts][m][n] partial sums of the K parts (unused with one part)
  uint32_t m, n, k;
  uint32_t tiles_per_wg;
  uint32_t blocks_per_part;
  uint32_t tiles_per_sync;   // tiles between two meetings of the wavefronts' partial sums
  uint32_t n_parts;          // 0: equal parts, gridDim.y of them; else the table below, gridDim.y = 1
  R16Part part[kMaxParts];
};

// 16 bytes from base + voff straight into LDS at lds_addr + 16 * lane (no register in between).
__device__ __forceinline__ void r16_dma16(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}

template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t dpp_umax16(uint32_t v) {
  const uint32_t moved = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), kCtrl, kRowMask, 0xF, false));
  return v > moved ? v : moved;
}
// Largest value over the 64 lanes of each of eight registers, DPP only; uniform results.
__device__ __forceinline__ void wave_umax16_x8(uint32_t (&v)[8]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = dpp_umax16<0xB1, 0xF>(v[i]);    // quad_perm [1,0,3,2]
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = dpp_umax16<0x4E, 0xF>(v[i]);    // quad_perm [2,3,0,1]
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = dpp_umax16<0x141, 0xF>(v[i]);   // row_half_mirror
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = dpp_umax16<0x140, 0xF>(v[i]);   // row_mirror
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = dpp_umax16<0x142, 0xA>(v[i]);   // row_bcast:15
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = dpp_umax16<0x143, 0xC>(v[i]);   // row_bcast:31
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v[i]), 63));
}
template <int kCtrl>
__device__ __forceinline__ float dpp_fadd16(float v) {
  return v + bit_cast<float>(__builtin_amdgcn_update_dpp(0, bit_cast<int>(v), kCtrl, 0xF, 0xF, false));
}

// LDS layout: [unit rings: W x RING][Sx: W x BW x MT x 8 x 8][1/s: W x BW x MT x 8][the conversion
// areas (W x kConvRows rows) during the prologue, then the partials (tiles per sync x W x (8 MT) x 16)]
__host__ __device__ inline uint32_t r16_shared_area_bytes(uint32_t waves, uint32_t mt, uint32_t tiles_per_sync) {
  const uint32_t conv = waves * kConvRows * kARowBytes, part = tiles_per_sync * waves * 8u * mt * 16u * 4u;
  return conv > part ? conv : part;
}
__host__ __device__ inline uint32_t r16_fixed_lds_bytes(uint32_t waves, uint32_t mt, uint32_t bw, uint32_t ring) {
  return waves * ring * kUnitBytes + waves * bw * mt * (64u + 8u) * 4u;
}
__host__ __device__ inline uint32_t r16_lds_bytes(uint32_t waves, uint32_t mt, uint32_t bw, uint32_t ring, uint32_t tiles_per_sync) {
  return r16_fixed_lds_bytes(waves, mt, bw, ring) + r16_shared_area_bytes(waves, mt, tiles_per_sync);
}

// MT = 16-row matrix tiles of activations (8 activation rows each), BW = block columns a wavefront
// owns, RING = weight units a wavefront keeps in flight.
template <int MT, int BW, int RING>
__global__ __launch_bounds__(768) void q4k_rows16_kernel(R16Args p) {
  static_assert(MT * BW <= 2, "the activation operands of a wavefront take 32 registers per tile and column");
  static_assert((RING - 1) * kKL <= 63, "vmcnt is a 6-bit counter");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t waves = blockDim.x >> 6;
  const uint32_t nrow = lane & 15u, gq = lane >> 4;        // weight row of the tile, K chunk of a sub-block
  uint32_t nbp = p.blocks_per_part, b0 = blockIdx.y * nbp;   // block columns of this K part
  uint32_t tiles_per_wg = p.tiles_per_wg, tiles_per_sync = p.tiles_per_sync, wg = blockIdx.x;
  uint32_t part_index = blockIdx.y, n_parts = gridDim.y;
  if (p.n_parts != 0u) {
    part_index = 0;
    for (uint32_t i = 1; i < p.n_parts; ++i) part_index = blockIdx.x >= p.part[i].first_wg ? i : part_index;
    const R16Part& pt = p.part[part_index];
    nbp = pt.nbp, b0 = pt.b0, tiles_per_wg = pt.tiles_per_wg, tiles_per_sync = pt.tiles_per_sync;
    wg = blockIdx.x - pt.first_wg, n_parts = p.n_parts;
  }
  // wavefronts of the launch that this part has no column for leave before the first barrier
  // (a barrier waits for the surviving wavefronts only)
  const uint32_t live_waves = (nbp + BW - 1u) / BW;
  if (wave >= live_waves) return;
  const uint32_t sbs = p.k / 256u, row_bytes = sbs * 144u;
  const uint32_t tiles_total = (p.n + kTile - 1u) / kTile;
  const uint32_t tile0 = wg * tiles_per_wg;
  if (tile0 >= tiles_total) return;                        // whole workgroup leaves together
  const uint32_t tiles = tile0 + tiles_per_wg <= tiles_total ? tiles_per_wg : tiles_total - tile0;
  const uint32_t row0 = tile0 * kTile;

  uint8_t* ring = lds + wave * (RING * kUnitBytes);
  const uint32_t ring_addr = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)ring));
  float* sx_all = reinterpret_cast<float*>(lds + waves * (RING * kUnitBytes));
  float* sx = sx_all + wave * (BW * MT * 64u);                               // [BW][MT][8 sub-blocks][8 rows]
  float* inv_all = sx_all + waves * (BW * MT * 64u);
  float* invs = inv_all + wave * (BW * MT * 8u);                             // [BW][MT][8 rows]
  float* part = inv_all + waves * (BW * MT * 8u);                            // [tiles per sync][W][8 MT][16]
  uint8_t* conv = reinterpret_cast<uint8_t*>(part) + wave * kConvRows * kARowBytes;   // prologue only, same memory as `part`

  // Block columns of this wavefront inside the part: wave, wave + W (BW = 2); one past the part
  // is computed with zero activations on the part's last block.
  auto col_live = [&](uint32_t jb) { return wave + jb * live_waves < nbp; };
  auto col = [&](uint32_t jb) { return b0 + (col_live(jb) ? wave + jb * live_waves : nbp - 1u); };

  // ---- the activations are requested first: a wavefront's loads return in order, so behind the
  // weight ring they would wait for it.  Requested by hand, because the compiler's own waits count
  // only the loads it knows of and would wait for the ring as well.  Between the request and the
  // wait below nothing names xv, and the kernel must not spill (a copy of a register that its load
  // has not filled yet would go unnoticed): tests/test_kernel_resources.py compiles this file and
  // fails on any scratch use.
  float4_t xv[BW * MT][8];
#pragma unroll
  for (int jb = 0; jb < BW; ++jb)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r8 = 0; r8 < 8; ++r8) {
        const uint32_t r = mt * 8u + r8;
        const float* src = p.a + static_cast<size_t>(r < p.m ? r : 0u) * p.k + col(jb) * 256u + lane * 4u;
        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(xv[jb * MT + mt][r8]) : "v"(src) : "memory");
      }

  // ---- weight units: piece pc = i * 64 + lane of a unit is 16 bytes pc % 9 of row pc / 9, brought
  // straight into the ring slot (the third instruction by sixteen lanes only)
  uint32_t piece_row[kKL], piece_off[kKL];
#pragma unroll
  for (int i = 0; i < kKL; ++i) {
    uint32_t pc = i * 64u + lane;
    pc = pc < kTile * 9u ? pc : kTile * 9u - 1u;
    piece_row[i] = pc / 9u;
    piece_off[i] = (pc - piece_row[i] * 9u) * 16u;
  }
  const uint32_t n_units = tiles * BW;
  // Every wavefront has asked for its activations before any asks for weights: the requests of a
  // CU are served in the order made, and the last wavefront's activations behind the others'
  // weight units would hold the whole workgroup at the end of the prologue.
  __builtin_amdgcn_s_barrier();
  uint32_t issued = 0, fill_slot = 0;
  auto next_unit = [&]() {
    // unit u = (tile u / BW, column u % BW); past the last one the last is read again (the loads
    // stay unconditional so that outstanding loads are counted exactly; the bytes come from L2,
    // and the slot they land in has been consumed)
    const uint32_t u = issued < n_units ? issued : n_units - 1u;
    const uint32_t tl = u / BW, jb = u % BW;
    const uint32_t first_row = row0 + tl * kTile;
    const uint32_t last = p.n - 1u - first_row;             // rows past the matrix: the last row, never stored
    const uint8_t* base = p.w + static_cast<size_t>(col(jb)) * 144u + static_cast<size_t>(first_row) * row_bytes;
    const uint32_t dst = ring_addr + fill_slot * kUnitBytes;
#pragma unroll
    for (int i = 0; i < kKL; ++i) {
      const uint32_t off = (piece_row[i] < last ? piece_row[i] : last) * row_bytes + piece_off[i];
      if (i + 1 < kKL) {
        r16_dma16(base, off, dst + i * 1024u);
      } else if (lane < kTile * 9u - 128u) {
        r16_dma16(base, off, dst + i * 1024u);
      }
    }
    ++issued;
    fill_slot = fill_slot + 1u == RING ? 0u : fill_slot + 1u;
  };
#pragma unroll
  for (int i = 0; i < RING; ++i) next_unit();
  // the activations have arrived when only the ring is outstanding
  asm volatile("s_waitcnt vmcnt(%0)" :: "n"(RING * kKL) : "memory");
#pragma unroll
  for (int q = 0; q < BW * MT; ++q)
#pragma unroll
    for (int r8 = 0; r8 < 8; ++r8) asm volatile("" : "+v"(xv[q][r8]));

  // ---- activations of this wavefront's block columns -> matrix-core operands in registers
  half8_t afrag[BW][MT][8];
#pragma unroll
  for (int jb = 0; jb < BW; ++jb) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      // largest magnitude of each row's block as bits (integer order = magnitude order; NaN and
      // infinity sort above every finite value, so the same reduction finds them); the eight
      // reductions go step by step side by side, so that no step waits for its predecessor
      uint32_t mx[8];
#pragma unroll
      for (int r8 = 0; r8 < 8; ++r8) {
        const float4_t v = xv[jb * MT + mt][r8];
        const uint32_t m0 = bit_cast<uint32_t>(v[0]) & 0x7FFFFFFFu, m1 = bit_cast<uint32_t>(v[1]) & 0x7FFFFFFFu;
        const uint32_t m2 = bit_cast<uint32_t>(v[2]) & 0x7FFFFFFFu, m3 = bit_cast<uint32_t>(v[3]) & 0x7FFFFFFFu;
        mx[r8] = max(max(m0, m1), max(m2, m3));
      }
      wave_umax16_x8(mx);
#pragma unroll
      for (int r8 = 0; r8 < 8; ++r8) {
        const uint32_t r = mt * 8u + r8;
        const uint32_t cr = 2u * (r8 & 3);      // matrix rows 2 r8 and 2 r8 + 1, four activation rows at a time
        typedef _Float16 half4v __attribute__((ext_vector_type(4)));
        typedef _Float16 half2v __attribute__((ext_vector_type(2)));
        typedef float float2v __attribute__((ext_vector_type(2)));
        if (r >= p.m || !col_live(jb)) {
          // a row the call does not have (the same for the whole wavefront): zero operands
          const half4v z = {0, 0, 0, 0};
          *reinterpret_cast<half4v*>(conv + cr * kARowBytes + lane * 8u) = z;
          *reinterpret_cast<half4v*>(conv + (cr + 1u) * kARowBytes + lane * 8u) = z;
          if ((lane & 7u) == 0u) sx[((jb * MT + mt) * 8u + (lane >> 3)) * 8u + r8] = 0.0f;
          if (lane == 0u) invs[(jb * MT + mt) * 8u + r8] = 1.0f;
        } else {
          const float4_t v = xv[jb * MT + mt][r8];
          const uint32_t e = mx[r8] >> 23;
          int se = 262 - static_cast<int>(e);                       // amax * s in [2^8, 2^9)
          se = se < 1 ? 1 : (se > 254 ? 254 : se);
          const float s = (e == 0u || e == 0xFFu) ? 1.0f : bit_cast<float>(static_cast<uint32_t>(se) << 23);
          // NaN or infinity anywhere in the block: the block's factor becomes NaN, as the reference's sum would
          const float inv = e == 0xFFu ? bit_cast<float>(0x7FC00000u)
                                       : (e == 0u ? 1.0f : bit_cast<float>(static_cast<uint32_t>(254 - se) << 23));
          // the nibble masks deliver a chunk's elements in the order 0, 2, 1, 3 | 4, 6, 5, 7
          float2v xa = {v[0] * s, v[2] * s}, xb = {v[1] * s, v[3] * s};
          if (e == 0xFFu) xa = xb = float2v{0.0f, 0.0f};
          const half2v ha = __builtin_convertvector(xa, half2v), hb = __builtin_convertvector(xb, half2v);
          const half2v la = __builtin_convertvector(xa - __builtin_convertvector(ha, float2v), half2v);
          const half2v lb = __builtin_convertvector(xb - __builtin_convertvector(hb, float2v), half2v);
          *reinterpret_cast<half4v*>(conv + cr * kARowBytes + lane * 8u) = half4v{ha[0], ha[1], hb[0], hb[1]};
          *reinterpret_cast<half4v*>(conv + (cr + 1u) * kARowBytes + lane * 8u) = half4v{la[0], la[1], lb[0], lb[1]};
          // sub-block sums (eight consecutive lanes) of the scaled values: what the matrix core
          // sees is these to 22 bits, and exactly these for a row of powers of two
          float seen = (xa[0] + xa[1]) + (xb[0] + xb[1]);
          seen = dpp_fadd16<0xB1>(seen);     // quad_perm [1,0,3,2]
          seen = dpp_fadd16<0x4E>(seen);     // quad_perm [2,3,0,1]
          seen = dpp_fadd16<0x141>(seen);    // row_half_mirror
          if ((lane & 7u) == 0u) sx[((jb * MT + mt) * 8u + (lane >> 3)) * 8u + r8] = seen;
          if (lane == 0u) invs[(jb * MT + mt) * 8u + r8] = inv;
        }
        if ((r8 & 3) == 3) {
          // matrix row i = 2 r8 + {hi, lo} is lane % 16; K chunk gq of sub-block sb.  The lanes
          // of the eight rows just converted pick theirs up before the area is written again.
          if ((nrow >> 3) == static_cast<uint32_t>(r8 >> 2)) {
#pragma unroll
            for (int sb = 0; sb < 8; ++sb) {
              afrag[jb][mt][sb] = *reinterpret_cast<const half8_t*>(conv + (nrow & 7u) * kARowBytes + (sb * 32u + gq * 8u) * 2u);
            }
          }
        }
      }
    }
  }
  lds_barrier();     // every wavefront is done with its conversion area: the partials take that memory over

  // Operand of the min term: matrix row 2 r (lanes with an even nrow) holds the sub-block sums of
  // activation row r as fp16 hi (K elements 0..7, lanes gq = 0) and lo (8..15, gq = 1), in the
  // order the mins are unpacked in; every other element is zero.
  half8_t amin[BW][MT];
#pragma unroll
  for (int jb = 0; jb < BW; ++jb)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (gq < 2u && (nrow & 1u) == 0u) {
        const float* s = sx + ((jb * MT + mt) * 8u) * 8u + (nrow >> 1);
        constexpr int kOrder[8] = {0, 2, 1, 3, 4, 6, 5, 7};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float sum = s[kOrder[j] * 8];
          const _Float16 hi = static_cast<_Float16>(sum);
          v[j] = gq == 0u ? hi : static_cast<_Float16>(sum - static_cast<float>(hi));
        }
      }
      amin[jb][mt] = v;
    }

  // a lane's results: weight row nrow, matrix rows 4 gq + e, i.e. activation rows 2 gq + {0, 1} of each MT
  float tileacc[MT][2];
  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  uint32_t read_slot = 0;
  auto consume = [&](int jb) {
    const uint8_t* blk = ring + read_slot * kUnitBytes + nrow * 144u;
    const uint4 h = *reinterpret_cast<const uint4*>(blk);
    uint2 wq[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) wq[g] = *reinterpret_cast<const uint2*>(blk + 16 + g * 32 + gq * 8);
    const float d24 = half_bits_to_float(h.x & 0xFFFFu) * 0x1p24f;
    const float dmin24 = half_bits_to_float(h.x >> 16) * 0x1p24f;
    const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    // An integer n < 2048 in a 16-bit half is the fp16 value n * 2^-24, so nibble * scale (<= 945)
    // is one 24-bit multiply for two weights and the matrix core adds a super-block's sub-blocks
    // up by itself; the mins (<= 63) go the same way against the sub-block sums.
    float4_t acc[MT], mres[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[mt] = zero4;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint32_t x = wq[g].x, y = wq[g].y;
      constexpr uint32_t kM = 0x000F000Fu;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int sb = 2 * g + half;
        const uint32_t sc = ((sb < 4 ? sc_lo : sc_hi) >> (8 * (sb & 3))) & 0xFFu;
        const int4v_t b = {static_cast<int>(__umul24((x >> (4 * half)) & kM, sc)), static_cast<int>(__umul24((x >> (8 + 4 * half)) & kM, sc)),
                           static_cast<int>(__umul24((y >> (4 * half)) & kM, sc)), static_cast<int>(__umul24((y >> (8 + 4 * half)) & kM, sc))};
        const half8_t bop = bit_cast<half8_t>(b);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[jb][mt][sb], bop, acc[mt], 0, 0, 0);
      }
    }
    {
      constexpr uint32_t kB = 0x00FF00FFu;
      const int4v_t b = {static_cast<int>(mn_lo & kB), static_cast<int>((mn_lo >> 8) & kB), static_cast<int>(mn_hi & kB),
                         static_cast<int>((mn_hi >> 8) & kB)};
      const half8_t bop = bit_cast<half8_t>(b);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) mres[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(amin[jb][mt], bop, zero4, 0, 0, 0);
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float f = acc[mt][2 * j] + acc[mt][2 * j + 1];
        const float v = fmaf(d24, f, -(dmin24 * mres[mt][2 * j]));
        tileacc[mt][j] = fmaf(v, invs[(jb * MT + mt) * 8u + 2u * gq + j], tileacc[mt][j]);
      }
  };

  // ---- tiles.  Every wavefront walks the same tiles, so the barriers match.
  const size_t region = static_cast<size_t>(p.m) * p.n;
  float* cpart = n_parts == 1u ? p.c : p.ws + part_index * region;
  // One tile: its BW units, then the wavefront's partial tile into LDS.  A unit is waited for when
  // RING - 1 later ones are all that may still be under way (stores of the sums count as well and
  // only make the wait longer); its slot is asked for again as soon as its words are in registers.
  auto do_tile = [&](uint32_t ti) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) tileacc[mt][0] = tileacc[mt][1] = 0.0f;
#pragma unroll
    for (int jb = 0; jb < BW; ++jb) {
      asm volatile("s_waitcnt vmcnt(%0)" :: "n"((RING - 1) * kKL) : "memory");
      consume(jb);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      next_unit();
      read_slot = read_slot + 1u == RING ? 0u : read_slot + 1u;
    }
    float* dst = part + ((ti * live_waves + wave) * (8u * MT)) * 16u;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j) dst[(mt * 8u + 2u * gq + j) * 16u + nrow] = tileacc[mt][j];
  };
  // The wavefronts run through a group of tiles on their own (no wavefront waits for another
  // while its ring is being refilled) and meet once a group: normally once a workgroup.
  for (uint32_t g0 = 0; g0 < tiles; g0 += tiles_per_sync) {
    const uint32_t in_group = tiles - g0 < tiles_per_sync ? tiles - g0 : tiles_per_sync;
    for (uint32_t ti = 0; ti < in_group; ++ti) do_tile(ti);
    lds_barrier();
    // sum the wavefronts' partial tiles per output in wavefront order and store
    for (uint32_t o = t; o < in_group * 8u * MT * 16u; o += live_waves * 64u) {
      const uint32_t nn = o & 15u, r = (o >> 4) % (8u * MT), ti = o / (128u * MT);
      const uint32_t row = row0 + (g0 + ti) * kTile + nn;
      if (r >= p.m || row >= p.n) continue;
      float sum = 0.0f;
      for (uint32_t wv = 0; wv < live_waves; ++wv) sum += part[((ti * live_waves + wv) * (8u * MT) + r) * 16u + nn];
      cpart[static_cast<size_t>(r) * p.n + row] = sum;
    }
    if (g0 + tiles_per_sync < tiles) lds_barrier();      // the table is written again
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive its workgroup
}

struct R16Plan {
  uint32_t parts, waves, bw, mt, tiles_per_wg, row_groups, ring, tiles_per_sync;
  uint32_t n_table;              // unequal parts: entries of `table`, row_groups = all workgroups
  R16Part table[kMaxParts];
};

constexpr uint32_t kR16Lds = 160u * 1024u - 64u;

// Tiles between two meetings: as many as the LDS beside the rings holds, in equal groups.
uint32_t r16_sync_tiles(uint32_t layout_waves, uint32_t live_waves, uint32_t mt, uint32_t bw, uint32_t ring, uint32_t per) {
  const uint32_t tile_bytes = live_waves * 8u * mt * 16u * 4u;
  uint32_t tps = (kR16Lds - r16_fixed_lds_bytes(layout_waves, mt, bw, ring)) / tile_bytes;
  tps = tps > per ? per : tps;
  const uint32_t syncs = (per + tps - 1u) / tps;
  return (per + syncs - 1u) / syncs;
}

// Unequal K parts of twelve and eight block columns.  The launch lasts as long as the SIMD with the
// most wavefronts works, and a wavefront's time goes to its instructions, not to waiting for
// weights: ten columns a workgroup put three wavefronts on two SIMDs and two on the others.  Parts
// of 12 and 8 columns fill the four SIMDs evenly (3 and 2 wavefronts each); a workgroup of an
// 8-column part takes one and a half times the tiles, and the CUs are shared out accordingly
// (`prologue` = the conversion of a wavefront's activations in units of one tile's work).  Measured
// 17408 x 5120: 8 rows 20.0 -> 18.9 us, 5120 x 17408: 8 rows 23.6 -> 21.2, 16 rows 31.9 -> 27.9 us.
bool r16_plan_unequal(uint32_t nb, uint32_t mt, uint32_t tiles_total, uint32_t cus, R16Plan& pl) {
  if (nb % 4u != 0u || nb < 20u) return false;
  uint32_t twelves = nb / 12u;
  while ((nb - twelves * 12u) % 8u != 0u) --twelves;     // nb = 12 a + 8 b; a >= 1 for nb >= 20, nb % 4 == 0
  const uint32_t eights = (nb - twelves * 12u) / 8u;
  if (twelves == 0u || eights == 0u || twelves + eights > kMaxParts) return false;
  const uint32_t prologue = 2;   // measured: 1..3 alike, 5 and more slower, for 8 and for 16 rows
  uint32_t t12 = 0, t8 = 0;
  for (uint32_t t = tiles_total / cus > 1u ? tiles_total / cus : 1u; t <= tiles_total; ++t) {   // a part alone needs tiles / t <= CUs
    const uint32_t u = (3u * (prologue + t)) / 2u - prologue;
    const uint32_t g12 = (tiles_total + t - 1u) / t, g8 = (tiles_total + u - 1u) / u;
    if (twelves * g12 + eights * g8 <= cus) {
      t12 = t, t8 = u;
      break;
    }
  }
  if (t12 == 0u) return false;
  const uint32_t waves = 12, bw = 1;
  uint32_t ring = 4;
  while (ring > 2u && r16_lds_bytes(waves, mt, bw, ring, 1) > kR16Lds) --ring;
  if (r16_lds_bytes(waves, mt, bw, ring, 1) > kR16Lds) return false;
  pl = R16Plan{};
  pl.parts = twelves + eights, pl.waves = waves, pl.bw = bw, pl.mt = mt, pl.ring = ring, pl.n_table = twelves + eights;
  // partial tiles (one wavefront's share of a tile) the LDS table holds, a whole number of
  // twelve-wavefront tiles: the launch sizes the table as tiles x 12 wavefronts
  const uint32_t table_units = (kR16Lds - r16_fixed_lds_bytes(waves, mt, bw, ring)) / (8u * mt * 16u * 4u) / waves * waves;
  uint32_t wg = 0, b0 = 0, max_sync = 1;
  for (uint32_t i = 0; i < pl.n_table; ++i) {
    const uint32_t cols = i < twelves ? 12u : 8u, per = i < twelves ? t12 : t8;
    uint32_t tps = table_units / cols;
    tps = tps > per ? per : tps;
    const uint32_t syncs = (per + tps - 1u) / tps;
    tps = (per + syncs - 1u) / syncs;
    pl.table[i] = R16Part{wg, per, b0, cols, tps};
    max_sync = tps * cols > max_sync ? tps * cols : max_sync;
    wg += (tiles_total + per - 1u) / per;
    b0 += cols;
  }
  pl.row_groups = wg;
  pl.tiles_per_wg = t12;
  pl.tiles_per_sync = (max_sync + waves - 1u) / waves;   // sizes the LDS table: tiles x wavefronts of the largest entry
  return true;
}

// K parts: the fewest (a divisor of the block count) whose block columns fit the twelve wavefronts
// of a workgroup, one column each, or two when 8 rows or fewer leave the registers for it --
// preferring one column each when that costs only twice the parts; then the rows are cut into
// equal runs of tiles, a workgroup per CU and part.
bool r16_plan(uint64_t m, uint64_t n, uint64_t k, R16Plan& pl) {
  if (m < 2 || m > 16 || k % 256 != 0 || n == 0 || n > 0x7FFFFFFFull || k > (1ull << 24)) return false;
  const uint32_t nb = static_cast<uint32_t>(k / 256), mt = m > 8 ? 2u : 1u, bw_max = mt == 1 ? 2u : 1u;
  const uint32_t tiles_total = static_cast<uint32_t>((n + kTile - 1) / kTile);
  const uint32_t cus = static_cast<uint32_t>(num_cus());
  if (r16_plan_unequal(nb, mt, tiles_total, cus, pl)) return true;
  for (uint32_t parts = 1; parts <= nb; ++parts) {
    if (nb % parts != 0) continue;
    const uint32_t nbp = nb / parts;
    uint32_t bw = 1;
    if (nbp > 12u) {
      bw = 2;
      if (bw > bw_max || nbp > 24u) continue;
      if (nb % (parts * 2u) == 0 && nb / (parts * 2u) <= 12u && nb / (parts * 2u) >= 6u) continue;
    }
    const uint32_t waves = (nbp + bw - 1u) / bw;
    if (waves < 4u && parts < nb) continue;              // too few wavefronts to hide the load latency
    uint32_t groups = cus / parts;
    if (groups == 0) groups = 1;
    if (groups > tiles_total) groups = tiles_total;
    const uint32_t per = (tiles_total + groups - 1u) / groups;
    // the deepest ring of weight units that fits beside the conversion areas, then as many
    // tiles between two meetings as the rest holds (equal groups)
    uint32_t ring = 4;
    while (ring > 2u && r16_lds_bytes(waves, mt, bw, ring, 1) > kR16Lds) --ring;
    if (r16_lds_bytes(waves, mt, bw, ring, 1) > kR16Lds) return false;
    const uint32_t tps = r16_sync_tiles(waves, waves, mt, bw, ring, per);
    pl = R16Plan{parts, waves, bw, mt, per, (tiles_total + per - 1u) / per, ring, tps, 0, {}};
    return true;
  }
  return false;
}

}  // namespace

bool gemv_q4k_rows16_supported(uint64_t m, uint64_t n, uint64_t k) {
  R16Plan pl;
  return r16_plan(m, n, k, pl);
}

// Floats of scratch the K parts' output regions need (none when one part writes C itself).
size_t gemv_q4k_rows16_workspace_bytes(uint64_t m, uint64_t n, uint64_t k) {
  R16Plan pl;
  if (!r16_plan(m, n, k, pl) || pl.parts == 1) return 0;
  return static_cast<size_t>(pl.parts) * m * n * 4;
}

// The kernels ask for more dynamic LDS than the default limit allows; the limit is raised once, at
// library initialisation (not inside a launch, which may be under stream capture).
namespace {
// Calls f with the instantiation that runs plan (mt, bw, ring).
template <typename F>
void r16_with_kernel(uint32_t mt, uint32_t bw, uint32_t ring, F&& f) {
  auto by_ring = [&](auto mtc, auto bwc) {
    constexpr int kMT = decltype(mtc)::value, kBW = decltype(bwc)::value;
    if (ring >= 4u) f(q4k_rows16_kernel<kMT, kBW, 4>);
    else if (ring == 3u) f(q4k_rows16_kernel<kMT, kBW, 3>);
    else f(q4k_rows16_kernel<kMT, kBW, 2>);
  };
  if (mt == 2u) by_ring(std::integral_constant<int, 2>{}, std::integral_constant<int, 1>{});
  else if (bw == 1u) by_ring(std::integral_constant<int, 1>{}, std::integral_constant<int, 1>{});
  else by_ring(std::integral_constant<int, 1>{}, std::integral_constant<int, 2>{});
}
}  // namespace

hipError_t gemv_q4k_rows16_prepare() {
  hipError_t err = hipSuccess;
  for (uint32_t shape = 0; shape < 3; ++shape)
    for (uint32_t ring = 2; ring <= 4; ++ring)
      r16_with_kernel(shape == 0 ? 2u : 1u, shape == 2 ? 2u : 1u, ring, [&](auto kernel) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 160 * 1024 - 64);
        if (e != hipSuccess && err == hipSuccess) err = e;
      });
  return err;
}

hipError_t launch_q4k_rows16(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m, uint32_t n,
                             uint32_t k, hipStream_t stream) {
  R16Plan pl;
  if (!r16_plan(m, n, k, pl)) return hipErrorInvalidValue;
  R16Args args{a, w, c, static_cast<float*>(workspace), m, n, k, pl.tiles_per_wg, static_cast<uint32_t>(k / 256) / pl.parts,
               pl.tiles_per_sync, pl.n_table, {}};
  for (uint32_t i = 0; i < pl.n_table; ++i) args.part[i] = pl.table[i];
  const dim3 grid(pl.row_groups, pl.n_table != 0u ? 1u : pl.parts), block(64 * pl.waves);
  const uint32_t lds = r16_lds_bytes(pl.waves, pl.mt, pl.bw, pl.ring, pl.tiles_per_sync);
  r16_with_kernel(pl.mt, pl.bw, pl.ring, [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, block, lds, stream, args); });
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (pl.parts > 1) return launch_vec_reduce(args.ws, c, static_cast<uint64_t>(m) * n, pl.parts, stream);
  return hipSuccess;
}

}  // namespace qmm
