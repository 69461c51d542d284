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
//    sub-block: eight nibbles of two dwords, masked in place and read as fp16 subnormals
//    (q * 2^-24, which the matrix core honours; 2^24 is folded into d).  The four results a lane
//    gets back belong to its own weight row, so the sub-block scale is applied by the lane that
//    unpacked it.
//  * A = 8 activation rows as 16 matrix rows: row r is hi = f16(x s) and lo = f16(x s - hi), s
//    the power of two that brings the largest magnitude of the row's 256-wide block to
//    [256, 512): 22 significant bits under the block's largest value, exact rescaling.  Products
//    of a 4-bit integer and an 11-bit value are exact in the fp32 accumulator.
//  * per super-block: f = sum_s sc_s * (D_hi + D_lo)_s, mm = sum_s mn_s * Sx_s (Sx = the sub-block
//    sums of what the matrix core sees), result += (d * f - dmin * mm) / s: for a one-hot row every
//    step is exact and the output is the reference's dequantized weight bit for bit.
//
// Work split.  A wavefront owns BW super-block columns of its workgroup's K part and keeps their
// activation operands in registers for the whole kernel (converted once in the prologue through a
// private LDS area); it walks all 16-row tiles of the workgroup's rows, loading each (tile, block)
// unit with coalesced 16-byte loads two units ahead, dropping it into a private LDS slot and
// reading it back in matrix-core order.  No activation is read inside the loop.  The wavefronts'
// partial tiles meet in LDS every kTilesPerSync tiles (one barrier, double buffered) and are added
// in wavefront order.  K parts (gridDim.y) write their sums to separate regions of a scratch buffer
// that a reduce launch adds in part order.  (A workgroup that arrives last adding the regions
// inside this kernel was measured four times slower: the device-scope release and acquire it needs
// write back and invalidate the L2 of its XCD under the workgroups still streaming weights.)

#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

constexpr uint32_t kTile = 16;            // weight rows per tile (the N of the instruction)
constexpr uint32_t kTilesPerSync = 4;
constexpr uint32_t kUnitBytes = kTile * 144u;
constexpr int kKL = 3;                    // 16-byte loads a lane makes per unit: ceil(16 * 9 / 64)
constexpr uint32_t kARowBytes = 256u * 2u + 16u;   // one matrix row of a block in the conversion area

struct R16Args {
  const float* a;          // m x k
  const uint8_t* w;        // n rows of k/256 blocks
  float* c;                // m x n, the result
  float* ws;               // [parts][m][n] partial sums of the K parts (unused with one part)
  uint32_t m, n, k;
  uint32_t tiles_per_wg;
  uint32_t blocks_per_part;
};

template <int kCtrl, int kRowMask>
__device__ __forceinline__ uint32_t dpp_umax16(uint32_t v) {
  const uint32_t moved = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), kCtrl, kRowMask, 0xF, false));
  return v > moved ? v : moved;
}
// Largest value over the 64 lanes, DPP only; uniform result.
__device__ __forceinline__ uint32_t wave_umax16(uint32_t v) {
  v = dpp_umax16<0xB1, 0xF>(v);    // quad_perm [1,0,3,2]
  v = dpp_umax16<0x4E, 0xF>(v);    // quad_perm [2,3,0,1]
  v = dpp_umax16<0x141, 0xF>(v);   // row_half_mirror
  v = dpp_umax16<0x140, 0xF>(v);   // row_mirror
  v = dpp_umax16<0x142, 0xA>(v);   // row_bcast:15
  v = dpp_umax16<0x143, 0xC>(v);   // row_bcast:31
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), 63));
}
template <int kCtrl>
__device__ __forceinline__ float dpp_fadd16(float v) {
  return v + bit_cast<float>(__builtin_amdgcn_update_dpp(0, bit_cast<int>(v), kCtrl, 0xF, 0xF, false));
}

// LDS layout: [unit slots: W][Sx: W x BW x MT x 8 x 8][1/s: W x BW x MT x 8][the conversion areas
// (W x 16 rows) during the prologue, then the partials (2 x kTilesPerSync x W x (8 MT) x 16)]
__host__ __device__ inline uint32_t r16_shared_area_bytes(uint32_t waves, uint32_t mt) {
  const uint32_t conv = waves * 16u * kARowBytes, part = 2u * kTilesPerSync * waves * 8u * mt * 16u * 4u;
  return conv > part ? conv : part;
}
__host__ __device__ inline uint32_t r16_lds_bytes(uint32_t waves, uint32_t mt, uint32_t bw) {
  return waves * kUnitBytes + waves * bw * mt * (64u + 8u) * 4u + r16_shared_area_bytes(waves, mt);
}

// MT = 16-row matrix tiles of activations (8 activation rows each), BW = block columns a wavefront owns.
template <int MT, int BW>
__global__ __launch_bounds__(768) void q4k_rows16_kernel(R16Args p) {
  static_assert(MT * BW <= 2, "the activation operands of a wavefront take 32 registers per tile and column");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t waves = blockDim.x >> 6;
  const uint32_t nrow = lane & 15u, gq = lane >> 4;        // weight row of the tile, K chunk of a sub-block
  const uint32_t nbp = p.blocks_per_part;
  const uint32_t b0 = blockIdx.y * nbp;                    // first block of this K part
  const uint32_t sbs = p.k / 256u, row_bytes = sbs * 144u;
  const uint32_t tiles_total = (p.n + kTile - 1u) / kTile;
  const uint32_t tile0 = blockIdx.x * p.tiles_per_wg;
  if (tile0 >= tiles_total) return;                        // whole workgroup leaves together
  const uint32_t tiles = tile0 + p.tiles_per_wg <= tiles_total ? p.tiles_per_wg : tiles_total - tile0;
  const uint32_t row0 = tile0 * kTile;

  uint8_t* slot = lds + wave * kUnitBytes;
  float* sx_all = reinterpret_cast<float*>(lds + waves * kUnitBytes);
  float* sx = sx_all + wave * (BW * MT * 64u);                               // [BW][MT][8 sub-blocks][8 rows]
  float* inv_all = sx_all + waves * (BW * MT * 64u);
  float* invs = inv_all + wave * (BW * MT * 8u);                             // [BW][MT][8 rows]
  float* part = inv_all + waves * (BW * MT * 8u);                            // [2][kTilesPerSync][W][8 MT][16]
  uint8_t* conv = reinterpret_cast<uint8_t*>(part) + wave * 16u * kARowBytes;   // prologue only, same memory as `part`

  // Block columns of this wavefront inside the part: wave, wave + W (BW = 2); one past the part
  // is computed with zero activations on the part's last block.
  auto col_live = [&](uint32_t jb) { return wave + jb * waves < nbp; };
  auto col = [&](uint32_t jb) { return b0 + (col_live(jb) ? wave + jb * waves : nbp - 1u); };

  // ---- weight units: piece pc = i * 64 + lane of a unit is 16 bytes pc % 9 of row pc / 9
  struct Unit {
    uint4 v[kKL];
  };
  uint32_t piece_row[kKL], piece_off[kKL];
#pragma unroll
  for (int i = 0; i < kKL; ++i) {
    uint32_t pc = i * 64u + lane;
    pc = pc < kTile * 9u ? pc : kTile * 9u - 1u;
    piece_row[i] = pc / 9u;
    piece_off[i] = (pc - piece_row[i] * 9u) * 16u;
  }
  const uint32_t n_units = tiles * BW;
  uint32_t issued = 0;
  auto next_unit = [&]() {
    // unit u = (tile u / BW, column u % BW); past the last one the last is read again (the loads
    // stay unconditional so that outstanding loads are counted exactly; the bytes come from L2)
    const uint32_t u = issued < n_units ? issued : n_units - 1u;
    const uint32_t tl = u / BW, jb = u % BW;
    const uint32_t first_row = row0 + tl * kTile;
    const uint8_t* base = p.w + static_cast<size_t>(col(jb)) * 144u;
    Unit un;
#pragma unroll
    for (int i = 0; i < kKL; ++i) {
      const uint32_t row = first_row + piece_row[i] < p.n ? first_row + piece_row[i] : p.n - 1u;   // past the matrix: the last row, never stored
      un.v[i] = *reinterpret_cast<const uint4*>(base + static_cast<size_t>(row) * row_bytes + piece_off[i]);
    }
    ++issued;
    return un;
  };
  // units in flight per wavefront (four measured no faster than two)
  constexpr int kAhead = 2;
  Unit wb[kAhead];
  wb[0] = next_unit();

  // ---- activations of this wavefront's block columns -> matrix-core operands in registers
  half8_t afrag[BW][MT][8];
#pragma unroll
  for (int jb = 0; jb < BW; ++jb) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      // with one column per wavefront all eight rows are requested before the first is converted
      constexpr int kPre = BW == 1 ? 8 : 1;
      float4 xv[kPre];
      auto row_ptr = [&](uint32_t r8) {
        const uint32_t r = mt * 8u + r8;
        return reinterpret_cast<const float4*>(p.a + static_cast<size_t>(r < p.m ? r : 0u) * p.k + col(jb) * 256u + lane * 4u);
      };
      if constexpr (kPre == 8) {
#pragma unroll
        for (int r8 = 0; r8 < 8; ++r8) xv[r8] = *row_ptr(r8);
      }
#pragma unroll
      for (int r8 = 0; r8 < 8; ++r8) {
        const uint32_t r = mt * 8u + r8;
        float4 v;
        if constexpr (kPre == 8) v = xv[r8]; else v = *row_ptr(r8);
        if (r >= p.m || !col_live(jb)) v = make_float4(0.f, 0.f, 0.f, 0.f);
        // largest magnitude of the block as bits (integer order = magnitude order; NaN and
        // infinity sort above every finite value, so the same reduction finds them)
        const uint32_t m0 = bit_cast<uint32_t>(v.x) & 0x7FFFFFFFu, m1 = bit_cast<uint32_t>(v.y) & 0x7FFFFFFFu;
        const uint32_t m2 = bit_cast<uint32_t>(v.z) & 0x7FFFFFFFu, m3 = bit_cast<uint32_t>(v.w) & 0x7FFFFFFFu;
        uint32_t mx = max(max(m0, m1), max(m2, m3));
        mx = wave_umax16(mx);
        const uint32_t e = mx >> 23;
        int se = 262 - static_cast<int>(e);                       // amax * s in [2^8, 2^9)
        se = se < 1 ? 1 : (se > 254 ? 254 : se);
        const float s = (e == 0u || e == 0xFFu) ? 1.0f : bit_cast<float>(static_cast<uint32_t>(se) << 23);
        // NaN or infinity anywhere in the block: the block's factor becomes NaN, as the reference's sum would
        const float inv = e == 0xFFu ? bit_cast<float>(0x7FC00000u)
                                     : (e == 0u ? 1.0f : bit_cast<float>(static_cast<uint32_t>(254 - se) << 23));
        float xs[4] = {v.x * s, v.y * s, v.z * s, v.w * s};
        _Float16 hi[4], lo[4];
        float seen = 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          if (e == 0xFFu) xs[c] = 0.0f;
          hi[c] = static_cast<_Float16>(xs[c]);
          lo[c] = static_cast<_Float16>(xs[c] - static_cast<float>(hi[c]));
          seen += static_cast<float>(hi[c]) + static_cast<float>(lo[c]);
        }
        // the nibble masks deliver a chunk's elements in the order 0, 2, 1, 3 | 4, 6, 5, 7
        typedef _Float16 half4v __attribute__((ext_vector_type(4)));
        *reinterpret_cast<half4v*>(conv + (2u * r8) * kARowBytes + lane * 8u) = half4v{hi[0], hi[2], hi[1], hi[3]};
        *reinterpret_cast<half4v*>(conv + (2u * r8 + 1u) * kARowBytes + lane * 8u) = half4v{lo[0], lo[2], lo[1], lo[3]};
        // sub-block sums: eight consecutive lanes
        seen = dpp_fadd16<0xB1>(seen);     // quad_perm [1,0,3,2]
        seen = dpp_fadd16<0x4E>(seen);     // quad_perm [2,3,0,1]
        seen = dpp_fadd16<0x141>(seen);    // row_half_mirror
        if ((lane & 7u) == 0u) sx[((jb * MT + mt) * 8u + (lane >> 3)) * 8u + r8] = seen;
        if (lane == 0u) invs[(jb * MT + mt) * 8u + r8] = inv;
      }
      // matrix row i = 2 r8 + {hi, lo} is lane % 16; K chunk gq of sub-block sb
#pragma unroll
      for (int sb = 0; sb < 8; ++sb) {
        afrag[jb][mt][sb] = *reinterpret_cast<const half8_t*>(conv + nrow * kARowBytes + (sb * 32u + gq * 8u) * 2u);
      }
    }
  }
#pragma unroll
  for (int i = 1; i < kAhead; ++i) wb[i] = next_unit();
  lds_barrier();     // every wavefront is done with its conversion area: the partials take that memory over

  // a lane's results: weight row nrow, matrix rows 4 gq + e, i.e. activation rows 2 gq + {0, 1} of each MT
  auto stash = [&](const Unit& u) {
#pragma unroll
    for (int i = 0; i < kKL; ++i) {
      if (i * 64u + lane < kTile * 9u) *reinterpret_cast<uint4*>(slot + (i * 64u + lane) * 16u) = u.v[i];
    }
  };

  float tileacc[MT][2];
  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  auto consume = [&](int jb) {
    const uint8_t* blk = slot + nrow * 144u;
    const uint4 h = *reinterpret_cast<const uint4*>(blk);
    uint2 wq[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) wq[g] = *reinterpret_cast<const uint2*>(blk + 16 + g * 32 + gq * 8);
    const float d24 = half_bits_to_float(h.x & 0xFFFFu) * 0x1p24f;
    const float dmin = half_bits_to_float(h.x >> 16);
    const uint32_t sc_lo = h.y & 0x3F3F3F3Fu, mn_lo = h.z & 0x3F3F3F3Fu;
    const uint32_t sc_hi = (h.w & 0x0F0F0F0Fu) | ((h.y >> 2) & 0x30303030u);
    const uint32_t mn_hi = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    float f[MT][2], mm[MT][2];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) f[mt][0] = f[mt][1] = mm[mt][0] = mm[mt][1] = 0.0f;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const uint32_t x = wq[g].x, y = wq[g].y;
      constexpr uint32_t kM = 0x000F000Fu;
      const int4v_t b_even = {static_cast<int>(x & kM), static_cast<int>((x >> 8) & kM), static_cast<int>(y & kM),
                              static_cast<int>((y >> 8) & kM)};
      const int4v_t b_odd = {static_cast<int>((x >> 4) & kM), static_cast<int>((x >> 12) & kM),
                             static_cast<int>((y >> 4) & kM), static_cast<int>((y >> 12) & kM)};
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int sb = 2 * g + half;
        const uint32_t scw = sb < 4 ? sc_lo : sc_hi, mnw = sb < 4 ? mn_lo : mn_hi;
        const float sc = static_cast<float>((scw >> (8 * (sb & 3))) & 0xFFu);
        const float mn = static_cast<float>((mnw >> (8 * (sb & 3))) & 0xFFu);
        const half8_t bop = bit_cast<half8_t>(half ? b_odd : b_even);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const float4_t dres = __builtin_amdgcn_mfma_f32_16x16x32_f16(afrag[jb][mt][sb], bop, zero4, 0, 0, 0);
          f[mt][0] = fmaf(sc, dres[0] + dres[1], f[mt][0]);
          f[mt][1] = fmaf(sc, dres[2] + dres[3], f[mt][1]);
          const float2 sxv = *reinterpret_cast<const float2*>(sx + ((jb * MT + mt) * 8u + sb) * 8u + 2u * gq);
          mm[mt][0] = fmaf(mn, sxv.x, mm[mt][0]);
          mm[mt][1] = fmaf(mn, sxv.y, mm[mt][1]);
        }
      }
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const float acc = fmaf(d24, f[mt][j], -(dmin * mm[mt][j]));
        tileacc[mt][j] = fmaf(acc, invs[(jb * MT + mt) * 8u + 2u * gq + j], tileacc[mt][j]);
      }
  };

  // ---- tiles.  Every wavefront walks the same tiles, so the barriers match.
  const size_t region = static_cast<size_t>(p.m) * p.n;
  float* cpart = gridDim.y == 1 ? p.c : p.ws + blockIdx.y * region;
  uint32_t buf = 0;
  // One tile: its BW units, then the wavefront's partial tile into LDS.  A unit's registers are
  // refilled, kAhead units ahead, as soon as it sits in the slot; unit u uses register set
  // u % kAhead, which is a constant of the tile's position in its group of kTilesPerSync.
  auto do_tile = [&](auto pos) {
    constexpr int ti = decltype(pos)::value;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) tileacc[mt][0] = tileacc[mt][1] = 0.0f;
#pragma unroll
    for (int jb = 0; jb < BW; ++jb) {
      constexpr int kSets = kAhead;
      const int set = (BW * ti + jb) % kSets;
      stash(wb[set]);
      wb[set] = next_unit();
      consume(jb);
    }
    float* dst = part + (((buf * kTilesPerSync + ti) * waves + wave) * (8u * MT)) * 16u;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int j = 0; j < 2; ++j) dst[(mt * 8u + 2u * gq + j) * 16u + nrow] = tileacc[mt][j];
  };
  static_assert(kTilesPerSync == 4 && (BW * kTilesPerSync) % kAhead == 0, "register sets repeat with the groups");
  for (uint32_t g0 = 0; g0 < tiles; g0 += kTilesPerSync) {
    const uint32_t in_group = tiles - g0 < kTilesPerSync ? tiles - g0 : kTilesPerSync;
    do_tile(std::integral_constant<int, 0>{});
    if (in_group > 1u) do_tile(std::integral_constant<int, 1>{});
    if (in_group > 2u) do_tile(std::integral_constant<int, 2>{});
    if (in_group > 3u) do_tile(std::integral_constant<int, 3>{});
    lds_barrier();
    // sum the wavefronts' partial tiles per output in wavefront order and store
    for (uint32_t o = t; o < in_group * 8u * MT * 16u; o += blockDim.x) {
      const uint32_t nn = o & 15u, r = (o >> 4) % (8u * MT), ti = o / (128u * MT);
      const uint32_t row = row0 + (g0 + ti) * kTile + nn;
      if (r >= p.m || row >= p.n) continue;
      float sum = 0.0f;
      for (uint32_t wv = 0; wv < waves; ++wv) sum += part[(((buf * kTilesPerSync + ti) * waves + wv) * (8u * MT) + r) * 16u + nn];
      cpart[static_cast<size_t>(r) * p.n + row] = sum;
    }
    buf ^= 1u;
  }
}

struct R16Plan {
  uint32_t parts, waves, bw, mt, tiles_per_wg, row_groups;
};

// K parts: the fewest (a divisor of the block count) whose block columns fit the twelve wavefronts
// of a workgroup, one column each, or two when 8 rows or fewer leave the registers for it --
// preferring one column each when that costs only twice the parts; then the rows are cut into
// equal runs of tiles, a workgroup per CU and part.
bool r16_plan(uint64_t m, uint64_t n, uint64_t k, R16Plan& pl) {
  if (m < 2 || m > 16 || k % 256 != 0 || n == 0 || n > 0x7FFFFFFFull || k > (1ull << 24)) return false;
  const uint32_t nb = static_cast<uint32_t>(k / 256), mt = m > 8 ? 2u : 1u, bw_max = mt == 1 ? 2u : 1u;
  const uint32_t tiles_total = static_cast<uint32_t>((n + kTile - 1) / kTile);
  const uint32_t cus = static_cast<uint32_t>(num_cus());
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
    pl = R16Plan{parts, waves, bw, mt, per, (tiles_total + per - 1u) / per};
    return r16_lds_bytes(waves, mt, bw) + 64u <= 160u * 1024u;
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
hipError_t gemv_q4k_rows16_prepare() {
  const void* kernels[3] = {reinterpret_cast<const void*>(q4k_rows16_kernel<1, 1>), reinterpret_cast<const void*>(q4k_rows16_kernel<1, 2>),
                            reinterpret_cast<const void*>(q4k_rows16_kernel<2, 1>)};
  for (const void* kern : kernels) {
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 64);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

hipError_t launch_q4k_rows16(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m, uint32_t n,
                             uint32_t k, hipStream_t stream) {
  R16Plan pl;
  if (!r16_plan(m, n, k, pl)) return hipErrorInvalidValue;
  R16Args args{a, w, c, static_cast<float*>(workspace), m, n, k, pl.tiles_per_wg, static_cast<uint32_t>(k / 256) / pl.parts};
  const dim3 grid(pl.row_groups, pl.parts), block(64 * pl.waves);
  const uint32_t lds = r16_lds_bytes(pl.waves, pl.mt, pl.bw);
  auto go = [&](auto kernel) { hipLaunchKernelGGL(kernel, grid, block, lds, stream, args); };
  if (pl.mt == 2) go(q4k_rows16_kernel<2, 1>);
  else if (pl.bw == 1) go(q4k_rows16_kernel<1, 1>);
  else go(q4k_rows16_kernel<1, 2>);
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (pl.parts > 1) return launch_vec_reduce(args.ws, c, static_cast<uint64_t>(m) * n, pl.parts, stream);
  return hipSuccess;
}

}  // namespace qmm
