// K-quant weights (Q4_K, Q5_K, Q6_K in GGUF order) x a few fp32 activation rows in ONE pass over the
// weights, on v_mfma_i32_16x16x64_i8, exact on the weight side.
//
//   C[r][n] = sum_k A[r][k] * deq(W)[n][k]
//   (layouts and decodes: src/core/numerics/quant.cpp:58-70,656-675 (Q4_K), :180-229 (Q5_K),
//   :299-342 (Q6_K); the reference's kernels for 2..5 rows, one 32-lane warp per output column:
//   src/backends/rocm/rocm_kernels_gemv.cpp:100-283).
//
// The activations of a 256-wide block become four signed 8-bit limbs under the block's power of two
// (i8_limbs.hpp), the quants go to the matrix core as they are stored (a mask per register), and
// what a floating-point kernel spends per weight (scale, min, convert) is spent here per sixteen or
// thirty-two weights on the integer sums that come back:
//
//  * B, 16 weight rows x 64 K: lane (n, g) loads eight bytes of row n and holds sixteen quants: the
//    low nibbles in its K slots 0..7, the high nibbles in slots 8..15, no byte loaded twice.  Q4_K /
//    Q5_K: the 64 K of "chunk" c are sub-blocks 2c (low nibbles) and 2c + 1 (high nibbles), bytes
//    [8g, 8g + 8) of the chunk's 32 per lane.  Q6_K: chunk (half h, p) is quarters p (low nibbles)
//    and p + 2 (high) of the half's 128 weights; with the two high bits the byte becomes 4 (q - 32),
//    so the format's offset costs nothing.
//  * A, 16 matrix rows x 64 K: Q4_K / Q5_K: rows 8 r + 4 par + l = limb l of activation row r
//    (two rows per instruction) with the K slots of the other sub-block parity zeroed, so that the
//    lane group that receives matrix rows 4 g'..4 g' + 3 has, for its own weight row, the four limb
//    sums of ONE sub-block and folds them with that sub-block's 6-bit scale by 24-bit integer
//    multiply-adds.  Q6_K has four scales per 64 K (per slot half and per pair of lane groups), so
//    all sixteen matrix rows go to one activation row: 4 v + l = limb l against the sixteen weights
//    under scale v of the chunk.
//  * per block and activation row the integer sums meet d, dmin and the block's power of two in fp32:
//    y += d * T * 2^-sh - dmin * sum_s mn_s S_s (S_s = the activations' sub-block sums), so a one-hot
//    activation returns the reference's dequantized weight RN(d * sc * q - dmin * mn) bit for bit.
//
// Work split.  A workgroup owns a range of weight rows over all of K (so nothing is left to add up
// in a second launch) and its wavefronts share the blocks of K: wavefront w takes blocks w, w + W, ...
// and, for each, walks the workgroup's 16-row tiles with the block's A operands in registers and two
// units of weights in flight.  It asks for the activations of its next block one block ahead and turns
// them into limbs when it gets there, row by row through one private 1 KB LDS slot; the sums of a
// tile live in a private LDS table; the wavefronts meet once, at the end, and their tables are added
// in wavefront order.  The row ranges are equal shares
// of the matrix whether or not that is a multiple of 16 rows: the CUs then stream equal byte counts,
// which is what sets the duration of a launch that is bound by memory.

#include "i8_limbs.hpp"
#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

using namespace i8limbs;

struct KqArgs {
  const uint8_t* w;
  const float* x;
  float* c;
  uint32_t m, n, nblk, rows_per_wg;
};

typedef uint4 uint4_u2 __attribute__((aligned(2)));
typedef uint2 uint2_u2 __attribute__((aligned(2)));
__device__ __forceinline__ uint4 load_u4_unaligned(const void* p) { return *reinterpret_cast<const uint4_u2*>(p); }
__device__ __forceinline__ uint2 load_u2_unaligned(const void* p) { return *reinterpret_cast<const uint2_u2*>(p); }

// The four limb sums of one lane times 256^l, as a float (each step exact while the total fits 24
// bits, which a one-hot row does).
__device__ __forceinline__ float join_limbs(const int (&acc)[4]) {
  float t = fmaf(static_cast<float>(acc[1]), 256.0f, static_cast<float>(acc[0]));
  t = fmaf(static_cast<float>(acc[2]), 65536.0f, t);
  return fmaf(static_cast<float>(acc[3]), 16777216.0f, t);
}

// ---- Q4_K and Q5_K: eight sub-blocks of 32 with 6-bit scales and mins ---------------------------
// The scales and mins of the four sub-blocks of parity par, from the twelve bytes in h.y, h.z, h.w
// (src/core/numerics/quant.cpp:58-70).
__device__ __forceinline__ void scales_of_parity(const uint4 h, uint32_t par, int (&sc)[4], float (&mn)[4]) {
  const uint32_t y = h.y >> (8u * par), z = h.z >> (8u * par), w = h.w >> (8u * par);
  sc[0] = static_cast<int>(y & 63u), sc[1] = static_cast<int>((y >> 16) & 63u);
  sc[2] = static_cast<int>((w & 15u) | ((y >> 2) & 0x30u)), sc[3] = static_cast<int>(((w >> 16) & 15u) | ((y >> 18) & 0x30u));
  mn[0] = static_cast<float>(z & 63u), mn[1] = static_cast<float>((z >> 16) & 63u);
  mn[2] = static_cast<float>(((w >> 4) & 15u) | ((z >> 2) & 0x30u));
  mn[3] = static_cast<float>(((w >> 20) & 15u) | ((z >> 18) & 0x30u));
}

template <bool kFiveBits>
struct Sub32Format {
  static constexpr uint32_t kBlock = kFiveBits ? 176u : 144u;
  static constexpr uint32_t kQs = kFiveBits ? 48u : 16u;
  static constexpr int kRowsPerSet = 2;     // activation rows one matrix instruction serves
  static constexpr uint32_t kMaxWaves[4] = {16u, 12u, 8u, 8u};
  struct Unit {
    uint4 h;
    uint2 qh;      // Q5_K: the fifth bits of the lane's eight byte positions, one bit per sub-block
    uint2 q[4];
  };
  struct Ctx {
    float4 S;      // sums of the four sub-blocks of the lane's parity, of the lane's activation row
    float f;       // 2^-sh of that row
  };

  // The lane's registers of a unit out of its row's block.
  static __device__ __forceinline__ void read(Unit& u, const uint8_t* blk, uint32_t g) {
    u.h = *reinterpret_cast<const uint4*>(blk);
    if (kFiveBits) u.qh = *reinterpret_cast<const uint2*>(blk + 16u + 8u * g);
#pragma unroll
    for (int c = 0; c < 4; ++c) u.q[c] = *reinterpret_cast<const uint2*>(blk + kQs + 32u * c + 8u * g);
  }

  // Activation row r has just been converted into `slot`: the lanes whose matrix rows carry it
  // take their A operands of set r / 2, and the lanes that will receive its sums what they need to
  // finish them.
  static __device__ __forceinline__ void fetch(int4v_t (&A)[4], Ctx& ctx, const uint8_t* slot, uint32_t r, uint32_t m,
                                               uint32_t lane) {
    const uint32_t ln = lane & 15u, g = lane >> 4;
    const uint32_t apar = (ln >> 2) & 1u;
    if ((ln >> 3) == (r & 1u)) {
      // eight weights' limbs in the K slots of the lane's parity, zeros in the other eight
      const uint8_t* a = slot + apar * 128u + (g >> 1) * 64u + (ln & 3u) * 16u + (g & 1u) * 8u;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        uint2 v = *reinterpret_cast<const uint2*>(a + c * 256);
        if (r >= m) v = make_uint2(0u, 0u);
        const int x = static_cast<int>(v.x), y = static_cast<int>(v.y);
        A[c] = apar ? int4v_t{0, 0, x, y} : int4v_t{x, y, 0, 0};
      }
    }
    if ((g >> 1) == (r & 1u)) {
      if (r < m) {
        ctx.S = *reinterpret_cast<const float4*>(slot + 1024u + (g & 1u) * 16u);
        ctx.f = __builtin_ldexpf(1.0f, -reinterpret_cast<const int*>(slot + 1056u)[0]);
      } else {
        ctx.S = make_float4(0.f, 0.f, 0.f, 0.f);
        ctx.f = 0.0f;
      }
    }
  }

  template <int NA>
  static __device__ __forceinline__ void dot(const Unit& u, const int4v_t (&A)[NA][4], const Ctx (&ctx)[NA],
                                             float (&val)[NA], uint32_t lane) {
    const uint32_t g = lane >> 4;
    int sc[4];
    float mn[4];
    scales_of_parity(u.h, g & 1u, sc, mn);
    const float d = half_bits_to_float(u.h.x & 0xFFFFu), dmin = half_bits_to_float(u.h.x >> 16);
    int4v_t B[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      constexpr uint32_t kN = 0x0F0F0F0Fu, kOne = 0x01010101u;
      uint32_t b0 = u.q[c].x & kN, b1 = u.q[c].y & kN, b2 = (u.q[c].x >> 4) & kN, b3 = (u.q[c].y >> 4) & kN;
      if (kFiveBits) {
        // bits 2c (low nibbles' sub-block) and 2c + 1 of the fifth-bit bytes -> bit 4
        b0 |= ((u.qh.x >> (2 * c)) & kOne) << 4, b1 |= ((u.qh.y >> (2 * c)) & kOne) << 4;
        b2 |= ((u.qh.x >> (2 * c + 1)) & kOne) << 4, b3 |= ((u.qh.y >> (2 * c + 1)) & kOne) << 4;
      }
      B[c] = int4v_t{static_cast<int>(b0), static_cast<int>(b1), static_cast<int>(b2), static_cast<int>(b3)};
    }
    const int4v_t zero = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < NA; ++s) {
      int acc[4] = {0, 0, 0, 0};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int4v_t D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[s][c], B[c], zero, 0, 0, 0);
#pragma unroll
        for (int l = 0; l < 4; ++l) {
          acc[l] = mad24(D[l], sc[c], acc[l]);
          asm("" : "+v"(acc[l]));   // one multiply-add per step, not a multiply and a three-way add later
        }
      }
      const float4 S = ctx[s].S;
      float accm = mn[0] * S.x;
      accm = fmaf(mn[1], S.y, accm), accm = fmaf(mn[2], S.z, accm), accm = fmaf(mn[3], S.w, accm);
      val[s] = fmaf(d, join_limbs(acc) * ctx[s].f, -(dmin * accm));
    }
  }

  // The output (tile-local row ln, activation row r) out of one wavefront's table of a tile.
  static __device__ __forceinline__ float gather(const float* tile_part, uint32_t r, uint32_t ln) {
    const float* p = tile_part + (r >> 1) * 64u + (r & 1u) * 32u + ln;
    return p[0] + p[16];
  }
};

// ---- Q6_K: sixteen groups of 16 with signed 8-bit scales, no mins ----------------------------------
struct Q6KFormat {
  static constexpr uint32_t kBlock = 210u;
  static constexpr int kRowsPerSet = 1;
  static constexpr uint32_t kMaxWaves[4] = {16u, 16u, 12u, 8u};
  struct Unit {
    uint2 ql[4];   // chunk 2h + p: bytes 64h + 32p + 8g ..
    uint2 qh[2];   // half h: bytes 128 + 32h + 8g ..
    uint4 sc;
    uint32_t d;
  };
  struct Ctx {
    float f;       // 2^-(sh + 2) of the set's activation row (NaN when the block holds a NaN or an infinity)
  };

  // (blocks of 210 bytes start on even addresses only)
  static __device__ __forceinline__ void read(Unit& u, const uint8_t* blk, uint32_t g) {
#pragma unroll
    for (int c = 0; c < 4; ++c) u.ql[c] = load_u2_unaligned(blk + 32u * c + 8u * g);
#pragma unroll
    for (int h = 0; h < 2; ++h) u.qh[h] = load_u2_unaligned(blk + 128u + 32u * h + 8u * g);
    u.sc = load_u4_unaligned(blk + 192u);
    u.d = *reinterpret_cast<const uint16_t*>(blk + 208u);
  }

  static __device__ __forceinline__ void fetch(int4v_t (&A)[4], Ctx& ctx, const uint8_t* slot, uint32_t r, uint32_t m,
                                               uint32_t lane) {
    const uint32_t ln = lane & 15u, g = lane >> 4;
    // Matrix row 4v + l: v = 2 (which half of a lane's K slots: quarter p or p + 2) + (which 16 of the
    // quarter's 32 weights: lanes g / 2).  Chunk 2h + p: sub-block 4h + p + 2 (v / 2), the lane's eight
    // weights [8g, 8g + 8) of it.
    const uint32_t v = ln >> 2;
    const bool live = (g >> 1) == (v & 1u) && r < m;
    const uint8_t* a = slot + (v >> 1) * 256u + (g >> 1) * 64u + (ln & 3u) * 16u + (g & 1u) * 8u;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      uint2 w = *reinterpret_cast<const uint2*>(a + (c >> 1) * 512 + (c & 1) * 128);
      if (!live) w = make_uint2(0u, 0u);
      const int x = static_cast<int>(w.x), y = static_cast<int>(w.y);
      A[c] = (v >> 1) ? int4v_t{0, 0, x, y} : int4v_t{x, y, 0, 0};
    }
    ctx.f = 0.0f;
    if (r < m) {
      // An infinity shows in the block's shift, a NaN (which the largest-magnitude search skips) in
      // the sub-block sums: either makes the block's factor NaN, as the reference's sum would be.
      const int sh = reinterpret_cast<const int*>(slot + 1056u)[0];
      const float4 s0 = *reinterpret_cast<const float4*>(slot + 1024u), s1 = *reinterpret_cast<const float4*>(slot + 1040u);
      const float total = ((s0.x + s0.y) + (s0.z + s0.w)) + ((s1.x + s1.y) + (s1.z + s1.w));
      ctx.f = sh == 156 - 255 || total != total ? bit_cast<float>(0x7FC00000u) : __builtin_ldexpf(1.0f, -sh - 2);
    }
  }

  template <int NA>
  static __device__ __forceinline__ void dot(const Unit& u, const int4v_t (&A)[NA][4], const Ctx (&ctx)[NA],
                                             float (&val)[NA], uint32_t lane) {
    const uint32_t g = lane >> 4, upper = g >> 1;
    const float d = half_bits_to_float(u.d);
    // the lane's scale in chunk 2h + p: group 8h + 2 (p + 2 upper) + g % 2
    const uint32_t scw[4] = {u.sc.x, u.sc.y, u.sc.z, u.sc.w};
    int sc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint32_t word = upper ? scw[2 * (c >> 1) + 1] : scw[2 * (c >> 1)];   // groups 8h + 4 upper ..
      sc[c] = static_cast<int>(static_cast<int8_t>((word >> (16u * (c & 1) + 8u * (g & 1u))) & 0xFFu));
    }
    int4v_t B[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const uint32_t l2[2] = {u.ql[c].x, u.ql[c].y}, h2[2] = {u.qh[c >> 1].x, u.qh[c >> 1].y};
      // nibble -> bits 2..5 (a rotation: what crosses a byte border is masked away), the two high bits
      // of the quarter (p for the low nibbles, p + 2 for the high ones) -> bits 6..7, and the sign
      // flipped: the byte is 4 (q - 32)
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const uint32_t rot_n = half ? 2u : 30u;
        const uint32_t rot_h = (26u + 2u * ((c & 1) + 2u * half)) & 31u;   // bit 2 quarter -> bit 6
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const uint32_t nib = __builtin_amdgcn_alignbit(l2[i], l2[i], rot_n) & 0x3C3C3C3Cu;
          const uint32_t hi = __builtin_amdgcn_alignbit(h2[i], h2[i], rot_h) & 0xC0C0C0C0u;
          B[c][2 * half + i] = static_cast<int>((nib | hi) ^ 0x80808080u);
        }
      }
    }
    const int4v_t zero = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < NA; ++s) {
      int acc[4] = {0, 0, 0, 0};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int4v_t D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[s][c], B[c], zero, 0, 0, 0);
#pragma unroll
        for (int l = 0; l < 4; ++l) {
          acc[l] = mad24(D[l], sc[c], acc[l]);
          asm("" : "+v"(acc[l]));
        }
      }
      val[s] = d * (join_limbs(acc) * ctx[s].f);
    }
  }

  static __device__ __forceinline__ float gather(const float* tile_part, uint32_t r, uint32_t ln) {
    const float* p = tile_part + r * 64u + ln;
    return (p[0] + p[16]) + (p[32] + p[48]);
  }
};

// NA = sets of A operands (matrix instructions per 64 K), WMAX = most wavefronts a workgroup may have.
template <class F, int NA, int WMAX>
__global__ __launch_bounds__(WMAX * 64) void kquant_rows_kernel(KqArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr uint32_t kRows = NA * F::kRowsPerSet;
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t W = blockDim.x >> 6;
  const uint32_t row0 = blockIdx.x * p.rows_per_wg;
  if (row0 >= p.n) return;
  const uint32_t rows = p.n - row0 < p.rows_per_wg ? p.n - row0 : p.rows_per_wg;
  const uint32_t tiles = (rows + 15u) >> 4;
  const uint32_t nmine = wave < p.nblk ? (p.nblk - wave + W - 1u) / W : 0u;
  const uint32_t part_floats = tiles * NA * 64u;
  const uint32_t wave_lds = kSlot + part_floats * 4u;
  uint8_t* slot = lds + wave * wave_lds;
  float* part = reinterpret_cast<float*>(slot + kSlot);
  for (uint32_t i = lane; i < part_floats; i += 64u) part[i] = 0.0f;

  const uint32_t ln = lane & 15u, g = lane >> 4;
  const uint32_t row_bytes = p.nblk * F::kBlock;
  const uint8_t* wbase = p.w + static_cast<size_t>(row0) * row_bytes + wave * F::kBlock;
  const uint32_t k = p.nblk * 256u;

  float4 xr[kRows];
  auto x_request = [&](uint32_t j) {
    const uint32_t b = wave + (j < nmine ? j : 0u) * W;
#pragma unroll
    for (uint32_t r = 0; r < kRows; ++r) {
      if (r < p.m) xr[r] = *reinterpret_cast<const float4*>(p.x + static_cast<size_t>(r) * k + (b < p.nblk ? b : 0u) * 256u + lane * 4u);
    }
  };
  // units in the order they are worked on: block after block, tile after tile
  uint32_t lj = 0, lt = 0;
  auto request = [&](typename F::Unit& u) {
    if (lj < nmine) {
      uint32_t rr = lt * 16u + ln;
      rr = rr < rows ? rr : rows - 1u;     // a row past the range repeats the last: never stored
      F::read(u, wbase + rr * row_bytes + lj * (W * F::kBlock), g);
      if (++lt == tiles) lt = 0, ++lj;
    }
  };
  // the activations first: loads return in order, and the conversion must not wait behind the weights
  x_request(0);
  typename F::Unit ua, ub;
  request(ua);
  request(ub);

  int4v_t A[NA][4];
  typename F::Ctx ctx[NA];
  uint32_t j = 0, t = 0;
  auto step = [&](const typename F::Unit& u) {
    if (j >= nmine) return;
    if (t == 0u) {
      // a new block: its activations become limbs, one row at a time through the one LDS slot
#pragma unroll
      for (uint32_t r = 0; r < kRows; ++r) {
        if (r < p.m) convert_block(xr[r], lane, slot);
        F::fetch(A[r / F::kRowsPerSet], ctx[r / F::kRowsPerSet], slot, r, p.m, lane);
      }
      x_request(j + 1u);
    }
    float* dst = part + t * (NA * 64u) + lane;
    float old[NA], val[NA];
#pragma unroll
    for (int s = 0; s < NA; ++s) old[s] = dst[s * 64];
    F::template dot<NA>(u, A, ctx, val, lane);
#pragma unroll
    for (int s = 0; s < NA; ++s) dst[s * 64] = old[s] + val[s];
    if (++t == tiles) t = 0, ++j;
  };
  while (j < nmine) {
    step(ua);
    request(ua);
    step(ub);
    request(ub);
  }
  __syncthreads();
  for (uint32_t o = threadIdx.x; o < tiles * kRows * 16u; o += blockDim.x) {
    const uint32_t nn = o & 15u, r = (o >> 4) % kRows, tl = o / (16u * kRows);
    const uint32_t row = tl * 16u + nn;
    if (r >= p.m || row >= rows) continue;
    float sum = 0.0f;
    for (uint32_t wv = 0; wv < W; ++wv) {   // wavefront order
      sum += F::gather(reinterpret_cast<const float*>(lds + wv * wave_lds + kSlot) + tl * (NA * 64u), r, nn);
    }
    p.c[static_cast<size_t>(r) * p.n + row0 + row] = sum;
  }
}

struct KqPlan {
  uint32_t waves, rows_per_wg, workgroups, lds;
};

constexpr uint32_t kKqLdsLimit = 160u * 1024u - 512u;

// Most wavefronts of a workgroup: what the registers of NA operand sets leave room for.
template <class F, int NA>
constexpr uint32_t kq_max_waves() {
  return F::kMaxWaves[NA - 1];
}

template <class F, int NA>
bool kq_plan(uint32_t n, uint32_t nblk, uint32_t cus, KqPlan& pl) {
  const uint32_t wmax = kq_max_waves<F, NA>();
  // Wavefronts: a CU runs them on four SIMDs (wavefront w on SIMD w % 4) and the launch lasts as
  // long as the SIMD with the most blocks to work through, so the count that makes that number
  // smallest, the larger count on a tie (more wavefronts hide more of each other's waits).
  uint32_t best = wmax, best_cost = ~0u;
  for (uint32_t w = wmax; w >= 4u; --w) {
    uint32_t cost = 0;
    for (uint32_t simd = 0; simd < 4u; ++simd) {
      uint32_t blocks = 0;
      for (uint32_t wv = simd; wv < w; wv += 4u) blocks += wv < nblk ? (nblk - wv + w - 1u) / w : 0u;
      cost = blocks > cost ? blocks : cost;
    }
    if (cost < best_cost) best = w, best_cost = cost;
  }
  // equal shares of the rows, one workgroup a CU; more rounds of workgroups when a share's tables
  // would not fit the LDS
  for (uint32_t rounds = 1; rounds <= 64u; ++rounds) {
    const uint32_t wgs = cus * rounds;
    const uint32_t share = (n + wgs - 1u) / wgs;
    const uint32_t tiles = (share + 15u) / 16u;
    const uint32_t lds = best * (kSlot + tiles * NA * 256u);
    if (lds <= kKqLdsLimit) {
      pl = KqPlan{best, share, (n + share - 1u) / share, lds};
      return true;
    }
  }
  return false;
}

template <class F, int NA>
hipError_t kq_launch(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t nblk, uint32_t cus,
                     hipStream_t stream) {
  KqPlan pl;
  if (!kq_plan<F, NA>(n, nblk, cus, pl)) return hipErrorInvalidValue;
  const KqArgs args{w, a, c, m, n, nblk, pl.rows_per_wg};
  hipLaunchKernelGGL((kquant_rows_kernel<F, NA, kq_max_waves<F, NA>()>), dim3(pl.workgroups), dim3(pl.waves * 64u), pl.lds, stream,
                     args);
  return hipGetLastError();
}

template <class F, int NA>
hipError_t kq_prepare_one() {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kquant_rows_kernel<F, NA, kq_max_waves<F, NA>()>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kKqLdsLimit));
}

// Rows a pass takes: Q4_K / Q5_K two per operand set and up to four sets, Q6_K one per set.
template <class F>
hipError_t kq_launch_rows(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k, hipStream_t stream) {
  const uint32_t nblk = k / 256u, cus = static_cast<uint32_t>(num_cus());
  constexpr uint32_t per_pass = 4u * F::kRowsPerSet;
  for (uint32_t r0 = 0; r0 < m; r0 += per_pass) {
    const uint32_t mr = m - r0 < per_pass ? m - r0 : per_pass;
    const uint32_t sets = (mr + F::kRowsPerSet - 1u) / F::kRowsPerSet;
    const float* ar = a + static_cast<size_t>(r0) * k;
    float* cr = c + static_cast<size_t>(r0) * n;
    hipError_t e;
    switch (sets) {
      case 1: e = kq_launch<F, 1>(ar, w, cr, mr, n, nblk, cus, stream); break;
      case 2: e = kq_launch<F, 2>(ar, w, cr, mr, n, nblk, cus, stream); break;
      case 3: e = kq_launch<F, 3>(ar, w, cr, mr, n, nblk, cus, stream); break;
      default: e = kq_launch<F, 4>(ar, w, cr, mr, n, nblk, cus, stream); break;
    }
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

template <class F>
hipError_t kq_prepare_format() {
  hipError_t e;
  if ((e = kq_prepare_one<F, 1>()) != hipSuccess) return e;
  if ((e = kq_prepare_one<F, 2>()) != hipSuccess) return e;
  if ((e = kq_prepare_one<F, 3>()) != hipSuccess) return e;
  return kq_prepare_one<F, 4>();
}

}  // namespace

hipError_t gemv_kquant_rows_prepare() {
  hipError_t e;
  if ((e = kq_prepare_format<Sub32Format<false>>()) != hipSuccess) return e;
  if ((e = kq_prepare_format<Sub32Format<true>>()) != hipSuccess) return e;
  return kq_prepare_format<Q6KFormat>();
}

bool gemv_kquant_rows_supported(uint64_t m, uint64_t n, uint64_t k) {
  return m >= 1 && n >= 1 && k >= 256 && k % 256 == 0 && k / 256 <= 0xFFFFu && n <= 0x7FFFFFFFull &&
         n * (k / 256) * 210ull <= 0xFFFFFFFFull * 16ull;
}

hipError_t launch_q4k_rows_i8(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                              hipStream_t stream) {
  return kq_launch_rows<Sub32Format<false>>(a, w, c, m, n, k, stream);
}
hipError_t launch_q5k_rows_i8(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                              hipStream_t stream) {
  return kq_launch_rows<Sub32Format<true>>(a, w, c, m, n, k, stream);
}
hipError_t launch_q6k_rows_i8(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                              hipStream_t stream) {
  return kq_launch_rows<Q6KFormat>(a, w, c, m, n, k, stream);
}

}  // namespace qmm
