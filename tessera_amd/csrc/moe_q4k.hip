// Routed experts (Q4_K) for a chunk of tokens, grouped by expert: every expert's weights are
// streamed once for all the tokens routed to it (reference per-row kernels:
// src/backends/rocm/rocm_kernels_moe.cpp:15-79; caller src/models/qwen3_5/moe.cpp:396-423).

#include "q4k_tile.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

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

}  // namespace

// ---- routed experts, a whole chunk of tokens grouped by expert -----------------------------
// (token, slot) pairs are sorted by expert so that each expert's weights are streamed once for
// all the tokens routed to it, and the three projections run as grouped MFMA GEMMs.
namespace {

// seg[e] = first sorted position of expert e (seg[experts] = pairs); pos[p] = sorted position
// of pair p; inv[pos[p]] = p.  Counting sort with LDS atomics: which position inside its expert's
// segment a pair gets depends on the order the atomics land in, but a row's result does not
// depend on where the row sits, so the outputs are the same on every run.  One workgroup of 1024.
__device__ __forceinline__ void moe_sort_pairs(const uint32_t* __restrict__ ids, uint32_t pairs, uint32_t experts,
                                               uint32_t* __restrict__ seg, uint32_t* __restrict__ pos,
                                               uint32_t* __restrict__ inv) {
  __shared__ uint32_t cursor[1024], wave_total[16];
  const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
  cursor[t] = 0;
  __syncthreads();
  for (uint32_t p = t; p < pairs; p += 1024u) {
    const uint32_t id = ids[p] < experts ? ids[p] : experts - 1u;   // a bad id cannot leave the tensor
    atomicAdd(&cursor[id], 1u);
  }
  __syncthreads();
  // exclusive prefix sum of the 1024 counts: inside each wavefront, then over the 16 totals
  const uint32_t count = cursor[t];
  uint32_t run = count;
#pragma unroll
  for (uint32_t d = 1; d < 64u; d *= 2u) {
    const uint32_t below = __shfl_up(run, d);
    if (lane >= d) run += below;
  }
  if (lane == 63u) wave_total[wave] = run;
  __syncthreads();
  uint32_t base = 0;
  for (uint32_t w = 0; w < wave; ++w) base += wave_total[w];
  const uint32_t first = base + run - count;
  __syncthreads();
  cursor[t] = first;
  if (t < experts) seg[t] = first;
  if (t == experts - 1u) seg[experts] = first + count;
  __syncthreads();
  for (uint32_t p = t; p < pairs; p += 1024u) {
    const uint32_t id = ids[p] < experts ? ids[p] : experts - 1u;
    const uint32_t at = atomicAdd(&cursor[id], 1u);
    pos[p] = at;
    inv[at] = p;
  }
}

__global__ __launch_bounds__(1024) void moe_sort_kernel(const uint32_t* __restrict__ ids, uint32_t pairs,
                                                        uint32_t experts, uint32_t* __restrict__ seg,
                                                        uint32_t* __restrict__ pos, uint32_t* __restrict__ inv) {
  moe_sort_pairs(ids, pairs, experts, seg, pos, inv);
}

// Half the sum of the 32 fp16 values of a Q4_K sub-block as an fp16 pair (hi, lo), for the
// min term of the routed-expert kernels (see moe_block_mma).  `v` is group g (8 values) of a row,
// held by four neighbouring lanes per sub-block; the row's sums live at `sums`, 16 halves a
// super-block: hi of sub-blocks 0..7, then lo.  Halved so that 32 values below 2048 stay below
// the largest fp16 number.
__device__ __forceinline__ void store_subblock_sum(const half8_t& v, uint32_t g, _Float16* sums) {
  float part = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) part += static_cast<float>(v[e]);
  part += __shfl_xor(part, 1);
  part += __shfl_xor(part, 2);
  if ((g & 3u) == 0) {
    const float half_sum = 0.5f * part;
    const _Float16 hi = static_cast<_Float16>(half_sum);
    const uint32_t at = (g >> 5) * 16u + ((g >> 2) & 7u);
    sums[at] = hi;
    sums[at + 8u] = static_cast<_Float16>(half_sum - static_cast<float>(hi));
  }
}

// The sort and the fp16 copy of the token rows do not depend on each other: workgroup 0 sorts,
// workgroup 1 + r converts row r of x (as rows_to_f16_kernel does: divided by the row's
// power-of-two scale, groups of 8 in the order the weight decode yields).
__global__ __launch_bounds__(1024) void moe_prepare_kernel(const uint32_t* __restrict__ ids, uint32_t pairs,
                                                           uint32_t experts, uint32_t* __restrict__ seg,
                                                           uint32_t* __restrict__ pos, uint32_t* __restrict__ inv,
                                                           const float* __restrict__ x, _Float16* __restrict__ a16,
                                                           _Float16* __restrict__ a_sums, float* __restrict__ a_scale,
                                                           uint32_t cols) {
  if (blockIdx.x == 0) {
    moe_sort_pairs(ids, pairs, experts, seg, pos, inv);
    return;
  }
  __shared__ float red[16];
  const uint32_t row = blockIdx.x - 1u, t = threadIdx.x;
  const float4* in = reinterpret_cast<const float4*>(x + static_cast<size_t>(row) * cols);
  float amax = 0.0f;
  for (uint32_t g = t; g < cols / 4u; g += 1024u) {
    const float4 v = in[g];
    amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fmaxf(fabsf(v.z), fabsf(v.w)), amax));
  }
  amax = wave_max(amax);
  if ((t & 63u) == 0) red[t >> 6] = amax;
  __syncthreads();
  amax = red[0];
#pragma unroll
  for (int w = 1; w < 16; ++w) amax = fmaxf(amax, red[w]);
  const float s = row_scale_for(amax), inv_s = 1.0f / s;
  half8_t* out = reinterpret_cast<half8_t*>(a16 + static_cast<size_t>(row) * cols);
  _Float16* sums = a_sums + static_cast<size_t>(row) * (cols / 16u);
  for (uint32_t g = t; g < cols / 8u; g += 1024u) {
    const half8_t v = to_f16_group(in[2 * g], in[2 * g + 1], inv_s);
    out[g] = v;
    store_subblock_sum(v, g, sums);
  }
  if (t == 0) a_scale[row] = s;
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

// ---- the chunk path for experts whose inner width fits LDS: two kernels ----------------------
// Both take 32 rows of an expert a pass and 32 columns a compute wavefront (so every weight is
// decoded once), stream raw super-blocks through a ring of S LDS stages with one barrier per
// super-block, and address rows through `inv` (sorted position -> pair), so no operand is
// gathered or scattered by a separate pass.  The direct loads are all issued by one extra
// wavefront that computes nothing: a CU accepts only so many vector-memory instructions at a
// time, a wavefront that issues into a full queue stands still until they are taken, and a
// wavefront that stores results must otherwise wait for its stores whenever it waits for loads
// (one counter covers both).  Measured on the 256-expert shape: the weight stream alone takes
// 68 us (gate and up) and 43 us (down), the arithmetic alone 24 and 12 us; with every
// wavefront loading its share the two added up.
template <int WAVES>
struct MoeTile {
  static constexpr uint32_t kBN = WAVES * 32u;                   // columns of a workgroup's tile
  static constexpr int kWBlocks = kBN * 144u / 1024u;            // 1 KB loads of a weight stage (exact)
  static constexpr uint32_t kWStage = kWBlocks * 1024u;
  static constexpr int kABlocks = 17;                            // 1 KB loads of an activation stage
  static constexpr uint32_t kARows = 32u * 512u;                 // one super-block of K for 32 rows, fp16 ...
  static constexpr uint32_t kAStage = kARows + 1024u;            // ... and the rows' 16 sub-block sums
  static constexpr uint32_t kThreads = (WAVES + 1) * 64u;        // compute wavefronts and the loader
  static_assert(kBN * 144u % 1024u == 0, "tile shape");
};

// The loader's source offsets of a weight stage: load b is chunks 64 b .. 64 b + 63 of the
// tile's 144-byte row pieces laid end to end (chunk q = 9 * row + part).
template <int WAVES>
__device__ __forceinline__ void moe_weight_offsets(uint32_t lane, uint32_t row_bytes, uint32_t (&src)[MoeTile<WAVES>::kWBlocks]) {
#pragma unroll
  for (int b = 0; b < MoeTile<WAVES>::kWBlocks; ++b) {
    const uint32_t q = b * 64u + lane;
    src[b] = (q / 9u) * row_bytes + (q % 9u) * 16u;
  }
}

template <int WAVES>
__device__ __forceinline__ void moe_issue_weights(const uint8_t* g, const uint32_t (&src)[MoeTile<WAVES>::kWBlocks],
                                                  uint32_t lds_stage) {
#pragma unroll
  for (int b = 0; b < MoeTile<WAVES>::kWBlocks; ++b) direct_load16(g, src[b], lds_stage + b * 1024u);
}

// The loader's barrier: at most BEHIND younger loads may still be in flight (loads complete in
// order), so the next stage has landed.  The compute wavefronts' barrier: their LDS reads of the
// stage they leave are done.
template <int BEHIND>
__device__ __forceinline__ void moe_loader_barrier(bool ring_full) {
  static_assert(BEHIND < 64, "vmcnt field");
  if (ring_full) {
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(BEHIND) : "memory");
  } else {
    asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  }
}
__device__ __forceinline__ void moe_compute_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One super-block (256 K values) of the (32 RT) x 32 product of a wavefront, added to `acc`.
//
// A Q4_K weight is d sc q - dmin mn (src/core/numerics/quant.cpp:656-675).  The matrix cores take
// q sc undecoded: an integer n < 2048 written into a 16-bit half IS the fp16 number n 2^-24
// (subnormal below 1024, the first normal binade above), so one 24-bit multiply of a masked
// nibble pair by the 6-bit scale makes two exact operands (q sc <= 945), and d is applied once to
// the block's sums.  The min term leaves the K loop: sum_k a_k dmin mn = sum_sb (dmin mn_sb) S_sb
// with S_sb the sum of the row's activations over sub-block sb, a 16-deep product of the rows'
// sums (fp16 hi/lo pairs, half the sum each, made where the fp16 rows are made) with 2 dmin mn
// (fp16 hi/lo pairs, exact: 11 x 6 bits); the lo x lo products (2^-22 of the term) are dropped.
// No weight is rounded, and the vector work per weight pair is a mask and a multiply (the
// v_fma_mixlo/hi_f16 pair that forms a rounded fp16 weight issues at half rate).
//
// `raw` is the lane's weight row in the raw stage, a_chunk(c) the address of 16-byte chunk c
// (8 K values) of the lane's activation row in the first 32 rows, `tile_bytes` the distance to
// the same row of the next 32; `sums` the lane's 16 bytes of its row's sums (hi for kg 0, lo for
// kg 1), `sums_tile_bytes` the distance to the next 32 rows' sums.  Every LDS read is requested
// well before its use: the lane's 80 bytes of the weight row, the sums and the first activation
// fragments up front, the fragments and quant words of a step one step before it (the scheduling
// barrier keeps them there).
template <int RT, typename AChunk>
__device__ __forceinline__ void moe_block_mma(const uint8_t* raw, uint32_t kg, AChunk&& a_chunk, uint32_t tile_bytes,
                                              const uint8_t* sums, uint32_t sums_tile_bytes, float16_t (&acc)[RT]) {
  const uint4 head_words = *reinterpret_cast<const uint4*>(raw);
  half8_t row_sums[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) row_sums[rt] = *reinterpret_cast<const half8_t*>(sums + rt * sums_tile_bytes);
  // Quant words of sub-block pair g (bytes 32 g + 8 kg + [0,8) and the same + 16 of the row's
  // quants) and the activation fragments of step j = 2 sb + tt, both fetched one step ahead.
  uint32_t q_next[4];
  auto load_q = [&](int g) {
    const uint8_t* qp = raw + 16 + g * 32 + kg * 8u;
    const uint2 q0 = *reinterpret_cast<const uint2*>(qp), q1 = *reinterpret_cast<const uint2*>(qp + 16);
    q_next[0] = q0.x, q_next[1] = q0.y, q_next[2] = q1.x, q_next[3] = q1.y;
  };
  half8_t a_next[RT];
  auto load_a = [&](int j) {
    const uint8_t* a = a_chunk((j >> 1) * 4u + (j & 1) * 2u + kg);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) a_next[rt] = *reinterpret_cast<const half8_t*>(a + rt * tile_bytes);
  };
  load_q(0);
  load_a(0);

  const float d24 = half_bits_to_float(head_words.x & 0xFFFFu) * 0x1p24f;
  const float ndmin2 = -2.0f * half_bits_to_float(head_words.x >> 16);
  const ScaleBytes sbytes = unpack_scales(head_words.y, head_words.z, head_words.w);

  // The min term: -2 dmin mn_sb as hi + lo (exact), hi against the sums' hi and lo, lo against
  // the sums' hi only (lanes of K half 1 hold the sums' lo and get zeros).
  {
    half8_t min_hi, min_lo;
#pragma unroll
    for (int sb = 0; sb < 8; ++sb) {
      const float p = static_cast<float>((sbytes.mn[sb >> 2] >> (8 * (sb & 3))) & 0xFFu) * ndmin2;
      const _Float16 hi = static_cast<_Float16>(p);
      min_hi[sb] = hi;
      min_lo[sb] = kg == 0 ? static_cast<_Float16>(p - static_cast<float>(hi)) : static_cast<_Float16>(0.0f);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      acc[rt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(row_sums[rt], min_hi, acc[rt], 0, 0, 0);
      acc[rt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(row_sums[rt], min_lo, acc[rt], 0, 0, 0);
    }
  }
  __builtin_amdgcn_sched_barrier(0);

  // The main term: sum_k a_k (q sc)_k 2^-24 over the block, then times d 2^24.
  float16_t blk[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int e = 0; e < 16; ++e) blk[rt][e] = 0.0f;
  }
  uint32_t qw[4];
  unrolled<16>([&](auto step) {
    constexpr int j = decltype(step)::value, sb = j >> 1, tt = j & 1;
    half8_t a_cur[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) a_cur[rt] = a_next[rt];
    if (j % 4 == 0) {   // an even sub-block brings the words; its odd successor takes their high nibbles
#pragma unroll
      for (int x = 0; x < 4; ++x) qw[x] = q_next[x];
      if (j < 12) load_q(j / 4 + 1);
    }
    if (j < 15) load_a(j + 1);
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t sc = (sbytes.sc[sb >> 2] >> (8 * (sb & 3))) & 0xFFu;
    // bytes 0 and 2 of a word are weights (k0, k2), bytes 1 and 3 (the word shifted down a byte)
    // (k1, k3): the order the fp16 rows are stored in
    auto pair = [&](uint32_t x, uint32_t down) { return __umul24((x >> (down + ((sb & 1) ? 4u : 0u))) & 0x000F000Fu, sc); };
    const uint4 words = make_uint4(pair(qw[2 * tt], 0u), pair(qw[2 * tt], 8u), pair(qw[2 * tt + 1], 0u), pair(qw[2 * tt + 1], 8u));
    const half8_t b = bit_cast<half8_t>(words);
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) blk[rt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_cur[rt], b, blk[rt], 0, 0, 0);
  });
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[rt][e] = fmaf(d24, blk[rt][e], acc[rt][e]);
  }
}

template <int RT>
__device__ __forceinline__ void zero_acc(float16_t (&acc)[RT]) {
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[rt][e] = 0.0f;
  }
}

// LDS of the gate/up kernel: a ring of three stages for passes of 32 rows, of two for 64.
template <int WAVES>
constexpr uint32_t moe_gate_up_ring_bytes() {
  using T = MoeTile<WAVES>;
  constexpr uint32_t one = 3u * (T::kAStage + T::kWStage), two = 2u * (2u * T::kAStage + T::kWStage);
  return one > two ? one : two;
}

struct MoeRowTables {
  alignas(16) uint32_t tok[64];
  alignas(16) uint32_t dst[64];
  alignas(16) float scale[64];
};

// One pass of moe_gate_up_kernel: rows m0 .. m0 + live of the sorted pairs (live <= 32 RT) against
// the workgroup's column tile, gate over all of K and then up, through a ring of S stages.
template <int WAVES, int S, int RT>
__device__ __forceinline__ void moe_gate_up_pass(uint8_t* lds, MoeRowTables& rows, const _Float16* __restrict__ a16,
                                                 const _Float16* __restrict__ a_sums, const float* __restrict__ a_scale,
                                                 const uint8_t* __restrict__ gate_e,
                                                 const uint8_t* __restrict__ up_e, float* __restrict__ phi,
                                                 const uint32_t* __restrict__ inv, uint32_t n, uint32_t k, uint32_t top_k,
                                                 uint32_t col0, uint32_t m0, uint32_t live) {
  using T = MoeTile<WAVES>;
  constexpr int kABlocks = T::kABlocks * RT, kRowBlocks = 16 * RT;   // 1 KB loads of a stage: all, rows only
  constexpr uint32_t kAStage = T::kAStage * RT;
  constexpr int kLoads = kABlocks + T::kWBlocks;   // of one stage
  static_assert(S == 2 || (S - 2) * kLoads < 64, "the loader's wait counts at most 63 loads");
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t row_blocks = k / 256u, row_bytes = row_blocks * 144u;
  const uint32_t total = 2u * row_blocks;
  const uint32_t lds_a = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)lds));
  const uint32_t lds_w = lds_a + S * kAStage;

  if (t < 32u * RT) {   // rows past the segment repeat its last row (computed, never stored)
    const uint32_t p = inv[m0 + (t < live ? t : live - 1u)];
    rows.tok[t] = p / top_k;
    rows.dst[t] = p;
    rows.scale[t] = a_scale[p / top_k];
  }
  __syncthreads();

  // Stage of iteration `it` is it % S.  Before iteration `it` the loads of it .. it + S - 2 are
  // issued and stage it has landed; during it the loader issues it + S - 1 into the stage every
  // wavefront left at the last barrier, then waits for it + 1.
  if (wave == WAVES) {
    // The offsets are the same in every pass; computed again behind an opaque copy of the lane
    // number, they do not sit in registers (of every wavefront) from one pass to the next.
    uint32_t ll = lane;
    asm volatile("" : "+v"(ll));
    uint32_t w_src[T::kWBlocks], a_src[kABlocks];
    moe_weight_offsets<WAVES>(ll, row_bytes, w_src);
    // Activation stage = 32 RT rows x 512 bytes, loaded as blocks of two rows; chunk c of row r
    // sits at position c ^ (r % 32) of the row, so that the 32 lanes of an MFMA operand read
    // (same chunk, 32 rows) touch every bank once.  Then the rows' sub-block sums, 32 bytes a
    // row: one load per 32 rows.
#pragma unroll
    for (int i = 0; i < kRowBlocks; ++i) {
      const uint32_t row = 2u * i + ll / 32u;
      a_src[i] = rows.tok[row] * (k * 2u) + (((ll % 32u) ^ (row & 31u)) * 16u);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) a_src[kRowBlocks + rt] = rows.tok[rt * 32u + ll / 2u] * (row_blocks * 32u) + (ll % 2u) * 16u;
    auto issue = [&](uint32_t it, uint32_t stage) {
      const uint32_t blk = it < row_blocks ? it : it - row_blocks;
      const uint8_t* ga = reinterpret_cast<const uint8_t*>(a16) + blk * 512u;
      const uint8_t* gs = reinterpret_cast<const uint8_t*>(a_sums) + blk * 32u;
#pragma unroll
      for (int i = 0; i < kRowBlocks; ++i) direct_load16(ga, a_src[i], lds_a + stage * kAStage + i * 1024u);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) direct_load16(gs, a_src[kRowBlocks + rt], lds_a + stage * kAStage + (kRowBlocks + rt) * 1024u);
      moe_issue_weights<WAVES>((it < row_blocks ? gate_e : up_e) + blk * 144u, w_src, lds_w + stage * T::kWStage);
    };
#pragma unroll
    for (int s = 0; s < S - 1; ++s) {
      if (static_cast<uint32_t>(s) < total) issue(s, s);
    }
    moe_loader_barrier<(S - 2) * kLoads>(total >= static_cast<uint32_t>(S - 1));
    uint32_t stage = 0;
    for (uint32_t it = 0; it < total; ++it) {
      const bool more = it + (S - 1) < total;
      if (more) issue(it + (S - 1), stage == 0 ? S - 1 : stage - 1u);
      moe_loader_barrier<(S - 2) * kLoads>(more);
      stage = stage + 1u == S ? 0u : stage + 1u;
    }
  } else {
    const uint32_t l32 = lane & 31u, kg = lane >> 5;
    const uint8_t* w_lane = lds + S * kAStage + (wave * 32u + l32) * 144u;
    const uint8_t* a_lane = lds + l32 * 512u;
    const uint8_t* s_lane = lds + kRowBlocks * 1024u + l32 * 32u + kg * 16u;
    float16_t acc[RT], acc_gate[RT];
    uint32_t stage = 0;
    moe_compute_barrier();
    auto run = [&]() {   // one tensor
      zero_acc<RT>(acc);
      for (uint32_t blk = 0; blk < row_blocks; ++blk) {
        moe_block_mma<RT>(w_lane + stage * T::kWStage, kg,
                          [&](uint32_t c) { return a_lane + stage * kAStage + ((c ^ l32) * 16u); }, T::kARows,
                          s_lane + stage * kAStage, 1024u, acc);
        moe_compute_barrier();
        stage = stage + 1u == S ? 0u : stage + 1u;
      }
    };
    run();
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) acc_gate[rt] = acc[rt];
    run();

    // lane holds column `col` and rows 32 rt + 8 g + 4 kg + [0,4), g = 0..3: four table entries a read
    const uint32_t col = col0 + wave * 32u + l32;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
      for (int g4 = 0; g4 < 4; ++g4) {
        const uint32_t row0 = rt * 32u + g4 * 8u + kg * 4u;
        const uint4 dst4 = *reinterpret_cast<const uint4*>(rows.dst + row0);
        const float4 sc4 = *reinterpret_cast<const float4*>(rows.scale + row0);
        const uint32_t dst[4] = {dst4.x, dst4.y, dst4.z, dst4.w};
        const float sc[4] = {sc4.x, sc4.y, sc4.z, sc4.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (row0 + i < live) {
            const float g = acc_gate[rt][g4 * 4 + i] * sc[i], u = acc[rt][g4 * 4 + i] * sc[i];
            phi[static_cast<size_t>(dst[i]) * n + col] = (g / (1.0f + expf(-g))) * u;
          }
        }
      }
    }
  }
  __syncthreads();   // the row tables and the ring are rewritten by the next pass
}

// phi[p][c] = silu((gate_e x_t)(c)) * (up_e x_t)(c) for the pairs p = (t, slot) of expert e and
// the columns of the workgroup's tile, written in pair order as fp32.  x comes as one fp16 copy
// per token (a16, scale a_scale): the direct loads of a pass fetch the tokens of its pairs.
// Gate runs over all of K, then up; the gate sums wait in registers.  An expert with more than
// 32 pairs left takes 64 a pass (two row tiles against one decode of the weights, ring of two
// stages), so that its weights are read and decoded once for up to 64 pairs.
template <int WAVES>
__global__ __launch_bounds__((WAVES + 1) * 64) void moe_gate_up_kernel(
    const _Float16* __restrict__ a16, const _Float16* __restrict__ a_sums, const float* __restrict__ a_scale,
    const uint8_t* __restrict__ gate, const uint8_t* __restrict__ up, uint64_t gate_stride, uint64_t up_stride,
    float* __restrict__ phi,
    const uint32_t* __restrict__ seg, const uint32_t* __restrict__ inv, uint32_t n, uint32_t k, uint32_t experts,
    uint32_t top_k) {
  using T = MoeTile<WAVES>;
  __shared__ __attribute__((aligned(16))) uint8_t lds[moe_gate_up_ring_bytes<WAVES>()];
  __shared__ MoeRowTables rows;
  // Grid as in q4k_gemm_grouped_kernel: an expert's tiles on one XCD, adjacent in dispatch order.
  const uint32_t tiles = n / T::kBN;
  const uint32_t slot = blockIdx.x / 8u;
  const uint32_t e = (slot / tiles) * 8u + blockIdx.x % 8u, tile = slot % tiles;
  if (e >= experts) return;
  const uint32_t r0 = seg[e], r1 = seg[e + 1];
  if (r1 <= r0) return;
  const size_t tile_off = static_cast<size_t>(tile) * T::kBN * (k / 256u * 144u);
  const uint8_t* gate_e = gate + e * gate_stride + tile_off;
  const uint8_t* up_e = up + e * up_stride + tile_off;
  for (uint32_t m0 = r0; m0 < r1;) {
    const uint32_t left = r1 - m0;
    if (left > 32u) {
      moe_gate_up_pass<WAVES, 2, 2>(lds, rows, a16, a_sums, a_scale, gate_e, up_e, phi, inv, n, k, top_k, tile * T::kBN, m0,
                                    left < 64u ? left : 64u);
      m0 += 64u;
    } else {
      moe_gate_up_pass<WAVES, 3, 1>(lds, rows, a16, a_sums, a_scale, gate_e, up_e, phi, inv, n, k, top_k, tile * T::kBN, m0, left);
      m0 += 32u;
    }
  }
}

// Dynamic LDS of the down kernel for passes of 32 RT rows: S weight stages, the row tables, the
// rows as fp16 (2k + 16 bytes each), their sub-block sums (k / 8 bytes each).
template <int WAVES>
__host__ __device__ constexpr size_t moe_down_lds_bytes(int stages, int rt, uint32_t inter) {
  return static_cast<size_t>(stages) * MoeTile<WAVES>::kWStage + 256u * rt +
         32u * rt * (2u * static_cast<size_t>(inter) + 16u + inter / 8u);
}

// One pass of moe_down_kernel: rows m0 .. m0 + live of the sorted pairs (live <= 32 RT) against
// column tiles tile0 .. tile1 of expert e.
template <int WAVES, int S, int RT>
__device__ __forceinline__ void moe_down_pass(uint8_t* dyn_lds, const float* __restrict__ phi,
                                              const uint8_t* __restrict__ down_e, float* __restrict__ rows,
                                              const uint32_t* __restrict__ inv, uint32_t n, uint32_t k, uint32_t tile0,
                                              uint32_t tile1, uint32_t m0, uint32_t live) {
  using T = MoeTile<WAVES>;
  float* row_scale = reinterpret_cast<float*>(dyn_lds + S * T::kWStage);
  uint32_t* row_dst = reinterpret_cast<uint32_t*>(dyn_lds + S * T::kWStage + 128 * RT);
  uint8_t* a_lds = dyn_lds + S * T::kWStage + 256 * RT;
  const uint32_t a_stride = 2u * k + 16u, sums_stride = k / 8u;
  uint8_t* sums_lds = a_lds + 32u * RT * a_stride;
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t row_blocks = k / 256u, row_bytes = row_blocks * 144u;
  const uint32_t total = (tile1 - tile0) * row_blocks;
  const uint32_t lds_w = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) uint8_t*)dyn_lds));

  // Iteration `it` is block it % row_blocks of tile tile0 + it / row_blocks; stages and waits
  // as in moe_gate_up_pass.  The loader requests the first weight stages while the other
  // wavefronts stage the rows.
  if (wave == WAVES) {
    uint32_t ll = lane;   // as in moe_gate_up_pass
    asm volatile("" : "+v"(ll));
    uint32_t w_src[T::kWBlocks];
    moe_weight_offsets<WAVES>(ll, row_bytes, w_src);
    uint32_t tile_i = tile0, blk_i = 0;   // S - 1 iterations ahead
    auto issue_next = [&](uint32_t stage) {
      moe_issue_weights<WAVES>(down_e + static_cast<size_t>(tile_i) * T::kBN * row_bytes + blk_i * 144u, w_src,
                               lds_w + stage * T::kWStage);
      if (++blk_i == row_blocks) blk_i = 0, ++tile_i;
    };
#pragma unroll
    for (int s = 0; s < S - 1; ++s) {
      if (static_cast<uint32_t>(s) < total) issue_next(s);
    }
    asm volatile("s_barrier" ::: "memory");   // the rows are staged; the weight loads stay in flight
    moe_loader_barrier<(S - 2) * T::kWBlocks>(total >= static_cast<uint32_t>(S - 1));
    uint32_t stage = 0;
    for (uint32_t it = 0; it < total; ++it) {
      const bool more = it + (S - 1) < total;
      if (more) issue_next(stage == 0 ? S - 1 : stage - 1u);
      moe_loader_barrier<(S - 2) * T::kWBlocks>(more);
      stage = stage + 1u == S ? 0u : stage + 1u;
    }
  } else {
    // The fp16 copy of the pass's rows: the compute wavefronts' (WAVES * 2) threads a row take its
    // largest magnitude, then write the groups of 8 in the order the decode yields.
    constexpr uint32_t kPer = WAVES * 2u;
    uint32_t tc = t;   // opaque, so that nothing derived from it is kept in registers between passes
    asm volatile("" : "+v"(tc));
#pragma nounroll
    for (int rt = 0; rt < RT; ++rt) {
      const uint32_t row = rt * 32u + tc / kPer, sub = tc % kPer;
      const uint32_t p = inv[m0 + (row < live ? row : live - 1u)];
      const float4* src = reinterpret_cast<const float4*>(phi + static_cast<size_t>(p) * k);
      float amax = 0.0f;
      for (uint32_t c = sub; c < k / 4u; c += kPer) {
        const float4 v = src[c];
        amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fmaxf(fabsf(v.z), fabsf(v.w)), amax));
      }
#pragma unroll
      for (uint32_t d = 1; d < kPer; d *= 2u) amax = fmaxf(amax, __shfl_xor(amax, d));
      const float s = row_scale_for(amax), inv_s = 1.0f / s;
      for (uint32_t c = sub; c < k / 8u; c += kPer) {   // neighbouring threads hold neighbouring groups
        const half8_t v = to_f16_group(src[2 * c], src[2 * c + 1], inv_s);
        *reinterpret_cast<half8_t*>(a_lds + row * a_stride + c * 16u) = v;
        store_subblock_sum(v, c, reinterpret_cast<_Float16*>(sums_lds + row * sums_stride));
      }
      if (sub == 0) row_scale[row] = s, row_dst[row] = p;
    }
    moe_compute_barrier();   // the staged rows
    uint32_t lc = lane;   // as the loader's copy
    asm volatile("" : "+v"(lc));
    const uint32_t l32 = lc & 31u, kg = lc >> 5;
    const uint8_t* w_lane = dyn_lds + (wave * 32u + l32) * 144u;
    const uint8_t* a_lane = a_lds + l32 * a_stride;
    const uint8_t* s_lane = sums_lds + l32 * sums_stride + kg * 16u;
    float16_t acc[RT];
    uint32_t stage = 0;
    moe_compute_barrier();
    for (uint32_t tile = tile0; tile < tile1; ++tile) {
      zero_acc<RT>(acc);
      for (uint32_t blk = 0; blk < row_blocks; ++blk) {
        moe_block_mma<RT>(w_lane + stage * T::kWStage, kg, [&](uint32_t c) { return a_lane + (blk * 32u + c) * 16u; },
                          32u * a_stride, s_lane + blk * 32u, 32u * sums_stride, acc);
        moe_compute_barrier();
        stage = stage + 1u == S ? 0u : stage + 1u;
      }
      // lane holds column `col` and rows 32 rt + 8 g + 4 kg + [0,4), g = 0..3: four table entries a read
      const uint32_t col = tile * T::kBN + wave * 32u + l32;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const uint32_t row0 = rt * 32u + g * 8u + kg * 4u;
          const uint4 dst4 = *reinterpret_cast<const uint4*>(row_dst + row0);
          const float4 sc4 = *reinterpret_cast<const float4*>(row_scale + row0);
          const uint32_t dst[4] = {dst4.x, dst4.y, dst4.z, dst4.w};
          const float sc[4] = {sc4.x, sc4.y, sc4.z, sc4.w};
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            if (row0 + i < live) rows[static_cast<size_t>(dst[i]) * n + col] = acc[rt][g * 4 + i] * sc[i];
          }
        }
      }
    }
  }
  __syncthreads();   // the rows, their tables and the ring are rewritten by the next pass
}

// rows[p][c] = (down_e phi[p])(c) for the pairs of expert e, in pair order as fp32.  The rows
// of a pass stay in LDS for the whole pass as fp16 under a power-of-two row scale (phi can
// exceed the fp16 range), converted here from the fp32 rows; the workgroup then streams the
// weights of `tiles_per_chunk` column tiles past them without a break between tiles.  A pass is
// 32 rows behind a ring of S stages, or (`wide`: the launch reserved the LDS for it) 64 rows
// behind a ring of two when the expert has more than 32 pairs left.
template <int WAVES, int S>
__global__ __launch_bounds__((WAVES + 1) * 64) void moe_down_kernel(
    const float* __restrict__ phi, const uint8_t* __restrict__ down, uint64_t down_stride, float* __restrict__ rows,
    const uint32_t* __restrict__ seg, const uint32_t* __restrict__ inv, uint32_t n, uint32_t k, uint32_t experts,
    uint32_t chunks, uint32_t tiles_per_chunk, bool wide) {
  using T = MoeTile<WAVES>;
  extern __shared__ __attribute__((aligned(16))) uint8_t dyn_lds[];
  const uint32_t tiles = n / T::kBN;
  const uint32_t slot = blockIdx.x / 8u;
  const uint32_t e = (slot / chunks) * 8u + blockIdx.x % 8u;
  const uint32_t tile0 = (slot % chunks) * tiles_per_chunk;
  if (e >= experts || tile0 >= tiles) return;
  const uint32_t tile1 = tile0 + tiles_per_chunk < tiles ? tile0 + tiles_per_chunk : tiles;
  const uint32_t r0 = seg[e], r1 = seg[e + 1];
  if (r1 <= r0) return;
  const uint8_t* down_e = down + e * down_stride;
  for (uint32_t m0 = r0; m0 < r1;) {
    const uint32_t left = r1 - m0;
    if (wide && left > 32u) {
      moe_down_pass<WAVES, 2, 2>(dyn_lds, phi, down_e, rows, inv, n, k, tile0, tile1, m0, left < 64u ? left : 64u);
      m0 += 64u;
    } else {
      moe_down_pass<WAVES, S, 1>(dyn_lds, phi, down_e, rows, inv, n, k, tile0, tile1, m0, left < 32u ? left : 32u);
      m0 += 32u;
    }
  }
}

// out[t][j] (+)= sum_slot wts[t][slot] * rows[t * top_k + slot][j], slots in order, four columns a thread.
__global__ __launch_bounds__(256) void moe_combine_pairs_kernel(const float4* __restrict__ rows, const float* __restrict__ wts,
                                                                float4* __restrict__ out, uint32_t tokens, uint32_t top_k,
                                                                uint32_t hidden4, bool accumulate) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (i >= static_cast<uint64_t>(tokens) * hidden4) return;
  const uint32_t t = static_cast<uint32_t>(i / hidden4), j = static_cast<uint32_t>(i % hidden4);
  float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  for (uint32_t s = 0; s < top_k; ++s) {
    const float w = wts[t * top_k + s];
    const float4 r = rows[static_cast<size_t>(t * top_k + s) * hidden4 + j];
    acc.x += w * r.x, acc.y += w * r.y, acc.z += w * r.z, acc.w += w * r.w;
  }
  if (accumulate) {
    const float4 o = out[i];
    acc.x += o.x, acc.y += o.y, acc.z += o.z, acc.w += o.w;
  }
  out[i] = acc;
}

size_t align256(size_t v) { return (v + 255) & ~size_t{255}; }

constexpr size_t kMoeLdsLimit = 160 * 1024 - 64;

// The two-kernel path needs an expert's 32 rows of phi in LDS next to the weight ring (eight
// compute wavefronts and three stages up to an inner width of 768, four and two up to 1792),
// whole column tiles, and 32-bit byte offsets into the fp16 token copy.
bool moe_resident_path(uint32_t hidden, uint32_t inter, uint32_t tokens) {
  return moe_down_lds_bytes<4>(2, 1, inter) <= kMoeLdsLimit && static_cast<uint64_t>(tokens) * hidden * 2 < (1ull << 32);
}

void launch_moe_gate_up_resident(const _Float16* a16, const _Float16* a_sums, const float* a_scale, const uint8_t* gate,
                                 const uint8_t* up,
                                 uint64_t gate_stride, uint64_t up_stride, float* phi, const uint32_t* seg,
                                 const uint32_t* inv, uint32_t hidden, uint32_t inter, uint32_t experts, uint32_t top_k,
                                 hipStream_t stream) {
  const uint32_t expert_groups = (experts + 7u) / 8u * 8u;
  hipLaunchKernelGGL((moe_gate_up_kernel<8>), dim3(expert_groups * (inter / 256u)), dim3(MoeTile<8>::kThreads), 0, stream, a16, a_sums, a_scale,
                     gate, up, gate_stride, up_stride, phi, seg, inv, inter, hidden, experts, top_k);
}

template <int WAVES, int S>
void launch_moe_down_tiles(const float* phi, const uint8_t* down, uint64_t down_stride, float* rows, const uint32_t* seg,
                           const uint32_t* inv, uint32_t hidden, uint32_t inter, uint32_t experts, uint32_t per_cu,
                           hipStream_t stream) {
  // As many column chunks per expert as give every CU its `per_cu` workgroups.
  const uint32_t tiles = hidden / MoeTile<WAVES>::kBN;
  const uint32_t want = (per_cu * static_cast<uint32_t>(num_cus()) + experts - 1u) / experts;
  const uint32_t chunks = want < 1u ? 1u : want > tiles ? tiles : want;
  const uint32_t tiles_per_chunk = (tiles + chunks - 1u) / chunks;
  const uint32_t expert_groups = (experts + 7u) / 8u * 8u;
  // 64-row passes where their rows fit next to a ring of two stages
  const size_t narrow = moe_down_lds_bytes<WAVES>(S, 1, inter), wide_bytes = moe_down_lds_bytes<WAVES>(2, 2, inter);
  const bool wide = wide_bytes <= kMoeLdsLimit;
  const size_t lds_bytes = wide && wide_bytes > narrow ? wide_bytes : narrow;
  hipLaunchKernelGGL((moe_down_kernel<WAVES, S>), dim3(expert_groups * chunks), dim3(MoeTile<WAVES>::kThreads), lds_bytes, stream, phi,
                     down, down_stride, rows, seg, inv, hidden, inter, experts, chunks, tiles_per_chunk, wide);
}

void launch_moe_down_resident(const float* phi, const uint8_t* down, uint64_t down_stride, float* rows, const uint32_t* seg,
                              const uint32_t* inv, uint32_t hidden, uint32_t inter, uint32_t experts, hipStream_t stream) {
  if (moe_down_lds_bytes<8>(3, 1, inter) <= kMoeLdsLimit) {
    launch_moe_down_tiles<8, 3>(phi, down, down_stride, rows, seg, inv, hidden, inter, experts, 1u, stream);
  } else {
    launch_moe_down_tiles<4, 2>(phi, down, down_stride, rows, seg, inv, hidden, inter, experts, 1u, stream);
  }
}

}  // namespace

bool moe_ffn_q4k_supported(uint64_t hidden, uint64_t inter, uint64_t experts) {
  return hidden % 256 == 0 && inter % 256 == 0 && hidden <= (1u << 16) && inter <= (1u << 16) && experts >= 1 &&
         experts <= 1024;
}

hipError_t moe_q4k_prepare() {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_down_kernel<8, 3>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kMoeLdsLimit));
  if (e != hipSuccess) return e;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_down_kernel<4, 2>), hipFuncAttributeMaxDynamicSharedMemorySize,
                             static_cast<int>(kMoeLdsLimit));
}

namespace {

// The workspace, carved the same way by the three entry points (each uses the parts it needs).
struct MoeWorkspace {
  uint32_t *seg, *pos, *inv;
  float *x_scale, *phi_scale;
  _Float16* a16;      // fp16 rows of x: one per token (resident path) or one per pair, gathered
  _Float16* a_sums;   // resident path: the token rows' sub-block sums, hidden / 16 halves a row
  float *g, *u;       // pairs x inter each; g doubles as phi (fp32, pair order) on the resident path
  _Float16* phi16;
  float* rows;        // pairs x hidden
  size_t bytes;
};
MoeWorkspace carve_moe_workspace(void* workspace, uint64_t pairs, uint64_t hidden, uint64_t inter, uint64_t experts) {
  uint8_t* const base = static_cast<uint8_t*>(workspace);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    uint8_t* p = base + off;
    off += align256(bytes);
    return p;
  };
  MoeWorkspace w;
  w.seg = reinterpret_cast<uint32_t*>(take((experts + 1) * 4));
  w.pos = reinterpret_cast<uint32_t*>(take(pairs * 4));
  w.inv = reinterpret_cast<uint32_t*>(take(pairs * 4));
  w.x_scale = reinterpret_cast<float*>(take((pairs + 256) * 4));
  w.phi_scale = reinterpret_cast<float*>(take((pairs + 256) * 4));
  w.a16 = reinterpret_cast<_Float16*>(take(pairs * hidden * 2));
  w.a_sums = reinterpret_cast<_Float16*>(take(pairs * hidden / 8));
  w.g = reinterpret_cast<float*>(take(pairs * inter * 4));
  w.u = reinterpret_cast<float*>(take(pairs * inter * 4));
  w.phi16 = reinterpret_cast<_Float16*>(take(pairs * inter * 2));
  w.rows = reinterpret_cast<float*>(take(pairs * hidden * 4));
  w.bytes = off;
  return w;
}

void launch_grouped(const _Float16* a16, const float* a_scale, const uint8_t* w, float* c, const uint32_t* seg,
                    uint64_t w_stride, uint32_t n, uint32_t k, uint32_t experts, const uint8_t* w2, float* c2,
                    uint64_t w2_stride, hipStream_t stream) {
  constexpr int BM = 32, BN = 64;
  const uint32_t expert_groups = (experts + 7u) / 8u * 8u, tensors = w2 != nullptr ? 2u : 1u;
  hipLaunchKernelGGL((q4k_gemm_grouped_kernel<BM, BN>), dim3(expert_groups * ((n + BN - 1) / BN) * tensors), dim3(BN * 2), 0,
                     stream, a16, a_scale, w, c, seg, w_stride, n, k, experts, tensors, w2, c2, w2_stride);
}

void launch_combine(const float* rows, const float* wts, float* out, uint32_t tokens, uint32_t top_k, uint32_t hidden,
                    bool accumulate, hipStream_t stream) {
  const uint64_t outs = static_cast<uint64_t>(tokens) * (hidden / 4u);
  hipLaunchKernelGGL(moe_combine_pairs_kernel, dim3(static_cast<uint32_t>((outs + 255) / 256)), dim3(256), 0, stream,
                     reinterpret_cast<const float4*>(rows), wts, reinterpret_cast<float4*>(out), tokens, top_k, hidden / 4u,
                     accumulate);
}

}  // namespace

size_t moe_ffn_q4k_workspace_bytes(uint64_t pairs, uint64_t hidden, uint64_t inter, uint64_t experts) {
  return carve_moe_workspace(nullptr, pairs, hidden, inter, experts).bytes;
}

// Two regimes.  Experts whose inner width fits LDS (moe_resident_path): x as one fp16 row per
// token, moe_gate_up_kernel, moe_down_kernel, a combine over consecutive rows.  Wider experts:
// the pairs' rows gathered as fp16, grouped GEMM tiles with the activations streamed in slices
// (q4k_gemm_grouped_kernel), silu and the fp16 copy of phi as a pass of their own.
hipError_t launch_moe_ffn_q4k(const float* x, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                              const uint32_t* ids, const float* wts, float* out, void* workspace,
                              uint32_t hidden, uint32_t inter, uint32_t top_k, uint64_t gate_stride,
                              uint64_t up_stride, uint64_t down_stride, uint32_t experts, uint32_t tokens,
                              bool accumulate, hipStream_t stream) {
  const uint32_t pairs = tokens * top_k;
  const MoeWorkspace ws = carve_moe_workspace(workspace, pairs, hidden, inter, experts);
  if (moe_resident_path(hidden, inter, tokens)) {
    hipLaunchKernelGGL(moe_prepare_kernel, dim3(1u + tokens), dim3(1024), 0, stream, ids, pairs, experts, ws.seg, ws.pos,
                       ws.inv, x, ws.a16, ws.a_sums, ws.x_scale, hidden);
    launch_moe_gate_up_resident(ws.a16, ws.a_sums, ws.x_scale, gate, up, gate_stride, up_stride, ws.g, ws.seg, ws.inv, hidden, inter,
                                experts, top_k, stream);
    launch_moe_down_resident(ws.g, down, down_stride, ws.rows, ws.seg, ws.inv, hidden, inter, experts, stream);
    launch_combine(ws.rows, wts, out, tokens, top_k, hidden, accumulate, stream);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, ws.seg, ws.pos, ws.inv);
  launch_rows_to_f16(x, ws.a16, ws.x_scale, pairs, hidden, ws.pos, top_k, stream);
  launch_grouped(ws.a16, ws.x_scale, gate, ws.g, ws.seg, gate_stride, inter, hidden, experts, up, ws.u, up_stride, stream);
  hipLaunchKernelGGL(moe_silu_mul_kernel, dim3(pairs), dim3(256), 0, stream, ws.g, ws.u, ws.phi16, ws.phi_scale, inter);
  launch_grouped(ws.phi16, ws.phi_scale, down, ws.rows, ws.seg, down_stride, hidden, inter, experts, nullptr, nullptr, 0,
                 stream);
  const uint64_t outs = static_cast<uint64_t>(tokens) * hidden;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(static_cast<uint32_t>((outs + 255) / 256)), dim3(256), 0, stream, ws.rows,
                     ws.pos, wts, out, tokens, top_k, hidden, accumulate);
  return hipGetLastError();
}

// The two halves of launch_moe_ffn_q4k behind the reference's own pair of ids
// ("moe_experts_gate_up_q4k_rows" then "moe_experts_down_q4k_rows",
// src/backends/rocm/rocm_kernels_moe.cpp:15-79) for a chunk of tokens: each sorts the pairs by
// expert for itself, so an expert's weights are read once per launch instead of once per token
// that chose it.  phi keeps the caller's layout (tokens x top_k x inter, fp32) between the two.
// Workspace as for launch_moe_ffn_q4k.
hipError_t launch_moe_gate_up_q4k_grouped(const float* x, const uint8_t* gate, const uint8_t* up, const uint32_t* ids,
                                          float* phi, void* workspace, uint32_t hidden, uint32_t inter, uint32_t top_k,
                                          uint64_t gate_stride, uint64_t up_stride, uint32_t experts, uint32_t tokens,
                                          hipStream_t stream) {
  const uint32_t pairs = tokens * top_k;
  const MoeWorkspace ws = carve_moe_workspace(workspace, pairs, hidden, inter, experts);
  if (moe_resident_path(hidden, inter, tokens)) {
    hipLaunchKernelGGL(moe_prepare_kernel, dim3(1u + tokens), dim3(1024), 0, stream, ids, pairs, experts, ws.seg, ws.pos,
                       ws.inv, x, ws.a16, ws.a_sums, ws.x_scale, hidden);
    launch_moe_gate_up_resident(ws.a16, ws.a_sums, ws.x_scale, gate, up, gate_stride, up_stride, phi, ws.seg, ws.inv, hidden, inter,
                                experts, top_k, stream);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, ws.seg, ws.pos, ws.inv);
  launch_rows_to_f16(x, ws.a16, ws.x_scale, pairs, hidden, ws.pos, top_k, stream);
  launch_grouped(ws.a16, ws.x_scale, gate, ws.g, ws.seg, gate_stride, inter, hidden, experts, up, ws.u, up_stride, stream);
  hipLaunchKernelGGL(moe_silu_scatter_kernel, dim3(pairs), dim3(256), 0, stream, ws.g, ws.u, ws.pos, phi, inter);
  return hipGetLastError();
}

hipError_t launch_moe_down_q4k_grouped(const float* phi, const uint8_t* down, const uint32_t* ids, const float* wts,
                                       float* out, void* workspace, uint32_t hidden, uint32_t inter, uint32_t top_k,
                                       uint64_t down_stride, uint32_t experts, uint32_t tokens, bool accumulate,
                                       hipStream_t stream) {
  const uint32_t pairs = tokens * top_k;
  const MoeWorkspace ws = carve_moe_workspace(workspace, pairs, hidden, inter, experts);
  hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), 0, stream, ids, pairs, experts, ws.seg, ws.pos, ws.inv);
  if (moe_resident_path(hidden, inter, tokens)) {
    launch_moe_down_resident(phi, down, down_stride, ws.rows, ws.seg, ws.inv, hidden, inter, experts, stream);
    launch_combine(ws.rows, wts, out, tokens, top_k, hidden, accumulate, stream);
    return hipGetLastError();
  }
  // source row of pair p is p itself (phi is pair-major): top_k = 1 in the gather
  launch_rows_to_f16(phi, ws.phi16, ws.phi_scale, pairs, inter, ws.pos, 1u, stream);
  launch_grouped(ws.phi16, ws.phi_scale, down, ws.rows, ws.seg, down_stride, hidden, inter, experts, nullptr, nullptr, 0,
                 stream);
  const uint64_t outs = static_cast<uint64_t>(tokens) * hidden;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(static_cast<uint32_t>((outs + 255) / 256)), dim3(256), 0, stream, ws.rows,
                     ws.pos, wts, out, tokens, top_k, hidden, accumulate);
  return hipGetLastError();
}

}  // namespace qmm
