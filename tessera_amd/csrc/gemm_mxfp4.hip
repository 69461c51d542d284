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
// Shape of the kernel.  A workgroup owns a BM x BN tile of C (256 x 256 with eight
// wavefronts for prefill: 64 x 128 and 128 accumulator registers per wavefront, two
// wavefronts per SIMD so that one's LDS reads run under the other's MFMAs) and walks K in
// steps of 128.  Operand tiles travel HBM -> LDS directly (global_load_lds, 16 bytes a
// lane), never through registers, into a ring of three LDS stages: while step s is
// multiplied, the loads of steps s+1 and s+2 are in flight, about 96 KB per CU, which is
// what the memory latency under load (about 2 microseconds) times the consumption rate
// asks for.  A direct load lands lane p's 16 bytes at position p of a 1 KB block, so rows
// cannot be padded; instead each lane fetches the chunk whose index is XOR-swizzled with
// its row, and the fragment reads undo the swizzle.  With that, the 16-byte fragment
// reads of 16 consecutive rows fall on 16 distinct bank groups.  Workgroups are
// persistent (one per CU) and the ring runs across tile boundaries.

#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

constexpr int kMaxTerms = 4;                // E4M3 terms an fp32 activation is split into at most
constexpr int kKS = 128;                    // K per step: one 32-bit word of E8M0 bytes per weight row
constexpr int kDmaPerStage = 13;            // direct loads a wavefront issues per stage (8 A, 4 B, 1 scales)

// Direct HBM -> LDS load: lane p's `bytes` at global `base + voff` land at LDS address
// lds_addr + p * bytes (base and lds_addr wave-uniform).  Issued as inline assembly so
// that the waits stay under this file's control: the kernel waits for exactly the stage
// it is about to publish (vmcnt counts direct loads in order) and keeps two younger
// stages in flight across its LDS reads.
__device__ __forceinline__ void direct_load16(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}
__device__ __forceinline__ void direct_load4(const void* base, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
               :: "v"(voff), "s"(base), "s"(lds_addr) : "memory", "m0");
}

// SPLIT: the activation is a sum of E4M3 terms (see split_rows_kernel): a8 holds kMaxTerms
// planes of m x k codes, term t weighing 2^(-4t); `need` says how many terms each row has.  A
// tile walks K once per term it needs, all into the same accumulators, the term's weight being
// the E8M0 scale of the A operand.
//
// WPERM: the nibble bytes of W are in the reference's 16-row fragment order (PermuteMxFp4ToWmma,
// src/core/numerics/quant.cpp:926-954: dword (tile t, 16-wide K step s, half h, row r) at
// ((t * k/16 + s) * 2 + h) * 16 + r; the scales stay row-major).  The 16 rows x 128 K of one
// direct-load block are still 1 KB of contiguous memory, only transposed inside, so the block is
// fetched dword by dword (global_load_lds_dword), each lane asking for the dword that belongs at
// its LDS position: the LDS image, and everything after it, is the row-major one.
template <int BM, int BN, int WM, int WN, bool SPLIT, bool WPERM = false>
__global__ __launch_bounds__(64 * WM * WN) void mxfp4_a8_gemm_kernel(
    const uint8_t* __restrict__ a8, const float* __restrict__ as, const uint8_t* __restrict__ w,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k, uint32_t n_begin, uint32_t n_end,
    const uint8_t* __restrict__ need) {
  constexpr int kWaves = WM * WN;
  static_assert(BM % (32 * WM) == 0 && BN % (32 * WN) == 0 && BN % 64 == 0, "tile shape");
  static_assert((BM / 8) % kWaves == 0 && (BN / 16) % kWaves == 0, "direct-load blocks divide among the wavefronts");
  constexpr int kTI = BM / WM / 32, kTJ = BN / WN / 32;      // MFMA tiles per wavefront
  constexpr int kABlk = BM / 8 / kWaves, kBBlk = BN / 16 / kWaves;  // 1 KB direct-load blocks per wavefront
  constexpr int kBLoads = WPERM ? 4 : 1;                     // load instructions per weight block
  constexpr int kDma = kABlk + kBBlk * kBLoads + 1;          // direct loads a wavefront issues per stage
  constexpr uint32_t kBBase = BM * kKS, kSBase = kBBase + BN * kKS / 2;
  constexpr uint32_t kStage = kSBase + BN * 4;
  __shared__ __attribute__((aligned(16))) uint8_t lds[3 * kStage];

  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t wm = wave / WN, wn = wave % WN;
  const uint32_t l32 = lane & 31u, kg = lane >> 5;        // MFMA row/column and K half
  const uint32_t row_bytes = k / 2, row_blocks = k / 32;
  const uint32_t tiles_n = (n_end - n_begin + BN - 1) / BN;
  const uint32_t tiles = tiles_n * ((m + BM - 1) / BM);
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)lds));

  // Direct loads of one tile.  Activation block L (1 KB, rows 8L..8L+7, eight 16-byte chunks
  // a row): lane p fetches row 8L + p/8, chunk (p%8) ^ ((row>>1)&7).  Weight block L (rows
  // 16L..16L+15, four chunks a row): row 16L + p/4, chunk (p%4) ^ ((row>>2)&3).  Scale block
  // (64 rows, one word a row): row 64L + p.  A wavefront moves kABlk + kBBlk + 1 blocks per
  // stage; rows past the matrix edge are clamped to the last row (never stored).
  struct Source {
    const uint8_t *a, *b, *s;           // tile origins (wave-uniform)
    uint32_t a_off[kABlk], b_off[kBBlk][kBLoads], s_off;
    uint32_t terms;                     // passes over K (SPLIT)
  };
  const size_t plane = static_cast<size_t>(m) * k;
  // Terms the rows m0 .. m0 + BM - 1 need: the largest of their `need` bytes (wave-uniform).
  auto tile_terms = [&](uint32_t m0) -> uint32_t {
    if (!SPLIT) return 1u;
    float most = 1.0f;
#pragma unroll
    for (int i = 0; i < (BM + 63) / 64; ++i) {
      const uint32_t row = m0 + i * 64u + lane;
      if (i * 64u + lane < BM && row < m) most = fmaxf(most, static_cast<float>(need[row]));
    }
    const uint32_t terms = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(wave_max(most)));
    return terms < static_cast<uint32_t>(kMaxTerms) ? terms : static_cast<uint32_t>(kMaxTerms);
  };
  auto locate = [&](uint32_t tile, Source& src) {
    const uint32_t m0 = (tile / tiles_n) * BM, n0 = n_begin + (tile % tiles_n) * BN;
    src.terms = tile_terms(m0);
    src.a = a8 + static_cast<size_t>(m0) * k;
    src.b = w + static_cast<size_t>(n0) * row_bytes;        // also the origin of 16-row tile n0 / 16 in fragment order
    src.s = w + static_cast<size_t>(n) * row_bytes + static_cast<size_t>(n0) * row_blocks;
#pragma unroll
    for (int i = 0; i < kABlk; ++i) {
      const uint32_t row = 8u * (wave * kABlk + i) + lane / 8u;
      const uint32_t chunk = (lane % 8u) ^ ((row >> 1) & 7u);
      src.a_off[i] = (m0 + row < m ? row : m - 1u - m0) * k + chunk * 16u;
    }
#pragma unroll
    for (int i = 0; i < kBBlk; ++i) {
      if constexpr (WPERM) {
        // LDS dword d = j * 64 + lane of the block is dword d % 4 of chunk position (d % 16) / 4 of
        // row d / 16, i.e. dword wd = 4 * (position ^ swizzle) + d % 4 of the row's 64 bytes.
        const uint32_t blk = wave * kBBlk + i;
        const uint32_t blk_in = n0 + 16u * blk < n ? blk : (n - 1u - n0) / 16u;    // n is a multiple of 16
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t d = j * 64u + lane, row = d / 16u, pos = (d % 16u) / 4u;
          const uint32_t wd = 4u * (pos ^ ((row >> 2) & 3u)) + d % 4u;
          src.b_off[i][j] = blk_in * 16u * row_bytes + (wd * 16u + row) * 4u;
        }
      } else {
        const uint32_t row = 16u * (wave * kBBlk + i) + lane / 4u;
        const uint32_t chunk = (lane % 4u) ^ ((row >> 2) & 3u);
        src.b_off[i][0] = (n0 + row < n ? row : n - 1u - n0) * row_bytes + chunk * 16u;
      }
    }
    const uint32_t row = 64u * (wave % (BN / 64)) + lane;
    src.s_off = (n0 + row < n ? row : n - 1u - n0) * row_blocks;
  };
  auto issue_stage = [&](uint32_t stage_off, const Source& src, uint32_t k0, uint32_t term) {
    const uint32_t stage = lds_base + stage_off;
    const uint8_t* ga = src.a + (SPLIT ? term * plane : 0) + k0;
    const uint8_t* gb = src.b + (WPERM ? k0 * 8u : k0 / 2);     // fragment order: 128 bytes per 16-wide K step of a tile
    const uint8_t* gs = src.s + k0 / 32;
#pragma unroll
    for (int i = 0; i < kABlk; ++i) direct_load16(ga, src.a_off[i], stage + (wave * kABlk + i) * 1024u);
#pragma unroll
    for (int i = 0; i < kBBlk; ++i) {
      if constexpr (WPERM) {
#pragma unroll
        for (int j = 0; j < 4; ++j) direct_load4(gb, src.b_off[i][j], stage + kBBase + (wave * kBBlk + i) * 1024u + j * 256u);
      } else {
        direct_load16(gb, src.b_off[i][0], stage + kBBase + (wave * kBBlk + i) * 1024u);
      }
    }
    direct_load4(gs, src.s_off, stage + kSBase + (wave % (BN / 64)) * 256u);
  };

  // Fragments of one 64-wide K slice.  8-bit A operand: a lane of K half `kg` supplies
  // k = 16*kg + [0,16) in its first four registers and k = 32 + 16*kg + [0,16) in the last
  // four (the instruction is two K=32 steps back to back), i.e. chunks 4*ks + kg and
  // 4*ks + 2 + kg of its row; the 4-bit B operand is k = 32*kg + [0,32), chunk 2*ks + kg.
  struct Frag {
    int8v_t a[kTI];
    uint4 b[kTJ];
  };
  uint32_t a_fr[2][2], b_fr[2];
  {
    const uint32_t row = wm * (BM / WM) + l32, swz = (l32 >> 1) & 7u;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int hi = 0; hi < 2; ++hi) a_fr[ks][hi] = row * 128u + (((ks * 4u + hi * 2u + kg) ^ swz) * 16u);
  }
  {
    const uint32_t row = wn * (BN / WN) + l32, swz = (l32 >> 2) & 3u;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) b_fr[ks] = kBBase + row * 64u + (((ks * 2u + kg) ^ swz) * 16u);
  }
  const uint32_t s_fr = kSBase + (wn * (BN / WN) + l32) * 4u;
  auto read_frags = [&](uint32_t stage_off, int ks, Frag& f) {
    const uint8_t* stage = lds + stage_off;
#pragma unroll
    for (int i = 0; i < kTI; ++i) {
      const uint4 lo = *reinterpret_cast<const uint4*>(stage + a_fr[ks][0] + i * 32 * 128);
      const uint4 hi = *reinterpret_cast<const uint4*>(stage + a_fr[ks][1] + i * 32 * 128);
      f.a[i] = int8v_t{static_cast<int>(lo.x), static_cast<int>(lo.y), static_cast<int>(lo.z),
                       static_cast<int>(lo.w), static_cast<int>(hi.x), static_cast<int>(hi.y),
                       static_cast<int>(hi.z), static_cast<int>(hi.w)};
    }
#pragma unroll
    for (int j = 0; j < kTJ; ++j) {
      f.b[j] = *reinterpret_cast<const uint4*>(stage + b_fr[ks] + j * 32 * 64);
    }
  };
  // Scale words of this lane's weight rows; block 2*ks + kg sits at byte 2*ks once lanes of
  // the upper K half have shifted their four bytes down by one (done at the use).
  auto read_scales = [&](uint32_t stage_off, uint32_t (&raw)[kTJ]) {
    const uint8_t* stage = lds + stage_off;
#pragma unroll
    for (int j = 0; j < kTJ; ++j) raw[j] = *reinterpret_cast<const uint32_t*>(stage + s_fr + j * 128);
  };

  float16_t acc[kTI][kTJ];
  // Every wavefront waits for its own direct loads of the stage about to be published (all
  // but the youngest stage's; loads complete in issue order, and stores issued in between
  // only make the wait longer), and for its LDS reads of the stage about to be overwritten,
  // before the barrier.
  auto publish = [&]() {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kDma) : "memory");
  };

  const uint32_t steps = k / kKS;
  Frag f0, f1;
  int sv[kTJ];
  uint32_t sv_raw[kTJ];
  uint32_t rd = 0, nx = kStage, ld = 2 * kStage;

  // One 64-wide K slice of matrix instructions on fragment `f`, with the LDS reads of another
  // fragment (`g`: slice g_ks of the stage at g_stage) issued in between, one read per matrix
  // instruction: a wavefront cannot issue anything else while it waits for the matrix pipe to take
  // its next instruction, so reads placed between them cost nothing, while reads in a block of their
  // own leave the pipe idle (all wavefronts leave the step's barrier together and would all read
  // first).  Worth 2-3 % at M = 2048 (0.2036 -> 0.1992 ms at 17408 x 5120); the matrix cores stay busy
  // 52 % of the cycles either way, the wavefronts spending 43 % of theirs in the step's wait for the
  // direct loads and the barrier behind it.
  auto mfmas_reading = [&](const Frag& f, auto ks_c, int sa, Frag& g, uint32_t g_stage, int g_ks) {
    constexpr int ks = decltype(ks_c)::value;
    constexpr int kReads = 2 * kTI + kTJ, kMfmas = kTI * kTJ;
    const uint8_t* stage = lds + g_stage;
    uint4 lo[kTI], hi[kTI];
    const int a_scale = SPLIT ? sa : 0x7F7F7F7F;
#pragma unroll
    for (int q = 0; q < (kReads > kMfmas ? kReads : kMfmas); ++q) {
      if (q < kMfmas) {
        const int j = q / kTI, i = q % kTI;
        const int8v_t bf = int8v_t{static_cast<int>(f.b[j].x), static_cast<int>(f.b[j].y),
                                   static_cast<int>(f.b[j].z), static_cast<int>(f.b[j].w), 0, 0, 0, 0};
        // A: E4M3 (cbsz 0) with unit scale (E8M0 127), or the term's weight; B: E2M1 (blgp 4)
        // with the block scale.
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(f.a[i], bf, acc[i][j], 0, 4, 0, a_scale, ks == 0 ? 0 : 2,
                                                                    sv[j]);
      }
      if (q < kReads) {
        if (q < 2 * kTI) {
          const int i = q / 2;
          const uint4 v = *reinterpret_cast<const uint4*>(stage + a_fr[g_ks][q & 1] + i * 32 * 128);
          if (q & 1) hi[i] = v;
          else lo[i] = v;
        } else {
          const int j = q - 2 * kTI;
          g.b[j] = *reinterpret_cast<const uint4*>(stage + b_fr[g_ks] + j * 32 * 64);
        }
      }
    }
#pragma unroll
    for (int q = 0; q < (kReads > kMfmas ? kReads : kMfmas); ++q) {
      if (q < kMfmas) __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one matrix instruction,
      if (q < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // then one LDS read
    }
#pragma unroll
    for (int i = 0; i < kTI; ++i) {
      g.a[i] = int8v_t{static_cast<int>(lo[i].x), static_cast<int>(lo[i].y), static_cast<int>(lo[i].z),
                       static_cast<int>(lo[i].w), static_cast<int>(hi[i].x), static_cast<int>(hi[i].y),
                       static_cast<int>(hi[i].z), static_cast<int>(hi[i].w)};
    }
  };

  // Persistent loop over this workgroup's tiles, flattened into one loop over K steps so
  // that the ring of stages never drains: the load cursor runs three steps ahead of the
  // multiply cursor and simply moves on to the next tile when a tile's K is exhausted, so
  // the first loads and fragment reads of a tile run under the previous tile's epilogue.
  // Past the last tile the cursor reloads a stage nobody reads rather than branching.
  uint32_t tile = blockIdx.x;
  if (tile >= tiles) return;
  const uint32_t my_tiles = (tiles - tile + gridDim.x - 1) / gridDim.x;
  Source src;
  locate(tile, src);
  uint32_t load_tile = tile, load_step = 0, load_term = 0;
  auto advance_load = [&]() {
    if (++load_step == steps) {          // uniform
      asm volatile("" ::: "memory");     // keeps this rare block a branch, not a chain of selects
      load_step = 0;
      if (SPLIT && ++load_term < src.terms) return;
      load_term = 0;
      load_tile += gridDim.x;
      if (load_tile < tiles) locate(load_tile, src);
    }
  };
  issue_stage(0, src, 0, 0);
  advance_load();
  issue_stage(kStage, src, load_step * kKS, load_term);
  advance_load();
  issue_stage(2 * kStage, src, load_step * kKS, load_term);
  advance_load();
  // the first stage has landed when only the two younger ones may be outstanding
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * kDma) : "memory");
  read_scales(rd, sv_raw);
  read_frags(rd, 0, f0);
#pragma unroll
  for (int i = 0; i < kTI; ++i)
#pragma unroll
    for (int j = 0; j < kTJ; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  for (uint32_t done_tiles = 0; done_tiles < my_tiles; ++done_tiles) {
    const uint32_t terms = tile_terms((tile / tiles_n) * BM);
    for (uint32_t term = 0; term < terms; ++term) {
      const int sa = 0x7F - 4 * static_cast<int>(term);      // E8M0 of 2^(-4 term), byte 0 is the one used
      for (uint32_t cur = 0; cur < steps; ++cur) {
        // One step of K on stage `rd`; `nx` holds the step after it, `ld` the one after that (its
        // loads were asked for half a step ago).  First half: the matrix instructions of the
        // step's first K slice, whose operands the previous step read, with the reads of the
        // second slice in between.  Then every wavefront has read all of `rd` and `nx` has landed
        // (publish), so `rd` is asked for again with the step three ahead.  Second half: the second
        // slice, with the reads of the NEXT step's first slice (and its scale words) in between.
#pragma unroll
        for (int j = 0; j < kTJ; ++j) sv[j] = static_cast<int>(sv_raw[j] >> (kg * 8u));
        mfmas_reading(f0, std::integral_constant<int, 0>{}, sa, f1, rd, 1);
        publish();
        issue_stage(rd, src, load_step * kKS, load_term);
        advance_load();
        mfmas_reading(f1, std::integral_constant<int, 1>{}, sa, f0, nx, 0);
        read_scales(nx, sv_raw);
        const uint32_t done = rd;
        rd = nx;
        nx = ld;
        ld = done;
      }
    }

    // Epilogue: lane holds column l32 and rows (e/4)*8 + kg*4 + e%4 of each 32 x 32 tile.
    const uint32_t m0 = (tile / tiles_n) * BM, n0 = n_begin + (tile % tiles_n) * BN;
    tile += gridDim.x;
#pragma unroll
    for (int i = 0; i < kTI; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const uint32_t row = m0 + wm * (BM / WM) + i * 32u + (e >> 2) * 8u + kg * 4u + (e & 3u);
        const float scale = as[row < m ? row : m - 1u];
#pragma unroll
        for (int j = 0; j < kTJ; ++j) {
          const uint32_t col = n0 + wn * (BN / WN) + j * 32u + l32;
          if (row < m && col < n_end) c[static_cast<size_t>(row) * n + col] = acc[i][j][e] * scale;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kTI; ++i)
#pragma unroll
      for (int j = 0; j < kTJ; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
  }
  // No direct load may still be writing LDS when the workgroup retires.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// ---- a few activation rows (speculative verify, m <= 32) ----------------------------------
// Bandwidth-bound: every weight byte is needed once and there is almost no reuse to stage
// for, so nothing goes through LDS on the way in.  v_mfma_scale_f32_16x16x128_f8f6f4 has the
// operand shape for that: a lane supplies 16 bytes of one weight row (32 E2M1 values = one
// MX block, K quarter lane/16), so one load instruction of a wavefront reads 64 contiguous
// bytes of each of 16 rows, and the E4M3 activation fragment is two such loads
// (k = 16q + [0,16) and 64 + 16q + [0,16) for K quarter q; layouts probed on hardware).
// A workgroup of eight wavefronts owns 64 weight rows (four 16-column tiles); the wavefronts
// split K among themselves and stream their share with a register prefetch; the eight partial
// tiles are summed in LDS in wavefront order (deterministic) and scaled by the row scale.  Two
// workgroups share a CU, so the 272 workgroups of N = 17408 are resident at once.
constexpr int kSkinnyWaves = 8;

template <int MT>   // 16-row activation tiles: 1 (m <= 16) or 2 (m <= 32)
__global__ __launch_bounds__(64 * kSkinnyWaves, 4) void mxfp4_a8_skinny_kernel(
    const uint8_t* __restrict__ a8, const float* __restrict__ as, const uint8_t* __restrict__ w,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k) {
  constexpr int kDepth = 2;
  typedef float float4v __attribute__((ext_vector_type(4)));
  __shared__ float red[kSkinnyWaves][MT][4][4][64];
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t l16 = lane & 15u, kq = lane >> 4;
  const uint32_t n0 = blockIdx.x * 64u;
  const uint32_t row_bytes = k / 2, row_blocks = k / 32;
  const uint8_t* scales = w + static_cast<size_t>(n) * row_bytes;

  // K steps (128 wide) of this wavefront: step index i stands for K step wave + 8 i, so that
  // at any moment the eight wavefronts read eight neighbouring 64-byte pieces of each row.
  const uint32_t total = k / 128u;
  const uint32_t s0 = 0, s1 = total > wave ? (total - wave + kSkinnyWaves - 1) / kSkinnyWaves : 0;

  // Loads use the lane order that coalesces: lane p fetches 16-byte chunk p%4 of row p/4, so
  // four neighbouring lanes cover 64 contiguous bytes.  The MFMA wants lane q*16 + r to hold
  // chunk q of row r; ds_bpermute moves the registers into that order (through the LDS
  // crossbar, no LDS memory), which is far cheaper than letting every lane of a quad address
  // a different row.
  const uint32_t ld_row = lane >> 2, ld_chunk = lane & 3u;
  const int take = static_cast<int>(((lane & 15u) * 4u + (lane >> 4)) * 4u);   // source lane * 4
  const uint8_t* wq[4];
  const uint8_t* ws[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t row = n0 + j * 16u + ld_row;
    row = row < n ? row : n - 1u;
    wq[j] = w + static_cast<size_t>(row) * row_bytes + ld_chunk * 16u;
    ws[j] = scales + static_cast<size_t>(row) * row_blocks;
  }
  const uint8_t* ap[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const uint32_t row = i * 16u + ld_row;
    ap[i] = a8 + static_cast<size_t>(row < m ? row : m - 1u) * k + ld_chunk * 16u;
  }

  struct Stage {
    uint4 q[4], lo[MT], hi[MT];
    uint32_t s[4];
  };
  auto fetch = [&](uint32_t index, Stage& st) {
    const uint32_t step = wave + kSkinnyWaves * index;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      st.q[j] = load_u4(wq[j] + step * 64u);
      st.s[j] = *reinterpret_cast<const uint32_t*>(ws[j] + 4u * step);   // blocks 4 step + 0..3
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      st.lo[i] = load_u4(ap[i] + step * 128u);
      st.hi[i] = load_u4(ap[i] + step * 128u + 64u);
    }
  };

  float4v acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = float4v{0.0f, 0.0f, 0.0f, 0.0f};

  auto to_mfma_order = [&](const uint4& v) {
    return int4v_t{__builtin_amdgcn_ds_bpermute(take, static_cast<int>(v.x)),
                   __builtin_amdgcn_ds_bpermute(take, static_cast<int>(v.y)),
                   __builtin_amdgcn_ds_bpermute(take, static_cast<int>(v.z)),
                   __builtin_amdgcn_ds_bpermute(take, static_cast<int>(v.w))};
  };
  auto consume = [&](const Stage& cur) {
    int8v_t af[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int4v_t lo = to_mfma_order(cur.lo[i]), hi = to_mfma_order(cur.hi[i]);
      af[i] = int8v_t{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int4v_t q = to_mfma_order(cur.q[j]);
      const int8v_t bf = int8v_t{q[0], q[1], q[2], q[3], 0, 0, 0, 0};
      // this lane's MX block is byte kq of its row's scale word
      const int sv = static_cast<int>(static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(take, static_cast<int>(cur.s[j]))) >> (kq * 8u));
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af[i], bf, acc[i][j], 0, 4, 0, 0x7F7F7F7F, 0, sv);
      }
    }
  };

  // Register pipeline of kDepth steps.  Full groups consume and refill unconditionally (a
  // refill past this wavefront's range re-reads its last step, a cache hit), so the compiler
  // counts outstanding loads exactly; the last partial group consumes without refilling.
  Stage st[kDepth];
  const uint32_t last = s1 > s0 ? s1 - 1u : s0;   // (a wavefront without steps reloads step `wave`: k >= 1024 keeps that in range)
#pragma unroll
  for (int d = 0; d < kDepth; ++d) fetch(s0 + d < s1 ? s0 + d : last, st[d]);
  uint32_t step = s0;
  for (; step + kDepth <= s1; step += kDepth) {
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      consume(st[d]);
      fetch(step + d + kDepth < s1 ? step + d + kDepth : last, st[d]);
    }
  }
#pragma unroll
  for (int d = 0; d < kDepth - 1; ++d) {
    if (step + d < s1) consume(st[d]);     // uniform
  }

  // Sum the wavefronts' partial tiles: lane holds column l16 and rows (lane/16)*4 + e.
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[wave][i][j][e][lane] = acc[i][j][e];
  __syncthreads();
  for (uint32_t o = t; o < m * 64u; o += 64u * kSkinnyWaves) {
    const uint32_t row = o / 64u, col = o % 64u;
    const uint32_t i = row / 16u, r = row % 16u, ln = (r / 4u) * 16u + col % 16u;
    float sum = 0.0f;
#pragma unroll
    for (int wv = 0; wv < kSkinnyWaves; ++wv) sum += red[wv][i][col / 16u][r % 4u][ln];
    if (n0 + col < n) c[static_cast<size_t>(row) * n + n0 + col] = sum * as[row];
  }
}

// ---- a few activation rows, streamed through LDS (k a multiple of 512) ----------------------
// Same arithmetic as the kernel above, fed differently: each direct load moves 256 contiguous
// bytes of a weight row (four rows per instruction) into a three-stage swizzled LDS ring, so
// HBM sees long row-contiguous runs instead of 64-byte pieces of sixteen rows, and the
// fragment reads do the row/K transposition for free.  A workgroup owns `rows_wg` weight rows (a
// multiple of 4, at most 80: the rows of the matrix shared out evenly over the CUs, because the
// bytes a CU's direct loads move set the pace -- 17408 rows as 272 groups of 64 took half as long
// again as 16384 rows as 256) and has two wavefronts per 16-row column tile; per stage (512 of
// K) the 4 K-steps of a tile are split two to a wavefront and the two wavefronts of a tile are
// summed through LDS at the end.  Activation rows the call does not have are not loaded (their
// rows of the product are never stored).
constexpr uint32_t kStreamMaxRows = 80;

// TERMS: the activation rows are fp32 rows split into kMaxTerms E4M3 planes (split_rows_kernel): matrix row
// t * rows + r is term t of row r, `a8` points at row 0 of plane 0, the planes lie `plane` bytes apart, `m` counts
// the matrix rows (kMaxTerms * rows), and the store adds a row's terms with their weights 16^-t.
template <int MT, bool TERMS = false>
__global__ __launch_bounds__(640) void mxfp4_a8_stream_kernel(
    const uint8_t* __restrict__ a8, const float* __restrict__ as, const uint8_t* __restrict__ w,
    float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k, uint32_t rows_wg, uint64_t plane = 0) {
  typedef float float4v __attribute__((ext_vector_type(4)));
  constexpr uint32_t kBBytes = kStreamMaxRows * 256, kABytes = MT * 16 * 512, kSBytes = kStreamMaxRows * 16;
  constexpr uint32_t kABase = kBBytes, kSBase = kABase + kABytes, kStage = kSBase + kSBytes;
  __shared__ __attribute__((aligned(16))) uint8_t lds[3 * kStage];

  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t tiles = (rows_wg + 15u) / 16u;           // blockDim.x = 128 * tiles
  const uint32_t l16 = lane & 15u, kq = lane >> 4;
  const uint32_t n0 = blockIdx.x * rows_wg;
  const uint32_t row_bytes = k / 2, row_blocks = k / 32;
  const uint8_t* w_tile = w + static_cast<size_t>(n0) * row_bytes;
  const uint8_t* s_tile = w + static_cast<size_t>(n) * row_bytes + static_cast<size_t>(n0) * row_blocks;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)lds));

  // Direct loads of one stage.  Weight block L (1 KB) = rows 4L..4L+3, sixteen 16-byte chunks
  // each: lane p fetches row 4L + p/16, chunk (p%16) ^ (row%16).  Activation block L = rows
  // 2L, 2L+1, thirty-two chunks each: row 2L + p/32, chunk (p%32) ^ (row%16).  Scale words: lane
  // p < 8 of wavefront v fetches the sixteen E8M0 bytes of row 8v + p.  Rows past the matrix
  // edge are clamped (never stored); blocks past the workgroup's rows or the call's activation
  // rows are not requested, so the loads a wavefront has in flight per stage differ: `my_dma`.
  constexpr int kAMax = 4 * MT;        // activation blocks a wavefront brings at most (two wavefronts: 8 MT blocks)
  const uint32_t waves = 2u * tiles;
  uint32_t b_src[2], a_src[kAMax], s_src;
  bool b_live[2], a_live[kAMax];
  uint32_t my_dma = 0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t row = 4u * (wave * 2u + i) + lane / 16u;
    const uint32_t chunk = (lane % 16u) ^ (row % 16u);
    b_src[i] = (n0 + row < n ? row : n - 1u - n0) * row_bytes + chunk * 16u;
    b_live[i] = 4u * (wave * 2u + i) < rows_wg;
    my_dma += b_live[i] ? 1u : 0u;
  }
#pragma unroll
  for (int i = 0; i < kAMax; ++i) {
    const uint32_t blk = wave + i * waves;               // blocks go round the wavefronts
    const uint32_t row = 2u * blk + lane / 32u;
    const uint32_t chunk = (lane % 32u) ^ (row % 16u);
    const uint32_t src_row = row < m ? row : m - 1u;
    if constexpr (TERMS) {
      const uint32_t real = m / kMaxTerms, term = src_row / real;
      a_src[i] = static_cast<uint32_t>(term * plane) + (src_row - term * real) * k + chunk * 16u;
    } else {
      a_src[i] = src_row * k + chunk * 16u;
    }
    a_live[i] = blk < 8u * MT && 2u * blk < m;
    my_dma += a_live[i] ? 1u : 0u;
  }
  const bool s_live = 8u * wave < rows_wg;
  {
    const uint32_t row = 8u * wave + (lane & 7u);
    s_src = (n0 + row < n ? row : n - 1u - n0) * row_blocks;
    my_dma += s_live ? 1u : 0u;
  }
  auto issue_stage = [&](uint32_t stage_off, uint32_t st) {
    const uint32_t stage = lds_base + stage_off;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if (b_live[i]) direct_load16(w_tile + st * 256u, b_src[i], stage + (wave * 2u + i) * 1024u);
    }
#pragma unroll
    for (int i = 0; i < kAMax; ++i) {
      if (a_live[i]) direct_load16(a8 + st * 512u, a_src[i], stage + kABase + (wave + i * waves) * 1024u);
    }
    if (s_live && lane < 8u) direct_load16(s_tile + st * 16u, s_src, stage + kSBase + wave * 128u);
  };
  // Everything but the stage requested last has landed, for every wavefront.
  auto publish = [&]() {
    switch (my_dma) {
      case 0: asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(1) lgkmcnt(0)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory"); break;
      case 3: asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory"); break;
      case 5: asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory"); break;
      case 6: asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory"); break;
      case 7: asm volatile("s_waitcnt vmcnt(7) lgkmcnt(0)" ::: "memory"); break;
      case 8: asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory"); break;
      case 9: asm volatile("s_waitcnt vmcnt(9) lgkmcnt(0)" ::: "memory"); break;
      case 10: asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(11) lgkmcnt(0)" ::: "memory"); break;
    }
    asm volatile("s_barrier" ::: "memory");
  };
  static_assert(2 + kAMax + 1 <= 11, "publish() counts up to eleven loads a stage");

  // This wavefront's share of a stage: column tile `tile`, K-steps 2*half and 2*half + 1.
  const uint32_t tile = wave % tiles, half = wave / tiles;
  const uint32_t b_row = tile * 16u + l16;
  float4v acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = float4v{0.0f, 0.0f, 0.0f, 0.0f};

  const uint32_t stages = k / 512u;
  issue_stage(0, 0);
  issue_stage(kStage, stages > 1 ? 1 : 0);
  publish();
  uint32_t rd = 0, nx = kStage, fill = 2 * kStage;
  for (uint32_t st = 0; st < stages; ++st) {
    issue_stage(fill, st + 2 < stages ? st + 2 : stages - 1u);
    const uint8_t* stage = lds + rd;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t step = half * 2u + u;
      const uint4 q = *reinterpret_cast<const uint4*>(stage + b_row * 256u + (((step * 4u + kq) ^ l16) * 16u));
      const int8v_t bf = int8v_t{static_cast<int>(q.x), static_cast<int>(q.y), static_cast<int>(q.z),
                                 static_cast<int>(q.w), 0, 0, 0, 0};
      const uint32_t sw = *reinterpret_cast<const uint32_t*>(stage + kSBase + b_row * 16u + step * 4u);
      const int sv = static_cast<int>(sw >> (kq * 8u));       // this lane's block is byte kq of the step's word
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const uint8_t* arow = stage + kABase + (i * 16u + l16) * 512u;
        const uint4 lo = *reinterpret_cast<const uint4*>(arow + (((step * 8u + kq) ^ l16) * 16u));
        const uint4 hi = *reinterpret_cast<const uint4*>(arow + (((step * 8u + 4u + kq) ^ l16) * 16u));
        const int8v_t af = int8v_t{static_cast<int>(lo.x), static_cast<int>(lo.y), static_cast<int>(lo.z),
                                   static_cast<int>(lo.w), static_cast<int>(hi.x), static_cast<int>(hi.y),
                                   static_cast<int>(hi.z), static_cast<int>(hi.w)};
        acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af, bf, acc[i], 0, 4, 0, 0x7F7F7F7F, 0, sv);
      }
    }
    publish();
    const uint32_t done = rd;
    rd = nx;
    nx = fill;
    fill = done;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive its workgroup
  __syncthreads();

  // Sum the two wavefronts of each tile (stage memory is free now): lane holds column l16 and
  // rows (lane/16)*4 + e of its 16 x 16 tile.
  float* red = reinterpret_cast<float*>(lds);          // [half][tile][MT][4][64]
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[(((half * tiles + tile) * MT + i) * 4u + e) * 64u + lane] = acc[i][e];
  __syncthreads();
  const uint32_t cols = tiles * 16u;
  auto tile_sum = [&](uint32_t row, uint32_t col) {
    const uint32_t i = row / 16u, r = row % 16u, ln = (r / 4u) * 16u + col % 16u, tl = col / 16u;
    return red[(((0u * tiles + tl) * MT + i) * 4u + r % 4u) * 64u + ln] +
           red[(((1u * tiles + tl) * MT + i) * 4u + r % 4u) * 64u + ln];
  };
  if constexpr (TERMS) {
    const uint32_t real = m / kMaxTerms;
    for (uint32_t o = t; o < real * cols; o += blockDim.x) {
      const uint32_t row = o / cols, col = o % cols;
      float sum = tile_sum((kMaxTerms - 1) * real + row, col);
#pragma unroll
      for (int term = kMaxTerms - 2; term >= 0; --term) sum = fmaf(sum, 0.0625f, tile_sum(term * real + row, col));
      if (col < rows_wg && n0 + col < n) c[static_cast<size_t>(row) * n + n0 + col] = sum * as[row];
    }
  } else {
    for (uint32_t o = t; o < m * cols; o += blockDim.x) {
      const uint32_t row = o / cols, col = o % cols;
      if (col < rows_wg && n0 + col < n) c[static_cast<size_t>(row) * n + n0 + col] = tile_sum(row, col) * as[row];
    }
  }
}

// ---- FP8 E4M3 weights x a few fp32 rows ("gemm_fp8", 2..16 rows), streamed the same way -----------
// The weights are E4M3 already, so they are the B operand of the same matrix instruction as they are
// stored (format E4M3 instead of E2M1, unit block scale); the fp32 rows go in as E4M3 terms as above
// (matrix row t * rows + r = term t of row r), the weight row's fp32 scale and the activation row's
// power of two are applied at the store.  A weight row is 512 bytes a stage instead of 256, so a
// direct load moves two rows and the workgroup's share of rows is sized to the LDS it leaves: the
// stage ring is dynamic shared memory of 3 x (rows x 512 + MT x 8192) bytes.
// BLOCK ("gemm_fp8_block"): `wscale` is one fp32 per 128 x 128 block of W, (n/128) x (k/128) row-major.
// An instruction covers 128 of K, i.e. exactly one block column, so its sum is taken by itself and
// multiplied by the block's scale before it joins the accumulator; the four scales a weight row
// needs per stage come with the stage (one more 16-byte direct load per row, rows x 16 more bytes).
template <int MT, bool BLOCK = false>
__global__ __launch_bounds__(640) void fp8_terms_stream_kernel(
    const uint8_t* __restrict__ a8, const float* __restrict__ as, const uint8_t* __restrict__ w,
    const float* __restrict__ wscale, float* __restrict__ c, uint32_t m, uint32_t n, uint32_t k, uint32_t rows_wg,
    uint64_t plane) {
  typedef float float4v __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const uint32_t kABase = rows_wg * 512u, kSBase = kABase + MT * 16u * 512u;
  const uint32_t kStage = kSBase + (BLOCK ? rows_wg * 16u : 0u);

  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t tiles = (rows_wg + 15u) / 16u;           // blockDim.x = 128 * tiles
  const uint32_t l16 = lane & 15u, kq = lane >> 4;
  const uint32_t n0 = blockIdx.x * rows_wg;
  const uint8_t* w_tile = w + static_cast<size_t>(n0) * k;
  const uint8_t* s_base = reinterpret_cast<const uint8_t*>(wscale);
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(
      (__attribute__((address_space(3))) uint8_t*)lds));

  // Direct loads of one stage.  Weight block L (1 KB) = rows 2L, 2L+1, thirty-two 16-byte chunks
  // each: lane p fetches row 2L + p/32, chunk (p%32) ^ (row%16); wavefront v brings blocks 4v..4v+3
  // (rows 8v..8v+7).  Activation blocks as in the kernel above.
  constexpr int kAMax = 4 * MT;
  const uint32_t waves = 2u * tiles;
  uint32_t b_src[4], a_src[kAMax];
  bool b_live[4], a_live[kAMax];
  uint32_t my_dma = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t blk = wave * 4u + i;
    const uint32_t row = 2u * blk + lane / 32u;
    const uint32_t chunk = (lane % 32u) ^ (row % 16u);
    b_src[i] = (n0 + row < n ? row : n - 1u - n0) * k + chunk * 16u;
    b_live[i] = 2u * blk < rows_wg;
    my_dma += b_live[i] ? 1u : 0u;
  }
#pragma unroll
  for (int i = 0; i < kAMax; ++i) {
    const uint32_t blk = wave + i * waves;
    const uint32_t row = 2u * blk + lane / 32u;
    const uint32_t chunk = (lane % 32u) ^ (row % 16u);
    const uint32_t src_row = row < m ? row : m - 1u;
    const uint32_t real = m / kMaxTerms, term = src_row / real;
    a_src[i] = static_cast<uint32_t>(term * plane) + (src_row - term * real) * k + chunk * 16u;
    a_live[i] = blk < 8u * MT && 2u * blk < m;
    my_dma += a_live[i] ? 1u : 0u;
  }
  // BLOCK: lane p < 8 of wavefront v fetches the stage's four scales (16 bytes) of row 8v + p
  const bool s_live = BLOCK && 8u * wave < rows_wg;
  uint32_t s_src = 0;
  if (BLOCK) {
    const uint32_t row = 8u * wave + (lane & 7u);
    s_src = ((n0 + row < n ? n0 + row : n - 1u) / 128u) * (k / 128u) * 4u;
    my_dma += s_live ? 1u : 0u;
  }
  auto issue_stage = [&](uint32_t stage_off, uint32_t st) {
    const uint32_t stage = lds_base + stage_off;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (b_live[i]) direct_load16(w_tile + st * 512u, b_src[i], stage + (wave * 4u + i) * 1024u);
    }
#pragma unroll
    for (int i = 0; i < kAMax; ++i) {
      if (a_live[i]) direct_load16(a8 + st * 512u, a_src[i], stage + kABase + (wave + i * waves) * 1024u);
    }
    // (rows_wg is a multiple of four, not of eight: the lanes past it stay out, their bytes would land in
    // the next stage)
    if (s_live && lane < 8u && 8u * wave + lane < rows_wg) direct_load16(s_base + st * 16u, s_src, stage + kSBase + wave * 128u);
  };
  // Everything but the stage requested last has landed, for every wavefront.
  auto publish = [&]() {
    switch (my_dma) {
      case 0: asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); break;
      case 1: asm volatile("s_waitcnt vmcnt(1) lgkmcnt(0)" ::: "memory"); break;
      case 2: asm volatile("s_waitcnt vmcnt(2) lgkmcnt(0)" ::: "memory"); break;
      case 3: asm volatile("s_waitcnt vmcnt(3) lgkmcnt(0)" ::: "memory"); break;
      case 4: asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory"); break;
      case 5: asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory"); break;
      case 6: asm volatile("s_waitcnt vmcnt(6) lgkmcnt(0)" ::: "memory"); break;
      case 7: asm volatile("s_waitcnt vmcnt(7) lgkmcnt(0)" ::: "memory"); break;
      case 8: asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory"); break;
      case 9: asm volatile("s_waitcnt vmcnt(9) lgkmcnt(0)" ::: "memory"); break;
      case 10: asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)" ::: "memory"); break;
      case 11: asm volatile("s_waitcnt vmcnt(11) lgkmcnt(0)" ::: "memory"); break;
      case 12: asm volatile("s_waitcnt vmcnt(12) lgkmcnt(0)" ::: "memory"); break;
      default: asm volatile("s_waitcnt vmcnt(13) lgkmcnt(0)" ::: "memory"); break;
    }
    asm volatile("s_barrier" ::: "memory");
  };
  static_assert(4 + kAMax + 1 <= 13, "publish() counts up to thirteen loads a stage");

  // This wavefront's share of a stage: column tile `tile`, K-steps 2*half and 2*half + 1.
  const uint32_t tile = wave % tiles, half = wave / tiles;
  const uint32_t b_row = tile * 16u + l16;
  float4v acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = float4v{0.0f, 0.0f, 0.0f, 0.0f};

  const uint32_t stages = k / 512u;
  issue_stage(0, 0);
  issue_stage(kStage, stages > 1 ? 1 : 0);
  publish();
  uint32_t rd = 0, nx = kStage, fill = 2 * kStage;
  for (uint32_t st = 0; st < stages; ++st) {
    issue_stage(fill, st + 2 < stages ? st + 2 : stages - 1u);
    const uint8_t* stage = lds + rd;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const uint32_t step = half * 2u + u;
      // a row of the last, partly filled tile past the workgroup's rows reads what follows the weight
      // area (activation bytes, still inside the stage): its column is never stored
      const uint8_t* brow = stage + b_row * 512u;
      const uint4 blo = *reinterpret_cast<const uint4*>(brow + (((step * 8u + kq) ^ l16) * 16u));
      const uint4 bhi = *reinterpret_cast<const uint4*>(brow + (((step * 8u + 4u + kq) ^ l16) * 16u));
      const int8v_t bf = int8v_t{static_cast<int>(blo.x), static_cast<int>(blo.y), static_cast<int>(blo.z),
                                 static_cast<int>(blo.w), static_cast<int>(bhi.x), static_cast<int>(bhi.y),
                                 static_cast<int>(bhi.z), static_cast<int>(bhi.w)};
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const uint8_t* arow = stage + kABase + (i * 16u + l16) * 512u;
        const uint4 lo = *reinterpret_cast<const uint4*>(arow + (((step * 8u + kq) ^ l16) * 16u));
        const uint4 hi = *reinterpret_cast<const uint4*>(arow + (((step * 8u + 4u + kq) ^ l16) * 16u));
        const int8v_t af = int8v_t{static_cast<int>(lo.x), static_cast<int>(lo.y), static_cast<int>(lo.z),
                                   static_cast<int>(lo.w), static_cast<int>(hi.x), static_cast<int>(hi.y),
                                   static_cast<int>(hi.z), static_cast<int>(hi.w)};
        // both operands E4M3 (cbsz 0, blgp 0) with unit E8M0 scales
        if constexpr (BLOCK) {
          const float4v d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af, bf, float4v{0.0f, 0.0f, 0.0f, 0.0f}, 0, 0, 0,
                                                                              0x7F7F7F7F, 0, 0x7F7F7F7F);
          const uint32_t s_row = b_row < rows_wg ? b_row : rows_wg - 1u;      // (a column past the rows is never stored)
          const float bs = *reinterpret_cast<const float*>(stage + kSBase + s_row * 16u + step * 4u);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[i][e] = fmaf(bs, d[e], acc[i][e]);
        } else {
          acc[i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(af, bf, acc[i], 0, 0, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
        }
      }
    }
    publish();
    const uint32_t done = rd;
    rd = nx;
    nx = fill;
    fill = done;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // no direct load may outlive its workgroup
  __syncthreads();

  // Sum the two wavefronts of each tile (stage memory is free now), add a row's terms, scale.
  float* red = reinterpret_cast<float*>(lds);          // [half][tile][MT][4][64]
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[(((half * tiles + tile) * MT + i) * 4u + e) * 64u + lane] = acc[i][e];
  __syncthreads();
  const uint32_t cols = tiles * 16u;
  auto tile_sum = [&](uint32_t row, uint32_t col) {
    const uint32_t i = row / 16u, r = row % 16u, ln = (r / 4u) * 16u + col % 16u, tl = col / 16u;
    return red[(((0u * tiles + tl) * MT + i) * 4u + r % 4u) * 64u + ln] +
           red[(((1u * tiles + tl) * MT + i) * 4u + r % 4u) * 64u + ln];
  };
  const uint32_t real = m / kMaxTerms;
  for (uint32_t o = t; o < real * cols; o += blockDim.x) {
    const uint32_t row = o / cols, col = o % cols;
    float sum = tile_sum((kMaxTerms - 1) * real + row, col);
#pragma unroll
    for (int term = kMaxTerms - 2; term >= 0; --term) sum = fmaf(sum, 0.0625f, tile_sum(term * real + row, col));
    if (col < rows_wg && n0 + col < n) {
      c[static_cast<size_t>(row) * n + n0 + col] = BLOCK ? sum * as[row] : sum * as[row] * wscale[n0 + col];
    }
  }
}

// Rows a workgroup of the FP8 kernel owns: the matrix shared out evenly over the CUs, in multiples
// of four rows, as many as the stage ring leaves room for (80 with one activation tile, 72 with two).
uint32_t fp8_rows_per_workgroup(uint32_t n, uint32_t max_rows) {
  const uint32_t cus = static_cast<uint32_t>(num_cus());
  const uint32_t rounds = (n + max_rows * cus - 1u) / (max_rows * cus);
  const uint32_t share = (n + cus * rounds - 1u) / (cus * rounds);
  uint32_t rows = (share + 3u) / 4u * 4u;
  rows = rows < 16u ? 16u : (rows > max_rows ? max_rows : rows);
  return rows;
}

// Rows a workgroup of the streamed kernel owns: the matrix shared out evenly over the CUs, as few
// rounds of workgroups as 80 rows each allow, in multiples of the four rows a direct load moves.
uint32_t stream_rows_per_workgroup(uint32_t n) {
  const uint32_t cus = static_cast<uint32_t>(num_cus());
  const uint32_t rounds = (n + kStreamMaxRows * cus - 1u) / (kStreamMaxRows * cus);
  const uint32_t share = (n + cus * rounds - 1u) / (cus * rounds);
  uint32_t rows = (share + 3u) / 4u * 4u;
  rows = rows < 16u ? 16u : (rows > kStreamMaxRows ? kStreamMaxRows : rows);
  return rows;
}


// ---- fp32 activations as a sum of E4M3 terms (for the ids whose contract is fp32 rows) -------
// A row is written as  a = s0 * (h0 + h1/16 + h2/256 + h3/4096),  s0 = 2^(floor(log2 rowmax) - 7),
// every h an E4M3 number: h0 is a/s0 (below 256) cut to its four leading significant bits, h1
// the same of 16 * (a/s0 - h0), and so on; the last term rounds instead of cutting.  All of it is
// exact fp32 arithmetic, so a value of 4T significant bits is reproduced exactly by T terms as
// long as its last bit is not below the E4M3 grid of the last term (2^-9 * 16^-(T-1) * s0, i.e.
// rowmax * 2^-(12+4T) at the least); what lies below is dropped.  `need` = terms the row's
// widest significand asks for: 2 for bf16-valued rows, 3 up to 12 bits, else 4 (16 bits kept).
// A non-finite element becomes the E4M3 NaN, which spoils its row of C.
__device__ __forceinline__ uint32_t e4m3_cut(float x, float& val) {        // |x| < 256
  const uint32_t b = bit_cast<uint32_t>(x), sign = (b >> 24) & 0x80u;
  if (fabsf(x) >= 0x1p-6f) {
    const uint32_t tb = b & 0xFFF00000u;                                  // sign, exponent, three mantissa bits
    val = bit_cast<float>(tb);
    return sign | ((((tb >> 23) & 0xFFu) - 120u) << 3) | ((tb >> 20) & 7u);
  }
  const uint32_t q = static_cast<uint32_t>(fabsf(x) * 512.0f);           // the subnormal grid, 2^-9
  val = copysignf(static_cast<float>(q) * 0x1p-9f, x);
  return sign | q;
}
__device__ __forceinline__ uint32_t e4m3_near(float x) {                  // |x| < 256, to nearest
  const uint32_t b = bit_cast<uint32_t>(x), sign = (b >> 24) & 0x80u, mag = b & 0x7FFFFFFFu;
  if (fabsf(x) >= 0x1p-6f) {
    const uint32_t r = mag + 0x7FFFFu + ((mag >> 20) & 1u);               // carry may reach the exponent (256 = 0x78)
    return sign | ((r >> 20) - (120u << 3));
  }
  return sign | static_cast<uint32_t>(rintf(fabsf(x) * 512.0f));         // 8 = 2^-6, the first normal code
}

// NV > 0: a thread keeps its NV 16-byte pieces of the row in registers between the two passes (the
// row is read once; k <= 4 * NV * blockDim.x).  NV = 0: the row is read again for the second pass.
template <int NV>
__global__ __launch_bounds__(1024) void split_rows_kernel(const float* __restrict__ a, uint8_t* __restrict__ planes,
                                                          float* __restrict__ as, uint8_t* __restrict__ need,
                                                          uint32_t m, uint32_t k) {
  __shared__ float s_max[16];
  __shared__ uint32_t s_or[16];
  const uint32_t row = blockIdx.x, t = threadIdx.x, stride = blockDim.x * 4u, waves = blockDim.x >> 6;
  const float* ar = a + static_cast<size_t>(row) * k;
  float amax = 0.0f;
  uint32_t low = 0;
  uint4 held[NV > 0 ? NV : 1];
  auto scan = [&](const uint4 v) {
    const uint32_t b[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const uint32_t mag = b[e] & 0x7FFFFFFFu;
      if (mag < 0x7F800000u) {
        amax = fmaxf(amax, bit_cast<float>(mag));
        if (mag != 0) low |= mag & 0x7FFFFFu;
      }
    }
  };
  if constexpr (NV > 0) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const uint32_t i = t * 4u + j * stride;
      held[j] = i < k ? load_u4(ar + i) : make_uint4(0u, 0u, 0u, 0u);                  // k is a multiple of 128
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) scan(held[j]);
  } else {
    for (uint32_t i = t * 4u; i < k; i += stride) scan(load_u4(ar + i));
  }
  amax = wave_max(amax);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) low |= __shfl_xor(low, off, kWave);
  if ((t & 63u) == 0) {
    s_max[t >> 6] = amax;
    s_or[t >> 6] = low;
  }
  __syncthreads();
  amax = 0.0f, low = 0;
  for (uint32_t wv = 0; wv < waves; ++wv) amax = fmaxf(amax, s_max[wv]), low |= s_or[wv];
  // floor(log2 amax), kept where both s0 and 1/s0 are normal numbers
  int e = static_cast<int>(bit_cast<uint32_t>(amax) >> 23) - 127;
  e = amax == 0.0f ? 7 : (e < -112 ? -112 : e);
  const float s0 = bit_cast<float>(static_cast<uint32_t>(e - 7 + 127) << 23);
  const float inv = bit_cast<float>(static_cast<uint32_t>(7 - e + 127) << 23);
  if (t == 0) {
    as[row] = s0;
    const uint32_t bits = 24u - static_cast<uint32_t>(__builtin_ctz(low | 0x800000u));
    need[row] = static_cast<uint8_t>(bits <= 8 ? 2 : (bits <= 12 ? 3 : 4));
  }
  const size_t plane = static_cast<size_t>(m) * k;
  uint8_t* out = planes + static_cast<size_t>(row) * k;
  auto emit = [&](const uint4 v, uint32_t i) {
    const uint32_t b[4] = {v.x, v.y, v.z, v.w};
    uint32_t code[kMaxTerms] = {0, 0, 0, 0};
#pragma unroll
    for (int el = 0; el < 4; ++el) {
      if ((b[el] & 0x7FFFFFFFu) >= 0x7F800000u) {
        code[0] |= 0x7Fu << (8 * el);
        continue;
      }
      float r = bit_cast<float>(b[el]) * inv;
#pragma unroll
      for (int term = 0; term < kMaxTerms - 1; ++term) {
        float val;
        code[term] |= e4m3_cut(r, val) << (8 * el);
        r = (r - val) * 16.0f;
      }
      code[kMaxTerms - 1] |= e4m3_near(r) << (8 * el);
    }
#pragma unroll
    for (int term = 0; term < kMaxTerms; ++term) *reinterpret_cast<uint32_t*>(out + term * plane + i) = code[term];
  };
  if constexpr (NV > 0) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const uint32_t i = t * 4u + j * stride;
      if (i < k) emit(held[j], i);
    }
  } else {
    for (uint32_t i = t * 4u; i < k; i += stride) emit(load_u4(ar + i), i);
  }
}

// A few rows: 1024 threads a row and the row kept in registers, so that the launch is one trip to
// memory and back (the split of 4 rows of 5120: 8.6 -> 4.7 us); many rows: 256 threads a row, several rows a CU.
void launch_split_rows(const float* a, uint8_t* planes, float* as, uint8_t* need, uint32_t m, uint32_t k,
                       hipStream_t stream) {
  if (m <= 64u && k <= 4096u * 8u) {
    const uint32_t threads = k >= 4096u ? 1024u : 256u;
    const uint32_t nv = (k + threads * 4u - 1u) / (threads * 4u);
    if (nv <= 1u) hipLaunchKernelGGL(split_rows_kernel<1>, dim3(m), dim3(threads), 0, stream, a, planes, as, need, m, k);
    else if (nv == 2u) hipLaunchKernelGGL(split_rows_kernel<2>, dim3(m), dim3(threads), 0, stream, a, planes, as, need, m, k);
    else if (nv <= 4u) hipLaunchKernelGGL(split_rows_kernel<4>, dim3(m), dim3(threads), 0, stream, a, planes, as, need, m, k);
    else hipLaunchKernelGGL(split_rows_kernel<8>, dim3(m), dim3(threads), 0, stream, a, planes, as, need, m, k);
    return;
  }
  hipLaunchKernelGGL(split_rows_kernel<0>, dim3(m), dim3(256), 0, stream, a, planes, as, need, m, k);
}

}  // namespace

bool gemm_mxfp4_a8_supported(uint64_t k) { return k % 128 == 0 && k <= (1u << 24); }

namespace {

template <int BM, int BN, int WM, int WN>
void launch_range(const uint8_t* a8, const float* as, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                  uint32_t k, uint32_t n_begin, uint32_t n_end, uint32_t max_groups, const uint8_t* need,
                  bool wperm, hipStream_t stream) {
  const uint32_t tiles = ((m + BM - 1) / BM) * ((n_end - n_begin + BN - 1) / BN);
  const uint32_t grid = tiles < max_groups ? tiles : max_groups;
  if (wperm) {
    hipLaunchKernelGGL((mxfp4_a8_gemm_kernel<BM, BN, WM, WN, false, true>), dim3(grid), dim3(64 * WM * WN), 0, stream,
                       a8, as, w, c, m, n, k, n_begin, n_end, need);
  } else if (need != nullptr) {
    hipLaunchKernelGGL((mxfp4_a8_gemm_kernel<BM, BN, WM, WN, true>), dim3(grid), dim3(64 * WM * WN), 0, stream,
                       a8, as, w, c, m, n, k, n_begin, n_end, need);
  } else {
    hipLaunchKernelGGL((mxfp4_a8_gemm_kernel<BM, BN, WM, WN, false>), dim3(grid), dim3(64 * WM * WN), 0, stream,
                       a8, as, w, c, m, n, k, n_begin, n_end, need);
  }
}

// Tiled launch of C = diag(as) . A8 . deq(W)^T; `need` non-null selects the split-activation form.
void launch_tiles(const uint8_t* a8, const float* as, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                  uint32_t k, const uint8_t* need, bool wperm, hipStream_t stream) {
  const uint32_t cus = static_cast<uint32_t>(num_cus());
  const uint32_t tiles_m = (m + 255u) / 256u, tiles_n = (n + 255u) / 256u;
  const uint32_t tiles = tiles_m * tiles_n;
  uint32_t main_tn = tiles_n;
  if (tiles > cus && tiles % cus != 0 && tiles % cus <= cus / 2) {
    main_tn = (tiles / cus) * cus / tiles_m;
  } else if (tiles < cus / 2) {
    main_tn = 0;                        // too few large tiles to fill the chip: small tiles throughout
  }
  const uint32_t n_split = main_tn * 256u < n ? main_tn * 256u : n;
  if (n_split > 0) launch_range<256, 256, 4, 2>(a8, as, w, c, m, n, k, 0u, n_split, cus, need, wperm, stream);
  if (n_split < n) launch_range<128, 64, 2, 2>(a8, as, w, c, m, n, k, n_split, n, 2u * cus, need, wperm, stream);
}

}  // namespace

// The bulk of C goes to persistent 256 x 256 tiles, whole rounds of one tile per CU; the
// columns left over when the tile count is not a multiple of the CU count would keep a
// few CUs busy for a whole extra round, so they are cut into 128 x 64 tiles that spread
// over every CU instead (two such workgroups share a CU).
hipError_t launch_mxfp4_a8_gemm(const uint8_t* a8, const float* as, const uint8_t* w, float* c,
                                uint32_t m, uint32_t n, uint32_t k, hipStream_t stream) {
  if (m <= 32 && k % 512 == 0) {
    const uint32_t rows = stream_rows_per_workgroup(n);
    const dim3 grid((n + rows - 1u) / rows), block(128u * ((rows + 15u) / 16u));
    if (m <= 16) {
      hipLaunchKernelGGL(mxfp4_a8_stream_kernel<1>, grid, block, 0, stream, a8, as, w, c, m, n, k, rows);
    } else {
      hipLaunchKernelGGL(mxfp4_a8_stream_kernel<2>, grid, block, 0, stream, a8, as, w, c, m, n, k, rows);
    }
    return hipGetLastError();
  }
  if (m <= 32 && k >= 128u * kSkinnyWaves) {   // every wavefront of the K split has a step
    const dim3 grid((n + 63u) / 64u), block(64 * kSkinnyWaves);
    if (m <= 16) {
      hipLaunchKernelGGL(mxfp4_a8_skinny_kernel<1>, grid, block, 0, stream, a8, as, w, c, m, n, k);
    } else {
      hipLaunchKernelGGL(mxfp4_a8_skinny_kernel<2>, grid, block, 0, stream, a8, as, w, c, m, n, k);
    }
    return hipGetLastError();
  }
  launch_tiles(a8, as, w, c, m, n, k, nullptr, false, stream);
  return hipGetLastError();
}

// The tiled kernel on weights in the reference's fragment order (n a multiple of 16, more than 32 rows).
bool gemm_mxfp4_a8_wperm_supported(uint64_t m, uint64_t n, uint64_t k) {
  return m > 32 && n % 16 == 0 && k >= 1024 && gemm_mxfp4_a8_supported(k);
}
hipError_t launch_mxfp4_a8_gemm_wperm(const uint8_t* a8, const float* as, const uint8_t* w, float* c, uint32_t m,
                                      uint32_t n, uint32_t k, hipStream_t stream) {
  launch_tiles(a8, as, w, c, m, n, k, nullptr, true, stream);
  return hipGetLastError();
}

bool gemm_mxfp4_f32_supported(uint64_t m, uint64_t k) { return m >= 17 && k >= 1024 && gemm_mxfp4_a8_supported(k); }

// 2..16 fp32 rows: the same E4M3 terms through the streamed kernel, eight rows (32 matrix rows) a pass.
bool gemm_mxfp4_f32_rows_supported(uint64_t m, uint64_t n, uint64_t k) {
  return m >= 2 && m <= 16 && k % 512 == 0 && k <= (1u << 20) && n >= 16 &&
         static_cast<uint64_t>(kMaxTerms) * m * k <= 0xFFFFFFFFull;
}
size_t gemm_mxfp4_f32_rows_workspace_bytes(uint64_t m, uint64_t k) { return gemm_mxfp4_f32_workspace_bytes(m, k); }

hipError_t launch_mxfp4_f32_rows(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m, uint32_t n,
                                 uint32_t k, hipStream_t stream) {
  uint8_t* planes = static_cast<uint8_t*>(workspace);
  float* as = reinterpret_cast<float*>(planes + static_cast<size_t>(kMaxTerms) * m * k);
  uint8_t* need = reinterpret_cast<uint8_t*>(as) + ((static_cast<size_t>(m) * 4 + 255) / 256) * 256;
  launch_split_rows(a, planes, as, need, m, k, stream);
  const uint32_t rows = stream_rows_per_workgroup(n);
  const dim3 grid((n + rows - 1u) / rows), block(128u * ((rows + 15u) / 16u));
  const uint64_t plane = static_cast<uint64_t>(m) * k;
  for (uint32_t r0 = 0; r0 < m; r0 += 8u) {
    const uint32_t real = m - r0 < 8u ? m - r0 : 8u;
    const uint8_t* a8 = planes + static_cast<size_t>(r0) * k;
    float* out = c + static_cast<size_t>(r0) * n;
    if (real <= 4u) {
      hipLaunchKernelGGL((mxfp4_a8_stream_kernel<1, true>), grid, block, 0, stream, a8, as + r0, w, out, kMaxTerms * real, n,
                         k, rows, plane);
    } else {
      hipLaunchKernelGGL((mxfp4_a8_stream_kernel<2, true>), grid, block, 0, stream, a8, as + r0, w, out, kMaxTerms * real, n,
                         k, rows, plane);
    }
  }
  return hipGetLastError();
}

size_t gemm_mxfp4_f32_workspace_bytes(uint64_t m, uint64_t k) {
  return static_cast<size_t>(kMaxTerms) * m * k + ((m * 4 + 255) / 256) * 256 + ((m + 255) / 256) * 256;
}

hipError_t launch_mxfp4_f32_gemm(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m,
                                 uint32_t n, uint32_t k, hipStream_t stream) {
  uint8_t* planes = static_cast<uint8_t*>(workspace);
  float* as = reinterpret_cast<float*>(planes + static_cast<size_t>(kMaxTerms) * m * k);
  uint8_t* need = reinterpret_cast<uint8_t*>(as) + ((static_cast<size_t>(m) * 4 + 255) / 256) * 256;
  launch_split_rows(a, planes, as, need, m, k, stream);
  launch_tiles(planes, as, w, c, m, n, k, need, false, stream);
  return hipGetLastError();
}

// ---- "gemm_fp8" with 2..16 fp32 rows on the scaled matrix instruction ---------------------------------
bool gemm_fp8_f32_rows_supported(uint64_t m, uint64_t n, uint64_t k) {
  return m >= 2 && m <= 16 && k % 512 == 0 && k <= (1u << 20) && n >= 16 && n <= 0x7FFFFFFFull &&
         static_cast<uint64_t>(kMaxTerms) * m * k <= 0xFFFFFFFFull;
}

hipError_t gemm_fp8_f32_rows_prepare() {
  const int lim = 160 * 1024 - 1024;
  const void* kernels[4] = {reinterpret_cast<const void*>(fp8_terms_stream_kernel<1>),
                            reinterpret_cast<const void*>(fp8_terms_stream_kernel<2>),
                            reinterpret_cast<const void*>(fp8_terms_stream_kernel<1, true>),
                            reinterpret_cast<const void*>(fp8_terms_stream_kernel<2, true>)};
  for (const void* kern : kernels) {
    const hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lim);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// Workspace as for the MXFP4 rows: the term planes, the rows' powers of two, the term counts.
hipError_t launch_fp8_f32_rows(const float* a, const uint8_t* w, const float* wscale, float* c, void* workspace,
                               uint32_t m, uint32_t n, uint32_t k, bool block_scales, hipStream_t stream) {
  uint8_t* planes = static_cast<uint8_t*>(workspace);
  float* as = reinterpret_cast<float*>(planes + static_cast<size_t>(kMaxTerms) * m * k);
  uint8_t* need = reinterpret_cast<uint8_t*>(as) + ((static_cast<size_t>(m) * 4 + 255) / 256) * 256;
  launch_split_rows(a, planes, as, need, m, k, stream);
  const uint64_t plane = static_cast<uint64_t>(m) * k;
  for (uint32_t r0 = 0; r0 < m; r0 += 8u) {
    const uint32_t real = m - r0 < 8u ? m - r0 : 8u;
    const uint32_t mt = real <= 4u ? 1u : 2u;
    // rows of a workgroup: what the stage ring leaves room for (a row takes 512 bytes of weights a stage,
    // 16 more with block scales)
    const uint32_t rows = fp8_rows_per_workgroup(n, mt == 1u ? 80u : (block_scales ? 68u : 72u));
    const dim3 grid((n + rows - 1u) / rows), block(128u * ((rows + 15u) / 16u));
    const uint32_t lds = 3u * (rows * (block_scales ? 528u : 512u) + mt * 16u * 512u);
    const uint8_t* a8 = planes + static_cast<size_t>(r0) * k;
    float* out = c + static_cast<size_t>(r0) * n;
    const uint32_t mrows = kMaxTerms * real;
    if (mt == 1u && !block_scales) {
      hipLaunchKernelGGL((fp8_terms_stream_kernel<1>), grid, block, lds, stream, a8, as + r0, w, wscale, out, mrows, n, k, rows, plane);
    } else if (!block_scales) {
      hipLaunchKernelGGL((fp8_terms_stream_kernel<2>), grid, block, lds, stream, a8, as + r0, w, wscale, out, mrows, n, k, rows, plane);
    } else if (mt == 1u) {
      hipLaunchKernelGGL((fp8_terms_stream_kernel<1, true>), grid, block, lds, stream, a8, as + r0, w, wscale, out, mrows, n, k, rows, plane);
    } else {
      hipLaunchKernelGGL((fp8_terms_stream_kernel<2, true>), grid, block, lds, stream, a8, as + r0, w, wscale, out, mrows, n, k, rows, plane);
    }
  }
  return hipGetLastError();
}

}  // namespace qmm
