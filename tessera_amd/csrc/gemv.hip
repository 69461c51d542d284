// Decode-regime GEMV for block-quantized weights on gfx950 (wave64, no MFMA).
//
// C[r, j] = sum_t A[r, t] * deq(W)[j, t] for a handful of activation rows r.
//
// The weight stream is the cost (HBM-bound), so the mapping is built around it:
//   * a row of W is cut into 16-byte "chunks"; thread t of a workgroup owns chunk
//     (t mod chunks_per_row) of every weight row the workgroup visits, so one
//     workgroup reads whole rows as contiguous 128-bit loads, row after row;
//   * because a thread's position along K never changes, its slice of the
//     activations is loaded once and lives in registers for the whole kernel (an
//     LDS- or cache-fed activation would cost 8 bytes of on-chip traffic per weight
//     byte and cap the kernel below the HBM rate);
//   * each thread's partial dot products are reduced across the wavefront with
//     cross-lane shuffles and across the wavefronts of the workgroup through a
//     few floats of LDS, one barrier per U weight rows, in a fixed order
//     (deterministic, no atomics).
// Codecs plug the block format into this skeleton.

#include <type_traits>

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

// Where a codec reads fp32 activations from: straight from global memory ...
struct GlobalX {
  const float* a;
  uint32_t k;
  __device__ __forceinline__ float4 operator()(int r, uint32_t elem) const {
    return *reinterpret_cast<const float4*>(a + static_cast<size_t>(r) * k + elem);
  }
};
// ... or from a piece of the activation rows staged in LDS.  A thread's slice is a
// few hundred contiguous bytes, so reading it straight from global memory makes every
// lane of a load touch its own cache line; the staged copy is filled with coalesced
// loads and padded by 4 floats per 64 so the strided reads spread over the banks.
struct StagedX {
  const float* lds;
  uint32_t base;    // first element of the staged piece
  uint32_t stride;  // padded floats per staged row
  static __device__ __forceinline__ uint32_t pad(uint32_t e) { return e + (e >> 6) * 4u; }
  __device__ __forceinline__ float4 operator()(int r, uint32_t elem) const {
    return *reinterpret_cast<const float4*>(lds + r * stride + pad(elem - base));
  }
};

// Per-thread byte offsets of a chunk relative to the (wavefront-uniform) start of a
// row group; the uniform part goes through scalar registers, so a load is one
// global_load with an SGPR base and a 32-bit VGPR offset.
struct Lane {
  uint32_t off0;
  uint32_t off1;
};

// ----------------------------------------------------------------------------
// Q4_K: 144-byte super-block = fp16 d, fp16 dmin, 12 bytes of 6-bit scales/mins,
// 128 quant bytes (reference layout: src/core/numerics/quant.hpp:11-15, decode
// src/core/numerics/quant.cpp:58-70,656-675).  A chunk is 16 quant bytes: chunk j
// of a block covers elements g*64 + h*16 + [0,16) in its low nibbles and the same
// + 32 in its high nibbles (g = j / 2, h = j % 2), i.e. half of sub-blocks 2g and
// 2g+1.
//
// sum_i x_i * (d*sc*q_i - dmin*mn) = d * sc * sum_i x_i q_i - dmin * mn * sum_i x_i,
// and sum_i x_i is a per-thread constant, so the inner loop is one fma per nibble.
// Nibbles become floats without integer->float converts: a nibble masked in place
// inside a 16-bit lane is the fp16 subnormal q * 2^-24 (q * 2^-20 for a nibble at
// bits 4..7, for which the activation is pre-divided by 16), which v_fma_mix_f32
// consumes directly; 2^24 is folded into d.  Every product that is exact in the
// reference decode stays exact here, so a one-hot activation returns the reference's
// dequantized weight bit for bit.
// ----------------------------------------------------------------------------
struct Q4KCodec {
  struct Args {
    const float* a;
    const uint8_t* w;
    uint32_t k;
  };
  template <int R>
  struct X {
    float lo[R][16];
    float hi[R][16];  // activation / 16
    float slo[R];
    float shi[R];
    uint32_t sh;      // 0 or 16: bit offset of the sub-block pair inside a scale word
    uint32_t lm, hm;  // byte-pair masks: 0x3F3F / 0 for groups 0,1; 0x0F0F / 0x3030 for 2,3
    bool upper;       // groups 2,3
  };
  struct Frag {
    uint4 q;
    uint4 h;
  };

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / 32u; }
  // Whether the skeleton stages fp32 activations through LDS for this codec, and the
  // first activation element a chunk needs (its slice stays inside that 64-aligned group
  // or starts there).
  static constexpr bool kStageX = true;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return (chunk >> 1) * 64u; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    const uint32_t blk = chunk >> 3, j = chunk & 7u, g = j >> 1;
    x.sh = (g & 1u) * 16u;
    x.upper = g >= 2u;
    x.lm = x.upper ? 0x0F0Fu : 0x3F3Fu;
    x.hm = x.upper ? 0x3030u : 0u;
    const uint32_t k0 = blk * 256u + g * 64u + (j & 1u) * 16u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float sl = 0.0f, sh = 0.0f;
#pragma unroll
      for (int i = 0; i < 16; i += 4) {
        float4 lo = src(r, k0 + i);
        float4 hi = src(r, k0 + 32 + i);
        if (!valid) lo = hi = make_float4(0.f, 0.f, 0.f, 0.f);
        x.lo[r][i] = lo.x, x.lo[r][i + 1] = lo.y, x.lo[r][i + 2] = lo.z, x.lo[r][i + 3] = lo.w;
        x.hi[r][i] = hi.x, x.hi[r][i + 1] = hi.y, x.hi[r][i + 2] = hi.z, x.hi[r][i + 3] = hi.w;
      }
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        sl += x.lo[r][i];
        sh += x.hi[r][i];
        x.hi[r][i] *= 0.0625f;
      }
      x.slo[r] = sl;
      x.shi[r] = sh;
    }
  }

  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk,
                                                   uint32_t prow) {
    const uint32_t hdr = prow * (cpr >> 3) * 144u + (chunk >> 3) * 144u;
    return Lane{hdr, hdr + 16u + (chunk & 7u) * 16u};
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f) {
    const uint8_t* base = p.w + static_cast<size_t>(row) * ((cpr >> 3) * 144u);
    f.h = load_u4(base + ln.off0);
    f.q = load_u4(base + ln.off1);
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    // 6-bit scale/min of sub-blocks 2g and 2g+1, kept as byte pairs (2g in byte 0,
    // 2g+1 in byte 1).  Groups 0,1 read six bits straight from bytes 2g, 2g+1 (+4 for
    // the mins); groups 2,3 join a nibble of bytes 8.. with the top two bits of the
    // bytes that groups 0,1 use.
    const uint32_t s0 = f.h.y, s1 = f.h.z, s2 = f.h.w;
    const uint32_t ls = x.upper ? s2 : s0;
    const uint32_t lmn = x.upper ? (s2 >> 4) : s1;
    const uint32_t sc2 = ((ls >> x.sh) & x.lm) | ((s0 >> (x.sh + 2u)) & x.hm);
    const uint32_t mn2 = ((lmn >> x.sh) & x.lm) | ((s1 >> (x.sh + 2u)) & x.hm);
    const float sca = static_cast<float>(sc2 & 0xFFu), scb = static_cast<float>((sc2 >> 8) & 0xFFu);
    const float mna = static_cast<float>(mn2 & 0xFFu), mnb = static_cast<float>((mn2 >> 8) & 0xFFu);
    const float d24 = half_bits_to_float(f.h.x & 0xFFFFu) * 0x1p24f;  // undoes the 2^-24 below
    const float dmin = half_bits_to_float(f.h.x >> 16);
    const uint32_t qw[4] = {f.q.x, f.q.y, f.q.z, f.q.w};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float al = 0.0f, ah = 0.0f;
#pragma unroll
      for (int wi = 0; wi < 4; ++wi) {
        const uint32_t w = qw[wi], w8 = w >> 8;
        const half2_t l02 = bit_cast<half2_t>(w & 0x000F000Fu);   // bytes 0,2 low nibbles
        const half2_t h02 = bit_cast<half2_t>(w & 0x00F000F0u);   // bytes 0,2 high nibbles * 16
        const half2_t l13 = bit_cast<half2_t>(w8 & 0x000F000Fu);  // bytes 1,3 low nibbles
        const half2_t h13 = bit_cast<half2_t>(w8 & 0x00F000F0u);  // bytes 1,3 high nibbles * 16
        al = fmaf(x.lo[r][4 * wi + 0], static_cast<float>(l02[0]), al);
        ah = fmaf(x.hi[r][4 * wi + 0], static_cast<float>(h02[0]), ah);
        al = fmaf(x.lo[r][4 * wi + 1], static_cast<float>(l13[0]), al);
        ah = fmaf(x.hi[r][4 * wi + 1], static_cast<float>(h13[0]), ah);
        al = fmaf(x.lo[r][4 * wi + 2], static_cast<float>(l02[1]), al);
        ah = fmaf(x.hi[r][4 * wi + 2], static_cast<float>(h02[1]), ah);
        al = fmaf(x.lo[r][4 * wi + 3], static_cast<float>(l13[1]), al);
        ah = fmaf(x.hi[r][4 * wi + 3], static_cast<float>(h13[1]), ah);
      }
      const float t1 = fmaf(scb, ah, sca * al);
      const float t2 = fmaf(mnb, x.shi[r], mna * x.slo[r]);
      out[r] = fmaf(d24, t1, -(dmin * t2));
    }
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args&, uint32_t, int, float v) {
    return v;
  }
};

// ----------------------------------------------------------------------------
// Routed-expert variants of the Q4_K codec (mixture-of-experts feed-forward; reference
// kernels src/backends/rocm/rocm_kernels_moe.cpp:15-79, launch protocol
// src/models/qwen3_5/moe.cpp:396-423).  Expert tensors are expert-major: expert e of a
// tensor starts `stride` bytes after expert e-1, rows inside it are ordinary Q4_K rows.
// The selected expert ids live in device memory, so the weight row is looked up in the
// kernel.  `batch` moves every per-token pointer to token y (grid.y).
// ----------------------------------------------------------------------------

// Gate and up of the `top_k` selected experts in one pass: output row slot*inter + j is row j of
// expert ids[slot]; a wavefront loads its activations once, takes that row of both tensors and
// stores silu(G x) * (U x) (the reference's single "moe_experts_gate_up_q4k" launch,
// src/backends/rocm/rocm_kernels_moe.cpp:15-49).
struct Q4KExpertGateUpCodec : Q4KCodec {
  static constexpr bool kTwoMatrices = true;
  struct Args {
    const float* a;
    const uint8_t* w;      // gate
    uint32_t k;            // hidden
    const uint32_t* ids;
    uint64_t stride;       // gate expert stride
    uint32_t inter, top_k;
    uint32_t n_experts;
    const uint8_t* up;
    uint64_t up_stride;
  };
  static __device__ __forceinline__ void batch(Args& p, uint32_t y) {
    p.a += static_cast<size_t>(y) * p.k;
    p.ids += static_cast<size_t>(y) * p.top_k;
  }
  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    Q4KCodec::load_x<R>(Q4KCodec::Args{p.a, p.w, p.k}, chunk, valid, x, src);
  }
  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk, uint32_t prow) {
    return Q4KCodec::make_lane(Q4KCodec::Args{}, cpr, chunk, prow);
  }
  // which = 0: gate, 1: up
  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row, uint32_t cpr,
                                              Frag& f, int which = 0) {
    const uint32_t slot = row / p.inter, j = row - slot * p.inter;
    const uint32_t e = p.ids[slot] < p.n_experts ? p.ids[slot] : p.n_experts - 1u;
    const uint8_t* base = (which ? p.up + e * p.up_stride : p.w + e * p.stride) +
                          static_cast<size_t>(j) * ((cpr >> 3) * 144u);
    f.h = load_u4(base + ln.off0);
    f.q = load_u4(base + ln.off1);
  }
  static __device__ __forceinline__ float combine(float g, float u) { return (g / (1.0f + expf(-g))) * u; }
};

// Down projection of the selected experts, summed with the routing weights:
// out[j] = sum_slot wts[slot] * (D_ids[slot] phi_slot)[j].  One output row is treated as a
// single dot product over K = top_k * inter whose weight blocks come from top_k experts and
// whose activations (phi, contiguous slot by slot) are scaled by their slot's weight.
struct Q4KExpertDownCodec : Q4KCodec {
  struct Args {
    const float* a;        // phi, top_k x inter
    const uint8_t* w;
    uint32_t k;            // top_k * inter
    const uint32_t* ids;
    uint64_t stride;
    uint32_t inter, top_k, hidden;
    uint32_t n_experts;    // ids are clamped below this
    const float* wts;
    const float* prev;     // the output itself when accumulating, else null
  };
  static __device__ __forceinline__ void batch(Args& p, uint32_t y) {
    p.a += static_cast<size_t>(y) * p.k;
    p.ids += static_cast<size_t>(y) * p.top_k;
    p.wts += static_cast<size_t>(y) * p.top_k;
    if (p.prev != nullptr) p.prev += static_cast<size_t>(y) * p.hidden;
  }
  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    Q4KCodec::load_x<R>(Q4KCodec::Args{p.a, p.w, p.k}, chunk, valid, x, src);
    const float wt = p.wts[chunk / (p.inter / 32u)];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        x.lo[r][i] *= wt;
        x.hi[r][i] *= wt;
      }
      x.slo[r] *= wt;
      x.shi[r] *= wt;
    }
  }
  // Offsets are relative to row 0 of expert 0; they stay below 4 GB (checked by the caller).
  static __device__ __forceinline__ Lane make_lane(const Args& p, uint32_t, uint32_t chunk, uint32_t prow) {
    const uint32_t per_slot = p.inter / 32u, slot = chunk / per_slot, cin = chunk - slot * per_slot;
    const uint32_t e = p.ids[slot] < p.n_experts ? p.ids[slot] : p.n_experts - 1u;
    const uint32_t hdr = static_cast<uint32_t>(e * p.stride) + prow * (p.inter / 256u) * 144u +
                         (cin >> 3) * 144u;
    return Lane{hdr, hdr + 16u + (cin & 7u) * 16u};
  }
  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row, uint32_t, Frag& f) {
    const uint8_t* base = p.w + static_cast<size_t>(row) * ((p.inter / 256u) * 144u);
    f.h = load_u4(base + ln.off0);
    f.q = load_u4(base + ln.off1);
  }
  template <int R>
  static __device__ __forceinline__ float finish(const Args& p, uint32_t row, int, float v) {
    return p.prev != nullptr ? p.prev[row] + v : v;
  }
};

// ----------------------------------------------------------------------------
// Q4_K, single activation row: the same arithmetic with a 32-byte chunk per thread
// (one whole group g of a block: sub-block 2g in the low nibbles, 2g+1 in the high
// nibbles), so the header decode, the cross-lane reduction and the loop overhead are
// paid once per 64 weights instead of once per 32.
// ----------------------------------------------------------------------------
struct Q4KPairCodec {
  using Args = Q4KCodec::Args;
  static constexpr bool kBalanceSimds = true;  // the decode, not the loads, paces the loop
  template <int R>
  struct X {
    float lo[R][32];
    float hi[R][32];
    float slo[R];
    float shi[R];
    uint32_t sh;
    uint32_t lm, hm;
    bool upper;
  };
  struct Frag {
    uint4 h;
    uint4 q0;
    uint4 q1;
  };

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / 64u; }
  // Whether the skeleton stages fp32 activations through LDS for this codec, and the
  // first activation element a chunk needs (its slice stays inside that 64-aligned group
  // or starts there).
  static constexpr bool kStageX = true;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return chunk * 64u; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    const uint32_t blk = chunk >> 2, g = chunk & 3u;
    x.sh = (g & 1u) * 16u;
    x.upper = g >= 2u;
    x.lm = x.upper ? 0x0F0Fu : 0x3F3Fu;
    x.hm = x.upper ? 0x3030u : 0u;
    const uint32_t k0 = blk * 256u + g * 64u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float sl = 0.0f, sh = 0.0f;
#pragma unroll
      for (int i = 0; i < 32; i += 4) {
        float4 lo = src(r, k0 + i);
        float4 hi = src(r, k0 + 32 + i);
        if (!valid) lo = hi = make_float4(0.f, 0.f, 0.f, 0.f);
        x.lo[r][i] = lo.x, x.lo[r][i + 1] = lo.y, x.lo[r][i + 2] = lo.z, x.lo[r][i + 3] = lo.w;
        x.hi[r][i] = hi.x, x.hi[r][i + 1] = hi.y, x.hi[r][i + 2] = hi.z, x.hi[r][i + 3] = hi.w;
      }
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        sl += x.lo[r][i];
        sh += x.hi[r][i];
      }
      x.slo[r] = sl;
      x.shi[r] = sh;
    }
  }

  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk,
                                                   uint32_t prow) {
    const uint32_t hdr = prow * (cpr >> 2) * 144u + (chunk >> 2) * 144u;
    return Lane{hdr, hdr + 16u + (chunk & 3u) * 32u};
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f) {
    const uint8_t* base = p.w + static_cast<size_t>(row) * ((cpr >> 2) * 144u);
    f.h = load_u4(base + ln.off0);
    f.q0 = load_u4(base + ln.off1);
    f.q1 = load_u4(base + ln.off1 + 16u);
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    const uint32_t s0 = f.h.y, s1 = f.h.z, s2 = f.h.w;
    const uint32_t ls = x.upper ? s2 : s0;
    const uint32_t lmn = x.upper ? (s2 >> 4) : s1;
    const uint32_t sc2 = ((ls >> x.sh) & x.lm) | ((s0 >> (x.sh + 2u)) & x.hm);
    const uint32_t mn2 = ((lmn >> x.sh) & x.lm) | ((s1 >> (x.sh + 2u)) & x.hm);
    const float sca = static_cast<float>(sc2 & 0xFFu), scb = static_cast<float>((sc2 >> 8) & 0xFFu);
    const float mna = static_cast<float>(mn2 & 0xFFu), mnb = static_cast<float>((mn2 >> 8) & 0xFFu);
    const float d24 = half_bits_to_float(f.h.x & 0xFFFFu) * 0x1p24f;
    const float dmin = half_bits_to_float(f.h.x >> 16);
    const uint32_t qw[8] = {f.q0.x, f.q0.y, f.q0.z, f.q0.w, f.q1.x, f.q1.y, f.q1.z, f.q1.w};
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float al = 0.0f, ah = 0.0f;
#pragma unroll
      for (int wi = 0; wi < 8; ++wi) {
        const uint32_t w = qw[wi], w8 = w >> 8;
        const half2_t l02 = bit_cast<half2_t>(w & 0x000F000Fu);
        const half2_t h02 = bit_cast<half2_t>(w & 0x00F000F0u);
        const half2_t l13 = bit_cast<half2_t>(w8 & 0x000F000Fu);
        const half2_t h13 = bit_cast<half2_t>(w8 & 0x00F000F0u);
        al = fmaf(x.lo[r][4 * wi + 0], static_cast<float>(l02[0]), al);
        ah = fmaf(x.hi[r][4 * wi + 0], static_cast<float>(h02[0]), ah);
        al = fmaf(x.lo[r][4 * wi + 1], static_cast<float>(l13[0]), al);
        ah = fmaf(x.hi[r][4 * wi + 1], static_cast<float>(h13[0]), ah);
        al = fmaf(x.lo[r][4 * wi + 2], static_cast<float>(l02[1]), al);
        ah = fmaf(x.hi[r][4 * wi + 2], static_cast<float>(h02[1]), ah);
        al = fmaf(x.lo[r][4 * wi + 3], static_cast<float>(l13[1]), al);
        ah = fmaf(x.hi[r][4 * wi + 3], static_cast<float>(h13[1]), ah);
      }
      // the high nibbles were masked in place (16 q): their 1/16 goes to the sub-block's scale, exactly
      const float t1 = fmaf(scb * 0.0625f, ah, sca * al);
      const float t2 = fmaf(mnb, x.shi[r], mna * x.slo[r]);
      out[r] = fmaf(d24, t1, -(dmin * t2));
    }
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args&, uint32_t, int, float v) {
    return v;
  }
};

// Gate and up projection of a dense feed-forward block in one pass, ending in
// silu(G x) * (U x) (the dense analogue of the routed-expert gate/up pass above; the
// reference runs two GEMVs and the "silu_mul" kernel, src/backends/rocm/rocm_kernels_basic.cpp:1882-1891).
// The two matrices share the skeleton's two pipeline stages: stage 0 holds the group's rows of
// the gate matrix, stage 1 the same rows of the up matrix, so both dot products of an output
// element are reduced in the same round and the thread that stores it has both, while the group
// shape (rows side by side, wavefronts per workgroup) stays the single-matrix one.  The
// activations are loaded once for the two matrices.
struct Q4KGateUpCodec : Q4KPairCodec {
  static constexpr bool kPairStages = true;
  struct Args {
    const float* a;
    const uint8_t* w;      // gate
    uint32_t k;
    const uint8_t* up;
  };
  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    Q4KPairCodec::load_x<R>(Q4KPairCodec::Args{p.a, p.w, p.k}, chunk, valid, x, src);
  }
  static __device__ __forceinline__ Lane make_lane(const Args& p, uint32_t cpr, uint32_t chunk, uint32_t prow) {
    return Q4KPairCodec::make_lane(Q4KPairCodec::Args{p.a, p.w, p.k}, cpr, chunk, prow);
  }
  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f, int stage) {
    const uint8_t* base = (stage ? p.up : p.w) + static_cast<size_t>(row) * ((cpr >> 2) * 144u);
    f.h = load_u4(base + ln.off0);
    f.q0 = load_u4(base + ln.off1);
    f.q1 = load_u4(base + ln.off1 + 16u);
  }
  static __device__ __forceinline__ float combine(float g, float u) { return (g / (1.0f + expf(-g))) * u; }
};

// Whether a codec spreads two matrices over the two pipeline stages (see Q4KGateUpCodec).
template <class Codec, class = void>
struct pair_stages : std::false_type {};
template <class Codec>
struct pair_stages<Codec, std::void_t<decltype(Codec::kPairStages)>> : std::bool_constant<Codec::kPairStages> {};

// Q4_K, single activation row, K cut into `gridDim.y` slices: workgroups of slice s take columns
// [s*k, (s+1)*k) of every weight row (k = the slice length) and write their partial dot products
// to output region s, so a workgroup stages only its slice of the activations and the caller's
// reduce over the regions ("gemm_vec_reduce", src/core/decode_internal.hpp:840-923) finishes the sum.
struct Q4KSliceCodec : Q4KPairCodec {
  static constexpr bool kSlices = true;
  struct Args {
    const float* a;
    const uint8_t* w;
    uint32_t k;           // slice length
    uint32_t row_bytes;   // bytes of a whole weight row
  };
  static __device__ __forceinline__ void select_slice(Args& p, uint32_t slice) {
    p.a += static_cast<size_t>(slice) * p.k;
    p.w += static_cast<size_t>(slice) * (p.k / 256u) * 144u;
  }
  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    Q4KPairCodec::load_x<R>(Q4KPairCodec::Args{p.a, p.w, p.k}, chunk, valid, x, src);
  }
  static __device__ __forceinline__ Lane make_lane(const Args& p, uint32_t, uint32_t chunk, uint32_t prow) {
    const uint32_t hdr = prow * p.row_bytes + (chunk >> 2) * 144u;
    return Lane{hdr, hdr + 16u + (chunk & 3u) * 32u};
  }
  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row, uint32_t, Frag& f) {
    const uint8_t* base = p.w + static_cast<size_t>(row) * p.row_bytes;
    f.h = load_u4(base + ln.off0);
    f.q0 = load_u4(base + ln.off1);
    f.q1 = load_u4(base + ln.off1 + 16u);
  }
  template <int R>
  static __device__ __forceinline__ float finish(const Args&, uint32_t, int, float v) {
    return v;
  }
};
template <class Codec, class = void>
struct k_slices : std::false_type {};
template <class Codec>
struct k_slices<Codec, std::void_t<decltype(Codec::kSlices)>> : std::bool_constant<Codec::kSlices> {};

// ----------------------------------------------------------------------------
// Q5_K: 176-byte super-block = fp16 d, fp16 dmin, 12 bytes of 6-bit scales/mins (packed as in
// Q4_K), qh[32] fifth bits, qs[128] low nibbles; value = d*sc*(nibble + 16*bit) - dmin*mn
// (reference decode src/core/numerics/quant.cpp:388-419, layout quant.hpp:592-595).  A chunk is
// one 64-weight group g of a block, as in Q4KPairCodec: 32 bytes of qs (sub-block 2g in the low
// nibbles, 2g+1 in the high nibbles) plus bits 2g and 2g+1 of the block's 32 qh bytes, which all
// four chunks of a block load.  Four five-bit quants are assembled per register with byte masks
// and converted with v_cvt_f32_ubyte*; d*sc, dmin*mn and sc*q are exact in fp32, so a one-hot
// activation returns the reference's dequantized weight bit for bit.
// ----------------------------------------------------------------------------
struct Q5KCodec {
  static constexpr bool kBalanceSimds = true;
  using Args = Q4KCodec::Args;
  template <int R>
  struct X {
    float lo[R][32];
    float hi[R][32];
    float slo[R];
    float shi[R];
    uint32_t sh;       // scale words: bit offset of the sub-block pair
    uint32_t lm, hm;   // scale byte-pair masks, as in Q4KPairCodec
    uint32_t hs;       // 2g: position of the group's bit pair in a qh byte
    bool upper;
  };
  struct Frag {
    uint4 h;
    uint4 qh0, qh1;
    uint4 q0, q1;
  };

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / 64u; }
  static constexpr bool kStageX = true;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return chunk * 64u; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    const uint32_t blk = chunk >> 2, g = chunk & 3u;
    x.sh = (g & 1u) * 16u;
    x.upper = g >= 2u;
    x.lm = x.upper ? 0x0F0Fu : 0x3F3Fu;
    x.hm = x.upper ? 0x3030u : 0u;
    x.hs = 2u * g;
    const uint32_t k0 = blk * 256u + g * 64u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float sl = 0.0f, sh = 0.0f;
#pragma unroll
      for (int i = 0; i < 32; i += 4) {
        float4 lo = src(r, k0 + i);
        float4 hi = src(r, k0 + 32 + i);
        if (!valid) lo = hi = make_float4(0.f, 0.f, 0.f, 0.f);
        x.lo[r][i] = lo.x, x.lo[r][i + 1] = lo.y, x.lo[r][i + 2] = lo.z, x.lo[r][i + 3] = lo.w;
        x.hi[r][i] = hi.x, x.hi[r][i + 1] = hi.y, x.hi[r][i + 2] = hi.z, x.hi[r][i + 3] = hi.w;
        sl += (lo.x + lo.y) + (lo.z + lo.w);
        sh += (hi.x + hi.y) + (hi.z + hi.w);
      }
      x.slo[r] = sl;
      x.shi[r] = sh;
    }
  }

  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk,
                                                   uint32_t prow) {
    const uint32_t hdr = prow * (cpr >> 2) * 176u + (chunk >> 2) * 176u;
    return Lane{hdr, hdr + 48u + (chunk & 3u) * 32u};
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f) {
    const uint8_t* base = p.w + static_cast<size_t>(row) * ((cpr >> 2) * 176u);
    f.h = load_u4(base + ln.off0);
    f.qh0 = load_u4(base + ln.off0 + 16u);
    f.qh1 = load_u4(base + ln.off0 + 32u);
    f.q0 = load_u4(base + ln.off1);
    f.q1 = load_u4(base + ln.off1 + 16u);
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    const uint32_t s0 = f.h.y, s1 = f.h.z, s2 = f.h.w;
    const uint32_t ls = x.upper ? s2 : s0;
    const uint32_t lmn = x.upper ? (s2 >> 4) : s1;
    const uint32_t sc2 = ((ls >> x.sh) & x.lm) | ((s0 >> (x.sh + 2u)) & x.hm);
    const uint32_t mn2 = ((lmn >> x.sh) & x.lm) | ((s1 >> (x.sh + 2u)) & x.hm);
    const float sca = static_cast<float>(sc2 & 0xFFu), scb = static_cast<float>((sc2 >> 8) & 0xFFu);
    const float mna = static_cast<float>(mn2 & 0xFFu), mnb = static_cast<float>((mn2 >> 8) & 0xFFu);
    const float d = half_bits_to_float(f.h.x & 0xFFFFu);
    const float dmin = half_bits_to_float(f.h.x >> 16);
    const uint32_t qw[8] = {f.q0.x, f.q0.y, f.q0.z, f.q0.w, f.q1.x, f.q1.y, f.q1.z, f.q1.w};
    const uint32_t hw[8] = {f.qh0.x, f.qh0.y, f.qh0.z, f.qh0.w, f.qh1.x, f.qh1.y, f.qh1.z, f.qh1.w};
    float al[R], ah[R];
#pragma unroll
    for (int r = 0; r < R; ++r) al[r] = ah[r] = 0.0f;
#pragma unroll
    for (int wi = 0; wi < 8; ++wi) {
      const uint32_t w = qw[wi], t = hw[wi] >> x.hs;
      const uint32_t lo4 = (w & 0x0F0F0F0Fu) | ((t & 0x01010101u) << 4);
      const uint32_t hi4 = ((w >> 4) & 0x0F0F0F0Fu) | ((t << 3) & 0x10101010u);
      const float l0 = static_cast<float>(lo4 & 0xFFu), l1 = static_cast<float>((lo4 >> 8) & 0xFFu);
      const float l2 = static_cast<float>((lo4 >> 16) & 0xFFu), l3 = static_cast<float>(lo4 >> 24);
      const float h0 = static_cast<float>(hi4 & 0xFFu), h1 = static_cast<float>((hi4 >> 8) & 0xFFu);
      const float h2 = static_cast<float>((hi4 >> 16) & 0xFFu), h3 = static_cast<float>(hi4 >> 24);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        al[r] = fmaf(x.lo[r][4 * wi + 0], l0, al[r]);
        ah[r] = fmaf(x.hi[r][4 * wi + 0], h0, ah[r]);
        al[r] = fmaf(x.lo[r][4 * wi + 1], l1, al[r]);
        ah[r] = fmaf(x.hi[r][4 * wi + 1], h1, ah[r]);
        al[r] = fmaf(x.lo[r][4 * wi + 2], l2, al[r]);
        ah[r] = fmaf(x.hi[r][4 * wi + 2], h2, ah[r]);
        al[r] = fmaf(x.lo[r][4 * wi + 3], l3, al[r]);
        ah[r] = fmaf(x.hi[r][4 * wi + 3], h3, ah[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float t1 = fmaf(scb, ah[r], sca * al[r]);
      const float t2 = fmaf(mnb, x.shi[r], mna * x.slo[r]);
      out[r] = fmaf(d, t1, -(dmin * t2));
    }
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args&, uint32_t, int, float v) {
    return v;
  }
};

// ----------------------------------------------------------------------------
// Q6_K: 210-byte super-block = ql[128] low nibbles, qh[64] two high bits each, 16 int8
// scales, fp16 d; value = d * s * (q - 32) (reference decode src/core/numerics/quant.cpp:421-450,
// layout quant.hpp:597-600, device twin src/backends/rocm/rocm_kernels_codec.hpp:132-176).
// A chunk is 64 weights: half n of the block, lanes l = is*16 .. is*16+15 of its four quarters
// (chunk = 4*block + 2*n + is), i.e. 16 bytes of ql at n*64 + is*16, 16 more 32 bytes further,
// 16 bytes of qh at 128 + n*32 + is*16, and the scales n*8 + is + {0,2,4,6}.  Blocks are only
// 2-byte aligned (210 = 2 * 105), so every load is an unaligned one.
//
// sum_i x_i * d*s*(q_i - 32) = d * s * (sum_i x_i q_i - 32 * sum_i x_i) per quarter, the second
// sum a per-thread constant.  The six-bit q of four lanes is assembled in one register (byte
// masks and shifts) and converted with v_cvt_f32_ubyte*.  d*s and s*(q-32) are exact in fp32, so
// a one-hot activation returns the reference's dequantized weight bit for bit.
// ----------------------------------------------------------------------------
struct Q6KCodec {
  static constexpr bool kBalanceSimds = true;
  struct Args {
    const float* a;
    const uint8_t* w;
    uint32_t k;
  };
  template <int R>
  struct X {
    float v[R][4][16];   // quarter j, lane l - is*16
    float s32[R][4];     // 32 * sum over the 16 lanes of quarter j
    uint32_t sc_shift;   // is * 8: byte of the scale words
  };
  struct Frag {
    uint4 ql0, ql1, qh;
    uint2 sc;            // the eight scales of half n
    uint32_t d;          // fp16 bits
  };
  typedef uint4 uint4_u __attribute__((aligned(2)));
  typedef uint2 uint2_u __attribute__((aligned(2)));

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / 64u; }
  static constexpr bool kStageX = true;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return (chunk >> 1) * 128u; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    const uint32_t is = chunk & 1u;
    x.sc_shift = is * 8u;
    const uint32_t k0 = (chunk >> 1) * 128u + is * 16u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i += 4) {
          float4 f = src(r, k0 + j * 32 + i);
          if (!valid) f = make_float4(0.f, 0.f, 0.f, 0.f);
          x.v[r][j][i] = f.x, x.v[r][j][i + 1] = f.y, x.v[r][j][i + 2] = f.z, x.v[r][j][i + 3] = f.w;
          sum += (f.x + f.y) + (f.z + f.w);
        }
        x.s32[r][j] = 32.0f * sum;
      }
    }
  }

  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk,
                                                   uint32_t prow) {
    const uint32_t blk = prow * (cpr >> 2) * 210u + (chunk >> 2) * 210u;
    const uint32_t n = (chunk >> 1) & 1u, is = chunk & 1u;
    return Lane{blk, n * 64u + is * 16u};   // block start; offset of this chunk's first ql bytes
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f) {
    const uint8_t* blk = p.w + static_cast<size_t>(row) * ((cpr >> 2) * 210u) + ln.off0;
    const uint32_t n = ln.off1 >> 6, is16 = ln.off1 & 16u;
    f.ql0 = *reinterpret_cast<const uint4_u*>(blk + ln.off1);
    f.ql1 = *reinterpret_cast<const uint4_u*>(blk + ln.off1 + 32u);
    f.qh = *reinterpret_cast<const uint4_u*>(blk + 128u + n * 32u + is16);
    f.sc = *reinterpret_cast<const uint2_u*>(blk + 192u + n * 8u);
    f.d = *reinterpret_cast<const uint16_t*>(blk + 208u);
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    const float d = half_bits_to_float(f.d);
    // scales n*8 + is + {0,2,4,6}: bytes is, is+2 of each word
    const uint32_t w0 = f.sc.x >> x.sc_shift, w1 = f.sc.y >> x.sc_shift;
    const float s[4] = {static_cast<float>(static_cast<int8_t>(w0 & 0xFFu)),
                        static_cast<float>(static_cast<int8_t>((w0 >> 16) & 0xFFu)),
                        static_cast<float>(static_cast<int8_t>(w1 & 0xFFu)),
                        static_cast<float>(static_cast<int8_t>((w1 >> 16) & 0xFFu))};
    const uint32_t a4[4] = {f.ql0.x, f.ql0.y, f.ql0.z, f.ql0.w};
    const uint32_t b4[4] = {f.ql1.x, f.ql1.y, f.ql1.z, f.ql1.w};
    const uint32_t h4[4] = {f.qh.x, f.qh.y, f.qh.z, f.qh.w};
    float acc[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[r][j] = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t a = a4[i], b = b4[i], h = h4[i];
      const uint32_t q[4] = {(a & 0x0F0F0F0Fu) | ((h & 0x03030303u) << 4),
                             (b & 0x0F0F0F0Fu) | ((h & 0x0C0C0C0Cu) << 2),
                             ((a >> 4) & 0x0F0F0F0Fu) | (h & 0x30303030u),
                             ((b >> 4) & 0x0F0F0F0Fu) | ((h >> 2) & 0x30303030u)};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float q0 = static_cast<float>(q[j] & 0xFFu), q1 = static_cast<float>((q[j] >> 8) & 0xFFu);
        const float q2 = static_cast<float>((q[j] >> 16) & 0xFFu), q3 = static_cast<float>(q[j] >> 24);
#pragma unroll
        for (int r = 0; r < R; ++r) {
          acc[r][j] = fmaf(x.v[r][j][4 * i + 0], q0, acc[r][j]);
          acc[r][j] = fmaf(x.v[r][j][4 * i + 1], q1, acc[r][j]);
          acc[r][j] = fmaf(x.v[r][j][4 * i + 2], q2, acc[r][j]);
          acc[r][j] = fmaf(x.v[r][j][4 * i + 3], q3, acc[r][j]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float t = 0.0f;
#pragma unroll
      for (int j = 0; j < 4; ++j) t = fmaf(d * s[j], acc[r][j] - x.s32[r][j], t);
      out[r] = t;
    }
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args&, uint32_t, int, float v) {
    return v;
  }
};

// Down projection of the selected experts with Q6_K expert tensors (reference kernel
// src/backends/rocm/rocm_kernels_moe.cpp:81-110, loaded next to the Q4_K one by
// src/models/qwen3_5/moe.cpp:107-115): a row is one dot product over top_k * inter, slot s
// reading expert ids[s], with the routing weight folded into the activations.
struct Q6KExpertDownCodec : Q6KCodec {
  using Args = Q4KExpertDownCodec::Args;
  static __device__ __forceinline__ void batch(Args& p, uint32_t y) { Q4KExpertDownCodec::batch(p, y); }
  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
    Q6KCodec::load_x<R>(Q6KCodec::Args{p.a, p.w, p.k}, chunk, valid, x, src);
    const float wt = p.wts[chunk / (p.inter / 64u)];
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int i = 0; i < 16; ++i) x.v[r][j][i] *= wt;
        x.s32[r][j] *= wt;
      }
    }
  }
  // Offsets are relative to row 0 of expert 0; they stay below 4 GB (checked by the caller).
  static __device__ __forceinline__ Lane make_lane(const Args& p, uint32_t, uint32_t chunk, uint32_t) {
    const uint32_t per_slot = p.inter / 64u, slot = chunk / per_slot, cin = chunk - slot * per_slot;
    const uint32_t e = p.ids[slot] < p.n_experts ? p.ids[slot] : p.n_experts - 1u;
    const uint32_t blk = static_cast<uint32_t>(e * p.stride) + (cin >> 2) * 210u;
    return Lane{blk, ((cin >> 1) & 1u) * 64u + (cin & 1u) * 16u};
  }
  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row, uint32_t, Frag& f) {
    const uint8_t* blk = p.w + static_cast<size_t>(row) * ((p.inter / 256u) * 210u) + ln.off0;
    const uint32_t n = ln.off1 >> 6, is16 = ln.off1 & 16u;
    f.ql0 = *reinterpret_cast<const uint4_u*>(blk + ln.off1);
    f.ql1 = *reinterpret_cast<const uint4_u*>(blk + ln.off1 + 32u);
    f.qh = *reinterpret_cast<const uint4_u*>(blk + 128u + n * 32u + is16);
    f.sc = *reinterpret_cast<const uint2_u*>(blk + 192u + n * 8u);
    f.d = *reinterpret_cast<const uint16_t*>(blk + 208u);
  }
  template <int R>
  static __device__ __forceinline__ float finish(const Args& p, uint32_t row, int, float v) {
    return p.prev != nullptr ? p.prev[row] + v : v;
  }
};

// ----------------------------------------------------------------------------
// MXFP4 with fp32 activations: packed buffer = n*k/2 nibble bytes (low nibble =
// even element) then n*k/32 E8M0 bytes (include/tessera/backend.hpp:195-201;
// src/core/numerics/gemm.cpp:311-344).  A 16-byte chunk is exactly one 32-element
// block, so the E8M0 scale multiplies the chunk's partial sum once.
// ----------------------------------------------------------------------------
struct MxFp4Codec {
  struct Args {
    const float* a;
    const uint8_t* w;
    const uint8_t* s;  // w + n*k/2
    uint32_t k;
  };
  template <int R>
  struct X {
    float v[R][32];
  };
  struct Frag {
    uint4 q;
    uint32_t s;
  };

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / 32u; }
  // Whether the skeleton stages fp32 activations through LDS for this codec, and the
  // first activation element a chunk needs (its slice stays inside that 64-aligned group
  // or starts there).
  static constexpr bool kStageX = true;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return chunk * 32u; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int i = 0; i < 32; i += 4) {
        float4 v = src(r, chunk * 32u + i);
        if (!valid) v = make_float4(0.f, 0.f, 0.f, 0.f);
        x.v[r][i] = v.x, x.v[r][i + 1] = v.y, x.v[r][i + 2] = v.z, x.v[r][i + 3] = v.w;
      }
    }
  }

  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk,
                                                   uint32_t prow) {
    const uint32_t c = prow * cpr + chunk;
    return Lane{c * 16u, c};
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f) {
    const size_t c = static_cast<size_t>(row) * cpr;
    f.q = load_u4(p.w + c * 16u + ln.off0);
    f.s = (p.s + c)[ln.off1];
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    const uint32_t qw[4] = {f.q.x, f.q.y, f.q.z, f.q.w};
    float2_t wv[16];
#pragma unroll
    for (int wi = 0; wi < 4; ++wi) {
      wv[4 * wi + 0] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[wi], 1.0f, 0);
      wv[4 * wi + 1] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[wi], 1.0f, 1);
      wv[4 * wi + 2] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[wi], 1.0f, 2);
      wv[4 * wi + 3] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[wi], 1.0f, 3);
    }
    const float scale = e8m0_to_float(f.s);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
      for (int b = 0; b < 16; ++b) {
        a0 = fmaf(x.v[r][2 * b], wv[b][0], a0);
        a1 = fmaf(x.v[r][2 * b + 1], wv[b][1], a1);
      }
      out[r] = (a0 + a1) * scale;
    }
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args&, uint32_t, int, float v) {
    return v;
  }
};

// MXFP4, single activation row: two MX blocks (64 weights, 32 nibble bytes, two scale bytes) per
// thread, so the reduction, the scale loads and the loop overhead are paid once per 64 weights
// (as Q4KPairCodec does for Q4_K).  K must be a multiple of 64.
struct MxFp4PairCodec {
  static constexpr bool kBalanceSimds = true;
  using Args = MxFp4Codec::Args;
  template <int R>
  struct X {
    float v[R][64];
  };
  struct Frag {
    uint4 q0, q1;
    uint32_t s;   // two E8M0 bytes
  };

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / 64u; }
  static constexpr bool kStageX = true;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return chunk * 64u; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args&, uint32_t chunk, bool valid, X<R>& x, const Src& src) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int i = 0; i < 64; i += 4) {
        float4 v = src(r, chunk * 64u + i);
        if (!valid) v = make_float4(0.f, 0.f, 0.f, 0.f);
        x.v[r][i] = v.x, x.v[r][i + 1] = v.y, x.v[r][i + 2] = v.z, x.v[r][i + 3] = v.w;
      }
    }
  }

  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk, uint32_t prow) {
    const uint32_t c = prow * cpr + chunk;
    return Lane{c * 32u, c * 2u};
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row, uint32_t cpr, Frag& f) {
    const size_t c = static_cast<size_t>(row) * cpr;
    const uint8_t* base = p.w + c * 32u + ln.off0;
    f.q0 = load_u4(base);
    f.q1 = load_u4(base + 16u);
    f.s = *reinterpret_cast<const uint16_t*>(p.s + c * 2u + ln.off1);
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    const uint32_t qw[8] = {f.q0.x, f.q0.y, f.q0.z, f.q0.w, f.q1.x, f.q1.y, f.q1.z, f.q1.w};
    const float scale[2] = {e8m0_to_float(f.s & 0xFFu), e8m0_to_float(f.s >> 8)};
#pragma unroll
    for (int r = 0; r < R; ++r) out[r] = 0.0f;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      float2_t wv[16];
#pragma unroll
      for (int wi = 0; wi < 4; ++wi) {
        wv[4 * wi + 0] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[4 * h + wi], 1.0f, 0);
        wv[4 * wi + 1] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[4 * h + wi], 1.0f, 1);
        wv[4 * wi + 2] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[4 * h + wi], 1.0f, 2);
        wv[4 * wi + 3] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(qw[4 * h + wi], 1.0f, 3);
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
        for (int b = 0; b < 16; ++b) {
          a0 = fmaf(x.v[r][32 * h + 2 * b], wv[b][0], a0);
          a1 = fmaf(x.v[r][32 * h + 2 * b + 1], wv[b][1], a1);
        }
        out[r] = fmaf(a0 + a1, scale[h], out[r]);
      }
    }
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args&, uint32_t, int, float v) {
    return v;
  }
};

// ----------------------------------------------------------------------------
// W4A8: MXFP4 weights, activations already quantized per token to E4M3 codes with
// one fp32 scale per row (quantize_fp8_pack).  The weight side is lossless:
// C[r, j] = As[r] * sum_b 2^(s_b - 127) * sum_{t in b} e4m3(a_t) * e2m1(w_t), which is
// the reference's QuantizeFp8Ref followed by GemmMxFp4Ref
// (src/core/numerics/quant.cpp:180-205, src/core/numerics/gemm.cpp:311-344) up to
// summation order.  Both operands convert exactly to fp16 and v_dot2_f32_f16 takes
// two products per instruction with fp32 accumulation.
// ----------------------------------------------------------------------------
struct MxFp4A8Codec {
  struct Args {
    const uint8_t* a;   // m x k e4m3 codes
    const float* as;    // m per-row scales
    const uint8_t* w;
    const uint8_t* s;
    uint32_t k;
  };
  template <int R>
  struct X {
    half2_t v[R][16];
  };
  struct Frag {
    uint4 q;
    uint32_t s;
  };

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / 32u; }
  // Whether the skeleton stages fp32 activations through LDS for this codec, and the
  // first activation element a chunk needs (its slice stays inside that 64-aligned group
  // or starts there).
  static constexpr bool kStageX = false;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return chunk * 32u; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint8_t* src = p.a + static_cast<size_t>(r) * p.k + chunk * 32u;
      uint4 c0 = load_u4(src), c1 = load_u4(src + 16);
      if (!valid) c0 = c1 = make_uint4(0, 0, 0, 0);
      const uint32_t cw[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        x.v[r][2 * i] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(cw[i], 1.0f, false);
        x.v[r][2 * i + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(cw[i], 1.0f, true);
      }
    }
  }

  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk,
                                                   uint32_t prow) {
    const uint32_t c = prow * cpr + chunk;
    return Lane{c * 16u, c};
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f) {
    const size_t c = static_cast<size_t>(row) * cpr;
    f.q = load_u4(p.w + c * 16u + ln.off0);
    f.s = (p.s + c)[ln.off1];
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    const uint32_t qw[4] = {f.q.x, f.q.y, f.q.z, f.q.w};
    half2_t wv[16];
#pragma unroll
    for (int wi = 0; wi < 4; ++wi) {
      wv[4 * wi + 0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw[wi], 1.0f, 0);
      wv[4 * wi + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw[wi], 1.0f, 1);
      wv[4 * wi + 2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw[wi], 1.0f, 2);
      wv[4 * wi + 3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(qw[wi], 1.0f, 3);
    }
    const float scale = e8m0_to_float(f.s);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float a0 = 0.0f, a1 = 0.0f;
#pragma unroll
      for (int b = 0; b < 16; b += 2) {
        a0 = __builtin_amdgcn_fdot2(wv[b], x.v[r][b], a0, false);
        a1 = __builtin_amdgcn_fdot2(wv[b + 1], x.v[r][b + 1], a1, false);
      }
      out[r] = (a0 + a1) * scale;
    }
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args& p, uint32_t, int r, float v) {
    return v * p.as[r];
  }
};

// ----------------------------------------------------------------------------
// FP8 E4M3 weights (n x k bytes) with one fp32 scale per weight row
// (include/tessera/backend.hpp:191-194; src/core/numerics/gemm.cpp:253-277).
// A chunk is 16 weights; the row scale multiplies the finished dot product.
// ----------------------------------------------------------------------------
// NQ = 16-byte pieces per chunk: a lane takes 16 * NQ consecutive weights of a row.  One piece
// for rows up to 16384 long, two beyond (a row must fit the 1024 threads of a workgroup).
// BLOCK: `s` holds one scale per 128 x 128 block of W instead ("gemm_fp8_block",
// include/tessera/backend.hpp:183-186; src/core/numerics/gemm.cpp:282-309): a chunk lies inside
// one block, so its partial dot product takes the block's scale before the lanes are summed.
template <int NQ, bool BLOCK = false>
struct Fp8CodecT {
  struct Args {
    const float* a;
    const uint8_t* w;
    const float* s;
    uint32_t k;
  };
  static constexpr uint32_t kChunk = 16u * NQ;
  template <int R>
  struct X {
    float v[R][16 * NQ];
  };
  struct Frag {
    uint4 q[NQ];
    float bs;   // BLOCK: the scale of the chunk's block
  };

  static __host__ __device__ __forceinline__ uint32_t chunks_per_row(uint32_t k) { return k / kChunk; }
  // Whether the skeleton stages fp32 activations through LDS for this codec, and the
  // first activation element a chunk needs (its slice stays inside that 64-aligned group
  // or starts there).
  static constexpr bool kStageX = true;
  static __device__ __forceinline__ uint32_t x_elem0(uint32_t chunk) { return chunk * kChunk; }

  template <int R, class Src>
  static __device__ __forceinline__ void load_x(const Args& p, uint32_t chunk, bool valid, X<R>& x,
                                                const Src& src) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
      for (int i = 0; i < 16 * NQ; i += 4) {
        float4 v = src(r, chunk * kChunk + i);
        if (!valid) v = make_float4(0.f, 0.f, 0.f, 0.f);
        x.v[r][i] = v.x, x.v[r][i + 1] = v.y, x.v[r][i + 2] = v.z, x.v[r][i + 3] = v.w;
      }
    }
  }

  // off1 (BLOCK): the lane's row inside the group and the 128-wide K block of its chunk
  static __device__ __forceinline__ Lane make_lane(const Args&, uint32_t cpr, uint32_t chunk,
                                                   uint32_t prow) {
    return Lane{(prow * cpr + chunk) * kChunk, BLOCK ? prow | ((chunk * kChunk / 128u) << 8) : 0u};
  }

  static __device__ __forceinline__ void load(const Args& p, const Lane& ln, uint32_t row,
                                              uint32_t cpr, Frag& f) {
    const uint8_t* base = p.w + static_cast<size_t>(row) * cpr * kChunk + ln.off0;
#pragma unroll
    for (int j = 0; j < NQ; ++j) f.q[j] = load_u4(base + 16 * j);
    if constexpr (BLOCK) f.bs = p.s[static_cast<size_t>((row + (ln.off1 & 0xFFu)) >> 7) * (p.k >> 7) + (ln.off1 >> 8)];
  }

  template <int R>
  static __device__ __forceinline__ void dot(const Frag& f, const X<R>& x, float (&out)[R]) {
    float a0[R], a1[R];
#pragma unroll
    for (int r = 0; r < R; ++r) a0[r] = a1[r] = 0.0f;
#pragma unroll
    for (int j = 0; j < NQ; ++j) {           // one 16-byte piece at a time keeps few converted values live
      const uint32_t qw[4] = {f.q[j].x, f.q[j].y, f.q[j].z, f.q[j].w};
      float2_t wv[8];
#pragma unroll
      for (int wi = 0; wi < 4; ++wi) {
        wv[2 * wi] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(qw[wi], 1.0f, false);
        wv[2 * wi + 1] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(qw[wi], 1.0f, true);
      }
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int b = 0; b < 8; ++b) {
          a0[r] = fmaf(x.v[r][16 * j + 2 * b], wv[b][0], a0[r]);
          a1[r] = fmaf(x.v[r][16 * j + 2 * b + 1], wv[b][1], a1[r]);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) out[r] = BLOCK ? (a0[r] + a1[r]) * f.bs : a0[r] + a1[r];
  }

  template <int R>
  static __device__ __forceinline__ float finish(const Args& p, uint32_t row, int, float v) {
    return BLOCK ? v : v * p.s[row];
  }
};
using Fp8Codec = Fp8CodecT<1>;
using Fp8WideCodec = Fp8CodecT<2>;
using Fp8QuadCodec = Fp8CodecT<4>;   // one activation row: 64 weights a lane

// ----------------------------------------------------------------------------
// The skeleton.  A workgroup owns a contiguous range of row groups; a group is P
// weight rows laid side by side over the threads (P * chunks_per_row slots, so the
// lanes stay full when a row's chunk count is not a multiple of 64).  Each thread
// keeps D row fragments in registers as a software pipeline: fragment d is consumed
// and at once refilled with the group D steps ahead, so D loads per thread stay in
// flight while the arithmetic runs.  One barrier per D groups publishes the
// per-wavefront partial sums; a few threads then add them in wavefront order and
// store (deterministic, no atomics).
// ----------------------------------------------------------------------------
template <class Codec, int R, int P, int D, int MAXT, uint32_t XP, bool LR = false>
__global__ __launch_bounds__(MAXT) void gemv_kernel(typename Codec::Args args, float* __restrict__ c,
                                                    uint32_t n, uint32_t cpr, uint32_t ldc,
                                                    uint32_t groups_per_wg) {
  // LR (rows shorter than a wavefront, whose lanes may then belong to three or more rows): a
  // lane leaves its partial in LDS and sixteen lanes per output add a row's partials after the
  // barrier.  Otherwise each wavefront reduces its (at most two) rows itself, which is faster
  // when rows are long.
  constexpr int kMaxWaves = MAXT / kWave;
  static_assert(MAXT <= 1024, "the row of a thread is found by a float division that is exact up to 1024");
  __shared__ float red[2][D][P][R][LR ? 1 : kMaxWaves];
  // Rows whose chunk count is a multiple of 16: an aligned run of 16 lanes never straddles two
  // rows, so one four-step sum per run replaces the two masked six-step sums over the wavefront,
  // and the threads that store add a row's runs instead of its wavefronts.
  __shared__ float red16[2][D][R][LR ? 1 : MAXT / 16];
  __shared__ float part[2][D][R][LR ? MAXT : 1];

  if constexpr (k_slices<Codec>::value) {     // blockIdx.y = K slice and output region
    Codec::select_slice(args, blockIdx.y);
    c += static_cast<size_t>(blockIdx.y) * R * ldc;
  }
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const uint32_t slots = P * cpr;
  const bool valid = t < slots;
  // t / cpr for t < 1024: (t + 1/2) / cpr is at least 1 / (2 cpr) away from an integer, far more than
  // the reciprocal's rounding moves it
  const uint32_t prow = valid ? static_cast<uint32_t>((static_cast<float>(t) + 0.5f) * __builtin_amdgcn_rcpf(static_cast<float>(cpr))) : 0u;
  const uint32_t chunk = valid ? t - prow * cpr : 0u;

  // Which of the P rows this wavefront's lanes belong to: at most two when a row has at least
  // 64 chunks (shorter rows take the LR path, which does not use these).
  const uint32_t first_slot = wave * 64u;
  const uint32_t last_slot = first_slot + 63u < slots ? first_slot + 63u : slots - 1u;
  const uint32_t row_a = first_slot / cpr, row_b = last_slot / cpr;
  const bool two = row_a != row_b;  // wavefront-uniform
  // Which sum a lane's partial goes into.  Selected, never multiplied by a 0/1 mask: a NaN or an
  // infinity among one row's weights must not reach its neighbour's sum (0 * inf = NaN), nor may
  // what an idle lane computed from the chunk it loaded for company.
  const bool to_a = valid && prow == row_a, to_b = valid && prow != row_a;
  const bool by16 = (cpr & 15u) == 0u;   // uniform

  // Groups [g0, g1) belong to this workgroup.  A group index past its end is clamped to its
  // last group for the loads (a prefetch must not pull the next workgroup's rows, which would
  // come from HBM a second time through another XCD's L2) and dropped at the store; rows past
  // n inside the last group re-read the group's first row.
  // A paired codec gives the two stages of the pipeline to its two matrices: a round then
  // covers one group (both matrices) instead of D groups.
  constexpr bool kPaired = pair_stages<Codec>::value;
  static_assert(!kPaired || D == 2, "a paired codec uses exactly two stages");
  constexpr uint32_t PR = P;
  constexpr uint32_t kGroupsPerRound = kPaired ? 1u : static_cast<uint32_t>(D);
  const uint32_t groups = (n + PR - 1) / PR;
  const uint32_t g0 = blockIdx.x * groups_per_wg;
  const uint32_t g1 = g0 + groups_per_wg < groups ? g0 + groups_per_wg : groups;
  const Lane ln = Codec::make_lane(args, cpr, chunk, prow);
  const Lane ln_tail = Codec::make_lane(args, cpr, chunk, (groups - 1u) * PR + prow < n ? prow : 0u);
  const bool ragged = n % PR != 0;
  // Stage d of the round that starts at group `gbase`: group gbase + d, or matrix d of gbase.
  auto fetch = [&](uint32_t gbase, int d, typename Codec::Frag& f) {
    uint32_t grp = kPaired ? gbase : gbase + static_cast<uint32_t>(d);
    grp = grp < g1 ? grp : g1 - 1u;
    const bool tail = ragged && grp == groups - 1u;
    if constexpr (kPaired) {
      Codec::load(args, tail ? ln_tail : ln, grp * PR, cpr, f, d);
    } else {
      Codec::load(args, tail ? ln_tail : ln, grp * PR, cpr, f);
    }
  };

  typename Codec::Frag frag[D];
  // Invalid lanes (past the last chunk) carry zero activations, so they add nothing.
  typename Codec::template X<R> x;
  if constexpr (Codec::kStageX) {
    constexpr uint32_t kPiece = XP;           // floats of one activation row resident in LDS
    constexpr uint32_t kStride = kPiece + kPiece / 16u;
    constexpr int kXPer = XP > 8192u ? 8 : 4; // float4 a thread may carry of a short activation row
    __shared__ __attribute__((aligned(16))) float xs[R * kStride];
    const uint32_t k = args.k;
    const uint32_t mine = Codec::x_elem0(chunk);
    if (R == 1 && k <= kPiece && k <= kXPer * 4u * blockDim.x) {   // uniform
      // Short single row: its loads are requested BEFORE the weight prefetch.  Loads return in
      // order, so requested after it they would sit behind D fragments per lane (over 100 KB
      // per workgroup) and the first dot product would start microseconds later.  Only the
      // first stage of weights is requested before the barrier, the others right after it: with
      // all D requested up front, the slowest wavefront's activations arrive behind everybody
      // else's burst (a third of a 50 MB matrix), the barrier opens when the burst has drained
      // and the memory system idles while the first stage is computed (3-4 % per launch).
      // (named registers, not an array: across the barrier below an array stays in scratch memory)
      auto x_load = [&](int i) {
        const uint32_t e = (t + i * blockDim.x) * 4u;
        return *reinterpret_cast<const float4*>(args.a + (e < k ? e : k - 4u));
      };
      auto x_store = [&](int i, const float4& v) {
        const uint32_t e = (t + i * blockDim.x) * 4u;
        if (e < k) *reinterpret_cast<float4*>(&xs[StagedX::pad(e)]) = v;
      };
      static_assert(kXPer == 4 || kXPer == 8, "x0..x7 below");
      const float4 x0 = x_load(0), x1 = x_load(1), x2 = x_load(2), x3 = x_load(3);
      float4 x4 = x0, x5 = x0, x6 = x0, x7 = x0;
      if constexpr (kXPer == 8) x4 = x_load(4), x5 = x_load(5), x6 = x_load(6), x7 = x_load(7);
      // A long row (the down projection: 70 KB to stage, 4 us before the first dot product) wants
      // the weights of two stages under way meanwhile.  A barrier that waits for nothing makes
      // sure every wavefront's activation requests are out before any weights, so that no
      // wavefront's activations queue behind the others' weights: 5120 x 17408 15.5 -> 13.8 us.
      // Short rows measured slower with two stages early (Q6_K 17408 x 5120: 19.0 -> 21.3 us) and
      // keep one stage, but take the barrier too (17408 x 5120: 12.23 -> 11.88 us).
      constexpr bool kTwoStagesEarly = kXPer == 8 && D > 1;
      {
        __builtin_amdgcn_sched_barrier(0);
        asm volatile("s_barrier");
        __builtin_amdgcn_sched_barrier(0);
      }
      fetch(g0, 0, frag[0]);
      if constexpr (kTwoStagesEarly) fetch(g0, 1, frag[1]);
      x_store(0, x0), x_store(1, x1), x_store(2, x2), x_store(3, x3);
      if constexpr (kXPer == 8) x_store(4, x4), x_store(5, x5), x_store(6, x6), x_store(7, x7);
      lds_barrier();
#pragma unroll
      for (int d = kTwoStagesEarly ? 2 : 1; d < D; ++d) fetch(g0, d, frag[d]);
      Codec::template load_x<R>(args, chunk, valid, x, StagedX{xs, 0u, kStride});
    } else {
      // Weight loads first, activations second: both are in flight before anything waits.
#pragma unroll
      for (int d = 0; d < D; ++d) fetch(g0, d, frag[d]);
      for (uint32_t base = 0; base < k; base += kPiece) {
        const uint32_t len = k - base < kPiece ? k - base : kPiece;
        if (base != 0) lds_barrier();  // the previous piece has been read
#pragma unroll
        for (int r = 0; r < R; ++r) {
          for (uint32_t e = t * 4u; e < len; e += blockDim.x * 4u) {
            *reinterpret_cast<float4*>(&xs[r * kStride + StagedX::pad(e)]) =
                *reinterpret_cast<const float4*>(args.a + static_cast<size_t>(r) * k + base + e);
          }
        }
        lds_barrier();
        if (mine >= base && mine < base + len) {
          Codec::template load_x<R>(args, chunk, valid, x, StagedX{xs, base, kStride});
        }
      }
    }
  } else {
#pragma unroll
    for (int d = 0; d < D; ++d) fetch(g0, d, frag[d]);
    Codec::template load_x<R>(args, chunk, valid, x, 0);
  }

  uint32_t buf = 0;
  // One round = D pipeline stages, one barrier.  `refill` rounds reload every
  // fragment they consume (unconditionally, so the compiler can count outstanding loads
  // exactly and never waits for more than the one fragment it needs); the last round
  // loads nothing and skips stages past the range.
  auto round_wave = [&](uint32_t g, auto refill) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (!kPaired && !decltype(refill)::value && g + d >= g1) break;
      float v[R];
      Codec::template dot<R>(frag[d], x, v);
      if constexpr (decltype(refill)::value) fetch(g + kGroupsPerRound, d, frag[d]);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        if (by16) {
          const float s16 = row16_sum(valid ? v[r] : 0.0f);
          if ((lane & 15u) == 0u) red16[buf][d][r][t >> 4] = s16;
        } else if (two) {
          const float sa = wave_sum_last(to_a ? v[r] : 0.0f);
          const float sb = wave_sum_last(to_b ? v[r] : 0.0f);
          if (lane == 63u) {
            red[buf][d][row_a][r][wave] = sa;
            red[buf][d][row_b][r][wave] = sb;
          }
        } else {
          const float sa = wave_sum_last(valid ? v[r] : 0.0f);
          if (lane == 63u) red[buf][d][row_a][r][wave] = sa;
        }
      }
    }
    lds_barrier();  // LDS only: the prefetched global loads stay in flight across it
    if (t < kGroupsPerRound * PR * R) {
      const uint32_t d = t / (PR * R), po = (t / R) % PR, r = t % R;
      const uint32_t row = (g + d) * PR + po;
      if (g + d < g1 && row < n) {
        auto slot_sum = [&](uint32_t stage) {
          float sum = 0.0f;
          if (by16) {
            for (uint32_t q = (po * cpr) >> 4; q < ((po + 1u) * cpr) >> 4; ++q) sum += red16[buf][stage][r][q];
          } else {
            const uint32_t w_lo = (po * cpr) >> 6, w_hi = ((po + 1u) * cpr - 1u) >> 6;
            for (uint32_t w = w_lo; w <= w_hi; ++w) sum += red[buf][stage][po][r][w];
          }
          return sum;
        };
        if constexpr (kPaired) {
          c[static_cast<size_t>(r) * ldc + row] = Codec::combine(slot_sum(0u), slot_sum(1u));
        } else {
          c[static_cast<size_t>(r) * ldc + row] = Codec::template finish<R>(args, row, r, slot_sum(d));
        }
      }
    }
    buf ^= 1u;
  };

  auto round_lds = [&](uint32_t g, auto refill) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      if (!kPaired && !decltype(refill)::value && g + d >= g1) break;
      float v[R];
      Codec::template dot<R>(frag[d], x, v);
      if constexpr (decltype(refill)::value) fetch(g + kGroupsPerRound, d, frag[d]);
      // Selected, never multiplied by a 0/1 mask (see to_a above).
#pragma unroll
      for (int r = 0; r < R; ++r) part[buf][d][r][t] = valid ? v[r] : 0.0f;
    }
    lds_barrier();  // LDS only: the prefetched global loads stay in flight across it
    for (uint32_t o = t >> 4; o < kGroupsPerRound * PR * R; o += blockDim.x >> 4) {
      const uint32_t d = o / (PR * R), po = (o / R) % PR, r = o % R;
      const uint32_t row = (g + d) * PR + po;
      const bool live = g + d < g1 && row < n;
      auto slot_sum = [&](uint32_t stage) {
        const float* src = &part[buf][stage][r][po * cpr];
        float sum = 0.0f;
        if (live) {
          for (uint32_t i = t & 15u; i < cpr; i += 16u) sum += src[i];
        }
        return row16_sum(sum);
      };
      float res;
      if constexpr (kPaired) {
        const float first = slot_sum(0u), second = slot_sum(1u);
        res = Codec::combine(first, second);
      } else {
        res = Codec::template finish<R>(args, live ? row : 0u, r, slot_sum(d));
      }
      if (live && (t & 15u) == 0u) c[static_cast<size_t>(r) * ldc + row] = res;
    }
    buf ^= 1u;
  };
  auto round = [&](uint32_t g, auto refill) {
    if constexpr (LR) round_lds(g, refill); else round_wave(g, refill);
  };

  uint32_t g = g0;
  for (; g + kGroupsPerRound < g1; g += kGroupsPerRound) round(g, std::true_type{});
  if (g < g1) round(g, std::false_type{});
}

// Small-K variant (a row has 8, 16 or 32 chunks): each wavefront owns 64 / cpr whole
// rows per pass and reduces inside aligned lane groups, no LDS and no barrier.
template <class Codec, int R, int U>
__global__ __launch_bounds__(256) void gemv_smallk_kernel(typename Codec::Args args,
                                                          float* __restrict__ c, uint32_t n,
                                                          uint32_t cpr, uint32_t ldc) {
  const uint32_t t = threadIdx.x, lane = t & 63u;
  const uint32_t rows_per_wave = 64u / cpr;
  const uint32_t chunk = lane % cpr, sub = lane / cpr;
  typename Codec::template X<R> x;
  if constexpr (Codec::kStageX) {
    Codec::template load_x<R>(args, chunk, true, x, GlobalX{args.a, args.k});
  } else {
    Codec::template load_x<R>(args, chunk, true, x, 0);
  }
  const Lane ln = Codec::make_lane(args, cpr, chunk, 0u);
  const uint32_t wave_global = blockIdx.x * (blockDim.x >> 6) + (t >> 6);
  const uint32_t waves_total = gridDim.x * (blockDim.x >> 6);
  const uint32_t groups = (n + rows_per_wave - 1) / rows_per_wave;
  for (uint32_t g0 = wave_global; g0 < groups; g0 += waves_total * U) {
    typename Codec::Frag frag[U];
    bool ok[U];
    uint32_t rows[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const uint32_t grp = g0 + u * waves_total;
      rows[u] = grp * rows_per_wave + sub;
      ok[u] = grp < groups && rows[u] < n;
      Codec::load(args, ln, ok[u] ? rows[u] : 0u, cpr, frag[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float v[R];
#pragma unroll
      for (int r = 0; r < R; ++r) v[r] = 0.0f;
      if (ok[u]) Codec::template dot<R>(frag[u], x, v);
#pragma unroll
      for (int r = 0; r < R; ++r) {
        float s = v[r];
        for (uint32_t off = cpr >> 1; off > 0; off >>= 1) {
          s += __shfl_xor(s, off, kWave);
        }
        if (ok[u] && chunk == 0) {
          c[static_cast<size_t>(r) * ldc + rows[u]] = Codec::template finish<R>(args, rows[u], r, s);
        }
      }
    }
  }
}

struct GemvPlan {
  uint32_t cpr;
  uint32_t threads;  // workgroup size, multiple of 64
  uint32_t p;        // weight rows per group
  bool smallk;
};

int g_num_cus = 256;

// Workgroup shape: rows per group P in 1..kMaxP and the thread count P*cpr rounded up
// to whole wavefronts; picks the P that idles the fewest lanes, larger P on ties
// (fewer, fuller workgroups share one copy of the activations).
template <uint32_t kMaxP>
GemvPlan plan_gemv(uint32_t cpr, uint32_t max_threads) {
  GemvPlan g{cpr, 0, 1, false};
  if (cpr == 4 || cpr == 8 || cpr == 16 || cpr == 32) {
    g.smallk = true;
    g.threads = 256;
    return g;
  }
  g.threads = (cpr + 63u) / 64u * 64u;
  if (cpr < 64) return g;  // a wavefront may span at most two rows
  double best = static_cast<double>(cpr) / g.threads;
  for (uint32_t p = 2; p <= kMaxP; ++p) {
    const uint32_t t = (p * cpr + 63u) / 64u * 64u;
    if (t > max_threads) break;
    const double fill = static_cast<double>(p * cpr) / t;
    if (fill >= best) {
      best = fill;
      g.p = p;
      g.threads = t;
    }
  }
  return g;
}

// The same choice for a codec whose loop is bound by its vector arithmetic rather than by the
// loads (kBalanceSimds): a CU runs its wavefronts on four SIMDs, so ten wavefronts put three on
// two of them and the launch lasts as long as those.  Cost of a candidate = wavefronts on the
// fullest SIMD x pipeline stages a workgroup runs; ties are ranked in the loop below, then go
// to fuller wavefronts, then to larger P.  At 17408x5120 Q4_K this picks 9 rows (12 wavefronts,
// 8 stages) over 8 rows (10 wavefronts, 9 stages).
template <uint32_t kMaxP>
GemvPlan plan_gemv_balanced(uint32_t cpr, uint32_t max_threads, uint32_t n) {
  GemvPlan g{cpr, (cpr + 63u) / 64u * 64u, 1, false};
  const uint32_t waves_per_simd = (max_threads / 64u + 3u) / 4u;
  const uint32_t cus = static_cast<uint32_t>(g_num_cus);
  uint64_t best_cost = ~0ull;
  uint32_t best_rank = 0;
  double best_fill = 0.0;
  for (uint32_t p = 1u; p <= kMaxP; ++p) {
    const uint32_t t = (p * cpr + 63u) / 64u * 64u;
    if (t > max_threads) break;
    const uint32_t w = t / 64u;
    uint32_t per_cu = (4u * waves_per_simd) / w;
    if (per_cu == 0) per_cu = 1;
    const uint32_t groups = (n + p - 1u) / p;
    uint32_t grid = cus * per_cu;
    if (grid > groups) grid = groups;
    const uint32_t per_wg = (groups + grid - 1u) / grid;
    grid = (groups + per_wg - 1u) / per_wg;
    const uint32_t resident = (grid + cus - 1u) / cus;
    const uint32_t cu_waves = w * resident;
    const uint64_t cost = static_cast<uint64_t>((cu_waves + 3u) / 4u) * per_wg;
    const double fill = static_cast<double>(p * cpr) / t;
    // Among equal costs: a long loop (four stages or more) likes one workgroup per CU with as
    // many wavefronts as fit (17408x5120: 9 rows, 12 wavefronts, 12.3 us; 6 rows, 8 wavefronts,
    // 12.9); a short one is mostly prologue and likes few wavefronts.
    const uint32_t rank = per_wg >= 4u ? (resident == 1u ? 100u : 0u) + cu_waves : 1000u - cu_waves;
    // Costs within 5 % of each other count as equal (the model is no finer than that:
    // 34816x5120 runs 21.0 us at cost 48 with twelve wavefronts, 21.5 at cost 46 with eight).
    const uint64_t gap = cost > best_cost ? cost - best_cost : best_cost - cost;
    const bool tie = best_cost != ~0ull && 20u * gap <= best_cost;
    const bool better = tie ? (rank > best_rank || (rank == best_rank && fill >= best_fill))
                            : cost < best_cost;
    if (better) best_cost = cost, best_rank = rank, best_fill = fill, g.p = p, g.threads = t;
  }
  return g;
}

template <class Codec, class = void>
struct balance_simds : std::false_type {};
template <class Codec>
struct balance_simds<Codec, std::void_t<decltype(Codec::kBalanceSimds)>> : std::bool_constant<Codec::kBalanceSimds> {};

template <class Codec, int R, int MAXT, int D, uint32_t P>
hipError_t launch_gemv_p(const typename Codec::Args& args, float* c, uint32_t n, uint32_t cpr,
                         uint32_t ldc, uint32_t threads, hipStream_t stream, uint32_t slices = 1) {
  // Resident workgroups per CU under __launch_bounds__(MAXT): the register budget
  // admits ceil(MAXT/256) wavefronts per SIMD whatever the block size.
  const uint32_t waves = threads / 64u;
  const uint32_t waves_per_simd = (MAXT / 64u + 3u) / 4u;
  uint32_t per_cu = (4u * waves_per_simd) / waves;
  if (per_cu == 0) per_cu = 1;
  constexpr uint32_t PR = P;
  const uint32_t groups = (n + PR - 1) / PR;
  uint32_t grid = static_cast<uint32_t>(g_num_cus) * per_cu / slices;     // workgroups per K slice
  if (grid == 0) grid = 1;
  if (grid > groups) grid = groups;
  uint32_t per_wg = (groups + grid - 1) / grid;
  grid = (groups + per_wg - 1) / per_wg;
  // Activation floats per row kept in LDS at a time.  A single long row (the down
  // projection) gets the 136 KB variant so that the whole row is staged by one round of
  // loads instead of three rounds in sequence; those workgroups are alone on their CU anyway.
  constexpr uint32_t kSmall = R == 1 ? 8192u : (R == 2 ? 4096u : 2048u);
  if constexpr (R == 1 && Codec::kStageX) {
    if (args.k > kSmall && args.k <= 32768u && per_cu == 1) {
      hipLaunchKernelGGL((gemv_kernel<Codec, R, P, D, MAXT, 32768u>), dim3(grid, slices), dim3(threads), 0,
                         stream, args, c, n, cpr, ldc, per_wg);
      return hipGetLastError();
    }
  }
  if (cpr < 64u) {
    hipLaunchKernelGGL((gemv_kernel<Codec, R, P, D, MAXT, kSmall, true>), dim3(grid, slices), dim3(threads), 0,
                       stream, args, c, n, cpr, ldc, per_wg);
    return hipGetLastError();
  }
  hipLaunchKernelGGL((gemv_kernel<Codec, R, P, D, MAXT, kSmall>), dim3(grid, slices), dim3(threads), 0, stream,
                     args, c, n, cpr, ldc, per_wg);
  return hipGetLastError();
}

template <class Codec, int R, int MAXT, int D, uint32_t kMaxP = 2>
hipError_t launch_gemv_r(const typename Codec::Args& args, float* c, uint32_t n, uint32_t k,
                         uint32_t ldc, hipStream_t stream, uint32_t slices = 1) {
  const uint32_t cpr = Codec::chunks_per_row(k);
  GemvPlan g = plan_gemv<kMaxP>(cpr, MAXT);
  // Rows shorter than a wavefront (and not of the small-K kernel's lengths) also go side by
  // side in a workgroup: plan_gemv would give each a workgroup of one partly idle wavefront.
  // Several activation rows make every codec's loop arithmetic-bound (a multiply-add per weight
  // and row), so those are planned by SIMD load as well: MXFP4 with four fp32 rows went from 2
  // rows a workgroup (5 wavefronts: 2,1,1,1 on the SIMDs) to 3 (8 wavefronts), 42.5 -> 32.4 us.
  if (!g.smallk && ((balance_simds<Codec>::value && R == 1) || cpr < 64u || R > 1)) {
    g = plan_gemv_balanced<kMaxP>(cpr, MAXT, n * slices);
  }
  if (slices > 1 && g.smallk) return hipErrorInvalidValue;
  if (pair_stages<Codec>::value && g.smallk) return hipErrorInvalidValue;
  if constexpr (!pair_stages<Codec>::value) {
    if (g.smallk) {
      constexpr int U = D > 4 ? 4 : D;
      const uint32_t rows_per_wave = 64u / cpr;
      const uint32_t groups = (n + rows_per_wave - 1) / rows_per_wave;
      uint32_t grid = (groups + 4u * U - 1) / (4u * U);
      const uint32_t cap = static_cast<uint32_t>(g_num_cus) * 8u;
      grid = grid > cap ? cap : (grid == 0 ? 1 : grid);
      hipLaunchKernelGGL((gemv_smallk_kernel<Codec, R, U>), dim3(grid), dim3(256), 0, stream, args, c,
                         n, cpr, ldc);
      return hipGetLastError();
    }
  }
  if (g.threads > MAXT) return hipErrorInvalidValue;
  switch (g.p) {
#define QMM_GEMV_CASE(PP)                                                                       \
  case PP:                                                                                      \
    if constexpr (kMaxP >= PP)                                                                  \
      return launch_gemv_p<Codec, R, MAXT, D, PP>(args, c, n, cpr, ldc, g.threads, stream, slices); \
    break;
    QMM_GEMV_CASE(1) QMM_GEMV_CASE(2) QMM_GEMV_CASE(3) QMM_GEMV_CASE(4) QMM_GEMV_CASE(5) QMM_GEMV_CASE(6)
    QMM_GEMV_CASE(7) QMM_GEMV_CASE(8) QMM_GEMV_CASE(9) QMM_GEMV_CASE(10) QMM_GEMV_CASE(11) QMM_GEMV_CASE(12)
#undef QMM_GEMV_CASE
    default: break;
  }
  return hipErrorInvalidValue;
}

// The activation row of the generic kernels, staged in LDS when it is short enough: a lane's
// slice is a few hundred contiguous bytes, so fetched straight from memory every lane of a load
// touches its own cache line (64 lines an instruction), which for the routed-expert rows (2048 or
// 4096 activations against two 1152-byte weight rows a wavefront) cost more than the weights.
// The workgroup copies the row with coalesced loads; the copy is padded as StagedX expects.
constexpr uint32_t kGenericXFloats = 8192;
__device__ __forceinline__ float* generic_x_area() {
  __shared__ __attribute__((aligned(16))) float xs[kGenericXFloats + kGenericXFloats / 16u];
  return xs;
}
template <class Codec>
__device__ __forceinline__ bool stage_generic_x(const typename Codec::Args& args) {
  if constexpr (Codec::kStageX) {
    if (args.k > kGenericXFloats) return false;   // uniform
    float* xs = generic_x_area();
    for (uint32_t e = threadIdx.x * 4u; e < args.k; e += blockDim.x * 4u) {
      *reinterpret_cast<float4*>(&xs[StagedX::pad(e)]) = *reinterpret_cast<const float4*>(args.a + e);
    }
    __syncthreads();
    return true;
  } else {
    return false;
  }
}

// Fallback for shapes the register-resident mapping does not cover (a row longer
// than 1024 chunks): one wavefront per weight row, lanes stride over the chunks and
// fetch their activations from LDS (short rows) or from memory each time.  Correct for any K the
// codec accepts; not tuned.
template <class Codec>
__global__ __launch_bounds__(256) void gemv_generic_kernel(typename Codec::Args args,
                                                           float* __restrict__ c, uint32_t n,
                                                           uint32_t cpr, uint32_t ldc) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if constexpr (requires { Codec::batch(args, 0u); }) {   // one activation row per grid.y
    Codec::batch(args, blockIdx.y);
    c += static_cast<size_t>(blockIdx.y) * ldc;
  }
  // A codec over two matrices (kTwoMatrices) takes the same row of both against one copy of the
  // activations and stores combine(first, second).
  constexpr bool kTwo = requires { Codec::kTwoMatrices; };
  // Order of the requests: the activation row (into registers, on its way to LDS), then the
  // fragments of the lane's first chunk; loads return in order, so the row is staged and the
  // barrier passed while the weights are still on their way (the barrier orders LDS only).
  constexpr int kXPer = kGenericXFloats / 4 / 256;
  bool staged = false;
  if constexpr (Codec::kStageX) staged = args.k <= kGenericXFloats;   // uniform
  const bool live = row < n;
  // rows and chunks past the end fetch the last ones (never used), so nothing here is conditional
  const uint32_t row_in = live ? row : n - 1u, chunk_in = lane < cpr ? lane : cpr - 1u;
  typename Codec::Frag f, f2;
  if constexpr (Codec::kStageX) {
    float4 x0, x1, x2, x3, x4, x5, x6, x7;
    static_assert(kXPer == 8, "eight 16-byte pieces a thread");
    const uint32_t last = args.k - 4u;
    auto piece = [&](uint32_t i) {
      const uint32_t e = (threadIdx.x + i * 256u) * 4u;
      return *reinterpret_cast<const float4*>(args.a + (staged && e < args.k ? e : last));
    };
    x0 = piece(0), x1 = piece(1), x2 = piece(2), x3 = piece(3), x4 = piece(4), x5 = piece(5), x6 = piece(6), x7 = piece(7);
    {
      const Lane ln = Codec::make_lane(args, cpr, chunk_in, 0u);
      Codec::load(args, ln, row_in, cpr, f);
      if constexpr (kTwo) Codec::load(args, ln, row_in, cpr, f2, 1);
    }
    if (staged) {
      float* xs = generic_x_area();
      auto put = [&](uint32_t i, const float4& v) {
        const uint32_t e = (threadIdx.x + i * 256u) * 4u;
        if (e < args.k) *reinterpret_cast<float4*>(&xs[StagedX::pad(e)]) = v;
      };
      put(0, x0), put(1, x1), put(2, x2), put(3, x3), put(4, x4), put(5, x5), put(6, x6), put(7, x7);
      lds_barrier();
    }
  } else {
    const Lane ln = Codec::make_lane(args, cpr, chunk_in, 0u);
    Codec::load(args, ln, row_in, cpr, f);
    if constexpr (kTwo) Codec::load(args, ln, row_in, cpr, f2, 1);
  }
  if (!live) return;  // whole wavefront leaves together
  float acc = 0.0f, acc2 = 0.0f;
  for (uint32_t chunk = lane; chunk < cpr; chunk += 64u) {
    typename Codec::template X<1> x;
    if (chunk != lane) {   // later chunks: fetched here
      const Lane ln = Codec::make_lane(args, cpr, chunk, 0u);
      Codec::load(args, ln, row, cpr, f);
      if constexpr (kTwo) Codec::load(args, ln, row, cpr, f2, 1);
    }
    if constexpr (Codec::kStageX) {
      if (staged) {
        Codec::template load_x<1>(args, chunk, true, x, StagedX{generic_x_area(), 0u, kGenericXFloats + kGenericXFloats / 16u});
      } else {
        Codec::template load_x<1>(args, chunk, true, x, GlobalX{args.a, args.k});
      }
    } else {
      Codec::template load_x<1>(args, chunk, true, x, 0);
    }
    float v[1];
    Codec::template dot<1>(f, x, v);
    acc += v[0];
    if constexpr (kTwo) {
      Codec::template dot<1>(f2, x, v);
      acc2 += v[0];
    }
  }
  acc = wave_sum(acc);
  if constexpr (kTwo) {
    acc2 = wave_sum(acc2);
    if (lane == 0) c[row] = Codec::combine(acc, acc2);
  } else {
    if (lane == 0) c[row] = Codec::template finish<1>(args, row, 0, acc);
  }
  (void)ldc;
}

// The same with RPW consecutive weight rows a wavefront, for launches with many rows (several
// tokens' expert rows): a lane's activations are fetched once per chunk and serve RPW rows, whose
// fragments are all requested before the first is used.  With one row a wavefront the activation
// fetch -- every lane its own 128-byte slice, 64 cache lines an instruction -- is repeated for
// every row and outweighs the weight fetch several times over.
template <class Codec, int RPW>
__global__ __launch_bounds__(256) void gemv_generic_rows_kernel(typename Codec::Args args, float* __restrict__ c,
                                                                uint32_t n, uint32_t cpr, uint32_t ldc) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t row0 = (blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) * RPW;
  if constexpr (requires { Codec::batch(args, 0u); }) {   // one activation row per grid.y
    Codec::batch(args, blockIdx.y);
    c += static_cast<size_t>(blockIdx.y) * ldc;
  }
  const bool staged = stage_generic_x<Codec>(args);
  if (row0 >= n) return;  // whole wavefront leaves together
  constexpr bool kTwo = requires { Codec::kTwoMatrices; };
  float acc[RPW], acc2[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) acc[r] = acc2[r] = 0.0f;
  for (uint32_t chunk = lane; chunk < cpr; chunk += 64u) {
    typename Codec::template X<1> x;
    if constexpr (Codec::kStageX) {
      if (staged) {
        Codec::template load_x<1>(args, chunk, true, x, StagedX{generic_x_area(), 0u, kGenericXFloats + kGenericXFloats / 16u});
      } else {
        Codec::template load_x<1>(args, chunk, true, x, GlobalX{args.a, args.k});
      }
    } else {
      Codec::template load_x<1>(args, chunk, true, x, 0);
    }
    const Lane ln = Codec::make_lane(args, cpr, chunk, 0u);
    typename Codec::Frag f[RPW], f2[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      const uint32_t row = row0 + r < n ? row0 + r : n - 1u;   // rows past the end repeat the last one
      Codec::load(args, ln, row, cpr, f[r]);
      if constexpr (kTwo) Codec::load(args, ln, row, cpr, f2[r], 1);
    }
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      float v[1];
      Codec::template dot<1>(f[r], x, v);
      acc[r] += v[0];
      if constexpr (kTwo) {
        Codec::template dot<1>(f2[r], x, v);
        acc2[r] += v[0];
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) {
    const float s = wave_sum(acc[r]);
    const uint32_t row = row0 + r;
    if constexpr (kTwo) {
      const float s2 = wave_sum(acc2[r]);
      if (lane == 0 && row < n) c[row] = Codec::combine(s, s2);
    } else {
      if (lane == 0 && row < n) c[row] = Codec::template finish<1>(args, row, 0, s);
    }
  }
  (void)ldc;
}

template <class Codec>
hipError_t launch_gemv_generic(const typename Codec::Args& args, float* c, uint32_t n, uint32_t k,
                               hipStream_t stream) {
  const uint32_t cpr = Codec::chunks_per_row(k);
  hipLaunchKernelGGL((gemv_generic_kernel<Codec>), dim3((n + 3u) / 4u), dim3(256), 0, stream, args,
                     c, n, cpr, n);
  return hipGetLastError();
}

}  // namespace

int num_cus() { return g_num_cus; }

void set_num_cus(int cus) {
  g_num_cus = cus > 0 ? cus : 256;
}

// Rows longer than the register-resident mapping holds (one chunk per thread, a row inside one
// workgroup) take the wave-per-row kernel, correct and untuned: any K of a format's granularity works.

hipError_t launch_q4k_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                           uint32_t k, hipStream_t stream) {
  if (k / 32u > 1024u) {   // longer rows than a workgroup holds: one wavefront per weight row, row by row
    for (uint32_t r = 0; r < m; ++r) {
      const hipError_t e = launch_gemv_generic<Q4KCodec>(Q4KCodec::Args{a + static_cast<size_t>(r) * k, w, k},
                                                         c + static_cast<size_t>(r) * n, n, k, stream);
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  // A lane keeps the 32 activations of its chunk for every row of the pass in registers: 128
  // registers at four rows, which fits only with two wavefronts per SIMD (workgroups of up to
  // 512 threads, k <= 16384); two rows fit 768-thread workgroups (k <= 24576); beyond that the
  // rows run one at a time.
  const uint32_t row_threads = (k / 32u + 63u) / 64u * 64u;
  for (uint32_t r0 = 0; r0 < m;) {
    const uint32_t left = m - r0;
    Q4KCodec::Args args{a + static_cast<size_t>(r0) * k, w, k};
    float* out = c + static_cast<size_t>(r0) * n;
    hipError_t e;
    uint32_t took;
    if (left >= 4 && row_threads <= 512u) {
      e = launch_gemv_r<Q4KCodec, 4, 512, 2, 6>(args, out, n, k, n, stream), took = 4;
    } else if (left == 3 && row_threads <= 512u) {
      e = launch_gemv_r<Q4KCodec, 3, 512, 2, 6>(args, out, n, k, n, stream), took = 3;
    } else if (left >= 2 && row_threads <= 768u) {
      e = launch_gemv_r<Q4KCodec, 2, 768, 2, 6>(args, out, n, k, n, stream), took = 2;
    } else {
      // Two fragments in flight per lane: a third makes the opening burst larger and the
      // launch longer (5120x17408 16.3 us against 15.1; 17408x5120 the same within noise).
      e = launch_gemv_r<Q4KPairCodec, 1, 768, 2, 9>(args, out, n, k, n, stream), took = 1;
    }
    if (e != hipSuccess) return e;
    r0 += took;
  }
  return hipSuccess;
}

// One activation row with K cut into `split` slices, partial sums to `split` output regions of n
// floats: slices of 64 to 512 chunks (4096..32768 weights) on matrices large enough to fill the chip.
bool q4k_gemv_split_supported(uint64_t n, uint64_t k, uint64_t split) {
  if (split < 2 || split > 8 || k % (256 * split) != 0) return false;
  const uint64_t slice = k / split;
  return slice >= 4096 && slice <= 32768 && n * k >= (1ull << 24) && n <= 0xFFFFFFFFull / split;
}

hipError_t launch_q4k_gemv_split(const float* a, const uint8_t* w, float* c, uint32_t n, uint32_t k, uint32_t split,
                                 hipStream_t stream) {
  const uint32_t slice = k / split;
  Q4KSliceCodec::Args args{a, w, slice, (k / 256u) * 144u};
  return launch_gemv_r<Q4KSliceCodec, 1, 768, 2, 12>(args, c, n, slice, n, stream, split);
}

// silu(G x) * (U x) for one activation row, one launch: a row of 64 to 384 chunks of 64 weights
// (two slot rows of it must fit a 768-thread workgroup and a wavefront may span two rows at most).
bool ffn_gate_up_q4k_supported(uint64_t k) { return k % 256 == 0 && k >= 4096 && k <= 24576; }

hipError_t launch_ffn_gate_up_q4k(const float* x, const uint8_t* gate, const uint8_t* up, float* out,
                                  uint32_t n, uint32_t k, hipStream_t stream) {
  Q4KGateUpCodec::Args args{x, gate, k, up};
  return launch_gemv_r<Q4KGateUpCodec, 1, 768, 2, 9>(args, out, n, k, n, stream);
}

// Q5_K: one row per weight pass (a lane keeps 64 activations and five 16-byte loads per stage).

hipError_t launch_q5k_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                           uint32_t k, hipStream_t stream) {
  if (k / 64u > 768u) {
    for (uint32_t r = 0; r < m; ++r) {
      const hipError_t e = launch_gemv_generic<Q5KCodec>(Q5KCodec::Args{a + static_cast<size_t>(r) * k, w, k},
                                                         c + static_cast<size_t>(r) * n, n, k, stream);
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  for (uint32_t r0 = 0; r0 < m; ++r0) {
    Q5KCodec::Args args{a + static_cast<size_t>(r0) * k, w, k};
    const hipError_t e = launch_gemv_r<Q5KCodec, 1, 768, 2, 9>(args, c + static_cast<size_t>(r0) * n, n, k, n, stream);
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// Q6_K: a lane keeps the 64 activations of its chunk per row in registers, so two rows share a
// weight pass (k <= 32768) and further rows take further passes.

hipError_t launch_q6k_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                           uint32_t k, hipStream_t stream) {
  if (k / 64u > 768u) {
    for (uint32_t r = 0; r < m; ++r) {
      const hipError_t e = launch_gemv_generic<Q6KCodec>(Q6KCodec::Args{a + static_cast<size_t>(r) * k, w, k},
                                                         c + static_cast<size_t>(r) * n, n, k, stream);
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  const uint32_t row_threads = (k / 64u + 63u) / 64u * 64u;
  for (uint32_t r0 = 0; r0 < m;) {
    Q6KCodec::Args args{a + static_cast<size_t>(r0) * k, w, k};
    float* out = c + static_cast<size_t>(r0) * n;
    hipError_t e;
    uint32_t took;
    if (m - r0 >= 2 && row_threads <= 512u) {
      // One fragment in flight per lane: with two, the 256 registers of a 512-thread workgroup
      // spill a few values, and a kernel with a scratch segment takes microseconds longer to
      // dispatch (two rows of 17408 x 5120: 38 us with depth 2, 29 us with depth 1).
      e = launch_gemv_r<Q6KCodec, 2, 512, 1, 6>(args, out, n, k, n, stream), took = 2;
    } else {
      e = launch_gemv_r<Q6KCodec, 1, 768, 2, 9>(args, out, n, k, n, stream), took = 1;
    }
    if (e != hipSuccess) return e;
    r0 += took;
  }
  return hipSuccess;
}

hipError_t launch_mxfp4_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                             uint32_t k, hipStream_t stream) {
  const uint8_t* s = w + static_cast<size_t>(n) * k / 2;
  if (k / 32u > 1024u) {
    for (uint32_t r = 0; r < m; ++r) {
      const hipError_t e = launch_gemv_generic<MxFp4Codec>(MxFp4Codec::Args{a + static_cast<size_t>(r) * k, w, s, k},
                                                           c + static_cast<size_t>(r) * n, n, k, stream);
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  // Register budgets as for Q4_K: four or three rows need two wavefronts per SIMD, two rows three.
  const uint32_t row_threads = (k / 32u + 63u) / 64u * 64u;
  for (uint32_t r0 = 0; r0 < m;) {
    const uint32_t left = m - r0;
    MxFp4Codec::Args args{a + static_cast<size_t>(r0) * k, w, s, k};
    float* out = c + static_cast<size_t>(r0) * n;
    hipError_t e;
    uint32_t took;
    if (left >= 4 && row_threads <= 512u) {
      e = launch_gemv_r<MxFp4Codec, 4, 512, 2, 6>(args, out, n, k, n, stream), took = 4;
    } else if (left == 3 && row_threads <= 512u) {
      e = launch_gemv_r<MxFp4Codec, 3, 512, 2, 6>(args, out, n, k, n, stream), took = 3;
    } else if (left >= 2 && row_threads <= 768u) {
      e = launch_gemv_r<MxFp4Codec, 2, 768, 2, 6>(args, out, n, k, n, stream), took = 2;
    } else {
      // one row: 64 weights a lane where K allows (and the row is long enough for the main kernel)
      e = hipErrorInvalidValue;
      const uint32_t cpr2 = k / 64u;
      if (k % 64u == 0 && !(cpr2 == 4 || cpr2 == 8 || cpr2 == 16 || cpr2 == 32)) {
        e = launch_gemv_r<MxFp4PairCodec, 1, 768, 2, 9>(args, out, n, k, n, stream);
      }
      if (e == hipErrorInvalidValue) e = launch_gemv_r<MxFp4Codec, 1, 1024, 4>(args, out, n, k, n, stream);
      took = 1;
    }
    if (e != hipSuccess) return e;
    r0 += took;
  }
  return hipSuccess;
}

hipError_t launch_mxfp4_a8_gemv(const uint8_t* a8, const float* as, const uint8_t* w, float* c,
                                uint32_t m, uint32_t n, uint32_t k, hipStream_t stream) {
  const uint8_t* s = w + static_cast<size_t>(n) * k / 2;
  if (k / 32u > 1024u) {
    for (uint32_t r = 0; r < m; ++r) {
      const hipError_t e = launch_gemv_generic<MxFp4A8Codec>(
          MxFp4A8Codec::Args{a8 + static_cast<size_t>(r) * k, as + r, w, s, k}, c + static_cast<size_t>(r) * n, n, k, stream);
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  for (uint32_t r0 = 0; r0 < m;) {
    const uint32_t left = m - r0;
    MxFp4A8Codec::Args args{a8 + static_cast<size_t>(r0) * k, as + r0, w, s, k};
    float* out = c + static_cast<size_t>(r0) * n;
    hipError_t e;
    uint32_t took;
    if (left >= 4) {
      e = launch_gemv_r<MxFp4A8Codec, 4, 1024, 2, 6>(args, out, n, k, n, stream), took = 4;
    } else if (left >= 2) {
      e = launch_gemv_r<MxFp4A8Codec, 2, 1024, 4, 6>(args, out, n, k, n, stream), took = 2;
    } else {
      e = launch_gemv_r<MxFp4A8Codec, 1, 1024, 4>(args, out, n, k, n, stream), took = 1;
    }
    if (e != hipSuccess) return e;
    r0 += took;
  }
  return hipSuccess;
}

namespace {
template <bool BLOCK>
hipError_t launch_fp8_gemv_as(const float* a, const uint8_t* w, const float* s, float* c, uint32_t m,
                              uint32_t n, uint32_t k, hipStream_t stream) {
  using Fp8Codec = Fp8CodecT<1, BLOCK>;
  using Fp8WideCodec = Fp8CodecT<2, BLOCK>;
  using Fp8QuadCodec = Fp8CodecT<4, BLOCK>;
  if (k / 32u > 1024u || (k / 16u > 1024u && k % 32u != 0)) {
    for (uint32_t r = 0; r < m; ++r) {
      const hipError_t e = launch_gemv_generic<Fp8Codec>(typename Fp8Codec::Args{a + static_cast<size_t>(r) * k, w, s, k},
                                                         c + static_cast<size_t>(r) * n, n, k, stream);
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  const uint32_t cpr4 = k / 64u;
  if (m == 1 && k % 64u == 0 && cpr4 >= 64u && cpr4 <= 768u) {
    // one row: 64 weights a lane, so the reduction and the loop overhead are paid once per 64
    typename Fp8QuadCodec::Args args{a, w, s, k};
    return launch_gemv_r<Fp8QuadCodec, 1, 768, 2, 9>(args, c, n, k, n, stream);
  }
  if (k / 16u > 1024u) {
    // rows of 16385..32768 weights: 32 weights a lane, one or two activation rows per weight pass
    for (uint32_t r0 = 0; r0 < m;) {
      typename Fp8WideCodec::Args args{a + static_cast<size_t>(r0) * k, w, s, k};
      float* out = c + static_cast<size_t>(r0) * n;
      hipError_t e;
      uint32_t took;
      // (with block scales two rows a pass no longer fit the registers of a 1024-thread
      // workgroup, and a kernel that spills pays for its scratch segment at every dispatch)
      if constexpr (!BLOCK) {
        if (m - r0 >= 2) {
          e = launch_gemv_r<Fp8WideCodec, 2, 1024, 2, 1>(args, out, n, k, n, stream), took = 2;
          if (e != hipSuccess) return e;
          r0 += took;
          continue;
        }
      }
      {
        e = launch_gemv_r<Fp8WideCodec, 1, 1024, 2, 1>(args, out, n, k, n, stream), took = 1;
      }
      if (e != hipSuccess) return e;
      r0 += took;
    }
    return hipSuccess;
  }
  for (uint32_t r0 = 0; r0 < m;) {
    const uint32_t left = m - r0;
    typename Fp8Codec::Args args{a + static_cast<size_t>(r0) * k, w, s, k};
    float* out = c + static_cast<size_t>(r0) * n;
    hipError_t e;
    uint32_t took;
    if (left >= 4) {
      e = launch_gemv_r<Fp8Codec, 4, 1024, 2, 6>(args, out, n, k, n, stream), took = 4;
    } else if (left >= 2) {
      e = launch_gemv_r<Fp8Codec, 2, 1024, 4, 6>(args, out, n, k, n, stream), took = 2;
    } else {
      e = launch_gemv_r<Fp8Codec, 1, 1024, 4>(args, out, n, k, n, stream), took = 1;
    }
    if (e != hipSuccess) return e;
    r0 += took;
  }
  return hipSuccess;
}
}  // namespace

hipError_t launch_fp8_gemv(const float* a, const uint8_t* w, const float* s, float* c, uint32_t m,
                           uint32_t n, uint32_t k, hipStream_t stream) {
  return launch_fp8_gemv_as<false>(a, w, s, c, m, n, k, stream);
}

// One scale per 128 x 128 block of W (n and k multiples of 128).
hipError_t launch_fp8_block_gemv(const float* a, const uint8_t* w, const float* s, float* c, uint32_t m,
                                 uint32_t n, uint32_t k, hipStream_t stream) {
  return launch_fp8_gemv_as<true>(a, w, s, c, m, n, k, stream);
}

// ---- mixture-of-experts (Q4_K experts) ------------------------------------------------

// Weight rows a wavefront takes in the per-token expert kernels: four when that still leaves
// every SIMD of the chip two wavefronts, else one (measured: 256 experts, 2048/512, top-8, gate/up and
// down together: 4 tokens 27.8 -> 21.6 us, 8 tokens 47 -> 33 us, 16 tokens 89 -> 56 us).
constexpr uint32_t kMoeRowsPerWave = 4;
static uint32_t moe_rows_per_wave(uint32_t n, uint32_t tokens) {
  const uint64_t waves = static_cast<uint64_t>(n) * tokens / kMoeRowsPerWave;
  return waves >= static_cast<uint64_t>(num_cus()) * 8u ? kMoeRowsPerWave : 1u;
}

hipError_t launch_moe_gate_up_q4k(const float* x, const uint8_t* gate, const uint8_t* up,
                                  const uint32_t* ids, float* phi, uint32_t hidden, uint32_t inter,
                                  uint32_t top_k, uint64_t gate_stride, uint64_t up_stride,
                                  uint32_t n_experts, uint32_t rows, hipStream_t stream) {
  const uint32_t n = top_k * inter, cpr = Q4KCodec::chunks_per_row(hidden);
  Q4KExpertGateUpCodec::Args a{x, gate, hidden, ids, gate_stride, inter, top_k, n_experts, up, up_stride};
  if (moe_rows_per_wave(n, rows) > 1u) {   // enough rows to fill the chip four rows a wavefront
    hipLaunchKernelGGL((gemv_generic_rows_kernel<Q4KExpertGateUpCodec, kMoeRowsPerWave>),
                       dim3((n + 4u * kMoeRowsPerWave - 1u) / (4u * kMoeRowsPerWave), rows), dim3(256), 0, stream, a, phi, n,
                       cpr, n);
  } else {
    hipLaunchKernelGGL((gemv_generic_kernel<Q4KExpertGateUpCodec>), dim3((n + 3u) / 4u, rows), dim3(256), 0, stream, a,
                       phi, n, cpr, n);
  }
  return hipGetLastError();
}

hipError_t launch_moe_down_q4k(const float* phi, const uint8_t* down, const uint32_t* ids,
                               const float* wts, float* out, uint32_t hidden, uint32_t inter,
                               uint32_t top_k, uint64_t down_stride, bool accumulate, uint32_t n_experts,
                               uint32_t rows, hipStream_t stream) {
  const uint32_t k = top_k * inter, cpr = Q4KCodec::chunks_per_row(k);
  Q4KExpertDownCodec::Args a{phi, down, k, ids, down_stride, inter, top_k, hidden, n_experts, wts,
                             accumulate ? out : nullptr};
  if (moe_rows_per_wave(hidden, rows) > 1u) {
    hipLaunchKernelGGL((gemv_generic_rows_kernel<Q4KExpertDownCodec, kMoeRowsPerWave>),
                       dim3((hidden + 4u * kMoeRowsPerWave - 1u) / (4u * kMoeRowsPerWave), rows), dim3(256), 0, stream, a, out,
                       hidden, cpr, hidden);
  } else {
    hipLaunchKernelGGL((gemv_generic_kernel<Q4KExpertDownCodec>), dim3((hidden + 3u) / 4u, rows), dim3(256), 0,
                       stream, a, out, hidden, cpr, hidden);
  }
  return hipGetLastError();
}

hipError_t launch_moe_down_q6k(const float* phi, const uint8_t* down, const uint32_t* ids,
                               const float* wts, float* out, uint32_t hidden, uint32_t inter,
                               uint32_t top_k, uint64_t down_stride, bool accumulate, uint32_t n_experts,
                               uint32_t rows, hipStream_t stream) {
  const uint32_t k = top_k * inter, cpr = Q6KCodec::chunks_per_row(k);
  Q6KExpertDownCodec::Args a{phi, down, k, ids, down_stride, inter, top_k, hidden, n_experts, wts,
                             accumulate ? out : nullptr};
  if (moe_rows_per_wave(hidden, rows) > 1u) {
    hipLaunchKernelGGL((gemv_generic_rows_kernel<Q6KExpertDownCodec, kMoeRowsPerWave>),
                       dim3((hidden + 4u * kMoeRowsPerWave - 1u) / (4u * kMoeRowsPerWave), rows), dim3(256), 0, stream, a, out,
                       hidden, cpr, hidden);
  } else {
    hipLaunchKernelGGL((gemv_generic_kernel<Q6KExpertDownCodec>), dim3((hidden + 3u) / 4u, rows), dim3(256), 0,
                       stream, a, out, hidden, cpr, hidden);
  }
  return hipGetLastError();
}

}  // namespace qmm
