// The non-matmul pieces of a transformer block that sit between the projections, as plain correct
// kernels so that a trunk can run on this backend end to end: rotary embeddings, softmax attention
// over a key/value cache, the query/gate split of gated attention.  Contracts:
// include/tessera/backend.hpp:162-179,378-390; CPU statements src/core/numerics/attention.cpp.
// None of them is tuned: they move kilobytes where the projections move megabytes.

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

// One thread per (row, head, pair): (x[j], x[j + pairs]) rotated by pos * theta^(-2j / rope_dim).
// The angle, its cosine and sine are formed in double and rounded to fp32 once, as RopeRef does
// (src/core/numerics/attention.cpp:11-44); `pos3` non-null selects the multimodal form, where pair
// j takes the temporal, height or width position of its row (MropeRef, attention.cpp:227-264).
__global__ __launch_bounds__(256) void rope_kernel(float* __restrict__ data, const uint64_t* __restrict__ pos3, uint64_t rows,
                                                   uint64_t heads, uint64_t head_dim, uint64_t rope_dim, uint64_t pos_base,
                                                   float theta, uint64_t sec_t, uint64_t sec_h) {
  const uint64_t pairs = rope_dim / 2;
  const uint64_t t = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (t >= rows * heads * pairs) return;
  const uint64_t row = t / (heads * pairs), rem = t % (heads * pairs), head = rem / pairs, j = rem % pairs;
  uint64_t p = pos_base + row;
  if (pos3 != nullptr) p = pos3[row * 3 + (j < sec_t ? 0 : (j < sec_t + sec_h ? 1 : 2))];
  const double angle = static_cast<double>(p) * pow(static_cast<double>(theta), -2.0 * static_cast<double>(j) / static_cast<double>(rope_dim));
  const float c = static_cast<float>(cos(angle)), s = static_cast<float>(sin(angle));
  float* base = data + (row * heads + head) * head_dim;
  const float x1 = base[j], x2 = base[j + pairs];
  base[j] = x1 * c - x2 * s;
  base[j + pairs] = x1 * s + x2 * c;
}

// One workgroup of four wavefronts per (query row, head).  Keys are taken 64 at a time: a
// wavefront forms the score of a key with its lanes across head_dim (coalesced key reads, a DPP
// sum), the first wavefront turns the 64 scores into weights against the running maximum, and
// thread e accumulates weight * v[key][e] (coalesced value reads): the usual running softmax, so
// the result differs from AttentionRef (src/core/numerics/attention.cpp:158-225) in summation
// order only.
// KV: how keys and values are stored.  The quantized kinds hold codes and one fp32 scale per key
// row (all kv heads of a position), and an element is code * scale as in AttentionQ8Ref /
// AttentionQ4Ref / AttentionFp8Ref (src/core/numerics/attention.cpp:45-121).
enum class KvKind { F32, F16, Q8, Q4, Fp8 };

// SPLIT (the flash-decoding ids, src/backends/rocm/rocm_kernels_basic.cpp:275-440): workgroup
// (row, head, s) covers chunk s of ceil(span / split) keys of the row's key range and leaves the
// unnormalized sum, the chunk's largest score and its sum of weights in pacc / pmax / psum at
// index (row * heads + head) * split + s (an empty chunk: 0, -1e30, 0); attention_combine_kernel
// merges them.
struct SplitOut {
  float *pacc, *pmax, *psum;
  uint64_t split;
};

template <KvKind KV, bool SPLIT>
__global__ __launch_bounds__(256) void attention_kernel(const float* __restrict__ q, const void* __restrict__ k,
                                                        const void* __restrict__ v, const float* __restrict__ k_scale,
                                                        const float* __restrict__ v_scale, float* __restrict__ out,
                                                        SplitOut part, uint64_t n, uint64_t heads, uint64_t kv_heads,
                                                        uint64_t head_dim, uint64_t q_base, uint64_t row_base, uint64_t window,
                                                        uint64_t causal) {
  constexpr uint32_t kKeys = 64;
  __shared__ float sc[kKeys], wt[kKeys], bc[2];
  const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
  const uint64_t g = blockIdx.x, rest = SPLIT ? g / part.split : g;
  const uint64_t i = rest / heads, h = rest % heads, kv = h / (heads / kv_heads);
  const uint64_t pos = q_base + i;
  uint64_t last = causal != 0 ? (pos >= n ? n - 1 : pos) : n - 1;
  uint64_t start = 0;
  if (causal != 0) {
    start = (window != 0 && pos + 1 > window) ? pos + 1 - window : 0;
    if (start > last) start = last;
  }
  if constexpr (SPLIT) {
    const uint64_t chunk = (last + 1 - start + part.split - 1) / part.split;
    const uint64_t cstart = start + (g % part.split) * chunk;
    if (cstart > last) {   // workgroup-uniform
      if (t < head_dim) part.pacc[g * head_dim + t] = 0.0f;
      if (t == 0) part.pmax[g] = -1e30f, part.psum[g] = 0.0f;
      return;
    }
    last = cstart + chunk - 1 < last ? cstart + chunk - 1 : last;
    start = cstart;
  }
  const float scale = 1.0f / sqrtf(static_cast<float>(head_dim));
  const uint64_t qb = ((row_base + i) * heads + h) * head_dim;
  auto kv_at = [&](const void* base, const float* row_scale, uint64_t key, uint64_t idx) {
    if constexpr (KV == KvKind::F16) {
      return half_bits_to_float(static_cast<const uint16_t*>(base)[idx]);
    } else if constexpr (KV == KvKind::F32) {
      return static_cast<const float*>(base)[idx];
    } else if constexpr (KV == KvKind::Q8) {
      return static_cast<float>(static_cast<const int8_t*>(base)[idx]) * row_scale[key];
    } else if constexpr (KV == KvKind::Q4) {
      const int nib = (static_cast<const uint8_t*>(base)[idx >> 1] >> ((idx & 1u) * 4u)) & 0xF;
      return static_cast<float>((nib & 8) ? nib - 16 : nib) * row_scale[key];
    } else {
      return e4m3_to_float(static_cast<const uint8_t*>(base)[idx]) * row_scale[key];
    }
  };
  float qr[4];                       // head_dim <= 256: up to four elements a lane
#pragma unroll
  for (int cc = 0; cc < 4; ++cc) qr[cc] = lane + 64u * cc < head_dim ? q[qb + lane + 64u * cc] : 0.0f;

  float run_max = -INFINITY, run_sum = 0.0f, acc = 0.0f;
  for (uint64_t j0 = start; j0 <= last; j0 += kKeys) {
    const uint32_t count = last - j0 + 1 < kKeys ? static_cast<uint32_t>(last - j0 + 1) : kKeys;
    for (uint32_t kk = wave; kk < kKeys; kk += 4u) {
      float dot = 0.0f;
      if (kk < count) {
        const uint64_t kb = ((j0 + kk) * kv_heads + kv) * head_dim;
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
          if (lane + 64u * cc < head_dim) dot = fmaf(qr[cc], kv_at(k, k_scale, j0 + kk, kb + lane + 64u * cc), dot);
        }
      }
      dot = wave_sum(dot);
      if (lane == 0) sc[kk] = kk < count ? dot * scale : -INFINITY;
    }
    __syncthreads();
    if (wave == 0) {
      const float s = sc[lane];
      const float m_new = fmaxf(run_max, wave_max(s));
      const float w = lane < count ? expf(s - m_new) : 0.0f;
      wt[lane] = w;
      const float l = wave_sum(w);
      if (lane == 0) {
        bc[0] = m_new;
        bc[1] = l;
      }
    }
    __syncthreads();
    const float m_new = bc[0];
    const float corr = expf(run_max - m_new);      // 0 on the first tile (run_max = -inf)
    run_sum = fmaf(corr, run_sum, bc[1]);
    run_max = m_new;
    if (t < head_dim) {
      float a = 0.0f;
      for (uint32_t kk = 0; kk < count; ++kk) {
        a = fmaf(wt[kk], kv_at(v, v_scale, j0 + kk, ((j0 + kk) * kv_heads + kv) * head_dim + t), a);
      }
      acc = fmaf(corr, acc, a);
    }
    __syncthreads();
  }
  if constexpr (SPLIT) {
    if (t < head_dim) part.pacc[g * head_dim + t] = acc;
    if (t == 0) part.pmax[g] = run_max, part.psum[g] = run_sum;
  } else {
    if (t < head_dim) out[qb + t] = acc / run_sum;
  }
}

// out[row][head] = sum_s w_s pacc_s / sum_s w_s psum_s with w_s = exp(pmax_s - max_s pmax_s)
// (src/backends/rocm/rocm_kernels_basic.cpp:664-690).  One workgroup per (row, head).
__global__ __launch_bounds__(256) void attention_combine_kernel(const float* __restrict__ pacc, const float* __restrict__ pmax,
                                                                const float* __restrict__ psum, float* __restrict__ out,
                                                                uint64_t head_dim, uint64_t split) {
  const uint64_t g = blockIdx.x, base = g * split;
  const uint32_t e = threadIdx.x;
  float top = -1e30f;
  for (uint64_t s = 0; s < split; ++s) top = fmaxf(top, pmax[base + s]);
  if (e < head_dim) {
    float num = 0.0f, den = 0.0f;
    for (uint64_t s = 0; s < split; ++s) {
      const float w = expf(pmax[base + s] - top);
      num = fmaf(w, pacc[(base + s) * head_dim + e], num);
      den = fmaf(w, psum[base + s], den);
    }
    out[g * head_dim + e] = num / den;
  }
}

__global__ __launch_bounds__(256) void qgate_split_kernel(const float* __restrict__ fused, float* __restrict__ q,
                                                          float* __restrict__ gate, uint64_t head_dim, uint64_t total) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (i >= total) return;
  const uint64_t rh = i / head_dim, e = i % head_dim;
  q[i] = fused[rh * 2 * head_dim + e];
  gate[i] = fused[rh * 2 * head_dim + head_dim + e];
}

// Per-row symmetric quantizer of the quantized key/value caches (QuantizeQ8Ref / QuantizeQ4Ref,
// src/core/numerics/quant.cpp:123-178): scale = amax / QMAX (1 for an all-zero row), code =
// x / scale rounded half away from zero and clamped to +-QMAX; int8 codes a byte each, 4-bit codes
// two a byte, low nibble first.  One workgroup per row.
template <int BITS>
__global__ __launch_bounds__(256) void quantize_kv_kernel(const float* __restrict__ in, uint8_t* __restrict__ out,
                                                          float* __restrict__ scale, uint64_t cols) {
  constexpr float kMax = BITS == 8 ? 127.0f : 7.0f;
  __shared__ float red[4];
  const uint32_t t = threadIdx.x;
  const float* row = in + static_cast<size_t>(blockIdx.x) * cols;
  float amax = 0.0f;
  for (uint64_t c = t; c < cols; c += 256u) amax = fmaxf(amax, fabsf(row[c]));
  amax = wave_max(amax);
  if ((t & 63u) == 0) red[t >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float s = amax > 0.0f ? amax / kMax : 1.0f;
  if (t == 0) scale[blockIdx.x] = s;
  auto code = [&](float x) {
    const float r = roundf(x / s);                       // half away from zero, as lround
    return static_cast<int>(fminf(fmaxf(r, -kMax), kMax));
  };
  if constexpr (BITS == 8) {
    uint8_t* dst = out + static_cast<size_t>(blockIdx.x) * cols;
    for (uint64_t c = t; c < cols; c += 256u) dst[c] = static_cast<uint8_t>(static_cast<int8_t>(code(row[c])));
  } else {
    uint8_t* dst = out + static_cast<size_t>(blockIdx.x) * (cols / 2);
    for (uint64_t c = t; c < cols / 2; c += 256u) {
      dst[c] = static_cast<uint8_t>((code(row[2 * c]) & 0xF) | ((code(row[2 * c + 1]) & 0xF) << 4));
    }
  }
}

// fp32 -> binary16 with the significand cut toward zero, magnitudes from 2^16 up (and NaN) to
// infinity, below 2^-24 to zero: the conversion of the "cast_f32_f16" built-in
// (src/backends/rocm/rocm_kernels.hpp:26-45), not the hardware's round-to-nearest.
__device__ __forceinline__ uint32_t float_to_fp16_cut(float value) {
  const uint32_t bits = bit_cast<uint32_t>(value);
  const uint32_t sign = (bits >> 16) & 0x8000u;
  const int exponent = static_cast<int>((bits >> 23) & 0xFFu) - 127;
  const uint32_t mantissa = bits & 0x7FFFFFu;
  if (exponent > 15) return sign | 0x7C00u;
  if (exponent < -24) return sign;
  if (exponent < -14) return sign | ((mantissa | 0x800000u) >> static_cast<uint32_t>(-exponent - 1));
  return sign | (static_cast<uint32_t>(exponent + 15) << 10) | (mantissa >> 13);
}

__global__ __launch_bounds__(256) void cast_f32_f16_kernel(const float* __restrict__ in, uint32_t* __restrict__ out, uint64_t pairs) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (i >= pairs) return;
  const float2 v = reinterpret_cast<const float2*>(in)[i];
  out[i] = float_to_fp16_cut(v.x) | (float_to_fp16_cut(v.y) << 16);
}

dim3 blocks_for(uint64_t count) { return dim3(static_cast<uint32_t>((count + 255) / 256)); }

}  // namespace

hipError_t launch_rope(float* data, const uint64_t* pos3, uint64_t rows, uint64_t heads, uint64_t head_dim, uint64_t rope_dim,
                       uint64_t pos_base, float theta, uint64_t sec_t, uint64_t sec_h, hipStream_t stream) {
  hipLaunchKernelGGL(rope_kernel, blocks_for(rows * heads * (rope_dim / 2)), dim3(256), 0, stream, data, pos3, rows, heads,
                     head_dim, rope_dim, pos_base, theta, sec_t, sec_h);
  return hipGetLastError();
}

namespace {
// kind: 0 fp32, 1 fp16 keys and values; 2 int8, 3 4-bit, 4 E4M3 codes with one scale per key row.
template <bool SPLIT>
hipError_t launch_attention_as(uint32_t kind, dim3 grid, const float* q, const void* k, const void* v, const float* k_scale,
                               const float* v_scale, float* out, SplitOut part, uint64_t n, uint64_t heads, uint64_t kv_heads,
                               uint64_t head_dim, uint64_t q_base, uint64_t row_base, uint64_t window, bool causal,
                               hipStream_t stream) {
  auto go = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, q, k, v, k_scale, v_scale, out, part, n, heads, kv_heads, head_dim,
                       q_base, row_base, window, causal ? 1ull : 0ull);
  };
  switch (kind) {
    case 0: go(attention_kernel<KvKind::F32, SPLIT>); break;
    case 1: go(attention_kernel<KvKind::F16, SPLIT>); break;
    case 2: go(attention_kernel<KvKind::Q8, SPLIT>); break;
    case 3: go(attention_kernel<KvKind::Q4, SPLIT>); break;
    default: go(attention_kernel<KvKind::Fp8, SPLIT>); break;
  }
  return hipGetLastError();
}
}  // namespace

hipError_t launch_attention(const float* q, const void* k, const void* v, float* out, uint64_t m, uint64_t n, uint64_t heads,
                            uint64_t kv_heads, uint64_t head_dim, uint64_t q_base, uint64_t row_base, uint64_t window,
                            bool kv_f16, bool causal, hipStream_t stream) {
  return launch_attention_as<false>(kv_f16 ? 1u : 0u, dim3(static_cast<uint32_t>(m * heads)), q, k, v, nullptr, nullptr, out,
                                    SplitOut{}, n, heads, kv_heads, head_dim, q_base, row_base, window, causal, stream);
}

// kind: 0 int8, 1 4-bit, 2 E4M3 keys and values with one scale per key row; always causal.
hipError_t launch_attention_quant(const float* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                  float* out, uint64_t m, uint64_t n, uint64_t heads, uint64_t kv_heads, uint64_t head_dim,
                                  uint64_t q_base, uint64_t row_base, uint64_t window, uint32_t kind, hipStream_t stream) {
  return launch_attention_as<false>(2u + kind, dim3(static_cast<uint32_t>(m * heads)), q, k, v, k_scale, v_scale, out, SplitOut{},
                                    n, heads, kv_heads, head_dim, q_base, row_base, window, true, stream);
}

// The split-N form: kv_kind as launch_attention_as (0 fp32, 1 fp16, 2.. quantized with scales).
hipError_t launch_attention_split(const float* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                  float* pacc, float* pmax, float* psum, uint64_t m, uint64_t n, uint64_t heads,
                                  uint64_t kv_heads, uint64_t head_dim, uint64_t q_base, uint64_t window, uint32_t kv_kind,
                                  bool causal, uint64_t split, hipStream_t stream) {
  return launch_attention_as<true>(kv_kind, dim3(static_cast<uint32_t>(m * heads * split)), q, k, v, k_scale, v_scale, nullptr,
                                   SplitOut{pacc, pmax, psum, split}, n, heads, kv_heads, head_dim, q_base, 0, window, causal,
                                   stream);
}

hipError_t launch_attention_combine(const float* pacc, const float* pmax, const float* psum, float* out, uint64_t m,
                                    uint64_t heads, uint64_t head_dim, uint64_t split, hipStream_t stream) {
  hipLaunchKernelGGL(attention_combine_kernel, dim3(static_cast<uint32_t>(m * heads)), dim3(256), 0, stream, pacc, pmax, psum, out,
                     head_dim, split);
  return hipGetLastError();
}

hipError_t launch_quantize_kv(const float* in, uint8_t* out, float* scale, uint64_t rows, uint64_t cols, uint32_t bits,
                              hipStream_t stream) {
  if (bits == 8) {
    hipLaunchKernelGGL(quantize_kv_kernel<8>, dim3(static_cast<uint32_t>(rows)), dim3(256), 0, stream, in, out, scale, cols);
  } else {
    hipLaunchKernelGGL(quantize_kv_kernel<4>, dim3(static_cast<uint32_t>(rows)), dim3(256), 0, stream, in, out, scale, cols);
  }
  return hipGetLastError();
}

hipError_t launch_cast_f32_f16(const float* in, void* out, uint64_t n, hipStream_t stream) {
  hipLaunchKernelGGL(cast_f32_f16_kernel, blocks_for(n / 2), dim3(256), 0, stream, in, static_cast<uint32_t*>(out), n / 2);
  return hipGetLastError();
}

hipError_t launch_qgate_split(const float* fused, float* q, float* gate, uint64_t heads, uint64_t head_dim, uint64_t rows,
                              hipStream_t stream) {
  const uint64_t total = rows * heads * head_dim;
  hipLaunchKernelGGL(qgate_split_kernel, blocks_for(total), dim3(256), 0, stream, fused, q, gate, head_dim, total);
  return hipGetLastError();
}

}  // namespace qmm
