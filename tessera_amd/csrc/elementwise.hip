// Small kernels around the matmul path: split-K reduce, per-token E4M3 activation
// quantization, MXFP4 row reference exponents, and fp32 dumps of the block decodes
// (the bit-exact level of the parity tests).

#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

constexpr float kE4M3Max = 448.0f;
constexpr float kE4M3MinScale = 1.0f / (448.0f * 512.0f);

// c[i] = sum_s part[s * total + i], s ascending ("gemm_vec_reduce",
// src/backends/rocm/rocm_kernels_gemv.cpp:53-66; "gemm_mxfp4_wmma_reduce",
// src/backends/rocm/rocm_kernels_basic.cpp:1497-1510).
__global__ __launch_bounds__(256) void vec_reduce_kernel(const float* __restrict__ part,
                                                         float* __restrict__ c, uint64_t total,
                                                         uint64_t split) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float acc = 0.0f;
  for (uint64_t s = 0; s < split; ++s) acc += part[s * total + i];
  c[i] = acc;
}

__global__ __launch_bounds__(256) void fill_f32_kernel(float* __restrict__ dst, float value,
                                                       uint64_t count) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) dst[i] = value;
}

// "silu_mul": o = silu(g) * u elementwise, the reference's expression
// (src/backends/rocm/rocm_kernels_basic.cpp:1882-1891).  o may alias g or u.
__global__ __launch_bounds__(256) void silu_mul_kernel(const float* g, const float* u, float* o, uint64_t n) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const float gate = g[i];
  o[i] = (gate / (1.0f + expf(-gate))) * u[i];
}

// "round_bf16": every fp32 value rounded in place to bfloat16 precision, nearest even, by the
// reference's integer arithmetic on the bits (src/backends/rocm/rocm_kernels_basic.cpp:885-899;
// NaN payloads and infinities go through the same add, as there).
__global__ __launch_bounds__(256) void round_bf16_kernel(uint32_t* __restrict__ x, uint64_t n) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  uint32_t bits = x[i];
  bits += 0x7FFFu + ((bits >> 16) & 1u);
  x[i] = bits & 0xFFFF0000u;
}

// "add": o = a + b elementwise (src/backends/rocm/rocm_kernels_basic.cpp:1870-1880).
__global__ __launch_bounds__(256) void add_kernel(const float* a, const float* b, float* o, uint64_t n) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) o[i] = a[i] + b[i];
}

// "fill": every int32 element set to the low 32 bits of the value
// (src/backends/rocm/rocm_kernels_basic.cpp:10-19).
__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t* __restrict__ out, int32_t value, uint64_t n) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) out[i] = value;
}

// "rmsnorm": y = x / sqrt(mean(x^2) + eps) * w per row, one workgroup per row
// (src/backends/rocm/rocm_kernels_basic.cpp:1586-1616).  The sum of squares is a strided fma chain
// per thread, a butterfly inside each wavefront and the four wavefront sums in order: the
// reference's tree adds the same partials in another order, so results agree to rounding.
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                      float* __restrict__ y, uint64_t cols, float eps) {
  __shared__ float part[4];
  const float* xr = x + static_cast<uint64_t>(blockIdx.x) * cols;
  float* yr = y + static_cast<uint64_t>(blockIdx.x) * cols;
  float sum = 0.0f;
  for (uint64_t c = threadIdx.x; c < cols; c += 256u) sum = fmaf(xr[c], xr[c], sum);
  sum = wave_sum(sum);
  if ((threadIdx.x & 63u) == 0) part[threadIdx.x >> 6] = sum;
  __syncthreads();
  const float mean = (((part[0] + part[1]) + part[2]) + part[3]) / static_cast<float>(cols);
  const float gain = 1.0f / sqrtf(mean + eps);
  for (uint64_t c = threadIdx.x; c < cols; c += 256u) yr[c] = xr[c] * gain * w[c];
}

// "embedding_f32" / "embedding_bf16" / "embedding_q4k": out[row] = table[ids[row]], a zero row for
// an id outside the table (src/backends/rocm/rocm_kernels_embedding.cpp:15-108).  KIND 0: fp32
// table, 1: bf16 (the high half of the fp32 bits), 2: Q4_K rows of cols/256 super-blocks, decoded
// as (d*sc)*q - dmin*mn with exact products and one rounding.
template <int KIND>
__global__ __launch_bounds__(256) void embedding_kernel(const uint32_t* __restrict__ ids, const void* __restrict__ table,
                                                        float* __restrict__ out, uint64_t rows, uint64_t cols,
                                                        uint64_t vocab) {
  const uint64_t g = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (g >= rows * cols) return;
  const uint64_t row = g / cols, i = g % cols;
  const uint64_t id = ids[row];
  if (id >= vocab) {
    out[g] = 0.0f;
    return;
  }
  if constexpr (KIND == 0) {
    out[g] = static_cast<const float*>(table)[id * cols + i];
  } else if constexpr (KIND == 1) {
    out[g] = bit_cast<float>(static_cast<uint32_t>(static_cast<const uint16_t*>(table)[id * cols + i]) << 16);
  } else {
    const uint64_t b = i / kQ4KBlockElems;
    const uint32_t e = static_cast<uint32_t>(i % kQ4KBlockElems);
    const uint8_t* base = static_cast<const uint8_t*>(table) + (id * (cols / kQ4KBlockElems) + b) * kQ4KBlockBytes;
    const uint32_t grp = e / 64u, half = (e % 64u) / 32u, l = e % 32u, sb = 2u * grp + half;
    const uint8_t* p = base + 4;
    uint32_t sc, mn;
    if (sb < 4) {
      sc = p[sb] & 63u;
      mn = p[sb + 4] & 63u;
    } else {
      sc = (p[sb + 4] & 15u) | ((p[sb - 4] >> 6) << 4);
      mn = (p[sb + 4] >> 4) | ((p[sb] >> 6) << 4);
    }
    const float d = half_bits_to_float(base[0] | (static_cast<uint32_t>(base[1]) << 8));
    const float dmin = half_bits_to_float(base[2] | (static_cast<uint32_t>(base[3]) << 8));
    const uint32_t byte = base[16 + grp * 32u + l];
    const uint32_t q = half ? byte >> 4 : byte & 15u;
    out[g] = (d * static_cast<float>(sc)) * static_cast<float>(q) - dmin * static_cast<float>(mn);
  }
}

// Workgroup-wide max of non-negative values; every thread returns it.
__device__ __forceinline__ float block_max_256(float v, float* lds) {
  v = wave_max(v);
  if ((threadIdx.x & 63u) == 0) lds[threadIdx.x >> 6] = v;
  __syncthreads();
  const float r = fmaxf(fmaxf(lds[0], lds[1]), fmaxf(lds[2], lds[3]));
  __syncthreads();
  return r;
}

__device__ __forceinline__ float e4m3_clamp_quotient(float x, float s) {
  const float q = x / s;  // correctly rounded fp32 division, as on the host
  return fminf(fmaxf(q, -kE4M3Max), kE4M3Max);
}

// Per-row dynamic E4M3 quantize-dequantize in place ("quantize_fp8",
// include/tessera/backend.hpp:296-302; src/core/numerics/quant.cpp:180-205).
// One workgroup per row.
__global__ __launch_bounds__(256) void quantize_fp8_kernel(float* __restrict__ data,
                                                           float* __restrict__ scale,
                                                           uint64_t cols) {
  __shared__ float lds[4];
  float* row = data + static_cast<uint64_t>(blockIdx.x) * cols;
  float amax = 0.0f;
  for (uint64_t c = threadIdx.x; c < cols; c += 256) amax = fmaxf(amax, fabsf(row[c]));
  amax = block_max_256(amax, lds);
  const float s = fmaxf(amax / kE4M3Max, kE4M3MinScale);
  if (threadIdx.x == 0) scale[blockIdx.x] = s;
  for (uint64_t c = threadIdx.x; c < cols; c += 256) {
    const uint32_t code = float_to_e4m3(e4m3_clamp_quotient(row[c], s));
    row[c] = e4m3_to_float(code) * s;
  }
}

__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return bit_cast<float>(b << 16); }

// Per-row dynamic E4M3 quantize to packed codes + scale ("quantize_fp8_pack",
// "quantize_fp8_pack_rows"; include/tessera/backend.hpp:303-307;
// src/core/numerics/quant.cpp:207-229).  cols is a multiple of 4; one workgroup per
// row.  kBf16 = true reads bf16 activations instead of fp32 (same values, half the
// bytes).
template <bool kBf16>
__global__ __launch_bounds__(256) void quantize_fp8_pack_kernel(const void* __restrict__ in,
                                                                uint8_t* __restrict__ out,
                                                                float* __restrict__ scale,
                                                                uint64_t cols) {
  __shared__ float lds[4];
  const uint64_t quads = cols / 4;
  const uint64_t base = static_cast<uint64_t>(blockIdx.x) * cols;
  auto load4 = [&](uint64_t q, float (&v)[4]) {
    if constexpr (kBf16) {
      const uint2 raw = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(in) + base + q * 4);
      v[0] = bf16_bits_to_float(raw.x & 0xFFFFu);
      v[1] = bf16_bits_to_float(raw.x >> 16);
      v[2] = bf16_bits_to_float(raw.y & 0xFFFFu);
      v[3] = bf16_bits_to_float(raw.y >> 16);
    } else {
      const float4 raw = *reinterpret_cast<const float4*>(static_cast<const float*>(in) + base + q * 4);
      v[0] = raw.x, v[1] = raw.y, v[2] = raw.z, v[3] = raw.w;
    }
  };
  float amax = 0.0f;
  for (uint64_t q = threadIdx.x; q < quads; q += 256) {
    float v[4];
    load4(q, v);
    amax = fmaxf(fmaxf(amax, fmaxf(fabsf(v[0]), fabsf(v[1]))), fmaxf(fabsf(v[2]), fabsf(v[3])));
  }
  amax = block_max_256(amax, lds);
  const float s = fmaxf(amax / kE4M3Max, kE4M3MinScale);
  if (threadIdx.x == 0 && blockIdx.y == 0) scale[blockIdx.x] = s;
  uint32_t* dst = reinterpret_cast<uint32_t*>(out + base);
  // grid.y workgroups share a row: each finds the row's maximum for itself (a few tens of KB
  // from L2) and rounds its own interleaved share of the quads, so the divisions and E4M3
  // roundings of a long row -- most of this kernel's time when only a few rows exist -- are spread
  // over several CUs.
  for (uint64_t q = blockIdx.y * 256ull + threadIdx.x; q < quads; q += 256ull * gridDim.y) {
    float v[4];
    load4(q, v);
    uint32_t word = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      word |= float_to_e4m3(e4m3_clamp_quotient(v[b], s)) << (8 * b);
    }
    dst[q] = word;
  }
}

// wref[r] = max over the row's E8M0 block exponents ("mxfp4_row_ref",
// src/backends/rocm/rocm_kernels_basic.cpp:1284-1303).  One wavefront per row.
__global__ __launch_bounds__(256) void mxfp4_row_ref_kernel(const uint8_t* __restrict__ w,
                                                            uint8_t* __restrict__ wref, uint64_t n,
                                                            uint64_t k) {
  const uint64_t r = static_cast<uint64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (r >= n) return;
  const uint64_t blocks = k / 32;
  const uint8_t* s = w + n * k / 2 + r * blocks;
  uint32_t ref = 0;
  for (uint64_t b = threadIdx.x & 63u; b < blocks; b += 64) ref = max(ref, static_cast<uint32_t>(s[b]));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ref = max(ref, static_cast<uint32_t>(__shfl_xor(static_cast<int>(ref), off, kWave)));
  if ((threadIdx.x & 63u) == 0) wref[r] = static_cast<uint8_t>(ref);
}

// fp32 dump of Q5_K blocks, one thread per quant byte (group g, lane l): the two values that
// share qs[g*32 + l].  Same arithmetic as the reference decode
// (src/core/numerics/quant.cpp:388-419): (d*sc)*q - dmin*mn, products exact, one rounding.
__global__ __launch_bounds__(256) void dequant_q5k_kernel(const uint8_t* __restrict__ w,
                                                          float* __restrict__ out, uint64_t nitems) {
  const uint64_t t = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= nitems) return;
  const uint64_t blk = t >> 7;
  const uint32_t g = static_cast<uint32_t>(t >> 5) & 3u, l = static_cast<uint32_t>(t) & 31u;
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
  const float d = half_bits_to_float(static_cast<uint32_t>(base[0]) | (static_cast<uint32_t>(base[1]) << 8));
  const float dmin = half_bits_to_float(static_cast<uint32_t>(base[2]) | (static_cast<uint32_t>(base[3]) << 8));
  const uint32_t low = base[48 + g * 32 + l], high = base[16 + l];
  const float q0 = static_cast<float>((low & 15u) + (((high >> (2 * g)) & 1u) << 4));
  const float q1 = static_cast<float>((low >> 4) + (((high >> (2 * g + 1)) & 1u) << 4));
  float* dst = out + blk * 256 + g * 64 + l;
  dst[0] = d * static_cast<float>(sca) * q0 - dmin * static_cast<float>(mna);
  dst[32] = d * static_cast<float>(scb) * q1 - dmin * static_cast<float>(mnb);
}

// fp32 dump of Q6_K blocks, one thread per (half n, lane l): the four values that share the
// bytes ql[n*64 + l], ql[n*64 + 32 + l] and qh[n*32 + l].  Same arithmetic as the reference
// decode (src/core/numerics/quant.cpp:421-450): (d * s) * (q - 32), both products exact.
__global__ __launch_bounds__(256) void dequant_q6k_kernel(const uint8_t* __restrict__ w,
                                                          float* __restrict__ out, uint64_t nitems) {
  const uint64_t t = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= nitems) return;
  const uint64_t blk = t >> 6;
  const uint32_t n = static_cast<uint32_t>(t >> 5) & 1u, l = static_cast<uint32_t>(t) & 31u, is = l >> 4;
  const uint8_t* base = w + blk * 210u;
  const uint32_t a = base[n * 64 + l], b = base[n * 64 + 32 + l], h = base[128 + n * 32 + l];
  const float d = half_bits_to_float(static_cast<uint32_t>(base[208]) | (static_cast<uint32_t>(base[209]) << 8));
  const int q[4] = {static_cast<int>((a & 15u) | ((h & 3u) << 4)), static_cast<int>((b & 15u) | (((h >> 2) & 3u) << 4)),
                    static_cast<int>((a >> 4) | (((h >> 4) & 3u) << 4)), static_cast<int>((b >> 4) | ((h >> 6) << 4))};
  float* dst = out + blk * 256 + n * 128 + l;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float s = static_cast<float>(static_cast<int8_t>(base[192 + n * 8 + is + 2 * j]));
    dst[32 * j] = d * s * static_cast<float>(q[j] - 32);
  }
}

// fp32 dump of Q4_K blocks, one thread per 16-byte quant chunk (32 values).  Same
// arithmetic as the reference decode (src/core/numerics/quant.cpp:656-675):
// (d*sc)*q - dmin*mn with exact products and one rounding.
__global__ __launch_bounds__(256) void dequant_q4k_kernel(const uint8_t* __restrict__ w,
                                                          float* __restrict__ out,
                                                          uint64_t nchunks) {
  const uint64_t c = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (c >= nchunks) return;
  const uint64_t blk = c >> 3;
  const uint32_t j = static_cast<uint32_t>(c & 7u), g = j >> 1, h = j & 1u;
  const uint8_t* base = w + blk * kQ4KBlockBytes;
  const uint4 hd = load_u4(base);
  const uint4 q = load_u4(base + 16 + j * 16);
  // byte i of the 12 scale bytes, picked out of the header's words (an indexed byte array would
  // live in scratch memory)
  auto p = [&](uint32_t i) {
    const uint32_t word = i < 4u ? hd.y : i < 8u ? hd.z : hd.w;
    return (word >> (8u * (i & 3u))) & 0xFFu;
  };
  auto scale_min = [&](uint32_t sb, uint32_t& sc, uint32_t& mn) {
    if (sb < 4) {
      sc = p(sb) & 63u;
      mn = p(sb + 4) & 63u;
    } else {
      sc = (p(sb + 4) & 15u) | ((p(sb - 4) >> 6) << 4);
      mn = (p(sb + 4) >> 4) | ((p(sb) >> 6) << 4);
    }
  };
  uint32_t sca, mna, scb, mnb;
  scale_min(2 * g, sca, mna);
  scale_min(2 * g + 1, scb, mnb);
  const float d = half_bits_to_float(hd.x & 0xFFFFu), dmin = half_bits_to_float(hd.x >> 16);
  const float s0 = d * static_cast<float>(sca), o0 = dmin * static_cast<float>(mna);
  const float s1 = d * static_cast<float>(scb), o1 = dmin * static_cast<float>(mnb);
  float* dst = out + blk * kQ4KBlockElems + g * 64 + h * 16;
  const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const uint32_t byte = (qw[i >> 2] >> (8 * (i & 3))) & 0xFFu;
    dst[i] = s0 * static_cast<float>(byte & 15u) - o0;
    dst[32 + i] = s1 * static_cast<float>(byte >> 4) - o1;
  }
}

// fp32 dump of packed MXFP4 weights, one thread per 32-element block.
__global__ __launch_bounds__(256) void dequant_mxfp4_kernel(const uint8_t* __restrict__ w,
                                                            float* __restrict__ out,
                                                            uint64_t nblocks, uint64_t blob_bytes) {
  const uint64_t b = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (b >= nblocks) return;
  const uint4 q = load_u4(w + b * 16);
  const float scale = e8m0_to_float(w[blob_bytes + b]);
  const uint32_t qw[4] = {q.x, q.y, q.z, q.w};
  float* dst = out + b * 32;
#pragma unroll
  for (int wi = 0; wi < 4; ++wi) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      dst[wi * 8 + j] = scale * e2m1_to_float((qw[wi] >> (4 * j)) & 15u);
    }
  }
}

// o = a + f[idx] * b ("moe_scale_add", src/backends/rocm/rocm_kernels_basic.cpp:1932-1942).
__global__ __launch_bounds__(256) void moe_scale_add_kernel(const float* __restrict__ a,
                                                            const float* __restrict__ b,
                                                            const float* __restrict__ f,
                                                            float* __restrict__ o, uint64_t n,
                                                            uint64_t idx) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) o[i] = a[i] + f[idx] * b[i];
}

// "moe_gate" (src/backends/rocm/rocm_kernels_basic.cpp:1896-1929): softmax over the top_k
// selected router logits (wts), and the shared expert's sigmoid gate sig = sigmoid(x . w).
// One workgroup of four wavefronts: the dot product is summed per wavefront with cross-lane
// adds and the four partials in order; the softmax (top_k is a handful of values) runs in the
// first wavefront, one value per lane, with wavefront-wide max and sum.  Sums are taken in
// another order than the reference's halving tree, so sig agrees to fp32 rounding, not bitwise.
__global__ __launch_bounds__(256) void moe_gate_kernel(const float* __restrict__ vals,
                                                       const float* __restrict__ x,
                                                       const float* __restrict__ w,
                                                       float* __restrict__ wts, float* __restrict__ sig,
                                                       uint32_t top_k, uint32_t hidden) {
  __shared__ float part[4];
  const uint32_t tid = threadIdx.x, lane = tid & 63u;
  float dot = 0.0f;
  for (uint32_t t = tid; t < hidden; t += 256u) dot = fmaf(x[t], w[t], dot);
  dot = wave_sum(dot);
  if (lane == 0u) part[tid >> 6] = dot;
  __syncthreads();
  if (tid < 64u) {
    // softmax over the selected logits, 64 at a time
    float m = -3.402823466e+38f;
    for (uint32_t p = lane; p < top_k; p += 64u) m = fmaxf(m, vals[p]);
    m = wave_max(m);
    float sum = 0.0f;
    for (uint32_t p = lane; p < top_k; p += 64u) sum += expf(vals[p] - m);
    sum = wave_sum(sum);
    for (uint32_t p = lane; p < top_k; p += 64u) wts[p] = expf(vals[p] - m) / sum;
    if (lane == 0u) sig[0] = 1.0f / (1.0f + expf(-(((part[0] + part[1]) + part[2]) + part[3])));
  }
}

// "top_k_rows" (src/backends/rocm/rocm_kernels_basic.cpp:3176-3243): per-row top-k of
// `vocab` fp32 logits in descending order, one workgroup per row.  Pass p selects the
// largest value not yet taken; ties go to the earlier column inside a thread's strided
// share and to the lower thread across threads, as in the reference's strict-greater merge.
__global__ __launch_bounds__(256) void top_k_rows_kernel(const float* __restrict__ logits,
                                                         uint32_t* __restrict__ ids,
                                                         float* __restrict__ vals, uint64_t vocab,
                                                         uint32_t top_k, uint64_t row_base) {
  __shared__ float rv[256];
  __shared__ uint32_t ri[256];
  __shared__ uint32_t rown[256];
  const uint32_t tid = threadIdx.x;
  const float* row = logits + (row_base + blockIdx.x) * vocab;
  // Columns this thread has already given away: they are the thread's largest, in order, so
  // "not yet taken" is "smaller than the last one given, or equal to it at a later column".
  float last_v = 0.0f;
  uint64_t last_c = 0;
  bool any = false;
  for (uint32_t p = 0; p < top_k; ++p) {
    float best = -INFINITY;
    uint64_t best_c = ~0ull;
    for (uint64_t c = tid; c < vocab; c += 256u) {
      const float v = row[c];
      const bool open = !any || v < last_v || (v == last_v && c > last_c);
      if (open && (best_c == ~0ull || v > best)) {
        best = v;
        best_c = c;
      }
    }
    rv[tid] = best_c != ~0ull ? best : -INFINITY;
    ri[tid] = best_c != ~0ull ? static_cast<uint32_t>(best_c) : 0u;
    rown[tid] = tid;
    __syncthreads();
    for (uint32_t s = 128u; s > 0u; s >>= 1) {
      if (tid < s && rv[tid + s] > rv[tid]) {
        rv[tid] = rv[tid + s];
        ri[tid] = ri[tid + s];
        rown[tid] = rown[tid + s];
      }
      __syncthreads();
    }
    if (tid == 0u) {
      vals[static_cast<size_t>(blockIdx.x) * top_k + p] = rv[0];
      ids[static_cast<size_t>(blockIdx.x) * top_k + p] = ri[0];
    }
    const uint32_t owner = rown[0];
    __syncthreads();
    if (tid == owner && best_c != ~0ull) {
      last_v = best;
      last_c = best_c;
      any = true;
    }
  }
}

inline dim3 grid_for(uint64_t count, uint32_t per_block) {
  return dim3(static_cast<uint32_t>((count + per_block - 1) / per_block));
}

}  // namespace

hipError_t launch_vec_reduce(const float* part, float* c, uint64_t total, uint64_t split,
                             hipStream_t stream) {
  hipLaunchKernelGGL(vec_reduce_kernel, grid_for(total, 256), dim3(256), 0, stream, part, c, total,
                     split);
  return hipGetLastError();
}

hipError_t launch_fill_f32(float* dst, float value, uint64_t count, hipStream_t stream) {
  if (count == 0) return hipSuccess;
  hipLaunchKernelGGL(fill_f32_kernel, grid_for(count, 256), dim3(256), 0, stream, dst, value, count);
  return hipGetLastError();
}

hipError_t launch_add(const float* a, const float* b, float* o, uint64_t n, hipStream_t stream) {
  hipLaunchKernelGGL(add_kernel, grid_for(n, 256), dim3(256), 0, stream, a, b, o, n);
  return hipGetLastError();
}

// Streaming read of `n16` 16-byte words, nothing else: the time a kernel that only has to fetch
// that many bytes takes on this device, launch ramp and tail included (the measured ceiling the
// GEMV kernels are compared with).  Each workgroup owns a contiguous range and every thread keeps
// eight 16-byte loads in flight; the xor of all words goes to out[0] only if it equals a value
// chosen so that the loads cannot be dropped.
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* __restrict__ p, size_t n16, uint32_t* out) {
  constexpr int U = 8;
  const size_t per = (n16 + gridDim.x - 1) / gridDim.x;
  const size_t lo = static_cast<size_t>(blockIdx.x) * per, hi = lo + per < n16 ? lo + per : n16;
  if (lo >= hi) return;
  uint32_t acc = 0;
  uint4 v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t i = lo + threadIdx.x + static_cast<size_t>(u) * 256u;
    v[u] = p[i < hi ? i : hi - 1];
  }
  for (size_t i = lo + threadIdx.x; i < hi; i += U * 256u) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
      const size_t nx = i + static_cast<size_t>(U + u) * 256u;
      v[u] = p[nx < hi ? nx : hi - 1];
    }
  }
  if (acc == 0x9E3779B9u) out[0] = acc;
}

hipError_t launch_read_probe(const void* src, uint32_t* out, uint64_t bytes, hipStream_t stream) {
  hipLaunchKernelGGL(read_probe_kernel, dim3(2048), dim3(256), 0, stream, static_cast<const uint4*>(src),
                     static_cast<size_t>(bytes / 16), out);
  return hipGetLastError();
}

// Ceiling of the matrix cores as the GEMMs meet it (the "mfma_probe" id): a register-only loop of one
// matrix instruction, four independent accumulators per wavefront, four wavefronts per SIMD, operands
// either constant (few bits toggle between instructions) or hashed (random bits, which is what real
// weights and activations look like and what the part's power limit prices).  kind 0:
// v_mfma_f32_32x32x16_f16, 1: v_mfma_scale_f32_32x32x64_f8f6f4 with an E4M3 and an E2M1 operand (the
// W4A8 prefill's instruction), 2: v_mfma_i32_16x16x64_i8 (the row-group decode GEMV's).
template <int KIND, bool RANDOM>
__global__ __launch_bounds__(256) void mfma_probe_kernel(float* out, uint32_t iters) {
  auto hash = [](uint32_t v) {
    v *= 2654435761u, v ^= v >> 15, v *= 2246822519u, v ^= v >> 13, v *= 3266489917u, v ^= v >> 16;
    return v;
  };
  const uint32_t seed = threadIdx.x * 8u + blockIdx.x * 977u;
  float result = 0.0f;
  if constexpr (KIND == 0) {
    half8_t a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      // random: values in [1, 2) with random mantissas and signs; constant: small integers
      const uint32_t ha = hash(seed + e), hb = hash(seed + 64u + e);
      a[e] = RANDOM ? bit_cast<_Float16>(static_cast<uint16_t>(0x3C00u | (ha & 0x83FFu))) : static_cast<_Float16>(1.0f);
      b[e] = RANDOM ? bit_cast<_Float16>(static_cast<uint16_t>(0x3C00u | (hb & 0x83FFu))) : static_cast<_Float16>(0.5f);
    }
    float16_t acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) result += acc[i][e];
  } else if constexpr (KIND == 1) {
    int8v_t a, b;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[e] = RANDOM ? static_cast<int>(hash(seed + e) & 0x77777777u) : 0x38383838;   // E4M3, exponent capped
      b[e] = RANDOM ? static_cast<int>(hash(seed + 64u + e)) : 0x22222222;           // E2M1 in the low half
    }
    float16_t acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][e] = 0.0f;
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i], 0, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) result += acc[i][e];
  } else {
    int4v_t a, b;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      a[e] = RANDOM ? static_cast<int>(hash(seed + e)) : 0x01010101;
      b[e] = RANDOM ? static_cast<int>(hash(seed + 64u + e) & 0x0F0F0F0Fu) : 0x03030303;
    }
    int4v_t acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = int4v_t{0, 0, 0, 0};
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[i], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) result += static_cast<float>(acc[i][0] ^ acc[i][1] ^ acc[i][2] ^ acc[i][3]);
  }
  out[static_cast<size_t>(blockIdx.x) * 256u + threadIdx.x] = result;
}

hipError_t launch_mfma_probe(float* out, uint32_t kind, bool random, uint32_t iters, uint32_t workgroups,
                             hipStream_t stream) {
#define QMM_PROBE(K)                                                                                          \
  if (kind == K) {                                                                                            \
    if (random) hipLaunchKernelGGL((mfma_probe_kernel<K, true>), dim3(workgroups), dim3(256), 0, stream, out, iters); \
    else hipLaunchKernelGGL((mfma_probe_kernel<K, false>), dim3(workgroups), dim3(256), 0, stream, out, iters);       \
    return hipGetLastError();                                                                                 \
  }
  QMM_PROBE(0) QMM_PROBE(1) QMM_PROBE(2)
#undef QMM_PROBE
  return hipErrorInvalidValue;
}

hipError_t launch_fill_i32(int32_t* out, int32_t value, uint64_t n, hipStream_t stream) {
  hipLaunchKernelGGL(fill_i32_kernel, grid_for(n, 256), dim3(256), 0, stream, out, value, n);
  return hipGetLastError();
}

hipError_t launch_rmsnorm(const float* x, const float* w, float* y, uint64_t rows, uint64_t cols, float eps,
                          hipStream_t stream) {
  hipLaunchKernelGGL(rmsnorm_kernel, dim3(static_cast<uint32_t>(rows)), dim3(256), 0, stream, x, w, y, cols, eps);
  return hipGetLastError();
}

// kind 0: fp32 table, 1: bf16, 2: Q4_K
hipError_t launch_embedding(int kind, const uint32_t* ids, const void* table, float* out, uint64_t rows,
                            uint64_t cols, uint64_t vocab, hipStream_t stream) {
  const dim3 grid = grid_for(rows * cols, 256);
  if (kind == 0) {
    hipLaunchKernelGGL(embedding_kernel<0>, grid, dim3(256), 0, stream, ids, table, out, rows, cols, vocab);
  } else if (kind == 1) {
    hipLaunchKernelGGL(embedding_kernel<1>, grid, dim3(256), 0, stream, ids, table, out, rows, cols, vocab);
  } else {
    hipLaunchKernelGGL(embedding_kernel<2>, grid, dim3(256), 0, stream, ids, table, out, rows, cols, vocab);
  }
  return hipGetLastError();
}

hipError_t launch_silu_mul(const float* g, const float* u, float* o, uint64_t n, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(silu_mul_kernel, grid_for(n, 256), dim3(256), 0, stream, g, u, o, n);
  return hipGetLastError();
}

hipError_t launch_round_bf16(float* x, uint64_t n, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  hipLaunchKernelGGL(round_bf16_kernel, grid_for(n, 256), dim3(256), 0, stream, reinterpret_cast<uint32_t*>(x), n);
  return hipGetLastError();
}

hipError_t launch_quantize_fp8(float* data, float* scale, uint64_t rows, uint64_t cols,
                               hipStream_t stream) {
  hipLaunchKernelGGL(quantize_fp8_kernel, dim3(static_cast<uint32_t>(rows)), dim3(256), 0, stream,
                     data, scale, cols);
  return hipGetLastError();
}

// Workgroups per row of the pack kernel: one per 1024 columns while the rows alone cannot fill
// the chip, one otherwise.
static dim3 quantize_pack_grid(uint64_t rows, uint64_t cols) {
  uint64_t per_row = 1;
  if (rows < 256) {
    per_row = (cols + 1023) / 1024;
    if (per_row > 16) per_row = 16;
    if (per_row == 0) per_row = 1;
  }
  return dim3(static_cast<uint32_t>(rows), static_cast<uint32_t>(per_row));
}

hipError_t launch_quantize_fp8_pack(const float* in, uint8_t* out, float* scale, uint64_t rows,
                                    uint64_t cols, hipStream_t stream) {
  hipLaunchKernelGGL(quantize_fp8_pack_kernel<false>, quantize_pack_grid(rows, cols), dim3(256),
                     0, stream, static_cast<const void*>(in), out, scale, cols);
  return hipGetLastError();
}

hipError_t launch_quantize_fp8_pack_bf16(const uint16_t* in, uint8_t* out, float* scale,
                                         uint64_t rows, uint64_t cols, hipStream_t stream) {
  hipLaunchKernelGGL(quantize_fp8_pack_kernel<true>, quantize_pack_grid(rows, cols), dim3(256), 0,
                     stream, static_cast<const void*>(in), out, scale, cols);
  return hipGetLastError();
}

// Packed MXFP4 nibble bytes between row-major and the reference's 16-row fragment order
// (PermuteMxFp4ToWmma, src/core/numerics/quant.cpp:926-954): dword (t, r, s, h) of the row-major
// matrix, ((t*16 + r) * k/16 + s) * 2 + h, sits at ((t * k/16 + s) * 2 + h) * 16 + r.  One thread per
// dword; the threads past the nibble bytes copy the scale bytes unchanged.
__global__ __launch_bounds__(256) void permute_mxfp4_wmma_kernel(const uint32_t* __restrict__ in, uint32_t* __restrict__ out,
                                                                 uint64_t n, uint64_t k, int inverse) {
  const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  const uint64_t blob_dwords = n * k / 8, scale_dwords = n * k / 32 / 4;
  if (i >= blob_dwords + scale_dwords) return;
  if (i >= blob_dwords) {
    out[i] = in[i];
    return;
  }
  const uint64_t ks = k / 16;
  // i indexes the fragment order: r fastest, then h, then s, then t
  const uint64_t r = i % 16, h = (i / 16) % 2, s_ = (i / 32) % ks, t = i / (32 * ks);
  const uint64_t row_major = ((t * 16 + r) * ks + s_) * 2 + h;
  if (inverse) {
    out[row_major] = in[i];
  } else {
    out[i] = in[row_major];
  }
}

hipError_t launch_permute_mxfp4_wmma(const uint8_t* in, uint8_t* out, uint64_t n, uint64_t k, bool inverse,
                                     hipStream_t stream) {
  const uint64_t dwords = n * k / 8 + n * k / 128;
  hipLaunchKernelGGL(permute_mxfp4_wmma_kernel, grid_for(dwords, 256), dim3(256), 0, stream,
                     reinterpret_cast<const uint32_t*>(in), reinterpret_cast<uint32_t*>(out), n, k, inverse ? 1 : 0);
  return hipGetLastError();
}

hipError_t launch_mxfp4_row_ref(const uint8_t* w, uint8_t* wref, uint64_t n, uint64_t k,
                                hipStream_t stream) {
  hipLaunchKernelGGL(mxfp4_row_ref_kernel, grid_for(n, 4), dim3(256), 0, stream, w, wref, n, k);
  return hipGetLastError();
}

hipError_t launch_dequant_q5k(const uint8_t* w, float* out, uint64_t nblocks, hipStream_t stream) {
  hipLaunchKernelGGL(dequant_q5k_kernel, grid_for(nblocks * 128, 256), dim3(256), 0, stream, w, out,
                     nblocks * 128);
  return hipGetLastError();
}

hipError_t launch_dequant_q6k(const uint8_t* w, float* out, uint64_t nblocks, hipStream_t stream) {
  hipLaunchKernelGGL(dequant_q6k_kernel, grid_for(nblocks * 64, 256), dim3(256), 0, stream, w, out,
                     nblocks * 64);
  return hipGetLastError();
}

hipError_t launch_dequant_q4k(const uint8_t* w, float* out, uint64_t nblocks, hipStream_t stream) {
  hipLaunchKernelGGL(dequant_q4k_kernel, grid_for(nblocks * 8, 256), dim3(256), 0, stream, w, out,
                     nblocks * 8);
  return hipGetLastError();
}

hipError_t launch_dequant_mxfp4(const uint8_t* w, float* out, uint64_t n, uint64_t k,
                                hipStream_t stream) {
  const uint64_t nblocks = n * k / 32;
  hipLaunchKernelGGL(dequant_mxfp4_kernel, grid_for(nblocks, 256), dim3(256), 0, stream, w, out,
                     nblocks, n * k / 2);
  return hipGetLastError();
}

hipError_t launch_moe_scale_add(const float* a, const float* b, const float* f, float* o,
                                uint64_t n, uint64_t idx, hipStream_t stream) {
  hipLaunchKernelGGL(moe_scale_add_kernel, grid_for(n, 256), dim3(256), 0, stream, a, b, f, o, n,
                     idx);
  return hipGetLastError();
}

hipError_t launch_moe_gate(const float* vals, const float* x, const float* w, float* wts, float* sig,
                           uint32_t top_k, uint32_t hidden, hipStream_t stream) {
  hipLaunchKernelGGL(moe_gate_kernel, dim3(1), dim3(256), 0, stream, vals, x, w, wts, sig, top_k, hidden);
  return hipGetLastError();
}

hipError_t launch_top_k_rows(const float* logits, uint32_t* ids, float* vals, uint32_t rows,
                             uint64_t vocab, uint32_t top_k, uint64_t row_base, hipStream_t stream) {
  hipLaunchKernelGGL(top_k_rows_kernel, dim3(rows), dim3(256), 0, stream, logits, ids, vals, vocab, top_k,
                     row_base);
  return hipGetLastError();
}

}  // namespace qmm
