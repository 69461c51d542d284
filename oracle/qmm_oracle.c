/*
 * CPU oracle for the quantized-matmul path: TEST INFRASTRUCTURE ONLY.
 *
 * A plain-C restatement of the host reference numerics of Quackster/tessera
 * (src/core/numerics/{quant,gemm,moe_cpu}.cpp).  Nothing in the product may
 * call into this file: it is the checker used by tests/, by the smoke check
 * and by the CPU-baseline leg of the benchmark, never the thing shipped or
 * measured as the product.
 *
 * Every routine cites the reference lines it follows.  Each is pinned by
 * tests/test_oracle_*.py against closed forms, exhaustive sweeps against
 * numpy/torch IEEE conversions, brute-force layout extraction and the few
 * known-answer values the reference documents (see the test files).  The
 * reference ships no test fixtures for this path, and its own sources do not
 * compile in this image (they need the C++23 <expected> header), so no
 * compiled-reference cross-check exists.
 *
 * Pin status:
 *   fp16/bf16/e4m3/e8m0/e2m1 codecs ......... pinned (exhaustive)
 *   Q4_K scale unpack + block decode ........ pinned (bit-serial brute force, closed form)
 *   Q5_K block decode + gemm ................ pinned (bit-serial extraction from the layout text,
 *                                             closed form RN32(d*sc*q - dmin*mn), one-hot)
 *   Q6_K block decode + gemm ................ pinned (bit-serial extraction from the layout text,
 *                                             closed form d*s*(q-32) exact in fp32, one-hot)
 *   fp8 per-row quantize (QDQ and pack) ..... pinned (invariants + torch.float8_e4m3fn)
 *   gemm_* sequential-fma references ........ pinned (one-hot identity, float64 bound)
 *   MXFP4->e4m3 fold table .................. pinned (the reference's literal 16x8 table, kept
 *                                             as a golden fixture; equals the encoder except 3
 *                                             tie entries)
 *   MoE expert forward / gate ............... pinned (composition of pinned parts; softmax
 *                                             vs torch)
 *   rmsnorm ................................. pinned (float64 evaluation, scale invariance, unit
 *                                             rows)
 *   embedding gather ........................ pinned (composition of the pinned decoders with an
 *                                             index; out-of-range ids give zero rows)
 *   silu_mul ................................ pinned (float64 evaluation within 2 ulp, silu(0) = 0,
 *                                             silu(x) - silu(-x) = x, large |x| limits)
 *   MXFP4 fragment-order permutation ........ pinned (an axis transpose of the bytes, numpy)
 *   rope / mrope ............................ pinned (complex multiplication by exp(i angle) in
 *                                             float64, position 0 = identity, pair norms kept,
 *                                             mrope with equal positions = rope)
 *   attention (fp32 and fp16 keys/values) ... pinned (torch softmax(q k^T / sqrt(d)) v with the
 *                                             causal / window mask built independently; one key =
 *                                             its value row)
 *   qgate_split ............................. pinned (numpy reshape)
 *   quantize_q8 / quantize_q4 ............... pinned (float64 half-away rounding written with floor,
 *                                             |x - q s| <= s / 2, extremes map to +-127 / +-7)
 *   attention over int8 / 4-bit / E4M3 keys . pinned (numpy / torch decode of the codes fed to torch
 *                                             softmax attention)
 *   attention_split / attention_combine ..... pinned (each chunk's pacc / psum equals torch attention
 *                                             over that chunk's keys alone, pmax the float64 maximum;
 *                                             combine(split) equals the unsplit attention)
 *   cast_f32_f16 (significand cut) .......... pinned (numpy float16 stepped toward zero when the
 *                                             nearest value lies above the input)
 *
 * Status codes mirror tessera::StatusCode (include/tessera/types.hpp:36-48).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORC_OK 0
#define ORC_INVALID_ARGUMENT 1
#define ORC_UNSUPPORTED 4
#define ORC_OOM 5

#define Q4K_ELEMS 256u
#define Q4K_BYTES 144u
#define Q5K_BYTES 176u
#define Q6K_BYTES 210u
#define MX_BLOCK 32u

/* quant.hpp:58-64 */
static const float kE4M3Max = 448.0f;
static const float kE4M3MinScale = 1.0f / (448.0f * 512.0f);

static uint32_t f32_bits(float v) {
  uint32_t b;
  memcpy(&b, &v, 4);
  return b;
}
static float bits_f32(uint32_t b) {
  float v;
  memcpy(&v, &b, 4);
  return v;
}

/* ---- IEEE binary16 -> binary32, exact (quant.cpp:74-91) ---- */
float orc_fp16_to_float(uint16_t h) {
  const uint32_t s = h >> 15, e = (h >> 10) & 31u, m = h & 1023u;
  float v;
  if (e == 0) {
    v = (float)m * 0x1p-24f;
  } else if (e == 31) {
    v = m ? nanf("") : INFINITY;
  } else {
    v = (1.0f + (float)m / 1024.0f) * ldexpf(1.0f, (int)e - 15);
  }
  return s ? -v : v;
}

/* Right shift with round-to-nearest-even (quant.cpp:42-52). */
static uint32_t shift_rne(uint32_t v, int sh) {
  const uint32_t rem = v & ((1u << sh) - 1u), half = 1u << (sh - 1);
  uint32_t r = v >> sh;
  if (rem > half || (rem == half && (r & 1u))) ++r;
  return r;
}

/* ---- binary32 -> binary16 bits, RNE (quant.cpp:606-654) ---- */
uint16_t orc_fp32_to_half_bits(float v) {
  const uint32_t b = f32_bits(v);
  const uint32_t s = b >> 31, ef = (b >> 23) & 255u, m = b & 0x7FFFFFu;
  const uint16_t inf = (uint16_t)((s << 15) | 0x7C00u);
  if (ef == 255u) return (uint16_t)(inf | (m ? 0x200u : 0u));
  if (ef == 0u) return (uint16_t)(s << 15);
  const int e = (int)ef - 127;
  if (e > 15) return inf;
  if (e < -14) {
    const int sh = -e - 1;
    if (sh >= 32) return (uint16_t)(s << 15);
    const uint32_t r = shift_rne(m + (1u << 23), sh);
    if (r > 1023u) return (uint16_t)((s << 15) | 0x0400u);
    return (uint16_t)((s << 15) | r);
  }
  const uint32_t m10 = shift_rne(m, 13);
  if (m10 > 1023u) {
    if (e + 1 > 15) return inf;
    return (uint16_t)((s << 15) | ((uint32_t)(e + 1 + 15) << 10));
  }
  return (uint16_t)((s << 15) | ((uint32_t)(e + 15) << 10) | m10);
}

/* ---- fp32 -> nearest bf16 value kept in fp32 storage (quant.cpp:231-243) ---- */
void orc_round_bf16(float* x, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    uint32_t b = f32_bits(x[i]);
    b += 0x7FFFu + ((b >> 16) & 1u);
    b &= 0xFFFF0000u;
    x[i] = bits_f32(b);
  }
}

/* ---- OCP FP8 E4M3 byte -> fp32 (quant.cpp:258-277) ---- */
float orc_fp8_e4m3_to_float(uint8_t c) {
  const uint32_t s = c >> 7, e = (c >> 3) & 15u, m = c & 7u;
  float v;
  if (e == 0) {
    v = (float)m * 0x1p-9f;
  } else if (e == 15) {
    if (m == 7) return nanf("");
    v = (1.0f + (float)m / 8.0f) * 256.0f;
  } else {
    v = (1.0f + (float)m / 8.0f) * ldexpf(1.0f, (int)e - 7);
  }
  return s ? -v : v;
}

/* ---- E8M0 shared exponent -> fp32: 2^(s-127) (quant.cpp:279-281) ---- */
float orc_e8m0_to_float(uint8_t s) { return ldexpf(1.0f, (int)s - 127); }

/* ---- OCP E2M1 nibble -> fp32 (quant.cpp:283-297) ---- */
float orc_f4e2m1_to_float(uint8_t nib) {
  const uint32_t s = (nib >> 3) & 1u, e = (nib >> 1) & 3u, m = nib & 1u;
  float v;
  if (e == 0) {
    v = (float)m * 0.5f;
  } else {
    v = (1.0f + (float)m / 2.0f) * ldexpf(1.0f, (int)e - 1);
  }
  return s ? -v : v;
}

/* ---- fp32 -> OCP FP8 E4M3 byte, RNE, NaN and |x|>448 -> 0x7F (quant.cpp:299-342) ---- */
uint8_t orc_fp32_to_fp8_e4m3(float v) {
  const uint32_t b = f32_bits(v);
  const uint32_t s = b >> 31;
  if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint8_t)((s << 7) | 0x7Fu);
  const float a = v < 0 ? -v : v;
  if (a == 0.0f) return (uint8_t)(s << 7);
  if (a > 448.0f) return (uint8_t)((s << 7) | 0x7Fu);
  int ex = 0;
  const float fr = frexpf(a, &ex); /* a = fr * 2^ex, fr in [0.5, 1) */
  int field = ex + 6;
  if (field < 1) {
    long long m = llrintf(a * 512.0f);
    if (m > 7) m = 7;
    return (uint8_t)((s << 7) | (uint32_t)m);
  }
  long long m = llrintf((fr * 2.0f - 1.0f) * 8.0f);
  if (m == 8) {
    m = 0;
    ++field;
  }
  if (field > 15) field = 15;
  if (field == 15 && m > 6) m = 6;
  return (uint8_t)((s << 7) | ((uint32_t)field << 3) | (uint32_t)m);
}

/* ---- Q4_K 6-bit (scale, min) pair of sub-block j from the 12-byte packing
 *      (quant.cpp:58-70; layout text quant.hpp:11-15) ---- */
void orc_get_scale_min(size_t j, const uint8_t* p, uint8_t* sc, uint8_t* mn) {
  if (j < 4) {
    *sc = p[j] & 63u;
    *mn = p[j + 4] & 63u;
  } else {
    *sc = (uint8_t)((p[j + 4] & 15u) | ((p[j - 4] >> 6) << 4));
    *mn = (uint8_t)((p[j + 4] >> 4) | ((p[j] >> 6) << 4));
  }
}

/* ---- one 144-byte Q4_K super-block -> 256 fp32 (quant.cpp:656-675) ---- */
void orc_dequantize_q4k(const uint8_t* blk, float* out) {
  const float d = orc_fp16_to_float((uint16_t)(blk[0] | (blk[1] << 8)));
  const float dmin = orc_fp16_to_float((uint16_t)(blk[2] | (blk[3] << 8)));
  const uint8_t* sp = blk + 4;
  const uint8_t* qs = blk + 16;
  for (size_t g = 0; g < 4; ++g) {
    uint8_t sc0, mn0, sc1, mn1;
    orc_get_scale_min(2 * g, sp, &sc0, &mn0);
    orc_get_scale_min(2 * g + 1, sp, &sc1, &mn1);
    const float s0 = d * (float)sc0, o0 = dmin * (float)mn0;
    const float s1 = d * (float)sc1, o1 = dmin * (float)mn1;
    for (size_t l = 0; l < 32; ++l) {
      const uint8_t q = qs[32 * g + l];
      out[64 * g + l] = s0 * (float)(q & 15u) - o0;
      out[64 * g + 32 + l] = s1 * (float)(q >> 4) - o1;
    }
  }
}

void orc_dequantize_q4k_rows(const uint8_t* w, float* out, size_t nblocks) {
  for (size_t b = 0; b < nblocks; ++b) orc_dequantize_q4k(w + b * Q4K_BYTES, out + b * Q4K_ELEMS);
}

static uint32_t round_half_even_u32(float v) {
  const long long r = llrint((double)v);
  return r < 0 ? 0u : (uint32_t)r;
}

/* ---- 256 fp32 -> one Q4_K super-block, fixture builder (quant.cpp:677-739) ---- */
void orc_quantize_q4k(const float* x, uint8_t* blk) {
  memset(blk, 0, Q4K_BYTES);
  float amax = 0.0f;
  for (size_t i = 0; i < Q4K_ELEMS; ++i) amax = fmaxf(amax, fabsf(x[i]));
  if (amax == 0.0f) return;
  const uint16_t db = orc_fp32_to_half_bits(amax / 32.0f);
  const float d = orc_fp16_to_float(db), dm = d;
  blk[0] = blk[2] = (uint8_t)(db & 255u);
  blk[1] = blk[3] = (uint8_t)(db >> 8);
  uint8_t* sp = blk + 4;
  uint8_t* qs = blk + 16;
  for (size_t j = 0; j < 8; ++j) {
    const float* sub = x + 32 * j;
    float lo = sub[0], hi = sub[0];
    for (size_t i = 1; i < 32; ++i) {
      lo = fminf(lo, sub[i]);
      hi = fmaxf(hi, sub[i]);
    }
    const float emin = fminf(lo, 0.0f);
    const float step = (hi - emin) / 15.0f;
    uint32_t sc = round_half_even_u32(step / d);
    if (sc > 63u) sc = 63u;
    uint32_t m = 0;
    if (lo < 0.0f) {
      m = round_half_even_u32(-lo / dm);
      if (m > 63u) m = 63u;
    }
    if (j < 4) {
      sp[j] = (uint8_t)sc;
      sp[j + 4] = (uint8_t)m;
    } else {
      sp[j + 4] = (uint8_t)((sc & 15u) | ((m & 15u) << 4));
      sp[j - 4] |= (uint8_t)((sc >> 4) << 6);
      sp[j] |= (uint8_t)((m >> 4) << 6);
    }
    const float off = dm * (float)m, scale = d * (float)sc;
    for (size_t i = 0; i < 32; ++i) {
      uint32_t q = 0;
      if (sc != 0) {
        q = round_half_even_u32((sub[i] + off) / scale);
        if (q > 15u) q = 15u;
      }
      const size_t el = 32 * j + i;
      const size_t at = 32 * (el / 64) + el % 32;
      if ((el / 32) % 2 == 1) {
        qs[at] |= (uint8_t)(q << 4);
      } else {
        qs[at] |= (uint8_t)(q & 15u);
      }
    }
  }
}

/* orc_fp32_to_fp8_e4m3 over an array, spread over OpenMP threads (for sweeps over all inputs). */
void orc_fp32_to_fp8_e4m3_many(const float* v, uint8_t* out, size_t n) {
#pragma omp parallel for schedule(static)
  for (long long i = 0; i < (long long)n; ++i) out[i] = orc_fp32_to_fp8_e4m3(v[i]);
}

/* ---- per-row dynamic E4M3 quantize-dequantize in place (quant.cpp:180-205) ---- */
int orc_quantize_fp8_ref(float* data, float* scale, size_t rows, size_t cols) {
  if (rows == 0 || cols == 0) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    float* row = data + r * cols;
    float amax = 0.0f;
    for (size_t c = 0; c < cols; ++c) amax = fmaxf(amax, fabsf(row[c]));
    const float s = fmaxf(amax / kE4M3Max, kE4M3MinScale);
    scale[r] = s;
    for (size_t c = 0; c < cols; ++c) {
      float q = row[c] / s;
      q = q < -kE4M3Max ? -kE4M3Max : (q > kE4M3Max ? kE4M3Max : q);
      row[c] = orc_fp8_e4m3_to_float(orc_fp32_to_fp8_e4m3(q)) * s;
    }
  }
  return ORC_OK;
}

/* ---- per-row dynamic E4M3 quantize to packed bytes + scale (quant.cpp:207-229) ---- */
int orc_quantize_fp8_pack_ref(const float* in, uint8_t* out, float* scale, size_t rows,
                              size_t cols) {
  if (rows == 0 || cols == 0 || cols % 4 != 0) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    const float* row = in + r * cols;
    float amax = 0.0f;
    for (size_t c = 0; c < cols; ++c) amax = fmaxf(amax, fabsf(row[c]));
    const float s = fmaxf(amax / kE4M3Max, kE4M3MinScale);
    scale[r] = s;
    for (size_t c = 0; c < cols; ++c) {
      float q = row[c] / s;
      q = q < -kE4M3Max ? -kE4M3Max : (q > kE4M3Max ? kE4M3Max : q);
      out[r * cols + c] = orc_fp32_to_fp8_e4m3(q);
    }
  }
  return ORC_OK;
}

/* ---- C = A . deq(W)^T, Q4_K rows, sequential fp32 fma over t = 0..k-1
 *      (gemm.cpp:18-41,62-73) ---- */
int orc_gemm_q4k_ref(const float* a, const uint8_t* w, float* c, size_t m, size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0 || k % Q4K_ELEMS != 0) return ORC_INVALID_ARGUMENT;
  const size_t bpr = k / Q4K_ELEMS;
  float* row = (float*)malloc(k * sizeof(float));
  if (!row) return ORC_OOM;
  for (size_t j = 0; j < n; ++j) {
    orc_dequantize_q4k_rows(w + j * bpr * Q4K_BYTES, row, bpr);
    for (size_t i = 0; i < m; ++i) {
      const float* ar = a + i * k;
      float acc = 0.0f;
      for (size_t t = 0; t < k; ++t) acc = fmaf(ar[t], row[t], acc);
      c[i * n + j] = acc;
    }
  }
  free(row);
  return ORC_OK;
}

/* ---- Q5_K block decode (quant.cpp:388-419; layout quant.hpp:592-595): 176 bytes = fp16 d, fp16
 *      dmin, 12 bytes of 6-bit scales/mins packed as in Q4_K, qh[32] high bits, qs[128] low
 *      nibbles; 256 values.  For group g in 0..3 and l in 0..31:
 *        out[g*64 + l]      = d*sc[2g]   * ((qs[g*32+l] & 15) + 16*bit(qh[l], 2g))   - dmin*mn[2g]
 *        out[g*64 + 32 + l] = d*sc[2g+1] * ((qs[g*32+l] >> 4) + 16*bit(qh[l], 2g+1)) - dmin*mn[2g+1]
 *      with d*sc and dmin*mn formed first in fp32 (both exact), one rounding at the subtract. ---- */
void orc_dequantize_q5k(const uint8_t* blk, float* out) {
  const float d = orc_fp16_to_float((uint16_t)(blk[0] | (blk[1] << 8)));
  const float dmin = orc_fp16_to_float((uint16_t)(blk[2] | (blk[3] << 8)));
  const uint8_t* scales = blk + 4;
  const uint8_t* qh = blk + 16;
  const uint8_t* qs = blk + 48;
  for (size_t g = 0; g < 4; ++g) {
    uint8_t sc0, mn0, sc1, mn1;
    orc_get_scale_min(2 * g, scales, &sc0, &mn0);
    orc_get_scale_min(2 * g + 1, scales, &sc1, &mn1);
    const float d1 = d * (float)sc0, m1 = dmin * (float)mn0;
    const float d2 = d * (float)sc1, m2 = dmin * (float)mn1;
    for (size_t l = 0; l < 32; ++l) {
      const uint8_t low = qs[g * 32 + l], high = qh[l];
      out[g * 64 + l] = d1 * ((float)(low & 0xF) + (((high >> (2 * g)) & 1) ? 16.0f : 0.0f)) - m1;
      out[g * 64 + 32 + l] = d2 * ((float)(low >> 4) + (((high >> (2 * g + 1)) & 1) ? 16.0f : 0.0f)) - m2;
    }
  }
}

void orc_dequantize_q5k_rows(const uint8_t* w, float* out, size_t nblocks) {
  for (size_t b = 0; b < nblocks; ++b) orc_dequantize_q5k(w + b * Q5K_BYTES, out + b * Q4K_ELEMS);
}

/* ---- C = A . deq(W)^T, Q5_K rows, sequential fp32 fma (gemm.cpp:18-41,75-86). ---- */
int orc_gemm_q5k_ref(const float* a, const uint8_t* w, float* c, size_t m, size_t n, size_t k,
                     int threads) {
  if (m == 0 || n == 0 || k == 0 || k % Q4K_ELEMS != 0) return ORC_INVALID_ARGUMENT;
  const size_t bpr = k / Q4K_ELEMS;
  int failed = 0;
#pragma omp parallel if (threads)
  {
    float* row = (float*)malloc(k * sizeof(float));
    if (!row) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp for schedule(static)
    for (long long j = 0; j < (long long)n; ++j) {
      if (!row) continue;
      orc_dequantize_q5k_rows(w + (size_t)j * bpr * Q5K_BYTES, row, bpr);
      for (size_t i = 0; i < m; ++i) {
        const float* ar = a + i * k;
        float acc = 0.0f;
        for (size_t t = 0; t < k; ++t) acc = fmaf(ar[t], row[t], acc);
        c[i * n + (size_t)j] = acc;
      }
    }
    free(row);
  }
  return failed ? ORC_OOM : ORC_OK;
}

/* ---- Q6_K block decode (quant.cpp:421-450; layout quant.hpp:597-600): 210 bytes = ql[128]
 *      low nibbles, qh[64] two high bits each, 16 int8 scales, fp16 d; 256 values.  For half
 *      n in 0..1 and l in 0..31, is = l / 16:
 *        out[n*128 +  0 + l] = d * s[n*8 + is + 0] * (((ql[n*64 + l]      & 15) | ((qh[n*32+l] >> 0 & 3) << 4)) - 32)
 *        out[n*128 + 32 + l] = d * s[n*8 + is + 2] * (((ql[n*64 + 32 + l] & 15) | ((qh[n*32+l] >> 2 & 3) << 4)) - 32)
 *        out[n*128 + 64 + l] = d * s[n*8 + is + 4] * (((ql[n*64 + l]      >> 4) | ((qh[n*32+l] >> 4 & 3) << 4)) - 32)
 *        out[n*128 + 96 + l] = d * s[n*8 + is + 6] * (((ql[n*64 + 32 + l] >> 4) | ((qh[n*32+l] >> 6 & 3) << 4)) - 32)
 *      evaluated as (d * s) * (q - 32) in fp32, both products exact (11 + 8 + 6 bits). ---- */
void orc_dequantize_q6k(const uint8_t* blk, float* out) {
  const uint8_t* ql = blk;
  const uint8_t* qh = blk + 128;
  const int8_t* sc = (const int8_t*)(blk + 192);
  const float d = orc_fp16_to_float((uint16_t)(blk[208] | (blk[209] << 8)));
  for (size_t n = 0; n < 2; ++n) {
    for (size_t l = 0; l < 32; ++l) {
      const size_t is = l / 16;
      const uint8_t h = qh[n * 32 + l];
      const int q1 = (ql[n * 64 + l] & 0xF) | (((h >> 0) & 3) << 4);
      const int q2 = (ql[n * 64 + 32 + l] & 0xF) | (((h >> 2) & 3) << 4);
      const int q3 = (ql[n * 64 + l] >> 4) | (((h >> 4) & 3) << 4);
      const int q4 = (ql[n * 64 + 32 + l] >> 4) | (((h >> 6) & 3) << 4);
      out[n * 128 + l] = d * (float)sc[n * 8 + is + 0] * (float)(q1 - 32);
      out[n * 128 + 32 + l] = d * (float)sc[n * 8 + is + 2] * (float)(q2 - 32);
      out[n * 128 + 64 + l] = d * (float)sc[n * 8 + is + 4] * (float)(q3 - 32);
      out[n * 128 + 96 + l] = d * (float)sc[n * 8 + is + 6] * (float)(q4 - 32);
    }
  }
}

void orc_dequantize_q6k_rows(const uint8_t* w, float* out, size_t nblocks) {
  for (size_t b = 0; b < nblocks; ++b) orc_dequantize_q6k(w + b * Q6K_BYTES, out + b * Q4K_ELEMS);
}

/* ---- C = A . deq(W)^T, Q6_K rows, sequential fp32 fma (gemm.cpp:18-41,88-99); weight rows
 *      spread over OpenMP threads when `threads` is non-zero (each output keeps its chain). ---- */
int orc_gemm_q6k_ref(const float* a, const uint8_t* w, float* c, size_t m, size_t n, size_t k,
                     int threads) {
  if (m == 0 || n == 0 || k == 0 || k % Q4K_ELEMS != 0) return ORC_INVALID_ARGUMENT;
  const size_t bpr = k / Q4K_ELEMS;
  int failed = 0;
#pragma omp parallel if (threads)
  {
    float* row = (float*)malloc(k * sizeof(float));
    if (!row) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp for schedule(static)
    for (long long j = 0; j < (long long)n; ++j) {
      if (!row) continue;
      orc_dequantize_q6k_rows(w + (size_t)j * bpr * Q6K_BYTES, row, bpr);
      for (size_t i = 0; i < m; ++i) {
        const float* ar = a + i * k;
        float acc = 0.0f;
        for (size_t t = 0; t < k; ++t) acc = fmaf(ar[t], row[t], acc);
        c[i * n + (size_t)j] = acc;
      }
    }
    free(row);
  }
  return failed ? ORC_OOM : ORC_OK;
}

/* Same arithmetic, weight rows spread over OpenMP threads.  Each output keeps
 * the sequential-t fma chain, so results equal orc_gemm_q4k_ref bit for bit.
 * Used only to time a multi-core CPU baseline. */
int orc_gemm_q4k_ref_omp(const float* a, const uint8_t* w, float* c, size_t m, size_t n,
                         size_t k) {
  if (m == 0 || n == 0 || k == 0 || k % Q4K_ELEMS != 0) return ORC_INVALID_ARGUMENT;
  const size_t bpr = k / Q4K_ELEMS;
  int failed = 0;
#pragma omp parallel
  {
    float* row = (float*)malloc(k * sizeof(float));
    if (!row) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp for schedule(static)
    for (long long j = 0; j < (long long)n; ++j) {
      if (!row) continue;
      orc_dequantize_q4k_rows(w + (size_t)j * bpr * Q4K_BYTES, row, bpr);
      for (size_t i = 0; i < m; ++i) {
        const float* ar = a + i * k;
        float acc = 0.0f;
        for (size_t t = 0; t < k; ++t) acc = fmaf(ar[t], row[t], acc);
        c[i * n + (size_t)j] = acc;
      }
    }
    free(row);
  }
  return failed ? ORC_OOM : ORC_OK;
}

/* ---- C = A . deq(W)^T, MXFP4 blob + E8M0 scales given separately
 *      (gemm.cpp:311-344); low nibble = even element ---- */
int orc_gemm_mxfp4_ref(const float* a, const uint8_t* w, const uint8_t* s, float* c, size_t m,
                       size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0 || k % MX_BLOCK != 0) return ORC_INVALID_ARGUMENT;
  const size_t nb = k / MX_BLOCK;
  for (size_t i = 0; i < m; ++i) {
    for (size_t j = 0; j < n; ++j) {
      float acc = 0.0f;
      for (size_t b = 0; b < nb; ++b) {
        const float sc = orc_e8m0_to_float(s[j * nb + b]);
        for (size_t l = 0; l < MX_BLOCK; ++l) {
          const size_t t = b * MX_BLOCK + l;
          const uint8_t byte = w[(j * k + t) / 2];
          const uint8_t nib = (t % 2 == 0) ? (byte & 15u) : (byte >> 4);
          acc = fmaf(a[i * k + t], sc * orc_f4e2m1_to_float(nib), acc);
        }
      }
      c[i * n + j] = acc;
    }
  }
  return ORC_OK;
}

/* Same arithmetic with the weight rows spread over OpenMP threads: a row is decoded once (the
 * same product sc * e2m1 as above), every output keeps its sequential fma chain, so the result
 * equals orc_gemm_mxfp4_ref bit for bit (checked in tests/test_oracle_gemm.py). */
int orc_gemm_mxfp4_ref_omp(const float* a, const uint8_t* w, const uint8_t* s, float* c, size_t m,
                           size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0 || k % MX_BLOCK != 0) return ORC_INVALID_ARGUMENT;
  const size_t nb = k / MX_BLOCK;
  int failed = 0;
#pragma omp parallel
  {
    float* row = (float*)malloc(k * sizeof(float));
    if (!row) {
#pragma omp atomic write
      failed = 1;
    }
#pragma omp for schedule(static)
    for (long long j = 0; j < (long long)n; ++j) {
      if (!row) continue;
      for (size_t t = 0; t < k; ++t) {
        const uint8_t byte = w[((size_t)j * k + t) / 2];
        const uint8_t nib = (t % 2 == 0) ? (byte & 15u) : (byte >> 4);
        row[t] = orc_e8m0_to_float(s[(size_t)j * nb + t / MX_BLOCK]) * orc_f4e2m1_to_float(nib);
      }
      for (size_t i = 0; i < m; ++i) {
        const float* ar = a + i * k;
        float acc = 0.0f;
        for (size_t t = 0; t < k; ++t) acc = fmaf(ar[t], row[t], acc);
        c[i * n + (size_t)j] = acc;
      }
    }
    free(row);
  }
  return failed ? ORC_OOM : ORC_OK;
}

/* MXFP4 weights -> fp32, n x k, from the packed device layout (blob then scales,
 * include/tessera/backend.hpp:195-201). */
int orc_dequantize_mxfp4(const uint8_t* packed, float* out, size_t n, size_t k) {
  if (n == 0 || k == 0 || k % MX_BLOCK != 0) return ORC_INVALID_ARGUMENT;
  const uint8_t* s = packed + n * k / 2;
  const size_t nb = k / MX_BLOCK;
  for (size_t j = 0; j < n; ++j) {
    for (size_t t = 0; t < k; ++t) {
      const uint8_t byte = packed[(j * k + t) / 2];
      const uint8_t nib = (t % 2 == 0) ? (byte & 15u) : (byte >> 4);
      out[j * k + t] = orc_e8m0_to_float(s[j * nb + t / MX_BLOCK]) * orc_f4e2m1_to_float(nib);
    }
  }
  return ORC_OK;
}

/* ---- C = A . (diag(s) W)^T, E4M3 weights with one fp32 scale per row
 *      (gemm.cpp:253-277) ---- */
int orc_gemm_fp8_ref(const float* a, const uint8_t* w, const float* s, float* c, size_t m,
                     size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0) return ORC_INVALID_ARGUMENT;
  for (size_t i = 0; i < m; ++i) {
    for (size_t j = 0; j < n; ++j) {
      const float sc = s[j];
      float acc = 0.0f;
      for (size_t t = 0; t < k; ++t) {
        acc = fmaf(a[i * k + t], sc * orc_fp8_e4m3_to_float(w[j * k + t]), acc);
      }
      c[i * n + j] = acc;
    }
  }
  return ORC_OK;
}

/* ---- the same with one fp32 scale per 128 x 128 block of W (gemm.cpp:282-309):
 *      s is (n/128) x (k/128), n and k multiples of 128 ---- */
int orc_gemm_fp8_block_ref(const float* a, const uint8_t* w, const float* s, float* c, size_t m,
                           size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0 || n % 128 != 0 || k % 128 != 0) return ORC_INVALID_ARGUMENT;
  const size_t k_blocks = k / 128;
  for (size_t i = 0; i < m; ++i) {
    for (size_t j = 0; j < n; ++j) {
      const float* s_row = s + (j / 128) * k_blocks;
      float acc = 0.0f;
      for (size_t t = 0; t < k; ++t) {
        acc = fmaf(a[i * k + t], s_row[t / 128] * orc_fp8_e4m3_to_float(w[j * k + t]), acc);
      }
      c[i * n + j] = acc;
    }
  }
  return ORC_OK;
}

/* e4m3 byte of (E2M1 magnitude code mag) * 2^-d, derived from the encoder with
 * round-to-nearest-even.  Agrees with the reference's literal table below except in
 * three tie entries (the tests list them). */
uint8_t orc_fold_entry_rne(unsigned d, unsigned mag) {
  const float v = ldexpf(orc_f4e2m1_to_float((uint8_t)(mag & 7u)), -(int)d);
  return orc_fp32_to_fp8_e4m3(v);
}

/* The reference's fold table as data (quant.cpp:846-863): entry [d][mag].  Where a
 * scaled magnitude falls exactly between two e4m3 subnormals (1.5 units: [9][3],
 * [10][5], [11][7]) the table holds the lower code, not the even one, so it cannot be
 * regenerated from the encoder and is kept literally. */
static const uint8_t kFoldTable[16][8] = {
    {0x00, 0x30, 0x38, 0x3c, 0x40, 0x44, 0x48, 0x4c}, {0x00, 0x28, 0x30, 0x34, 0x38, 0x3c, 0x40, 0x44},
    {0x00, 0x20, 0x28, 0x2c, 0x30, 0x34, 0x38, 0x3c}, {0x00, 0x18, 0x20, 0x24, 0x28, 0x2c, 0x30, 0x34},
    {0x00, 0x10, 0x18, 0x1c, 0x20, 0x24, 0x28, 0x2c}, {0x00, 0x08, 0x10, 0x14, 0x18, 0x1c, 0x20, 0x24},
    {0x00, 0x04, 0x08, 0x0c, 0x10, 0x14, 0x18, 0x1c}, {0x00, 0x02, 0x04, 0x06, 0x08, 0x0c, 0x10, 0x14},
    {0x00, 0x01, 0x02, 0x03, 0x04, 0x06, 0x08, 0x0c}, {0x00, 0x00, 0x01, 0x01, 0x02, 0x03, 0x04, 0x06},
    {0x00, 0x00, 0x00, 0x01, 0x01, 0x01, 0x02, 0x03}, {0x00, 0x00, 0x00, 0x00, 0x00, 0x01, 0x01, 0x01},
    {0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x01}, {0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x00},
    {0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x00}, {0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x00, 0x00},
};

uint8_t orc_fold_entry(unsigned d, unsigned mag) { return kFoldTable[d & 15u][mag & 7u]; }

/* ---- MXFP4 -> e4m3 bytes relative to the per-row max exponent
 *      (quant.cpp:865-898) ---- */
int orc_fold_mxfp4_to_fp8(const uint8_t* w, const uint8_t* s, uint8_t* out, uint8_t* wref,
                          size_t rows, size_t cols) {
  if (rows == 0 || cols == 0 || cols % MX_BLOCK != 0) return ORC_INVALID_ARGUMENT;
  const size_t nb = cols / MX_BLOCK;
  for (size_t r = 0; r < rows; ++r) {
    uint8_t ref = 0;
    for (size_t b = 0; b < nb; ++b) ref = s[r * nb + b] > ref ? s[r * nb + b] : ref;
    wref[r] = ref;
    for (size_t c = 0; c < cols; ++c) {
      const uint8_t byte = w[(r * cols + c) / 2];
      const uint8_t nib = (c % 2 == 0) ? (byte & 15u) : (byte >> 4);
      int d = (int)ref - (int)s[r * nb + c / MX_BLOCK];
      d = d < 0 ? 0 : (d > 15 ? 15 : d);
      out[r * cols + c] = (uint8_t)(orc_fold_entry((unsigned)d, nib & 7u) | ((nib & 8u) ? 0x80u : 0u));
    }
  }
  return ORC_OK;
}

/* ---- MXFP4 nibble bytes, row-major -> the 16-row fragment order of the fp8 tensor-core kernel
 *      (PermuteMxFp4ToWmma, quant.cpp:926-954): input byte (t, r, s, h, b) =
 *      (((t*16 + r)*ks + s)*2 + h)*4 + b goes to (((t*ks + s)*2 + h)*16 + r)*4 + b, ks = cols/16 ---- */
int orc_permute_mxfp4_to_wmma(const uint8_t* packed, uint8_t* out, size_t rows, size_t cols) {
  if (rows == 0 || cols == 0 || rows % 16 != 0 || cols % 16 != 0) return ORC_INVALID_ARGUMENT;
  const size_t nt = rows / 16, ks = cols / 16;
  for (size_t t = 0; t < nt; ++t) {
    for (size_t s = 0; s < ks; ++s) {
      for (size_t h = 0; h < 2; ++h) {
        for (size_t r = 0; r < 16; ++r) {
          const size_t in = (((t * 16 + r) * ks + s) * 2 + h) * 4;
          const size_t o = (((t * ks + s) * 2 + h) * 16 + r) * 4;
          for (size_t b = 0; b < 4; ++b) out[o + b] = packed[in + b];
        }
      }
    }
  }
  return ORC_OK;
}

/* ---- Q4_K row groups: the load-time copy that the gfx950 int8 matrix kernel reads.  No counterpart
 *      in the reference (its own load-time hook is PermuteMxFp4ToWmma above); this is the layout's
 *      definition, element by element, for checking the device's permutation against:
 *      rows [g*R, g*R+rows) of group g keep, per 256-wide block b, rows*144 bytes at
 *      (g*R*nblk + b*rows)*144: first the tiles' quants, then the rows' 16-byte headers.
 *      Tile t (rows 16t..16t+rt-1 of the group) has two pieces c = 0,1 of rt*64 bytes at
 *      t*2048 + c*rt*64; row nn of the tile, lane group q = 0..3, owns the 16 bytes at (q*rt + nn)*16
 *      of a piece; byte P of them holds in its low nibble weight 16*(q%2)+P of sub-block 2c + q/2 and
 *      in its high nibble the same weight of sub-block 2c + 4 + q/2 minus 8 (mod 16).
 *      Header: d, dmin as in GGUF; then byte i of the next three words = sc[2i] | (mn[2i+1] & 3) << 6,
 *      sc[2i+1] | (mn[2i+1] >> 2 & 3) << 6, mn[2i] | (mn[2i+1] >> 4) << 6 (sc, mn from GetScaleMin). ---- */
static uint32_t orc_q4k_nibble(const uint8_t* block, int sub, int l) {
  const uint8_t byte = block[16 + (sub / 2) * 32 + l];
  return (sub & 1) ? (uint32_t)(byte >> 4) : (uint32_t)(byte & 15);
}
int orc_permute_q4k_rowgroup(const uint8_t* in, uint8_t* out, size_t n, size_t k, size_t R, int inverse) {
  if (n == 0 || k == 0 || k % 256 != 0 || R == 0 || R > 64) return ORC_INVALID_ARGUMENT;
  const size_t nblk = k / 256;
  for (size_t r = 0; r < n; ++r) {
    const size_t row0 = r / R * R, rows = n - row0 < R ? n - row0 : R, rr = r - row0;
    const size_t tile = rr / 16, nn = rr % 16, rt = rows - tile * 16 < 16 ? rows - tile * 16 : 16;
    for (size_t b = 0; b < nblk; ++b) {
      const size_t gguf = (r * nblk + b) * 144, region = (row0 * nblk + b * rows) * 144;
      const size_t hdr = region + rows * 128 + rr * 16;
      if (!inverse) {
        const uint8_t* blk = in + gguf;
        uint8_t sc[8], mn[8];
        for (int j = 0; j < 8; ++j) orc_get_scale_min(j, blk + 4, &sc[j], &mn[j]);
        memcpy(out + hdr, blk, 4);
        for (int i = 0; i < 4; ++i) {
          const uint8_t mo = mn[2 * i + 1];
          out[hdr + 4 + i] = (uint8_t)(sc[2 * i] | ((mo & 3) << 6));
          out[hdr + 8 + i] = (uint8_t)(sc[2 * i + 1] | (((mo >> 2) & 3) << 6));
          out[hdr + 12 + i] = (uint8_t)(mn[2 * i] | (((mo >> 4) & 3) << 6));
        }
        for (int c = 0; c < 2; ++c) {
          for (int q = 0; q < 4; ++q) {
            uint8_t* piece = out + region + tile * 2048 + (size_t)c * rt * 64 + ((size_t)q * rt + nn) * 16;
            for (int P = 0; P < 16; ++P) {
              const int l = 16 * (q % 2) + P;
              const uint32_t lo = orc_q4k_nibble(blk, 2 * c + q / 2, l);
              const uint32_t hi = (orc_q4k_nibble(blk, 2 * c + 4 + q / 2, l) + 8u) & 15u;   /* minus 8 mod 16 */
              piece[P] = (uint8_t)(lo | (hi << 4));
            }
          }
        }
      } else {
        const uint8_t* h = in + hdr;
        uint8_t* blk = out + gguf;
        uint8_t sc[8], mn[8];
        for (int i = 0; i < 4; ++i) {
          sc[2 * i] = h[4 + i] & 63;
          sc[2 * i + 1] = h[8 + i] & 63;
          mn[2 * i] = h[12 + i] & 63;
          mn[2 * i + 1] = (uint8_t)((h[4 + i] >> 6) | ((h[8 + i] >> 6) << 2) | ((h[12 + i] >> 6) << 4));
        }
        memcpy(blk, h, 4);
        /* the reference's packing of the twelve scale bytes (quant.cpp:712-720) */
        for (int j = 0; j < 4; ++j) {
          blk[4 + j] = (uint8_t)(sc[j] | ((sc[j + 4] >> 4) << 6));
          blk[8 + j] = (uint8_t)(mn[j] | ((mn[j + 4] >> 4) << 6));
          blk[12 + j] = (uint8_t)((sc[j + 4] & 15) | ((mn[j + 4] & 15) << 4));
        }
        memset(blk + 16, 0, 128);
        for (int c = 0; c < 2; ++c) {
          for (int q = 0; q < 4; ++q) {
            const uint8_t* piece = in + region + tile * 2048 + (size_t)c * rt * 64 + ((size_t)q * rt + nn) * 16;
            for (int P = 0; P < 16; ++P) {
              const int l = 16 * (q % 2) + P, shift = (q / 2) * 4;
              const uint32_t lo = piece[P] & 15u, hi = ((uint32_t)(piece[P] >> 4) + 8u) & 15u;
              blk[16 + c * 32 + l] |= (uint8_t)(lo << shift);          /* sub-block 2c + q/2 */
              blk[16 + (c + 2) * 32 + l] |= (uint8_t)(hi << shift);    /* sub-block 2c + 4 + q/2 */
            }
          }
        }
      }
    }
  }
  return ORC_OK;
}

/* ---- folded W4A8 GEMM: (sum fma(a8, w8)) * As[m] * 2^(wref-127)
 *      (quant.cpp:900-924) ---- */
int orc_gemm_mxfp4_fp8_ref(const uint8_t* a8, const float* as, const uint8_t* w8,
                           const uint8_t* wref, float* c, size_t m, size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0) return ORC_INVALID_ARGUMENT;
  for (size_t i = 0; i < m; ++i) {
    for (size_t j = 0; j < n; ++j) {
      const float ws = exp2f((float)wref[j] - 127.0f);
      float acc = 0.0f;
      for (size_t t = 0; t < k; ++t) {
        acc = fmaf(orc_fp8_e4m3_to_float(a8[i * k + t]), orc_fp8_e4m3_to_float(w8[j * k + t]), acc);
      }
      c[i * n + j] = acc * as[i] * ws;
    }
  }
  return ORC_OK;
}

/* ---- W4A8 with the lossless weight side: per-token E4M3 QDQ of the activation
 *      (QuantizeFp8Ref) followed by GemmMxFp4Ref, computed from the packed codes:
 *      a = e4m3(code) * As[i].  Equals orc_quantize_fp8_ref + orc_gemm_mxfp4_ref
 *      bit for bit because the QDQ value is exactly that product. ---- */
int orc_gemm_mxfp4_w4a8_ref(const uint8_t* a8, const float* as, const uint8_t* w,
                            const uint8_t* s, float* c, size_t m, size_t n, size_t k) {
  if (m == 0 || n == 0 || k == 0 || k % MX_BLOCK != 0) return ORC_INVALID_ARGUMENT;
  float* a = (float*)malloc(m * k * sizeof(float));
  if (!a) return ORC_OOM;
  for (size_t i = 0; i < m; ++i) {
    for (size_t t = 0; t < k; ++t) a[i * k + t] = orc_fp8_e4m3_to_float(a8[i * k + t]) * as[i];
  }
  const int st = orc_gemm_mxfp4_ref(a, w, s, c, m, n, k);
  free(a);
  return st;
}

/* ---- router weights: softmax over the selected top-k logits
 *      (src/backends/rocm/rocm_kernels_basic.cpp:1915-1926) ---- */
void orc_moe_gate(const float* vals, float* wts, size_t top_k) {
  float mx = -3.402823466e+38f;
  for (size_t p = 0; p < top_k; ++p) mx = fmaxf(mx, vals[p]);
  float sum = 0.0f;
  for (size_t p = 0; p < top_k; ++p) sum += expf(vals[p] - mx);
  for (size_t p = 0; p < top_k; ++p) wts[p] = expf(vals[p] - mx) / sum;
}

/* ---- top-k of one row by descending value; on equal values the lower column
 *      wins (the reference kernel's exact tie order differs and depends on its
 *      thread layout, src/backends/rocm/rocm_kernels_basic.cpp:3173-3243; the
 *      generators assert tie-free inputs) ---- */
void orc_top_k_row(const float* logits, size_t n, size_t top_k, uint32_t* ids, float* vals) {
  for (size_t p = 0; p < top_k; ++p) {
    size_t best = (size_t)-1;
    for (size_t c = 0; c < n; ++c) {
      int taken = 0;
      for (size_t q = 0; q < p; ++q) taken |= (ids[q] == c);
      if (taken) continue;
      if (best == (size_t)-1 || logits[c] > logits[best]) best = c;
    }
    ids[p] = (uint32_t)best;
    vals[p] = logits[best];
  }
}

/* ---- y = x / sqrt(mean(x^2) + eps) * w per row, the sum of squares one sequential fma chain
 *      (src/core/numerics/norm.cpp:7-32) ---- */
int orc_rmsnorm(const float* x, const float* w, float* y, size_t rows, size_t cols, float eps) {
  if (rows == 0 || cols == 0 || eps < 0.0f) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    const float* xr = x + r * cols;
    float mean = 0.0f;
    for (size_t c = 0; c < cols; ++c) mean = fmaf(xr[c], xr[c], mean);
    mean /= (float)cols;
    const float gain = 1.0f / sqrtf(mean + eps);
    for (size_t c = 0; c < cols; ++c) y[r * cols + c] = xr[c] * gain * w[c];
  }
  return ORC_OK;
}

/* ---- out[row] = table[ids[row]], a zero row for an id outside the table; kind 0: fp32 table,
 *      1: bf16 (the high half of the fp32 bits), 2: Q4_K rows
 *      (src/backends/rocm/rocm_kernels_embedding.cpp:10-108) ---- */
int orc_embedding(int kind, const uint32_t* ids, const void* table, float* out, size_t rows, size_t cols,
                  size_t vocab) {
  if (rows == 0 || cols == 0 || vocab == 0 || (kind == 2 && cols % 256 != 0)) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    float* o = out + r * cols;
    const size_t id = ids[r];
    if (id >= vocab) {
      memset(o, 0, cols * sizeof(float));
    } else if (kind == 0) {
      memcpy(o, (const float*)table + id * cols, cols * sizeof(float));
    } else if (kind == 1) {
      const uint16_t* t = (const uint16_t*)table + id * cols;
      for (size_t c = 0; c < cols; ++c) o[c] = bits_f32((uint32_t)t[c] << 16);
    } else {
      orc_dequantize_q4k_rows((const uint8_t*)table + id * (cols / 256) * 144, o, cols / 256);
    }
  }
  return ORC_OK;
}

/* ---- rotary embedding in place, NeoX pairing (j, j + rope_dim/2) per head, angle
 *      (pos_base + row) * theta^(-2j/rope_dim) in double, cos and sin rounded to fp32
 *      (src/core/numerics/attention.cpp:11-44) ---- */
int orc_rope(float* io, size_t rows, size_t heads, size_t head_dim, size_t rope_dim, uint64_t pos_base, double theta) {
  if (rows == 0 || heads == 0 || head_dim == 0 || rope_dim == 0 || rope_dim > head_dim || rope_dim % 2 != 0 || !(theta > 0.0)) {
    return ORC_INVALID_ARGUMENT;
  }
  const size_t half = rope_dim / 2;
  for (size_t r = 0; r < rows; ++r) {
    const double pos = (double)(pos_base + r);
    for (size_t h = 0; h < heads; ++h) {
      float* base = io + (r * heads + h) * head_dim;
      for (size_t j = 0; j < half; ++j) {
        const double angle = pos * pow(theta, -2.0 * (double)j / (double)rope_dim);
        const float c = (float)cos(angle), s = (float)sin(angle);
        const float x1 = base[j], x2 = base[j + half];
        base[j] = x1 * c - x2 * s;
        base[j + half] = x1 * s + x2 * c;
      }
    }
  }
  return ORC_OK;
}

/* ---- multimodal rotary embedding: pair j uses the temporal, height or width position of its
 *      row by section (pairs past the sections reuse the width id)
 *      (src/core/numerics/attention.cpp:227-264) ---- */
int orc_mrope(float* io, const uint64_t* pos, size_t rows, size_t heads, size_t head_dim, size_t rope_dim,
              size_t sec_t, size_t sec_h, size_t sec_w, double theta) {
  if (rows == 0 || heads == 0 || head_dim == 0 || rope_dim == 0 || rope_dim > head_dim || rope_dim % 2 != 0 || !(theta > 0.0)) {
    return ORC_INVALID_ARGUMENT;
  }
  const size_t pairs = rope_dim / 2;
  if (sec_t + sec_h + sec_w > pairs) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    for (size_t h = 0; h < heads; ++h) {
      float* base = io + (r * heads + h) * head_dim;
      for (size_t j = 0; j < pairs; ++j) {
        const uint64_t section_pos = j < sec_t ? pos[r * 3] : (j < sec_t + sec_h ? pos[r * 3 + 1] : pos[r * 3 + 2]);
        const double angle = (double)section_pos * pow(theta, -2.0 * (double)j / (double)rope_dim);
        const float c = (float)cos(angle), s = (float)sin(angle);
        const float x1 = base[j], x2 = base[j + pairs];
        base[j] = x1 * c - x2 * s;
        base[j + pairs] = x1 * s + x2 * c;
      }
    }
  }
  return ORC_OK;
}

/* ---- softmax(q k^T / sqrt(head_dim)) v per query row and head, grouped kv heads; query row i
 *      sits at position q_base + i and, when causal, attends keys max(0, pos + 1 - window) .. min(pos,
 *      n - 1) (window 0 = all of the prefix); sequential fp32 fma dots, weights divided by the sum
 *      before they multiply v (src/core/numerics/attention.cpp:158-225).  kv_f16: keys and values are
 *      binary16 (AttentionRefF16, attention.cpp:128-156). ---- */
int orc_attention(const float* q, const void* k, const void* v, float* out, size_t m, size_t n, size_t heads,
                  size_t kv_heads, size_t head_dim, uint64_t q_base, size_t window, int kv_f16, int causal) {
  if (m == 0 || n == 0 || heads == 0 || kv_heads == 0 || head_dim == 0 || heads % kv_heads != 0) return ORC_INVALID_ARGUMENT;
  const size_t count = n * kv_heads * head_dim;
  float* kf = (float*)malloc(count * sizeof(float));
  float* vf = (float*)malloc(count * sizeof(float));
  float* scores = (float*)malloc(n * sizeof(float));
  if (!kf || !vf || !scores) {
    free(kf), free(vf), free(scores);
    return ORC_OOM;
  }
  for (size_t i = 0; i < count; ++i) {
    kf[i] = kv_f16 ? orc_fp16_to_float(((const uint16_t*)k)[i]) : ((const float*)k)[i];
    vf[i] = kv_f16 ? orc_fp16_to_float(((const uint16_t*)v)[i]) : ((const float*)v)[i];
  }
  const size_t group = heads / kv_heads;
  const float scale = 1.0f / sqrtf((float)head_dim);
  for (size_t i = 0; i < m; ++i) {
    const size_t pos = (size_t)(q_base + i);
    const size_t last = causal ? (pos >= n ? n - 1 : pos) : n - 1;
    size_t start = 0;
    if (causal) {
      start = window != 0 && pos + 1 > window ? pos + 1 - window : 0;
      if (start > last) start = last;
    }
    for (size_t h = 0; h < heads; ++h) {
      const size_t kv = h / group;
      const float* q_row = q + (i * heads + h) * head_dim;
      float row_max = 0.0f;
      int first = 1;
      for (size_t j = start; j <= last; ++j) {
        const float* k_row = kf + (j * kv_heads + kv) * head_dim;
        float dot = 0.0f;
        for (size_t e = 0; e < head_dim; ++e) dot = fmaf(q_row[e], k_row[e], dot);
        dot *= scale;
        scores[j] = dot;
        if (first || dot > row_max) row_max = dot, first = 0;
      }
      float denom = 0.0f;
      for (size_t j = start; j <= last; ++j) {
        scores[j] = expf(scores[j] - row_max);
        denom += scores[j];
      }
      float* o_row = out + (i * heads + h) * head_dim;
      for (size_t e = 0; e < head_dim; ++e) {
        float acc = 0.0f;
        for (size_t j = start; j <= last; ++j) acc = fmaf(scores[j] / denom, vf[(j * kv_heads + kv) * head_dim + e], acc);
        o_row[e] = acc;
      }
    }
  }
  free(kf), free(vf), free(scores);
  return ORC_OK;
}

/* ---- quantized key/value caches: symmetric per-row int8 (scale amax / 127) and 4-bit (amax / 7,
 *      two codes a byte, low nibble first) with round half away from zero, an all-zero row taking
 *      scale 1 (quant.cpp:123-178) ---- */
int orc_quantize_q8(const float* in, uint8_t* out, float* scale, size_t rows, size_t cols) {
  if (rows == 0 || cols == 0 || cols % 4 != 0) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    float amax = 0.0f;
    for (size_t c = 0; c < cols; ++c) amax = fmaxf(amax, fabsf(in[r * cols + c]));
    const float s = amax > 0.0f ? amax / 127.0f : 1.0f;
    scale[r] = s;
    for (size_t c = 0; c < cols; ++c) {
      long q = lroundf(in[r * cols + c] / s);
      q = q < -127 ? -127 : (q > 127 ? 127 : q);
      out[r * cols + c] = (uint8_t)(int8_t)q;
    }
  }
  return ORC_OK;
}

int orc_quantize_q4(const float* in, uint8_t* out, float* scale, size_t rows, size_t cols) {
  if (rows == 0 || cols == 0 || cols % 8 != 0) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    float amax = 0.0f;
    for (size_t c = 0; c < cols; ++c) amax = fmaxf(amax, fabsf(in[r * cols + c]));
    const float s = amax > 0.0f ? amax / 7.0f : 1.0f;
    scale[r] = s;
    for (size_t c = 0; c < cols; c += 2) {
      uint8_t packed = 0;
      for (size_t h = 0; h < 2; ++h) {
        long q = lroundf(in[r * cols + c + h] / s);
        q = q < -7 ? -7 : (q > 7 ? 7 : q);
        packed |= (uint8_t)(((uint8_t)q & 0xFu) << (4 * h));
      }
      out[r * cols / 2 + c / 2] = packed;
    }
  }
  return ORC_OK;
}

/* ---- attention over a quantized cache: every key / value element is code * scale of its key row
 *      (kind 0: int8, 1: signed 4-bit, two a byte, 2: E4M3), then orc_attention, causal
 *      (attention.cpp:45-121) ---- */
int orc_attention_quant(const float* q, const uint8_t* k, const uint8_t* v, const float* k_scale, const float* v_scale,
                        float* out, size_t m, size_t n, size_t heads, size_t kv_heads, size_t head_dim, uint64_t q_base,
                        size_t window, int kind) {
  if (m == 0 || n == 0 || heads == 0 || kv_heads == 0 || head_dim == 0 || heads % kv_heads != 0 || kind < 0 || kind > 2) {
    return ORC_INVALID_ARGUMENT;
  }
  const size_t width = kv_heads * head_dim, count = n * width;
  float* kf = (float*)malloc(count * sizeof(float));
  float* vf = (float*)malloc(count * sizeof(float));
  if (!kf || !vf) {
    free(kf), free(vf);
    return ORC_OOM;
  }
  for (size_t j = 0; j < n; ++j) {
    for (size_t d = 0; d < width; ++d) {
      const size_t i = j * width + d;
      float kc, vc;
      if (kind == 0) {
        kc = (float)(int8_t)k[i], vc = (float)(int8_t)v[i];
      } else if (kind == 1) {
        int kn = (k[i / 2] >> ((i % 2) * 4)) & 0xF, vn = (v[i / 2] >> ((i % 2) * 4)) & 0xF;
        kc = (float)((kn & 8) ? kn - 16 : kn), vc = (float)((vn & 8) ? vn - 16 : vn);
      } else {
        kc = orc_fp8_e4m3_to_float(k[i]), vc = orc_fp8_e4m3_to_float(v[i]);
      }
      kf[i] = kc * k_scale[j], vf[i] = vc * v_scale[j];
    }
  }
  const int rc = orc_attention(q, kf, vf, out, m, n, heads, kv_heads, head_dim, q_base, window, 0, 1);
  free(kf), free(vf);
  return rc;
}

/* ---- flash-decoding partials: the key range of (row, head) is cut into `split` chunks of
 *      ceil(span / split) keys; chunk s leaves pacc = sum_j exp(score_j - pmax) v_j (not
 *      normalised), pmax = its largest score, psum = sum_j exp(score_j - pmax) at index
 *      (row * heads + head) * split + s; an empty chunk leaves 0, -1e30, 0
 *      (src/backends/rocm/rocm_kernels_basic.cpp:275-440; sequential sums here).  k, v are fp32. ---- */
int orc_attention_split(const float* q, const float* k, const float* v, float* pacc, float* pmax, float* psum, size_t m,
                        size_t n, size_t heads, size_t kv_heads, size_t head_dim, uint64_t q_base, size_t window, int causal,
                        size_t split) {
  if (m == 0 || n == 0 || heads == 0 || kv_heads == 0 || head_dim == 0 || heads % kv_heads != 0 || split == 0) {
    return ORC_INVALID_ARGUMENT;
  }
  float* scores = (float*)malloc(n * sizeof(float));
  if (!scores) return ORC_OOM;
  const size_t group = heads / kv_heads;
  const float scale = 1.0f / sqrtf((float)head_dim);
  for (size_t i = 0; i < m; ++i) {
    const size_t pos = (size_t)(q_base + i);
    const size_t last = causal ? (pos >= n ? n - 1 : pos) : n - 1;
    size_t start = 0;
    if (causal) {
      start = window != 0 && pos + 1 > window ? pos + 1 - window : 0;
      if (start > last) start = last;
    }
    const size_t chunk = (last + 1 - start + split - 1) / split;
    for (size_t h = 0; h < heads; ++h) {
      const size_t kv = h / group;
      const float* q_row = q + (i * heads + h) * head_dim;
      for (size_t sidx = 0; sidx < split; ++sidx) {
        const size_t base = (i * heads + h) * split + sidx;
        const size_t cstart = start + sidx * chunk;
        if (cstart > last) {
          for (size_t e = 0; e < head_dim; ++e) pacc[base * head_dim + e] = 0.0f;
          pmax[base] = -1e30f, psum[base] = 0.0f;
          continue;
        }
        const size_t cend = cstart + chunk - 1 < last ? cstart + chunk - 1 : last;
        float top = 0.0f;
        for (size_t j = cstart; j <= cend; ++j) {
          float dot = 0.0f;
          for (size_t e = 0; e < head_dim; ++e) dot = fmaf(q_row[e], k[(j * kv_heads + kv) * head_dim + e], dot);
          scores[j] = dot * scale;
          if (j == cstart || scores[j] > top) top = scores[j];
        }
        float denom = 0.0f;
        for (size_t j = cstart; j <= cend; ++j) {
          scores[j] = expf(scores[j] - top);
          denom += scores[j];
        }
        for (size_t e = 0; e < head_dim; ++e) {
          float acc = 0.0f;
          for (size_t j = cstart; j <= cend; ++j) acc = fmaf(scores[j], v[(j * kv_heads + kv) * head_dim + e], acc);
          pacc[base * head_dim + e] = acc;
        }
        pmax[base] = top, psum[base] = denom;
      }
    }
  }
  free(scores);
  return ORC_OK;
}

/* ---- merge of the partials (rocm_kernels_basic.cpp:664-690) ---- */
int orc_attention_combine(const float* pacc, const float* pmax, const float* psum, float* out, size_t m, size_t heads,
                          size_t head_dim, size_t split) {
  if (m == 0 || heads == 0 || head_dim == 0 || split == 0) return ORC_INVALID_ARGUMENT;
  for (size_t g = 0; g < m * heads; ++g) {
    const size_t base = g * split;
    float top = -1e30f;
    for (size_t s = 0; s < split; ++s) top = fmaxf(top, pmax[base + s]);
    for (size_t e = 0; e < head_dim; ++e) {
      float num = 0.0f, den = 0.0f;
      for (size_t s = 0; s < split; ++s) {
        const float w = expf(pmax[base + s] - top);
        num = fmaf(w, pacc[(base + s) * head_dim + e], num);
        den = fmaf(w, psum[base + s], den);
      }
      out[g * head_dim + e] = num / den;
    }
  }
  return ORC_OK;
}

/* ---- fp32 -> binary16 as the "cast_f32_f16" built-in does it: the significand is cut, not rounded
 *      (toward zero), magnitudes of 2^16 and more -- and NaN -- give infinity, magnitudes below
 *      2^-24 give zero (src/backends/rocm/rocm_kernels.hpp:26-45) ---- */
uint16_t orc_float_to_fp16_cut(float value) {
  uint32_t bits;
  memcpy(&bits, &value, sizeof(bits));
  const uint32_t sign = (bits >> 16) & 0x8000u;
  const int exponent = (int)((bits >> 23) & 0xFFu) - 127;
  uint32_t mantissa = bits & 0x7FFFFFu;
  if (exponent > 15) return (uint16_t)(sign | 0x7C00u);
  if (exponent < -24) return (uint16_t)sign;
  if (exponent < -14) {
    mantissa |= 0x800000u;
    return (uint16_t)(sign | (mantissa >> (uint32_t)(-exponent - 14 + 13)));
  }
  return (uint16_t)(sign | ((uint32_t)(exponent + 15) << 10) | (mantissa >> 13));
}

void orc_cast_f32_f16(const float* in, uint16_t* out, size_t n) {
  for (size_t i = 0; i < n; ++i) out[i] = orc_float_to_fp16_cut(in[i]);
}

/* ---- fused gated-attention projection (rows x heads x [query | gate]) -> queries, gates
 *      (src/core/numerics/attention.cpp:287-309) ---- */
int orc_qgate_split(const float* fused, float* q, float* gate, size_t heads, size_t head_dim, size_t rows) {
  if (heads == 0 || head_dim == 0 || rows == 0) return ORC_INVALID_ARGUMENT;
  for (size_t r = 0; r < rows; ++r) {
    for (size_t h = 0; h < heads; ++h) {
      const float* src = fused + (r * heads + h) * 2 * head_dim;
      for (size_t e = 0; e < head_dim; ++e) {
        q[(r * heads + h) * head_dim + e] = src[e];
        gate[(r * heads + h) * head_dim + e] = src[head_dim + e];
      }
    }
  }
  return ORC_OK;
}

/* ---- o = silu(g) * u elementwise (src/core/numerics/norm.cpp:211-226; the device kernel
 *      src/backends/rocm/rocm_kernels_basic.cpp:1882-1891 is the same expression) ---- */
void orc_silu_mul(const float* g, const float* u, float* o, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    const float silu = g[i] / (1.0f + expf(-g[i]));
    o[i] = silu * u[i];
  }
}

/* ---- one Q4_K expert on one token: down(silu(gate x) * (up x))
 *      (moe_cpu.cpp:39-64) ---- */
int orc_moe_expert_forward_q4k(const float* x, const uint8_t* gate, const uint8_t* up,
                               const uint8_t* down, size_t hidden, size_t inter, float* out) {
  if (hidden == 0 || inter == 0) return ORC_INVALID_ARGUMENT;
  float* g = (float*)malloc(3 * inter * sizeof(float));
  if (!g) return ORC_OOM;
  float* u = g + inter;
  float* phi = u + inter;
  int st = orc_gemm_q4k_ref(x, gate, g, 1, inter, hidden);
  if (st == ORC_OK) st = orc_gemm_q4k_ref(x, up, u, 1, inter, hidden);
  if (st == ORC_OK) {
    for (size_t j = 0; j < inter; ++j) phi[j] = (g[j] / (1.0f + expf(-g[j]))) * u[j];
    st = orc_gemm_q4k_ref(phi, down, out, 1, hidden, inter);
  }
  free(g);
  return st;
}

/* ---- routed sum over the selected experts of one token, slots in order:
 *      acc[j] += sum_slot wts[slot] * expert(ids[slot])(x)[j]
 *      (moe_cpu.cpp:66-129 with one partial per slot, which is what its thread
 *      pool produces when it has at least top_k threads; the device kernel
 *      src/backends/rocm/rocm_kernels_moe.cpp:51-79 sums slots the same way) ---- */
int orc_moe_experts_forward_q4k(const float* x, const uint32_t* ids, const float* wts,
                                size_t top_k, const uint8_t* gate, size_t gate_stride,
                                const uint8_t* up, size_t up_stride, const uint8_t* down,
                                size_t down_stride, size_t hidden, size_t inter, float* acc) {
  float* out = (float*)malloc(hidden * sizeof(float));
  float* sum = (float*)calloc(hidden, sizeof(float));
  if (!out || !sum) {
    free(out);
    free(sum);
    return ORC_OOM;
  }
  int st = ORC_OK;
  for (size_t c = 0; c < top_k && st == ORC_OK; ++c) {
    const size_t e = ids[c];
    st = orc_moe_expert_forward_q4k(x, gate + e * gate_stride, up + e * up_stride,
                                    down + e * down_stride, hidden, inter, out);
    if (st != ORC_OK) break;
    for (size_t j = 0; j < hidden; ++j) sum[j] += wts[c] * out[j];
  }
  if (st == ORC_OK) {
    for (size_t j = 0; j < hidden; ++j) acc[j] += sum[j];
  }
  free(out);
  free(sum);
  return st;
}

/* Tokens of a batch spread over OpenMP threads; each token is the sequential
 * routine above, so results do not depend on the thread count. */
int orc_moe_batch_forward_q4k(const float* x, const uint32_t* ids, const float* wts, size_t rows,
                              size_t top_k, const uint8_t* gate, size_t gate_stride,
                              const uint8_t* up, size_t up_stride, const uint8_t* down,
                              size_t down_stride, size_t hidden, size_t inter, float* out) {
  int bad = 0;
#pragma omp parallel for schedule(dynamic)
  for (long long r = 0; r < (long long)rows; ++r) {
    memset(out + (size_t)r * hidden, 0, hidden * sizeof(float));
    const int st = orc_moe_experts_forward_q4k(
        x + (size_t)r * hidden, ids + (size_t)r * top_k, wts + (size_t)r * top_k, top_k, gate,
        gate_stride, up, up_stride, down, down_stride, hidden, inter, out + (size_t)r * hidden);
    if (st != ORC_OK) {
#pragma omp atomic write
      bad = st;
    }
  }
  return bad;
}
