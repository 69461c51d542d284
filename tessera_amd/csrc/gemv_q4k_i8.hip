// Q4_K decode GEMV over a load-time copy of the weights in "row-group" order, on the int8 matrix cores.
//
// The GGUF order (reference layout src/core/numerics/quant.hpp:11-15) keeps a row's super-blocks
// together, which is what a CPU walks; on gfx950 the decode GEMV over it is bound by vector issue
// slots (a mask per two weights and a multiply-add per weight), not by HBM.  The reference has a hook
// for a load-time re-ordering of a weight tensor (PermuteMxFp4ToWmma, src/core/numerics/quant.cpp:926-954,
// selected per launch by the `wperm` scalar); this file is that hook for Q4_K on this part:
//
//   * rows are cut into groups of R consecutive rows, one workgroup each (R is the caller's choice up to
//     64; 32, two full tiles, is the default);
//   * a group stores, per 256-wide block of K, first the quants of its 16-row tiles and then the
//     16-byte headers of its rows: R * 144 bytes, the GGUF byte count, nothing padded;
//   * a tile's quants are two pieces ("pair sets" c = 0, 1) of rows x 64 bytes: lane (n, g) of a
//     wavefront (row n of the tile, g = 0..3) owns 16 bytes per piece whose low nibbles are the 16
//     weights [16 (g % 2), +16) of sub-block 2c + g / 2 and whose high nibbles are the same weights of
//     sub-block 2c + 4 + g / 2, stored minus eight as 4-bit two's complement.  One v_and_b32 per
//     register therefore yields the B operand of v_mfma_i32_16x16x64_i8: the low nibbles as they are,
//     the high ones as signed bytes 16 (q - 8);
//   * a header is d, dmin (as in GGUF) and the sixteen 6-bit scales and mins re-packed so that the
//     lanes of even and of odd sub-blocks each find theirs in one register.
//
// The activations of a block become four signed 8-bit limbs under the block's power of two (30 bits
// below the block's largest magnitude: a one-hot or power-of-two row is exact, any row keeps more
// than the 24 bits of its fp32 values near the maximum), laid out as the A operand: matrix rows
// 0..3 carry the limbs for the even sub-block of a 64-wide K pair, 4..7 for the odd one, and rows
// 8..15 the same for a second tile whose product is accumulated into the same registers, so that
// after two matrix instructions every lane holds, for its own weight row and sub-block parity, the
// four limb dot products -- which it folds with its own 6-bit scale by integer multiply-adds.
// The sums are exact integers; d, dmin and the power of two enter once per block in fp32:
//   y_row += d * (T * 2^-sh + 8 * sum_{high} sc_s S_s) - dmin * sum_s mn_s S_s,   S_s = sum of x over sub-block s.
// A one-hot activation returns RN(d * sc * q - dmin * mn), the reference's dequantized weight
// (src/core/numerics/quant.cpp:656-675), bit for bit.

#include "i8_limbs.hpp"
#include "qmm_device.hpp"
#include "qmm_kernels.hpp"

namespace qmm {
namespace {

using namespace i8limbs;

// ---- the twelve scale bytes ------------------------------------------------------------------
// GGUF (src/core/numerics/quant.cpp:58-70): j < 4: sc = b[j] & 63, mn = b[j+4] & 63; j >= 4:
// sc = (b[j+4] & 15) | (b[j-4] >> 6) << 4, mn = (b[j+4] >> 4) | (b[j] >> 6) << 4.
__device__ __forceinline__ void gguf_scales(const uint8_t (&b)[12], uint32_t (&sc)[8], uint32_t (&mn)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    sc[j] = b[j] & 63u;
    mn[j] = b[j + 4] & 63u;
    sc[j + 4] = (b[j + 8] & 15u) | ((b[j] >> 6) << 4);
    mn[j + 4] = (b[j + 8] >> 4) | ((b[j + 4] >> 6) << 4);
  }
}
// Row-group header words: y = scales of the even sub-blocks, z = of the odd ones, w = mins of the even
// ones, one per byte; the mins of the odd sub-blocks ride in the top two bits of those twelve bytes.
__device__ __forceinline__ void pack_header(const uint32_t (&sc)[8], const uint32_t (&mn)[8], uint32_t& y,
                                            uint32_t& z, uint32_t& w) {
  y = z = w = 0u;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t mo = mn[2 * i + 1];
    y |= (sc[2 * i] | ((mo & 3u) << 6)) << (8 * i);
    z |= (sc[2 * i + 1] | (((mo >> 2) & 3u) << 6)) << (8 * i);
    w |= (mn[2 * i] | (((mo >> 4) & 3u) << 6)) << (8 * i);
  }
}
__device__ __forceinline__ uint32_t odd_mins(uint32_t y, uint32_t z, uint32_t w) {
  return ((y >> 6) & 0x03030303u) | ((z >> 4) & 0x0C0C0C0Cu) | ((w >> 2) & 0x30303030u);
}

// Where row `rr` of a group of `rows` rows keeps block-local things: byte offset of its piece
// (c, g) and of its header inside the block's rows * 144 bytes.
__device__ __forceinline__ uint32_t piece_offset(uint32_t rows, uint32_t rr, uint32_t c, uint32_t g) {
  const uint32_t tile = rr >> 4, nn = rr & 15u;
  const uint32_t rt = rows - tile * 16u < 16u ? rows - tile * 16u : 16u;
  return tile * 2048u + c * rt * 64u + (g * rt + nn) * 16u;
}
__device__ __forceinline__ uint32_t header_offset(uint32_t rows, uint32_t rr) { return rows * 128u + rr * 16u; }

// One thread per (row, block): GGUF -> row groups, or back.
__global__ __launch_bounds__(256) void q4k_rowgroup_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out,
                                                          uint32_t n, uint32_t nblk, uint32_t R, bool inverse) {
  const uint64_t idx = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
  if (idx >= static_cast<uint64_t>(n) * nblk) return;
  const uint32_t r = static_cast<uint32_t>(idx / nblk), b = static_cast<uint32_t>(idx - static_cast<uint64_t>(r) * nblk);
  const uint32_t row0 = r / R * R, rows = n - row0 < R ? n - row0 : R, rr = r - row0;
  const size_t gguf = (static_cast<size_t>(r) * nblk + b) * 144u;
  const size_t region = static_cast<size_t>(row0) * nblk * 144u + static_cast<size_t>(b) * rows * 144u;
  if (!inverse) {
    const uint8_t* blk = in + gguf;
    uint8_t* reg = out + region;
    uint4 qs[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) qs[i] = load_u4(blk + 16 + 16 * i);
    const uint4 h = load_u4(blk);
    const uint32_t hw[3] = {h.y, h.z, h.w};
    uint8_t sb[12];
#pragma unroll
    for (int i = 0; i < 12; ++i) sb[i] = static_cast<uint8_t>(hw[i >> 2] >> (8 * (i & 3)));
    uint32_t sc[8], mn[8], y, z, w;
    gguf_scales(sb, sc, mn);
    pack_header(sc, mn, y, z, w);
    *reinterpret_cast<uint4*>(reg + header_offset(rows, rr)) = make_uint4(h.x, y, z, w);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        // 16 bytes of GGUF group c (sub-blocks 2c, 2c+1) and of group c+2, weights [16 (g%2), +16)
        const uint4 a = qs[c * 2 + (g & 1)], hi = qs[(c + 2) * 2 + (g & 1)];
        const uint32_t av[4] = {a.x, a.y, a.z, a.w}, hv[4] = {hi.x, hi.y, hi.z, hi.w};
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t lo = (g >> 1) ? (av[i] >> 4) & 0x0F0F0F0Fu : av[i] & 0x0F0F0F0Fu;
          const uint32_t up = ((g >> 1) ? (hv[i] >> 4) & 0x0F0F0F0Fu : hv[i] & 0x0F0F0F0Fu) ^ 0x08080808u;
          o[i] = lo | (up << 4);
        }
        *reinterpret_cast<uint4*>(reg + piece_offset(rows, rr, c, g)) = make_uint4(o[0], o[1], o[2], o[3]);
      }
    }
  } else {
    const uint8_t* reg = in + region;
    uint8_t* blk = out + gguf;
    const uint4 h = load_u4(reg + header_offset(rows, rr));
    const uint32_t dm = odd_mins(h.y, h.z, h.w);
    uint32_t sc[8], mn[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      sc[2 * i] = (h.y >> (8 * i)) & 63u;
      sc[2 * i + 1] = (h.z >> (8 * i)) & 63u;
      mn[2 * i] = (h.w >> (8 * i)) & 63u;
      mn[2 * i + 1] = (dm >> (8 * i)) & 63u;
    }
    // the reference's packing (src/core/numerics/quant.cpp:712-720)
    uint32_t sw[3] = {0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      sw[0] |= (sc[j] | ((sc[j + 4] >> 4) << 6)) << (8 * j);
      sw[1] |= (mn[j] | ((mn[j + 4] >> 4) << 6)) << (8 * j);
      sw[2] |= ((sc[j + 4] & 15u) | ((mn[j + 4] & 15u) << 4)) << (8 * j);
    }
    *reinterpret_cast<uint4*>(blk) = make_uint4(h.x, sw[0], sw[1], sw[2]);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const uint4 p0 = load_u4(reg + piece_offset(rows, rr, c, half));       // low nibbles of the GGUF bytes
        const uint4 p1 = load_u4(reg + piece_offset(rows, rr, c, 2 + half));   // high nibbles
        const uint32_t a[4] = {p0.x, p0.y, p0.z, p0.w}, bb[4] = {p1.x, p1.y, p1.z, p1.w};
        uint32_t lo[4], up[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          lo[i] = (a[i] & 0x0F0F0F0Fu) | ((bb[i] & 0x0F0F0F0Fu) << 4);
          up[i] = (((a[i] >> 4) & 0x0F0F0F0Fu) ^ 0x08080808u) | ((((bb[i] >> 4) & 0x0F0F0F0Fu) ^ 0x08080808u) << 4);
        }
        *reinterpret_cast<uint4*>(blk + 16 + (c * 2 + half) * 16) = make_uint4(lo[0], lo[1], lo[2], lo[3]);
        *reinterpret_cast<uint4*>(blk + 16 + ((c + 2) * 2 + half) * 16) = make_uint4(up[0], up[1], up[2], up[3]);
      }
    }
  }
}

// Quants of one tile pair x one block for a lane ([tile][pair set]) and the header of its row.
struct Unit {
  uint4 q[4];
  uint4 h;
};

// One unit against the block's limbs.  The lane ends up with the dot product of row
// (tile lane / 32, lane % 16) over the four sub-blocks of its parity (lane / 16 % 2).
__device__ __forceinline__ float unit_dot(const Unit& f, const uint8_t* a0, const uint8_t* a1, const uint8_t* slot,
                                          bool odd) {
  const uint32_t y = f.h.y, z = f.h.z, w = f.h.w;
  const uint32_t scw = odd ? z : y;
  const uint32_t mnw = odd ? odd_mins(y, z, w) : (w & 0x3F3F3F3Fu);
  int sc[4];
  float mn[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    sc[j] = (scw >> (8 * j)) & 63u;
    mn[j] = static_cast<float>((mnw >> (8 * j)) & 0xFFu);
  }
  const float4 S4 = *reinterpret_cast<const float4*>(slot + 1024u + (odd ? 16u : 0u));
  const float S[4] = {S4.x, S4.y, S4.z, S4.w};
  int acc[4] = {0, 0, 0, 0};
  const int4v_t zero = {0, 0, 0, 0};
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const uint4 v0 = f.q[c], v1 = f.q[2 + c];
    int4v_t B0, B1, H0, H1;
    B0[0] = v0.x & 0x0F0F0F0Fu, B0[1] = v0.y & 0x0F0F0F0Fu, B0[2] = v0.z & 0x0F0F0F0Fu, B0[3] = v0.w & 0x0F0F0F0Fu;
    B1[0] = v1.x & 0x0F0F0F0Fu, B1[1] = v1.y & 0x0F0F0F0Fu, B1[2] = v1.z & 0x0F0F0F0Fu, B1[3] = v1.w & 0x0F0F0F0Fu;
    H0[0] = v0.x & 0xF0F0F0F0u, H0[1] = v0.y & 0xF0F0F0F0u, H0[2] = v0.z & 0xF0F0F0F0u, H0[3] = v0.w & 0xF0F0F0F0u;
    H1[0] = v1.x & 0xF0F0F0F0u, H1[1] = v1.y & 0xF0F0F0F0u, H1[2] = v1.z & 0xF0F0F0F0u, H1[3] = v1.w & 0xF0F0F0F0u;
    // K pair c from the low nibbles (scale times 16 so that both kinds carry the same factor) ...
    const int4v_t A0 = *reinterpret_cast<const int4v_t*>(a0 + c * 256);
    const int4v_t A1 = *reinterpret_cast<const int4v_t*>(a1 + c * 256);
    int4v_t D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A0, B0, zero, 0, 0, 0);
    D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, B1, D, 0, 0, 0);
    const int sl = sc[c] << 4;
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      acc[m] = mad24(D[m], sl, acc[m]);
      asm("" : "+v"(acc[m]));   // one multiply-add per step, not a multiply and a three-way add later
    }
    // ... and K pair c + 2 from the high ones, which are 16 (q - 8)
    const int4v_t A2 = *reinterpret_cast<const int4v_t*>(a0 + (c + 2) * 256);
    const int4v_t A3 = *reinterpret_cast<const int4v_t*>(a1 + (c + 2) * 256);
    int4v_t E = __builtin_amdgcn_mfma_i32_16x16x64_i8(A2, H0, zero, 0, 0, 0);
    E = __builtin_amdgcn_mfma_i32_16x16x64_i8(A3, H1, E, 0, 0, 0);
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      acc[m] = mad24(E[m], sc[c + 2], acc[m]);
      asm("" : "+v"(acc[m]));
    }
  }
  float accm = mn[0] * S[0];
  accm = fmaf(mn[1], S[1], accm), accm = fmaf(mn[2], S[2], accm), accm = fmaf(mn[3], S[3], accm);
  const float acc8 = fmaf(static_cast<float>(sc[3]), S[3], static_cast<float>(sc[2]) * S[2]);
  float T = fmaf(static_cast<float>(acc[1]), 256.0f, static_cast<float>(acc[0]));
  T = fmaf(static_cast<float>(acc[2]), 65536.0f, T);
  T = fmaf(static_cast<float>(acc[3]), 16777216.0f, T);
  T = __builtin_ldexpf(T, -4 - reinterpret_cast<const int*>(slot + 1056u)[0]);
  const float d = half_bits_to_float(f.h.x & 0xFFFFu);
  const float dmin = half_bits_to_float(f.h.x >> 16);
  return fmaf(d, fmaf(8.0f, acc8, T), -(dmin * accm));
}

// Workgroup i owns rows [i*R, i*R+R) over all of K as U tile pairs (the last tile may be short, the
// last pair single); wavefront w takes blocks w, w+W, ...; PD blocks of quants in flight.  A
// wavefront converts the activations of its own blocks, one block ahead, into two private LDS
// slots, so there is no barrier before the final sum over the wavefronts.
template <int U, int W, int PD>
__global__ __launch_bounds__(W * 64) void q4k_i8_gemv_kernel(const uint8_t* __restrict__ wq,
                                                             const float* __restrict__ x, float* __restrict__ c,
                                                             uint32_t n, uint32_t nblk, uint32_t R) {
  // the first kilobyte stays zero: the A operand of the lanes whose matrix rows carry nothing
  __shared__ __attribute__((aligned(16))) uint8_t lds[1024u + W * 2u * kSlot];
  __shared__ float part[W * U * 32];
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t row0 = blockIdx.x * R;
  const uint32_t rows = n - row0 < R ? n - row0 : R;
  const uint32_t T = (rows + 15u) / 16u;
  const uint32_t nmine = wave < nblk ? (nblk - wave + W - 1u) / W : 0u;
  const uint8_t* wbase = wq + static_cast<size_t>(row0) * nblk * 144u;
  const uint32_t bstride = rows * 144u;
  const uint32_t ln = lane & 15u, g = lane >> 4, lt = lane >> 5;
  // Per-lane offsets of its pieces inside a block's bytes.  A tile past the last one repeats the
  // last, a row past a short tile's last repeats that row: those lanes' sums are never stored.
  uint32_t qoff[U][4], hoff[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      uint32_t tile = 2u * u + t;
      tile = tile < T ? tile : T - 1u;
      const uint32_t rt = rows - tile * 16u < 16u ? rows - tile * 16u : 16u;
      const uint32_t nn = ln < rt ? ln : rt - 1u;
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) qoff[u][t * 2 + cc] = tile * 2048u + cc * rt * 64u + (g * rt + nn) * 16u;
      if (t == static_cast<int>(lt)) hoff[u] = rows * 128u + (tile * 16u + nn) * 16u;
    }
  }
  auto load_unit = [&](uint32_t j, int u, Unit& f) {
    const uint8_t* p = wbase + static_cast<size_t>(wave + j * W) * bstride;
#pragma unroll
    for (int q = 0; q < 4; ++q) f.q[q] = load_u4(p + qoff[u][q]);
    f.h = load_u4(p + hoff[u]);
  };
  auto x_load = [&](uint32_t j) {
    const uint32_t b = wave + (j < nmine ? j : 0u) * W;
    return *reinterpret_cast<const float4*>(x + (b < nblk ? b : 0u) * 256u + lane * 4u);
  };
  // activations first: loads return in order, and the conversion must not wait behind the weights
  float4 xr = x_load(0);
  Unit buf[PD][U];
#pragma unroll
  for (int p = 0; p < PD; ++p) {
    if (static_cast<uint32_t>(p) < nmine) {
#pragma unroll
      for (int u = 0; u < U; ++u) load_unit(p, u, buf[p][u]);
    }
  }
  // every wavefront zeroes the shared kilobyte itself (same values), so it waits for nobody
  reinterpret_cast<uint4*>(lds)[lane] = make_uint4(0u, 0u, 0u, 0u);
  uint8_t* myslots = lds + 1024u + wave * 2u * kSlot;
  float4 xn = x_load(1);
  if (nmine > 0u) convert_block(xr, lane, myslots);
  xr = xn;
  const bool odd = (g & 1u) != 0u;
  // matrix rows 0..3 / 4..7 of tile 0 and 8..11 / 12..15 of tile 1 carry limbs for the K halves
  // their lane group covers; every other lane reads zeros
  const bool live0 = (ln < 4u && g < 2u) || (ln >= 4u && ln < 8u && g >= 2u);
  const bool live1 = (ln >= 8u && ln < 12u && g < 2u) || (ln >= 12u && g >= 2u);
  const uint32_t aoff = ((ln >> 2) & 1u) * 128u + (g & 1u) * 64u + (ln & 3u) * 16u;
  float row[U];
#pragma unroll
  for (int u = 0; u < U; ++u) row[u] = 0.0f;
  for (uint32_t j0 = 0; j0 < nmine; j0 += PD) {
#pragma unroll
    for (int p = 0; p < PD; ++p) {
      const uint32_t j = j0 + p;
      if (j < nmine) {
        const uint8_t* slot = myslots + (j & 1u) * kSlot;
        const uint8_t* a0 = live0 ? slot + aoff : lds;
        const uint8_t* a1 = live1 ? slot + aoff : lds;
#pragma unroll
        for (int u = 0; u < U; ++u) {
          row[u] += unit_dot(buf[p][u], a0, a1, slot, odd);
          if (j + PD < nmine) load_unit(j + PD, u, buf[p][u]);
        }
        if (j + 1u < nmine) {
          xn = x_load(j + 2u);
          convert_block(xr, lane, myslots + ((j + 1u) & 1u) * kSlot);
          xr = xn;
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    // the two parities of a row sit 16 lanes apart
    const float other = bit_cast<float>(__builtin_amdgcn_ds_swizzle(bit_cast<int>(row[u]), 0x401F));
    const float v = row[u] + other;
    if (!odd) part[(wave * U + u) * 32u + lt * 16u + ln] = v;
  }
  __syncthreads();
  for (uint32_t o = threadIdx.x; o < U * 32u; o += W * 64u) {
    float s = 0.0f;
    for (int w = 0; w < W; ++w) s += part[w * U * 32u + o];   // wavefront order: deterministic
    if (o < rows) c[row0 + o] = s;
  }
}

template <int U, int W, int PD>
hipError_t launch_uwp(const uint8_t* wq, const float* x, float* c, uint32_t n, uint32_t nblk, uint32_t R,
                      hipStream_t stream) {
  hipLaunchKernelGGL((q4k_i8_gemv_kernel<U, W, PD>), dim3((n + R - 1u) / R), dim3(W * 64), 0, stream, wq, x, c, n,
                     nblk, R);
  return hipGetLastError();
}

template <int U>
hipError_t launch_u(const uint8_t* wq, const float* x, float* c, uint32_t n, uint32_t nblk, uint32_t R,
                    hipStream_t stream) {
  // Wavefronts per workgroup: a count that divides the blocks of a row evenly where there is one, as
  // many as the register budget of the unit count allows otherwise.
  constexpr int kPD = U == 1 ? 2 : 1;
  if (nblk % 16u == 0u) return launch_uwp<U, 16, kPD>(wq, x, c, n, nblk, R, stream);
  if (nblk % 10u == 0u) return launch_uwp<U, 10, kPD>(wq, x, c, n, nblk, R, stream);
  if (nblk % 8u == 0u || nblk < 10u) return launch_uwp<U, 8, kPD>(wq, x, c, n, nblk, R, stream);
  return launch_uwp<U, 16, kPD>(wq, x, c, n, nblk, R, stream);
}

}  // namespace

uint32_t q4k_rowgroup_default_rows(uint64_t n) {
  // Every CU the same number of rows where the matrix is tall enough for that to matter; two full
  // tiles otherwise.
  (void)n;
  return 32u;   // two full tiles: one unit per block, the least vector work per weight
}

bool q4k_rowgroup_supported(uint64_t n, uint64_t k, uint64_t rows_per_group) {
  return rows_per_group >= 1 && rows_per_group <= kQ4KRowGroupMaxRows && k % 256 == 0 && k / 256 <= 0xFFFFu &&
         n <= 0x7FFFFFFFull && n * (k / 256) <= 0xFFFFFFFFull * 64ull;
}

hipError_t launch_q4k_rowgroup(const uint8_t* in, uint8_t* out, uint32_t n, uint32_t k, uint32_t rows_per_group,
                               bool inverse, hipStream_t stream) {
  const uint32_t nblk = k / 256u;
  const uint64_t total = static_cast<uint64_t>(n) * nblk;
  hipLaunchKernelGGL(q4k_rowgroup_kernel, dim3(static_cast<uint32_t>((total + 255u) / 256u)), dim3(256), 0, stream, in,
                     out, n, nblk, rows_per_group, inverse);
  return hipGetLastError();
}

hipError_t launch_q4k_i8_gemv(const float* a, const uint8_t* w, float* c, uint32_t n, uint32_t k,
                              uint32_t rows_per_group, hipStream_t stream) {
  const uint32_t nblk = k / 256u, R = rows_per_group;
  const uint32_t tiles = (R + 15u) / 16u;
  switch ((tiles + 1u) / 2u) {
    case 1: return launch_u<1>(w, a, c, n, nblk, R, stream);
    case 2: return launch_u<2>(w, a, c, n, nblk, R, stream);
    default: return hipErrorInvalidValue;
  }
}

}  // namespace qmm
