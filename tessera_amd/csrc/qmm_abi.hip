// C ABI of the kernel library: device bring-up, the built-in kernel table, launch
// validation and per-id dispatch.  See include/tessera_qmm.h for the contract of each
// entry point and the reference interface it stands behind.

#include "../../include/tessera_qmm.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "qmm_kernels.hpp"

namespace {

struct LaunchCtx {
  void* const* buf;
  const size_t* bytes;  // may be null: sizes unknown, skip size checks
  size_t nbuf;
  const uint64_t* sc;
  size_t nsc;
  hipStream_t stream;
  bool no_alloc = false;  // qmm_launch_static: scratch comes from the static device array only

  template <class T>
  T* ptr(size_t i) const { return static_cast<T*>(buf[i]); }
  // Buffer i holds at least `need` bytes (or sizes were not given).
  bool fits(size_t i, unsigned __int128 need) const {
    return bytes == nullptr || static_cast<unsigned __int128>(bytes[i]) >= need;
  }
};

using qmm_fn = qmm_status (*)(const LaunchCtx&);

thread_local std::string g_last_error;
thread_local int t_device = -1;  // device this thread last made current
std::mutex g_init_mutex;
int g_device = -1;
std::string g_device_name;

qmm_status map_hip(hipError_t e) {
  if (e == hipSuccess) return QMM_OK;
  g_last_error = hipGetErrorString(e);
  // Same mapping as the reference backend (src/backends/rocm/rocm_backend.cpp:38-45).
  if (e == hipErrorOutOfMemory) return QMM_OUT_OF_MEMORY;
  if (e == hipErrorInvalidValue) return QMM_INVALID_ARGUMENT;
  return QMM_DEVICE_ERROR;
}

qmm_status bad(const std::string& why) {
  g_last_error = why;
  return QMM_INVALID_ARGUMENT;
}

using u128 = unsigned __int128;
constexpr uint64_t kMaxDim = 0x7FFFFFFFull;  // kernels index rows/cols with 32 bits

bool counts(const LaunchCtx& c, size_t nbuf, size_t nsc) { return c.nbuf == nbuf && c.nsc == nsc; }

bool dims_ok(uint64_t m, uint64_t n, uint64_t k) {
  return m != 0 && n != 0 && k != 0 && m <= kMaxDim && n <= kMaxDim && k <= kMaxDim;
}

u128 q4k_bytes(uint64_t n, uint64_t k) { return static_cast<u128>(n) * (k / 256) * 144; }
u128 mxfp4_bytes(uint64_t n, uint64_t k) { return static_cast<u128>(n) * k / 2 + static_cast<u128>(n) * k / 32; }

// ---- Q4_K --------------------------------------------------------------------
// Regime choice inside the Q4_K ids: the caller names an id by the reference's
// regime table (src/models/qwen3_5/project.cpp:233-366); every Q4_K GEMM id has the
// same buffers and m, n, k scalars, so each id accepts every m and picks the gfx950
// kernel that fits it.
// Device scratch owned by the library (the fp16 copy of the activations that the Q4_K MFMA
// GEMM reads).  Grown on demand; a block that has been handed to a launch is never freed before
// the process ends (a recorded graph or another thread's launch may still point at it), so growth
// retires the old block instead.  Growing allocates, which a stream under capture cannot do: such
// a launch is refused.  Launches that use the block are ordered by the caller's stream.
void* g_workspace = nullptr;
size_t g_workspace_bytes = 0;
std::vector<void*> g_retired_workspaces;
// A workspace the caller owns (qmm_set_workspace): while one is set the library neither grows nor
// frees anything in qmm_launch; a launch that needs more than it holds is refused.
void* g_user_workspace = nullptr;
size_t g_user_workspace_bytes = 0;
// Scratch of the decode-sized kernels (the few-row Q4_K path's activation operand): allocated
// once by qmm_init and never moved or freed, so a decode step recorded into a HIP graph keeps
// pointing at live memory whatever the prefill-sized workspace above does later.
constexpr size_t kDecodeScratchBytes = size_t{16} << 20;
void* g_decode_scratch = nullptr;
std::mutex g_workspace_mutex;

// Scratch of qmm_launch_static, the entry point that allocates nothing: a device array that is
// part of the code object, so it exists on every device the library is loaded on from load time
// to process end.  In host code the array's name is only a handle for hipGetSymbolAddress;
// g_static_scratch[device] holds the device address (resolved by qmm_init with that device
// current) and is what every launch uses.
constexpr size_t kStaticScratchBytes = QMM_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
void* g_static_scratch[kMaxDevices] = {};

qmm_status workspace(const LaunchCtx& c, size_t bytes, void** out) {
  if (c.no_alloc) {
    if (bytes > kStaticScratchBytes) {
      g_last_error = "qmm_launch_static: this launch needs " + std::to_string(bytes) +
                     " bytes of scratch, the static scratch holds " + std::to_string(kStaticScratchBytes);
      return QMM_INVALID_ARGUMENT;
    }
    *out = g_static_scratch[g_device];
    return QMM_OK;
  }
  std::lock_guard<std::mutex> lock(g_workspace_mutex);
  if (g_user_workspace != nullptr) {
    if (bytes > g_user_workspace_bytes) {
      g_last_error = "qmm_launch: this launch needs " + std::to_string(bytes) + " bytes of workspace, the one set with "
                     "qmm_set_workspace holds " + std::to_string(g_user_workspace_bytes);
      return QMM_INVALID_ARGUMENT;
    }
    *out = g_user_workspace;
    return QMM_OK;
  }
  if (bytes > g_workspace_bytes) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(c.stream, &capturing) != hipSuccess) (void)hipGetLastError();
    if (capturing != hipStreamCaptureStatusNone) {
      g_last_error = "qmm_launch: this launch needs " + std::to_string(bytes) + " bytes of workspace and the library's holds " +
                     std::to_string(g_workspace_bytes) + "; it cannot grow while the stream is being captured (hand one over "
                     "with qmm_set_workspace, or make one eager call of this size first)";
      return QMM_INVALID_ARGUMENT;
    }
    // at least double, so that the retired blocks together stay below the live one
    size_t want = (bytes + (size_t{1} << 24) - 1) & ~((size_t{1} << 24) - 1);
    if (want < 2 * g_workspace_bytes) want = 2 * g_workspace_bytes;
    void* fresh = nullptr;
    const hipError_t e = hipMalloc(&fresh, want);
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return map_hip(e);
    }
    if (g_workspace != nullptr) g_retired_workspaces.push_back(g_workspace);
    g_workspace = fresh;
    g_workspace_bytes = want;
  }
  *out = g_workspace;
  return QMM_OK;
}

// The fixed-address scratch of the decode-sized kernels: qmm_init's allocation, or the first
// kDecodeScratchBytes of the static array for qmm_launch_static.
void* decode_scratch(const LaunchCtx& c) {
  static_assert(kDecodeScratchBytes <= kStaticScratchBytes, "the static scratch holds the decode scratch");
  return c.no_alloc ? g_static_scratch[g_device] : g_decode_scratch;
}

// Q4_K regimes by activation rows.  One row and small matrices: the VALU GEMV.  2..16 rows of a
// matrix with at least kQ4KFewRowsMinWeights weights: the exact few-row MFMA kernels (weights read
// once).  The tiled fp16 MFMA GEMM, whose operands are rounded to fp16 as in the reference's
// tensor-core tile: "gemm_q4k_wmma" from kQ4KGemmMinRows rows, the other ids from
// g_q4k_tensor_rows rows -- 64 by default, where the reference's own regime table switches to its
// fp16 tile (kGemmWmmaMinRows, src/core/decode_internal.hpp:1428; src/models/qwen3_5/project.cpp:307), so that below it results keep the fp32
// contract of the reference's tiled kernel; more rows than 16 below that run sixteen at a time
// through the exact kernels.  qmm_set_q4k_tensor_rows lowers it (at least kQ4KGemmMinRows).
constexpr uint64_t kQ4KGemmMinRows = 17;
constexpr uint64_t kQ4KTensorRowsDefault = 64;
std::atomic<uint64_t> g_q4k_tensor_rows{kQ4KTensorRowsDefault};
constexpr uint64_t kMxfp4GemmMinRows = 17;   // below: the VALU GEMV passes, exact fp32 order
constexpr uint64_t kQ4KFewRowsMinWeights = uint64_t{16} << 20;
constexpr uint64_t kQ4KRows16MinRows = 3;      // from here the 16x16x32 kernel, below the 4x4x4 one
constexpr uint64_t kQ4KFewRowsMaxK = 262144;   // its activation operand must fit the decode scratch
constexpr uint64_t kQ4KRowsI8MaxK = 5120;      // up to here the int8 one-pass kernel leads for two rows

qmm_status q4k_matmul(const LaunchCtx& ctx, const float* a, const uint8_t* w, float* c, uint64_t m, uint64_t n,
                      uint64_t k, uint64_t f16_from) {
  const hipStream_t s = ctx.stream;
  if (m >= f16_from && qmm::gemm_q4k_supported(m, k)) {
    void* ws = nullptr;
    const qmm_status st = workspace(ctx, qmm::gemm_q4k_workspace_bytes(m, k), &ws);
    if (st != QMM_OK) return st;
    return map_hip(qmm::launch_q4k_gemm(a, w, c, ws, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                        static_cast<uint32_t>(k), s));
  }
  if (m > 16 && (n * k >= kQ4KFewRowsMinWeights || qmm::gemv_q4k_rows16_supported(16, n, k))) {
    // exact, sixteen rows at a time (each chunk takes the regime of its own row count)
    for (uint64_t r = 0; r < m; r += 16) {
      const qmm_status st = q4k_matmul(ctx, a + r * k, w, c + r * n, m - r < 16 ? m - r : 16, n, k, f16_from);
      if (st != QMM_OK) return st;
    }
    return QMM_OK;
  }
  // Two rows against weight rows of up to 5120: one pass on the int8 matrix cores with the activations
  // as 8-bit limbs, whole K per workgroup, nothing left for a second launch to add up.  Measured
  // against the kernels below: 17408 x 5120 14.6..16.6 against 17.7..18.2 us, 4096 x 4096 6.6 against
  // 8.1, 32768 x 1024 7.8 against 11.7; longer rows go the other way (8192 x 8192 15.6 against 14.2),
  // and three and four rows are level with the 16x16x32 kernel (17.3 / 17.8 against 17.7 / 18.4 us in
  // one harness, 19.5 against 18.9 in another), so they stay there.
  if (m == 2 && k <= kQ4KRowsI8MaxK && n * k >= kQ4KFewRowsMinWeights &&
      qmm::gemv_kquant_rows_supported(m, n, k)) {
    return map_hip(qmm::launch_q4k_rows_i8(a, w, c, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                           static_cast<uint32_t>(k), s));
  }
  // 3..16 rows of a large matrix: one pass over the weights on the 16x16x32 MFMA.
  // (two rows as well when the weight rows are long: 5120 x 17408 20.5 against 24.8 us on the
  // resident kernel, 4096 x 14336 15.3 against 18.5; at 8192 and below the resident kernel leads)
  // From five rows on it leads at any size (1024 x 1024, 8 rows: 5.1 against 14.5 us on the
  // multiply-add passes; four rows are level with them below 16 M weights).
  if ((m >= kQ4KRows16MinRows || (m == 2 && k > 8192)) && m <= 16 && (n * k >= kQ4KFewRowsMinWeights || m >= 5) &&
      qmm::gemv_q4k_rows16_supported(m, n, k) &&
      qmm::gemv_q4k_rows16_workspace_bytes(m, n, k) <= kDecodeScratchBytes) {
    void* ws = decode_scratch(ctx);
    if (ws == nullptr) {
      g_last_error = "Q4_K: decode scratch missing";
      return QMM_DEVICE_ERROR;
    }
    return map_hip(qmm::launch_q4k_rows16(a, w, c, ws, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                          static_cast<uint32_t>(k), s));
  }
  if (m >= 2 && m <= 16 && n * k >= kQ4KFewRowsMinWeights && k <= kQ4KFewRowsMaxK &&
      qmm::gemv_q4k_mfma_supported(1, n, k)) {
    void* ws = decode_scratch(ctx);   // fixed address: a recorded decode step stays valid
    if (ws == nullptr || qmm::gemv_q4k_mfma_workspace_bytes(8, k) > kDecodeScratchBytes) {
      g_last_error = "Q4_K: decode scratch missing or too small for this k";
      return QMM_DEVICE_ERROR;
    }
    for (uint64_t r = 0; r < m; r += 8) {
      const uint64_t rows = m - r < 8 ? m - r : 8;
      const hipError_t e = qmm::launch_q4k_gemv_mfma(a + r * k, w, c + r * n, ws, static_cast<uint32_t>(rows),
                                                     static_cast<uint32_t>(n), static_cast<uint32_t>(k), s);
      if (e != hipSuccess) return map_hip(e);
    }
    return QMM_OK;
  }
  return map_hip(qmm::launch_q4k_gemv(a, w, c, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                      static_cast<uint32_t>(k), s));
}
qmm_status q4k_matmul(const LaunchCtx& ctx, const float* a, const uint8_t* w, float* c, uint64_t m, uint64_t n,
                      uint64_t k) {
  return q4k_matmul(ctx, a, w, c, m, n, k, g_q4k_tensor_rows.load(std::memory_order_relaxed));
}

// Weights handed over as the load-time row-group copy (`layout` = its rows per group; 0 = GGUF order):
// one activation row runs on the int8 matrix kernel that the copy was made for; every other regime
// gets the GGUF order back in the workspace first (behind what that regime itself keeps there) and
// then runs as usual -- correct for every id, at the price of one more pass over the weights.
bool q4k_layout_ok(uint64_t n, uint64_t k, uint64_t layout) {
  return layout == 0 || qmm::q4k_rowgroup_supported(n, k, layout);
}
size_t q4k_regime_workspace(uint64_t m, uint64_t k, uint64_t f16_from) {
  return m >= f16_from && qmm::gemm_q4k_supported(m, k) ? (qmm::gemm_q4k_workspace_bytes(m, k) + 255) & ~size_t{255} : 0;
}
qmm_status q4k_matmul_layout(const LaunchCtx& ctx, const float* a, const uint8_t* w, float* c, uint64_t m, uint64_t n,
                             uint64_t k, uint64_t f16_from, uint64_t layout) {
  if (layout == 0) return q4k_matmul(ctx, a, w, c, m, n, k, f16_from);
  if (m == 1) {
    return map_hip(qmm::launch_q4k_i8_gemv(a, w, c, static_cast<uint32_t>(n), static_cast<uint32_t>(k),
                                           static_cast<uint32_t>(layout), ctx.stream));
  }
  const size_t front = q4k_regime_workspace(m, k, f16_from);
  void* ws = nullptr;
  qmm_status st = workspace(ctx, front + static_cast<size_t>(q4k_bytes(n, k)), &ws);
  if (st != QMM_OK) return st;
  uint8_t* gguf = static_cast<uint8_t*>(ws) + front;
  st = map_hip(qmm::launch_q4k_rowgroup(w, gguf, static_cast<uint32_t>(n), static_cast<uint32_t>(k),
                                        static_cast<uint32_t>(layout), true, ctx.stream));
  if (st != QMM_OK) return st;
  return q4k_matmul(ctx, a, gguf, c, m, n, k, f16_from);
}

// "gemm_q4k", "gemm_q4k_row", "gemm_q4k_batched", "gemm_q4k_wmma": buffers A, W, C;
// scalars m, n, k (include/tessera/backend.hpp:153-161,207-209,397-415;
// src/core/decode_internal.hpp:1484-1504), optionally followed by `layout` (see q4k_matmul_layout).
qmm_status run_gemm_q4k_id(const LaunchCtx& c, bool wmma) {
  if (!counts(c, 3, 3) && !counts(c, 3, 4)) return bad("gemm_q4k: expects 3 buffers and 3 scalars (a fourth: layout)");
  const uint64_t m = c.sc[0], n = c.sc[1], k = c.sc[2], layout = c.nsc > 3 ? c.sc[3] : 0;
  if (!dims_ok(m, n, k) || k % 256 != 0) return bad("gemm_q4k: m, n, k must be non-zero and k a multiple of 256");
  if (!q4k_layout_ok(n, k, layout)) return bad("gemm_q4k: layout is 0 (GGUF order) or the rows per group of a row-group copy (1..64)");
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, q4k_bytes(n, k)) ||
      !c.fits(2, static_cast<u128>(m) * n * 4)) {
    return bad("gemm_q4k: a buffer is smaller than m, n, k require");
  }
  return q4k_matmul_layout(c, c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<float>(2), m, n, k,
                           wmma ? kQ4KGemmMinRows : g_q4k_tensor_rows.load(std::memory_order_relaxed), layout);
}
qmm_status run_gemm_q4k(const LaunchCtx& c) { return run_gemm_q4k_id(c, false); }
qmm_status run_gemm_q4k_wmma(const LaunchCtx& c) { return run_gemm_q4k_id(c, true); }

// "gemm_q4k_vec" and "gemm_q4k_rows{R}": buffers A, W, C; scalars m, n, k, split
// (src/backends/rocm/rocm_kernels_gemv.cpp:17-24,103-156), optionally followed by `layout`.  C has `split` regions of
// m*n floats whose sum is the result: either every region receives the partial sums of its K
// slice (one row, slices of 4096 weights or more), or region 0 receives the whole dot product and
// regions 1..split-1 are zeroed; "gemm_vec_reduce" over them yields the result either way.
qmm_status run_gemm_q4k_split(const LaunchCtx& c, uint64_t rows_required) {
  if (!counts(c, 3, 4) && !counts(c, 3, 5)) return bad("gemm_q4k_vec/rows: expects 3 buffers and 4 scalars (a fifth: layout)");
  const uint64_t m = c.sc[0], n = c.sc[1], k = c.sc[2], split = c.sc[3], layout = c.nsc > 4 ? c.sc[4] : 0;
  if (!dims_ok(m, n, k) || k % 256 != 0) return bad("gemm_q4k_vec/rows: bad m, n, k");
  if (!q4k_layout_ok(n, k, layout)) return bad("gemm_q4k_vec/rows: layout is 0 (GGUF order) or the rows per group of a row-group copy (1..64)");
  if (rows_required != 0 && m != rows_required) return bad("gemm_q4k_rowsR: m must equal R");
  if (split == 0 || split > 64 || (k / 256) % split != 0) return bad("gemm_q4k_vec/rows: split must divide k/256");
  const u128 region = static_cast<u128>(m) * n * 4;
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, q4k_bytes(n, k)) || !c.fits(2, region * split)) {
    return bad("gemm_q4k_vec/rows: a buffer is smaller than m, n, k, split require");
  }
  float* out = c.ptr<float>(2);
  // One row of a large matrix with long enough slices: real partial sums, one region per slice,
  // each workgroup staging only its slice of the activations.
  if (layout == 0 && m == 1 && n <= 0xFFFFFFFFull && k <= 0xFFFFFFFFull && qmm::q4k_gemv_split_supported(n, k, split)) {
    return map_hip(qmm::launch_q4k_gemv_split(c.ptr<const float>(0), c.ptr<const uint8_t>(1), out, static_cast<uint32_t>(n),
                                              static_cast<uint32_t>(k), static_cast<uint32_t>(split), c.stream));
  }
  qmm_status st = q4k_matmul_layout(c, c.ptr<const float>(0), c.ptr<const uint8_t>(1), out, m, n, k,
                                    g_q4k_tensor_rows.load(std::memory_order_relaxed), layout);
  if (st == QMM_OK && split > 1) {
    st = map_hip(qmm::launch_fill_f32(out + m * n, 0.0f, (split - 1) * m * n, c.stream));
  }
  return st;
}
qmm_status run_gemm_q4k_vec(const LaunchCtx& c) { return run_gemm_q4k_split(c, 0); }
qmm_status run_gemm_q4k_rows2(const LaunchCtx& c) { return run_gemm_q4k_split(c, 2); }
qmm_status run_gemm_q4k_rows3(const LaunchCtx& c) { return run_gemm_q4k_split(c, 3); }
qmm_status run_gemm_q4k_rows4(const LaunchCtx& c) { return run_gemm_q4k_split(c, 4); }
qmm_status run_gemm_q4k_rows5(const LaunchCtx& c) { return run_gemm_q4k_split(c, 5); }

// "gemm_vec_reduce" / "gemm_mxfp4_wmma_reduce": buffers part, c; scalars total, split.
qmm_status run_vec_reduce(const LaunchCtx& c) {
  if (!counts(c, 2, 2)) return bad("gemm_vec_reduce: expects 2 buffers and 2 scalars");
  const uint64_t total = c.sc[0], split = c.sc[1];
  if (total == 0 || split == 0 || total > (1ull << 40) || split > 4096) return bad("gemm_vec_reduce: bad total or split");
  if (!c.fits(0, static_cast<u128>(total) * split * 4) || !c.fits(1, static_cast<u128>(total) * 4)) {
    return bad("gemm_vec_reduce: a buffer is smaller than total, split require");
  }
  return map_hip(qmm::launch_vec_reduce(c.ptr<const float>(0), c.ptr<float>(1), total, split, c.stream));
}

// "silu_mul": buffers G, U, O (fp32, n each); scalar n.  O = silu(G) * U
// (include/tessera/backend.hpp:257-259,618-625).
qmm_status run_silu_mul(const LaunchCtx& c) {
  if (!counts(c, 3, 1)) return bad("silu_mul: expects 3 buffers and 1 scalar");
  const uint64_t n = c.sc[0];
  if (n == 0 || n > (1ull << 40)) return bad("silu_mul: n must be non-zero");
  const u128 bytes = static_cast<u128>(n) * 4;
  if (!c.fits(0, bytes) || !c.fits(1, bytes) || !c.fits(2, bytes)) return bad("silu_mul: a buffer is smaller than n requires");
  return map_hip(qmm::launch_silu_mul(c.ptr<const float>(0), c.ptr<const float>(1), c.ptr<float>(2), n, c.stream));
}

// "add": buffers A, B, O (fp32, n each); scalar n (include/tessera/backend.hpp:255-256,618-625).
qmm_status run_add(const LaunchCtx& c) {
  if (!counts(c, 3, 1)) return bad("add: expects 3 buffers and 1 scalar");
  const uint64_t n = c.sc[0];
  if (n == 0 || n > (1ull << 40)) return bad("add: n must be non-zero");
  const u128 bytes = static_cast<u128>(n) * 4;
  if (!c.fits(0, bytes) || !c.fits(1, bytes) || !c.fits(2, bytes)) return bad("add: a buffer is smaller than n requires");
  return map_hip(qmm::launch_add(c.ptr<const float>(0), c.ptr<const float>(1), c.ptr<float>(2), n, c.stream));
}

// "read_probe" (not a reference id; a measuring aid): buffers Src, Out (at least 4 bytes, left
// untouched); scalar bytes (a multiple of 16).  Reads Src once and does nothing else.
qmm_status run_read_probe(const LaunchCtx& c) {
  if (!counts(c, 2, 1)) return bad("read_probe: expects 2 buffers and 1 scalar");
  const uint64_t bytes = c.sc[0];
  if (bytes == 0 || bytes % 16 != 0 || !c.fits(0, bytes) || !c.fits(1, 4)) return bad("read_probe: bytes must be a non-zero multiple of 16 within the buffer");
  return map_hip(qmm::launch_read_probe(c.ptr<const void>(0), c.ptr<uint32_t>(1), bytes, c.stream));
}

// "mfma_probe" (not a reference id; the matrix-core ceiling the prefill GEMMs are compared with, as
// "read_probe" is the memory one): buffer out (workgroups * 256 fp32); scalars kind (0: fp16 32x32x16,
// 1: scaled E4M3 x E2M1 32x32x64, 2: int8 16x16x64), random (0: constant operands, 1: hashed), iters,
// workgroups.  Executes workgroups * 4 * 4 * iters matrix instructions and nothing else.
qmm_status run_mfma_probe(const LaunchCtx& c) {
  if (!counts(c, 1, 4)) return bad("mfma_probe: expects 1 buffer and 4 scalars");
  const uint64_t kind = c.sc[0], random = c.sc[1], iters = c.sc[2], wgs = c.sc[3];
  if (kind > 2 || random > 1 || iters == 0 || iters > (1u << 24) || wgs == 0 || wgs > 65536 || !c.fits(0, wgs * 1024)) {
    return bad("mfma_probe: kind 0..2, random 0 or 1, 1..2^24 iterations, 1..65536 workgroups, out of workgroups * 256 floats");
  }
  return map_hip(qmm::launch_mfma_probe(c.ptr<float>(0), static_cast<uint32_t>(kind), random == 1, static_cast<uint32_t>(iters),
                                        static_cast<uint32_t>(wgs), c.stream));
}

// "fill": buffer 0 is an int32 array; scalars value, count (include/tessera/backend.hpp:151-152,393-396).
qmm_status run_fill(const LaunchCtx& c) {
  if (!counts(c, 1, 2)) return bad("fill: expects 1 buffer and 2 scalars");
  const uint64_t n = c.sc[1];
  if (n > (1ull << 40) || !c.fits(0, static_cast<u128>(n) * 4)) return bad("fill: the buffer is smaller than the count requires");
  if (n == 0) return QMM_OK;
  return map_hip(qmm::launch_fill_i32(c.ptr<int32_t>(0), static_cast<int32_t>(c.sc[0]), n, c.stream));
}

// "rmsnorm": buffers X (rows x cols), W (cols), Y (rows x cols); scalars rows, cols, fp32 bits of
// epsilon (include/tessera/backend.hpp:212-216,557-564).
qmm_status run_rmsnorm(const LaunchCtx& c) {
  if (!counts(c, 3, 3)) return bad("rmsnorm: expects 3 buffers and 3 scalars");
  const uint64_t rows = c.sc[0], cols = c.sc[1];
  if (rows == 0 || cols == 0 || rows > (1u << 30) || cols > (1ull << 32)) return bad("rmsnorm: rows and cols must be non-zero");
  const u128 bytes = static_cast<u128>(rows) * cols * 4;
  if (!c.fits(0, bytes) || !c.fits(1, static_cast<u128>(cols) * 4) || !c.fits(2, bytes)) {
    return bad("rmsnorm: a buffer is smaller than rows, cols require");
  }
  const uint32_t eps_bits = static_cast<uint32_t>(c.sc[2]);
  float eps;
  std::memcpy(&eps, &eps_bits, 4);
  return map_hip(qmm::launch_rmsnorm(c.ptr<const float>(0), c.ptr<const float>(1), c.ptr<float>(2), rows, cols, eps, c.stream));
}

// "rope": buffer X (rows x heads x head_dim fp32, rotated in place); scalars rows, heads, head_dim,
// rope_dim, pos_base, fp32 bits of theta (include/tessera/backend.hpp:162-166,417-428).
// "mrope": buffers X, Pos (rows x 3 u64: temporal, height, width); scalars rows, heads, head_dim,
// rope_dim, fp32 bits of theta, sec_t, sec_h, sec_w (backend.hpp:378-385,805-818).
qmm_status run_rope_common(const LaunchCtx& c, bool multimodal) {
  if (!counts(c, multimodal ? 2 : 1, multimodal ? 8 : 6)) return bad("rope/mrope: wrong number of buffers or scalars");
  const uint64_t rows = c.sc[0], heads = c.sc[1], head_dim = c.sc[2], rope_dim = c.sc[3];
  if (rows == 0 || heads == 0 || head_dim == 0 || rope_dim == 0 || rope_dim > head_dim || head_dim % 2 != 0 || rope_dim % 2 != 0 ||
      rows > (1u << 30) || heads > (1u << 20) || head_dim > (1u << 20)) {
    return bad("rope/mrope: rows, heads, head_dim, rope_dim must be non-zero, the dims even, rope_dim <= head_dim");
  }
  const uint64_t sec_t = multimodal ? c.sc[5] : 0, sec_h = multimodal ? c.sc[6] : 0, sec_w = multimodal ? c.sc[7] : 0;
  if (multimodal && (sec_t > rope_dim || sec_h > rope_dim || sec_w > rope_dim || sec_t + sec_h + sec_w > rope_dim / 2)) {
    return bad("mrope: the sections hold more pairs than rope_dim / 2");
  }
  if (!c.fits(0, static_cast<u128>(rows) * heads * head_dim * 4) || (multimodal && !c.fits(1, static_cast<u128>(rows) * 24))) {
    return bad("rope/mrope: a buffer is smaller than rows, heads, head_dim require");
  }
  const uint32_t theta_bits = static_cast<uint32_t>(c.sc[multimodal ? 4 : 5]);
  float theta;
  std::memcpy(&theta, &theta_bits, 4);
  if (!(theta > 0.0f)) return bad("rope/mrope: theta must be positive");
  return map_hip(qmm::launch_rope(c.ptr<float>(0), multimodal ? c.ptr<const uint64_t>(1) : nullptr, rows, heads, head_dim, rope_dim,
                                  multimodal ? 0 : c.sc[4], theta, sec_t, sec_h, c.stream));
}
qmm_status run_rope(const LaunchCtx& c) { return run_rope_common(c, false); }
qmm_status run_mrope(const LaunchCtx& c) { return run_rope_common(c, true); }

// "attention": buffers Q (rows x heads*head_dim fp32), K, V (n x kv_heads*head_dim, fp32 or fp16), Out
// (as Q); scalars m, n, heads, kv_heads, head_dim, q_base, row_base, window, kv_f16, causal
// (include/tessera/backend.hpp:167-179,429-440).  Q and Out hold at least row_base + m rows.
qmm_status run_attention(const LaunchCtx& c) {
  if (!counts(c, 4, 10)) return bad("attention: expects 4 buffers and 10 scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], heads = c.sc[2], kv_heads = c.sc[3], head_dim = c.sc[4], q_base = c.sc[5],
                 row_base = c.sc[6], window = c.sc[7], kv_f16 = c.sc[8], causal = c.sc[9];
  if (m == 0 || n == 0 || heads == 0 || kv_heads == 0 || head_dim == 0 || heads % kv_heads != 0) {
    return bad("attention: m, n, heads, kv_heads, head_dim must be non-zero and heads a multiple of kv_heads");
  }
  if (head_dim > 256) return bad("attention: head_dim must be at most 256");
  if (m > (1u << 24) || n > (1ull << 32) || heads > (1u << 16) || row_base > (1ull << 32) || q_base > (1ull << 40) ||
      m * heads > 0x7FFFFFFFull || kv_f16 > 1 || causal > 1) {
    return bad("attention: a scalar is out of range");
  }
  const u128 q_bytes = static_cast<u128>(row_base + m) * heads * head_dim * 4;
  const u128 kv_bytes = static_cast<u128>(n) * kv_heads * head_dim * (kv_f16 ? 2 : 4);
  if (!c.fits(0, q_bytes) || !c.fits(1, kv_bytes) || !c.fits(2, kv_bytes) || !c.fits(3, q_bytes)) {
    return bad("attention: a buffer is smaller than the scalars require");
  }
  return map_hip(qmm::launch_attention(c.ptr<const float>(0), c.ptr<const void>(1), c.ptr<const void>(2), c.ptr<float>(3), m, n,
                                       heads, kv_heads, head_dim, q_base, row_base, window, kv_f16 == 1, causal == 1, c.stream));
}

// "attention_q8", "attention_q4", "attention_fp8": buffers q, K and V codes (n x kv_heads*head_dim int8
// / nibbles, two a byte / E4M3), one fp32 scale per key row for K and for V, out; scalars m, n, heads,
// kv_heads, head_dim, q_base, row_base, window, kind (0..2; the id fixes the decode, as in the
// reference's kernels) (include/tessera/backend.hpp:284-309,679-691; always causal).
qmm_status run_attention_quant(const LaunchCtx& c, uint32_t kind) {
  if (!counts(c, 6, 9)) return bad("attention_q8/q4/fp8: expects 6 buffers and 9 scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], heads = c.sc[2], kv_heads = c.sc[3], head_dim = c.sc[4], q_base = c.sc[5],
                 row_base = c.sc[6], window = c.sc[7];
  if (m == 0 || n == 0 || heads == 0 || kv_heads == 0 || head_dim == 0 || heads % kv_heads != 0 || c.sc[8] > 2) {
    return bad("attention_q8/q4/fp8: m, n, heads, kv_heads, head_dim must be non-zero, heads a multiple of kv_heads, kind 0..2");
  }
  if (head_dim > 256) return bad("attention_q8/q4/fp8: head_dim must be at most 256");
  if (kind == 1 && (kv_heads * head_dim) % 2 != 0) return bad("attention_q4: a key row must hold an even number of codes");
  if (m > (1u << 24) || n > (1ull << 32) || heads > (1u << 16) || row_base > (1ull << 32) || q_base > (1ull << 40) ||
      m * heads > 0x7FFFFFFFull) {
    return bad("attention_q8/q4/fp8: a scalar is out of range");
  }
  const u128 q_bytes = static_cast<u128>(row_base + m) * heads * head_dim * 4;
  const u128 codes = static_cast<u128>(n) * kv_heads * head_dim;
  const u128 kv_bytes = kind == 1 ? codes / 2 : codes;
  if (!c.fits(0, q_bytes) || !c.fits(1, kv_bytes) || !c.fits(2, kv_bytes) || !c.fits(3, static_cast<u128>(n) * 4) ||
      !c.fits(4, static_cast<u128>(n) * 4) || !c.fits(5, q_bytes)) {
    return bad("attention_q8/q4/fp8: a buffer is smaller than the scalars require");
  }
  return map_hip(qmm::launch_attention_quant(c.ptr<const float>(0), c.ptr<const void>(1), c.ptr<const void>(2),
                                             c.ptr<const float>(3), c.ptr<const float>(4), c.ptr<float>(5), m, n, heads,
                                             kv_heads, head_dim, q_base, row_base, window, kind, c.stream));
}
qmm_status run_attention_q8(const LaunchCtx& c) { return run_attention_quant(c, 0); }
qmm_status run_attention_q4(const LaunchCtx& c) { return run_attention_quant(c, 1); }
qmm_status run_attention_fp8(const LaunchCtx& c) { return run_attention_quant(c, 2); }

// The flash-decoding forms.  "attention_split" / "attention_split_gqa": buffers q, k, v, pacc
// (m*heads*split x head_dim), pmax, psum (m*heads*split each); scalars m, n, heads, kv_heads,
// head_dim, q_base, window, kv_f16, causal, split (the gqa id: m = 1 and at most 6 heads a kv head;
// same partials, so this backend runs it as the plain split).  "attention_q8_split" / "_q4_split" /
// "_fp8_split": buffers q, k, v, ks, vs, pacc, pmax, psum; scalars m, n, heads, kv_heads, head_dim,
// q_base, window, kind, split (include/tessera/backend.hpp:310-329,441-466,692-705).
qmm_status run_attention_split_common(const LaunchCtx& c, const char* id, bool quant, uint32_t kind, bool gqa) {
  if (!counts(c, quant ? 8 : 6, quant ? 9 : 10)) return bad(std::string(id) + ": wrong number of buffers or scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], heads = c.sc[2], kv_heads = c.sc[3], head_dim = c.sc[4], q_base = c.sc[5],
                 window = c.sc[6];
  const uint64_t split = quant ? c.sc[8] : c.sc[9];
  if (m == 0 || n == 0 || heads == 0 || kv_heads == 0 || head_dim == 0 || heads % kv_heads != 0 || split == 0) {
    return bad(std::string(id) + ": m, n, heads, kv_heads, head_dim, split must be non-zero and heads a multiple of kv_heads");
  }
  if (quant ? c.sc[7] > 2 : (c.sc[7] > 1 || c.sc[8] > 1)) return bad(std::string(id) + ": kind, kv_f16 or causal out of range");
  if (gqa && (m != 1 || heads / kv_heads > 6)) return bad(std::string(id) + ": m must be 1 and heads / kv_heads at most 6");
  if (head_dim > 256) return bad(std::string(id) + ": head_dim must be at most 256");
  if (quant && kind == 1 && (kv_heads * head_dim) % 2 != 0) return bad(std::string(id) + ": a key row must hold an even number of codes");
  if (m > (1u << 24) || n > (1ull << 32) || heads > (1u << 16) || q_base > (1ull << 40) || split > (1u << 16) ||
      static_cast<u128>(m) * heads * split > 0x7FFFFFFFull) {
    return bad(std::string(id) + ": a scalar is out of range");
  }
  const u128 q_bytes = static_cast<u128>(m) * heads * head_dim * 4;
  const u128 codes = static_cast<u128>(n) * kv_heads * head_dim;
  const u128 kv_bytes = !quant ? codes * (c.sc[7] ? 2 : 4) : kind == 1 ? codes / 2 : codes;
  const u128 parts = static_cast<u128>(m) * heads * split;
  const size_t p0 = quant ? 5 : 3;
  bool ok = c.fits(0, q_bytes) && c.fits(1, kv_bytes) && c.fits(2, kv_bytes) && c.fits(p0, parts * head_dim * 4) &&
            c.fits(p0 + 1, parts * 4) && c.fits(p0 + 2, parts * 4);
  if (quant) ok = ok && c.fits(3, static_cast<u128>(n) * 4) && c.fits(4, static_cast<u128>(n) * 4);
  if (!ok) return bad(std::string(id) + ": a buffer is smaller than the scalars require");
  const uint32_t kv_kind = quant ? 2u + kind : static_cast<uint32_t>(c.sc[7]);
  const bool causal = quant ? true : c.sc[8] == 1;
  return map_hip(qmm::launch_attention_split(c.ptr<const float>(0), c.ptr<const void>(1), c.ptr<const void>(2),
                                             quant ? c.ptr<const float>(3) : nullptr, quant ? c.ptr<const float>(4) : nullptr,
                                             c.ptr<float>(p0), c.ptr<float>(p0 + 1), c.ptr<float>(p0 + 2), m, n, heads, kv_heads,
                                             head_dim, q_base, window, kv_kind, causal, split, c.stream));
}
qmm_status run_attention_split(const LaunchCtx& c) { return run_attention_split_common(c, "attention_split", false, 0, false); }
qmm_status run_attention_split_gqa(const LaunchCtx& c) { return run_attention_split_common(c, "attention_split_gqa", false, 0, true); }
qmm_status run_attention_q8_split(const LaunchCtx& c) { return run_attention_split_common(c, "attention_q8_split", true, 0, false); }
qmm_status run_attention_q4_split(const LaunchCtx& c) { return run_attention_split_common(c, "attention_q4_split", true, 1, false); }
qmm_status run_attention_fp8_split(const LaunchCtx& c) { return run_attention_split_common(c, "attention_fp8_split", true, 2, false); }

// "attention_combine": buffers pacc, pmax, psum, out (m x heads*head_dim); scalars m, heads, head_dim,
// split (include/tessera/backend.hpp:330-333,467-475).
qmm_status run_attention_combine(const LaunchCtx& c) {
  if (!counts(c, 4, 4)) return bad("attention_combine: expects 4 buffers and 4 scalars");
  const uint64_t m = c.sc[0], heads = c.sc[1], head_dim = c.sc[2], split = c.sc[3];
  if (m == 0 || heads == 0 || head_dim == 0 || split == 0) return bad("attention_combine: m, heads, head_dim, split must be non-zero");
  if (head_dim > 256 || m > (1u << 24) || heads > (1u << 16) || split > (1u << 16) || m * heads > 0x7FFFFFFFull) {
    return bad("attention_combine: a scalar is out of range");
  }
  const u128 parts = static_cast<u128>(m) * heads * split;
  if (!c.fits(0, parts * head_dim * 4) || !c.fits(1, parts * 4) || !c.fits(2, parts * 4) ||
      !c.fits(3, static_cast<u128>(m) * heads * head_dim * 4)) {
    return bad("attention_combine: a buffer is smaller than the scalars require");
  }
  return map_hip(qmm::launch_attention_combine(c.ptr<const float>(0), c.ptr<const float>(1), c.ptr<const float>(2), c.ptr<float>(3),
                                               m, heads, head_dim, split, c.stream));
}

// "quantize_q8" / "quantize_q4": buffers In (rows x cols fp32), Out (int8 codes / 4-bit codes, two a
// byte), one fp32 scale per row; scalars rows, cols (a multiple of 4 / of 8)
// (include/tessera/backend.hpp:280-283,292-295,670-678,706-714).
qmm_status run_quantize_kv(const LaunchCtx& c, uint32_t bits) {
  if (!counts(c, 3, 2)) return bad("quantize_q8/q4: expects 3 buffers and 2 scalars");
  const uint64_t rows = c.sc[0], cols = c.sc[1];
  if (rows == 0 || cols == 0 || cols % (bits == 8 ? 4 : 8) != 0 || rows > 0x7FFFFFFFull || cols > (1ull << 32)) {
    return bad("quantize_q8/q4: rows and cols must be non-zero, cols a multiple of 4 (q8) or 8 (q4)");
  }
  if (!c.fits(0, static_cast<u128>(rows) * cols * 4) || !c.fits(1, static_cast<u128>(rows) * cols * bits / 8) ||
      !c.fits(2, static_cast<u128>(rows) * 4)) {
    return bad("quantize_q8/q4: a buffer is smaller than rows and cols require");
  }
  return map_hip(qmm::launch_quantize_kv(c.ptr<const float>(0), c.ptr<uint8_t>(1), c.ptr<float>(2), rows, cols, bits, c.stream));
}
qmm_status run_quantize_q8(const LaunchCtx& c) { return run_quantize_kv(c, 8); }
qmm_status run_quantize_q4(const LaunchCtx& c) { return run_quantize_kv(c, 4); }

// "cast_f32_f16": buffers In (n fp32), Out (n binary16, two per 32-bit word); scalar n, even
// (include/tessera/backend.hpp:334-336,732-740).
qmm_status run_cast_f32_f16(const LaunchCtx& c) {
  if (!counts(c, 2, 1)) return bad("cast_f32_f16: expects 2 buffers and 1 scalar");
  const uint64_t n = c.sc[0];
  if (n == 0 || n % 2 != 0 || n > (1ull << 40)) return bad("cast_f32_f16: n must be non-zero and even");
  if (!c.fits(0, static_cast<u128>(n) * 4) || !c.fits(1, static_cast<u128>(n) * 2)) return bad("cast_f32_f16: a buffer is smaller than n requires");
  return map_hip(qmm::launch_cast_f32_f16(c.ptr<const float>(0), c.ptr<void>(1), n, c.stream));
}

// "qgate_split": buffers Fused (rows x heads x 2*head_dim: per head the query then the gate), Q, G
// (rows x heads*head_dim each); scalars heads, head_dim, rows (include/tessera/backend.hpp:386-390,819-826).
qmm_status run_qgate_split(const LaunchCtx& c) {
  if (!counts(c, 3, 3)) return bad("qgate_split: expects 3 buffers and 3 scalars");
  const uint64_t heads = c.sc[0], head_dim = c.sc[1], rows = c.sc[2];
  if (heads == 0 || head_dim == 0 || rows == 0 || heads > (1u << 20) || head_dim > (1u << 20) || rows > (1u << 30)) {
    return bad("qgate_split: heads, head_dim and rows must be non-zero");
  }
  const u128 part = static_cast<u128>(rows) * heads * head_dim * 4;
  if (!c.fits(0, part * 2) || !c.fits(1, part) || !c.fits(2, part)) return bad("qgate_split: a buffer is smaller than the scalars require");
  return map_hip(qmm::launch_qgate_split(c.ptr<const float>(0), c.ptr<float>(1), c.ptr<float>(2), heads, head_dim, rows, c.stream));
}

// "embedding_f32", "embedding_bf16", "embedding_q4k": buffers ids (u32, rows), table (vocab x cols),
// Out (fp32 rows x cols); scalars rows, cols, vocab (include/tessera/backend.hpp:260-265,827-839).
qmm_status run_embedding(const LaunchCtx& c, int kind) {
  if (!counts(c, 3, 3)) return bad("embedding: expects 3 buffers and 3 scalars");
  const uint64_t rows = c.sc[0], cols = c.sc[1], vocab = c.sc[2];
  if (rows == 0 || cols == 0 || vocab == 0 || rows > (1u << 30) || cols > (1u << 30) || vocab > (1u << 30)) {
    return bad("embedding: rows, cols and vocab must be non-zero");
  }
  if (kind == 2 && cols % 256 != 0) return bad("embedding_q4k: cols must be a multiple of 256");
  const u128 table = kind == 0 ? static_cast<u128>(vocab) * cols * 4
                     : kind == 1 ? static_cast<u128>(vocab) * cols * 2
                                 : static_cast<u128>(vocab) * (cols / 256) * 144;
  if (!c.fits(0, static_cast<u128>(rows) * 4) || !c.fits(1, table) || !c.fits(2, static_cast<u128>(rows) * cols * 4)) {
    return bad("embedding: a buffer is smaller than rows, cols, vocab require");
  }
  return map_hip(qmm::launch_embedding(kind, c.ptr<const uint32_t>(0), c.ptr<const void>(1), c.ptr<float>(2), rows, cols,
                                       vocab, c.stream));
}
qmm_status run_embedding_f32(const LaunchCtx& c) { return run_embedding(c, 0); }
qmm_status run_embedding_bf16(const LaunchCtx& c) { return run_embedding(c, 1); }
qmm_status run_embedding_q4k(const LaunchCtx& c) { return run_embedding(c, 2); }

// "round_bf16": buffer 0 is the fp32 data rounded in place to bfloat16 precision; scalar n
// (include/tessera/backend.hpp:337-339,740-747; src/models/qwen3_5/project.cpp:351-364).
qmm_status run_round_bf16(const LaunchCtx& c) {
  if (!counts(c, 1, 1)) return bad("round_bf16: expects 1 buffer and 1 scalar");
  const uint64_t n = c.sc[0];
  if (n == 0 || n > (1ull << 40)) return bad("round_bf16: n must be non-zero");
  if (!c.fits(0, static_cast<u128>(n) * 4)) return bad("round_bf16: the buffer is smaller than n requires");
  return map_hip(qmm::launch_round_bf16(c.ptr<float>(0), n, c.stream));
}

// "ffn_gate_up_silu_q4k" (not a reference id; the dense analogue of "moe_experts_gate_up_q4k"):
// buffers X (fp32 m x k), Gate, Up (Q4_K, n rows of k each), Out (fp32 m x n); scalars m, n, k.
// Where the up product of "ffn_gate_up_silu_q4k" with several rows lives.  Below the tensor-tile
// threshold: in the fixed decode scratch, behind the room the few-row kernels may use for their
// activation operand or their K parts, so nothing is allocated (a recorded decode step stays
// valid) -- when it fits.  Otherwise in the workspace, behind whatever the Q4_K GEMM keeps at its
// start (a request for that smaller size returns the same base, so the two do not overlap).
struct FfnScratch {
  bool in_decode_scratch;
  size_t up_off;
  size_t workspace_bytes;
};
FfnScratch ffn_scratch(uint64_t m, uint64_t n, uint64_t k) {
  const size_t up_bytes = static_cast<size_t>(m) * n * 4;
  const bool f16 = m >= g_q4k_tensor_rows.load(std::memory_order_relaxed) && qmm::gemm_q4k_supported(m, k);
  if (!f16) {
    const uint64_t chunk = m < 16 ? m : 16, tail = m % 16;
    size_t room = qmm::gemv_q4k_mfma_workspace_bytes(8, k);
    const size_t parts = qmm::gemv_q4k_rows16_workspace_bytes(chunk, n, k);
    const size_t parts_tail = tail >= 2 ? qmm::gemv_q4k_rows16_workspace_bytes(tail, n, k) : 0;
    room = room > parts ? room : parts;
    room = room > parts_tail ? room : parts_tail;
    const size_t up_off = (room + 255) & ~size_t{255};
    if (up_off + up_bytes <= kDecodeScratchBytes) return FfnScratch{true, up_off, 0};
    // In the workspace, but still behind the few-row kernels' room: qmm_launch_static serves the
    // workspace and the decode scratch from the same array, where offset 0 would be under their
    // partial sums.
    return FfnScratch{false, up_off, up_off + up_bytes};
  }
  const size_t up_off = (qmm::gemm_q4k_workspace_bytes(m, k) + 255) & ~size_t{255};
  return FfnScratch{false, up_off, up_off + up_bytes};
}

// Out = silu(X Gate^T) * (X Up^T), what the reference computes with two "gemm_q4k*" launches
// and "silu_mul" (src/models/qwen3_5/trunk.cpp:294-304).  One row of a supported k is a single launch that
// reads the activations once for both matrices; anything else runs the two products through the
// Q4_K regimes above (the up product into library scratch) and multiplies.
qmm_status run_ffn_gate_up_silu_q4k(const LaunchCtx& c) {
  if (!counts(c, 4, 3)) return bad("ffn_gate_up_silu_q4k: expects 4 buffers and 3 scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], k = c.sc[2];
  if (!dims_ok(m, n, k) || k % 256 != 0) return bad("ffn_gate_up_silu_q4k: m, n, k must be non-zero and k a multiple of 256");
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, q4k_bytes(n, k)) || !c.fits(2, q4k_bytes(n, k)) ||
      !c.fits(3, static_cast<u128>(m) * n * 4)) {
    return bad("ffn_gate_up_silu_q4k: a buffer is smaller than m, n, k require");
  }
  const float* x = c.ptr<const float>(0);
  const uint8_t* gate = c.ptr<const uint8_t>(1);
  const uint8_t* up = c.ptr<const uint8_t>(2);
  float* out = c.ptr<float>(3);
  if (m == 1 && qmm::ffn_gate_up_q4k_supported(k)) {
    return map_hip(qmm::launch_ffn_gate_up_q4k(x, gate, up, out, static_cast<uint32_t>(n), static_cast<uint32_t>(k), c.stream));
  }
  const FfnScratch lay = ffn_scratch(m, n, k);
  float* u = nullptr;
  qmm_status st = QMM_OK;
  if (lay.in_decode_scratch && decode_scratch(c) != nullptr) {
    u = reinterpret_cast<float*>(static_cast<uint8_t*>(decode_scratch(c)) + lay.up_off);
  } else {
    void* ws = nullptr;
    st = workspace(c, lay.workspace_bytes, &ws);
    if (st != QMM_OK) return st;
    u = reinterpret_cast<float*>(static_cast<uint8_t*>(ws) + lay.up_off);
  }
  st = q4k_matmul(c, x, gate, out, m, n, k);
  if (st == QMM_OK) st = q4k_matmul(c, x, up, u, m, n, k);
  if (st == QMM_OK) st = map_hip(qmm::launch_silu_mul(out, u, out, m * n, c.stream));
  return st;
}

// "dequant_q4k" (not a reference id): buffers W, Out (fp32); scalar nblocks.
qmm_status run_dequant_q4k(const LaunchCtx& c) {
  if (!counts(c, 2, 1)) return bad("dequant_q4k: expects 2 buffers and 1 scalar");
  const uint64_t nb = c.sc[0];
  if (nb == 0 || nb > (1ull << 32)) return bad("dequant_q4k: bad block count");
  if (!c.fits(0, static_cast<u128>(nb) * 144) || !c.fits(1, static_cast<u128>(nb) * 1024)) {
    return bad("dequant_q4k: a buffer is smaller than nblocks requires");
  }
  return map_hip(qmm::launch_dequant_q4k(c.ptr<const uint8_t>(0), c.ptr<float>(1), nb, c.stream));
}

// Q5_K / Q6_K from kQ4KGemmMinRows rows up: weights decoded once to fp16 in the library
// workspace, then the dense fp16 MFMA GEMM.
qmm_status kquant_prefill(const LaunchCtx& c, uint32_t block_bytes, uint64_t m, uint64_t n, uint64_t k,
                          uint64_t split) {
  void* ws = nullptr;
  qmm_status st = workspace(c, qmm::gemm_kquant_f16_workspace_bytes(m, n, k), &ws);
  if (st != QMM_OK) return st;
  float* out = c.ptr<float>(2);
  st = map_hip(qmm::launch_kquant_f16_gemm(c.ptr<const float>(0), c.ptr<const uint8_t>(1), block_bytes, out, ws,
                                           static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                           static_cast<uint32_t>(k), c.stream));
  if (st == QMM_OK && split > 1) st = map_hip(qmm::launch_fill_f32(out + m * n, 0.0f, (split - 1) * m * n, c.stream));
  return st;
}

// ---- Q5_K ---------------------------------------------------------------------
// "gemm_q5k", "gemm_q5k_batched", "gemm_q5k_vec", "gemm_q5k_rows{R}": as the Q6_K ids below, with
// 176-byte blocks (include/tessera/backend.hpp:202-206,524-536; rocm_backend.cpp:95-101).
qmm_status q5k_matmul(const LaunchCtx& c, uint64_t m, uint64_t n, uint64_t k, uint64_t split, const char* who) {
  if (!dims_ok(m, n, k) || k % 256 != 0) return bad(std::string(who) + ": m, n, k must be non-zero and k a multiple of 256");
  if (split == 0 || split > 64 || (k / 256) % split != 0) return bad(std::string(who) + ": split must divide k/256");
  const u128 region = static_cast<u128>(m) * n * 4;
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, static_cast<u128>(n) * (k / 256) * 176) ||
      !c.fits(2, region * split)) {
    return bad(std::string(who) + ": a buffer is smaller than m, n, k require");
  }
  float* out = c.ptr<float>(2);
  if (m >= kQ4KGemmMinRows && qmm::gemm_kquant_f16_supported(m, n, k)) {
    return kquant_prefill(c, 176, m, n, k, split);
  }
  // Several rows: one pass over the weights for up to eight of them on the int8 matrix cores
  // (17408 x 5120: 2 rows 17.6 us against 30.3 on a multiply-add pass per row, 8 rows 31 against 121).
  const bool one_pass = m >= 2 && qmm::gemv_kquant_rows_supported(m, n, k);
  const auto launch = one_pass ? qmm::launch_q5k_rows_i8 : qmm::launch_q5k_gemv;
  qmm_status st = map_hip(launch(c.ptr<const float>(0), c.ptr<const uint8_t>(1), out, static_cast<uint32_t>(m),
                                 static_cast<uint32_t>(n), static_cast<uint32_t>(k), c.stream));
  if (st == QMM_OK && split > 1) st = map_hip(qmm::launch_fill_f32(out + m * n, 0.0f, (split - 1) * m * n, c.stream));
  return st;
}
qmm_status run_gemm_q5k(const LaunchCtx& c) {
  if (!counts(c, 3, 3)) return bad("gemm_q5k: expects 3 buffers and 3 scalars");
  return q5k_matmul(c, c.sc[0], c.sc[1], c.sc[2], 1, "gemm_q5k");
}
qmm_status run_gemm_q5k_split(const LaunchCtx& c, uint64_t rows_required) {
  if (!counts(c, 3, 4)) return bad("gemm_q5k_vec/rows: expects 3 buffers and 4 scalars");
  if (rows_required != 0 && c.sc[0] != rows_required) return bad("gemm_q5k_rowsR: m must equal R");
  return q5k_matmul(c, c.sc[0], c.sc[1], c.sc[2], c.sc[3], "gemm_q5k_vec/rows");
}
qmm_status run_gemm_q5k_vec(const LaunchCtx& c) { return run_gemm_q5k_split(c, 0); }
qmm_status run_gemm_q5k_rows2(const LaunchCtx& c) { return run_gemm_q5k_split(c, 2); }
qmm_status run_gemm_q5k_rows3(const LaunchCtx& c) { return run_gemm_q5k_split(c, 3); }
qmm_status run_gemm_q5k_rows4(const LaunchCtx& c) { return run_gemm_q5k_split(c, 4); }
qmm_status run_gemm_q5k_rows5(const LaunchCtx& c) { return run_gemm_q5k_split(c, 5); }

// "dequant_q5k" (not a reference id): buffers W, Out (fp32); scalar nblocks.
qmm_status run_dequant_q5k(const LaunchCtx& c) {
  if (!counts(c, 2, 1)) return bad("dequant_q5k: expects 2 buffers and 1 scalar");
  const uint64_t nb = c.sc[0];
  if (nb == 0 || nb > (1ull << 32)) return bad("dequant_q5k: bad block count");
  if (!c.fits(0, static_cast<u128>(nb) * 176) || !c.fits(1, static_cast<u128>(nb) * 1024)) {
    return bad("dequant_q5k: a buffer is smaller than nblocks requires");
  }
  return map_hip(qmm::launch_dequant_q5k(c.ptr<const uint8_t>(0), c.ptr<float>(1), nb, c.stream));
}

// ---- Q6_K ---------------------------------------------------------------------
// "gemm_q6k", "gemm_q6k_batched": buffers A, W, C; scalars m, n, k, k a multiple of 256
// (include/tessera/backend.hpp:202-206,524-536).  "gemm_q6k_vec", "gemm_q6k_rows{R}": the same
// plus `split`, with the partials contract of the Q4_K ids
// (src/backends/rocm/rocm_backend.cpp:102-108; rocm_kernels_gemv.cpp:19-24,107-156).
u128 q6k_bytes(uint64_t n, uint64_t k) { return static_cast<u128>(n) * (k / 256) * 210; }

qmm_status q6k_matmul(const LaunchCtx& c, uint64_t m, uint64_t n, uint64_t k, uint64_t split, const char* who) {
  if (!dims_ok(m, n, k) || k % 256 != 0) return bad(std::string(who) + ": m, n, k must be non-zero and k a multiple of 256");
  if (split == 0 || split > 64 || (k / 256) % split != 0) return bad(std::string(who) + ": split must divide k/256");
  const u128 region = static_cast<u128>(m) * n * 4;
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, q6k_bytes(n, k)) || !c.fits(2, region * split)) {
    return bad(std::string(who) + ": a buffer is smaller than m, n, k require");
  }
  float* out = c.ptr<float>(2);
  if (m >= kQ4KGemmMinRows && qmm::gemm_kquant_f16_supported(m, n, k)) {
    return kquant_prefill(c, 210, m, n, k, split);
  }
  // From three rows: one pass over the weights for up to four of them on the int8 matrix cores
  // (17408 x 5120: 4 rows 32 us against 52 on multiply-add passes of two rows, 8 rows 61 against 103;
  // two rows stay on the multiply-add pass, 26 against 29 us).
  const bool one_pass = m >= 3 && qmm::gemv_kquant_rows_supported(m, n, k);
  const auto launch = one_pass ? qmm::launch_q6k_rows_i8 : qmm::launch_q6k_gemv;
  qmm_status st = map_hip(launch(c.ptr<const float>(0), c.ptr<const uint8_t>(1), out, static_cast<uint32_t>(m),
                                 static_cast<uint32_t>(n), static_cast<uint32_t>(k), c.stream));
  if (st == QMM_OK && split > 1) st = map_hip(qmm::launch_fill_f32(out + m * n, 0.0f, (split - 1) * m * n, c.stream));
  return st;
}

qmm_status run_gemm_q6k(const LaunchCtx& c) {
  if (!counts(c, 3, 3)) return bad("gemm_q6k: expects 3 buffers and 3 scalars");
  return q6k_matmul(c, c.sc[0], c.sc[1], c.sc[2], 1, "gemm_q6k");
}
qmm_status run_gemm_q6k_split(const LaunchCtx& c, uint64_t rows_required) {
  if (!counts(c, 3, 4)) return bad("gemm_q6k_vec/rows: expects 3 buffers and 4 scalars");
  if (rows_required != 0 && c.sc[0] != rows_required) return bad("gemm_q6k_rowsR: m must equal R");
  return q6k_matmul(c, c.sc[0], c.sc[1], c.sc[2], c.sc[3], "gemm_q6k_vec/rows");
}
qmm_status run_gemm_q6k_vec(const LaunchCtx& c) { return run_gemm_q6k_split(c, 0); }
qmm_status run_gemm_q6k_rows2(const LaunchCtx& c) { return run_gemm_q6k_split(c, 2); }
qmm_status run_gemm_q6k_rows3(const LaunchCtx& c) { return run_gemm_q6k_split(c, 3); }
qmm_status run_gemm_q6k_rows4(const LaunchCtx& c) { return run_gemm_q6k_split(c, 4); }
qmm_status run_gemm_q6k_rows5(const LaunchCtx& c) { return run_gemm_q6k_split(c, 5); }

// "dequant_q6k" (not a reference id): buffers W, Out (fp32); scalar nblocks.
qmm_status run_dequant_q6k(const LaunchCtx& c) {
  if (!counts(c, 2, 1)) return bad("dequant_q6k: expects 2 buffers and 1 scalar");
  const uint64_t nb = c.sc[0];
  if (nb == 0 || nb > (1ull << 32)) return bad("dequant_q6k: bad block count");
  if (!c.fits(0, static_cast<u128>(nb) * 210) || !c.fits(1, static_cast<u128>(nb) * 1024)) {
    return bad("dequant_q6k: a buffer is smaller than nblocks requires");
  }
  return map_hip(qmm::launch_dequant_q6k(c.ptr<const uint8_t>(0), c.ptr<float>(1), nb, c.stream));
}

// ---- MXFP4 / FP8 ---------------------------------------------------------------
// "gemm_mxfp4", "gemm_mxfp4_rows", "gemm_mxfp4_batched": buffers A, W, C; scalars
// m, n, k with k a multiple of 32 (include/tessera/backend.hpp:195-201,513-523;
// src/backends/rocm/rocm_kernels_basic.cpp:1092-1214).
qmm_status run_gemm_mxfp4(const LaunchCtx& c) {
  if (!counts(c, 3, 3)) return bad("gemm_mxfp4: expects 3 buffers and 3 scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], k = c.sc[2];
  if (!dims_ok(m, n, k) || k % 32 != 0) return bad("gemm_mxfp4: m, n, k must be non-zero and k a multiple of 32");
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, mxfp4_bytes(n, k)) ||
      !c.fits(2, static_cast<u128>(m) * n * 4)) {
    return bad("gemm_mxfp4: a buffer is smaller than m, n, k require");
  }
  // From 17 rows on the weights go through the matrix cores as they are (E2M1 operand, E8M0 block
  // scale) and the fp32 rows as a short sum of E4M3 terms (gemm_mxfp4.hip).
  if (m >= kMxfp4GemmMinRows && m <= 0xFFFFFFFFull && n <= 0xFFFFFFFFull && qmm::gemm_mxfp4_f32_supported(m, k)) {
    void* ws = nullptr;
    const qmm_status st = workspace(c, qmm::gemm_mxfp4_f32_workspace_bytes(m, k), &ws);
    if (st != QMM_OK) return st;
    return map_hip(qmm::launch_mxfp4_f32_gemm(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<float>(2), ws,
                                              static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                              static_cast<uint32_t>(k), c.stream));
  }
  // 2..16 rows of a matrix large enough to be worth a second launch: the same terms through the streamed
  // few-row kernel (weights read once per eight rows) instead of four rows a pass on the vector unit.
  if (m >= 2 && m <= 16 && n * k >= kQ4KFewRowsMinWeights && qmm::gemm_mxfp4_f32_rows_supported(m, n, k) &&
      qmm::gemm_mxfp4_f32_rows_workspace_bytes(m, k) <= kDecodeScratchBytes && decode_scratch(c) != nullptr) {
    return map_hip(qmm::launch_mxfp4_f32_rows(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<float>(2),
                                              decode_scratch(c), static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                              static_cast<uint32_t>(k), c.stream));
  }
  return map_hip(qmm::launch_mxfp4_gemv(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<float>(2),
                                        static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                        static_cast<uint32_t>(k), c.stream));
}
qmm_status run_gemm_mxfp4_rows(const LaunchCtx& c) {
  if (c.nsc >= 1 && c.sc[0] > 16) return bad("gemm_mxfp4_rows: m must be 1..16");
  return run_gemm_mxfp4(c);
}

// "mxfp4_row_ref": buffers W, Wref (n bytes); scalars n, k
// (src/backends/rocm/rocm_kernels_basic.cpp:1284-1303).
qmm_status run_mxfp4_row_ref(const LaunchCtx& c) {
  if (!counts(c, 2, 2)) return bad("mxfp4_row_ref: expects 2 buffers and 2 scalars");
  const uint64_t n = c.sc[0], k = c.sc[1];
  if (!dims_ok(1, n, k) || k % 32 != 0) return bad("mxfp4_row_ref: bad n or k");
  if (!c.fits(0, mxfp4_bytes(n, k)) || !c.fits(1, n)) return bad("mxfp4_row_ref: buffer too small");
  return map_hip(qmm::launch_mxfp4_row_ref(c.ptr<const uint8_t>(0), c.ptr<uint8_t>(1), n, k, c.stream));
}

// "gemm_mxfp4_wmma": buffers A (m x k E4M3 codes), W (packed MXFP4), As (m fp32),
// Wref (n bytes), C; scalars m, n, k, split, wperm
// (src/backends/rocm/rocm_kernels_basic.cpp:1310-1493; src/models/qwen3_5/project.cpp:207-215).
// gfx950 multiplies E2M1 by E4M3 natively, so the weights are not folded to E4M3 and
// Wref is unused: the result is As[r] * sum_t e4m3(a_t) * 2^(s-127) * e2m1(w_t), which
// equals the reference's folded result wherever its fold is exact.  Split regions as
// for "gemm_q4k_vec".  wperm (pre-permuted weights) must be 0, as the reference
// always passes.
qmm_status run_gemm_mxfp4_wmma(const LaunchCtx& c) {
  if (!counts(c, 5, 5)) return bad("gemm_mxfp4_wmma: expects 5 buffers and 5 scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], k = c.sc[2], split = c.sc[3], wperm = c.sc[4];
  if (!dims_ok(m, n, k) || k % 32 != 0) return bad("gemm_mxfp4_wmma: bad m, n, k");
  if (split == 0 || split > 64) return bad("gemm_mxfp4_wmma: bad split");
  if (wperm > 1 || (wperm == 1 && (n % 16 != 0 || k % 16 != 0))) {
    return bad("gemm_mxfp4_wmma: wperm is 0 or 1, and fragment-ordered weights have n and k multiples of 16");
  }
  const u128 region = static_cast<u128>(m) * n * 4;
  if (!c.fits(0, static_cast<u128>(m) * k) || !c.fits(1, mxfp4_bytes(n, k)) || !c.fits(2, m * 4) ||
      !c.fits(3, n) || !c.fits(4, region * split)) {
    return bad("gemm_mxfp4_wmma: a buffer is smaller than m, n, k, split require");
  }
  float* out = c.ptr<float>(4);
  const uint8_t* w = c.ptr<const uint8_t>(1);
  if (wperm == 1) {
    // Weights in the reference's fragment order (PermuteMxFp4ToWmma, quant.cpp:926-954): the tiled
    // kernel reads them as they are; the few-row and single-row kernels want row-major runs, so
    // for them the matrix is put back into row-major order in the workspace first.
    if (m <= 0xFFFFFFFFull && n <= 0xFFFFFFFFull && qmm::gemm_mxfp4_a8_wperm_supported(m, n, k)) {
      qmm_status st = map_hip(qmm::launch_mxfp4_a8_gemm_wperm(
          c.ptr<const uint8_t>(0), c.ptr<const float>(2), w, out, static_cast<uint32_t>(m), static_cast<uint32_t>(n),
          static_cast<uint32_t>(k), c.stream));
      if (st == QMM_OK && split > 1) st = map_hip(qmm::launch_fill_f32(out + m * n, 0.0f, (split - 1) * m * n, c.stream));
      return st;
    }
    void* ws = nullptr;
    qmm_status st = workspace(c, static_cast<size_t>(mxfp4_bytes(n, k)), &ws);
    if (st != QMM_OK) return st;
    st = map_hip(qmm::launch_permute_mxfp4_wmma(w, static_cast<uint8_t*>(ws), n, k, true, c.stream));
    if (st != QMM_OK) return st;
    w = static_cast<const uint8_t*>(ws);
  }
  // Regime: a single row stays on the VALU GEMV; from two rows on the scaled MFMA takes over
  // (a streaming kernel up to 32 rows, the tiled GEMM above that).
  // (The streaming kernel would be faster for one row of a wide matrix as well -- 17408 x 5120:
  // 11.1 against 12.4 us -- but its sums do not meet the single row's tolerance against the
  // fp32 reference, so one row keeps the fp32 multiply-adds.)
  if (m > 1 && k >= 1024 && qmm::gemm_mxfp4_a8_supported(k)) {
    qmm_status st = map_hip(qmm::launch_mxfp4_a8_gemm(
        c.ptr<const uint8_t>(0), c.ptr<const float>(2), w, out,
        static_cast<uint32_t>(m), static_cast<uint32_t>(n), static_cast<uint32_t>(k), c.stream));
    if (st == QMM_OK && split > 1) {
      st = map_hip(qmm::launch_fill_f32(out + m * n, 0.0f, (split - 1) * m * n, c.stream));
    }
    return st;
  }
  qmm_status st = map_hip(qmm::launch_mxfp4_a8_gemv(
      c.ptr<const uint8_t>(0), c.ptr<const float>(2), w, out,
      static_cast<uint32_t>(m), static_cast<uint32_t>(n), static_cast<uint32_t>(k), c.stream));
  if (st == QMM_OK && split > 1) {
    st = map_hip(qmm::launch_fill_f32(out + m * n, 0.0f, (split - 1) * m * n, c.stream));
  }
  return st;
}

// "permute_mxfp4_wmma" (not a reference id; the device form of the reference's load-time
// PermuteMxFp4ToWmma, src/core/numerics/quant.cpp:926-954): buffers In, Out (packed MXFP4, n*k/2
// nibble bytes then n*k/32 scale bytes); scalars n, k (multiples of 16 and 32), inverse (0: row-major
// -> fragment order, 1: back).  The scale bytes are copied unchanged.
qmm_status run_permute_mxfp4_wmma(const LaunchCtx& c) {
  if (!counts(c, 2, 3)) return bad("permute_mxfp4_wmma: expects 2 buffers and 3 scalars");
  const uint64_t n = c.sc[0], k = c.sc[1], inverse = c.sc[2];
  if (!dims_ok(1, n, k) || n % 16 != 0 || k % 32 != 0 || inverse > 1) return bad("permute_mxfp4_wmma: n a multiple of 16, k of 32, inverse 0 or 1");
  if (!c.fits(0, mxfp4_bytes(n, k)) || !c.fits(1, mxfp4_bytes(n, k))) return bad("permute_mxfp4_wmma: buffer too small");
  if (c.buf[0] == c.buf[1]) return bad("permute_mxfp4_wmma: not in place");
  return map_hip(qmm::launch_permute_mxfp4_wmma(c.ptr<const uint8_t>(0), c.ptr<uint8_t>(1), n, k, inverse == 1, c.stream));
}

// "permute_q4k_rowgroup" (not a reference id; the Q4_K counterpart of the hook above, for this part's
// int8 matrix instruction): buffers In, Out (n x k/256 Q4_K blocks each); scalars n, k, rows per group
// (1..64; 0 = the default, 32), inverse (0: GGUF order -> row groups, 1: back).
qmm_status run_permute_q4k_rowgroup(const LaunchCtx& c) {
  if (!counts(c, 2, 4)) return bad("permute_q4k_rowgroup: expects 2 buffers and 4 scalars");
  const uint64_t n = c.sc[0], k = c.sc[1], inverse = c.sc[3];
  const uint64_t rows = c.sc[2] == 0 ? qmm::q4k_rowgroup_default_rows(n) : c.sc[2];
  if (!dims_ok(1, n, k) || k % 256 != 0 || inverse > 1 || !qmm::q4k_rowgroup_supported(n, k, rows)) {
    return bad("permute_q4k_rowgroup: k a multiple of 256, 1..64 rows per group, inverse 0 or 1");
  }
  if (!c.fits(0, q4k_bytes(n, k)) || !c.fits(1, q4k_bytes(n, k))) return bad("permute_q4k_rowgroup: buffer too small");
  if (c.buf[0] == c.buf[1]) return bad("permute_q4k_rowgroup: not in place");
  return map_hip(qmm::launch_q4k_rowgroup(c.ptr<const uint8_t>(0), c.ptr<uint8_t>(1), static_cast<uint32_t>(n),
                                          static_cast<uint32_t>(k), static_cast<uint32_t>(rows), inverse == 1, c.stream));
}

// "dequant_mxfp4" (not a reference id): buffers W (packed), Out (n x k fp32); scalars n, k.
qmm_status run_dequant_mxfp4(const LaunchCtx& c) {
  if (!counts(c, 2, 2)) return bad("dequant_mxfp4: expects 2 buffers and 2 scalars");
  const uint64_t n = c.sc[0], k = c.sc[1];
  if (!dims_ok(1, n, k) || k % 32 != 0) return bad("dequant_mxfp4: bad n or k");
  if (!c.fits(0, mxfp4_bytes(n, k)) || !c.fits(1, static_cast<u128>(n) * k * 4)) return bad("dequant_mxfp4: buffer too small");
  return map_hip(qmm::launch_dequant_mxfp4(c.ptr<const uint8_t>(0), c.ptr<float>(1), n, k, c.stream));
}

// "quantize_fp8": buffers data (rows x cols fp32, in place), scale; scalars rows, cols
// (include/tessera/backend.hpp:296-302,715-722).
qmm_status run_quantize_fp8(const LaunchCtx& c) {
  if (!counts(c, 2, 2)) return bad("quantize_fp8: expects 2 buffers and 2 scalars");
  const uint64_t rows = c.sc[0], cols = c.sc[1];
  if (!dims_ok(rows, 1, cols)) return bad("quantize_fp8: rows and cols must be non-zero");
  if (!c.fits(0, static_cast<u128>(rows) * cols * 4) || !c.fits(1, static_cast<u128>(rows) * 4)) return bad("quantize_fp8: buffer too small");
  return map_hip(qmm::launch_quantize_fp8(c.ptr<float>(0), c.ptr<float>(1), rows, cols, c.stream));
}

// "quantize_fp8_pack" / "quantize_fp8_pack_rows": buffers In (fp32), Out (codes), scale;
// scalars rows, cols with cols a multiple of 4 (include/tessera/backend.hpp:303-307,723-730).
qmm_status run_quantize_fp8_pack(const LaunchCtx& c) {
  if (!counts(c, 3, 2)) return bad("quantize_fp8_pack: expects 3 buffers and 2 scalars");
  const uint64_t rows = c.sc[0], cols = c.sc[1];
  if (!dims_ok(rows, 1, cols) || cols % 4 != 0) return bad("quantize_fp8_pack: cols must be a non-zero multiple of 4");
  if (!c.fits(0, static_cast<u128>(rows) * cols * 4) || !c.fits(1, static_cast<u128>(rows) * cols) ||
      !c.fits(2, static_cast<u128>(rows) * 4)) {
    return bad("quantize_fp8_pack: buffer too small");
  }
  return map_hip(qmm::launch_quantize_fp8_pack(c.ptr<const float>(0), c.ptr<uint8_t>(1), c.ptr<float>(2), rows, cols, c.stream));
}

// "quantize_fp8_pack_a16" (not a reference id): as "quantize_fp8_pack" with bf16 input.
qmm_status run_quantize_fp8_pack_a16(const LaunchCtx& c) {
  if (!counts(c, 3, 2)) return bad("quantize_fp8_pack_a16: expects 3 buffers and 2 scalars");
  const uint64_t rows = c.sc[0], cols = c.sc[1];
  if (!dims_ok(rows, 1, cols) || cols % 4 != 0) return bad("quantize_fp8_pack_a16: cols must be a non-zero multiple of 4");
  if (!c.fits(0, static_cast<u128>(rows) * cols * 2) || !c.fits(1, static_cast<u128>(rows) * cols) ||
      !c.fits(2, static_cast<u128>(rows) * 4)) {
    return bad("quantize_fp8_pack_a16: buffer too small");
  }
  return map_hip(qmm::launch_quantize_fp8_pack_bf16(c.ptr<const uint16_t>(0), c.ptr<uint8_t>(1), c.ptr<float>(2), rows, cols, c.stream));
}

// "gemm_fp8": buffers A, W (n x k E4M3 bytes), S (n fp32), C; scalars m, n, k
// (include/tessera/backend.hpp:191-194,504-512).
qmm_status run_gemm_fp8(const LaunchCtx& c) {
  if (!counts(c, 4, 3)) return bad("gemm_fp8: expects 4 buffers and 3 scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], k = c.sc[2];
  if (!dims_ok(m, n, k)) return bad("gemm_fp8: m, n, k must be non-zero");
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, static_cast<u128>(n) * k) ||
      !c.fits(2, static_cast<u128>(n) * 4) || !c.fits(3, static_cast<u128>(m) * n * 4)) {
    return bad("gemm_fp8: a buffer is smaller than m, n, k require");
  }
  // 2..16 rows of a large matrix: the weights through the matrix cores as they are (E4M3 operand), the
  // fp32 rows as E4M3 terms, weights read once per eight rows (gemm_mxfp4.hip).
  if (m >= 2 && m <= 16 && n * k >= kQ4KFewRowsMinWeights && qmm::gemm_fp8_f32_rows_supported(m, n, k) &&
      qmm::gemm_mxfp4_f32_rows_workspace_bytes(m, k) <= kDecodeScratchBytes && decode_scratch(c) != nullptr) {
    return map_hip(qmm::launch_fp8_f32_rows(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const float>(2),
                                            c.ptr<float>(3), decode_scratch(c), static_cast<uint32_t>(m),
                                            static_cast<uint32_t>(n), static_cast<uint32_t>(k), false, c.stream));
  }
  return map_hip(qmm::launch_fp8_gemv(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const float>(2),
                                      c.ptr<float>(3), static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                      static_cast<uint32_t>(k), c.stream));
}

// "gemm_fp8_block": buffers A, W (n x k E4M3 bytes), S ((n/128) x (k/128) fp32 block scales), C;
// scalars m, n, k with n and k multiples of 128 (include/tessera/backend.hpp:183-186,476-485;
// reference kernel src/backends/rocm/rocm_kernels_basic.cpp:1066-1089).
qmm_status run_gemm_fp8_block(const LaunchCtx& c) {
  if (!counts(c, 4, 3)) return bad("gemm_fp8_block: expects 4 buffers and 3 scalars");
  const uint64_t m = c.sc[0], n = c.sc[1], k = c.sc[2];
  if (!dims_ok(m, n, k) || n % 128 != 0 || k % 128 != 0) return bad("gemm_fp8_block: m, n, k must be non-zero, n and k multiples of 128");
  if (!c.fits(0, static_cast<u128>(m) * k * 4) || !c.fits(1, static_cast<u128>(n) * k) ||
      !c.fits(2, static_cast<u128>(n / 128) * (k / 128) * 4) || !c.fits(3, static_cast<u128>(m) * n * 4)) {
    return bad("gemm_fp8_block: a buffer is smaller than m, n, k require");
  }
  // 2..16 rows of a large matrix: the matrix cores as for gemm_fp8, an instruction's sum (128 of K: one
  // block column) times the block's scale
  if (m >= 2 && m <= 16 && n * k >= kQ4KFewRowsMinWeights && qmm::gemm_fp8_f32_rows_supported(m, n, k) &&
      qmm::gemm_mxfp4_f32_rows_workspace_bytes(m, k) <= kDecodeScratchBytes && decode_scratch(c) != nullptr) {
    return map_hip(qmm::launch_fp8_f32_rows(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const float>(2),
                                            c.ptr<float>(3), decode_scratch(c), static_cast<uint32_t>(m),
                                            static_cast<uint32_t>(n), static_cast<uint32_t>(k), true, c.stream));
  }
  return map_hip(qmm::launch_fp8_block_gemv(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const float>(2),
                                            c.ptr<float>(3), static_cast<uint32_t>(m), static_cast<uint32_t>(n),
                                            static_cast<uint32_t>(k), c.stream));
}

// "moe_scale_add": buffers a, b, f, o; scalars n, idx
// (src/backends/rocm/rocm_kernels_basic.cpp:1932-1942).
qmm_status run_moe_scale_add(const LaunchCtx& c) {
  if (!counts(c, 4, 2)) return bad("moe_scale_add: expects 4 buffers and 2 scalars");
  const uint64_t n = c.sc[0], idx = c.sc[1];
  if (n == 0 || n > (1ull << 40)) return bad("moe_scale_add: bad n");
  if (!c.fits(0, static_cast<u128>(n) * 4) || !c.fits(1, static_cast<u128>(n) * 4) ||
      !c.fits(2, (static_cast<u128>(idx) + 1) * 4) || !c.fits(3, static_cast<u128>(n) * 4)) {
    return bad("moe_scale_add: buffer too small");
  }
  return map_hip(qmm::launch_moe_scale_add(c.ptr<const float>(0), c.ptr<const float>(1), c.ptr<const float>(2),
                                           c.ptr<float>(3), n, idx, c.stream));
}

// ---- routed experts ------------------------------------------------------------------
// "moe_experts_gate_up_q4k": buffers x, gate, up, ids, phi; scalars hidden, inter, top_k,
// gate_stride, up_stride (src/backends/rocm/rocm_kernels_moe.cpp:15-47;
// src/models/qwen3_5/moe.cpp:396-404).  "..._rows" (not a reference id) adds a trailing
// scalar `rows`: x is rows x hidden, ids rows x top_k, phi rows x top_k x inter, one token
// per row in a single launch.
constexpr uint64_t kMoeGroupedMinRows = 17;   // as kQ4KGemmMinRows: past the largest speculative-verify batch

qmm_status run_moe_gate_up_n(const LaunchCtx& c, bool batched) {
  if (!counts(c, 5, batched ? 6 : 5)) return bad("moe_experts_gate_up_q4k: expects 5 buffers and 5 (6) scalars");
  const uint64_t hidden = c.sc[0], inter = c.sc[1], top_k = c.sc[2], gs = c.sc[3], us = c.sc[4];
  const uint64_t rows = batched ? c.sc[5] : 1;
  if (hidden == 0 || inter == 0 || hidden % 256 != 0 || inter % 256 != 0 || hidden > (1u << 20) ||
      inter > (1u << 20) || top_k == 0 || top_k > 64 || rows == 0 || rows > 65535) {
    return bad("moe_experts_gate_up_q4k: bad hidden, inter, top_k or rows");
  }
  const u128 expert = q4k_bytes(inter, hidden);
  if (gs < expert || us < expert) return bad("moe_experts_gate_up_q4k: expert stride smaller than one expert");
  if (!c.fits(0, static_cast<u128>(rows) * hidden * 4) || !c.fits(1, expert) || !c.fits(2, expert) ||
      !c.fits(3, static_cast<u128>(rows) * top_k * 4) || !c.fits(4, static_cast<u128>(rows) * top_k * inter * 4)) {
    return bad("moe_experts_gate_up_q4k: a buffer is smaller than the shape requires");
  }
  // Experts the smaller of the two tensors holds (all of them when sizes were not given).
  uint64_t experts = 0xFFFFFFFFull;
  if (c.bytes != nullptr) {
    const uint64_t eg = (c.bytes[1] - static_cast<uint64_t>(expert)) / gs + 1, eu = (c.bytes[2] - static_cast<uint64_t>(expert)) / us + 1;
    experts = eg < eu ? eg : eu;
    if (experts > 0xFFFFFFFFull) experts = 0xFFFFFFFFull;
  }
  // A chunk of tokens (prefill): grouped by expert on the MFMA path, each expert's weights read
  // once per launch; that overtakes one exact pass per token at about 16 tokens (256 experts,
  // top-8: 89 against 81 us).
  if (batched && rows >= kMoeGroupedMinRows && c.bytes != nullptr && rows * top_k <= (1u << 20) &&
      qmm::moe_ffn_q4k_supported(hidden, inter, experts)) {
    void* ws = nullptr;
    const qmm_status st = workspace(c, qmm::moe_ffn_q4k_workspace_bytes(rows * top_k, hidden, inter, experts), &ws);
    if (st != QMM_OK) return st;
    return map_hip(qmm::launch_moe_gate_up_q4k_grouped(
        c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const uint8_t>(2), c.ptr<const uint32_t>(3), c.ptr<float>(4),
        ws, static_cast<uint32_t>(hidden), static_cast<uint32_t>(inter), static_cast<uint32_t>(top_k), gs, us,
        static_cast<uint32_t>(experts), static_cast<uint32_t>(rows), c.stream));
  }
  return map_hip(qmm::launch_moe_gate_up_q4k(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const uint8_t>(2),
                                             c.ptr<const uint32_t>(3), c.ptr<float>(4), static_cast<uint32_t>(hidden),
                                             static_cast<uint32_t>(inter), static_cast<uint32_t>(top_k), gs, us,
                                             static_cast<uint32_t>(experts), static_cast<uint32_t>(rows), c.stream));
}
qmm_status run_moe_gate_up(const LaunchCtx& c) { return run_moe_gate_up_n(c, false); }
qmm_status run_moe_gate_up_rows(const LaunchCtx& c) { return run_moe_gate_up_n(c, true); }

// "moe_experts_down_q4k": buffers phi, down, ids, wts, out; scalars hidden, inter, top_k,
// down_stride, accumulate (src/backends/rocm/rocm_kernels_moe.cpp:49-79;
// src/models/qwen3_5/moe.cpp:413-423).  "..._rows" adds a trailing `rows` as above.
qmm_status run_moe_down_n(const LaunchCtx& c, bool batched, bool q6k) {
  const char* who = q6k ? "moe_experts_down_q6k" : "moe_experts_down_q4k";
  if (!counts(c, 5, batched ? 6 : 5)) return bad(std::string(who) + ": expects 5 buffers and 5 (6) scalars");
  const uint64_t hidden = c.sc[0], inter = c.sc[1], top_k = c.sc[2], ds = c.sc[3], acc = c.sc[4];
  const uint64_t rows = batched ? c.sc[5] : 1;
  if (hidden == 0 || inter == 0 || inter % 256 != 0 || hidden > (1u << 24) || inter > (1u << 20) ||
      top_k == 0 || top_k > 64 || top_k * inter / 32 > 32768 || rows == 0 || rows > 65535) {
    return bad(std::string(who) + ": bad hidden, inter, top_k or rows");
  }
  const u128 expert_bytes = q6k ? q6k_bytes(hidden, inter) : q4k_bytes(hidden, inter);
  if (ds < expert_bytes) return bad(std::string(who) + ": expert stride smaller than one expert");
  if (!c.fits(0, static_cast<u128>(rows) * top_k * inter * 4) || !c.fits(1, expert_bytes) ||
      !c.fits(2, static_cast<u128>(rows) * top_k * 4) || !c.fits(3, static_cast<u128>(rows) * top_k * 4) ||
      !c.fits(4, static_cast<u128>(rows) * hidden * 4)) {
    return bad(std::string(who) + ": a buffer is smaller than the shape requires");
  }
  // The expert ids are clamped to the tensor and the kernels address it with 32-bit offsets, so
  // the tensor's size must be known and below 4 GB.
  if (c.bytes == nullptr) return bad(std::string(who) + ": buffer sizes are required (they bound the expert ids)");
  if (c.bytes[1] >= (1ull << 32)) {
    g_last_error = std::string(who) + ": expert tensors of 4 GB and more are not implemented";
    return QMM_UNSUPPORTED_FEATURE;
  }
  const uint64_t experts = (c.bytes[1] - static_cast<uint64_t>(expert_bytes)) / ds + 1;
  if (!q6k && batched && rows >= kMoeGroupedMinRows && rows * top_k <= (1u << 20) &&
      qmm::moe_ffn_q4k_supported(hidden, inter, experts)) {
    void* ws = nullptr;
    const qmm_status st = workspace(c, qmm::moe_ffn_q4k_workspace_bytes(rows * top_k, hidden, inter, experts), &ws);
    if (st != QMM_OK) return st;
    return map_hip(qmm::launch_moe_down_q4k_grouped(
        c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const uint32_t>(2), c.ptr<const float>(3), c.ptr<float>(4), ws,
        static_cast<uint32_t>(hidden), static_cast<uint32_t>(inter), static_cast<uint32_t>(top_k), ds,
        static_cast<uint32_t>(experts), static_cast<uint32_t>(rows), acc != 0, c.stream));
  }
  const auto launch = q6k ? qmm::launch_moe_down_q6k : qmm::launch_moe_down_q4k;
  return map_hip(launch(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const uint32_t>(2),
                        c.ptr<const float>(3), c.ptr<float>(4), static_cast<uint32_t>(hidden),
                        static_cast<uint32_t>(inter), static_cast<uint32_t>(top_k), ds, acc != 0,
                        static_cast<uint32_t>(experts), static_cast<uint32_t>(rows), c.stream));
}
qmm_status run_moe_down(const LaunchCtx& c) { return run_moe_down_n(c, false, false); }
qmm_status run_moe_down_rows(const LaunchCtx& c) { return run_moe_down_n(c, true, false); }
// "moe_experts_down_q6k": the same contract with Q6_K expert tensors
// (src/backends/rocm/rocm_kernels_moe.cpp:81-110).
qmm_status run_moe_down_q6k(const LaunchCtx& c) { return run_moe_down_n(c, false, true); }
qmm_status run_moe_down_q6k_rows(const LaunchCtx& c) { return run_moe_down_n(c, true, true); }

// "moe_gate": buffers vals (top_k), x, w (hidden), wts (top_k), sig (1); scalars top_k, hidden
// (src/backends/rocm/rocm_kernels_basic.cpp:1896-1929).
qmm_status run_moe_gate(const LaunchCtx& c) {
  if (!counts(c, 5, 2)) return bad("moe_gate: expects 5 buffers and 2 scalars");
  const uint64_t top_k = c.sc[0], hidden = c.sc[1];
  if (top_k == 0 || top_k > 4096 || hidden == 0 || hidden > (1u << 24)) return bad("moe_gate: bad top_k or hidden");
  if (!c.fits(0, top_k * 4) || !c.fits(1, hidden * 4) || !c.fits(2, hidden * 4) || !c.fits(3, top_k * 4) ||
      !c.fits(4, 4)) {
    return bad("moe_gate: buffer too small");
  }
  return map_hip(qmm::launch_moe_gate(c.ptr<const float>(0), c.ptr<const float>(1), c.ptr<const float>(2),
                                      c.ptr<float>(3), c.ptr<float>(4), static_cast<uint32_t>(top_k),
                                      static_cast<uint32_t>(hidden), c.stream));
}

// "top_k_rows": buffers logits, ids, vals; scalars rows, vocab, top_k, row_base
// (src/backends/rocm/rocm_kernels_basic.cpp:3170-3243; top_k is at most 32 there).
qmm_status run_top_k_rows(const LaunchCtx& c) {
  if (!counts(c, 3, 4)) return bad("top_k_rows: expects 3 buffers and 4 scalars");
  const uint64_t rows = c.sc[0], vocab = c.sc[1], top_k = c.sc[2], base = c.sc[3];
  if (rows == 0 || rows > kMaxDim || vocab == 0 || vocab > kMaxDim || top_k == 0 || top_k > 32 || top_k > vocab ||
      base > kMaxDim) {
    return bad("top_k_rows: bad rows, vocab, top_k (1..32) or row_base");
  }
  if (!c.fits(0, static_cast<u128>(base + rows) * vocab * 4) || !c.fits(1, static_cast<u128>(rows) * top_k * 4) ||
      !c.fits(2, static_cast<u128>(rows) * top_k * 4)) {
    return bad("top_k_rows: buffer too small");
  }
  return map_hip(qmm::launch_top_k_rows(c.ptr<const float>(0), c.ptr<uint32_t>(1), c.ptr<float>(2),
                                        static_cast<uint32_t>(rows), vocab, static_cast<uint32_t>(top_k), base,
                                        c.stream));
}

// "moe_experts_ffn_q4k_rows" (not a reference id): the routed-expert feed-forward of a chunk
// of tokens in one call, tokens grouped by expert.  Buffers x (rows x hidden), gate, up, down
// (expert tensors), ids, wts (rows x top_k), out (rows x hidden); scalars hidden, inter, top_k,
// gate_stride, up_stride, down_stride, rows, accumulate.  Same result as gate_up_rows followed
// by down_rows, on the fp16 MFMA path (bound as for the Q4_K prefill GEMM).
qmm_status run_moe_ffn_rows(const LaunchCtx& c) {
  if (!counts(c, 7, 8)) return bad("moe_experts_ffn_q4k_rows: expects 7 buffers and 8 scalars");
  const uint64_t hidden = c.sc[0], inter = c.sc[1], top_k = c.sc[2], gs = c.sc[3], us = c.sc[4], ds = c.sc[5];
  const uint64_t rows = c.sc[6], acc = c.sc[7];
  if (c.bytes == nullptr) return bad("moe_experts_ffn_q4k_rows: buffer sizes are required (they bound the expert ids)");
  if (hidden == 0 || inter == 0 || top_k == 0 || top_k > 64 || rows == 0 || rows * top_k > (1u << 20)) {
    return bad("moe_experts_ffn_q4k_rows: bad hidden, inter, top_k or rows");
  }
  const u128 eg = q4k_bytes(inter, hidden), ed = q4k_bytes(hidden, inter);
  if (hidden % 256 != 0 || inter % 256 != 0 || gs < eg || us < eg || ds < ed) {
    return bad("moe_experts_ffn_q4k_rows: shapes must be multiples of 256 and strides hold one expert");
  }
  if (!c.fits(0, static_cast<u128>(rows) * hidden * 4) || !c.fits(1, eg) || !c.fits(2, eg) || !c.fits(3, ed) ||
      !c.fits(4, static_cast<u128>(rows) * top_k * 4) || !c.fits(5, static_cast<u128>(rows) * top_k * 4) ||
      !c.fits(6, static_cast<u128>(rows) * hidden * 4)) {
    return bad("moe_experts_ffn_q4k_rows: a buffer is smaller than the shape requires");
  }
  uint64_t experts = (c.bytes[1] - static_cast<uint64_t>(eg)) / gs + 1;
  const uint64_t eu = (c.bytes[2] - static_cast<uint64_t>(eg)) / us + 1, edn = (c.bytes[3] - static_cast<uint64_t>(ed)) / ds + 1;
  experts = experts < eu ? experts : eu;
  experts = experts < edn ? experts : edn;
  if (!qmm::moe_ffn_q4k_supported(hidden, inter, experts)) {
    g_last_error = "moe_experts_ffn_q4k_rows: more than 1024 experts or a dimension above 65536 is not implemented";
    return QMM_UNSUPPORTED_FEATURE;
  }
  void* ws = nullptr;
  const qmm_status st = workspace(c, qmm::moe_ffn_q4k_workspace_bytes(rows * top_k, hidden, inter, experts), &ws);
  if (st != QMM_OK) return st;
  return map_hip(qmm::launch_moe_ffn_q4k(c.ptr<const float>(0), c.ptr<const uint8_t>(1), c.ptr<const uint8_t>(2),
                                         c.ptr<const uint8_t>(3), c.ptr<const uint32_t>(4), c.ptr<const float>(5),
                                         c.ptr<float>(6), ws, static_cast<uint32_t>(hidden), static_cast<uint32_t>(inter),
                                         static_cast<uint32_t>(top_k), gs, us, ds, static_cast<uint32_t>(experts),
                                         static_cast<uint32_t>(rows), acc != 0, c.stream));
}

struct Entry {
  const char* id;
  qmm_fn fn;
};

const Entry kTable[] = {
    {"gemm_q4k", run_gemm_q4k},
    {"gemm_q4k_row", run_gemm_q4k},
    {"gemm_q4k_batched", run_gemm_q4k},
    {"gemm_q4k_wmma", run_gemm_q4k_wmma},
    {"gemm_q4k_vec", run_gemm_q4k_vec},
    {"gemm_q4k_rows2", run_gemm_q4k_rows2},
    {"gemm_q4k_rows3", run_gemm_q4k_rows3},
    {"gemm_q4k_rows4", run_gemm_q4k_rows4},
    {"gemm_q4k_rows5", run_gemm_q4k_rows5},
    {"gemm_vec_reduce", run_vec_reduce},
    {"silu_mul", run_silu_mul},
    {"add", run_add},
    {"fill", run_fill},
    {"read_probe", run_read_probe},
    {"mfma_probe", run_mfma_probe},
    {"rmsnorm", run_rmsnorm},
    {"rope", run_rope},
    {"mrope", run_mrope},
    {"attention", run_attention},
    {"attention_q8", run_attention_q8},
    {"attention_q4", run_attention_q4},
    {"attention_fp8", run_attention_fp8},
    {"attention_split", run_attention_split},
    {"attention_split_gqa", run_attention_split_gqa},
    {"attention_q8_split", run_attention_q8_split},
    {"attention_q4_split", run_attention_q4_split},
    {"attention_fp8_split", run_attention_fp8_split},
    {"attention_combine", run_attention_combine},
    {"quantize_q8", run_quantize_q8},
    {"quantize_q4", run_quantize_q4},
    {"cast_f32_f16", run_cast_f32_f16},
    {"qgate_split", run_qgate_split},
    {"embedding_f32", run_embedding_f32},
    {"embedding_bf16", run_embedding_bf16},
    {"embedding_q4k", run_embedding_q4k},
    {"round_bf16", run_round_bf16},
    {"ffn_gate_up_silu_q4k", run_ffn_gate_up_silu_q4k},
    {"gemm_mxfp4", run_gemm_mxfp4},
    {"gemm_mxfp4_rows", run_gemm_mxfp4_rows},
    {"gemm_mxfp4_batched", run_gemm_mxfp4},
    {"mxfp4_row_ref", run_mxfp4_row_ref},
    {"gemm_mxfp4_wmma", run_gemm_mxfp4_wmma},
    {"gemm_mxfp4_wmma_reduce", run_vec_reduce},
    {"quantize_fp8", run_quantize_fp8},
    {"quantize_fp8_pack", run_quantize_fp8_pack},
    {"quantize_fp8_pack_rows", run_quantize_fp8_pack},
    {"gemm_fp8", run_gemm_fp8},
    {"gemm_fp8_block", run_gemm_fp8_block},
    {"moe_scale_add", run_moe_scale_add},
    {"moe_experts_gate_up_q4k", run_moe_gate_up},
    {"moe_experts_down_q4k", run_moe_down},
    {"moe_experts_gate_up_q4k_rows", run_moe_gate_up_rows},
    {"moe_experts_down_q4k_rows", run_moe_down_rows},
    {"moe_experts_down_q6k", run_moe_down_q6k},
    {"moe_experts_down_q6k_rows", run_moe_down_q6k_rows},
    {"moe_experts_ffn_q4k_rows", run_moe_ffn_rows},
    {"moe_gate", run_moe_gate},
    {"top_k_rows", run_top_k_rows},
    {"dequant_q4k", run_dequant_q4k},
    {"gemm_q5k", run_gemm_q5k},
    {"gemm_q5k_batched", run_gemm_q5k},
    {"gemm_q5k_wmma", run_gemm_q5k},
    {"gemm_q5k_vec", run_gemm_q5k_vec},
    {"gemm_q5k_rows2", run_gemm_q5k_rows2},
    {"gemm_q5k_rows3", run_gemm_q5k_rows3},
    {"gemm_q5k_rows4", run_gemm_q5k_rows4},
    {"gemm_q5k_rows5", run_gemm_q5k_rows5},
    {"dequant_q5k", run_dequant_q5k},
    {"gemm_q6k", run_gemm_q6k},
    {"gemm_q6k_batched", run_gemm_q6k},
    {"gemm_q6k_wmma", run_gemm_q6k},
    {"gemm_q6k_vec", run_gemm_q6k_vec},
    {"gemm_q6k_rows2", run_gemm_q6k_rows2},
    {"gemm_q6k_rows3", run_gemm_q6k_rows3},
    {"gemm_q6k_rows4", run_gemm_q6k_rows4},
    {"gemm_q6k_rows5", run_gemm_q6k_rows5},
    {"dequant_q6k", run_dequant_q6k},
    {"dequant_mxfp4", run_dequant_mxfp4},
    {"permute_mxfp4_wmma", run_permute_mxfp4_wmma},
    {"permute_q4k_rowgroup", run_permute_q4k_rowgroup},
    {"quantize_fp8_pack_a16", run_quantize_fp8_pack_a16},
};
constexpr size_t kTableSize = sizeof(kTable) / sizeof(kTable[0]);

}  // namespace

extern "C" {

qmm_status qmm_init(int device) {
  std::lock_guard<std::mutex> lock(g_init_mutex);
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess) return map_hip(e) == QMM_INVALID_ARGUMENT ? QMM_DEVICE_ERROR : map_hip(e);
  if (device < 0 || device >= count) return bad("qmm_init: device index out of range");
  if (g_device == device) return QMM_OK;
  if ((e = hipSetDevice(device)) != hipSuccess) return map_hip(e);
  hipDeviceProp_t prop;
  if ((e = hipGetDeviceProperties(&prop, device)) != hipSuccess) return map_hip(e);
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    g_last_error = std::string("qmm_init: device is ") + prop.gcnArchName + ", this library holds gfx950 code only";
    return QMM_UNSUPPORTED_FEATURE;
  }
  g_device_name = prop.name[0] != '\0' ? prop.name : prop.gcnArchName;   // some hosts report no marketing name
  qmm::set_num_cus(prop.multiProcessorCount);
  g_device = device;
  if (device < kMaxDevices && g_static_scratch[device] == nullptr) {
    // Each device holds its own copy of the array at its own address; `device` is current here.
    void* p = nullptr;
    if ((e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) != hipSuccess) {
      g_device = -1;
      return map_hip(e);
    }
    g_static_scratch[device] = p;
  }
  if ((e = qmm::gemv_q4k_rows16_prepare()) != hipSuccess || (e = qmm::moe_q4k_prepare()) != hipSuccess ||
      (e = qmm::gemv_kquant_rows_prepare()) != hipSuccess || (e = qmm::gemm_fp8_f32_rows_prepare()) != hipSuccess) {
    g_device = -1;
    return map_hip(e);
  }
  if (g_decode_scratch == nullptr) {
    if ((e = hipMalloc(&g_decode_scratch, kDecodeScratchBytes)) != hipSuccess) {
      g_decode_scratch = nullptr;
      g_device = -1;
      return map_hip(e);
    }
  }
  return QMM_OK;
}

const char* qmm_device_name(void) { return g_device_name.c_str(); }

qmm_status qmm_memory_info(uint64_t* total_bytes, uint64_t* free_bytes) {
  if (total_bytes == nullptr || free_bytes == nullptr) return bad("qmm_memory_info: null output");
  size_t f = 0, t = 0;
  const hipError_t e = hipMemGetInfo(&f, &t);
  if (e != hipSuccess) return map_hip(e);
  *total_bytes = t;
  *free_bytes = f;
  return QMM_OK;
}

qmm_status qmm_alloc(size_t bytes, void** out_device_ptr) {
  if (bytes == 0 || out_device_ptr == nullptr) return bad("qmm_alloc: zero bytes or null output");
  void* p = nullptr;
  const hipError_t e = hipMalloc(&p, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return map_hip(e);
  }
  *out_device_ptr = p;
  return QMM_OK;
}

qmm_status qmm_free(void* device_ptr) {
  if (device_ptr == nullptr) return QMM_OK;
  return map_hip(hipFree(device_ptr));
}

qmm_status qmm_copy_h2d(void* dst_device, const void* src_host, size_t bytes, void* stream) {
  if (bytes == 0) return QMM_OK;
  if (dst_device == nullptr || src_host == nullptr) return bad("qmm_copy_h2d: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  return map_hip(e);
}

qmm_status qmm_copy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream) {
  if (bytes == 0) return QMM_OK;
  if (dst_host == nullptr || src_device == nullptr) return bad("qmm_copy_d2h: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e = hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  return map_hip(e);
}

qmm_status qmm_copy_d2d(void* dst_device, const void* src_device, size_t bytes, void* stream) {
  if (bytes == 0) return QMM_OK;
  if (dst_device == nullptr || src_device == nullptr) return bad("qmm_copy_d2d: null pointer");
  return map_hip(hipMemcpyAsync(dst_device, src_device, bytes, hipMemcpyDeviceToDevice,
                                static_cast<hipStream_t>(stream)));
}

qmm_status qmm_load(const char* id, qmm_kernel* out) {
  if (id == nullptr || out == nullptr) return bad("qmm_load: null argument");
  for (size_t i = 0; i < kTableSize; ++i) {
    if (std::strcmp(kTable[i].id, id) == 0) {
      *out = static_cast<qmm_kernel>(i + 1);
      return QMM_OK;
    }
  }
  *out = 0;
  g_last_error = std::string("qmm_load: no built-in named ") + id;
  return QMM_UNSUPPORTED_FEATURE;
}

const char* qmm_kernel_id(qmm_kernel kernel) {
  return (kernel == 0 || kernel > kTableSize) ? nullptr : kTable[kernel - 1].id;
}

size_t qmm_kernel_count(void) { return kTableSize; }

const char* qmm_kernel_name(size_t index) { return index < kTableSize ? kTable[index].id : nullptr; }

namespace {

qmm_status launch_checked(qmm_kernel kernel, const uint32_t grid[3], const uint32_t block[3],
                          void* const* buffers, const size_t* buf_bytes, size_t nbuffers,
                          const uint64_t* scalars, size_t nscalars, void* stream, bool no_alloc) {
  if (kernel == 0 || kernel > kTableSize) return bad("qmm_launch: bad kernel handle");
  if (grid == nullptr || block == nullptr) return bad("qmm_launch: null grid or block");
  for (int i = 0; i < 3; ++i) {
    if (grid[i] == 0 || block[i] == 0) return bad("qmm_launch: zero grid or block dimension");
  }
  if (nbuffers > QMM_MAX_BOUND_BUFFERS || nscalars > QMM_MAX_SCALARS) return bad("qmm_launch: too many buffers or scalars");
  if ((nbuffers != 0 && buffers == nullptr) || (nscalars != 0 && scalars == nullptr)) return bad("qmm_launch: null argument array");
  for (size_t i = 0; i < nbuffers; ++i) {
    if (buffers[i] == nullptr) return bad("qmm_launch: null buffer");
    // The kernels use 16-byte vector and direct-to-LDS loads from the start of each operand;
    // device allocations are aligned far beyond that, a pointer into the middle of one may not be.
    if (reinterpret_cast<uintptr_t>(buffers[i]) % 16 != 0) return bad("qmm_launch: buffers must be 16-byte aligned");
  }
  if (g_device < 0) {
    g_last_error = "qmm_launch: qmm_init has not succeeded";
    return QMM_DEVICE_ERROR;
  }
  if (no_alloc && (g_device >= kMaxDevices || g_static_scratch[g_device] == nullptr)) {
    g_last_error = "qmm_launch_static: the static scratch was not resolved on this device";
    return QMM_DEVICE_ERROR;
  }
  if (t_device != g_device) {  // callers may hop threads; HIP's current device is per thread
    const hipError_t e = hipSetDevice(g_device);
    if (e != hipSuccess) return map_hip(e);
    t_device = g_device;
  }
  const LaunchCtx ctx{buffers, buf_bytes, nbuffers, scalars, nscalars, static_cast<hipStream_t>(stream), no_alloc};
  return kTable[kernel - 1].fn(ctx);
}

}  // namespace

qmm_status qmm_launch(qmm_kernel kernel, const uint32_t grid[3], const uint32_t block[3],
                      void* const* buffers, const size_t* buf_bytes, size_t nbuffers,
                      const uint64_t* scalars, size_t nscalars, void* stream) {
  return launch_checked(kernel, grid, block, buffers, buf_bytes, nbuffers, scalars, nscalars, stream, false);
}

qmm_status qmm_launch_static(qmm_kernel kernel, const uint32_t grid[3], const uint32_t block[3],
                             void* const* buffers, const size_t* buf_bytes, size_t nbuffers,
                             const uint64_t* scalars, size_t nscalars, void* stream) {
  return launch_checked(kernel, grid, block, buffers, buf_bytes, nbuffers, scalars, nscalars, stream, true);
}

size_t qmm_static_scratch_bytes(void) { return kStaticScratchBytes; }

qmm_status qmm_workspace_bytes(qmm_kernel kernel, const uint64_t* scalars, size_t nscalars, size_t* out_bytes) {
  if (kernel == 0 || kernel > kTableSize || out_bytes == nullptr || (nscalars != 0 && scalars == nullptr)) {
    return bad("qmm_workspace_bytes: bad kernel handle or null argument");
  }
  *out_bytes = 0;
  const std::string id = kTable[kernel - 1].id;
  auto sc = [&](size_t i) { return i < nscalars ? scalars[i] : uint64_t{0}; };
  auto starts = [&](const char* prefix) { return id.rfind(prefix, 0) == 0; };
  if (starts("gemm_q4k")) {
    const uint64_t m = sc(0), n = sc(1), k = sc(2);
    const bool split_id = id == "gemm_q4k_vec" || starts("gemm_q4k_rows");
    const uint64_t layout = sc(split_id ? 4 : 3);
    const uint64_t from = id == "gemm_q4k_wmma" ? kQ4KGemmMinRows : g_q4k_tensor_rows.load(std::memory_order_relaxed);
    if (m >= from && qmm::gemm_q4k_supported(m, k)) *out_bytes = qmm::gemm_q4k_workspace_bytes(m, k);
    if (layout != 0 && m > 1 && k % 256 == 0) *out_bytes = q4k_regime_workspace(m, k, from) + static_cast<size_t>(q4k_bytes(n, k));
  } else if (id == "ffn_gate_up_silu_q4k") {
    const uint64_t m = sc(0), n = sc(1), k = sc(2);
    if (m >= 2 && n != 0 && k != 0) *out_bytes = ffn_scratch(m, n, k).workspace_bytes;
  } else if (id == "gemm_mxfp4_wmma") {
    const uint64_t m = sc(0), n = sc(1), k = sc(2), wperm = sc(4);
    if (wperm == 1 && !qmm::gemm_mxfp4_a8_wperm_supported(m, n, k)) *out_bytes = static_cast<size_t>(mxfp4_bytes(n, k));
  } else if (id == "gemm_mxfp4" || id == "gemm_mxfp4_batched") {
    const uint64_t m = sc(0), k = sc(2);
    if (m >= kMxfp4GemmMinRows && qmm::gemm_mxfp4_f32_supported(m, k)) *out_bytes = qmm::gemm_mxfp4_f32_workspace_bytes(m, k);
  } else if (starts("gemm_q5k") || starts("gemm_q6k")) {
    const uint64_t m = sc(0), n = sc(1), k = sc(2);
    if (m >= kQ4KGemmMinRows && qmm::gemm_kquant_f16_supported(m, n, k)) *out_bytes = qmm::gemm_kquant_f16_workspace_bytes(m, n, k);
  } else if (id == "moe_experts_gate_up_q4k_rows" || id == "moe_experts_down_q4k_rows") {
    const uint64_t hidden = sc(0), inter = sc(1), top_k = sc(2), rows = sc(5);
    if (rows >= kMoeGroupedMinRows) *out_bytes = qmm::moe_ffn_q4k_workspace_bytes(rows * top_k, hidden, inter, 1024);
  } else if (id == "moe_experts_ffn_q4k_rows") {
    const uint64_t hidden = sc(0), inter = sc(1), top_k = sc(2), rows = sc(6);
    *out_bytes = qmm::moe_ffn_q4k_workspace_bytes(rows * top_k, hidden, inter, 1024);
  }
  return QMM_OK;
}

qmm_status qmm_set_q4k_tensor_rows(uint32_t rows) {
  if (rows == 0) rows = static_cast<uint32_t>(kQ4KTensorRowsDefault);
  if (rows < kQ4KGemmMinRows) return bad("qmm_set_q4k_tensor_rows: at least 17 rows (the verify batch of up to 16 stays exact)");
  g_q4k_tensor_rows.store(rows, std::memory_order_relaxed);
  return QMM_OK;
}

uint32_t qmm_q4k_tensor_rows(void) { return static_cast<uint32_t>(g_q4k_tensor_rows.load(std::memory_order_relaxed)); }

qmm_status qmm_set_workspace(void* device_ptr, size_t bytes) {
  if ((device_ptr == nullptr) != (bytes == 0)) return bad("qmm_set_workspace: pointer and size must both be set or both be zero");
  if (reinterpret_cast<uintptr_t>(device_ptr) % 256 != 0) return bad("qmm_set_workspace: the workspace must be 256-byte aligned");
  std::lock_guard<std::mutex> lock(g_workspace_mutex);
  g_user_workspace = device_ptr;
  g_user_workspace_bytes = bytes;
  return QMM_OK;
}

qmm_status qmm_sync(void* stream) { return map_hip(hipStreamSynchronize(static_cast<hipStream_t>(stream))); }

const char* qmm_last_error(void) { return g_last_error.c_str(); }

}  // extern "C"
