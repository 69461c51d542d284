// Host-side projection helpers over the Backend: the reference's regime table
// (src/models/qwen3_5/project.cpp:233-366, thresholds src/core/decode_internal.hpp:1349-1441)
// and split-K rule (src/core/decode_internal.hpp:840-885), with the same function names.
// ProjectBatch computes C (m x n fp32) = A (m x k fp32) . deq(W)^T for a quantized weight.
#pragma once

#include <cstdlib>
#include <map>
#include <string>

#include "backend.hpp"

namespace tessera_amd {

// src/core/decode_internal.hpp:840-885.
constexpr std::size_t kGemmVecOutputsPerBlock = 8;
constexpr std::size_t kGemmVecSplitTargetBlocks = 2048;
constexpr std::size_t kGemmVecMaxSplit = 8;
// src/core/decode_internal.hpp:1349-1361 (tile sizes), 1425-1441 (kGemmWmmaMinRows at 1428).
constexpr std::size_t kGemmWmmaMinRows = 64;
constexpr std::size_t kGemmWmmaMinCols = 32;
constexpr std::size_t kTiledMinRows = 16;

// Largest divisor of k/256 that brings the workgroup count of a "_vec"/"_rows" launch up to
// `target`, capped at kGemmVecMaxSplit; 1 keeps the plain grid.
inline std::size_t GemmVecSplit(std::size_t outputs, std::size_t k, std::size_t target = kGemmVecSplitTargetBlocks) {
  const std::size_t blocks_x = (outputs + kGemmVecOutputsPerBlock - 1) / kGemmVecOutputsPerBlock;
  if (blocks_x == 0 || blocks_x >= target) return 1;
  const std::size_t superblocks = k / 256;
  std::size_t split = (target + blocks_x - 1) / blocks_x;
  if (split > kGemmVecMaxSplit) split = kGemmVecMaxSplit;
  for (; split > 1; --split) {
    if (superblocks % split == 0) return split;
  }
  return 1;
}

// Kernels and scratch a sequence of projections shares (the part of Qwen35State that
// ProjectBatch and ProjectWmma touch: src/models/qwen3_5/internal.hpp:104-199).
struct ProjectState {
  std::map<std::string, std::unique_ptr<Kernel>> kernels;
  std::unique_ptr<Buffer> gemv_part;                     // split-K partials
  std::unique_ptr<Buffer> wmma_a, wmma_as;               // E4M3 codes and row scales of A
  std::map<const Buffer*, std::unique_ptr<Buffer>> mxfp4_wref;
  // Q4_K tensors kept as this backend's load-time row-group copy (RowGroupCopyQ4K below): the rows
  // per group that the Q4_K GEMM ids then receive as their trailing `layout` scalar -- what the
  // reference does for MXFP4 with PermuteMxFp4ToWmma and `wperm` (src/models/qwen3_5/project.cpp:212).
  std::map<const Buffer*, std::uint64_t> q4k_layout;
  // The reference splits K to fill a 96-CU card; this backend takes any split (it writes the
  // whole result to region 0) but gains nothing from it, so the default passes split = 1.
  bool honour_reference_split = false;
  // Take the reference's three launches for the dense gate/up/silu even where the fused id exists.
  bool no_fused_ffn = false;
  // MXFP4: the per-token E4M3 activation path (ProjectWmma).  As in the reference
  // (src/models/qwen3_5/project.cpp:236-250) it is on unless TESSERA_MXFP4_WMMA=0 and serves
  // m <= 16; more rows keep fp32 activations ("gemm_mxfp4_batched", which this backend runs on the
  // matrix cores without quantizing the activation).
  bool mxfp4_wmma = [] {
    const char* env = std::getenv("TESSERA_MXFP4_WMMA");
    return env == nullptr || std::atoi(env) != 0;
  }();
  // Opt-in, not a reference setting: also send m > 16 through ProjectWmma (k % 128 == 0).  Half
  // the time of the fp32-row id, at the price of the E4M3 rounding of the activation (about 2^-4
  // per element) that the reference's prefill does not have.
  bool mxfp4_fp8_prefill = false;
};

inline Expected<const Kernel*> CachedKernel(Backend& backend, ProjectState& h, const std::string& id) {
  auto it = h.kernels.find(id);
  if (it == h.kernels.end()) {
    auto loaded = backend.LoadKernel(id);
    if (!loaded) return unexpected(loaded.error());
    it = h.kernels.emplace(id, std::move(*loaded)).first;
  }
  return it->second.get();
}

inline Expected<void> Grow(Backend& backend, std::unique_ptr<Buffer>& slot, std::size_t bytes) {
  if (slot != nullptr && slot->Size() >= bytes) return {};
  auto buf = backend.AllocateBuffer(bytes);
  if (!buf) return unexpected(buf.error());
  slot = std::move(*buf);
  return {};
}

// "_vec" / "_rows{R}" launch with the split-K partials and the reduce pass
// (ProjectGemvDevice / ProjectGemvRowsDevice, src/models/qwen3_5/internal.hpp:104-199).
inline Expected<void> ProjectGemvDevice(Backend& backend, ProjectState& h, const Kernel& gemm, const Buffer& a,
                                        const Buffer& w, Buffer& out, std::size_t m, std::size_t n, std::size_t k,
                                        std::uint64_t layout = 0) {
  const std::size_t split = h.honour_reference_split ? GemmVecSplit(m * n, k) : 1;
  const Buffer* dst = &out;
  if (split > 1) {
    if (auto ok = Grow(backend, h.gemv_part, split * m * n * 4); !ok) return ok;
    dst = h.gemv_part.get();
  }
  KernelLaunch l;
  l.grid_x = static_cast<std::uint32_t>((m * n + kGemmVecOutputsPerBlock - 1) / kGemmVecOutputsPerBlock);
  l.grid_y = static_cast<std::uint32_t>(split);
  l.buffers = {&a, &w, dst};
  l.scalars = {m, n, k, split};
  if (layout != 0) l.scalars.push_back(layout);
  if (auto ok = backend.LaunchKernel(gemm, l); !ok) return ok;
  if (split > 1) {
    auto reduce = CachedKernel(backend, h, "gemm_vec_reduce");
    if (!reduce) return unexpected(reduce.error());
    KernelLaunch r;
    r.grid_x = static_cast<std::uint32_t>((m * n + 255) / 256);
    r.buffers = {h.gemv_part.get(), &out};
    r.scalars = {m * n, split};
    return backend.LaunchKernel(**reduce, r);
  }
  return {};
}

// Load-time hook, not a reference function: replaces a Q4_K tensor of n rows x k by this backend's
// row-group copy (same byte count) and remembers its layout, so that every later ProjectBatch on
// the returned buffer passes the `layout` scalar.  A loader would call it for the tensors it wants
// kept that way (one row against long weight rows gains: 5120 x 17408 13.3 against 14.0 us) right
// after upload and drop the GGUF-order buffer.  Returns UnsupportedFeature where the backend has no such id.
inline Expected<std::unique_ptr<Buffer>> RowGroupCopyQ4K(Backend& backend, ProjectState& h, const Buffer& w,
                                                         std::size_t n, std::size_t k, std::uint64_t rows_per_group = 32) {
  auto perm = CachedKernel(backend, h, "permute_q4k_rowgroup");
  if (!perm) return unexpected(perm.error());
  auto copy = backend.AllocateBuffer(w.Size());
  if (!copy) return unexpected(copy.error());
  KernelLaunch l;
  l.buffers = {&w, copy->get()};
  l.scalars = {n, k, rows_per_group, 0};
  if (auto ok = backend.LaunchKernel(**perm, l); !ok) return unexpected(ok.error());
  h.q4k_layout[copy->get()] = rows_per_group;
  return std::move(*copy);
}

// MXFP4 weights with per-token E4M3 activations (ProjectWmma,
// src/models/qwen3_5/project.cpp:100-232): quantize_fp8_pack_rows, mxfp4_row_ref once per
// weight, gemm_mxfp4_wmma.  Returns false when the backend lacks the kernel.
inline Expected<bool> ProjectWmma(Backend& backend, ProjectState& h, const Buffer& a, const Buffer& w, Buffer& out,
                                  std::size_t m, std::size_t n, std::size_t k) {
  auto wmma = CachedKernel(backend, h, "gemm_mxfp4_wmma");
  if (!wmma) {
    if (wmma.error() == StatusCode::UnsupportedFeature) return false;
    return unexpected(wmma.error());
  }
  auto pack = CachedKernel(backend, h, "quantize_fp8_pack_rows");
  auto rowref = CachedKernel(backend, h, "mxfp4_row_ref");
  if (!pack) return unexpected(pack.error());
  if (!rowref) return unexpected(rowref.error());
  if (auto ok = Grow(backend, h.wmma_a, m * k); !ok) return unexpected(ok.error());
  if (auto ok = Grow(backend, h.wmma_as, m * 4); !ok) return unexpected(ok.error());
  auto it = h.mxfp4_wref.find(&w);
  if (it == h.mxfp4_wref.end()) {
    auto buf = backend.AllocateBuffer(n);
    if (!buf) return unexpected(buf.error());
    KernelLaunch rl;
    rl.grid_x = static_cast<std::uint32_t>((n + 255) / 256);
    rl.buffers = {&w, buf->get()};
    rl.scalars = {n, k};
    if (auto ok = backend.LaunchKernel(**rowref, rl); !ok) return unexpected(ok.error());
    it = h.mxfp4_wref.emplace(&w, std::move(*buf)).first;
  }
  KernelLaunch ql;
  ql.grid_x = static_cast<std::uint32_t>(m);
  ql.block_x = 1024;
  ql.buffers = {&a, h.wmma_a.get(), h.wmma_as.get()};
  ql.scalars = {m, k};
  if (auto ok = backend.LaunchKernel(**pack, ql); !ok) return unexpected(ok.error());
  KernelLaunch wl;
  wl.grid_x = static_cast<std::uint32_t>((n + 63) / 64);
  wl.block_x = 128;
  wl.buffers = {h.wmma_a.get(), &w, h.wmma_as.get(), it->second.get(), &out};
  wl.scalars = {m, n, k, 1, 0};
  if (auto ok = backend.LaunchKernel(**wmma, wl); !ok) return unexpected(ok.error());
  return true;
}

// The regime table.  On this backend every id of a format accepts every m and picks its own
// gfx950 kernel, so the table only has to name an id the caller's contract allows.
inline Expected<void> ProjectBatch(Backend& backend, ProjectState& h, DType dtype, const Buffer& a, const Buffer& w,
                                   Buffer& out, std::size_t m, std::size_t n, std::size_t k) {
  if (m == 0 || n == 0 || k == 0) return unexpected(StatusCode::InvalidArgument);
  if (dtype == DType::F4E2M1) {
    if (h.mxfp4_wmma && (m <= 16 || (h.mxfp4_fp8_prefill && k % 128 == 0))) {
      auto done = ProjectWmma(backend, h, a, w, out, m, n, k);
      if (!done) return unexpected(done.error());
      if (*done) return {};
    }
    auto gemm = CachedKernel(backend, h, m == 1 ? "gemm_mxfp4" : (m <= 16 ? "gemm_mxfp4_rows" : "gemm_mxfp4_batched"));
    if (!gemm) return unexpected(gemm.error());
    KernelLaunch l;
    // the reference's shapes: a warp per column for one row and for up to 16 rows
    // (src/backends/rocm/rocm_kernels_basic.cpp:1097-1214), 32 x 32 tiles for the batched kernel; the
    // library picks its own geometry from m, n, k either way
    l.grid_x = static_cast<std::uint32_t>(m <= 16 ? (n + 7) / 8 : ((m + 31) / 32) * ((n + 31) / 32));
    l.buffers = {&a, &w, &out};
    l.scalars = {m, n, k};
    return backend.LaunchKernel(**gemm, l);
  }
  if (dtype == DType::Q4K || dtype == DType::Q5K || dtype == DType::Q6K) {
    // The K-quant formats share one table (src/core/decode_internal.hpp:1256-1276,1365-1460):
    // rows{m} for m in 2..4 (the ids exist up to 5), the tensor-core tile from 64 rows and 32
    // columns, the batched id from kTiledMinRows, the vec id otherwise.
    if (k % 256 != 0) return unexpected(StatusCode::InvalidArgument);
    const std::string fmt = dtype == DType::Q4K ? "q4k" : dtype == DType::Q5K ? "q5k" : "q6k";
    std::uint64_t layout = 0;
    if (dtype == DType::Q4K) {
      if (auto it = h.q4k_layout.find(&w); it != h.q4k_layout.end()) layout = it->second;
    }
    if (m >= 2 && m <= 4) {
      auto rows = CachedKernel(backend, h, "gemm_" + fmt + "_rows" + std::to_string(m));
      if (!rows) return unexpected(rows.error());
      return ProjectGemvDevice(backend, h, **rows, a, w, out, m, n, k, layout);
    }
    if (m >= kGemmWmmaMinRows && n >= kGemmWmmaMinCols) {
      auto wmma = CachedKernel(backend, h, "gemm_" + fmt + "_wmma");
      if (!wmma) return unexpected(wmma.error());
      KernelLaunch l;
      l.grid_x = static_cast<std::uint32_t>((n + 63) / 64);
      l.grid_y = static_cast<std::uint32_t>((m + 127) / 128);
      l.buffers = {&a, &w, &out};
      l.scalars = {m, n, k};
      if (layout != 0) l.scalars.push_back(layout);
      return backend.LaunchKernel(**wmma, l);
    }
    if (m >= kTiledMinRows) {
      auto tiled = CachedKernel(backend, h, "gemm_" + fmt + "_batched");
      if (!tiled) return unexpected(tiled.error());
      KernelLaunch l;
      l.grid_x = static_cast<std::uint32_t>(((m + 31) / 32) * ((n + 31) / 32));
      l.buffers = {&a, &w, &out};
      l.scalars = {m, n, k};
      if (layout != 0) l.scalars.push_back(layout);
      return backend.LaunchKernel(**tiled, l);
    }
    auto vec = CachedKernel(backend, h, "gemm_" + fmt + "_vec");
    if (!vec) return unexpected(vec.error());
    return ProjectGemvDevice(backend, h, **vec, a, w, out, m, n, k, layout);
  }
  return unexpected(StatusCode::UnsupportedFeature);
}

// Front half of the dense feed-forward block: mlp = silu(xn Gate^T) * (xn Up^T)
// (src/models/qwen3_5/trunk.cpp:294-304: ProjectBatch for gate, ProjectBatch for up,
// SiluMulDevice).  When both tensors are Q4_K the backend's fused id does it in one launch;
// a backend without the id (UnsupportedFeature) or other formats take the reference's three
// launches, with `gate_out` and `up_out` as the intermediates the reference keeps in h.fgate/h.fup.
inline Expected<void> FfnGateUpSilu(Backend& backend, ProjectState& h, DType gate_dtype, DType up_dtype,
                                    const Buffer& xn, const Buffer& gate, const Buffer& up, Buffer& gate_out,
                                    Buffer& up_out, Buffer& mlp, std::size_t m, std::size_t n, std::size_t k) {
  if (m == 0 || n == 0 || k == 0) return unexpected(StatusCode::InvalidArgument);
  if (gate_dtype == DType::Q4K && up_dtype == DType::Q4K && !h.no_fused_ffn) {
    auto fused = CachedKernel(backend, h, "ffn_gate_up_silu_q4k");
    if (fused) {
      KernelLaunch l;
      l.grid_x = static_cast<std::uint32_t>((m * n + 7) / 8);
      l.buffers = {&xn, &gate, &up, &mlp};
      l.scalars = {m, n, k};
      return backend.LaunchKernel(**fused, l);
    }
    if (fused.error() != StatusCode::UnsupportedFeature) return unexpected(fused.error());
  }
  if (auto st = ProjectBatch(backend, h, gate_dtype, xn, gate, gate_out, m, n, k); !st) return st;
  if (auto st = ProjectBatch(backend, h, up_dtype, xn, up, up_out, m, n, k); !st) return st;
  auto silu = CachedKernel(backend, h, "silu_mul");
  if (!silu) return unexpected(silu.error());
  KernelLaunch l;
  l.grid_x = static_cast<std::uint32_t>((m * n + 255) / 256);     // src/core/decode_internal.hpp:976-986
  l.buffers = {&gate_out, &up_out, &mlp};
  l.scalars = {m * n};
  return backend.LaunchKernel(**silu, l);
}

}  // namespace tessera_amd
