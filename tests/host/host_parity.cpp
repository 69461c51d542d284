// Parity of the C++ host side (tessera_amd/host) against the CPU oracle, through the C ABI.
// Test infrastructure: links oracle/liboracle.so as the checker.  Prints one line per case and
// exits non-zero on the first failure.  `--list` prints the cases without touching a GPU.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "../../tessera_amd/host/project.hpp"

extern "C" {
int orc_gemm_q4k_ref(const float* a, const uint8_t* w, float* c, size_t m, size_t n, size_t k);
int orc_gemm_q5k_ref(const float* a, const uint8_t* w, float* c, size_t m, size_t n, size_t k, int threads);
int orc_gemm_q6k_ref(const float* a, const uint8_t* w, float* c, size_t m, size_t n, size_t k, int threads);
int orc_gemm_mxfp4_ref(const float* a, const uint8_t* w, const uint8_t* s, float* c, size_t m, size_t n, size_t k);
int orc_quantize_fp8_ref(float* data, float* scale, size_t rows, size_t cols);
void orc_silu_mul(const float* g, const float* u, float* o, size_t n);
}

using namespace tessera_amd;

namespace {

std::mt19937_64 rng(7);

std::vector<uint8_t> Q4KWeights(size_t n, size_t k) {
  std::vector<uint8_t> w(n * (k / 256) * 144);
  for (auto& b : w) b = static_cast<uint8_t>(rng());
  for (size_t blk = 0; blk < w.size() / 144; ++blk) {   // fp16 d, dmin around 1e-2
    w[blk * 144 + 0] = static_cast<uint8_t>(rng()); w[blk * 144 + 1] = 0x20 + (rng() & 3);
    w[blk * 144 + 2] = static_cast<uint8_t>(rng()); w[blk * 144 + 3] = 0x20 + (rng() & 3);
  }
  return w;
}
std::vector<uint8_t> Q5KWeights(size_t n, size_t k) {
  std::vector<uint8_t> w(n * (k / 256) * 176);
  for (auto& b : w) b = static_cast<uint8_t>(rng());
  for (size_t blk = 0; blk < w.size() / 176; ++blk) {   // fp16 d, dmin around 1e-2
    w[blk * 176 + 1] = 0x20 + (rng() & 3);
    w[blk * 176 + 3] = 0x20 + (rng() & 3);
  }
  return w;
}
std::vector<uint8_t> Q6KWeights(size_t n, size_t k) {
  std::vector<uint8_t> w(n * (k / 256) * 210);
  for (auto& b : w) b = static_cast<uint8_t>(rng());
  for (size_t blk = 0; blk < w.size() / 210; ++blk) w[blk * 210 + 209] = 0x14 + (rng() & 3);   // fp16 d around 1e-3
  return w;
}
std::vector<uint8_t> MxFp4Weights(size_t n, size_t k) {
  std::vector<uint8_t> w(n * k / 2 + n * k / 32);
  for (size_t i = 0; i < n * k / 2; ++i) w[i] = static_cast<uint8_t>(rng());
  for (size_t i = n * k / 2; i < w.size(); ++i) w[i] = static_cast<uint8_t>(119 + rng() % 5);
  return w;
}
std::vector<float> Activations(size_t m, size_t k) {
  std::normal_distribution<float> nd(0.0f, 1.0f);
  std::vector<float> a(m * k);
  for (auto& v : a) {
    v = nd(rng);
    uint32_t bits; std::memcpy(&bits, &v, 4);             // bf16-valued, like the prefill configuration
    bits = (bits + 0x7FFFu + ((bits >> 16) & 1u)) & 0xFFFF0000u;
    std::memcpy(&v, &bits, 4);
  }
  return a;
}

template <class T>
std::unique_ptr<Buffer> Upload(Backend& b, const std::vector<T>& v) {
  auto buf = b.AllocateBuffer(v.size() * sizeof(T));
  if (!buf || !b.CopyH2D(**buf, std::as_bytes(std::span<const T>(v)))) std::exit(3);
  return std::move(*buf);
}

// largest |got - ref| over max(|ref|, 0.05 rms(ref)), and over rms(ref)
void Errors(const std::vector<float>& got, const std::vector<float>& ref, double& rel, double& rms_rel) {
  double ss = 0;
  for (float v : ref) ss += double(v) * v;
  const double rms = std::sqrt(ss / ref.size());
  rel = rms_rel = 0;
  for (size_t i = 0; i < ref.size(); ++i) {
    const double d = std::fabs(double(got[i]) - ref[i]);
    rel = std::max(rel, d / std::max(std::fabs(double(ref[i])), 0.05 * rms));
    rms_rel = std::max(rms_rel, d / rms);
  }
}

struct Case {
  const char* name;
  DType dtype;
  size_t m, n, k;
  bool reference_split;
  double rel_tol, rms_tol;     // see tests/test_gpu_q4k.py, test_gpu_gemm_q4k.py, test_gpu_gemm_mxfp4.py, test_gpu_gemm_mxfp4_f32.py
  bool fp8_prefill = false;    // ProjectState::mxfp4_fp8_prefill: E4M3 activations beyond 16 rows (reference: QDQ + GemmMxFp4Ref)
  bool row_groups = false;     // the Q4_K tensor is replaced by RowGroupCopyQ4K's copy before the projection
};
const Case kCases[] = {
    {"q4k decode m=1 (gemm_q4k_vec)", DType::Q4K, 1, 640, 5120, false, 1e-3, 1e-3},
    {"q4k decode m=1, reference split-K + gemm_vec_reduce", DType::Q4K, 1, 640, 5120, true, 1e-3, 1e-3},
    {"q4k verify m=3 (gemm_q4k_rows3)", DType::Q4K, 3, 333, 2048, true, 1e-3, 1e-3},
    {"q4k m=7 (gemm_q4k_vec, m rows)", DType::Q4K, 7, 129, 1280, false, 1e-3, 1e-3},
    {"q4k m=16 (gemm_q4k_batched)", DType::Q4K, 16, 256, 1024, false, 1e-3, 1e-3},
    {"q4k prefill m=192 (gemm_q4k_wmma, fp16 MFMA)", DType::Q4K, 192, 320, 1024, false, 1.0, 4e-3},
    {"q4k decode m=1 over the load-time row-group copy (layout scalar)", DType::Q4K, 1, 650, 5120, false, 1e-3, 1e-3, false, true},
    {"q4k verify m=3 over the row-group copy, reference split-K", DType::Q4K, 3, 333, 2048, true, 1e-3, 1e-3, false, true},
    {"q4k prefill m=192 over the row-group copy (gemm_q4k_wmma)", DType::Q4K, 192, 320, 1024, false, 1.0, 4e-3, false, true},
    {"q6k decode m=1, reference split-K (gemm_q6k_vec)", DType::Q6K, 1, 640, 5120, true, 1e-3, 1e-3},
    {"q6k verify m=3 (gemm_q6k_rows3)", DType::Q6K, 3, 333, 2048, true, 1e-3, 1e-3},
    {"q6k prefill m=192 (gemm_q6k_wmma, fp16 MFMA)", DType::Q6K, 192, 320, 1024, false, 1.0, 4e-3},
    {"q5k decode m=1 (gemm_q5k_vec)", DType::Q5K, 1, 640, 5120, false, 1e-3, 1e-3},
    {"q5k m=16 (gemm_q5k_batched)", DType::Q5K, 16, 256, 1024, false, 1e-3, 1e-3},
    {"q5k prefill m=100 (gemm_q5k_wmma, fp16 MFMA)", DType::Q5K, 100, 257, 2304, false, 1.0, 4e-3},
    {"mxfp4 w4a8 m=1 (quantize_fp8_pack_rows + gemm_mxfp4_wmma)", DType::F4E2M1, 1, 512, 1024, false, 1e-3, 1e-3},
    {"mxfp4 w4a8 m=16 (streaming scaled MFMA)", DType::F4E2M1, 16, 512, 2048, false, 1e-2, 5e-4},
    {"mxfp4 w4a8 m=300 (tiled scaled MFMA, opt-in)", DType::F4E2M1, 300, 384, 1024, false, 1e-2, 5e-4, true},
    {"mxfp4 prefill m=300, the reference's rule (gemm_mxfp4_batched, fp32 rows on the scaled MFMA)", DType::F4E2M1, 300, 384,
     1024, false, 2e-3, 1e-4},
    {"mxfp4 m=17 (gemm_mxfp4_batched)", DType::F4E2M1, 17, 200, 2048, false, 2e-3, 1e-4},
};

// Front half of the dense feed-forward block through FfnGateUpSilu, fused id or three launches.
struct FfnCase {
  const char* name;
  size_t m, n, k;
  bool three_launches;
  double rel_tol;
};
const FfnCase kFfnCases[] = {
    {"ffn gate/up/silu m=1 (ffn_gate_up_silu_q4k, one launch)", 1, 1027, 5120, false, 1e-3},
    {"ffn gate/up/silu m=1, the reference's three launches", 1, 1027, 5120, true, 1e-3},
    {"ffn gate/up/silu m=3 (fused id, composed inside the library)", 3, 200, 2048, false, 1e-3},
};

bool RunFfn(Backend& backend, const FfnCase& c) {
  ProjectState h;
  h.no_fused_ffn = c.three_launches;
  const auto x = Activations(c.m, c.k);
  const auto gate = Q4KWeights(c.n, c.k), up = Q4KWeights(c.n, c.k);
  std::vector<float> g(c.m * c.n), u(c.m * c.n), ref(c.m * c.n), got(c.m * c.n);
  orc_gemm_q4k_ref(x.data(), gate.data(), g.data(), c.m, c.n, c.k);
  orc_gemm_q4k_ref(x.data(), up.data(), u.data(), c.m, c.n, c.k);
  orc_silu_mul(g.data(), u.data(), ref.data(), ref.size());
  auto dx = Upload(backend, x);
  auto dg = Upload(backend, gate);
  auto du = Upload(backend, up);
  auto og = backend.AllocateBuffer(ref.size() * 4), ou = backend.AllocateBuffer(ref.size() * 4);
  auto out = backend.AllocateBuffer(ref.size() * 4);
  auto st = FfnGateUpSilu(backend, h, DType::Q4K, DType::Q4K, *dx, *dg, *du, **og, **ou, **out, c.m, c.n, c.k);
  backend.Synchronize();
  if (!st) {
    std::printf("FAIL %s: status %d (%s)\n", c.name, static_cast<int>(st.error()), backend.LastError());
    return false;
  }
  if (!backend.CopyD2H(**out, std::as_writable_bytes(std::span<float>(got)))) std::exit(3);
  double rel, rms;
  Errors(got, ref, rel, rms);
  const bool launches_ok = (h.kernels.count("ffn_gate_up_silu_q4k") == 1) != c.three_launches;
  const bool ok = rel <= c.rel_tol && launches_ok;
  std::printf("%s %s: rel %.2e (<= %.0e)%s\n", ok ? "ok  " : "FAIL", c.name, rel, c.rel_tol,
              launches_ok ? "" : " [wrong launch sequence]");
  return ok;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc > 1 && std::strcmp(argv[1], "--list") == 0) {
    for (const Case& c : kCases) std::printf("%s\n", c.name);
    for (const FfnCase& c : kFfnCases) std::printf("%s\n", c.name);
    return 0;
  }
  auto backend = CreateBackend();
  if (auto ok = backend->Init(); !ok) {
    std::printf("Init failed: status %d (%s)\n", static_cast<int>(ok.error()), backend->LastError());
    return 2;
  }
  // Error behaviour of the reference interface.
  if (auto k = backend->LoadKernel("delta_step_heads"); k || k.error() != StatusCode::UnsupportedFeature) return 4;
  const std::byte blob[4] = {};
  if (auto k = backend->LoadKernel("gemm_q4k", std::span<const std::byte>(blob)); k || k.error() != StatusCode::UnsupportedFeature) return 4;
  if (auto b = backend->AllocateBuffer(0); b || b.error() != StatusCode::InvalidArgument) return 4;
  {
    auto k = backend->LoadKernel("gemm_q4k");
    auto buf = backend->AllocateBuffer(1024);
    KernelLaunch l;
    l.buffers = {buf->get(), buf->get(), buf->get()};
    l.scalars = {1, 8, 100};                                // k not a multiple of 256
    if (auto st = backend->LaunchKernel(**k, l); st || st.error() != StatusCode::InvalidArgument) return 4;
  }
  std::printf("ok   error behaviour (unknown id, non-empty code, zero-byte buffer, bad k)\n");

  int failed = 0;
  for (const Case& c : kCases) {
    ProjectState h;
    h.honour_reference_split = c.reference_split;
    h.mxfp4_fp8_prefill = c.fp8_prefill;
    const auto a = Activations(c.m, c.k);
    const auto w = c.dtype == DType::Q4K   ? Q4KWeights(c.n, c.k)
                   : c.dtype == DType::Q5K ? Q5KWeights(c.n, c.k)
                   : c.dtype == DType::Q6K ? Q6KWeights(c.n, c.k)
                                           : MxFp4Weights(c.n, c.k);
    std::vector<float> ref(c.m * c.n), got(c.m * c.n);
    if (c.dtype == DType::Q4K) {
      orc_gemm_q4k_ref(a.data(), w.data(), ref.data(), c.m, c.n, c.k);
    } else if (c.dtype == DType::Q5K) {
      orc_gemm_q5k_ref(a.data(), w.data(), ref.data(), c.m, c.n, c.k, 1);
    } else if (c.dtype == DType::Q6K) {
      orc_gemm_q6k_ref(a.data(), w.data(), ref.data(), c.m, c.n, c.k, 1);
    } else {
      std::vector<float> qdq = a, scale(c.m);               // QuantizeFp8Ref (m <= 16 or opted in) then GemmMxFp4Ref
      if (c.m <= 16 || c.fp8_prefill) orc_quantize_fp8_ref(qdq.data(), scale.data(), c.m, c.k);
      orc_gemm_mxfp4_ref(qdq.data(), w.data(), w.data() + c.n * c.k / 2, ref.data(), c.m, c.n, c.k);
    }
    auto da = Upload(*backend, a);
    auto dw = Upload(*backend, w);
    if (c.row_groups) {
      auto copy = RowGroupCopyQ4K(*backend, h, *dw, c.n, c.k);
      if (!copy) {
        std::printf("FAIL %s: RowGroupCopyQ4K status %d (%s)\n", c.name, static_cast<int>(copy.error()), backend->LastError());
        ++failed;
        continue;
      }
      dw = std::move(*copy);     // the loader drops the GGUF-order buffer
    }
    auto out = backend->AllocateBuffer(c.m * c.n * 4);
    auto st = ProjectBatch(*backend, h, c.dtype, *da, *dw, **out, c.m, c.n, c.k);
    backend->Synchronize();
    if (!st) {
      std::printf("FAIL %s: status %d (%s)\n", c.name, static_cast<int>(st.error()), backend->LastError());
      ++failed;
      continue;
    }
    if (!backend->CopyD2H(**out, std::as_writable_bytes(std::span<float>(got)))) return 3;
    double rel, rms;
    Errors(got, ref, rel, rms);
    const bool ok = rel <= c.rel_tol && rms <= c.rms_tol;
    std::printf("%s %s: rel %.2e (<= %.0e) rms %.2e (<= %.0e)\n", ok ? "ok  " : "FAIL", c.name, rel, c.rel_tol, rms, c.rms_tol);
    failed += ok ? 0 : 1;
  }
  for (const FfnCase& c : kFfnCases) failed += RunFfn(*backend, c) ? 0 : 1;
  return failed == 0 ? 0 : 1;
}
