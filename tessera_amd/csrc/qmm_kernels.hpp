// Host-callable launchers of the gfx950 kernels.  Every launcher enqueues on
// `stream` and returns the HIP launch status; none allocates or synchronises.
// Shapes are validated by the caller (qmm_abi.hip) before any of these runs.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace qmm {

void set_num_cus(int cus);
int num_cus();

// ---- decode GEMV family (gemv.hip) -----------------------------------------

// C (m x n fp32) = A (m x k fp32) . deq(W)^T, W = n rows of k/256 Q4_K blocks.
hipError_t launch_q4k_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                           uint32_t k, hipStream_t stream);
// W = n rows of k/256 Q5_K blocks (176 bytes each).
hipError_t launch_q5k_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                           uint32_t k, hipStream_t stream);
// W = n rows of k/256 Q6_K blocks (210 bytes each).
hipError_t launch_q6k_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                           uint32_t k, hipStream_t stream);
// W = packed MXFP4 (n*k/2 nibble bytes, then n*k/32 E8M0 bytes).
hipError_t launch_mxfp4_gemv(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n,
                             uint32_t k, hipStream_t stream);
// A = m x k E4M3 codes with per-row scales `as`; W packed MXFP4; lossless weight side.
hipError_t launch_mxfp4_a8_gemv(const uint8_t* a8, const float* as, const uint8_t* w, float* c,
                                uint32_t m, uint32_t n, uint32_t k, hipStream_t stream);
// W = n x k E4M3 bytes, s = one fp32 scale per weight row.
hipError_t launch_fp8_gemv(const float* a, const uint8_t* w, const float* s, float* c, uint32_t m,
                           uint32_t n, uint32_t k, hipStream_t stream);
hipError_t launch_fp8_block_gemv(const float* a, const uint8_t* w, const float* s, float* c, uint32_t m,
                           uint32_t n, uint32_t k, hipStream_t stream);   // s: (n/128) x (k/128) block scales

// Q4_K times 1..4 activation rows on the 4x4x4 fp16 MFMA (gemv_q4k_mfma.hip).  `workspace`
// holds the fp16 hi/lo activation operand (gemv_q4k_mfma_workspace_bytes).
bool gemv_q4k_mfma_supported(uint64_t m, uint64_t n, uint64_t k);
size_t gemv_q4k_mfma_workspace_bytes(uint64_t m, uint64_t k);
hipError_t launch_q4k_gemv_mfma(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m,
                                uint32_t n, uint32_t k, hipStream_t stream);

// Q4_K in row-group order (gemv_q4k_i8.hip): a load-time copy of a GGUF Q4_K matrix, same byte count, in which
// `rows_per_group` consecutive rows (at most kQ4KRowGroupMaxRows; the last group may be shorter) are stored
// together block by block in the operand order of the int8 matrix instruction.
constexpr uint32_t kQ4KRowGroupMaxRows = 64;
uint32_t q4k_rowgroup_default_rows(uint64_t n);
bool q4k_rowgroup_supported(uint64_t n, uint64_t k, uint64_t rows_per_group);
// GGUF -> row groups (inverse: back); not in place.
hipError_t launch_q4k_rowgroup(const uint8_t* in, uint8_t* out, uint32_t n, uint32_t k, uint32_t rows_per_group,
                               bool inverse, hipStream_t stream);
// c (n fp32) = deq(W) . a for one activation row, W in row-group order.
hipError_t launch_q4k_i8_gemv(const float* a, const uint8_t* w, float* c, uint32_t n, uint32_t k,
                              uint32_t rows_per_group, hipStream_t stream);

// ---- routed experts, Q4_K (gemv.hip) ----------------------------------------------
// phi[t][slot*inter + j] = silu(G_e x_t)[j] * (U_e x_t)[j], e = ids[t][slot]; `rows` tokens.
hipError_t launch_moe_gate_up_q4k(const float* x, const uint8_t* gate, const uint8_t* up,
                                  const uint32_t* ids, float* phi, uint32_t hidden, uint32_t inter,
                                  uint32_t top_k, uint64_t gate_stride, uint64_t up_stride,
                                  uint32_t n_experts, uint32_t rows, hipStream_t stream);
// out[t][j] (+)= sum_slot wts[t][slot] * (D_e phi[t][slot])[j].
hipError_t launch_moe_down_q4k(const float* phi, const uint8_t* down, const uint32_t* ids,
                               const float* wts, float* out, uint32_t hidden, uint32_t inter,
                               uint32_t top_k, uint64_t down_stride, bool accumulate, uint32_t n_experts,
                               uint32_t rows, hipStream_t stream);

// The same with Q6_K expert tensors.
hipError_t launch_moe_down_q6k(const float* phi, const uint8_t* down, const uint32_t* ids,
                               const float* wts, float* out, uint32_t hidden, uint32_t inter,
                               uint32_t top_k, uint64_t down_stride, bool accumulate, uint32_t n_experts,
                               uint32_t rows, hipStream_t stream);

// ---- MFMA GEMMs (gemm_mxfp4.hip, gemm_q4k.hip) --------------------------------------
bool gemm_mxfp4_a8_supported(uint64_t k);
// W4A8 on the scaled MFMA: A = m x k E4M3 codes + per-row scales, W packed MXFP4.
hipError_t launch_mxfp4_a8_gemm(const uint8_t* a8, const float* as, const uint8_t* w, float* c,
                                uint32_t m, uint32_t n, uint32_t k, hipStream_t stream);

// The same with W's nibble bytes in the reference's 16-row fragment order (PermuteMxFp4ToWmma,
// src/core/numerics/quant.cpp:926-954), tiled kernel only.
bool gemm_mxfp4_a8_wperm_supported(uint64_t m, uint64_t n, uint64_t k);
hipError_t launch_mxfp4_a8_gemm_wperm(const uint8_t* a8, const float* as, const uint8_t* w, float* c, uint32_t m,
                                      uint32_t n, uint32_t k, hipStream_t stream);
// Packed MXFP4 (nibble bytes then scales) between row-major and that fragment order; the scales are copied.
hipError_t launch_permute_mxfp4_wmma(const uint8_t* in, uint8_t* out, uint64_t n, uint64_t k, bool inverse,
                                     hipStream_t stream);

// MXFP4 weights, fp32 activation rows (17 or more): the rows are split into E4M3 terms in the
// workspace and multiplied on the same scaled MFMA, one pass over K per term.
bool gemm_mxfp4_f32_supported(uint64_t m, uint64_t k);
// 2..16 fp32 rows (k a multiple of 512): the same terms through the streamed few-row kernel, the weights read
// once per eight rows.
bool gemm_mxfp4_f32_rows_supported(uint64_t m, uint64_t n, uint64_t k);
size_t gemm_mxfp4_f32_rows_workspace_bytes(uint64_t m, uint64_t k);
hipError_t launch_mxfp4_f32_rows(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m, uint32_t n,
                                 uint32_t k, hipStream_t stream);
// "gemm_fp8" / "gemm_fp8_block" with 2..16 fp32 rows: E4M3 weights as the matrix instruction's other
// operand, the rows as E4M3 terms; same workspace as gemm_mxfp4_f32_rows_workspace_bytes.  `wscale`:
// one fp32 per weight row, or (block_scales) one per 128 x 128 block, (n/128) x (k/128).  prepare()
// once per device.
bool gemm_fp8_f32_rows_supported(uint64_t m, uint64_t n, uint64_t k);
hipError_t gemm_fp8_f32_rows_prepare();
hipError_t launch_fp8_f32_rows(const float* a, const uint8_t* w, const float* wscale, float* c, void* workspace,
                               uint32_t m, uint32_t n, uint32_t k, bool block_scales, hipStream_t stream);
size_t gemm_mxfp4_f32_workspace_bytes(uint64_t m, uint64_t k);
hipError_t launch_mxfp4_f32_gemm(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m,
                                 uint32_t n, uint32_t k, hipStream_t stream);

// Q4_K prefill GEMM on fp16 MFMA (gemm_q4k.hip).  `workspace` holds m*k fp16 values.
bool gemm_q4k_supported(uint64_t m, uint64_t k);
size_t gemm_q4k_workspace_bytes(uint64_t m, uint64_t k);
hipError_t launch_q4k_gemm(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m,
                           uint32_t n, uint32_t k, hipStream_t stream);

// Q5_K (block_bytes 176) and Q6_K (210) prefill: weights decoded once to fp16 in the workspace,
// then a dense fp16 MFMA GEMM (gemm_q4k.hip).
bool gemm_kquant_f16_supported(uint64_t m, uint64_t n, uint64_t k);
size_t gemm_kquant_f16_workspace_bytes(uint64_t m, uint64_t n, uint64_t k);
hipError_t launch_kquant_f16_gemm(const float* a, const uint8_t* w, uint32_t block_bytes, float* c, void* workspace,
                                  uint32_t m, uint32_t n, uint32_t k, hipStream_t stream);

// Routed experts for a chunk of tokens, grouped by expert (moe_q4k.hip): out[t] (+)= sum over
// the token's top_k experts of wts * down_e(silu(gate_e x) * up_e x), as grouped MFMA GEMMs.
// fp16 copy of fp32 rows, each divided by a power-of-two scale written to scale[row] (gemm_q4k.hip).
// With `pos`, destination row pos[p] takes source row p / top_k.
void launch_rows_to_f16(const float* src, _Float16* dst, float* scale, uint32_t rows, uint32_t cols, const uint32_t* pos,
                        uint32_t top_k, hipStream_t stream);
bool moe_ffn_q4k_supported(uint64_t hidden, uint64_t inter, uint64_t experts);
size_t moe_ffn_q4k_workspace_bytes(uint64_t pairs, uint64_t hidden, uint64_t inter, uint64_t experts);
hipError_t launch_moe_gate_up_q4k_grouped(const float* x, const uint8_t* gate, const uint8_t* up, const uint32_t* ids,
                                          float* phi, void* workspace, uint32_t hidden, uint32_t inter, uint32_t top_k,
                                          uint64_t gate_stride, uint64_t up_stride, uint32_t experts, uint32_t tokens,
                                          hipStream_t stream);
hipError_t launch_moe_down_q4k_grouped(const float* phi, const uint8_t* down, const uint32_t* ids, const float* wts,
                                       float* out, void* workspace, uint32_t hidden, uint32_t inter, uint32_t top_k,
                                       uint64_t down_stride, uint32_t experts, uint32_t tokens, bool accumulate,
                                       hipStream_t stream);
hipError_t launch_moe_ffn_q4k(const float* x, const uint8_t* gate, const uint8_t* up, const uint8_t* down,
                              const uint32_t* ids, const float* wts, float* out, void* workspace,
                              uint32_t hidden, uint32_t inter, uint32_t top_k, uint64_t gate_stride,
                              uint64_t up_stride, uint64_t down_stride, uint32_t experts, uint32_t tokens,
                              bool accumulate, hipStream_t stream);

// ---- element-wise helpers (elementwise.hip) ---------------------------------
hipError_t launch_vec_reduce(const float* part, float* c, uint64_t total, uint64_t split,
                             hipStream_t stream);
hipError_t launch_fill_f32(float* dst, float value, uint64_t count, hipStream_t stream);
hipError_t launch_add(const float* a, const float* b, float* o, uint64_t n, hipStream_t stream);
hipError_t launch_fill_i32(int32_t* out, int32_t value, uint64_t n, hipStream_t stream);
// Register-only loop of one matrix instruction (kind 0: fp16 32x32x16, 1: scaled fp8 x fp4 32x32x64, 2: int8
// 16x16x64), `workgroups` x 4 wavefronts x 4 accumulators x `iters`; out holds workgroups * 256 floats.
hipError_t launch_mfma_probe(float* out, uint32_t kind, bool random, uint32_t iters, uint32_t workgroups,
                             hipStream_t stream);
hipError_t launch_read_probe(const void* src, uint32_t* out, uint64_t bytes, hipStream_t stream);
hipError_t launch_rmsnorm(const float* x, const float* w, float* y, uint64_t rows, uint64_t cols, float eps,
                          hipStream_t stream);
hipError_t launch_embedding(int kind, const uint32_t* ids, const void* table, float* out, uint64_t rows,
                            uint64_t cols, uint64_t vocab, hipStream_t stream);
hipError_t launch_silu_mul(const float* g, const float* u, float* o, uint64_t n, hipStream_t stream);
hipError_t launch_round_bf16(float* x, uint64_t n, hipStream_t stream);

// Q4_K x 2..16 activation rows in one pass over the weights on the 16x16x32 fp16 MFMA, exact on the
// weight side (gemv_q4k_rows16.hip).  `workspace` holds the K parts' output regions.
hipError_t gemv_q4k_rows16_prepare();   // once per device, from qmm_init
hipError_t moe_q4k_prepare();           // once per device, from qmm_init (moe_q4k.hip)

// Q4_K / Q5_K / Q6_K x a few fp32 rows in one pass over the weights on the int8 matrix cores
// (gemv_kquant_rows.hip); any m, taken some rows a pass (eight, eight, four).
hipError_t gemv_kquant_rows_prepare();   // once per device, from qmm_init
bool gemv_kquant_rows_supported(uint64_t m, uint64_t n, uint64_t k);
hipError_t launch_q4k_rows_i8(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                              hipStream_t stream);
hipError_t launch_q5k_rows_i8(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                              hipStream_t stream);
hipError_t launch_q6k_rows_i8(const float* a, const uint8_t* w, float* c, uint32_t m, uint32_t n, uint32_t k,
                              hipStream_t stream);
bool gemv_q4k_rows16_supported(uint64_t m, uint64_t n, uint64_t k);
size_t gemv_q4k_rows16_workspace_bytes(uint64_t m, uint64_t n, uint64_t k);
hipError_t launch_q4k_rows16(const float* a, const uint8_t* w, float* c, void* workspace, uint32_t m, uint32_t n,
                             uint32_t k, hipStream_t stream);

// Q4_K, one activation row, K cut into `split` slices whose partial sums go to `split` output
// regions of n floats (the caller's reduce adds them).
bool q4k_gemv_split_supported(uint64_t n, uint64_t k, uint64_t split);
hipError_t launch_q4k_gemv_split(const float* a, const uint8_t* w, float* c, uint32_t n, uint32_t k, uint32_t split,
                                 hipStream_t stream);

// Dense feed-forward gate and up projections with the activation fused, one activation row:
// out[j] = silu(G x)[j] * (U x)[j], both matrices n rows of Q4_K.
bool ffn_gate_up_q4k_supported(uint64_t k);
hipError_t launch_ffn_gate_up_q4k(const float* x, const uint8_t* gate, const uint8_t* up, float* out,
                                  uint32_t n, uint32_t k, hipStream_t stream);
hipError_t launch_quantize_fp8(float* data, float* scale, uint64_t rows, uint64_t cols,
                               hipStream_t stream);
hipError_t launch_quantize_fp8_pack(const float* in, uint8_t* out, float* scale, uint64_t rows,
                                    uint64_t cols, hipStream_t stream);
hipError_t launch_quantize_fp8_pack_bf16(const uint16_t* in, uint8_t* out, float* scale,
                                         uint64_t rows, uint64_t cols, hipStream_t stream);
hipError_t launch_mxfp4_row_ref(const uint8_t* w, uint8_t* wref, uint64_t n, uint64_t k,
                                hipStream_t stream);
hipError_t launch_dequant_q4k(const uint8_t* w, float* out, uint64_t nblocks, hipStream_t stream);
hipError_t launch_dequant_q5k(const uint8_t* w, float* out, uint64_t nblocks, hipStream_t stream);
hipError_t launch_dequant_q6k(const uint8_t* w, float* out, uint64_t nblocks, hipStream_t stream);
hipError_t launch_dequant_mxfp4(const uint8_t* w, float* out, uint64_t n, uint64_t k,
                                hipStream_t stream);
hipError_t launch_moe_gate(const float* vals, const float* x, const float* w, float* wts, float* sig,
                           uint32_t top_k, uint32_t hidden, hipStream_t stream);
hipError_t launch_top_k_rows(const float* logits, uint32_t* ids, float* vals, uint32_t rows,
                             uint64_t vocab, uint32_t top_k, uint64_t row_base, hipStream_t stream);
hipError_t launch_moe_scale_add(const float* a, const float* b, const float* f, float* o,
                                uint64_t n, uint64_t idx, hipStream_t stream);

// ---- non-matmul trunk pieces (trunk.hip) ---------------------------------------
// pos3 null: "rope" (positions pos_base + row); else "mrope" (per-row (t, h, w) triples, section sizes).
hipError_t launch_rope(float* data, const uint64_t* pos3, uint64_t rows, uint64_t heads, uint64_t head_dim, uint64_t rope_dim,
                       uint64_t pos_base, float theta, uint64_t sec_t, uint64_t sec_h, hipStream_t stream);
hipError_t launch_attention(const float* q, const void* k, const void* v, float* out, uint64_t m, uint64_t n, uint64_t heads,
                            uint64_t kv_heads, uint64_t head_dim, uint64_t q_base, uint64_t row_base, uint64_t window,
                            bool kv_f16, bool causal, hipStream_t stream);
hipError_t launch_attention_quant(const float* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                  float* out, uint64_t m, uint64_t n, uint64_t heads, uint64_t kv_heads, uint64_t head_dim,
                                  uint64_t q_base, uint64_t row_base, uint64_t window, uint32_t kind, hipStream_t stream);
hipError_t launch_attention_split(const float* q, const void* k, const void* v, const float* k_scale, const float* v_scale,
                                  float* pacc, float* pmax, float* psum, uint64_t m, uint64_t n, uint64_t heads,
                                  uint64_t kv_heads, uint64_t head_dim, uint64_t q_base, uint64_t window, uint32_t kv_kind,
                                  bool causal, uint64_t split, hipStream_t stream);
hipError_t launch_attention_combine(const float* pacc, const float* pmax, const float* psum, float* out, uint64_t m,
                                    uint64_t heads, uint64_t head_dim, uint64_t split, hipStream_t stream);
hipError_t launch_quantize_kv(const float* in, uint8_t* out, float* scale, uint64_t rows, uint64_t cols, uint32_t bits,
                              hipStream_t stream);
hipError_t launch_cast_f32_f16(const float* in, void* out, uint64_t n, hipStream_t stream);
hipError_t launch_qgate_split(const float* fused, float* q, float* gate, uint64_t heads, uint64_t head_dim, uint64_t rows,
                              hipStream_t stream);

}  // namespace qmm
