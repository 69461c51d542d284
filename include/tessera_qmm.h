/*
 * tessera_qmm.h -- C ABI of the MI355X (gfx950) quantized-matmul kernel library.
 *
 * The library is the device side of a tessera `Backend` for the quantized matmul
 * path only.  Tessera has no C ABI of its own: its backends are C++ classes linked
 * into the binary (tessera::CreateBackend, include/tessera/backend.hpp:1062-1071).
 * Each entry point below therefore names the Backend virtual, or the piece of
 * RocmBackend, that a thin C++ adapter implements by calling it.
 *
 * Conventions
 *   - plain pointers and sizes only; every device pointer is a HIP device address
 *     on the device chosen by qmm_init;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream).  All work
 *     is asynchronous on that stream, like RocmBackend's single stream
 *     (src/backends/rocm/rocm_backend.cpp:311-330,716-722);
 *   - every function returns a qmm_status whose integer values are identical to
 *     tessera::StatusCode (include/tessera/types.hpp:36-48);
 *   - no exceptions cross the boundary;
 *   - device memory: qmm_alloc allocates what the caller asks for; qmm_init allocates the 16 MB
 *     scratch of the decode-sized kernels once; prefill-sized launches (Q4_K/Q5_K/Q6_K from 17
 *     rows, the grouped routed-expert ids) need a workspace, which is the caller's when one was
 *     set with qmm_set_workspace and otherwise a library-owned block that qmm_launch grows on
 *     demand with hipMalloc.  A block that a launch has used is never freed (growth allocates a
 *     new one of at least twice the size and keeps the old until the process ends, so a launch
 *     recorded into a HIP graph keeps a valid pointer); growth while `stream` is being captured
 *     returns InvalidArgument with a message: grow before capturing, or set a workspace.
 *     qmm_launch_static never allocates.
 */
#ifndef TESSERA_QMM_H_
#define TESSERA_QMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t qmm_status;
enum {
  QMM_OK = 0,
  QMM_INVALID_ARGUMENT = 1,
  QMM_FILE_NOT_FOUND = 2,
  QMM_MALFORMED_FILE = 3,
  QMM_UNSUPPORTED_FEATURE = 4,
  QMM_OUT_OF_MEMORY = 5,
  QMM_DEVICE_ERROR = 6,
  QMM_NON_FINITE = 7,
  QMM_NETWORK_ERROR = 8
};

/* Binding limits of one launch (include/tessera/backend.hpp:45-48). */
#define QMM_MAX_BOUND_BUFFERS 16
#define QMM_MAX_SCALARS 16

/* Opaque kernel handle: table index + 1, never 0 for a loaded kernel.  Same
 * representation as RocmBackend (src/backends/rocm/rocm_backend.cpp:639-670). */
typedef uintptr_t qmm_kernel;

/* Backend::SetDeviceIndex + Backend::Init (backend.hpp:869-889;
 * rocm_backend.cpp:270-333).  Selects the device, checks that it is a gfx950 part
 * and that the library's code object loads, and allocates the 16 MB scratch of the
 * decode-sized kernels (held until the process ends, at a fixed address, so decode
 * launches never allocate and may be recorded into a HIP graph).  Ok when already
 * initialised on the same device; InvalidArgument for an index out of range;
 * UnsupportedFeature on a device that is not gfx950; OutOfMemory / DeviceError for a
 * HIP failure. */
qmm_status qmm_init(int device);

/* Backend::DeviceName (backend.hpp:853-854).  Valid after qmm_init; "" before. */
const char* qmm_device_name(void);

/* Backend::MemoryInfo (backend.hpp:856-859). */
qmm_status qmm_memory_info(uint64_t* total_bytes, uint64_t* free_bytes);

/* Backend::AllocateBuffer(bytes, MemoryKind::Device) / Backend::FreeBuffer
 * (backend.hpp:891-906; rocm_backend.cpp:335-376).  0 bytes is InvalidArgument;
 * hipErrorOutOfMemory maps to OutOfMemory. */
qmm_status qmm_alloc(size_t bytes, void** out_device_ptr);
qmm_status qmm_free(void* device_ptr);

/* Backend::CopyH2DAt / CopyD2HAt / CopyD2D (backend.hpp:912-965;
 * rocm_backend.cpp:378-408,523-550).  The adapter does the bounds check against its
 * Buffer sizes and passes already-offset pointers.  H2D and D2H return after the
 * copy has completed (they synchronise the stream, as the reference does); D2D is
 * asynchronous. */
qmm_status qmm_copy_h2d(void* dst_device, const void* src_host, size_t bytes, void* stream);
qmm_status qmm_copy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream);
qmm_status qmm_copy_d2d(void* dst_device, const void* src_device, size_t bytes, void* stream);

/* Backend::LoadKernel(name, {}) for built-ins (backend.hpp:1004-1017;
 * rocm_backend.cpp:639-670).  An id this library does not implement returns
 * UnsupportedFeature, which the callers rely on to fall through to another regime
 * (src/models/qwen3_5/project.cpp:109-112,285,303,319,331). */
qmm_status qmm_load(const char* id, qmm_kernel* out);

/* Kernel::Id() of a loaded handle; NULL for a bad handle. */
const char* qmm_kernel_id(qmm_kernel kernel);

/* The ids qmm_load accepts, for diagnostics: count, then name by index. */
size_t qmm_kernel_count(void);
const char* qmm_kernel_name(size_t index);

/* Backend::LaunchKernel (backend.hpp:1022-1026; rocm_backend.cpp:672-729) with
 * KernelLaunch flattened: grid[3], block[3], buffers in kernel parameter order, then
 * 64-bit scalars (floats travel as fp32 bit patterns in the low 32 bits).
 *
 * Validation happens before any device work and returns InvalidArgument: zero grid or
 * block dimensions, more than 16 buffers or scalars (ValidateLaunch,
 * backend.hpp:138-148), the per-id argument counts and shape rules of
 * CheckBuiltInArgs (backend.hpp:391-841), a NULL buffer, a buffer pointer that is not
 * 16-byte aligned (device allocations are; the kernels use 16-byte vector loads), and --
 * when `buf_bytes` is not NULL -- any buffer smaller than the launch's scalars require.  `buf_bytes[i]` is
 * Buffer::Size() of buffer i; pass NULL to skip the size check (the routed-expert ids that clamp
 * expert ids to their tensor -- "moe_experts_down_*", "moe_experts_ffn_q4k_rows" -- need the sizes
 * and return InvalidArgument without them).
 *
 * Geometry: the ids keep the reference's argument contracts, but a gfx950 kernel has
 * its own natural launch shape, so `grid` and `block` are validated and otherwise
 * ignored: the library picks the launch shape from the scalars.  (The Vulkan backend
 * ignores block_* the same way, backend.hpp:50-55.)  Split-K ids
 * ("gemm_q4k_vec", "gemm_q4k_rows{2..5}", "gemm_mxfp4_wmma") honour the `split` scalar
 * of their contract: the sum over the `split` output regions equals the result (real
 * per-slice partial sums for one row of a large Q4_K matrix, else everything in region 0 and
 * zeros in the others), so the reference's reduce pass ("gemm_vec_reduce",
 * "gemm_mxfp4_wmma_reduce") still works.
 *
 * Ids and scalars beyond the reference's table (each optional; a caller that never uses them sees
 * the reference's contracts unchanged):
 *   - "permute_q4k_rowgroup": buffers In, Out; scalars n, k, rows_per_group (0 = the default, 32;
 *     at most 64), inverse (0 = GGUF order -> row groups, 1 = back).  The gfx950 counterpart of the
 *     reference's load-time re-ordering hook (PermuteMxFp4ToWmma, src/core/numerics/quant.cpp:926-954):
 *     a copy of a Q4_K tensor, same byte count, laid out for the int8 matrix cores.
 *   - the Q4_K GEMM ids ("gemm_q4k", "_row", "_vec", "_rows{2..5}", "_batched", "_wmma") take one
 *     more trailing scalar, `layout`: absent or 0 = W is in GGUF order; R = W is the copy made by
 *     "permute_q4k_rowgroup" with rows_per_group R (as `wperm` selects the re-ordered MXFP4 tensor,
 *     src/models/qwen3_5/project.cpp:212).  One row runs on the copy directly; more rows have it put
 *     back into GGUF order in the workspace first (qmm_workspace_bytes counts that).
 *   - "gemm_mxfp4", "gemm_mxfp4_rows", "gemm_mxfp4_batched" keep the reference's contract (fp32
 *     activations, no activation quantization).  Where they run on the matrix cores (2..16 rows of a
 *     matrix of 16 M weights or more with k a multiple of 512; from 17 rows with k a multiple of 128)
 *     each activation is carried to 16 significant bits under its row's largest magnitude (exactly,
 *     when it has no more); one row and the small shapes carry the full fp32 value.
 *   - "gemm_fp8" and "gemm_fp8_block" likewise: 2..16 rows of a matrix of 16 M weights or more with k a
 *     multiple of 512 run on the matrix cores (E4M3 weights as stored, activations to 16 significant
 *     bits, the matrix core's own accumulation: within 2e-4 of the rms output of the reference's fp32
 *     loop, 2e-3 with x20 outlier channels); other shapes on the vector unit in fp32.
 *   - "mfma_probe": buffer Out (workgroups * 256 floats); scalars kind (0 fp16 32x32x16, 1 scaled
 *     fp8 x fp4 32x32x64, 2 int8 16x16x64), random (0 constant operands, 1 hashed), iterations,
 *     workgroups.  "read_probe": a plain read of a buffer.  Measurement ids: the matrix-core and the
 *     read ceiling of the part the library runs on, for the benchmark's roofline.
 */
qmm_status qmm_launch(qmm_kernel kernel, const uint32_t grid[3], const uint32_t block[3],
                      void* const* buffers, const size_t* buf_bytes, size_t nbuffers,
                      const uint64_t* scalars, size_t nscalars, void* stream);

/* qmm_launch for callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its
 * scratch lives in the caller's arch state).  Same arguments, validation and results as
 * qmm_launch, but every kernel that needs scratch beyond its inputs and outputs (the Q4_K
 * few-row operand, the fp16 copies of the MFMA GEMMs, the fused feed-forward's up product, the
 * grouped routed-expert tables) takes it from one device array of QMM_STATIC_SCRATCH_BYTES that
 * is part of the library's code object: it calls no hipMalloc or hipFree, and a launch that
 * needs more returns InvalidArgument with the two sizes in qmm_last_error.  Each device the
 * library is loaded on holds that array until the process ends.  All calls on a device share
 * it and it keeps the last call's contents (no kernel here needs it zeroed): launches through
 * this entry point on one device must be ordered (one stream, or events); overlapping ones
 * race on the scratch. */
#define QMM_STATIC_SCRATCH_BYTES (32u << 20)
qmm_status qmm_launch_static(qmm_kernel kernel, const uint32_t grid[3], const uint32_t block[3],
                             void* const* buffers, const size_t* buf_bytes, size_t nbuffers,
                             const uint64_t* scalars, size_t nscalars, void* stream);
size_t qmm_static_scratch_bytes(void);

/* Caller-owned scratch, as the reference keeps it in the arch state and grows it on demand
 * (src/models/qwen3_5/project.cpp:127-155,198-206: gemv_part, wmma_a, wmma_as, wmma_part).
 * qmm_workspace_bytes returns what a launch of `kernel` with these scalars needs (0 for
 * decode-sized launches and ids without scratch; for the grouped routed-expert ids an upper bound
 * over the expert count).  qmm_set_workspace hands the library a device block of that size
 * (256-byte aligned) to use for every later qmm_launch on any stream, in stream order, until it
 * is replaced or cleared with (NULL, 0); while one is set, qmm_launch allocates nothing and a
 * launch that needs more returns InvalidArgument.  The caller must not free or replace the
 * block while launches that use it are in flight. */
qmm_status qmm_workspace_bytes(qmm_kernel kernel, const uint64_t* scalars, size_t nscalars, size_t* out_bytes);
qmm_status qmm_set_workspace(void* device_ptr, size_t bytes);

/* The row count from which the Q4_K ids other than "gemm_q4k_wmma" ("gemm_q4k", "gemm_q4k_batched",
 * "ffn_gate_up_silu_q4k") use the fp16 tensor-core tile, whose operands are rounded to fp16.
 * Default 64: the reference's regime table switches to its own fp16 tile there (kGemmWmmaMinRows,
 * src/core/decode_internal.hpp:1428, used at src/models/qwen3_5/project.cpp:307) and keeps fp32
 * activations below (src/models/qwen3_5/project.cpp:307-322), so by default a result carries the fp16 operand
 * rounding exactly where the reference's does; 17..63 rows then run sixteen at a time through the
 * exact kernels (about 28 us per 16 rows of a 17408 x 5120 matrix, against 35..46 us for the
 * tile).  A caller that prefers the tile's speed there sets a lower count, at least 17 (up to 16
 * rows, the speculative-verify batch, always stay exact); a higher count keeps more rows on the
 * exact kernels, sixteen at a time; 0 restores the default.
 * "gemm_q4k_wmma" itself uses the tile from 17 rows whatever this says.  Process-wide; not a
 * reference interface (its table is compiled in). */
qmm_status qmm_set_q4k_tensor_rows(uint32_t rows);
uint32_t qmm_q4k_tensor_rows(void);

/* Backend::Synchronize (backend.hpp:1028-1029; rocm_backend.cpp:731-739). */
qmm_status qmm_sync(void* stream);

/* Text of the last HIP error seen by this thread ("" if none), for the adapter's
 * diagnostics channel (Backend::SetDiagnostics, backend.hpp:861-863). */
const char* qmm_last_error(void);

#ifdef __cplusplus
} /* extern "C" */
#endif

#endif /* TESSERA_QMM_H_ */
