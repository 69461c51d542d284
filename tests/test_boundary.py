"""The C-ABI boundary: exported symbols, kernel table, and the validation rules of
Backend::LaunchKernel (include/tessera/backend.hpp:138-148,391-841).  The CPU part runs
without a GPU (no compute calls); the GPU part checks that every validation error is raised
before any device work and that the reference's error codes come back."""
import ctypes
import os
import re

import numpy as np
import pytest

import tessera_amd
from tessera_amd import Backend, KernelLaunch, StatusCode, StatusError, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

REFERENCE_IDS = [
    "gemm_q4k", "gemm_q4k_row", "gemm_q4k_vec", "gemm_q4k_rows2", "gemm_q4k_rows3", "gemm_q4k_rows4",
    "gemm_q4k_rows5", "gemm_q4k_batched", "gemm_q4k_wmma", "gemm_vec_reduce", "gemm_mxfp4",
    "gemm_mxfp4_rows", "gemm_mxfp4_batched", "mxfp4_row_ref", "gemm_mxfp4_wmma",
    "gemm_mxfp4_wmma_reduce", "quantize_fp8", "quantize_fp8_pack", "quantize_fp8_pack_rows",
    "gemm_fp8", "gemm_fp8_block", "moe_scale_add", "moe_experts_gate_up_q4k", "moe_experts_down_q4k", "moe_gate",
    "top_k_rows", "gemm_q6k", "gemm_q6k_vec", "gemm_q6k_rows2", "gemm_q6k_rows3", "gemm_q6k_rows4",
    "gemm_q6k_rows5", "gemm_q6k_batched", "gemm_q5k", "gemm_q5k_vec", "gemm_q5k_rows2", "gemm_q5k_rows3",
    "gemm_q5k_rows4", "gemm_q5k_rows5", "gemm_q5k_batched", "moe_experts_down_q6k", "gemm_q5k_wmma", "gemm_q6k_wmma",
    "silu_mul", "round_bf16", "add", "fill", "rmsnorm", "embedding_f32", "embedding_bf16", "embedding_q4k",
    "rope", "mrope", "attention", "qgate_split", "attention_q8", "attention_q4", "attention_fp8", "quantize_q8",
    "quantize_q4", "cast_f32_f16", "attention_split", "attention_split_gqa", "attention_combine", "attention_q8_split",
    "attention_q4_split", "attention_fp8_split",
]


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "tessera_qmm.h")).read()
    declared = sorted(set(re.findall(r"\b(qmm_[a-z0-9_]+)\s*\(", header)))
    assert len(declared) >= 14
    lib = ctypes.CDLL(tessera_amd.backend.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in include/tessera_qmm.h but not exported"


def test_status_codes_match_reference_values():
    header = open(os.path.join(ROOT, "include", "tessera_qmm.h")).read()
    pairs = dict(re.findall(r"QMM_([A-Z_]+) = (\d)", header))
    want = {"OK": 0, "INVALID_ARGUMENT": 1, "FILE_NOT_FOUND": 2, "MALFORMED_FILE": 3,
            "UNSUPPORTED_FEATURE": 4, "OUT_OF_MEMORY": 5, "DEVICE_ERROR": 6, "NON_FINITE": 7,
            "NETWORK_ERROR": 8}
    assert {k: int(v) for k, v in pairs.items()} == want
    assert [c.value for c in StatusCode] == list(range(9))


def test_kernel_table_and_unknown_ids_without_a_device():
    b = Backend()
    names = b.KernelNames()
    for kid in REFERENCE_IDS:
        assert kid in names
        assert b.LoadKernel(kid).Id() == kid
    for kid in ("gemm_q3k", "delta_step_heads", "", "gemm_q4k "):
        with pytest.raises(StatusError) as e:
            b.LoadKernel(kid)
        assert e.value.code == StatusCode.UnsupportedFeature   # callers fall through on this code
    with pytest.raises(StatusError) as e:
        b.LoadKernel("gemm_q4k", code=b"\x03\x02\x23\x07")      # built-ins only, like RocmBackend
    assert e.value.code == StatusCode.UnsupportedFeature
    with pytest.raises(StatusError) as e:
        b.AllocateBuffer(0)
    assert e.value.code == StatusCode.InvalidArgument


def test_generic_launch_validation_without_a_device():
    b = Backend()
    k = b.LoadKernel("gemm_q4k")
    fake = b.WrapBuffer(0x1000, 1 << 20)
    cases = [
        KernelLaunch(grid_x=0, buffers=[fake] * 3, scalars=[1, 1, 256]),
        KernelLaunch(block_y=0, buffers=[fake] * 3, scalars=[1, 1, 256]),
        KernelLaunch(buffers=[fake] * 17, scalars=[1, 1, 256]),
        KernelLaunch(buffers=[fake] * 3, scalars=[1] * 17),
        KernelLaunch(buffers=[fake, b.WrapBuffer(0, 16), fake], scalars=[1, 1, 256]),
    ]
    for launch in cases:
        with pytest.raises(StatusError) as e:
            b.LaunchKernel(k, launch)
        assert e.value.code == StatusCode.InvalidArgument


@pytest.mark.gpu
def test_backend_identity(backend):
    assert backend.Name() == "mi355x"
    assert backend.DeviceName()
    info = backend.MemoryInfo()
    assert info.total_bytes > 100 << 30 and 0 < info.free_bytes <= info.total_bytes
    backend.Init()   # Ok when already initialised


@pytest.mark.gpu
def test_per_id_validation_on_device(backend):
    g = synth.rng(1)
    n, k = 64, 512
    w = backend.Upload(synth.q4k_weights(g, n, k))
    a = backend.Upload(synth.activations_f32(g, 1, k))
    c = backend.AllocateBuffer(4 * n)
    backend.CopyH2D(c, np.full(n, 7.0, np.float32))

    def expect_invalid(name, bufs, scalars):
        with pytest.raises(StatusError) as e:
            backend.LaunchKernel(backend.LoadKernel(name), KernelLaunch(buffers=bufs, scalars=scalars))
        assert e.value.code == StatusCode.InvalidArgument, (name, scalars)

    expect_invalid("gemm_q4k", [a, w], [1, n, k])                # buffer count
    off = backend.WrapBuffer(a.Handle() + 4, a.Size() - 4)          # a pointer into the middle of an allocation
    expect_invalid("gemm_q4k", [off, w, c], [1, n, k - 256])     # not 16-byte aligned
    expect_invalid("gemm_q4k", [a, w, c], [1, n])                # scalar count
    expect_invalid("gemm_q4k", [a, w, c], [0, n, k])             # zero m
    expect_invalid("gemm_q4k", [a, w, c], [1, n, 500])           # k % 256
    expect_invalid("gemm_q4k", [a, w, c], [1, n + 1, k])         # weights too small for n
    expect_invalid("gemm_q4k", [a, w, c], [2, n, k])             # A and C too small for m
    expect_invalid("gemm_q4k_vec", [a, w, c], [1, n, k, 3])      # split must divide k/256
    expect_invalid("gemm_q4k_vec", [a, w, c], [1, n, k, 2])      # C too small for 2 regions
    expect_invalid("gemm_mxfp4", [a, w, c], [1, n, 48])          # k % 32
    expect_invalid("gemm_mxfp4_rows", [a, w, c], [17, n, 512])   # m must be 1..16
    expect_invalid("quantize_fp8", [a, c], [0, k])
    expect_invalid("quantize_fp8_pack", [a, c, c], [1, 510])     # cols % 4
    expect_invalid("gemm_fp8", [a, w, c], [1, n, k])             # 4 buffers
    expect_invalid("gemm_vec_reduce", [c, c], [n, 2])            # partials too small
    backend.Synchronize()
    # nothing ran: C still holds its sentinel
    assert np.all(backend.CopyD2H(c, dtype=np.float32) == 7.0)
    with pytest.raises(StatusError) as e:
        backend.CopyH2DAt(c, 4 * n - 4, np.zeros(2, np.float32))  # bounds-checked copies
    assert e.value.code == StatusCode.InvalidArgument
    with pytest.raises(StatusError) as e:
        backend.CopyD2HAt(c, 8, 4 * n)
    assert e.value.code == StatusCode.InvalidArgument


@pytest.mark.gpu
def test_routed_expert_down_ids_need_buffer_sizes(backend):
    """The expert ids are clamped to the tensor, whose size only the buffer sizes tell: without
    them (buf_bytes = NULL, which other ids accept) the call is refused before any device work."""
    import ctypes as C
    g = synth.rng(2)
    experts, hidden, inter, top_k = 4, 256, 256, 2
    down = backend.Upload(synth.q4k_weights(g, experts * hidden, inter))
    phi = backend.Upload(np.zeros(top_k * inter, np.float32))
    ids = backend.Upload(np.array([1, 3], np.uint32))
    wts = backend.Upload(np.array([0.5, 0.5], np.float32))
    out = backend.AllocateBuffer(4 * hidden)
    backend.CopyH2D(out, np.full(hidden, 7.0, np.float32))
    ds = hidden * (inter // 256) * 144
    lib = backend._lib
    grid, block = (C.c_uint32 * 3)(1, 1, 1), (C.c_uint32 * 3)(256, 1, 1)
    bufs = (C.c_void_p * 5)(phi.Handle(), down.Handle(), ids.Handle(), wts.Handle(), out.Handle())
    for name, scalars in (("moe_experts_down_q4k", [hidden, inter, top_k, ds, 0]),
                          ("moe_experts_down_q4k_rows", [hidden, inter, top_k, ds, 0, 1])):
        scal = (C.c_uint64 * len(scalars))(*scalars)
        kern = backend.LoadKernel(name)
        rc = lib.qmm_launch(kern.Handle(), grid, block, bufs, None, 5, scal, len(scalars), None)
        assert rc == StatusCode.InvalidArgument, name
        assert b"sizes" in lib.qmm_last_error()
    backend.Synchronize()
    assert np.all(backend.CopyD2H(out, dtype=np.float32) == 7.0)
