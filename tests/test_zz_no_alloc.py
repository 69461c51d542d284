"""``qmm_launch_static``: the launch entry point that allocates nothing (scratch from the library's
static device array) must give, bit for bit, what ``qmm_launch`` gives for the ids that use
scratch, on two calls in a row with the second one smaller (the array keeps the first call's
contents), and must refuse a launch whose scratch exceeds the array."""
import numpy as np
import pytest

from tessera_amd import KernelLaunch, StatusCode, StatusError, synth

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _both(backend, name, buffers, out, scalars, grid_x):
    """Run one launch through qmm_launch and through qmm_launch_static; return both outputs."""
    res = []
    kern = backend.LoadKernel(name)
    for no_alloc in (False, True):
        backend.CopyH2D(out, np.full(out.Size() // 4, np.nan, np.float32))
        backend.LaunchKernel(kern, KernelLaunch(grid_x=grid_x, buffers=buffers, scalars=scalars), no_alloc=no_alloc)
        backend.Synchronize()
        res.append(backend.CopyD2H(out, dtype=np.float32).copy())
    return res


def test_static_scratch_matches_allocating_entry_point(backend):
    assert backend.StaticScratchBytes() == 32 << 20
    g = synth.rng(4242)
    n, k = 4100, 4096                     # 16.8 M weights: 2..16 rows take the few-row path (operand in scratch)
    w = synth.q4k_weights(g, n, k)
    up = synth.q4k_weights(g, n, k)
    dw, dup = backend.Upload(w), backend.Upload(up)
    # two calls in a row per id, the second with the smaller input
    for m_first, m_second in ((64, 24), (8, 3)):
        for m in (m_first, m_second):
            a = synth.activations_f32(g, m, k)
            da = backend.Upload(a)
            out = backend.AllocateBuffer(4 * m * n)
            ref, got = _both(backend, "gemm_q4k_batched", [da, dw, out], out, [m, n, k], (m * n + 7) // 8)
            assert np.isfinite(ref).all()
            assert np.array_equal(_bits(got), _bits(ref)), ("gemm_q4k_batched", m)
            ref, got = _both(backend, "ffn_gate_up_silu_q4k", [da, dw, dup, out], out, [m, n, k], (m * n + 7) // 8)
            assert np.isfinite(ref).all()
            assert np.array_equal(_bits(got), _bits(ref)), ("ffn_gate_up_silu_q4k", m)


def test_static_scratch_up_product_that_does_not_fit_the_decode_room(backend):
    """ffn_gate_up_silu_q4k with 40 rows of a wide matrix: the up product (21 MB) does not fit beside the
    few-row kernels' partial sums in the first 16 MB, so it goes behind them in the same static array and
    must not be overwritten by the second 16-row chunk's partials; then a smaller call."""
    g = synth.rng(4245)
    n, k = 131072, 2048
    base = synth.q4k_weights(g, 4096, k)
    w = np.tile(np.asarray(base).reshape(-1), n // 4096)
    up = np.roll(w, 144 * 77)
    dw, dup = backend.Upload(w), backend.Upload(up)
    for m in (40, 18):
        a = synth.activations_f32(g, m, k)
        da = backend.Upload(a)
        out = backend.AllocateBuffer(4 * m * n)
        ref, got = _both(backend, "ffn_gate_up_silu_q4k", [da, dw, dup, out], out, [m, n, k], (m * n + 7) // 8)
        assert np.isfinite(ref).all()
        assert np.array_equal(_bits(got), _bits(ref)), m


def test_static_scratch_fp32_rows_on_the_scaled_matrix_instruction(backend):
    """MXFP4 and FP8 weights with 2..16 fp32 rows keep the rows' E4M3 terms in scratch; 12 rows then 3."""
    g = synth.rng(4246)
    n, k = 4100, 4096
    mx = backend.Upload(synth.mxfp4_weights(g, n, k, -8, -4))
    codes, scales = synth.fp8_weights(g, n, k)
    dcodes, dscales = backend.Upload(codes), backend.Upload(scales)
    for m in (12, 3):
        da = backend.Upload(synth.activations_f32(g, m, k))
        out = backend.AllocateBuffer(4 * m * n)
        ref, got = _both(backend, "gemm_mxfp4_rows", [da, mx, out], out, [m, n, k], (m * n + 7) // 8)
        assert np.isfinite(ref).all()
        assert np.array_equal(_bits(got), _bits(ref)), ("gemm_mxfp4_rows", m)
        ref, got = _both(backend, "gemm_fp8", [da, dcodes, dscales, out], out, [m, n, k], (m * n + 255) // 256)
        assert np.isfinite(ref).all()
        assert np.array_equal(_bits(got), _bits(ref)), ("gemm_fp8", m)


def test_static_scratch_grouped_experts_then_smaller_chunk(backend):
    g = synth.rng(4243)
    experts, hidden, inter, top_k = 16, 512, 256, 4
    gate = synth.q4k_weights(g, experts * inter, hidden)
    up = synth.q4k_weights(g, experts * inter, hidden)
    down = synth.q4k_weights(g, experts * hidden, inter)
    gs, ds = inter * (hidden // 256) * 144, hidden * (inter // 256) * 144
    dg, du, dd = backend.Upload(gate), backend.Upload(up), backend.Upload(down)
    for rows in (96, 40):
        x = synth.activations_bf16(g, rows, hidden)
        ids, vals = synth.moe_routing(g, rows, experts, top_k)
        e = np.exp(vals - vals.max(axis=1, keepdims=True))
        wts = (e / e.sum(axis=1, keepdims=True)).astype(np.float32)
        dx, di, dwt = backend.Upload(x), backend.Upload(ids), backend.Upload(wts)
        out = backend.AllocateBuffer(4 * rows * hidden)
        ref, got = _both(backend, "moe_experts_ffn_q4k_rows", [dx, dg, du, dd, di, dwt, out], out,
                         [hidden, inter, top_k, gs, gs, ds, rows, 0], 1)
        assert np.isfinite(ref).all()
        assert np.array_equal(_bits(got), _bits(ref)), rows


def test_static_scratch_rejects_what_does_not_fit(backend):
    g = synth.rng(4244)
    n, k, m = 64, 17408, 1024             # the fp16 copy of the activations alone is 35.6 MB
    w = synth.q4k_weights(g, n, k)
    dw = backend.Upload(w)
    da = backend.AllocateBuffer(4 * m * k)
    out = backend.AllocateBuffer(4 * m * n)
    kern = backend.LoadKernel("gemm_q4k_wmma")
    launch = KernelLaunch(grid_x=1, buffers=[da, dw, out], scalars=[m, n, k])
    with pytest.raises(StatusError) as err:
        backend.LaunchKernel(kern, launch, no_alloc=True)
    assert err.value.code == StatusCode.InvalidArgument
    assert "static scratch" in str(err.value)
