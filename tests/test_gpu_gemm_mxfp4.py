"""W4A8 GEMM on the scaled MFMA (gemm_mxfp4_wmma with m > 4) against the CPU oracle.

The MFMA multiplies exact E4M3 x E2M1 products; it differs from QuantizeFp8Ref + GemmMxFp4Ref
by how the 64 products of one instruction are summed (the matrix core aligns them to the
largest and keeps a fixed number of bits, so small products next to an outlier lose low bits)
and by the order of the fp32 accumulation across instructions.  Documented bound for this
path (measured against a float64 evaluation the oracle itself sits 1e-5 from): the largest
absolute error is at most 5e-4 of the rms output (measured 2e-4 with the x20 outlier channels
of the benchmark's activation generator, 2e-5 without them), at most 5e-5 in the 2-norm, and
at most 1e-2 under tests/util.py:rel_err."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import norm_err, rel_err, rms_err, run

pytestmark = pytest.mark.gpu


def w4a8(backend, x, w, m, n, k):
    dx, dw = backend.Upload(x), backend.Upload(w)
    da8, das = backend.AllocateBuffer(m * k), backend.AllocateBuffer(4 * m)
    dref, out = backend.AllocateBuffer(n), backend.AllocateBuffer(4 * m * n)
    run(backend, "quantize_fp8_pack_rows", [dx, da8, das], [m, k], grid=(m, 1, 1))
    run(backend, "gemm_mxfp4_wmma", [da8, dw, das, dref, out], [m, n, k, 1, 0], grid=((n + 63) // 64, 1, 1))
    backend.Synchronize()
    return backend.CopyD2H(out, dtype=np.float32).reshape(m, n)


@pytest.mark.parametrize("m,n,k", [(5, 64, 256), (16, 128, 512), (33, 100, 768), (128, 128, 256),
                                   (130, 257, 1024), (64, 192, 5120), (300, 50, 2048),
                                   # more rows than 64 a CU: the few-row kernel shares them out evenly
                                   # (68, 72, 80 rows a workgroup, ragged last workgroup, a second round)
                                   (5, 16500, 512), (20, 17001, 512), (16, 19999, 1024), (3, 20500, 512), (32, 18433, 512)])
def test_gemm_matches_oracle(backend, m, n, k):
    g = synth.rng(m * 7 + n * 3 + k)
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    x = synth.activations_bf16_outliers(g, m, k)
    codes, scale = oracle.quantize_fp8_pack(x, m, k)
    ref = oracle.gemm_mxfp4_w4a8(codes, scale, w, m, n, k)
    got = w4a8(backend, x, w, m, n, k)
    assert rms_err(got, ref) <= 5e-4, rms_err(got, ref)
    assert norm_err(got, ref) <= 5e-5, norm_err(got, ref)
    assert rel_err(got, ref) <= 1e-2, rel_err(got, ref)


def w4a8_oracle(x, w, m, n, k):
    """QuantizeFp8Ref then GemmMxFp4Ref on all host cores: the threaded fp32-activation oracle fed with
    the quantize-dequantized rows e4m3(code) * scale, which is what the single-threaded W4A8 oracle
    multiplies (checked bit for bit on two rows where this is used)."""
    codes, scale = oracle.quantize_fp8_pack(x, m, k)
    lut = np.array([oracle.fp8_e4m3_to_float(c) for c in range(256)], np.float32)
    qdq = (lut[codes] * scale.reshape(m, 1)).astype(np.float32)
    return oracle.gemm_mxfp4(qdq, w, m, n, k, threads=True)


def test_gemm_block_scales_and_codes_exact(backend):
    """Every E2M1 code under a wide spread of E8M0 exponents, one-hot E4M3 activations: each
    output is a single exact product, so the MFMA operand layout (which lane supplies which
    block, nibble order, scale byte selection) is checked bit for bit."""
    g = synth.rng(99)
    m, n, k = 64, 96, 512
    w = synth.mxfp4_weights(g, n, k, -30, 30)
    pos = [int(p) for p in g.permutation(k)[:m]]
    x = synth.one_hot_rows(k, pos) * np.float32(448.0)     # quantizes to code 0x7E, scale 1
    deq = oracle.dequantize_mxfp4(w, n, k)
    got = w4a8(backend, x, w, m, n, k)
    for r, t in enumerate(pos):
        want = (deq[:, t] * np.float32(448.0)).astype(np.float32)
        assert np.array_equal(got[r] + np.float32(0), want + np.float32(0)), (r, t)


def test_full_size_prefill_rows(backend):
    """BASELINE config 3, MXFP4 leg, at full size (M=2048, N=17408, K=5120): a sample of rows
    against the oracle, plus the tensor-parallel column shard N=8704, which must reproduce the
    first half of the columns exactly."""
    g = synth.rng(31337)
    m, n, k = 2048, 17408, 5120
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    x = synth.activations_bf16(g, m, k)
    got = w4a8(backend, x, w, m, n, k)
    # 72 rows: every position inside a 32-row MFMA tile, spread over all eight 256-row tiles, all
    # columns (the 256 x 256 tiles and the 128 x 64 ones that take the leftover columns)
    rows = sorted({(37 * i) % 2048 for i in range(64)} | {0, 31, 32, 255, 256, 1023, 2016, 2047})
    assert {r % 32 for r in rows} == set(range(32)) and {r // 256 for r in rows} == set(range(8))
    ref = w4a8_oracle(x[rows], w, len(rows), n, k)
    few = [0, 3]
    codes, scale = oracle.quantize_fp8_pack(x[rows][few], len(few), k)
    assert np.array_equal(ref[few], oracle.gemm_mxfp4_w4a8(codes, scale, w, len(few), n, k))
    print(f"configs[3] W4A8 2048x17408x5120, {len(rows)} rows: max|d|/rms {rms_err(got[rows], ref):.2e}, "
          f"2-norm {norm_err(got[rows], ref):.2e}, rel (floor 0.05 rms) {rel_err(got[rows], ref):.2e}")
    assert rms_err(got[rows], ref) <= 5e-4, rms_err(got[rows], ref)
    assert norm_err(got[rows], ref) <= 5e-5, norm_err(got[rows], ref)
    shard = synth.mxfp4_column_shard(w, n, k, 0, n // 2)
    got_shard = w4a8(backend, x, shard, m, n // 2, k)
    assert np.array_equal(got_shard, got[:, : n // 2])


def test_down_projection_shape_prefill_rows(backend):
    """The other FFN shape (N=5120, K=17408) at a ragged M: sampled rows against the oracle."""
    g = synth.rng(31338)
    m, n, k = 500, 5120, 17408
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    x = synth.activations_bf16(g, m, k)
    got = w4a8(backend, x, w, m, n, k)
    rows = sorted({(37 * i) % 500 for i in range(40)} | {0, 31, 32, 255, 256, 499})
    assert {r % 32 for r in rows} == set(range(32))
    ref = w4a8_oracle(x[rows], w, len(rows), n, k)
    assert rms_err(got[rows], ref) <= 5e-4, rms_err(got[rows], ref)


# ---- weights pre-permuted at load (the reference's PermuteMxFp4ToWmma, quant.cpp:926-954, wperm = 1) ----
@pytest.mark.parametrize("n,k", [(16, 32), (48, 256), (272, 1024), (1040, 5120)])
def test_permute_id_is_the_reference_permutation(backend, n, k):
    """permute_mxfp4_wmma on the device against the oracle's restatement, and back again."""
    g = synth.rng(n + k)
    w = synth.mxfp4_weights(g, n, k, -20, 20)
    want = oracle.permute_mxfp4_to_wmma(w, n, k)
    dw, dp, db = backend.Upload(w), backend.AllocateBuffer(w.size), backend.AllocateBuffer(w.size)
    run(backend, "permute_mxfp4_wmma", [dw, dp], [n, k, 0], grid=((w.size + 255) // 256, 1, 1))
    run(backend, "permute_mxfp4_wmma", [dp, db], [n, k, 1], grid=((w.size + 255) // 256, 1, 1))
    backend.Synchronize()
    assert np.array_equal(backend.CopyD2H(dp), want)
    assert np.array_equal(backend.CopyD2H(db), w)


@pytest.mark.parametrize("m,n,k", [(1, 64, 1024), (4, 272, 2048), (16, 128, 512), (32, 96, 1024), (33, 272, 1024),
                                   (130, 1040, 1024), (300, 64, 2048), (64, 336, 5120), (40, 48, 1056)])
def test_wperm_gives_the_same_result(backend, m, n, k):
    """gemm_mxfp4_wmma with wperm = 1 on the permuted copy equals wperm = 0 on the GGUF layout bit
    for bit, in every regime (single row, few rows, tiled; ragged last tiles; a K the tiled kernel
    does not take); the permuted copy's dequant dump after permuting back is the oracle's."""
    g = synth.rng(31 * m + n + k)
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    x = synth.activations_bf16_outliers(g, m, k)
    wp = oracle.permute_mxfp4_to_wmma(w, n, k)
    dx = backend.Upload(x)
    da8, das = backend.AllocateBuffer(m * k), backend.AllocateBuffer(4 * m)
    dref = backend.AllocateBuffer(n)
    run(backend, "quantize_fp8_pack_rows", [dx, da8, das], [m, k], grid=(m, 1, 1))
    outs = []
    for weights, wperm in ((w, 0), (wp, 1)):
        dw, out = backend.Upload(weights), backend.AllocateBuffer(4 * m * n)
        run(backend, "gemm_mxfp4_wmma", [da8, dw, das, dref, out], [m, n, k, 1, wperm], grid=((n + 63) // 64, 1, 1))
        backend.Synchronize()
        outs.append(backend.CopyD2H(out, dtype=np.float32))
    assert np.array_equal(outs[0], outs[1])
    codes, scale = oracle.quantize_fp8_pack(x, m, k)
    ref = oracle.gemm_mxfp4_w4a8(codes, scale, w, m, n, k)
    assert rms_err(outs[1].reshape(m, n), ref) <= 5e-4


def test_wperm_needs_whole_fragments(backend):
    from tessera_amd import StatusCode, StatusError
    g = synth.rng(8)
    m, n, k = 4, 40, 256                       # n is not a multiple of 16
    w = synth.mxfp4_weights(g, n, k)
    bufs = [backend.AllocateBuffer(m * k), backend.Upload(w), backend.AllocateBuffer(4 * m), backend.AllocateBuffer(n),
            backend.AllocateBuffer(4 * m * n)]
    with pytest.raises(StatusError) as e:
        run(backend, "gemm_mxfp4_wmma", bufs, [m, n, k, 1, 1])
    assert e.value.code == StatusCode.InvalidArgument
