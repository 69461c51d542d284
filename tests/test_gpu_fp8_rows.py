"""FP8 E4M3 weights (one fp32 scale per row, "gemm_fp8") times 2..16 fp32 rows on the matrix cores:
from 16 M weights on, with k a multiple of 512, the weights are the scaled matrix instruction's second
operand as stored and each fp32 row goes in as four E4M3 terms (16 significant bits kept per element),
eight rows a pass over the weights.  Reference kernel src/backends/rocm/rocm_kernels_basic.cpp:1039-1064,
CPU GemmFp8Ref.  The matrix core aligns the products of an instruction to the largest before adding
them (as for MXFP4 weights on the same instruction, tests/test_gpu_gemm_mxfp4_f32.py), which bounds the
result, not the terms: asserted max|d| <= 2e-4 of the rms output against the oracle (measured 6e-5 to
1.5e-4 over up to 525 k outputs; 2e-3 with x20 outlier channels, measured up to 9e-4) and 2e-5 / 1e-4 in the
2-norm (measured 1.5e-5 / 4.5e-5); single products (one-hot rows of up to 12 significant bits) bit for bit.

"gemm_fp8_block" (one fp32 scale per 128 x 128 block, src/backends/rocm/rocm_kernels_basic.cpp:1066-1089)
takes the same path: an instruction's 128 of K are one block column, its sum is multiplied by the block's
scale before it joins the fp32 accumulator.  Same bounds; one-hot rows of powers of two bit for bit."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import norm_err, rms_err, run, same_bits_zero_sign_free

pytestmark = pytest.mark.gpu
LUT = np.array([oracle.fp8_e4m3_to_float(c) for c in range(256)], np.float32)


def fp8_gemm(backend, a, codes, scales, m, n, k):
    da, dw, ds = backend.Upload(a), backend.Upload(codes), backend.Upload(scales)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_fp8", [da, dw, ds, dc], [m, n, k], grid=((m * n + 255) // 256, 1, 1))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


@pytest.mark.parametrize("m,n,k", [(2, 4100, 4096), (3, 8200, 2048), (4, 3300, 5120), (5, 16390, 1024), (7, 4100, 4096),
                                   (8, 3300, 5120), (9, 16390, 1024), (13, 1030, 17408), (16, 3300, 5120), (16, 32800, 512),
                                   (3, 33, 524288), (2, 17, 1048576)])      # the last two: a few very long rows
@pytest.mark.parametrize("kind", ["f32", "bf16_outliers"])
def test_rows_match_oracle(backend, m, n, k, kind):
    g = synth.rng(5100 * m + n + k)
    codes, scales = synth.fp8_weights(g, n, k)
    a = {"f32": synth.activations_f32, "bf16_outliers": synth.activations_bf16_outliers}[kind](g, m, k)
    ref = oracle.gemm_fp8(a, codes, scales, m, n, k)
    got = fp8_gemm(backend, a, codes, scales, m, n, k)
    tol, tol_norm = (2e-3, 1e-4) if kind == "bf16_outliers" else (2e-4, 2e-5 if k <= 65536 else 4e-5)   # (the oracle's own fp32 sum over half a million terms)
    print(f"gemm_fp8 {m}x{n}x{k} {kind}: max|d|/rms {rms_err(got, ref):.2e}, 2-norm {norm_err(got, ref):.2e}")
    assert rms_err(got, ref) <= tol and norm_err(got, ref) <= tol_norm


def test_one_hot_zero_and_non_finite_rows(backend):
    g = synth.rng(5200)
    m, n, k = 7, 4100, 4096
    codes, scales = synth.fp8_weights(g, n, k)
    lut = LUT[codes].reshape(n, k)
    pos = [0, 15, 16, 777, 4095, 2048]
    vals = np.array([1.0, 1.5, -0.8125, 3.99609375, 2.0 ** -20, -(2.0 ** 7)], np.float32)   # up to 12 significant bits
    a = np.zeros((m, k), np.float32)
    for r, (t, v) in enumerate(zip(pos, vals)):
        a[r, t] = v
    got = fp8_gemm(backend, a, codes, scales, m, n, k)
    for r, (t, v) in enumerate(zip(pos, vals)):
        # the device scales the sum of exact products by the weight row's scale: one rounding; for a
        # power of two that is the reference's a * (scale * w) bit for bit, otherwise within its last place
        assert same_bits_zero_sign_free(got[r], (lut[:, t] * v) * scales), (r, t)
        want = (scales * lut[:, t]) * v
        if float(np.log2(abs(v))).is_integer():
            assert same_bits_zero_sign_free(got[r], want), (r, t)
        else:
            assert np.all(np.abs(got[r] - want) <= np.spacing(np.abs(want))), (r, t)
    assert np.all(got[6] == 0.0)
    a = synth.activations_f32(g, m, k)
    a[2, 100] = np.inf
    a[4, 7] = np.nan
    got = fp8_gemm(backend, a, codes, scales, m, n, k)
    good = [0, 1, 3, 5, 6]
    assert not np.isfinite(got[[2, 4]]).any() and np.isfinite(got[good]).all()
    assert rms_err(got[good], oracle.gemm_fp8(a[good], codes, scales, 5, n, k)) <= 1e-4


@pytest.mark.parametrize("m", [2, 8])
def test_every_weight_code_through_the_matrix_operand(backend, m):
    """All 256 codes as weights (row r holds code r along its whole length) under unit scales and one-hot
    rows at every chunk position of a stage: the instruction's E4M3 decode against Fp8E4M3ToFloat,
    subnormal codes and both NaN codes included."""
    n, k = 256, 65536
    codes = np.repeat(np.arange(n, dtype=np.uint8), k)
    scales = np.ones(n, np.float32)
    g = synth.rng(5300 + m)
    pos = [int(t) for t in g.integers(0, k, m)]
    got = fp8_gemm(backend, synth.one_hot_rows(k, pos), codes, scales, m, n, k)
    nan = np.isnan(LUT)
    for r in range(m):
        assert np.array_equal(np.isnan(got[r]), nan)
        assert same_bits_zero_sign_free(got[r][~nan], LUT[~nan]), (m, r)


def test_a_nan_weight_stays_in_its_column(backend):
    g = synth.rng(5400)
    m, n, k = 4, 3300, 5120
    codes, scales = synth.fp8_weights(g, n, k)
    codes = codes.reshape(n, k).copy()
    bad = [0, 67, 68, 3299]
    for c in bad:
        codes[c, (37 * c) % k] = 0x7F
    codes = codes.reshape(-1)
    a = synth.activations_f32(g, m, k)
    got = fp8_gemm(backend, a, codes, scales, m, n, k)
    with np.errstate(invalid="ignore"):
        ref = oracle.gemm_fp8(a, codes, scales, m, n, k)
    good = [c for c in range(n) if c not in bad]
    assert np.isnan(got[:, bad]).all() and np.isnan(ref[:, bad]).all()
    assert rms_err(got[:, good], ref[:, good]) <= 1e-4


@pytest.mark.parametrize("n,k", [(17408, 5120), (5120, 17408)])
def test_full_size_rows(backend, n, k):
    """The 27B FFN shapes, 4 and 16 rows, every output against the oracle."""
    g = synth.rng(5500 + n)
    codes, scales = synth.fp8_weights(g, n, k)
    for m in (4, 16):
        a = synth.activations_f32(g, m, k)
        ref = oracle.gemm_fp8(a, codes, scales, m, n, k)
        got = fp8_gemm(backend, a, codes, scales, m, n, k)
        print(f"gemm_fp8 {m} rows {n}x{k}: max|d|/rms {rms_err(got, ref):.2e}, 2-norm {norm_err(got, ref):.2e}")
        assert rms_err(got, ref) <= 1e-4 and norm_err(got, ref) <= 2e-5


# ---- one scale per 128 x 128 block ----------------------------------------------------------------
def fp8_block_gemm(backend, a, codes, scales, m, n, k):
    da, dw, ds = backend.Upload(a), backend.Upload(codes), backend.Upload(scales)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_fp8_block", [da, dw, ds, dc], [m, n, k], grid=((m * n + 255) // 256, 1, 1))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


@pytest.mark.parametrize("m,n,k", [(2, 4096, 4096), (3, 8192, 2048), (4, 3328, 5120), (5, 16384, 1024), (8, 3328, 5120),
                                   (9, 4224, 4096), (13, 1024, 17408), (16, 3328, 5120), (16, 32768, 512),
                                   (3, 128, 262144)])
@pytest.mark.parametrize("kind", ["f32", "bf16_outliers"])
def test_block_scaled_rows_match_oracle(backend, m, n, k, kind):
    g = synth.rng(5600 * m + n + k)
    codes, scales = synth.fp8_block_weights(g, n, k)
    a = {"f32": synth.activations_f32, "bf16_outliers": synth.activations_bf16_outliers}[kind](g, m, k)
    ref = oracle.gemm_fp8_block(a, codes, scales, m, n, k)
    got = fp8_block_gemm(backend, a, codes, scales, m, n, k)
    tol, tol_norm = (2e-3, 1e-4) if kind == "bf16_outliers" else (2e-4, 2e-5 if k <= 65536 else 4e-5)
    print(f"gemm_fp8_block {m}x{n}x{k} {kind}: max|d|/rms {rms_err(got, ref):.2e}, 2-norm {norm_err(got, ref):.2e}")
    assert rms_err(got, ref) <= tol and norm_err(got, ref) <= tol_norm


def test_block_scaled_one_hot_rows_pick_their_block(backend):
    """One-hot rows of powers of two at positions in different block columns, on weight rows that span
    every block row: each output is code x block scale x value, so a scale taken from a neighbouring
    block (row or column) shows."""
    g = synth.rng(5700)
    m, n, k = 6, 4224, 4096              # 33 block rows (a workgroup's rows straddle them), 32 block columns
    codes, scales = synth.fp8_block_weights(g, n, k)
    lut = LUT[codes].reshape(n, k)
    sc = scales.reshape(n // 128, k // 128)
    pos = [0, 127, 128, 2049, 4095]
    vals = np.array([1.0, 2.0 ** -20, -(2.0 ** 7), 0.5, 2.0 ** 30], np.float32)
    a = np.zeros((m, k), np.float32)
    for r, (t, v) in enumerate(zip(pos, vals)):
        a[r, t] = v
    got = fp8_block_gemm(backend, a, codes, scales, m, n, k)
    for r, (t, v) in enumerate(zip(pos, vals)):
        want = (np.repeat(sc[:, t // 128], 128) * lut[:, t]) * v
        assert same_bits_zero_sign_free(got[r], want), (r, t)
    assert np.all(got[5] == 0.0)


def test_block_scaled_full_size_rows(backend):
    g = synth.rng(5800)
    n, k = 17408, 5120
    codes, scales = synth.fp8_block_weights(g, n, k)
    for m in (4, 16):
        a = synth.activations_f32(g, m, k)
        ref = oracle.gemm_fp8_block(a, codes, scales, m, n, k)
        got = fp8_block_gemm(backend, a, codes, scales, m, n, k)
        print(f"gemm_fp8_block {m} rows {n}x{k}: max|d|/rms {rms_err(got, ref):.2e}, 2-norm {norm_err(got, ref):.2e}")
        assert rms_err(got, ref) <= 2e-4 and norm_err(got, ref) <= 2e-5
