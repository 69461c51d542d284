"""MXFP4 weights times fp32 activation rows on the matrix cores (gemm_mxfp4 / gemm_mxfp4_batched from
17 rows on, the id ProjectBatch issues for MXFP4 prefill, src/core/decode_internal.hpp:1494-1504;
reference kernel src/backends/rocm/rocm_kernels_basic.cpp:1221-1282, CPU GemmMxFp4Ref).

The contract is fp32 activations, no activation quantization.  The device writes each row as a
sum of E4M3 terms, a = s0 (h0 + h1/16 + h2/256 + h3/4096) with s0 a power of two, each h the four
leading significant bits of what the terms before it left (`split_model` below restates it), and
multiplies every term by the unchanged E2M1 x E8M0 weights on the scaled MFMA, all terms into one
fp32 accumulator.  Rows whose values have at most 8 significant bits (bf16-valued, the prefill
configuration) take two terms and are reproduced exactly down to rowmax * 2^-20; up to 12 bits
three terms; other rows four terms, which keep 16 significant bits.  Two checks follow from that:

* against the float64 product of the split rows and the exact weights the device may differ by
  its accumulation only (products are exact).  The matrix core aligns the 64 products of an
  instruction to the largest before adding them, so an instruction that holds a x20 outlier
  channel drops low bits of its small products: asserted 1e-4 of the rms output (measured 2e-5 to
  5e-5) for N(0,1) rows, 5e-4 (measured 1.5e-4) with the x20 outlier channels of configs[2];
* against the oracle's fp32 GemmMxFp4Ref the same two bounds, and 2e-5 / 5e-5 in the 2-norm,
  bf16-valued or fp32-valued rows alike (16 kept bits cost 2^-17 per element, far below the
  accumulation).  These are the bounds of the W4A8 id on the same instruction
  (tests/test_gpu_gemm_mxfp4.py), without that id's E4M3 rounding of the activation."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import norm_err, rms_err, run, same_bits_zero_sign_free

pytestmark = pytest.mark.gpu
ACC_TOL, ORACLE_NORM = 1e-4, 2e-5                         # N(0,1) rows
ACC_TOL_OUTLIERS, ORACLE_NORM_OUTLIERS = 5e-4, 5e-5       # rows with x20 outlier channels


def mx_gemm(backend, name, a, w, m, n, k):
    da, dw = backend.Upload(a), backend.Upload(w)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, name, [da, dw, dc], [m, n, k], grid=((m * n + 7) // 8, 1, 1))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


def cut4(x):
    """|x| < 256 cut (toward zero) to the E4M3 grid: four significant bits from 2^-6 up, multiples
    of 2^-9 below."""
    ax = np.abs(x)
    mant, exp = np.frexp(ax)
    normal = np.ldexp(np.floor(mant * 16.0) / 16.0, exp)
    return np.copysign(np.where(ax >= 2.0 ** -6, normal, np.floor(ax * 512.0) / 512.0), x)


def near4(x):
    ax = np.abs(x)
    mant, exp = np.frexp(ax)
    normal = np.ldexp(np.rint(mant * 16.0) / 16.0, exp)            # ties to even, as the device
    return np.copysign(np.where(ax >= 2.0 ** -6, normal, np.rint(ax * 512.0) / 512.0), x)


def split_model(a, terms):
    """What `terms` E4M3 terms keep of fp32 rows, in float64 (all steps are exact in fp32 too)."""
    a = np.asarray(a, np.float32).astype(np.float64)
    amax = np.max(np.abs(a), axis=1)
    e = np.where(amax > 0, np.floor(np.log2(np.where(amax > 0, amax, 1.0))), 7.0)
    s0 = np.exp2(e - 7.0)[:, None]
    r = a / s0
    kept = np.zeros_like(r)
    for t in range(terms):
        h = near4(r) if t == 3 else cut4(r)
        kept += h / 16.0 ** t
        r = (r - h) * 16.0
    return kept * s0


def check(got, a, w, m, n, k, terms, ref, what, outliers=False):
    deq = oracle.dequantize_mxfp4(w, n, k).astype(np.float64)
    sim = split_model(a, terms) @ deq.T
    acc = rms_err(got, sim)
    print(f"{what}: vs split-row product {acc:.2e}; vs fp32 oracle max|d|/rms {rms_err(got, ref):.2e}, "
          f"2-norm {norm_err(got, ref):.2e}")
    tol, tol_norm = (ACC_TOL_OUTLIERS, ORACLE_NORM_OUTLIERS) if outliers else (ACC_TOL, ORACLE_NORM)
    assert acc <= tol, (what, acc)
    assert rms_err(got, ref) <= tol and norm_err(got, ref) <= tol_norm, (what, rms_err(got, ref), norm_err(got, ref))


SHAPES = [(17, 200, 1024), (20, 131, 5120), (33, 64, 2048), (64, 515, 1280), (100, 96, 4096), (130, 257, 1024),
          (300, 520, 2048), (513, 320, 1152)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("kind", ["bf16", "bf16_outliers", "f32"])
def test_gemm_matches_oracle(backend, m, n, k, kind):
    g = synth.rng(2100 * m + n + k)
    w = synth.mxfp4_weights(g, n, k)
    a = {"bf16": synth.activations_bf16, "bf16_outliers": synth.activations_bf16_outliers,
         "f32": synth.activations_f32}[kind](g, m, k)
    ref = oracle.gemm_mxfp4(a, w, m, n, k, threads=True)
    for name in ("gemm_mxfp4_batched", "gemm_mxfp4"):
        got = mx_gemm(backend, name, a, w, m, n, k)
        check(got, a, w, m, n, k, 4 if kind == "f32" else 2, ref, f"{name} {m}x{n}x{k} {kind}", kind == "bf16_outliers")


def test_split_keeps_what_it_says(backend):
    """One-hot rows (every output is one product, exact in fp32): values of 8 significant bits
    come back exactly, values of 12 bits too (three terms), a full fp32 value to 16 bits; block
    scales over a wide range; every E2M1 code."""
    g = synth.rng(41)
    m, n, k = 96, 128, 1024
    w = synth.mxfp4_weights(g, n, k, -30, 30)
    deq = oracle.dequantize_mxfp4(w, n, k)
    pos = [int(p) for p in g.permutation(k)[:m]]
    for bits in (8, 12, 24):
        vals = g.standard_normal(m).astype(np.float32) * np.exp2(g.integers(-20, 20, m)).astype(np.float32)
        if bits < 24:
            vals = (vals.view(np.uint32) & np.uint32((0xFFFFFFFF << (24 - bits)) & 0xFFFFFFFF)).view(np.float32)
        a = synth.one_hot_rows(k, pos) * vals[:, None]
        got = mx_gemm(backend, "gemm_mxfp4_batched", a, w, m, n, k)
        for r, t in enumerate(pos):
            want = deq[:, t] * vals[r]
            if bits < 24:
                assert same_bits_zero_sign_free(got[r], want), (bits, r, t)
            else:
                assert np.all(np.abs(got[r] - want) <= np.abs(want) * 2.0 ** -16), (bits, r, t)


def test_small_values_beside_a_large_one(backend):
    """A row's values far below its largest: exact down to rowmax * 2^-13 (two terms, bf16-valued),
    and within rowmax * 2^-20 per element below that."""
    g = synth.rng(43)
    m, n, k = 64, 64, 1024
    w = synth.mxfp4_weights(g, n, k, -2, 2)
    a = synth.activations_bf16(g, m, k) * np.exp2(-g.integers(0, 24, size=(m, k))).astype(np.float32)
    a[:, 0] = 200.0
    ref = oracle.gemm_mxfp4(a, w, m, n, k, threads=True)
    got = mx_gemm(backend, "gemm_mxfp4_batched", a, w, m, n, k)
    deq = oracle.dequantize_mxfp4(w, n, k).astype(np.float64)
    kept = split_model(a, 2)
    assert np.max(np.abs(kept - a)) <= 200.0 * 2.0 ** -20
    big = np.abs(a) >= 256.0 * 2.0 ** -13
    assert np.array_equal(kept[big], a.astype(np.float64)[big])
    assert rms_err(got, kept @ deq.T) <= ACC_TOL_OUTLIERS
    assert rms_err(got, ref) <= ACC_TOL_OUTLIERS


def test_rows_of_zeros_and_non_finite_rows(backend):
    """An all-zero row gives zeros; a row holding an infinity or a NaN comes back non-finite and
    leaves the other rows alone."""
    g = synth.rng(44)
    m, n, k = 40, 96, 1024
    w = synth.mxfp4_weights(g, n, k)
    a = synth.activations_bf16(g, m, k)
    a[3] = 0.0
    a[7, 100] = np.inf
    a[21, 5] = np.nan
    got = mx_gemm(backend, "gemm_mxfp4_batched", a, w, m, n, k)
    good = [r for r in range(m) if r not in (7, 21)]
    with np.errstate(invalid="ignore"):
        ref = oracle.gemm_mxfp4(a[good], w, len(good), n, k, threads=True)
    assert np.all(got[3] == 0.0)
    assert not np.isfinite(got[7]).any() and not np.isfinite(got[21]).any()
    assert rms_err(got[good], ref) <= ACC_TOL


def test_full_size_prefill_rows(backend):
    """BASELINE configs[3], MXFP4 leg with the reference's default id (fp32 rows, here bf16-valued):
    M=2048, N=17408, K=5120 and one rank's column shard N=8704.  Every element against the float64
    product of the split rows; 72 rows (every position of a 32-row MFMA tile, all eight 256-row
    tiles, all columns: the 256x256 tiles and the 128x64 ones that take the leftover columns)
    against the fp32 oracle; the shard equals the first half of the columns bit for bit."""
    g = synth.rng(31339)
    m, n, k = 2048, 17408, 5120
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    a = synth.activations_bf16(g, m, k)
    got = mx_gemm(backend, "gemm_mxfp4_batched", a, w, m, n, k)
    deq = oracle.dequantize_mxfp4(w, n, k).astype(np.float64)
    sim = split_model(a, 2) @ deq.T
    del deq
    assert rms_err(got, sim) <= ACC_TOL, rms_err(got, sim)
    rows = sorted({(37 * i) % 2048 for i in range(64)} | {0, 31, 32, 255, 256, 1023, 2016, 2047})
    assert {r % 32 for r in rows} == set(range(32)) and {r // 256 for r in rows} == set(range(8))
    ref = oracle.gemm_mxfp4(a[rows], w, len(rows), n, k, threads=True)
    print(f"configs[3] MXFP4 fp32-row id, 72 rows: vs fp32 oracle max|d|/rms {rms_err(got[rows], ref):.2e}, "
          f"2-norm {norm_err(got[rows], ref):.2e}; all rows vs split-row product {rms_err(got, sim):.2e}")
    assert rms_err(got[rows], ref) <= ACC_TOL and norm_err(got[rows], ref) <= ORACLE_NORM
    shard = synth.mxfp4_column_shard(w, n, k, 0, n // 2)
    got_shard = mx_gemm(backend, "gemm_mxfp4_batched", a, shard, m, n // 2, k)
    assert np.array_equal(got_shard, got[:, : n // 2])


# ---- 2..16 fp32 rows of a large matrix: the same terms through the streamed few-row kernel ----
@pytest.mark.parametrize("m,n,k", [(2, 4100, 4096), (4, 3300, 5120), (5, 4100, 4096), (8, 3300, 5120), (9, 4100, 4096),
                                   (13, 1030, 17408), (16, 3300, 5120)])
@pytest.mark.parametrize("kind", ["bf16", "bf16_outliers", "f32"])
def test_few_rows_on_the_matrix_cores_match_oracle(backend, m, n, k, kind):
    """gemm_mxfp4 / gemm_mxfp4_rows with 2..16 rows against 16 M weights or more (the reference's one
    warp per column with 16 accumulators, src/backends/rocm/rocm_kernels_basic.cpp:1153-1214): always
    four terms, eight rows a weight pass; same bounds as from 17 rows."""
    g = synth.rng(2300 * m + n + k)
    w = synth.mxfp4_weights(g, n, k)
    a = {"bf16": synth.activations_bf16, "bf16_outliers": synth.activations_bf16_outliers,
         "f32": synth.activations_f32}[kind](g, m, k)
    ref = oracle.gemm_mxfp4(a, w, m, n, k, threads=True)
    for name in ("gemm_mxfp4_rows", "gemm_mxfp4"):
        got = mx_gemm(backend, name, a, w, m, n, k)
        check(got, a, w, m, n, k, 4, ref, f"{name} {m}x{n}x{k} {kind}", kind == "bf16_outliers")


def test_few_rows_one_hot_and_zero_rows(backend):
    """One-hot rows of 8- and 12-bit values return single exact products (which lane supplies which
    block, the term order, the 16^-t weights); a zero row gives zeros; a non-finite element spoils its
    row only."""
    g = synth.rng(2400)
    m, n, k = 6, 4100, 4096
    w = synth.mxfp4_weights(g, n, k, -20, 20)
    deq = oracle.dequantize_mxfp4(w, n, k)
    pos = [0, 31, 32, 777, 4095]
    vals = np.array([1.0, 1.5, 0.8125, 3.99609375, 2.0 ** -20], np.float32)      # up to 12 significant bits
    a = np.zeros((m, k), np.float32)
    for r, (t, v) in enumerate(zip(pos, vals)):
        a[r, t] = v
    got = mx_gemm(backend, "gemm_mxfp4_rows", a, w, m, n, k)
    for r, (t, v) in enumerate(zip(pos, vals)):
        assert same_bits_zero_sign_free(got[r], deq[:, t] * v), (r, t)
    assert np.all(got[5] == 0.0)
    a = synth.activations_f32(g, m, k)
    a[2, 100] = np.inf
    a[4, 7] = np.nan
    got = mx_gemm(backend, "gemm_mxfp4_rows", a, w, m, n, k)
    assert not np.isfinite(got[[2, 4]]).any() and np.isfinite(got[[0, 1, 3, 5]]).all()
