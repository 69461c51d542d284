"""GPU parity of the one-pass several-row kernels for Q5_K and Q6_K (int8 matrix cores, weights read
once for up to eight resp. four activation rows) against the oracle: decode exactness through one-hot
rows, every row count of a pass and across passes, ragged and tiny shapes, the 27B FFN shapes.  The
same kernel takes Q4_K with two rows on matrices of 16 M weights or more whose rows are at most 5120
long: covered at the end (three and four rows of those shapes run beside it for comparison)."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import ref_grid_vec, rel_err, rms_err, run, same_bits_zero_sign_free, strict_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-3

FORMATS = {
    "q5k": (synth.q5k_weights, oracle.gemm_q5k, oracle.dequantize_q5k, 176),
    "q6k": (synth.q6k_weights, oracle.gemm_q6k, oracle.dequantize_q6k, 210),
}


def gemm(backend, name, a, w, m, n, k):
    da, dw = backend.Upload(a), backend.Upload(w)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, name, [da, dw, dc], [m, n, k], grid=ref_grid_vec(m, n))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
@pytest.mark.parametrize("m", [2, 3, 4, 5, 7, 8, 9, 13, 16])
def test_one_hot_rows_reproduce_dequant_bit_exact(backend, fmt, m):
    """Rows that are one-hot, scaled by powers of two over the fp32 range, return columns of
    deq(W) times that power: nibble and high-bit assembly, scales, mins or offset, the limb split of
    the activations and the per-block power of two are all exact."""
    make, _, deq_fn, _ = FORMATS[fmt]
    g = synth.rng(7100 + m)
    n, k = 83, 1536
    w = make(g, n, k)
    deq = deq_fn(w).reshape(n, k).astype(np.float64)
    for scale in (1.0, 2.0 ** -100, 2.0 ** 90, -(2.0 ** -3)):
        pos = [int(t) for t in g.integers(0, k, m)]
        a = synth.one_hot_rows(k, pos) * np.float32(scale)
        got = gemm(backend, f"gemm_{fmt}", a, w, m, n, k)
        for r, t in enumerate(pos):
            want = (deq[:, t] * scale).astype(np.float32)
            assert same_bits_zero_sign_free(got[r], want), (fmt, m, scale, r, t)


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
@pytest.mark.parametrize("m", [2, 3, 4, 6, 8, 11, 16])
@pytest.mark.parametrize("n,k", [(1, 256), (15, 512), (16, 256), (17, 768), (250, 1024), (1000, 2048), (4099, 2048),
                                 (3001, 4352), (700, 5120), (300, 17408)])
def test_rows_match_oracle(backend, fmt, m, n, k):
    if m > 8 and n * k > 4 << 20:
        pytest.skip("more than one pass of rows is covered on the smaller shapes and at full size")
    make, ref_fn, _, _ = FORMATS[fmt]
    g = synth.rng(7200 + 13 * m + n + k)
    w = make(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = ref_fn(a, w, m, n, k, threads=True)
    got = gemm(backend, f"gemm_{fmt}", a, w, m, n, k)
    assert rel_err(got, ref) <= TOL, (fmt, m, n, k, rel_err(got, ref))
    assert rms_err(got, ref) < 5e-5, (fmt, m, n, k, rms_err(got, ref))


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
def test_rows_with_wide_dynamic_range_inside_a_block(backend, fmt):
    """Activations whose magnitudes span 2^40 inside one 256-wide block: the four limbs keep 30 bits
    under the block's largest value, so what is lost stays below 2^-29 of that value per element."""
    make, ref_fn, _, _ = FORMATS[fmt]
    g = synth.rng(7300)
    m, n, k = 4, 333, 2048
    w = make(g, n, k)
    a = synth.activations_f32(g, m, k) * np.exp2(g.integers(-20, 21, (m, k))).astype(np.float32)
    ref = ref_fn(a, w, m, n, k, threads=True)
    got = gemm(backend, f"gemm_{fmt}", a, w, m, n, k)
    assert rel_err(got, ref) <= TOL and rms_err(got, ref) < 5e-5


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
def test_a_non_finite_activation_stays_in_its_row(backend, fmt):
    make, ref_fn, _, _ = FORMATS[fmt]
    g = synth.rng(7400)
    m, n, k = 5, 130, 1024
    w = make(g, n, k)
    for bad in (np.inf, -np.inf, np.nan):
        a = synth.activations_f32(g, m, k)
        a[2, 700] = bad
        got = gemm(backend, f"gemm_{fmt}", a, w, m, n, k)
        assert not np.isfinite(got[2]).any(), (fmt, bad)
        good = [0, 1, 3, 4]
        ref = ref_fn(a[good], w, 4, n, k)
        assert rel_err(got[good], ref) <= TOL


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
def test_a_non_finite_weight_block_stays_in_its_row(backend, fmt):
    make, ref_fn, _, bb = FORMATS[fmt]
    g = synth.rng(7500)
    m, n, k = 4, 67, 1280
    w = make(g, n, k).reshape(n, -1)
    d_at = 0 if fmt == "q5k" else 208
    bad_rows = [3, 40, 66]
    for r in bad_rows:
        blk = r % (k // 256)
        w[r, bb * blk + d_at:bb * blk + d_at + 2] = np.array([0x00, 0x7C], np.uint8)   # d = +inf
    w = w.reshape(-1)
    a = synth.activations_f32(g, m, k)
    got = gemm(backend, f"gemm_{fmt}", a, w, m, n, k)
    with np.errstate(invalid="ignore", over="ignore"):
        ref = ref_fn(a, w, m, n, k)
    good = [r for r in range(n) if r not in bad_rows]
    assert not np.isfinite(got[:, bad_rows]).any() and not np.isfinite(ref[:, bad_rows]).any()
    assert rel_err(got[:, good], ref[:, good]) <= TOL


@pytest.mark.parametrize("fmt,m", [("q5k", 2), ("q5k", 4), ("q5k", 8), ("q5k", 16), ("q6k", 3), ("q6k", 4), ("q6k", 8)])
@pytest.mark.parametrize("n,k", [(17408, 5120), (5120, 17408)])
def test_full_size_rows(backend, fmt, m, n, k):
    """The 27B FFN shapes, every output of every row against the threaded oracle; the figure with the
    small floor (1e-3 of the rms) is printed beside the asserted one."""
    make, ref_fn, _, _ = FORMATS[fmt]
    g = synth.rng(7600 + m + n)
    w = make(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = ref_fn(a, w, m, n, k, threads=True)
    got = gemm(backend, f"gemm_{fmt}", a, w, m, n, k)
    print(f"{fmt} {m} rows {n}x{k}: rel_err {rel_err(got, ref):.2e} (floor 0.05 rms), "
          f"{strict_rel_err(got, ref):.2e} (floor 1e-3 rms), max|d|/rms {rms_err(got, ref):.2e}")
    assert rel_err(got, ref) <= TOL and rms_err(got, ref) < 5e-5


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
def test_rows_ids_and_split_regions(backend, fmt):
    """The reference's per-row-count ids with a split: the sum in region 0, zeros behind."""
    make, ref_fn, _, _ = FORMATS[fmt]
    g = synth.rng(7700)
    n, k, split = 515, 2048, 4
    w = make(g, n, k)
    for rows in (2, 3, 4, 5):
        a = synth.activations_f32(g, rows, k)
        da, dw = backend.Upload(a), backend.Upload(w)
        dc = backend.AllocateBuffer(4 * rows * n * split)
        run(backend, f"gemm_{fmt}_rows{rows}", [da, dw, dc], [rows, n, k, split], grid=ref_grid_vec(rows, n))
        backend.Synchronize()
        got = backend.CopyD2H(dc, dtype=np.float32).reshape(split, rows, n)
        assert rel_err(got.sum(axis=0), ref_fn(a, w, rows, n, k)) <= TOL
        assert np.all(got[1:] == 0.0)


Q4K_SHAPES = [(3300, 5120), (8200, 2048), (16390, 1024), (4099, 4096), (17408, 5120)]


@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("n,k", Q4K_SHAPES[:4])
def test_q4k_one_hot_rows_bit_exact(backend, m, n, k):
    g = synth.rng(7800 + m + n)
    w = synth.q4k_weights(g, n, k)
    deq = oracle.dequantize_q4k(w).reshape(n, k).astype(np.float64)
    for scale in (1.0, 2.0 ** -100, 2.0 ** 90, -(2.0 ** -3)):
        pos = [int(t) for t in g.integers(0, k, m)]
        a = synth.one_hot_rows(k, pos) * np.float32(scale)
        got = gemm(backend, "gemm_q4k_batched", a, w, m, n, k)
        for r, t in enumerate(pos):
            assert same_bits_zero_sign_free(got[r], (deq[:, t] * scale).astype(np.float32)), (m, n, k, scale, r, t)


@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("n,k", Q4K_SHAPES)
def test_q4k_rows_match_oracle(backend, m, n, k):
    g = synth.rng(7900 + m + n)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    for name in ("gemm_q4k", "gemm_q4k_batched"):
        got = gemm(backend, name, a, w, m, n, k)
        assert rel_err(got, ref) <= TOL and rms_err(got, ref) < 5e-5, (name, m, n, k, rel_err(got, ref), rms_err(got, ref))


def test_q4k_non_finite_values_stay_in_their_row(backend):
    g = synth.rng(7950)
    m, n, k = 3, 3300, 5120
    w = synth.q4k_weights(g, n, k).reshape(n, -1)
    bad_rows = [5, 1700, 3299]
    for r in bad_rows:
        w[r, 144 * (r % 20):144 * (r % 20) + 2] = np.array([0x00, 0x7C], np.uint8)   # d = +inf
    w = w.reshape(-1)
    a = synth.activations_f32(g, m, k)
    a[1, 4000] = np.nan
    got = gemm(backend, "gemm_q4k_batched", a, w, m, n, k)
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.gemm_q4k(a[[0, 2]], w, 2, n, k, threads=True)
    good = [r for r in range(n) if r not in bad_rows]
    assert not np.isfinite(got[1]).any()
    assert not np.isfinite(got[:, bad_rows]).any()
    assert rel_err(got[[0, 2]][:, good], ref[:, good]) <= TOL
