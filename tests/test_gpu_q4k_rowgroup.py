"""GPU parity of the load-time row-group copy of a Q4_K matrix (`permute_q4k_rowgroup`, the `layout`
scalar of the Q4_K GEMM ids) and of the int8 matrix-core decode GEMV that reads it, through the C ABI.

The copy is a permutation of the GGUF bytes: the device's against the oracle's element-by-element
statement of the order, both ways, bit for bit.  The GEMV over it is held to what the GEMV over
the GGUF order is held to: one-hot rows return the reference's dequantized weight bit for bit, any
row lands within max relative error 1e-3 of the reference's fp32 sequential sum (it keeps 30 bits
of every activation under its block's largest, so it lands within the reference sum's own rounding noise, a few 1e-6 of the rms output at K = 5120;
the tests assert 5e-5)."""
import numpy as np
import pytest

import oracle
from tessera_amd import StatusCode, StatusError, synth
from util import ref_grid_vec, rel_err, rms_err, run, same_bits_zero_sign_free, strict_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-3


def to_rowgroups(backend, w, n, k, rows=0, inverse=False):
    dw = backend.Upload(w)
    out = backend.AllocateBuffer(np.asarray(w).nbytes)
    run(backend, "permute_q4k_rowgroup", [dw, out], [n, k, rows, int(inverse)])
    backend.Synchronize()
    return backend.CopyD2H(out, dtype=np.uint8)


def gemv(backend, name, a, wrg, m, n, k, layout, split=None):
    da, dw = backend.Upload(a), backend.Upload(wrg)
    regions = split or 1
    dc = backend.AllocateBuffer(4 * m * n * regions)
    scalars = [m, n, k] + ([split] if split is not None else []) + [layout]
    run(backend, name, [da, dw, dc], scalars, grid=ref_grid_vec(m, n))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(regions, m, n)


@pytest.mark.parametrize("n,k,rows", [(96, 512, 0), (70, 1024, 32), (33, 256, 16), (100, 768, 64), (5, 256, 7),
                                      (1000, 2048, 20), (67, 5120, 48), (1, 256, 1)])
def test_permutation_matches_the_layout_statement_both_ways(backend, n, k, rows):
    g = synth.rng(900 + n + k)
    w = synth.q4k_weights(g, n, k)
    want = oracle.permute_q4k_rowgroup(w, n, k, rows or 32)
    got = to_rowgroups(backend, w, n, k, rows)
    assert np.array_equal(got, want.reshape(-1))
    back = to_rowgroups(backend, got, n, k, rows, inverse=True)
    assert np.array_equal(back, np.asarray(w).reshape(-1))


@pytest.mark.parametrize("k,rows", [(256, 32), (512, 32), (1024, 20), (768, 64), (2048, 32), (5120, 32)])
def test_one_hot_rows_reproduce_the_block_decode_bit_for_bit(backend, k, rows):
    """The GEMV's own decode of the copy (nibbles minus eight in the high halves, re-packed scales, integer
    scale products, d and dmin last): column t of deq(W) for every position of the first block and a
    spread over the rest, at magnitudes from 2^-100 to 2^90."""
    g = synth.rng(910 + k)
    n = 96 if rows != 20 else 90
    w = synth.q4k_weights(g, n, k)
    deq = oracle.dequantize_q4k(w).reshape(n, k)
    wrg = to_rowgroups(backend, w, n, k, rows)
    pos = list(range(256)) + [int(t) for t in g.integers(0, k, 32)]
    for i, t in enumerate(pos):
        scale = np.float32(2.0) ** [0, -100, 90, -3][i % 4]
        x = synth.one_hot_rows(k, [t]) * scale
        c = gemv(backend, "gemm_q4k_vec", x, wrg, 1, n, k, rows, split=1)[0, 0]
        assert same_bits_zero_sign_free(c, deq[:, t] * scale), (k, t, float(scale))


@pytest.mark.parametrize("n,k,rows", [(64, 256, 32), (33, 512, 32), (100, 1024, 32), (17, 768, 16), (129, 1280, 64),
                                      (256, 2048, 32), (130, 5120, 32), (67, 17408, 32), (40, 4352, 20),
                                      (3001, 768, 32), (6007, 5120, 32), (523, 17408, 48), (1027, 8192, 32),
                                      (2051, 6400, 32), (5, 32768, 32)])
def test_single_row_matches_oracle(backend, n, k, rows):
    g = synth.rng(920 + n)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    wrg = to_rowgroups(backend, w, n, k, rows)
    ref = oracle.gemm_q4k(a, w, 1, n, k)
    for name, split in (("gemm_q4k_vec", 1), ("gemm_q4k", None), ("gemm_q4k_row", None)):
        got = gemv(backend, name, a, wrg, 1, n, k, rows, split=split)[0]
        assert rel_err(got, ref) < TOL and rms_err(got, ref) < 5e-5, (name, rel_err(got, ref), rms_err(got, ref))


def test_split_regions_sum_to_the_result(backend):
    g = synth.rng(930)
    n, k = 300, 5120
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    wrg = to_rowgroups(backend, w, n, k)
    parts = gemv(backend, "gemm_q4k_vec", a, wrg, 1, n, k, 32, split=4)
    assert rel_err(parts.sum(axis=0), oracle.gemm_q4k(a, w, 1, n, k)) < TOL


@pytest.mark.parametrize("m", [2, 4, 8, 16, 40])
def test_other_row_counts_go_through_the_gguf_order(backend, m):
    """More than one activation row: the copy is put back into GGUF order in the workspace and the
    usual regime of that row count runs; the result equals the one from the GGUF tensor bit for bit."""
    g = synth.rng(940 + m)
    n, k = 520, 2048
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    wrg = to_rowgroups(backend, w, n, k)
    name = "gemm_q4k_rows2" if m == 2 else ("gemm_q4k_rows4" if m == 4 else "gemm_q4k_batched")
    if name.startswith("gemm_q4k_rows"):
        got = gemv(backend, name, a, wrg, m, n, k, 32, split=1)[0]
        da, dw, dc = backend.Upload(a), backend.Upload(w), backend.AllocateBuffer(4 * m * n)
        run(backend, name, [da, dw, dc], [m, n, k, 1])
    else:
        got = gemv(backend, name, a, wrg, m, n, k, 32)[0]
        da, dw, dc = backend.Upload(a), backend.Upload(w), backend.AllocateBuffer(4 * m * n)
        run(backend, name, [da, dw, dc], [m, n, k])
    backend.Synchronize()
    direct = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
    assert np.array_equal(got.view(np.uint32), direct.view(np.uint32))
    assert rel_err(got, oracle.gemm_q4k(a, w, m, n, k)) < (TOL if m < 17 else 5e-3)


def test_non_finite_weight_row_stays_in_its_row(backend):
    g = synth.rng(950)
    n, k = 203, 5120
    w = synth.q4k_weights(g, n, k).reshape(n, -1)
    bad = [7, 40, 66, 201]
    for r in bad:
        w[r, 144 * (r % (k // 256)):144 * (r % (k // 256)) + 2] = np.array([0x00, 0x7C], np.uint8)   # d = +inf
    w = w.reshape(-1)
    good = [r for r in range(n) if r not in bad]
    a = synth.activations_f32(g, 1, k)
    wrg = to_rowgroups(backend, w, n, k)
    got = gemv(backend, "gemm_q4k_vec", a, wrg, 1, n, k, 32, split=1)[0, 0]
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.gemm_q4k(a, w, 1, n, k)[0]
    assert not np.isfinite(got[bad]).any() and not np.isfinite(ref[bad]).any()
    assert rel_err(got[good], ref[good]) < TOL


def test_non_finite_activation_spoils_every_output(backend):
    g = synth.rng(951)
    n, k = 64, 1024
    w = synth.q4k_weights(g, n, k)
    wrg = to_rowgroups(backend, w, n, k)
    for bad in (np.inf, np.nan):
        a = synth.activations_f32(g, 1, k)
        a[0, 300] = bad
        got = gemv(backend, "gemm_q4k_vec", a, wrg, 1, n, k, 32, split=1)[0, 0]
        assert not np.isfinite(got).any()


@pytest.mark.parametrize("n,k", [(17408, 5120), (5120, 17408), (5120, 5120)])
def test_full_size_configs_match_oracle(backend, n, k):
    """configs[1] (and configs[0]'s matrix) at full size through the row-group copy, every output
    against the threaded oracle; prints the per-element figure with the small floor as well."""
    g = synth.rng(960 + n)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    wrg = to_rowgroups(backend, w, n, k)
    assert np.array_equal(to_rowgroups(backend, wrg, n, k, inverse=True), np.asarray(w).reshape(-1))
    got = gemv(backend, "gemm_q4k_vec", a, wrg, 1, n, k, 32, split=1)[0]
    ref = oracle.gemm_q4k(a, w, 1, n, k)
    print(f"row-group gemv {n}x{k}: rel_err {rel_err(got, ref):.2e} (floor 0.05 rms), "
          f"{strict_rel_err(got, ref):.2e} (floor 1e-3 rms), max|d|/rms {rms_err(got, ref):.2e}")
    assert rel_err(got, ref) < TOL and rms_err(got, ref) < 5e-5


def test_bad_layout_is_refused(backend):
    g = synth.rng(970)
    n, k = 64, 512
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    with pytest.raises(StatusError) as e:
        gemv(backend, "gemm_q4k_vec", a, w, 1, n, k, 65, split=1)
    assert e.value.code == StatusCode.InvalidArgument
    with pytest.raises(StatusError) as e:
        to_rowgroups(backend, w, n, k, rows=100)
    assert e.value.code == StatusCode.InvalidArgument
