"""GPU parity of the Q4_K decode path against the CPU oracle, through the C ABI.

Two levels (as the path's contract states): dequantized weights bit-exact against the
reference block decode; GEMV outputs within max relative error 1e-3 of the reference's
fp32 sequential-fma result (tests/util.py:rel_err is the metric; the kernels actually land
near 1e-6, the bound is the contract's)."""
import numpy as np
import pytest

import oracle
from tessera_amd import StatusCode, StatusError, synth
from util import ref_grid_vec, rel_err, rms_err, run, same_bits, same_bits_zero_sign_free, strict_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-3


def gemm(backend, name, a, w, m, n, k, extra=()):
    da, dw = backend.Upload(a), backend.Upload(w)
    split = extra[0] if extra else 1
    dc = backend.AllocateBuffer(4 * m * n * split)
    run(backend, name, [da, dw, dc], [m, n, k, *extra], grid=ref_grid_vec(m, n))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(split, m, n)


def test_dequant_dump_bit_exact_all_blocks(backend):
    g = synth.rng(100)
    n, k = 1024, 5120
    w = synth.q4k_weights(g, n, k)
    # edge blocks: all-zero, all-ones quants with extreme scales, negative d, fp16 subnormal d
    blocks = w.reshape(-1, 144)
    blocks[0] = 0
    blocks[1, 4:16] = 0xFF
    blocks[1, 16:] = 0xFF
    blocks[2, 0:2] = np.array([-0.013], np.float16).view(np.uint8)
    blocks[3, 0:2] = np.array([3e-6], np.float16).view(np.uint8)
    nb = blocks.shape[0]
    dw = backend.Upload(w)
    out = backend.AllocateBuffer(nb * 1024)
    run(backend, "dequant_q4k", [dw, out], [nb])
    backend.Synchronize()
    got = backend.CopyD2H(out, dtype=np.float32)
    assert same_bits(got, oracle.dequantize_q4k(w))


def test_every_fp16_header_value_decodes_as_the_oracle(backend):
    """All 65536 fp16 bit patterns as d (and, mirrored, as dmin): the device's half-to-float
    conversion (subnormals, signed zeros, infinities, NaNs) against Fp16ToFloat through the dump
    and through the production GEMV (one-hot rows, k = 256).  Finite results bit for bit;
    where the oracle gives NaN the device must give NaN."""
    g = synth.rng(101)
    nb = 65536
    w = synth.q4k_weights(g, nb, 256).reshape(nb, 144)
    bits = np.arange(nb, dtype=np.uint16)
    w[:, 0:2] = bits.view(np.uint8).reshape(nb, 2)
    w[:, 2:4] = bits[::-1].copy().view(np.uint8).reshape(nb, 2)
    w = w.reshape(-1)
    with np.errstate(invalid="ignore", over="ignore"):
        want = oracle.dequantize_q4k(w).reshape(nb, 256)
    dw = backend.Upload(w)
    out = backend.AllocateBuffer(nb * 1024)
    run(backend, "dequant_q4k", [dw, out], [nb])
    backend.Synchronize()
    got = backend.CopyD2H(out, dtype=np.float32).reshape(nb, 256)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    # the GEMV's own decode: column t of deq(W) for a few t (rows = the 65536 blocks)
    pos = [0, 31, 32, 200, 255]
    x = synth.one_hot_rows(256, pos)
    dx, dc = backend.Upload(x), backend.AllocateBuffer(4 * len(pos) * nb)
    run(backend, "gemm_q4k", [dx, dw, dc], [len(pos), nb, 256])
    backend.Synchronize()
    c = backend.CopyD2H(dc, dtype=np.float32).reshape(len(pos), nb)
    for r, t in enumerate(pos):
        ok = np.isfinite(want).all(axis=1)      # a NaN or infinity anywhere in the block spreads through 0 * inf
        assert same_bits_zero_sign_free(c[r][ok], want[ok, t]), t


@pytest.mark.parametrize("k,n", [(1280, 67), (5120, 67), (17408, 67), (3072, 3001), (2560, 3001), (5120, 6007)])
def test_non_finite_weight_row_stays_in_its_row(backend, k, n):
    """An infinite d in one row: that row's output is not finite (as in the reference), its
    neighbours', which share wavefronts and workgroups with it, are untouched."""
    g = synth.rng(102 + k)
    w = synth.q4k_weights(g, n, k).reshape(n, -1)
    bad = [7, 40, 66] if n == 67 else [7, 40, 66, 1001, 1002, n - 2]
    for r in bad:
        w[r, 144 * (r % (k // 256)):144 * (r % (k // 256)) + 2] = np.array([0x00, 0x7C], np.uint8)   # +inf
    w = w.reshape(-1)
    good = [r for r in range(n) if r not in bad]
    for m in (1, 2, 4):
        a = synth.activations_f32(g, m, k)
        da, dw, dc = backend.Upload(a), backend.Upload(w), backend.AllocateBuffer(4 * m * n)
        run(backend, "gemm_q4k", [da, dw, dc], [m, n, k])
        backend.Synchronize()
        got = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
        with np.errstate(invalid="ignore", over="ignore"):
            ref = oracle.gemm_q4k(a, w, m, n, k)
        assert not np.isfinite(got[:, bad]).any() and not np.isfinite(ref[:, bad]).any()
        assert rel_err(got[:, good], ref[:, good]) < TOL


@pytest.mark.parametrize("k", [256, 512, 1024, 768, 2048, 5120])
def test_gemv_one_hot_reproduces_dequant_bit_exact(backend, k):
    """A one-hot activation makes the production GEMV return one column of deq(W): the
    kernel's own decode (nibble extraction, scale unpack, d*sc*q - dmin*mn) is bit-exact."""
    g = synth.rng(200 + k)
    n = 96
    w = synth.q4k_weights(g, n, k)
    deq = oracle.dequantize_q4k(w).reshape(n, k)
    # every position of the first block, then a spread over the rest of the row
    pos = list(range(256)) + [int(t) for t in g.integers(0, k, 64)]
    for r0 in range(0, len(pos), 4):
        sel = pos[r0:r0 + 4]
        c = gemm(backend, "gemm_q4k", synth.one_hot_rows(k, sel), w, len(sel), n, k)[0]
        for r, t in enumerate(sel):
            assert same_bits_zero_sign_free(c[r], deq[:, t]), (k, t)


SHAPES = [(64, 256), (33, 512), (100, 1024), (17, 768), (129, 1280), (256, 2048), (130, 5120),
          (67, 17408), (40, 4352), (1, 256), (5, 32768)]


@pytest.mark.parametrize("n,k", [(3001, 768), (3003, 1280), (2999, 1536), (3005, 2560), (4099, 3072), (3002, 3584),
                                 (3001, 4352), (6007, 5120), (2051, 6400), (1027, 8192), (523, 17408)])
def test_single_row_over_many_output_columns(backend, n, k):
    """One activation row against enough weight rows that a workgroup takes several rows side by
    side (which count depends on how K/64 divides into wavefronts, including rows shorter than a
    wavefront whose lanes then belong to two weight rows); ragged last group."""
    g = synth.rng(31 * n + k)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    ref = oracle.gemm_q4k(a, w, 1, n, k, threads=True)
    got = gemm(backend, "gemm_q4k", a, w, 1, n, k)[0]
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("n,k", [(3001, 768), (2999, 1536), (3005, 2560), (4099, 3072), (3002, 3584), (1030, 5120)])
@pytest.mark.parametrize("m", [2, 3, 4])
def test_few_rows_over_many_output_columns(backend, n, k, m):
    g = synth.rng(43 * n + k + m)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    got = gemm(backend, "gemm_q4k", a, w, m, n, k)[0]
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 7, 16])
def test_gemm_q4k_matches_oracle(backend, n, k, m):
    if m > 4 and k > 8192:
        pytest.skip("large-k multi-row cases are covered at m <= 4")
    g = synth.rng(1000 * m + n + k)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    for name in ("gemm_q4k", "gemm_q4k_batched") if m != 1 else ("gemm_q4k", "gemm_q4k_row"):
        got = gemm(backend, name, a, w, m, n, k)[0]
        assert rel_err(got, ref) <= TOL, (name, rel_err(got, ref))


@pytest.mark.parametrize("n,k,split", [(640, 5120, 4), (5120, 5120, 4), (333, 2048, 2), (64, 17408, 4), (64, 256, 1)])
def test_vec_split_contract_and_reduce(backend, n, k, split):
    """gemm_q4k_vec writes `split` regions whose ordered sum gemm_vec_reduce returns
    (src/models/qwen3_5/internal.hpp:104-145)."""
    g = synth.rng(n + k + split)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    ref = oracle.gemm_q4k(a, w, 1, n, k, threads=True)
    da, dw = backend.Upload(a), backend.Upload(w)
    part = backend.AllocateBuffer(4 * n * split)
    backend.CopyH2D(part, np.full(n * split, np.nan, np.float32))   # stale partials must not leak
    out = backend.AllocateBuffer(4 * n)
    run(backend, "gemm_q4k_vec", [da, dw, part], [1, n, k, split], grid=((n + 7) // 8, split, 1))
    run(backend, "gemm_vec_reduce", [part, out], [n, split], grid=((n + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(out, dtype=np.float32)
    assert rel_err(got, ref) <= TOL
    parts = backend.CopyD2H(part, dtype=np.float32).reshape(split, n)
    assert np.array_equal(parts.sum(axis=0, dtype=np.float32), got)


@pytest.mark.parametrize("n,k,split", [(5120, 17408, 4), (2001, 16384, 2), (1031, 32768, 8), (4099, 8192, 2), (5120, 17408, 2)])
def test_vec_split_regions_hold_partial_sums(backend, n, k, split):
    """One row of a large matrix with slices of 4096 weights or more (the down projection as the
    reference's caller issues it: GemmVecSplit(5120, 17408) = 4, src/core/decode_internal.hpp:840-885):
    region s holds the dot products over K slice s, each within the GEMV bound of the oracle's
    product over that slice, and gemm_vec_reduce returns their ordered sum."""
    g = synth.rng(3 * n + k + split)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    ref = oracle.gemm_q4k(a, w, 1, n, k, threads=True)
    da, dw = backend.Upload(a), backend.Upload(w)
    part = backend.AllocateBuffer(4 * n * split)
    backend.CopyH2D(part, np.full(n * split, np.nan, np.float32))
    out = backend.AllocateBuffer(4 * n)
    run(backend, "gemm_q4k_vec", [da, dw, part], [1, n, k, split], grid=((n + 7) // 8, split, 1))
    run(backend, "gemm_vec_reduce", [part, out], [n, split], grid=((n + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(out, dtype=np.float32)
    parts = backend.CopyD2H(part, dtype=np.float32).reshape(split, n)
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)
    assert np.array_equal(parts.sum(axis=0, dtype=np.float32), got)
    blocks = w.reshape(n, k // 256, 144)
    per = k // 256 // split
    for s_ in range(split):
        ws = np.ascontiguousarray(blocks[:, s_ * per:(s_ + 1) * per]).reshape(-1)
        ref_s = oracle.gemm_q4k(a[:, s_ * per * 256:(s_ + 1) * per * 256], ws, 1, n, per * 256, threads=True)
        assert rel_err(parts[s_], ref_s) <= TOL, (s_, rel_err(parts[s_], ref_s))


@pytest.mark.parametrize("rows", [2, 3, 4, 5])
def test_rows_kernels(backend, rows):
    g = synth.rng(rows)
    n, k, split = 200, 2048, 2
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, rows, k)
    ref = oracle.gemm_q4k(a, w, rows, n, k)
    got = gemm(backend, f"gemm_q4k_rows{rows}", a, w, rows, n, k, extra=(split,))
    assert rel_err(got.sum(axis=0), ref) <= TOL
    with pytest.raises(StatusError) as e:          # the id fixes the row count
        gemm(backend, f"gemm_q4k_rows{rows}", a[:1], w, 1, n, k, extra=(1,))
    assert e.value.code == StatusCode.InvalidArgument


# Matrices of 16M weights and more take 2..16 rows through the few-row MFMA kernels (eight rows a
# pass, activations as fp16 hi/lo pairs with a per-row power-of-two scale; up to four rows with
# the activations resident in LDS when n is a multiple of 4, else streamed per stage); the shapes
# cover k/256 divisible by 4, by 2 only and odd (the tilings), k/256 not a multiple of 8 (ragged
# stages), n not a multiple of 4, and every pass count.
FEW_ROW_SHAPES = [(4096, 4096), (2060, 8192), (1030, 17408), (8200, 2048), (7400, 2304), (11000, 1536), (8194, 2048),
                  (65540, 256), (65538, 256), (16388, 1024), (3300, 5120), (1180, 14336)]


@pytest.mark.parametrize("n,k", FEW_ROW_SHAPES)
@pytest.mark.parametrize("m", [2, 3, 4, 5, 8, 9, 12, 16])
def test_few_rows_match_oracle(backend, n, k, m):
    if m > 9 and (n, k) != FEW_ROW_SHAPES[0]:
        pytest.skip("several passes are covered on the first shape")
    g = synth.rng(77 * m + n + k)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    got = gemm(backend, "gemm_q4k_batched", a, w, m, n, k)[0]
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)
    assert rms_err(got, ref) <= 1e-4, rms_err(got, ref)     # the split activations keep 22 bits


# Five rows and more take the one-pass kernel whatever the matrix size (two K parts of unequal
# size at k = 5120, a single wavefront's column at k = 256, ragged last tiles), 17..63 rows sixteen
# at a time with a short last chunk.
@pytest.mark.parametrize("n,k", [(100, 1024), (1030, 2304), (515, 5120), (64, 17408), (3001, 256)])
@pytest.mark.parametrize("m", [5, 9, 16, 17, 21, 33])
def test_five_rows_and_more_on_small_matrices(backend, n, k, m):
    g = synth.rng(91 * m + n + k)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    got = gemm(backend, "gemm_q4k_batched", a, w, m, n, k)[0]
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)
    assert rms_err(got, ref) <= 1e-4, rms_err(got, ref)


def test_few_rows_scaling_and_exactness(backend):
    n, k = 4096, 4096
    g = synth.rng(31337)
    w = synth.q4k_weights(g, n, k)
    deq = oracle.dequantize_q4k(w).reshape(n, k)
    # one-hot rows reproduce the fp32 block decode bit for bit, whatever the magnitude
    a = np.zeros((3, k), np.float32)
    a[0, 5], a[1, 4095], a[2, 1234] = 1.0, 2.0 ** -100, -(2.0 ** 90)
    got = gemm(backend, "gemm_q4k_batched", a, w, 3, n, k)[0]
    assert same_bits_zero_sign_free(got[0], deq[:, 5])
    assert same_bits_zero_sign_free(got[1], deq[:, 4095] * np.float32(2.0 ** -100))
    assert same_bits_zero_sign_free(got[2], deq[:, 1234] * np.float32(-(2.0 ** 90)))
    # the same through the kernels that take 5..8 and 9..16 rows in one pass
    for rows in (6, 13):
        a = np.zeros((rows, k), np.float32)
        pos = [int(p) for p in g.permutation(k)[:rows]]
        vals = np.array([1.0, 2.0 ** -100, -(2.0 ** 90), 3.0, -0.375, 2.0 ** 20, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0], np.float32)
        for r, t_ in enumerate(pos):
            a[r, t_] = vals[r]
        got = gemm(backend, "gemm_q4k_batched", a, w, rows, n, k)[0]
        for r, t_ in enumerate(pos):
            assert same_bits_zero_sign_free(got[r], deq[:, t_] * vals[r]), (rows, r, t_)
    # rows of very different magnitude, a zero row, and a row with a 1000x outlier
    a = synth.activations_f32(g, 5, k)
    a[0] *= np.float32(1e-30)
    a[1] *= np.float32(1e25)
    a[2] = 0.0
    a[3, 77] = 1000.0 * np.abs(a[3]).max()
    ref = oracle.gemm_q4k(a, w, 5, n, k, threads=True)
    got = gemm(backend, "gemm_q4k_batched", a, w, 5, n, k)[0]
    assert np.all(got[2] == 0.0)
    for r in (0, 1, 3, 4):
        assert rel_err(got[r], ref[r]) <= TOL, (r, rel_err(got[r], ref[r]))
    # a power-of-two multiple of the input gives exactly that multiple of the output
    got4 = gemm(backend, "gemm_q4k_batched", 4 * a, w, 5, n, k)[0]
    assert np.array_equal(got4[3:], 4 * got[3:])


def test_few_rows_full_size(backend):
    """configs[1] shapes with 4, 8 and 16 rows (speculative verify; the split of K into parts depends
    on both N and the row count), every row and column against the threaded oracle."""
    for seed, (n, k, m) in enumerate([(17408, 5120, 4), (5120, 17408, 8), (17408, 5120, 16), (5120, 17408, 16),
                                      (17408, 5120, 9), (5120, 17408, 2)]):
        g = synth.rng(909 + seed)
        w = synth.q4k_weights(g, n, k)
        a = synth.activations_f32(g, m, k)
        ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
        got = gemm(backend, f"gemm_q4k_rows{m}" if m <= 5 else "gemm_q4k_batched", a, w, m, n, k,
                   extra=(1,) if m <= 5 else ())[0]
        print(f"Q4_K {m} rows {n}x{k}: rel_err {rel_err(got, ref):.2e} (floor 0.05 rms), "
              f"{strict_rel_err(got, ref):.2e} (floor 1e-3 rms), max|d|/rms {rms_err(got, ref):.2e}")
        assert rel_err(got, ref) <= TOL, (n, k, m, rel_err(got, ref))
        # each row equals the single-row kernel's answer to fp32 summation-order noise
        one = gemm(backend, "gemm_q4k_vec", a[:1], w, 1, n, k, extra=(1,))[0]
        assert rms_err(got[:1], one) <= 2e-5


def test_special_inputs(backend):
    g = synth.rng(7)
    n, k = 77, 1024
    w = synth.q4k_weights(g, n, k)
    assert np.all(gemm(backend, "gemm_q4k", np.zeros((1, k), np.float32), w, 1, n, k) == 0.0)
    zero_w = np.zeros_like(w)
    a = synth.activations_f32(g, 2, k)
    assert np.all(gemm(backend, "gemm_q4k", a, zero_w, 2, n, k) == 0.0)


def test_full_size_configs(backend):
    """BASELINE configs 0 and 1 at full size: 5120x5120, 17408x5120 (gate/up), 5120x17408 (down)."""
    for seed, (n, k) in enumerate([(5120, 5120), (17408, 5120), (5120, 17408)]):
        g = synth.rng(4242 + seed)
        w = synth.q4k_weights(g, n, k)
        a = synth.activations_f32(g, 1, k)
        ref = oracle.gemm_q4k(a, w, 1, n, k, threads=True)
        got = gemm(backend, "gemm_q4k_vec", a, w, 1, n, k, extra=(1,))[0]
        print(f"Q4_K gemv {n}x{k}: rel_err {rel_err(got, ref):.2e} (floor 0.05 rms), "
              f"{strict_rel_err(got, ref):.2e} (floor 1e-3 rms), max|d|/rms {rms_err(got, ref):.2e}")
        assert rel_err(got, ref) <= TOL, (n, k, rel_err(got, ref))
        # linearity, a size-independent property: W(2a) == 2 W a exactly (power-of-two scaling)
        got2 = gemm(backend, "gemm_q4k_vec", 2 * a, w, 1, n, k, extra=(1,))[0]
        assert np.array_equal(got2, 2 * got)
