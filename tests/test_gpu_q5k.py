"""GPU parity of the Q5_K ids (dequant dump, GEMV with 1..5 rows, split contract) against the oracle."""
import numpy as np
import pytest

import oracle
from tessera_amd import StatusCode, StatusError, synth
from util import ref_grid_vec, rel_err, run, same_bits, same_bits_zero_sign_free

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
    g = synth.rng(600)
    n, k = 512, 5120
    w = synth.q5k_weights(g, n, k)
    blocks = w.reshape(-1, 176)
    blocks[0] = 0
    blocks[1, 4:] = 0xFF
    blocks[2, 0:2] = np.array([-0.013], np.float16).view(np.uint8)
    blocks[3, 0:2] = np.array([3e-6], np.float16).view(np.uint8)
    nb = blocks.shape[0]
    dw = backend.Upload(w)
    out = backend.AllocateBuffer(nb * 1024)
    run(backend, "dequant_q5k", [dw, out], [nb])
    backend.Synchronize()
    assert same_bits(backend.CopyD2H(out, dtype=np.float32), oracle.dequantize_q5k(w))


@pytest.mark.parametrize("k", [256, 512, 768, 2048, 5120])
def test_gemv_one_hot_reproduces_dequant_bit_exact(backend, k):
    """A one-hot activation makes the production GEMV return one column of deq(W): the kernel's
    own decode (nibble and fifth-bit assembly, scale unpack, d*sc*q - dmin*mn) is bit-exact."""
    g = synth.rng(610 + k)
    n = 96
    w = synth.q5k_weights(g, n, k)
    deq = oracle.dequantize_q5k(w).reshape(n, k)
    pos = list(range(256)) + [int(t) for t in g.integers(0, k, 32)]
    for r0 in range(0, len(pos), 2):
        sel = pos[r0:r0 + 2]
        c = gemm(backend, "gemm_q5k", synth.one_hot_rows(k, sel), w, len(sel), n, k)[0]
        for r, t in enumerate(sel):
            assert same_bits_zero_sign_free(c[r], deq[:, t]), (k, t)


SHAPES = [(64, 256), (33, 512), (100, 1024), (17, 768), (129, 1280), (256, 2048), (130, 5120),
          (67, 17408), (40, 4352), (1, 256), (5, 32768), (3, 49152)]


@pytest.mark.parametrize("n,k", [(3001, 768), (3003, 1280), (2999, 1536), (3005, 2560), (4099, 3072), (3002, 3584),
                                 (3001, 4352), (6007, 5120), (2051, 6400), (1027, 8192), (523, 17408)])
def test_single_row_over_many_output_columns(backend, n, k):
    """One activation row against enough weight rows that a workgroup takes several rows side by
    side (which count depends on how K/64 divides into wavefronts, including rows shorter than a
    wavefront whose lanes then belong to two weight rows); ragged last group."""
    g = synth.rng(31 * n + k)
    w = synth.q5k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    ref = oracle.gemm_q5k(a, w, 1, n, k, threads=True)
    got = gemm(backend, "gemm_q5k", a, w, 1, n, k)[0]
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("n,k", [(3001, 768), (2999, 1536), (3005, 2560), (4099, 3072), (3002, 3584), (1030, 5120)])
@pytest.mark.parametrize("m", [2, 3, 4])
def test_few_rows_over_many_output_columns(backend, n, k, m):
    g = synth.rng(43 * n + k + m)
    w = synth.q5k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q5k(a, w, m, n, k, threads=True)
    got = gemm(backend, "gemm_q5k", a, w, m, n, k)[0]
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("n,k", SHAPES)
@pytest.mark.parametrize("m", [1, 2, 3, 5, 16])
def test_gemm_q5k_matches_oracle(backend, n, k, m):
    if m > 3 and k > 8192:
        pytest.skip("large-k multi-row cases are covered at m <= 3")
    g = synth.rng(2000 * m + n + k)
    w = synth.q5k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q5k(a, w, m, n, k, threads=True)
    for name in ("gemm_q5k", "gemm_q5k_batched"):
        got = gemm(backend, name, a, w, m, n, k)[0]
        assert rel_err(got, ref) <= TOL, (name, rel_err(got, ref))


@pytest.mark.parametrize("rows", [2, 3, 4, 5])
def test_rows_and_split_contract(backend, rows):
    g = synth.rng(rows + 640)
    n, k, split = 200, 2048, 2
    w = synth.q5k_weights(g, n, k)
    a = synth.activations_f32(g, rows, k)
    ref = oracle.gemm_q5k(a, w, rows, n, k)
    got = gemm(backend, f"gemm_q5k_rows{rows}", a, w, rows, n, k, extra=(split,))
    assert rel_err(got.sum(axis=0), ref) <= TOL
    assert np.all(got[1:] == 0.0)
    got1 = gemm(backend, "gemm_q5k_vec", a[:1], w, 1, n, k, extra=(4,))
    assert rel_err(got1.sum(axis=0), ref[:1]) <= TOL
    with pytest.raises(StatusError) as e:
        gemm(backend, f"gemm_q5k_rows{rows}", a[:1], w, 1, n, k, extra=(1,))
    assert e.value.code == StatusCode.InvalidArgument
    with pytest.raises(StatusError) as e:
        gemm(backend, "gemm_q5k", a[:, :200], w, rows, n, 200)
    assert e.value.code == StatusCode.InvalidArgument


def test_full_size_and_linearity(backend):
    """The 27B FFN shapes with Q5_K weights: gate/up 17408x5120 and down 5120x17408, one row."""
    for seed, (n, k) in enumerate([(17408, 5120), (5120, 17408)]):
        g = synth.rng(6600 + seed)
        w = synth.q5k_weights(g, n, k)
        a = synth.activations_f32(g, 1, k)
        ref = oracle.gemm_q5k(a, w, 1, n, k, threads=True)
        got = gemm(backend, "gemm_q5k_vec", a, w, 1, n, k, extra=(1,))[0]
        assert rel_err(got, ref) <= TOL, (n, k, rel_err(got, ref))
        got2 = gemm(backend, "gemm_q5k_vec", 2 * a, w, 1, n, k, extra=(1,))[0]
        assert np.array_equal(got2, 2 * got)
# From 17 rows up the weights are decoded once to fp16 and multiplied on the fp16 MFMA: weights
# carry one rounding of 2^-11, activations a second (per-row scaled), accumulation is fp32.
RMS_TOL, NORM_TOL = 4e-3, 1e-3


@pytest.mark.parametrize("m,n,k", [(17, 300, 512), (64, 512, 1024), (100, 257, 2304), (300, 1000, 5120), (256, 256, 256)])
def test_prefill_fp16_mfma_matches_oracle(backend, m, n, k):
    from util import norm_err, rms_err
    g = synth.rng(5900 + m + n + k)
    w = synth.q5k_weights(g, n, k)
    a = synth.activations_bf16(g, m, k)
    ref = oracle.gemm_q5k(a, w, m, n, k, threads=True)
    for name in ("gemm_q5k_wmma", "gemm_q5k_batched"):
        got = gemm(backend, name, a, w, m, n, k)[0]
        assert rms_err(got, ref) <= RMS_TOL, (name, rms_err(got, ref))
        assert norm_err(got, ref) <= NORM_TOL, (name, norm_err(got, ref))
    # one-hot rows return the fp16 rounding of the exact decode
    hot = synth.one_hot_rows(k, [t % k for t in range(0, 32 * 37, 37)])
    deq = oracle.dequantize_q5k(w).reshape(n, k)
    got = gemm(backend, "gemm_q5k_wmma", hot, w, 32, n, k)[0]
    for r, t in enumerate([t % k for t in range(0, 32 * 37, 37)]):
        assert same_bits_zero_sign_free(got[r], deq[:, t].astype(np.float16).astype(np.float32)), t
