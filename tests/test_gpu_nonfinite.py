"""A non-finite weight (an infinite Q4_K d, an E8M0 byte of 0xFF) spoils its own output column and
nothing else, in every regime: the few-row MFMA kernels, the tiled MFMA GEMMs, the W4A8 kernels
and the routed-expert paths.  (The single-row VALU GEMV is covered in test_gpu_q4k.py.)"""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import rms_err, run

pytestmark = pytest.mark.gpu


def check(got, ref, bad, n, tol):
    good = np.array([r for r in range(n) if r not in bad])
    assert not np.isfinite(got[:, bad]).any()
    assert np.isfinite(got[:, good]).all()
    assert rms_err(got[:, good], ref[:, good]) < tol


@pytest.mark.parametrize("m,tol", [(2, 1e-4), (4, 1e-4), (8, 1e-4), (16, 1e-4), (17, 4e-3), (70, 4e-3), (300, 4e-3)])
def test_q4k_rows_with_an_infinite_scale(backend, m, tol):
    g = synth.rng(1300 + m)
    n, k = 4100, 4096                     # 16.8 M weights: the few-row kernels below 17 rows
    w = synth.q4k_weights(g, n, k).reshape(n, -1)
    bad = [0, 5, 1030, 2049, 4099]
    for r in bad:
        w[r, 144 * (r % 16):144 * (r % 16) + 2] = np.array([0x00, 0x7C], np.uint8)
    w = w.reshape(-1)
    a = synth.activations_bf16(g, m, k)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_q4k_batched", [backend.Upload(a), backend.Upload(w), dc], [m, n, k])
    backend.Synchronize()
    got = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
    rows = list(range(min(m, 3)))
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.gemm_q4k(a[rows], w, len(rows), n, k, threads=True)
    check(got[rows], ref, bad, n, tol)
    good = np.array([r for r in range(n) if r not in bad])
    assert np.isfinite(got[:, good]).all() and not np.isfinite(got[:, bad]).any()


@pytest.mark.parametrize("m", [1, 4, 16, 40, 300])
def test_w4a8_rows_with_an_infinite_block_scale(backend, m):
    g = synth.rng(1320 + m)
    n, k = 520, 2048
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    bad = [0, 63, 64, 300, 519]
    scales = w[n * k // 2:].reshape(n, k // 32)
    for r in bad:
        scales[r, r % (k // 32)] = 0xFF
    x = synth.activations_bf16(g, m, k)
    dx, dw = backend.Upload(x), backend.Upload(w)
    da8, das = backend.AllocateBuffer(m * k), backend.AllocateBuffer(4 * m)
    dref, out = backend.AllocateBuffer(n), backend.AllocateBuffer(4 * m * n)
    run(backend, "quantize_fp8_pack_rows", [dx, da8, das], [m, k], grid=(m, 1, 1))
    run(backend, "gemm_mxfp4_wmma", [da8, dw, das, dref, out], [m, n, k, 1, 0], grid=((n + 63) // 64, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(out, dtype=np.float32).reshape(m, n)
    codes, scale = oracle.quantize_fp8_pack(x, m, k)
    with np.errstate(invalid="ignore", over="ignore"):
        ref = oracle.gemm_mxfp4_w4a8(codes, scale, w, m, n, k)
    check(got, ref, bad, n, 5e-4)


@pytest.mark.parametrize("m", [2, 4, 8, 16, 17, 70])
@pytest.mark.parametrize("n,k", [(4100, 4096), (130, 5120)])
def test_q4k_a_non_finite_activation_row_stays_in_its_row(backend, m, n, k):
    """One activation row holds an infinity and a NaN: that output row is not finite, the other
    rows are what they would be without it (rows share weight passes, tiles and scratch)."""
    g = synth.rng(1340 + m + n)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_bf16(g, m, k)
    a[1, 7], a[1, k - 1] = np.inf, np.nan
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_q4k_batched", [backend.Upload(a), backend.Upload(w), dc], [m, n, k])
    backend.Synchronize()
    got = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
    assert not np.isfinite(got[1]).any()
    rows = [0] + list(range(2, min(m, 4)))
    ref = oracle.gemm_q4k(a[rows], w, len(rows), n, k, threads=True)
    assert np.isfinite(np.delete(got, 1, axis=0)).all()
    assert rms_err(got[rows], ref) < (1e-4 if m < 17 else 4e-3)
