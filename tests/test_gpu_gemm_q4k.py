"""Q4_K prefill GEMM on fp16 MFMA (the Q4_K GEMM ids from 17 rows on) against the CPU oracle.

The kernel multiplies fp16 activations by fp16 weights decoded in registers as
w16 = fma(q, RN16(d*sc), -RN16(dmin*mn)) and accumulates in fp32, like the reference's WMMA
kernel, which also stages both operands as fp16 (src/backends/rocm/rocm_kernels_wmma.cpp:334-431).
bf16-valued activations (the prefill configuration) convert to fp16 exactly, so the only error
against GemmQ4KRef is the fp16 rounding of the weights, three roundings of relative size 2^-11
on terms that partly cancel, random in sign over K, plus fp32 summation order.  Documented bound
for this path: largest absolute error at most 4e-3 of the rms output, 2-norm error at most 1e-3
(measured about 1.5e-3 and 3e-4); general fp32 activations add their own fp16 rounding (2^-11
relative per element) and are held to the same bound."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import norm_err, rms_err, run, same_bits_zero_sign_free

pytestmark = pytest.mark.gpu
RMS_TOL, NORM_TOL = 4e-3, 1e-3


def gemm(backend, name, a, w, m, n, k):
    da, dw = backend.Upload(a), backend.Upload(w)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, name, [da, dw, dc], [m, n, k], grid=((n + 63) // 64, (m + 127) // 128, 1))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


SHAPES = [(17, 96, 512), (24, 64, 256), (32, 100, 512), (64, 64, 768), (130, 257, 1024), (256, 256, 2048),
          (300, 50, 5120), (100, 600, 1280), (513, 320, 256)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("kind", ["bf16", "f32"])
def test_gemm_matches_oracle(backend, m, n, k, kind):
    g = synth.rng(m * 5 + n * 11 + k)
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_bf16(g, m, k) if kind == "bf16" else synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    for name in ("gemm_q4k_wmma", "gemm_q4k_batched"):
        got = gemm(backend, name, a, w, m, n, k)
        assert rms_err(got, ref) <= RMS_TOL, (name, rms_err(got, ref))
        assert norm_err(got, ref) <= NORM_TOL, (name, norm_err(got, ref))


def test_gemm_one_hot_is_the_fp16_dequant(backend):
    """One-hot activations: each output is one decoded weight, so operand layouts (which lane
    decodes which nibble, the order inside groups of 8, scale/min extraction for all eight
    sub-blocks) are checked exactly: the result must equal fma(q, RN16(d*sc), -RN16(dmin*mn))
    evaluated in fp16, which is within one fp16 ulp-and-a-half of the bit-exact dequant."""
    g = synth.rng(77)
    m, n, k = 256, 96, 512
    w = synth.q4k_weights(g, n, k)
    pos = [int(p) for p in g.permutation(k)[:m]]
    a = synth.one_hot_rows(k, pos)
    got = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    deq = oracle.dequantize_q4k(w).reshape(n, k)
    blocks = w.reshape(n, k // 256, 144)
    d = blocks[:, :, 0:2].copy().view(np.float16).astype(np.float32)[:, :, 0]
    dmin = blocks[:, :, 2:4].copy().view(np.float16).astype(np.float32)[:, :, 0]
    for r, t in enumerate(pos):
        b, e = divmod(t, 256)
        sb = e // 32
        sc = np.empty(n, np.float32)
        mn = np.empty(n, np.float32)
        for j in range(n):
            s, mm = oracle.get_scale_min(sb, blocks[j, b, 4:16])
            sc[j], mn[j] = s, mm
        byte = blocks[:, b, 16 + (sb // 2) * 32 + e % 32]
        q = ((byte >> 4) if sb % 2 else (byte & 15)).astype(np.float64)
        s16 = (d[:, b] * sc).astype(np.float16).astype(np.float64)
        m16 = (dmin[:, b] * mn).astype(np.float16).astype(np.float64)
        want = (q * s16 - m16).astype(np.float16).astype(np.float32)   # exact product, one rounding
        assert same_bits_zero_sign_free(got[r], want), (r, t)
        assert np.max(np.abs(want - deq[:, t])) <= 2.0 ** -9 * np.max(np.abs(deq[:, t])) + 1e-6


def test_full_size_prefill_rows(backend):
    """BASELINE configs[3] shape (M=2048, N=17408, K=5120, bf16 activations) and one rank's
    column shard (N=8704 = the first half of the rows of W): sampled rows against the oracle,
    and the shard must equal the corresponding columns of the full product bit for bit."""
    g = synth.rng(3)
    m, n, k = 2048, 17408, 5120
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_bf16(g, m, k)
    got = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    rows = [0, 1, 255, 256, 1023, 2047]
    ref = oracle.gemm_q4k(a[rows], w, len(rows), n, k, threads=True)
    assert rms_err(got[rows], ref) <= RMS_TOL, rms_err(got[rows], ref)
    assert norm_err(got[rows], ref) <= NORM_TOL
    shard = gemm(backend, "gemm_q4k_wmma", a, w[: 8704 * (k // 256) * 144], m, 8704, k)
    assert np.array_equal(shard, got[:, :8704])


def test_down_projection_shape_prefill_rows(backend):
    """The other FFN shape (N=5120, K=17408: 68 super-blocks a row, 544 K-steps a tile) at M=512,
    with a row count that leaves a ragged last row tile: sampled rows against the oracle."""
    g = synth.rng(5)
    m, n, k = 500, 5120, 17408
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_bf16(g, m, k)
    got = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    rows = [0, 255, 256, 499]
    ref = oracle.gemm_q4k(a[rows], w, len(rows), n, k, threads=True)
    assert rms_err(got[rows], ref) <= RMS_TOL, rms_err(got[rows], ref)
    assert norm_err(got[rows], ref) <= NORM_TOL
