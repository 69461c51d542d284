"""Q4_K prefill GEMM on fp16 MFMA against the CPU oracle: gemm_q4k_wmma from 17 rows on, the other
Q4_K ids from 64 rows on (the reference's regime table, src/core/decode_internal.hpp:1349-1361;
below that they keep fp32 activations, sixteen rows at a time through the exact kernels) or from
the row count set with SetQ4KTensorRows.

The kernel multiplies fp16 activations by fp16 weights and accumulates in fp32, like the
reference's tensor-core tile (src/backends/rocm/rocm_kernels_wmma.cpp:334-431).  Its weights are
the reference's: the fp32 block decode rounded once to fp16 (`__float2half_rn(dsc*nib - dmm)`,
rocm_kernels_wmma.cpp:73-77); its activations are the fp32 rows divided by a power of two per row
and rounded to fp16 (exact for the bf16-valued rows of the prefill configuration).  So there are
two references here:

* `f16_operands_product`: the same two fp16 operands multiplied in float64 (the weights as
  `q4k_weights_f16` states them).  The device result
  may differ from it by fp32 accumulation only (asserted: 3e-5 of the rms output).
* the oracle's fp32 GemmQ4KRef.  The distance of `f16_operands_product` from it is what rounding
  the operands to fp16 costs (measured 3e-4 of the rms output as largest error, 8e-5 in 2-norm,
  with K = 5120); the device is held to 1.2 times that distance plus the accumulation allowance.
  The per-element figure with the small floor, max |d| / max(|ref|, 1e-3 rms), is printed beside it."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import norm_err, rel_err, rms_err, run, same_bits_zero_sign_free

pytestmark = pytest.mark.gpu
ACC_TOL = 3e-5          # fp32 accumulation order, in units of the rms output


def gemm(backend, name, a, w, m, n, k):
    da, dw = backend.Upload(a), backend.Upload(w)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, name, [da, dw, dc], [m, n, k], grid=((n + 63) // 64, (m + 127) // 128, 1))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


def q4k_weights_f16(w, n, k):
    """The tile's fp16 weights: fma(nibble, d*sc, -dmin*mn) on the fp32 products d*sc and dmin*mn,
    rounded once to fp16 (float64 holds the fma exactly).  The reference's expression
    `__float2half_rn(dsc*nib - dmm)` rounds the same fma to fp32 first; the two differ only where
    that fp32 value lands on the midpoint of two fp16 numbers (about one weight in 3e7, by one
    fp16 unit in the last place, this one being the nearer to the exact value)."""
    blk = np.asarray(w, np.uint8).reshape(-1, 144)
    hdr = blk[:, :4].copy().view(np.float16).astype(np.float32)
    sp = blk[:, 4:16]
    sc = np.empty((blk.shape[0], 8), np.float32)
    mn = np.empty_like(sc)
    sc[:, :4], mn[:, :4] = sp[:, 0:4] & 63, sp[:, 4:8] & 63
    sc[:, 4:] = (sp[:, 8:12] & 15) | ((sp[:, 0:4] >> 6) << 4)
    mn[:, 4:] = (sp[:, 8:12] >> 4) | ((sp[:, 4:8] >> 6) << 4)
    dsc = (hdr[:, 0:1] * sc).astype(np.float64)
    dmm = (hdr[:, 1:2] * mn).astype(np.float64)
    qs = blk[:, 16:].reshape(-1, 4, 32)
    out = np.empty((blk.shape[0], 8, 32), np.float16)
    with np.errstate(over="ignore"):
        out[:, 0::2] = dsc[:, 0::2, None] * (qs & 15) - dmm[:, 0::2, None]
        out[:, 1::2] = dsc[:, 1::2, None] * (qs >> 4) - dmm[:, 1::2, None]
    return out.reshape(n, k)


def f16_operands_product(a, w, m, n, k):
    """float64 product of the two fp16 operands the tensor-core path multiplies: the weights of
    q4k_weights_f16; activation rows divided by the power of two that brings their largest
    magnitude to [1024, 2048), rounded to fp16, multiplied back."""
    w16 = q4k_weights_f16(w, n, k).astype(np.float64)
    a = np.asarray(a, np.float32).reshape(m, k)
    amax = np.max(np.abs(a), axis=1)
    e = np.floor(np.log2(np.where(amax > 0, amax, 1.0)))
    s = np.where(amax > 0, np.exp2(e - 10.0), 1.0).astype(np.float32)
    a16 = (a / s[:, None]).astype(np.float16).astype(np.float64) * s[:, None].astype(np.float64)
    return a16 @ w16.T


def rel_err_floored(got, ref):
    """max |got - ref| / max(|ref|, eps), eps = 1e-3 rms(ref): the per-element figure with the
    small floor, reported (not asserted: an output that cancels to 1e-3 of the rms cannot be
    reproduced to 1e-3 of itself by any operand rounding)."""
    got = np.asarray(got, np.float64).reshape(-1)
    ref = np.asarray(ref, np.float64).reshape(-1)
    eps = 1e-3 * np.sqrt(np.mean(ref * ref)) + 1e-30
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), eps)))


def check(got, a, w, m, n, k, ref, what):
    """Device result against both references (see the module docstring)."""
    sim = f16_operands_product(a, w, m, n, k)
    assert rms_err(got, sim) <= ACC_TOL, (what, "device vs fp16-operand product", rms_err(got, sim))
    sim_rms, sim_norm = rms_err(sim, ref), norm_err(sim, ref)
    got_rms, got_norm = rms_err(got, ref), norm_err(got, ref)
    print(f"{what}: vs fp32 oracle max|d|/rms {got_rms:.2e} (fp16-operand product {sim_rms:.2e}), "
          f"2-norm {got_norm:.2e} ({sim_norm:.2e}), max|d|/max(|ref|,1e-3 rms) {rel_err_floored(got, ref):.2e}")
    assert got_rms <= 1.2 * sim_rms + ACC_TOL, (what, got_rms, sim_rms)
    assert got_norm <= 1.2 * sim_norm + ACC_TOL, (what, got_norm, sim_norm)
    assert got_rms <= 4e-3 and got_norm <= 1e-3, (what, got_rms, got_norm)     # absolute ceiling of the path (fp32 rows, short K)


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
        if name == "gemm_q4k_batched" and m < 64:
            # fp32 activations, as the reference's tiled kernel below its tensor-core regime
            assert rel_err(got, ref) <= 1e-3 and rms_err(got, ref) <= 1e-4, (name, m, rel_err(got, ref), rms_err(got, ref))
        else:
            check(got, a, w, m, n, k, ref, f"{name} {m}x{n}x{k} {kind}")


def test_tensor_rows_setting(backend):
    """gemm_q4k_batched between 17 and 63 rows: exact by default (the one-pass few-row kernel,
    sixteen rows at a time), the fp16 tile -- bit for bit gemm_q4k_wmma's result -- once the caller
    lowers the threshold; fewer than 17 is refused; 0 restores the default."""
    g = synth.rng(515)
    m, n, k = 40, 4100, 4096                  # 16.8 M weights: the few-row kernels take it
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    assert backend.Q4KTensorRows() == 64
    exact = gemm(backend, "gemm_q4k_batched", a, w, m, n, k)
    tile = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    assert rel_err(exact, ref) <= 1e-3 and rms_err(exact, ref) <= 1e-4
    assert rms_err(tile, ref) > rms_err(exact, ref)
    try:
        backend.SetQ4KTensorRows(17)
        assert backend.Q4KTensorRows() == 17
        assert np.array_equal(gemm(backend, "gemm_q4k_batched", a, w, m, n, k), tile)
        with pytest.raises(Exception):
            backend.SetQ4KTensorRows(16)
    finally:
        backend.SetQ4KTensorRows(0)
    assert backend.Q4KTensorRows() == 64
    assert np.array_equal(gemm(backend, "gemm_q4k_batched", a, w, m, n, k), exact)


def test_gemm_one_hot_is_the_fp16_dequant(backend):
    """One-hot activations: each output is one decoded weight, so operand layouts (which lane
    decodes which nibble, the order inside groups of 8, scale/min extraction for all eight
    sub-blocks) and the decode's arithmetic are checked exactly: the result must be the bit-exact
    fp32 dequant rounded once to fp16, the reference tile's weight."""
    g = synth.rng(77)
    m, n, k = 256, 96, 512
    w = synth.q4k_weights(g, n, k)
    pos = [int(p) for p in g.permutation(k)[:m]]
    a = synth.one_hot_rows(k, pos)
    got = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    w16 = q4k_weights_f16(w, n, k)
    assert np.array_equal(w16, oracle.dequantize_q4k(w).reshape(n, k).astype(np.float16))   # no midpoint case here
    for r, t in enumerate(pos):
        assert same_bits_zero_sign_free(got[r], w16[:, t].astype(np.float32)), (r, t)


@pytest.mark.parametrize("lo,hi", [(1e-6, 1e-4), (2e-8, 3e-6)])
def test_gemm_small_block_scales(backend, lo, hi):
    """Block headers of the size real checkpoints have (1e-6 .. 1e-4, down to fp16 subnormals):
    the decode works in fp32, so nothing is lost before the one rounding to fp16 that the
    reference tile also makes; weights below the fp16 normal range keep fewer bits in both."""
    g = synth.rng(78)
    m, n, k = 96, 160, 1024
    w = synth.q4k_weights(g, n, k).reshape(-1, 144)
    nb = w.shape[0]
    w[:, 0:2] = g.uniform(lo, hi, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    w[:, 2:4] = g.uniform(lo, hi, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    w = w.reshape(-1)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_q4k(a, w, m, n, k, threads=True)
    got = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    sim = f16_operands_product(a, w, m, n, k)
    assert rms_err(got, sim) <= ACC_TOL, rms_err(got, sim)
    print(f"headers in [{lo:g}, {hi:g}]: vs fp32 oracle max|d|/rms {rms_err(got, ref):.2e} "
          f"(fp16-operand product {rms_err(sim, ref):.2e})")
    assert rms_err(got, ref) <= 1.2 * rms_err(sim, ref) + ACC_TOL


def test_full_size_prefill_rows(backend):
    """BASELINE configs[3] shape (M=2048, N=17408, K=5120, bf16 activations) and one rank's
    column shard (N=8704 = the first half of the rows of W).  Every element of the product is
    compared with the float64 product of the same fp16 operands; 72 rows -- every position inside
    a 32-row MFMA tile, spread over all eight 256-row tiles -- are compared with the fp32 oracle
    over all columns, i.e. the 256x256 tiles and the 128x64 tiles that take the leftover columns;
    the shard must equal the corresponding columns of the full product bit for bit."""
    g = synth.rng(3)
    m, n, k = 2048, 17408, 5120
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_bf16(g, m, k)
    got = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    sim = f16_operands_product(a, w, m, n, k)
    assert rms_err(got, sim) <= ACC_TOL, rms_err(got, sim)
    rows = sorted({(37 * i) % 2048 for i in range(64)} | {0, 31, 32, 255, 256, 1023, 2016, 2047})
    assert {r % 32 for r in rows} == set(range(32)) and {r // 256 for r in rows} == set(range(8))
    ref = oracle.gemm_q4k(a[rows], w, len(rows), n, k, threads=True)
    check(got[rows], a[rows], w, len(rows), n, k, ref, "configs[3] Q4_K 2048x17408x5120, 72 rows")
    shard = gemm(backend, "gemm_q4k_wmma", a, w[: 8704 * (k // 256) * 144], m, 8704, k)
    assert np.array_equal(shard, got[:, :8704])


def test_down_projection_shape_prefill_rows(backend):
    """The other FFN shape (N=5120, K=17408: 68 super-blocks a row, 544 K-steps a tile) at M=500,
    a row count that leaves a ragged last row tile: all of it against the fp16-operand product,
    some 65 rows (every 32-row tile position) against the fp32 oracle."""
    g = synth.rng(5)
    m, n, k = 500, 5120, 17408
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_bf16(g, m, k)
    got = gemm(backend, "gemm_q4k_wmma", a, w, m, n, k)
    sim = f16_operands_product(a, w, m, n, k)
    assert rms_err(got, sim) <= ACC_TOL, rms_err(got, sim)
    rows = sorted({(37 * i) % 500 for i in range(32)} | set(range(224, 256)) | {0, 256, 499})
    assert {r % 32 for r in rows} == set(range(32))
    ref = oracle.gemm_q4k(a[rows], w, len(rows), n, k, threads=True)
    check(got[rows], a[rows], w, len(rows), n, k, ref, "down shape Q4_K 500x5120x17408")
