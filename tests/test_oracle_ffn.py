"""Pins of the oracle's dense feed-forward pieces (silu_mul): no reference fixture covers them, so
they are held to what the mathematics fixes."""
import numpy as np

import oracle


def test_silu_mul_against_float64_and_identities():
    g = np.random.default_rng(41)
    x = np.concatenate([g.standard_normal(20000) * 4, g.standard_normal(2000) * 40,
                        np.array([0.0, -0.0, 1.0, -1.0, 88.0, -88.0, 104.0, -104.0, 1e-20, -1e-20])]).astype(np.float32)
    u = g.standard_normal(x.size).astype(np.float32)
    got = oracle.silu_mul(x, u).astype(np.float64)
    x64, u64 = x.astype(np.float64), u.astype(np.float64)
    with np.errstate(over="ignore"):
        want = x64 / (1.0 + np.exp(-x64)) * u64
    # three fp32 roundings (exp, divide, multiply) around a well-conditioned expression; below
    # x = -88.7 expf(-x) overflows to inf and the fp32 expression returns -0 where the exact
    # value is about x * e^x < 1e-36
    tol = 4 * np.spacing(np.abs(want).astype(np.float32)).astype(np.float64) + 1e-36
    assert np.all(np.abs(got - want) <= tol)
    # silu(0) = 0 whatever u; silu(x) - silu(-x) = x; silu(x) -> x and silu(-x) -> -0 for large x
    assert np.all(oracle.silu_mul(np.zeros(4, np.float32), np.array([1, -1, 1e30, -1e30], np.float32)) == 0)
    ones = np.ones_like(x)
    diff = oracle.silu_mul(x, ones).astype(np.float64) - oracle.silu_mul(-x, ones).astype(np.float64)
    assert np.all(np.abs(diff - x64) <= 4 * np.spacing(np.abs(x)).astype(np.float64) + 1e-36)
    big = np.array([104.0, 200.0, 1e10], np.float32)
    assert np.array_equal(oracle.silu_mul(big, np.ones(3, np.float32)), big)
    assert np.all(oracle.silu_mul(-big, np.ones(3, np.float32)) == 0)


def test_ffn_gate_up_is_the_composition_of_pinned_parts():
    from tessera_amd import synth
    g = synth.rng(43)
    n, k = 24, 512
    gate, up = synth.q4k_weights(g, n, k), synth.q4k_weights(g, n, k)
    x = synth.activations_f32(g, 2, k)
    got = oracle.ffn_gate_up_silu_q4k(x, gate, up, 2, n, k)
    gg, uu = oracle.gemm_q4k(x, gate, 2, n, k), oracle.gemm_q4k(x, up, 2, n, k)
    assert np.array_equal(got, oracle.silu_mul(gg, uu).reshape(2, n))
    # a zero gate matrix gives silu(0) * u = 0 everywhere
    zero = np.zeros_like(gate)
    assert np.all(oracle.ffn_gate_up_silu_q4k(x, zero, up, 2, n, k) == 0)


def test_rmsnorm_against_float64_and_invariants():
    g = np.random.default_rng(44)
    rows, cols, eps = 5, 5120, 1e-6
    x = (g.standard_normal((rows, cols)) * 3).astype(np.float32)
    w = (1 + 0.1 * g.standard_normal(cols)).astype(np.float32)
    got = oracle.rmsnorm(x, w, rows, cols, eps).astype(np.float64)
    x64 = x.astype(np.float64)
    want = x64 / np.sqrt((x64 * x64).mean(axis=1, keepdims=True) + eps) * w.astype(np.float64)
    # a sequential fp32 sum of 5120 squares: relative error about sqrt(cols) * 2^-24
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-12)) < 2e-5
    # a row of equal values c with eps = 0 and unit weights normalises to sign(c) (all ones)
    ones = oracle.rmsnorm(np.full((1, 256), -3.0, np.float32), np.ones(256, np.float32), 1, 256, 0.0)
    assert np.allclose(ones, -1.0, rtol=0, atol=1e-6)
    # scaling the row by a power of two leaves the result unchanged when eps = 0 (exact scaling)
    a = oracle.rmsnorm(x, w, rows, cols, 0.0)
    b = oracle.rmsnorm(x * np.float32(8), w, rows, cols, 0.0)
    assert np.array_equal(a, b)
    import pytest
    with pytest.raises(oracle.OracleError):
        oracle.rmsnorm(x, w, 0, cols, eps)


def test_embedding_gathers_decoded_rows_and_zero_fills_bad_ids():
    from tessera_amd import synth
    g = synth.rng(45)
    vocab, cols = 37, 512
    ids = np.array([0, 36, 5, 37, 4000000000, 5], dtype=np.uint32)
    f32 = g.standard_normal((vocab, cols)).astype(np.float32)
    out = oracle.embedding("f32", ids, f32, ids.size, cols, vocab)
    assert np.array_equal(out[[0, 1, 2, 5]], f32[[0, 36, 5, 5]]) and np.all(out[[3, 4]] == 0)
    bf16 = (f32.view(np.uint32) >> 16).astype(np.uint16)
    out = oracle.embedding("bf16", ids, bf16, ids.size, cols, vocab)
    assert np.array_equal(out[[0, 1, 2]].view(np.uint32), (bf16[[0, 36, 5]].astype(np.uint32) << 16))
    assert np.all(out[[3, 4]] == 0)
    q4k = synth.q4k_weights(g, vocab, cols)
    deq = oracle.dequantize_q4k(q4k).reshape(vocab, cols)
    out = oracle.embedding("q4k", ids, q4k, ids.size, cols, vocab)
    assert np.array_equal(out[[0, 1, 2, 5]].view(np.uint32), deq[[0, 36, 5, 5]].view(np.uint32))
    assert np.all(out[[3, 4]] == 0)
