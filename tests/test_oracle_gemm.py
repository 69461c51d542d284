"""Pins the oracle's MXFP4 / FP8 / W4A8 / MoE routines: float64 bounds, one-hot identities,
torch.float8_e4m3fn, the reference's literal fold table (tests/golden/kmag_table.json) and
torch.softmax."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
from tessera_amd import synth

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def numpy_dequant_mxfp4(packed, n, k):
    """Independent decode: table lookup, low nibble = even element, 2^(s-127) per 32."""
    table = np.array([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], np.float64)
    blob = packed[: n * k // 2].reshape(n, k // 2)
    sc = packed[n * k // 2:].reshape(n, k // 32).astype(np.int64)
    nib = np.empty((n, k), dtype=np.uint8)
    nib[:, 0::2] = blob & 15
    nib[:, 1::2] = blob >> 4
    return table[nib] * np.repeat(np.ldexp(1.0, sc - 127), 32, axis=1)


def test_mxfp4_dequant_and_gemm():
    g = synth.rng(2)
    n, k = 20, 256
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    w[n * k // 2] = 0          # the 2^-127 subnormal scale
    w[n * k // 2 + 1] = 250    # a huge scale whose products still fit fp32
    deq64 = numpy_dequant_mxfp4(w, n, k)
    deq = oracle.dequantize_mxfp4(w, n, k)
    assert np.array_equal(deq.astype(np.float64), deq64)       # products are exact
    pos = [0, 1, 31, 32, 33, 255]
    c = oracle.gemm_mxfp4(synth.one_hot_rows(k, pos), w, len(pos), n, k)
    for r, t in enumerate(pos):
        # a dot product starts from +0, so a -0 weight comes out as +0: compare -0 as 0
        assert np.array_equal((c[r] + 0.0).view(np.uint32), (deq[:, t] + 0.0).view(np.uint32))
    w2 = synth.mxfp4_weights(g, n, k)
    d2 = numpy_dequant_mxfp4(w2, n, k)
    a = synth.activations_f32(g, 4, k)
    c = oracle.gemm_mxfp4(a, w2, 4, n, k)
    ref = a.astype(np.float64) @ d2.T
    bound = k * 2.0 ** -24 * (np.abs(a).astype(np.float64) @ np.abs(d2).T)
    assert np.all(np.abs(c - ref) <= bound)
    # the threaded entry keeps every output's fma chain
    assert np.array_equal(oracle.gemm_mxfp4(a, w2, 4, n, k, threads=True).view(np.uint32), c.view(np.uint32))
    with pytest.raises(oracle.OracleError) as err:     # k not a multiple of 32
        oracle.gemm_mxfp4(a[:, :48], w2[: n * 48 // 2 + n * 48 // 32], 4, n, 48)
    assert err.value.code == 1


def test_permute_mxfp4_to_wmma():
    """The fragment-order permutation against an independent statement of it (an axis transpose of
    the nibble bytes seen as [tile][row][k step][half][4 bytes]); the scales do not move."""
    g = synth.rng(12)
    n, k = 48, 96
    w = synth.mxfp4_weights(g, n, k)
    got = oracle.permute_mxfp4_to_wmma(w, n, k)
    blob = w[: n * k // 2].reshape(n // 16, 16, k // 16, 2, 4)
    assert np.array_equal(got[: n * k // 2], blob.transpose(0, 2, 3, 1, 4).reshape(-1))
    assert np.array_equal(got[n * k // 2:], w[n * k // 2:])
    assert sorted(got[: n * k // 2].tolist()) == sorted(w[: n * k // 2].tolist())
    with pytest.raises(oracle.OracleError):
        oracle.permute_mxfp4_to_wmma(synth.mxfp4_weights(g, 40, 96), 40, 96)     # rows not a multiple of 16


def test_gemm_fp8():
    g = synth.rng(3)
    n, k = 12, 96
    codes, scales = synth.fp8_weights(g, n, k)
    wv = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy().reshape(n, k)
    pos = [0, 5, 95]
    c = oracle.gemm_fp8(synth.one_hot_rows(k, pos), codes, scales, len(pos), n, k)
    for r, t in enumerate(pos):
        want = (scales * wv[:, t].astype(np.float32)).astype(np.float32)
        assert np.array_equal(c[r].view(np.uint32), want.view(np.uint32))
    a = synth.activations_f32(g, 2, k)
    c = oracle.gemm_fp8(a, codes, scales, 2, n, k)
    ref = a.astype(np.float64) @ (wv * scales[:, None].astype(np.float64)).T
    assert np.allclose(c, ref, rtol=0, atol=1e-4 * np.abs(ref).max())


def test_gemm_fp8_block():
    """One scale per 128 x 128 block: a one-hot row returns scale[block] * weight bit for bit (torch's
    E4M3 decode, block picked by integer division written out here), a dense row stays within the
    float64 product's rounding bound, and with every block of a row band given that band's row
    scale the result equals gemm_fp8's bit for bit."""
    g = synth.rng(31)
    n, k = 256, 384
    codes, scales = synth.fp8_block_weights(g, n, k)
    wv = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy().reshape(n, k)
    sc = scales.reshape(n // 128, k // 128)
    pos = [0, 127, 128, 200, 383]
    c = oracle.gemm_fp8_block(synth.one_hot_rows(k, pos), codes, scales, len(pos), n, k)
    for r, t in enumerate(pos):
        per_row = np.repeat(sc[:, t // 128], 128)
        want = (per_row * wv[:, t].astype(np.float32)).astype(np.float32)
        assert np.array_equal(c[r].view(np.uint32), want.view(np.uint32))
    a = synth.activations_f32(g, 2, k)
    c = oracle.gemm_fp8_block(a, codes, scales, 2, n, k)
    full = np.repeat(np.repeat(sc, 128, axis=0), 128, axis=1).astype(np.float64)
    ref = a.astype(np.float64) @ (wv * full).T
    assert np.allclose(c, ref, rtol=0, atol=1e-4 * np.abs(ref).max())
    band = g.uniform(0.5, 2.0, n // 128).astype(np.float32)
    uniform = np.repeat(band[:, None], k // 128, axis=1).reshape(-1)
    assert np.array_equal(oracle.gemm_fp8_block(a, codes, uniform, 2, n, k),
                          oracle.gemm_fp8(a, codes, np.repeat(band, 128), 2, n, k))
    with pytest.raises(oracle.OracleError):
        oracle.gemm_fp8_block(a[:, :320], codes[: n * 320], scales, 2, n, 320)   # k not a multiple of 128


def test_quantize_fp8_invariants():
    g = synth.rng(4)
    rows, cols = 6, 512
    x = synth.activations_bf16_outliers(g, rows, cols)
    x[3] = 0.0                                   # all-zero row
    x[4] *= 1e-9                                 # below the scale floor
    qdq, s = oracle.quantize_fp8(x, rows, cols)
    codes, s2 = oracle.quantize_fp8_pack(x, rows, cols)
    assert np.array_equal(s, s2)
    amax = np.abs(x).max(axis=1)
    floor = np.float32(1.0) / (np.float32(448.0) * np.float32(512.0))
    want_s = np.maximum((amax / np.float32(448.0)).astype(np.float32), floor)
    assert np.array_equal(s.view(np.uint32), want_s.view(np.uint32))
    assert s[3] == floor and np.all(codes[3] == 0)
    for r in (0, 1, 2, 5):
        assert (codes[r, np.argmax(np.abs(x[r]))] & 0x7F) == 0x7E      # the max encodes to +-448
    assert not np.any((codes & 0x7F) == 0x7F)                          # never the NaN code
    # pack then decode * scale == QDQ output, bit for bit
    dec = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal((dec * s[:, None]).view(np.uint32), qdq.view(np.uint32))
    # codes equal torch's RNE cast of the clamped quotient (away from the subnormal-cap interval)
    q = np.clip(x / s[:, None], -448, 448).astype(np.float32)
    keep = ~((np.abs(q) >= 7.5 * 2.0 ** -9) & (np.abs(q) < 2.0 ** -6))
    tcodes = torch.from_numpy(q).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(codes[keep], tcodes[keep])
    # idempotent: the row max is unchanged by QDQ, so a second pass is the identity
    qdq2, s3 = oracle.quantize_fp8(qdq, rows, cols)
    assert np.array_equal(s3, s) and np.array_equal(qdq2.view(np.uint32), qdq.view(np.uint32))
    with pytest.raises(oracle.OracleError):
        oracle.quantize_fp8_pack(x[:, :6], rows, 6)


def test_fold_table_is_the_reference_table_and_where_it_leaves_the_encoder():
    table = json.load(open(os.path.join(GOLDEN, "kmag_table.json")))["table"]
    diff = []
    for d in range(16):
        for n in range(8):
            assert oracle.fold_entry(d, n) == int(table[d][n], 16)
            if oracle.fold_entry_rne(d, n) != int(table[d][n], 16):
                diff.append((d, n))
    # the three exact ties (1.5 subnormal units) go down in the table, to even in the encoder
    assert diff == [(9, 3), (10, 5), (11, 7)]
    mags = [0, .5, 1, 1.5, 2, 3, 4, 6]
    for d in range(9):          # exact through d = 8 (6 * 2^-8 = 3 * 2^-7 still fits 3 bits)
        for n in range(8):
            assert oracle.fp8_e4m3_to_float(oracle.fold_entry(d, n)) == mags[n] * 2.0 ** -d


def test_folded_w4a8_equals_lossless_when_fold_is_exact():
    g = synth.rng(6)
    m, n, k = 3, 10, 128
    w = synth.mxfp4_weights(g, n, k, -8, -4)     # exponent spread 4 <= 8: the fold is exact
    a = synth.activations_bf16_outliers(g, m, k)
    codes, s = oracle.quantize_fp8_pack(a, m, k)
    w8, wref = oracle.fold_mxfp4_to_fp8(w, n, k)
    assert np.array_equal(wref, w[n * k // 2:].reshape(n, -1).max(axis=1))
    folded = oracle.gemm_mxfp4_fp8(codes, s, w8, wref, m, n, k)
    lossless = oracle.gemm_mxfp4_w4a8(codes, s, w, m, n, k)
    qdq, _ = oracle.quantize_fp8(a, m, k)
    assert np.array_equal(lossless.view(np.uint32), oracle.gemm_mxfp4(qdq, w, m, n, k).view(np.uint32))
    # same real number, different rounding order: a few ulp apart
    assert np.allclose(folded, lossless, rtol=1e-5, atol=1e-6 * np.abs(lossless).max())
    exact = (torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy()
             * s[:, None].astype(np.float64)) @ np.asarray(
                 [[oracle.f4e2m1_to_float(int(x)) for x in row] for row in
                  np.stack([w[: n * k // 2].reshape(n, -1) & 15, w[: n * k // 2].reshape(n, -1) >> 4],
                           axis=2).reshape(n, k)], dtype=np.float64).T
    # scale columns by their block exponents before comparing
    sc = np.repeat(np.ldexp(1.0, w[n * k // 2:].reshape(n, -1).astype(np.int64) - 127), 32, axis=1)
    nib = np.stack([w[: n * k // 2].reshape(n, -1) & 15, w[: n * k // 2].reshape(n, -1) >> 4], axis=2).reshape(n, k)
    tab = np.array([oracle.f4e2m1_to_float(i) for i in range(16)])
    a64 = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy() * s[:, None].astype(np.float64)
    exact = a64 @ (tab[nib] * sc).T
    assert np.allclose(lossless, exact, rtol=1e-5, atol=1e-6 * np.abs(exact).max())


def test_moe_gate_and_topk():
    g = synth.rng(8)
    ids, vals = synth.moe_routing(g, 5, 64, 8)
    for r in range(5):
        w = oracle.moe_gate(vals[r])
        t = torch.softmax(torch.from_numpy(vals[r]), dim=0).numpy()
        assert np.allclose(w, t, rtol=2e-6, atol=0) and abs(w.sum() - 1) < 1e-6
        perm = g.permutation(8)
        assert np.allclose(oracle.moe_gate(vals[r][perm]), w[perm], rtol=2e-6)
    lg = g.standard_normal(64).astype(np.float32)
    oi, ov = oracle.top_k_row(lg, 8)
    tv, ti = torch.topk(torch.from_numpy(lg), 8)
    assert np.array_equal(oi, ti.numpy().astype(np.uint32)) and np.array_equal(ov, tv.numpy())


def test_moe_expert_forward_composition():
    g = synth.rng(9)
    hidden, inter, experts, top_k, rows = 256, 256, 6, 2, 3
    gate = synth.q4k_weights(g, experts * inter, hidden)
    up = synth.q4k_weights(g, experts * inter, hidden)
    down = synth.q4k_weights(g, experts * hidden, inter)
    x = synth.activations_bf16(g, rows, hidden)
    ids, vals = synth.moe_routing(g, rows, experts, top_k)
    wts = np.stack([oracle.moe_gate(v) for v in vals])
    out = oracle.moe_batch_forward_q4k(x, ids, wts, gate, up, down, hidden, inter)
    gs, ds = inter * 144, hidden * 144
    for r in range(rows):
        acc = np.zeros(hidden, dtype=np.float32)
        for c in range(top_k):
            e = int(ids[r, c])
            gv = oracle.gemm_q4k(x[r], gate[e * gs:(e + 1) * gs], 1, inter, hidden)[0]
            uv = oracle.gemm_q4k(x[r], up[e * gs:(e + 1) * gs], 1, inter, hidden)[0]
            phi = (gv / (np.float32(1) + np.exp(-gv, dtype=np.float32))) * uv
            dv = oracle.gemm_q4k(phi, down[e * ds:(e + 1) * ds], 1, hidden, inter)[0]
            acc += wts[r, c] * dv
        assert np.allclose(out[r], acc, rtol=1e-5, atol=1e-5 * np.abs(acc).max())
