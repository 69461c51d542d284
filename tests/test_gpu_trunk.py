"""The non-matmul trunk ids that sit between the projections (rope, mrope, attention, qgate_split;
contracts include/tessera/backend.hpp:162-179,378-390) against the oracle's restatements of
RopeRef / MropeRef / AttentionRef / QGateSplitRef (src/core/numerics/attention.cpp).  Plain
correct kernels: rope forms its angles in double as the CPU reference does (the reference's own
device kernel uses fp32 powf/cosf/sinf), attention is a running softmax, so it differs from the
reference in summation order only (bound 2e-6 of the largest output)."""
import numpy as np
import pytest

import oracle
from tessera_amd import StatusCode, StatusError, synth
from util import run

pytestmark = pytest.mark.gpu


def f32_bits(x):
    return int(np.float32(x).view(np.uint32))


@pytest.mark.parametrize("rows,heads,head_dim,rope_dim,pos_base,theta", [(5, 3, 64, 64, 0, 1e4), (33, 8, 128, 64, 100000, 1e6),
                                                                          (1, 1, 8, 2, 7, 10.0), (300, 2, 256, 256, 5, 1e4)])
def test_rope(backend, rows, heads, head_dim, rope_dim, pos_base, theta):
    g = synth.rng(rows + head_dim)
    x = g.standard_normal((rows, heads, head_dim)).astype(np.float32)
    want = oracle.rope(x, rows, heads, head_dim, rope_dim, pos_base, float(np.float32(theta)))
    dx = backend.Upload(x)
    run(backend, "rope", [dx], [rows, heads, head_dim, rope_dim, pos_base, f32_bits(theta)],
        grid=((rows * heads * (rope_dim // 2) + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(dx, dtype=np.float32).reshape(rows, heads, head_dim)
    # cos and sin may differ by one fp32 unit in the last place between the host's and the device's libm
    assert np.max(np.abs(got - want)) <= 3e-7 * np.max(np.abs(x))
    assert np.array_equal(got[..., rope_dim:], x[..., rope_dim:])


def test_mrope(backend):
    g = synth.rng(3)
    rows, heads, head_dim, rope_dim, theta = 40, 4, 128, 96, 1e4
    x = g.standard_normal((rows, heads, head_dim)).astype(np.float32)
    pos = g.integers(0, 5000, size=(rows, 3)).astype(np.uint64)
    sec = (20, 16, 8)
    want = oracle.mrope(x, pos, rows, heads, head_dim, rope_dim, *sec, theta)
    dx, dp = backend.Upload(x), backend.Upload(pos)
    run(backend, "mrope", [dx, dp], [rows, heads, head_dim, rope_dim, f32_bits(theta), *sec],
        grid=((rows * heads * (rope_dim // 2) + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(dx, dtype=np.float32).reshape(rows, heads, head_dim)
    assert np.max(np.abs(got - want)) <= 3e-7 * np.max(np.abs(x))
    with pytest.raises(StatusError) as e:
        run(backend, "mrope", [dx, dp], [rows, heads, head_dim, rope_dim, f32_bits(theta), 40, 8, 1])
    assert e.value.code == StatusCode.InvalidArgument


@pytest.mark.parametrize("m,n,heads,kv_heads,head_dim,q_base,window,kv_f16,causal", [
    (5, 12, 4, 2, 32, 7, 0, 0, 1), (3, 400, 8, 8, 64, 397, 16, 0, 1), (6, 9, 2, 1, 128, 0, 0, 1, 1),
    (4, 300, 4, 4, 16, 0, 0, 0, 0), (2, 5, 2, 2, 8, 20, 3, 1, 1), (1, 1000, 24, 4, 256, 999, 0, 1, 1),
    (7, 130, 6, 2, 100, 60, 0, 0, 1)])
def test_attention(backend, m, n, heads, kv_heads, head_dim, q_base, window, kv_f16, causal):
    g = synth.rng(m * 100 + n)
    q = g.standard_normal((m, heads * head_dim)).astype(np.float32)
    k = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    v = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    if kv_f16:
        k, v = k.astype(np.float16), v.astype(np.float16)
    want = oracle.attention(q, k, v, m, n, heads, kv_heads, head_dim, q_base, window, bool(kv_f16), bool(causal))
    # the rows of this sequence sit at row_base inside a larger batch buffer; its other rows stay as they are
    row_base, total = 2, m + 5
    qbuf = np.zeros((total, heads * head_dim), np.float32)
    qbuf[row_base:row_base + m] = q
    dq, dk, dv = backend.Upload(qbuf), backend.Upload(k), backend.Upload(v)
    dout = backend.Upload(np.full((total, heads * head_dim), 7.0, np.float32))
    run(backend, "attention", [dq, dk, dv, dout], [m, n, heads, kv_heads, head_dim, q_base, row_base, window, kv_f16, causal],
        grid=(m * heads, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(dout, dtype=np.float32).reshape(total, heads * head_dim)
    assert np.max(np.abs(got[row_base:row_base + m] - want)) <= 2e-6 * max(1.0, np.max(np.abs(want)))
    assert np.all(got[:row_base] == 7.0) and np.all(got[row_base + m:] == 7.0)


def test_attention_argument_errors(backend):
    b = [backend.AllocateBuffer(1 << 16) for _ in range(4)]
    for scalars in ([1, 4, 3, 2, 16, 0, 0, 0, 0, 1],       # heads not a multiple of kv_heads
                    [1, 4, 2, 2, 512, 0, 0, 0, 0, 1],      # head_dim above 256
                    [0, 4, 2, 2, 16, 0, 0, 0, 0, 1],       # no rows
                    [1, 1 << 20, 2, 2, 64, 0, 0, 0, 0, 1]):  # keys beyond the buffer
        with pytest.raises(StatusError) as e:
            run(backend, "attention", b, scalars)
        assert e.value.code == StatusCode.InvalidArgument


def test_qgate_split(backend):
    g = synth.rng(10)
    rows, heads, head_dim = 37, 6, 72
    fused = g.standard_normal((rows, heads, 2, head_dim)).astype(np.float32)
    df = backend.Upload(fused)
    dq, dg = backend.AllocateBuffer(4 * rows * heads * head_dim), backend.AllocateBuffer(4 * rows * heads * head_dim)
    run(backend, "qgate_split", [df, dq, dg], [heads, head_dim, rows], grid=((rows * heads * head_dim + 255) // 256, 1, 1))
    backend.Synchronize()
    want_q, want_g = oracle.qgate_split(fused, heads, head_dim, rows)
    assert np.array_equal(backend.CopyD2H(dq, dtype=np.float32), want_q)
    assert np.array_equal(backend.CopyD2H(dg, dtype=np.float32), want_g)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("rows,cols", [(1, 8), (5, 1024), (33, 2056)])
def test_quantize_kv_bit_exact(backend, bits, rows, cols):
    """quantize_q8 / quantize_q4 (the quantized cache's per-row quantizers): codes and scales equal
    QuantizeQ8Ref / QuantizeQ4Ref bit for bit, with an all-zero row, exact ties and an outlier."""
    g = synth.rng(rows * 10 + cols + bits)
    x = g.standard_normal((rows, cols)).astype(np.float32) * np.float32(2.5)
    x[0] = 0.0
    x[0, :8] = np.array([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 127.0 if bits == 8 else 7.0, -1.0], np.float32)   # scale 1: exact ties
    if rows > 2:
        x[1] = 0.0
        x[2, cols // 2] = 300.0
    want_codes, want_scale = oracle.quantize_kv(x, rows, cols, bits)
    din = backend.Upload(x)
    dout, dscale = backend.AllocateBuffer(rows * cols * bits // 8), backend.AllocateBuffer(4 * rows)
    run(backend, "quantize_q8" if bits == 8 else "quantize_q4", [din, dout, dscale], [rows, cols], grid=(rows, 1, 1))
    backend.Synchronize()
    assert np.array_equal(backend.CopyD2H(dscale, dtype=np.float32), want_scale)
    assert np.array_equal(backend.CopyD2H(dout), want_codes)
    with pytest.raises(StatusError) as e:
        run(backend, "quantize_q8" if bits == 8 else "quantize_q4", [din, dout, dscale], [rows, cols + 2])
    assert e.value.code == StatusCode.InvalidArgument


@pytest.mark.parametrize("kind", ["q8", "q4", "fp8"])
@pytest.mark.parametrize("m,n,heads,kv_heads,head_dim,q_base,window", [(5, 12, 4, 2, 32, 7, 0), (3, 200, 8, 8, 64, 197, 50),
                                                                        (1, 130, 6, 2, 128, 129, 0), (2, 70, 2, 1, 256, 68, 0)])
def test_attention_over_a_quantized_cache(backend, kind, m, n, heads, kv_heads, head_dim, q_base, window):
    """attention_q8 / attention_q4 / attention_fp8: a cache written by the matching quantizer, read back
    by the attention id, against AttentionQ8Ref / Q4Ref / Fp8Ref (summation order differs)."""
    g = synth.rng(m * 7 + n + len(kind) * 1000)
    width = kv_heads * head_dim
    q = g.standard_normal((m, heads * head_dim)).astype(np.float32)
    kf = g.standard_normal((n, width)).astype(np.float32)
    vf = g.standard_normal((n, width)).astype(np.float32)
    if kind == "fp8":
        k, ks = oracle.quantize_fp8_pack(kf, n, width)
        v, vs = oracle.quantize_fp8_pack(vf, n, width)
    else:
        k, ks = oracle.quantize_kv(kf, n, width, 8 if kind == "q8" else 4)
        v, vs = oracle.quantize_kv(vf, n, width, 8 if kind == "q8" else 4)
    want = oracle.attention_quant(q, k, v, ks, vs, m, n, heads, kv_heads, head_dim, kind, q_base, window)
    row_base, total = 1, m + 3
    qbuf = np.zeros((total, heads * head_dim), np.float32)
    qbuf[row_base:row_base + m] = q
    bufs = [backend.Upload(qbuf), backend.Upload(k), backend.Upload(v), backend.Upload(ks), backend.Upload(vs),
            backend.Upload(np.full((total, heads * head_dim), 7.0, np.float32))]
    run(backend, "attention_" + kind, bufs, [m, n, heads, kv_heads, head_dim, q_base, row_base, window, oracle.KV_KINDS[kind]],
        grid=(m * heads, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(bufs[5], dtype=np.float32).reshape(total, heads * head_dim)
    assert np.max(np.abs(got[row_base:row_base + m] - want)) <= 2e-6 * max(1.0, np.max(np.abs(want)))
    assert np.all(got[:row_base] == 7.0) and np.all(got[row_base + m:] == 7.0)
    with pytest.raises(StatusError) as e:   # kind above 2
        run(backend, "attention_" + kind, bufs, [m, n, heads, kv_heads, head_dim, q_base, row_base, window, 3])
    assert e.value.code == StatusCode.InvalidArgument


def test_cast_f32_f16_bit_exact(backend):
    g = synth.rng(78)
    x = np.concatenate([g.standard_normal(5000).astype(np.float32) * np.float32(10.0) ** g.integers(-9, 6, 5000).astype(np.float32),
                        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 65535.9, 65536.0, -70000.0, 2.0 ** -24, 2.0 ** -25,
                                  2.0 ** -14, np.inf, -np.inf, np.nan], np.float32)])
    din, dout = backend.Upload(x), backend.AllocateBuffer(2 * x.size)
    run(backend, "cast_f32_f16", [din, dout], [x.size], grid=((x.size // 2 + 255) // 256, 1, 1))
    backend.Synchronize()
    assert np.array_equal(backend.CopyD2H(dout, dtype=np.uint16), oracle.cast_f32_f16(x))
    with pytest.raises(StatusError) as e:   # n must be even
        run(backend, "cast_f32_f16", [din, dout], [x.size - 1])
    assert e.value.code == StatusCode.InvalidArgument


@pytest.mark.parametrize("m,n,heads,kv_heads,head_dim,q_base,window,kv_f16,causal,split,gqa", [
    (1, 300, 8, 2, 64, 299, 0, 0, 1, 4, True), (1, 77, 6, 1, 128, 76, 0, 1, 1, 8, True), (3, 90, 4, 4, 32, 80, 25, 0, 1, 3, False),
    (2, 11, 2, 1, 16, 0, 0, 0, 0, 16, False), (1, 5, 2, 2, 256, 4, 0, 0, 1, 1, False)])
def test_attention_split_and_combine(backend, m, n, heads, kv_heads, head_dim, q_base, window, kv_f16, causal, split, gqa):
    """attention_split / attention_split_gqa then attention_combine: the partials against the oracle's
    (chunks of ceil(span / split) keys, empty chunks 0 / -1e30 / 0), the merged rows against the unsplit
    attention."""
    g = synth.rng(m * 13 + n + split)
    q = g.standard_normal((m, heads * head_dim)).astype(np.float32)
    k = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    v = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    if kv_f16:
        k, v = k.astype(np.float16), v.astype(np.float16)
    kf, vf = np.asarray(k, np.float32), np.asarray(v, np.float32)
    want_acc, want_max, want_sum = oracle.attention_split(q, kf, vf, m, n, heads, kv_heads, head_dim, split, q_base, window, bool(causal))
    parts = m * heads * split
    dq, dk, dv = backend.Upload(q), backend.Upload(k), backend.Upload(v)
    dacc, dmax, dsum = backend.AllocateBuffer(4 * parts * head_dim), backend.AllocateBuffer(4 * parts), backend.AllocateBuffer(4 * parts)
    run(backend, "attention_split_gqa" if gqa else "attention_split", [dq, dk, dv, dacc, dmax, dsum],
        [m, n, heads, kv_heads, head_dim, q_base, window, kv_f16, causal, split], grid=(parts, 1, 1))
    dout = backend.AllocateBuffer(4 * m * heads * head_dim)
    run(backend, "attention_combine", [dacc, dmax, dsum, dout], [m, heads, head_dim, split], grid=(m * heads, 1, 1))
    backend.Synchronize()
    got_max, got_sum = backend.CopyD2H(dmax, dtype=np.float32), backend.CopyD2H(dsum, dtype=np.float32)
    got_acc = backend.CopyD2H(dacc, dtype=np.float32).reshape(parts, head_dim)
    empty = want_sum == 0
    assert np.array_equal(got_sum == 0, empty) and np.all(got_max[empty] == np.float32(-1e30)) and not got_acc[empty].any()
    assert np.max(np.abs(got_max[~empty] - want_max[~empty])) <= 2e-6 * max(1.0, np.max(np.abs(want_max[~empty])))
    assert np.max(np.abs(got_sum - want_sum)) <= 4e-6 * np.max(want_sum)
    assert np.max(np.abs(got_acc - want_acc)) <= 4e-6 * max(1.0, np.max(np.abs(want_acc)))
    want = oracle.attention(q, k, v, m, n, heads, kv_heads, head_dim, q_base, window, bool(kv_f16), bool(causal))
    got = backend.CopyD2H(dout, dtype=np.float32).reshape(m, heads * head_dim)
    assert np.max(np.abs(got - want)) <= 3e-6 * max(1.0, np.max(np.abs(want)))
    if gqa:
        with pytest.raises(StatusError) as e:   # the gqa form serves one row
            run(backend, "attention_split_gqa", [dq, dk, dv, dacc, dmax, dsum], [2, n, heads, kv_heads, head_dim, q_base, window, kv_f16, causal, split])
        assert e.value.code == StatusCode.InvalidArgument


@pytest.mark.parametrize("kind", ["q8", "q4", "fp8"])
def test_attention_split_over_a_quantized_cache(backend, kind):
    m, n, heads, kv_heads, head_dim, q_base, window, split = 1, 150, 8, 2, 64, 149, 0, 5
    g = synth.rng(len(kind) + 500)
    width = kv_heads * head_dim
    q = g.standard_normal((m, heads * head_dim)).astype(np.float32)
    kf = g.standard_normal((n, width)).astype(np.float32)
    vf = g.standard_normal((n, width)).astype(np.float32)
    if kind == "fp8":
        (k, ks), (v, vs) = oracle.quantize_fp8_pack(kf, n, width), oracle.quantize_fp8_pack(vf, n, width)
    else:
        bits = 8 if kind == "q8" else 4
        (k, ks), (v, vs) = oracle.quantize_kv(kf, n, width, bits), oracle.quantize_kv(vf, n, width, bits)
    kd, vd = oracle.dequant_kv(k, ks, n, width, kind), oracle.dequant_kv(v, vs, n, width, kind)
    want_acc, want_max, want_sum = oracle.attention_split(q, kd, vd, m, n, heads, kv_heads, head_dim, split, q_base, window, True)
    parts = m * heads * split
    bufs = [backend.Upload(q), backend.Upload(k), backend.Upload(v), backend.Upload(ks), backend.Upload(vs),
            backend.AllocateBuffer(4 * parts * head_dim), backend.AllocateBuffer(4 * parts), backend.AllocateBuffer(4 * parts)]
    run(backend, f"attention_{kind}_split", bufs, [m, n, heads, kv_heads, head_dim, q_base, window, oracle.KV_KINDS[kind], split],
        grid=(parts, 1, 1))
    dout = backend.AllocateBuffer(4 * m * heads * head_dim)
    run(backend, "attention_combine", bufs[5:] + [dout], [m, heads, head_dim, split], grid=(m * heads, 1, 1))
    backend.Synchronize()
    assert np.max(np.abs(backend.CopyD2H(bufs[5], dtype=np.float32).reshape(parts, head_dim) - want_acc)) <= 4e-6 * max(1.0, np.max(np.abs(want_acc)))
    assert np.max(np.abs(backend.CopyD2H(bufs[7], dtype=np.float32) - want_sum)) <= 4e-6 * np.max(want_sum)
    want = oracle.attention_quant(q, k, v, ks, vs, m, n, heads, kv_heads, head_dim, kind, q_base, window)
    got = backend.CopyD2H(dout, dtype=np.float32).reshape(m, heads * head_dim)
    assert np.max(np.abs(got - want)) <= 3e-6 * max(1.0, np.max(np.abs(want)))
