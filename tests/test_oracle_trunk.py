"""Pins the oracle's restatements of the non-matmul trunk pieces that sit around the projections:
RopeRef, MropeRef, AttentionRef (fp32 and fp16 keys/values), QGateSplitRef, the quantized key/value
caches (QuantizeQ8Ref, QuantizeQ4Ref, AttentionQ8Ref / Q4Ref / Fp8Ref) and the cast_f32_f16 conversion
(src/core/numerics/attention.cpp, quant.cpp:123-178, src/backends/rocm/rocm_kernels.hpp:26-45)."""
import numpy as np
import pytest
import torch

import oracle
from tessera_amd import synth


def complex_rope(x, angles, rope_dim):
    """(x1 + i x2) * exp(i angle) per NeoX pair, float64."""
    x = x.astype(np.float64).copy()
    half = rope_dim // 2
    z = (x[..., :half] + 1j * x[..., half:rope_dim]) * np.exp(1j * angles)
    x[..., :half], x[..., half:rope_dim] = z.real, z.imag
    return x


@pytest.mark.parametrize("rows,heads,head_dim,rope_dim,pos_base,theta", [(5, 3, 64, 64, 0, 1e4), (4, 2, 128, 64, 1000, 1e6),
                                                                          (1, 1, 8, 2, 7, 10.0)])
def test_rope(rows, heads, head_dim, rope_dim, pos_base, theta):
    g = synth.rng(rows + head_dim)
    x = g.standard_normal((rows, heads, head_dim)).astype(np.float32)
    got = oracle.rope(x, rows, heads, head_dim, rope_dim, pos_base, theta)
    j = np.arange(rope_dim // 2)
    angles = (pos_base + np.arange(rows))[:, None, None] * theta ** (-2.0 * j / rope_dim)[None, None, :]
    want = complex_rope(x, angles, rope_dim)
    assert np.max(np.abs(got - want)) <= 4e-7 * np.max(np.abs(x))
    assert np.array_equal(got[..., rope_dim:], x[..., rope_dim:])                     # the rest of a head is left alone
    half = rope_dim // 2
    assert np.allclose(got[..., :half] ** 2 + got[..., half:rope_dim] ** 2,
                       x[..., :half] ** 2 + x[..., half:rope_dim] ** 2, rtol=1e-5, atol=1e-6)
    if pos_base == 0:
        assert np.array_equal(got[0], x[0])                                           # position 0 is the identity
    with pytest.raises(oracle.OracleError):
        oracle.rope(x, rows, heads, head_dim, head_dim + 2, 0, theta)


def test_mrope():
    g = synth.rng(3)
    rows, heads, head_dim, rope_dim, theta = 6, 2, 64, 48, 1e4
    x = g.standard_normal((rows, heads, head_dim)).astype(np.float32)
    pos = g.integers(0, 500, size=(rows, 3)).astype(np.uint64)
    sec = (10, 8, 4)                       # 22 of 24 pairs; the last two reuse the width id
    got = oracle.mrope(x, pos, rows, heads, head_dim, rope_dim, *sec, theta)
    j = np.arange(rope_dim // 2)
    which = np.where(j < sec[0], 0, np.where(j < sec[0] + sec[1], 1, 2))
    angles = pos[:, which].astype(np.float64)[:, None, :] * theta ** (-2.0 * j / rope_dim)[None, None, :]
    want = complex_rope(x, angles, rope_dim)
    assert np.max(np.abs(got - want)) <= 4e-7 * np.max(np.abs(x))
    same = np.repeat(np.arange(100, 100 + rows, dtype=np.uint64)[:, None], 3, axis=1)
    assert np.array_equal(oracle.mrope(x, same, rows, heads, head_dim, rope_dim, *sec, theta),
                          oracle.rope(x, rows, heads, head_dim, rope_dim, 100, theta))
    with pytest.raises(oracle.OracleError):
        oracle.mrope(x, pos, rows, heads, head_dim, rope_dim, 20, 4, 1, theta)       # more section pairs than pairs


def torch_attention(q, k, v, m, n, heads, kv_heads, head_dim, q_base, window, causal):
    q = torch.from_numpy(q.astype(np.float64)).reshape(m, heads, head_dim)
    k = torch.from_numpy(k.astype(np.float64)).reshape(n, kv_heads, head_dim).repeat_interleave(heads // kv_heads, dim=1)
    v = torch.from_numpy(v.astype(np.float64)).reshape(n, kv_heads, head_dim).repeat_interleave(heads // kv_heads, dim=1)
    s = torch.einsum("mhd,nhd->hmn", q, k) / np.sqrt(np.float32(head_dim)).astype(np.float64)
    pos = torch.arange(m) + q_base
    keys = torch.arange(n)
    if causal:
        last = torch.clamp(pos, max=n - 1)
        start = torch.where(torch.tensor(window != 0) & (pos + 1 > window), pos + 1 - window, torch.zeros_like(pos))
        start = torch.minimum(start, last)
        mask = (keys[None, :] >= start[:, None]) & (keys[None, :] <= last[:, None])
        s = s.masked_fill(~mask[None], float("-inf"))
    w = torch.softmax(s, dim=-1)
    return torch.einsum("hmn,nhd->mhd", w, v).reshape(m, heads * head_dim).numpy()


@pytest.mark.parametrize("m,n,heads,kv_heads,head_dim,q_base,window,kv_f16,causal", [
    (5, 12, 4, 2, 32, 7, 0, False, True), (3, 40, 8, 8, 64, 37, 16, False, True), (6, 9, 2, 1, 128, 0, 0, True, True),
    (4, 30, 4, 4, 16, 0, 0, False, False), (2, 5, 2, 2, 8, 20, 3, True, True)])
def test_attention(m, n, heads, kv_heads, head_dim, q_base, window, kv_f16, causal):
    g = synth.rng(m * 100 + n)
    q = g.standard_normal((m, heads * head_dim)).astype(np.float32)
    k = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    v = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    if kv_f16:
        k, v = k.astype(np.float16), v.astype(np.float16)
    got = oracle.attention(q, k, v, m, n, heads, kv_heads, head_dim, q_base, window, kv_f16, causal)
    want = torch_attention(q, np.asarray(k, np.float32), np.asarray(v, np.float32), m, n, heads, kv_heads, head_dim, q_base,
                           window, causal)
    assert np.max(np.abs(got - want)) <= 2e-6 * max(1.0, np.max(np.abs(want)))


def test_attention_single_key_and_errors():
    g = synth.rng(9)
    heads, head_dim = 3, 16
    q = g.standard_normal((1, heads * head_dim)).astype(np.float32)
    k = g.standard_normal((4, heads * head_dim)).astype(np.float32)
    v = g.standard_normal((4, heads * head_dim)).astype(np.float32)
    got = oracle.attention(q, k, v, 1, 4, heads, heads, head_dim, q_base=0)          # position 0 sees key 0 only
    assert np.array_equal(got[0], v[0])
    with pytest.raises(oracle.OracleError):
        oracle.attention(q, k, v, 1, 4, heads, 2, head_dim)                          # heads not a multiple of kv_heads


def test_qgate_split():
    g = synth.rng(10)
    rows, heads, head_dim = 3, 4, 8
    fused = g.standard_normal((rows, heads, 2, head_dim)).astype(np.float32)
    q, gate = oracle.qgate_split(fused, heads, head_dim, rows)
    assert np.array_equal(q.reshape(rows, heads, head_dim), fused[:, :, 0])
    assert np.array_equal(gate.reshape(rows, heads, head_dim), fused[:, :, 1])


def half_away(x):
    """Round half away from zero, float64, written with floor (not the library's round)."""
    return np.sign(x) * np.floor(np.abs(x) + 0.5)


@pytest.mark.parametrize("bits,qmax", [(8, 127), (4, 7)])
def test_quantize_kv(bits, qmax):
    g = synth.rng(40 + bits)
    rows, cols = 7, 96
    x = g.standard_normal((rows, cols)).astype(np.float32) * np.float32(3.0)
    x[2] = 0.0                                                   # all-zero row: scale 1, codes 0
    x[3, 5] = 50.0                                               # one outlier sets the scale
    x[4, :8] = np.array([0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.49, -0.49], np.float32)
    x[4, 8] = np.float32(qmax)                                   # amax = qmax: scale exactly 1, the values above are exact ties
    x[4, 9:] = 0.0
    codes, scale = oracle.quantize_kv(x, rows, cols, bits)
    amax = np.abs(x).max(axis=1)
    want_scale = np.where(amax > 0, (amax / np.float32(qmax)).astype(np.float32), np.float32(1.0))
    assert np.array_equal(scale, want_scale)
    if bits == 8:
        q = codes.view(np.int8).reshape(rows, cols).astype(np.int64)
    else:
        nib = np.stack([codes & 0xF, codes >> 4], axis=-1).reshape(rows, cols).astype(np.int64)
        q = np.where(nib >= 8, nib - 16, nib)
    want = np.clip(half_away((x / scale[:, None]).astype(np.float32).astype(np.float64)), -qmax, qmax).astype(np.int64)
    assert np.array_equal(q, want)
    assert np.all(np.abs(q * scale[:, None].astype(np.float64) - x) <= scale[:, None] * 0.5000001)
    assert np.all(np.abs(q).max(axis=1)[amax > 0] == qmax) and np.all(q[2] == 0)
    assert scale[4] == 1.0 and q[4, :8].tolist() == [1, -1, 2, -2, 3, -3, 0, 0]
    with pytest.raises(oracle.OracleError):
        oracle.quantize_kv(x[:, :94], rows, 94, bits)           # cols not a multiple of 4 / 8


@pytest.mark.parametrize("kind", ["q8", "q4", "fp8"])
@pytest.mark.parametrize("m,n,heads,kv_heads,head_dim,q_base,window", [(4, 20, 4, 2, 32, 16, 0), (2, 33, 6, 6, 16, 40, 8)])
def test_attention_quant(kind, m, n, heads, kv_heads, head_dim, q_base, window):
    """The codes are decoded here with numpy / torch views (int8 view, nibble arithmetic, torch's E4M3) and
    fed to the torch attention; the oracle must agree to summation order."""
    g = synth.rng(m + n + len(kind))
    width = kv_heads * head_dim
    q = g.standard_normal((m, heads * head_dim)).astype(np.float32)
    ks = g.uniform(0.005, 0.02, n).astype(np.float32)
    vs = g.uniform(0.005, 0.02, n).astype(np.float32)
    if kind == "q4":
        k = g.integers(0, 256, n * width // 2, dtype=np.uint8)
        v = g.integers(0, 256, n * width // 2, dtype=np.uint8)
        def dec(c):
            nib = np.stack([c & 0xF, c >> 4], axis=-1).reshape(n, width).astype(np.int64)
            return np.where(nib >= 8, nib - 16, nib).astype(np.float64)
    elif kind == "q8":
        k = g.integers(0, 256, n * width, dtype=np.uint8)
        v = g.integers(0, 256, n * width, dtype=np.uint8)
        dec = lambda c: c.view(np.int8).reshape(n, width).astype(np.float64)
    else:
        k = g.integers(0, 0x7F, n * width, dtype=np.uint8) | (g.integers(0, 2, n * width, dtype=np.uint8) << 7)   # no NaN codes
        v = g.integers(0, 0x7F, n * width, dtype=np.uint8) | (g.integers(0, 2, n * width, dtype=np.uint8) << 7)
        dec = lambda c: torch.from_numpy(c.copy()).view(torch.float8_e4m3fn).to(torch.float64).numpy().reshape(n, width)
    got = oracle.attention_quant(q, k, v, ks, vs, m, n, heads, kv_heads, head_dim, kind, q_base, window)
    kf = (dec(k).astype(np.float32) * ks[:, None]).astype(np.float32)
    vf = (dec(v).astype(np.float32) * vs[:, None]).astype(np.float32)
    want = torch_attention(q, kf, vf, m, n, heads, kv_heads, head_dim, q_base, window, True)
    assert np.max(np.abs(got - want)) <= 2e-6 * max(1.0, np.max(np.abs(want)))
    assert np.array_equal(got, oracle.attention(q, kf, vf, m, n, heads, kv_heads, head_dim, q_base, window, False, True))


def test_cast_f32_f16_cuts_the_significand():
    """Toward zero: numpy's nearest binary16, stepped one value toward zero where it lies above the
    input in magnitude; 2^16 and more (and NaN) give infinity, below 2^-24 zero."""
    g = synth.rng(77)
    x = np.concatenate([g.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** g.integers(-9, 5, 4000).astype(np.float32),
                        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 65535.9, 65536.0, -70000.0, 2.0 ** -24, 2.0 ** -25,
                                  -(2.0 ** -24) * 1.5, 2.0 ** -14, 2.0 ** -14 * 0.999, np.inf, -np.inf], np.float32)])
    got = oracle.cast_f32_f16(x)
    with np.errstate(over="ignore"):
        near = x.astype(np.float16)
    above = np.abs(near.astype(np.float64)) > np.abs(x.astype(np.float64))
    cut = np.where(above, np.nextafter(near, np.float16(0.0)), near)
    big = np.abs(x) >= 65536.0
    want = np.where(big, np.where(np.signbit(x), np.float16(-np.inf), np.float16(np.inf)), cut).astype(np.float16)
    assert np.array_equal(got, want.view(np.uint16))
    assert oracle.cast_f32_f16(np.array([np.nan], np.float32))[0] & 0x7FFF == 0x7C00     # NaN becomes infinity


@pytest.mark.parametrize("m,n,heads,kv_heads,head_dim,q_base,window,causal,split", [
    (1, 50, 4, 2, 32, 49, 0, True, 4), (3, 40, 6, 6, 16, 30, 12, True, 5), (2, 9, 2, 1, 8, 0, 0, False, 16), (1, 7, 2, 2, 8, 6, 0, True, 1)])
def test_attention_split_and_combine(m, n, heads, kv_heads, head_dim, q_base, window, causal, split):
    """Every chunk on its own is an attention over that chunk's keys (torch, float64): pacc / psum is its
    output, pmax its largest score; merged, the chunks give the unsplit attention."""
    g = synth.rng(m * 31 + n + split)
    q = g.standard_normal((m, heads * head_dim)).astype(np.float32)
    k = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    v = g.standard_normal((n, kv_heads * head_dim)).astype(np.float32)
    pacc, pmax, psum = oracle.attention_split(q, k, v, m, n, heads, kv_heads, head_dim, split, q_base, window, causal)
    group = heads // kv_heads
    empties = 0
    for i in range(m):
        pos = q_base + i
        last = min(pos, n - 1) if causal else n - 1
        start = min(max(0, pos + 1 - window) if (causal and window) else 0, last)
        chunk = -(-(last + 1 - start) // split)
        for h in range(heads):
            for s in range(split):
                base = (i * heads + h) * split + s
                lo = start + s * chunk
                if lo > last:
                    assert pmax[base] == np.float32(-1e30) and psum[base] == 0 and not pacc[base].any()
                    empties += 1
                    continue
                hi = min(lo + chunk - 1, last)
                kk = k[lo:hi + 1].reshape(-1, kv_heads, head_dim)[:, h // group].astype(np.float64)
                vv = v[lo:hi + 1].reshape(-1, kv_heads, head_dim)[:, h // group].astype(np.float64)
                sc = kk @ q[i].reshape(heads, head_dim)[h].astype(np.float64) / np.sqrt(np.float32(head_dim)).astype(np.float64)
                w = np.exp(sc - sc.max())
                assert abs(pmax[base] - sc.max()) <= 2e-6 * max(1.0, abs(sc.max()))
                assert abs(psum[base] - w.sum()) <= 2e-6 * w.sum() and psum[base] >= 1.0
                assert np.max(np.abs(pacc[base] - w @ vv)) <= 4e-6 * max(1.0, np.max(np.abs(w @ vv)))
    if split > n:
        assert empties > 0
    merged = oracle.attention_combine(pacc, pmax, psum, m, heads, head_dim, split)
    want = torch_attention(q, k, v, m, n, heads, kv_heads, head_dim, q_base, window, causal)
    assert np.max(np.abs(merged - want)) <= 3e-6 * max(1.0, np.max(np.abs(want)))
