"""Pins the oracle's restatements of the non-matmul trunk pieces that sit around the projections:
RopeRef, MropeRef, AttentionRef (fp32 and fp16 keys/values), QGateSplitRef
(src/core/numerics/attention.cpp)."""
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
