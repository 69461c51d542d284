"""Seeded synthetic tensors in the reference's weight-buffer layouts.

One generator per benchmark configuration, shared by the tests and ``bench.py`` so the
CPU and GPU sides see identical bytes.  All randomness comes from
``numpy.random.Generator(PCG64(seed))``.

Layouts:
  * Q4_K: rows of 144-byte super-blocks -- fp16 d, fp16 dmin, 12 bytes packing eight
    (6-bit scale, 6-bit min) pairs, 128 quant bytes (src/core/numerics/quant.hpp:11-15;
    packing rule src/core/numerics/quant.cpp:58-70,712-720);
  * MXFP4: n*k/2 nibble bytes (low nibble = even element) followed by n*k/32 E8M0 bytes
    (include/tessera/backend.hpp:195-201; src/core/loaders/mxfp4.cpp:217-259);
  * FP8: n*k E4M3 bytes plus one fp32 scale per row (include/tessera/backend.hpp:191-194).
"""
from __future__ import annotations

import numpy as np

Q4K_ELEMS = 256
Q4K_BYTES = 144


def rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def pack_q4k_scales(sc: np.ndarray, mn: np.ndarray) -> np.ndarray:
    """(..., 8) 6-bit scales and mins -> (..., 12) packed bytes."""
    sc = sc.astype(np.uint8)
    mn = mn.astype(np.uint8)
    out = np.zeros(sc.shape[:-1] + (12,), dtype=np.uint8)
    out[..., 0:4] = (sc[..., 0:4] & 63) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = (mn[..., 0:4] & 63) | ((mn[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 15) | ((mn[..., 4:8] & 15) << 4)
    return out


def q4k_weights(g: np.random.Generator, n: int, k: int) -> np.ndarray:
    """n x k Q4_K matrix: d, dmin ~ U[1e-3, 2e-2] (rounded to fp16), scales/mins ~ U{0..63},
    quants ~ U{0..15}.  Returns a flat uint8 array of n * k/256 * 144 bytes."""
    assert k % Q4K_ELEMS == 0
    nb = n * (k // Q4K_ELEMS)
    blocks = np.empty((nb, Q4K_BYTES), dtype=np.uint8)
    d = g.uniform(1e-3, 2e-2, size=(nb, 2)).astype(np.float32).astype(np.float16)
    blocks[:, 0:4] = d.view(np.uint8).reshape(nb, 4)
    sc = g.integers(0, 64, size=(nb, 8), dtype=np.uint8)
    mn = g.integers(0, 64, size=(nb, 8), dtype=np.uint8)
    blocks[:, 4:16] = pack_q4k_scales(sc, mn)
    blocks[:, 16:] = g.integers(0, 256, size=(nb, 128), dtype=np.uint8)
    return blocks.reshape(-1)


Q5K_BYTES = 176
Q6K_BYTES = 210


def q5k_weights(g: np.random.Generator, n: int, k: int) -> np.ndarray:
    """n x k Q5_K matrix (176-byte super-blocks: fp16 d, dmin, 12 packed scale/min bytes, 32 bytes
    of high bits, 128 bytes of low nibbles): d, dmin ~ U[5e-4, 1e-2] (rounded to fp16),
    scales/mins ~ U{0..63}, quants uniform.  Flat uint8 array."""
    assert k % Q4K_ELEMS == 0
    nb = n * (k // Q4K_ELEMS)
    blocks = np.empty((nb, Q5K_BYTES), dtype=np.uint8)
    d = g.uniform(5e-4, 1e-2, size=(nb, 2)).astype(np.float32).astype(np.float16)
    blocks[:, 0:4] = d.view(np.uint8).reshape(nb, 4)
    sc = g.integers(0, 64, size=(nb, 8), dtype=np.uint8)
    mn = g.integers(0, 64, size=(nb, 8), dtype=np.uint8)
    blocks[:, 4:16] = pack_q4k_scales(sc, mn)
    blocks[:, 16:] = g.integers(0, 256, size=(nb, 160), dtype=np.uint8)
    return blocks.reshape(-1)


def q6k_weights(g: np.random.Generator, n: int, k: int) -> np.ndarray:
    """n x k Q6_K matrix (210-byte super-blocks: 128 low-nibble bytes, 64 bytes of 2-bit highs,
    16 int8 scales, fp16 d): quants and scales uniform over their whole ranges (scales include
    negative values and -128), d ~ U[1e-4, 2e-3] rounded to fp16.  Flat uint8 array."""
    assert k % Q4K_ELEMS == 0
    nb = n * (k // Q4K_ELEMS)
    blocks = np.empty((nb, Q6K_BYTES), dtype=np.uint8)
    blocks[:, 0:208] = g.integers(0, 256, size=(nb, 208), dtype=np.uint8)
    d = g.uniform(1e-4, 2e-3, size=(nb, 1)).astype(np.float32).astype(np.float16)
    blocks[:, 208:210] = d.view(np.uint8).reshape(nb, 2)
    return blocks.reshape(-1)


def mxfp4_weights(g: np.random.Generator, n: int, k: int, exp_lo: int = -8,
                  exp_hi: int = -4) -> np.ndarray:
    """Packed MXFP4: E2M1 codes uniform over the 16 values, E8M0 exponent uniform in
    [exp_lo, exp_hi].  Returns blob then scales, flat uint8."""
    assert k % 32 == 0
    blob = g.integers(0, 256, size=n * k // 2, dtype=np.uint8)
    scales = (127 + g.integers(exp_lo, exp_hi + 1, size=n * k // 32)).astype(np.uint8)
    return np.concatenate([blob, scales])


def mxfp4_column_shard(packed: np.ndarray, n: int, k: int, row0: int, rows: int) -> np.ndarray:
    """Rows [row0, row0+rows) of a packed MXFP4 matrix as a packed matrix of its own: blob rows
    and scale rows are sliced separately and re-concatenated (the tensor-parallel column slice,
    src/core/loaders/tensor_slice.cpp:63-78)."""
    blob = packed[: n * k // 2].reshape(n, k // 2)
    sc = packed[n * k // 2:].reshape(n, k // 32)
    return np.concatenate([blob[row0:row0 + rows].reshape(-1), sc[row0:row0 + rows].reshape(-1)])


def encode_e4m3(x: np.ndarray) -> np.ndarray:
    """fp32 -> OCP E4M3 codes, round to nearest even, |x| clamped to 448 (numpy, for
    generating weights; the kernels and the oracle have their own encoders)."""
    x = np.clip(np.ascontiguousarray(x, dtype=np.float32), -448.0, 448.0)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint32)
    mag = bits & 0x7FFFFFFF
    sub = np.rint(np.abs(x) * np.float32(512.0)).astype(np.uint32)          # below 2^-6
    r = mag + 0x7FFFF + ((mag >> 20) & 1)
    norm = (r >> 20) - (120 << 3)
    code = np.where(mag < 0x3C800000, sub, norm)
    return (sign | code).astype(np.uint8)


def fp8_weights(g: np.random.Generator, n: int, k: int) -> tuple[np.ndarray, np.ndarray]:
    """A per-row-scaled E4M3 weight matrix as a real checkpoint holds it: W ~ N(0, 0.02^2),
    scale[r] = amax(W[r]) / 448, codes = e4m3(W / scale).  Returns (codes n*k, scales n)."""
    w = (g.standard_normal(size=(n, k)) * 0.02).astype(np.float32)
    scales = (np.abs(w).max(axis=1) / np.float32(448.0)).astype(np.float32)
    codes = encode_e4m3(w / scales[:, None])
    return codes.reshape(-1), scales


def fp8_block_weights(g: np.random.Generator, n: int, k: int) -> tuple[np.ndarray, np.ndarray]:
    """E4M3 weights with one scale per 128 x 128 block (n and k multiples of 128): W ~ N(0, 0.02^2)
    with a per-block gain, scale = amax(block) / 448, codes = e4m3(W / scale).  Returns
    (codes n*k, scales (n/128)*(k/128) row-major)."""
    nb, kb = n // 128, k // 128
    gain = g.uniform(0.25, 4.0, size=(nb, kb)).astype(np.float32)
    w = (g.standard_normal(size=(n, k)) * 0.02).astype(np.float32).reshape(nb, 128, kb, 128) * gain[:, None, :, None]
    scales = (np.abs(w).max(axis=(1, 3)) / np.float32(448.0)).astype(np.float32)
    codes = encode_e4m3((w / scales[:, None, :, None]).reshape(n, k))
    return codes.reshape(-1), scales.reshape(-1)


def activations_f32(g: np.random.Generator, m: int, k: int) -> np.ndarray:
    return g.standard_normal(size=(m, k)).astype(np.float32)


def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """fp32 -> nearest-even bf16 value, kept in fp32 storage."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    b = (b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000
    return b.astype(np.uint32).view(np.float32).reshape(x.shape)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """bf16-valued fp32 array -> uint16 bit patterns."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def activations_bf16(g: np.random.Generator, m: int, k: int) -> np.ndarray:
    """N(0,1) rounded to bf16 (fp32 storage)."""
    return round_to_bf16(activations_f32(g, m, k))


def activations_bf16_outliers(g: np.random.Generator, m: int, k: int, frac: float = 0.01,
                              gain: float = 20.0) -> np.ndarray:
    """N(0,1) with a fixed random 1% of the k channels scaled x20 (the same channels for every
    row), then rounded to bf16 (fp32 storage)."""
    x = activations_f32(g, m, k)
    ch = g.choice(k, size=max(1, int(round(frac * k))), replace=False)
    x[:, ch] *= gain
    return round_to_bf16(x)


def moe_routing(g: np.random.Generator, rows: int, n_experts: int, top_k: int):
    """Router logits ~ N(0,1); top-k by descending value; softmax over the selected k.
    Returns (ids uint32 rows x top_k, selected logits fp32 rows x top_k).  Asserts that the
    top_k + 1 largest logits of every row are distinct."""
    logits = g.standard_normal(size=(rows, n_experts)).astype(np.float32)
    order = np.argsort(-logits, axis=1, kind="stable")[:, :top_k]
    vals = np.take_along_axis(logits, order, axis=1)
    # only ties among the selected values or at the selection boundary would make the
    # choice depend on the tie rule
    top = -np.sort(-logits, axis=1)[:, : top_k + 1]
    assert np.all(top[:, 1:] != top[:, :-1]), "router logits tie at the top-k boundary"
    return order.astype(np.uint32), vals


def one_hot_rows(k: int, positions) -> np.ndarray:
    a = np.zeros((len(positions), k), dtype=np.float32)
    for r, t in enumerate(positions):
        a[r, t] = 1.0
    return a
