"""Pins the oracle's Q6_K routines without running any reference code.

Independent sources: a bit-serial reading of the layout text (src/core/numerics/quant.hpp:597-600,
"128 low nibbles, 64 2-bit highs, 16 int8 scales, d"; ggml's block_q6_K / dequantize_row_q6_K,
which the reference says it ports), the closed form value = d * s * (q - 32), exact in fp32 and
evaluated here in float64, and the sequential-fma GEMM against a float64 dot product.
"""
import numpy as np

import oracle
from tessera_amd import synth


def bit_serial_q6k(block: np.ndarray) -> np.ndarray:
    """256 values of one block read bit by bit.  Element e = n*128 + j*32 + l (n half, j quarter,
    l lane): low four bits = nibble (j // 2) of byte ql[n*64 + (j % 2)*32 + l]; high two bits =
    bits [2j, 2j+2) of byte qh[n*32 + l]; scale = int8 sc[n*8 + 2*j + l // 16]."""
    bits = np.unpackbits(block, bitorder="little")
    d = float(block[208:210].view(np.float16)[0])
    out = np.empty(256, np.float64)
    for e in range(256):
        n, j, l = e // 128, (e % 128) // 32, e % 32
        lo_byte = n * 64 + (j % 2) * 32 + l
        lo = sum(int(bits[8 * lo_byte + 4 * (j // 2) + i]) << i for i in range(4))
        hi_byte = 128 + n * 32 + l
        hi = sum(int(bits[8 * hi_byte + 2 * j + i]) << i for i in range(2))
        s_byte = 192 + n * 8 + 2 * j + l // 16
        s = sum(int(bits[8 * s_byte + i]) << i for i in range(8))
        s = s - 256 if s >= 128 else s
        out[e] = d * s * ((lo | (hi << 4)) - 32)
    return out


def test_decode_matches_bit_serial_reading_exactly():
    g = synth.rng(61)
    w = synth.q6k_weights(g, 4, 1024).reshape(-1, 210)
    # edge blocks: zeros, all ones, extreme scales, negative and subnormal d
    w[0] = 0
    w[1, :208] = 0xFF
    w[2, 192:208] = np.array([-128, 127, -1, 1] * 4, np.int8).view(np.uint8)
    w[3, 208:210] = np.array([-0.0007], np.float16).view(np.uint8)
    w[4, 208:210] = np.array([3e-7], np.float16).view(np.uint8)
    got = oracle.dequantize_q6k(w.reshape(-1)).reshape(-1, 256)
    for b in range(w.shape[0]):
        ref = bit_serial_q6k(w[b])
        # d (11 bits) * s (8) * (q - 32) (6) fits fp32 exactly: float64 and fp32 agree bit for bit
        assert np.array_equal(got[b].astype(np.float64), ref), b
    assert np.all(got[0] == 0.0)


def test_gemm_one_hot_zero_and_float64_bound():
    g = synth.rng(62)
    n, k, m = 37, 1024, 3
    w = synth.q6k_weights(g, n, k)
    deq = oracle.dequantize_q6k(w).reshape(n, k)
    hot = np.zeros((4, k), np.float32)
    pos = [0, 255, 256 + 131, k - 1]
    for r, t in enumerate(pos):
        hot[r, t] = 1.0
    c = oracle.gemm_q6k(hot, w, 4, n, k)
    for r, t in enumerate(pos):
        assert np.array_equal(c[r], deq[:, t])
    assert np.all(oracle.gemm_q6k(np.zeros((1, k), np.float32), w, 1, n, k) == 0.0)
    a = synth.activations_f32(g, m, k)
    c = oracle.gemm_q6k(a, w, m, n, k)
    ref = a.astype(np.float64) @ deq.astype(np.float64).T
    bound = k * 2.0 ** -24 * (np.abs(a).astype(np.float64) @ np.abs(deq).astype(np.float64).T)
    assert np.all(np.abs(c - ref) <= bound + 1e-30)
    assert np.array_equal(oracle.gemm_q6k(a, w, m, n, k, threads=True), c)
    with np.testing.assert_raises(oracle.OracleError):
        oracle.gemm_q6k(a[:, :200], w, m, n, 200)
