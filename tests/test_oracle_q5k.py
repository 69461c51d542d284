"""Pins the oracle's Q5_K routines without running any reference code.

Independent sources: a bit-serial reading of the layout text (src/core/numerics/quant.hpp:592-595,
"d, dmin, 12 scale/min bytes, 32 high bits, 128 low nibbles"; ggml's block_q5_K, which the
reference says it ports; the scale/min packing is the Q4_K one, pinned in test_oracle_q4k.py),
the closed form value = RN32(d*sc*q - dmin*mn) with both products exact, evaluated in float64,
and the sequential-fma GEMM against a float64 dot product.
"""
import numpy as np

import oracle
from tessera_amd import synth
from test_oracle_q4k import bit_serial_scale_min


def bit_serial_q5k(block: np.ndarray) -> np.ndarray:
    """256 values of one block read bit by bit.  Element e = g*64 + h*32 + l (group g, half h,
    lane l): low four bits = nibble h of byte qs[g*32 + l] (block byte 48 + g*32 + l); fifth bit =
    bit 2g + h of byte qh[l] (block byte 16 + l); scale/min = sub-block 2g + h."""
    bits = np.unpackbits(block, bitorder="little")
    d = float(block[0:2].view(np.float16)[0])
    dmin = float(block[2:4].view(np.float16)[0])
    out = np.empty(256, np.float64)
    for e in range(256):
        g, h, l = e // 64, (e % 64) // 32, e % 32
        lo = sum(int(bits[8 * (48 + g * 32 + l) + 4 * h + i]) << i for i in range(4))
        hi = int(bits[8 * (16 + l) + 2 * g + h])
        sc, mn = bit_serial_scale_min(block[4:16], 2 * g + h)
        out[e] = np.float32(d * sc * (lo + 16 * hi) - dmin * mn)   # both products exact; one rounding
    return out


def test_decode_matches_bit_serial_reading_exactly():
    g = synth.rng(51)
    w = synth.q5k_weights(g, 4, 1024).reshape(-1, 176)
    w[0] = 0
    w[1, 4:] = 0xFF
    w[2, 0:2] = np.array([-0.013], np.float16).view(np.uint8)
    w[3, 0:2] = np.array([3e-6], np.float16).view(np.uint8)
    got = oracle.dequantize_q5k(w.reshape(-1)).reshape(-1, 256)
    for b in range(w.shape[0]):
        assert np.array_equal(got[b].astype(np.float64), bit_serial_q5k(w[b])), b
    assert np.all(got[0] == 0.0)


def test_gemm_one_hot_zero_and_float64_bound():
    g = synth.rng(52)
    n, k, m = 37, 1024, 3
    w = synth.q5k_weights(g, n, k)
    deq = oracle.dequantize_q5k(w).reshape(n, k)
    hot = np.zeros((4, k), np.float32)
    pos = [0, 255, 256 + 131, k - 1]
    for r, t in enumerate(pos):
        hot[r, t] = 1.0
    c = oracle.gemm_q5k(hot, w, 4, n, k)
    for r, t in enumerate(pos):
        assert np.array_equal(c[r], deq[:, t])
    assert np.all(oracle.gemm_q5k(np.zeros((1, k), np.float32), w, 1, n, k) == 0.0)
    a = synth.activations_f32(g, m, k)
    c = oracle.gemm_q5k(a, w, m, n, k)
    ref = a.astype(np.float64) @ deq.astype(np.float64).T
    bound = k * 2.0 ** -24 * (np.abs(a).astype(np.float64) @ np.abs(deq).astype(np.float64).T)
    assert np.all(np.abs(c - ref) <= bound + 1e-30)
    assert np.array_equal(oracle.gemm_q5k(a, w, m, n, k, threads=True), c)
