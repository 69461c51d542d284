"""Pins the oracle's Q4_K routines without running any reference code.

Independent sources: a bit-serial reading of the layout text
(src/core/numerics/quant.hpp:11-15: "12 bytes packing 8 x (6-bit scale, 6-bit min)";
ggml's get_scale_min_k4 bit positions), the closed form value = RN32(d*sc*q - dmin*mn)
evaluated in float64, and the quantizer's documented error bound
(src/core/numerics/quant.hpp:585-589).
"""
import numpy as np
import pytest

import oracle
from tessera_amd import synth


def bit_serial_scale_min(p12: np.ndarray, j: int) -> tuple[int, int]:
    """Scale/min of sub-block j read bit by bit from the 96-bit field.

    Bits of byte i are numbered 8*i .. 8*i+7 (LSB first).  Sub-blocks 0..3: scale = bits
    [8j, 8j+6), min = bits [8(j+4), 8(j+4)+6).  Sub-blocks 4..7: scale = low nibble of byte
    j+4 with bits 6..7 of byte j-4 on top; min = high nibble of byte j+4 with bits 6..7 of
    byte j on top."""
    bits = np.unpackbits(p12, bitorder="little")

    def field(start: int, width: int) -> int:
        return int(sum(int(bits[start + i]) << i for i in range(width)))

    if j < 4:
        return field(8 * j, 6), field(8 * (j + 4), 6)
    sc = field(8 * (j + 4), 4) | (field(8 * (j - 4) + 6, 2) << 4)
    mn = field(8 * (j + 4) + 4, 4) | (field(8 * j + 6, 2) << 4)
    return sc, mn


def test_get_scale_min_bruteforce_boundaries():
    edge = [0, 1, 15, 16, 31, 32, 47, 48, 62, 63]
    g = np.random.default_rng(0)
    for j in range(8):
        for sc in edge:
            for mn in edge:
                scs = g.integers(0, 64, 8)
                mns = g.integers(0, 64, 8)
                scs[j], mns[j] = sc, mn
                p = synth.pack_q4k_scales(scs[None, :], mns[None, :])[0]
                assert oracle.get_scale_min(j, p) == (sc, mn)
                assert bit_serial_scale_min(p, j) == (sc, mn)
    for _ in range(2000):  # arbitrary byte patterns, not only packer outputs
        p = g.integers(0, 256, 12, dtype=np.uint8)
        for j in range(8):
            assert oracle.get_scale_min(j, p) == bit_serial_scale_min(p, j)


def closed_form_block(block: np.ndarray) -> np.ndarray:
    """float64 evaluation of d*sc*q - dmin*mn, rounded once to fp32."""
    d = float(block[0:2].view(np.float16)[0])
    dmin = float(block[2:4].view(np.float16)[0])
    out = np.empty(256, dtype=np.float32)
    for sub in range(8):
        sc, mn = bit_serial_scale_min(block[4:16], sub)
        grp, hi = divmod(sub, 2)
        q = block[16 + 32 * grp: 16 + 32 * grp + 32]
        nib = (q >> 4) if hi else (q & 15)
        # d*sc*q <= 21 significant bits and dmin*mn <= 17: both exact in float64 and fp32
        out[32 * sub: 32 * sub + 32] = (d * sc * nib.astype(np.float64) - dmin * mn).astype(np.float32)
    return out


def test_dequantize_matches_closed_form():
    g = synth.rng(11)
    w = synth.q4k_weights(g, 16, 1024).reshape(-1, 144)
    got = oracle.dequantize_q4k(w).reshape(-1, 256)
    for b in range(w.shape[0]):
        assert np.array_equal(got[b].view(np.uint32), closed_form_block(w[b]).view(np.uint32))


def test_dequantize_special_blocks():
    zero = np.zeros(144, dtype=np.uint8)
    assert np.all(oracle.dequantize_q4k(zero) == 0.0)
    # one quant set, everything else neutral: d = 1, sc[0] = 1 -> element 0 == q
    blk = np.zeros(144, dtype=np.uint8)
    blk[0:2] = np.array([1.0], dtype=np.float16).view(np.uint8)
    blk[4] = 1
    blk[16] = 0x0B
    out = oracle.dequantize_q4k(blk)
    assert out[0] == 11.0 and np.count_nonzero(out) == 1
    # high nibble of qs byte 0 is element 32, scaled by sub-block 1
    blk[5] = 2
    blk[16] = 0xB0
    out = oracle.dequantize_q4k(blk)
    assert out[32] == 22.0 and np.count_nonzero(out) == 1
    # the min term: dmin = 0.5, mn[2] = 3 -> elements 64..95 == -1.5
    blk = np.zeros(144, dtype=np.uint8)
    blk[2:4] = np.array([0.5], dtype=np.float16).view(np.uint8)
    blk[4 + 6] = 3
    out = oracle.dequantize_q4k(blk)
    assert np.all(out[64:96] == -1.5) and np.count_nonzero(out) == 32


def test_quantize_roundtrip_bound():
    g = np.random.default_rng(5)
    x = g.standard_normal(256 * 40).astype(np.float32)
    w = oracle.quantize_q4k(x)
    y = oracle.dequantize_q4k(w)
    for b in range(40):
        xb, yb = x[b * 256:(b + 1) * 256], y[b * 256:(b + 1) * 256]
        d = float(w[b * 144: b * 144 + 2].view(np.float16)[0])
        for sub in range(8):
            sc, _ = oracle.get_scale_min(sub, w[b * 144 + 4: b * 144 + 16])
            err = np.max(np.abs(xb[32 * sub: 32 * sub + 32] - yb[32 * sub: 32 * sub + 32]))
            # step/2 + dm/2 as documented, plus the clipping a step rounded down by up to d/2
            # causes at q = 15 (15 * d/2); a small slack covers the fp32 arithmetic
            assert err <= (d * sc) / 2 + d / 2 + 7.5 * d + 1e-5
        rel = np.linalg.norm(xb - yb) / np.linalg.norm(xb)
        assert rel < 0.2
    assert np.all(oracle.quantize_q4k(np.zeros(256, np.float32)) == 0)


def test_gemm_q4k_one_hot_is_dequant_and_float64_bound():
    g = synth.rng(21)
    n, k = 24, 768
    w = synth.q4k_weights(g, n, k)
    deq = oracle.dequantize_q4k(w).reshape(n, k)
    pos = [0, 31, 32, 63, 64, 255, 256, 300, 767]
    a = synth.one_hot_rows(k, pos)
    c = oracle.gemm_q4k(a, w, len(pos), n, k)
    for r, t in enumerate(pos):
        assert np.array_equal(c[r].view(np.uint32), deq[:, t].view(np.uint32))
    a = synth.activations_f32(g, 3, k)
    c = oracle.gemm_q4k(a, w, 3, n, k)
    ref = a.astype(np.float64) @ deq.astype(np.float64).T
    bound = k * 2.0 ** -24 * (np.abs(a).astype(np.float64) @ np.abs(deq).astype(np.float64).T)
    assert np.all(np.abs(c - ref) <= bound)
    assert np.array_equal(oracle.gemm_q4k(a, w, 3, n, k, threads=True).view(np.uint32), c.view(np.uint32))
    assert np.all(oracle.gemm_q4k(np.zeros((1, k), np.float32), w, 1, n, k) == 0.0)


def test_gemm_q4k_rejects_bad_shapes():
    for m, n, k in [(0, 4, 256), (1, 0, 256), (1, 4, 0), (1, 4, 100)]:
        with pytest.raises(oracle.OracleError) as e:
            oracle.gemm_q4k(np.zeros(max(m * k, 1), np.float32), np.zeros(144, np.uint8), m, n, k)
        assert e.value.code == 1


def decode_rowgroups(buf: np.ndarray, n: int, k: int, R: int) -> np.ndarray:
    """deq(W) read straight from a row-group copy, following the layout's text only (no call into the
    oracle): group g keeps, per block, the tiles' quants and then the rows' headers; a weight of
    sub-block s < 4 is a low nibble of pair set s // 2, one of s >= 4 a high nibble (stored minus 8) of
    pair set (s - 4) // 2; value = RN32(d * sc * q - dmin * mn) from exact products."""
    buf = np.asarray(buf, np.uint8).reshape(-1)
    nblk = k // 256
    out = np.empty((n, k), np.float32)
    for r in range(n):
        row0 = r // R * R
        rows = min(R, n - row0)
        rr = r - row0
        tile, nn = divmod(rr, 16)
        rt = min(16, rows - tile * 16)
        for b in range(nblk):
            region = (row0 * nblk + b * rows) * 144
            h = buf[region + rows * 128 + rr * 16:][:16]
            d, dmin = (float(v) for v in h[:4].view(np.float16))
            for s in range(8):
                i, odd = divmod(s, 2)
                if odd:
                    sc = int(h[8 + i]) & 63
                    mn = (int(h[4 + i]) >> 6) | ((int(h[8 + i]) >> 6) << 2) | ((int(h[12 + i]) >> 6) << 4)
                else:
                    sc = int(h[4 + i]) & 63
                    mn = int(h[12 + i]) & 63
                c = (s % 4) // 2
                for l in range(32):
                    q4 = 2 * (s % 2) + l // 16
                    byte = int(buf[region + tile * 2048 + c * rt * 64 + (q4 * rt + nn) * 16 + l % 16])
                    q = (byte & 15) if s < 4 else (((byte >> 4) + 8) & 15)
                    out[r, b * 256 + s * 32 + l] = np.float32(d * sc * q - dmin * mn)   # float64, rounded once
    return out


@pytest.mark.parametrize("n,k,R", [(40, 512, 32), (21, 256, 16), (70, 256, 64), (9, 512, 7), (33, 256, 20)])
def test_rowgroup_copy_is_a_permutation_that_decodes_to_the_same_weights(n, k, R):
    g = synth.rng(77 + n)
    w = synth.q4k_weights(g, n, k)
    # every scale / min value somewhere, so that a wrong bit position in the re-packed header shows
    blocks = np.asarray(w).reshape(-1, 144)
    blocks[:, 4:16] = g.integers(0, 256, (blocks.shape[0], 12), dtype=np.uint8)
    w = blocks.reshape(-1)
    p = oracle.permute_q4k_rowgroup(w, n, k, R)
    assert p.shape == w.shape
    assert np.array_equal(oracle.permute_q4k_rowgroup(p, n, k, R, inverse=True), w)
    want = oracle.dequantize_q4k(w).reshape(n, k)
    got = decode_rowgroups(p, n, k, R)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
