"""Pins the oracle's scalar codecs against independent sources: numpy/torch IEEE
conversions, closed forms, and the known-answer values the reference documents in
src/core/numerics/quant.hpp (:21-22, :93-94, :101-102, :108-109, :564-565)."""
import math

import numpy as np
import pytest
import torch

import oracle


def test_documented_known_answers():
    assert oracle.fp16_to_float(0x3C00) == 1.0
    assert oracle.e8m0_to_float(127) == 1.0
    assert oracle.f4e2m1_to_float(3) == 1.5
    # quant.hpp:88-94 and :560-565 say "bias 8" and pair 0x40 with 1.0, but the code they
    # document (quant.cpp:258-277, 299-342) uses the OCP bias of 7, and so does the reference's
    # own fold table (quant.cpp:846-863 encodes magnitude 1.0 at shift 0 as 0x38).  The code and
    # the table are the contract: 1.0 <-> 0x38, 0x40 <-> 2.0.
    assert oracle.fp8_e4m3_to_float(0x38) == 1.0 and oracle.fp8_e4m3_to_float(0x40) == 2.0
    assert oracle.fp32_to_fp8_e4m3(1.0) == 0x38


def test_fp16_to_float_exhaustive_vs_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.fp16_to_float(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_fp32_to_half_bits_vs_numpy():
    g = np.random.default_rng(1)
    vals = np.concatenate([
        g.standard_normal(20000).astype(np.float32),
        (g.standard_normal(20000) * 1e-6).astype(np.float32),   # fp16 subnormal range
        (g.standard_normal(5000) * 7e4).astype(np.float32),     # overflow edge
        np.array([0.0, -0.0, 65504.0, 65520.0, 65519.99, 2.0**-24, 2.0**-25, 3 * 2.0**-25,
                  np.inf, -np.inf, 5.9604645e-08, 6.097555e-05], dtype=np.float32),
    ])
    want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.fp32_to_half_bits(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)
    # every fp16 value survives the round trip
    allh = np.arange(65536, dtype=np.uint16)
    fin = allh[(allh & 0x7C00) != 0x7C00]
    back = np.array([oracle.fp32_to_half_bits(float(f)) for f in fin.view(np.float16).astype(np.float32)],
                    dtype=np.uint16)
    assert np.array_equal(back, fin)


def test_e8m0_all_codes():
    for s in range(255):
        assert oracle.e8m0_to_float(s) == math.ldexp(1.0, s - 127)
    assert oracle.e8m0_to_float(0) == 2.0 ** -127 and oracle.e8m0_to_float(0) > 0
    assert math.isinf(oracle.e8m0_to_float(255))


def test_e2m1_all_codes():
    table = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for nib in range(16):
        v = oracle.f4e2m1_to_float(nib)
        assert abs(v) == table[nib & 7]
        assert math.copysign(1.0, v) == (-1.0 if nib & 8 else 1.0)


def test_e4m3_decode_all_codes_vs_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).to(torch.float32).numpy()
    got = np.array([oracle.fp8_e4m3_to_float(c) for c in range(256)], dtype=np.float32)
    nan = np.isnan(want)
    assert nan.sum() == 2 and np.array_equal(np.isnan(got), nan)       # 0x7F and 0xFF only
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert oracle.fp8_e4m3_to_float(0x38) == 1.0 and oracle.fp8_e4m3_to_float(0x7E) == 448.0
    assert oracle.fp8_e4m3_to_float(0x01) == 2.0 ** -9


def _e4m3_values():
    return np.array([oracle.fp8_e4m3_to_float(c) for c in range(0x7F)], dtype=np.float64)


def test_e4m3_encode_roundtrip_midpoints_and_saturation():
    vals = _e4m3_values()
    for c in range(0x7F):
        assert oracle.fp32_to_fp8_e4m3(float(vals[c])) == c
        if c:
            assert oracle.fp32_to_fp8_e4m3(-float(vals[c])) == (c | 0x80)
    assert oracle.fp32_to_fp8_e4m3(-0.0) == 0x80
    # Midpoints between neighbours go to the even mantissa; just off a midpoint goes to the
    # nearer neighbour.  The one exception is the reference's subnormal branch, which caps the
    # mantissa at 7: [7.5 * 2^-9, 2^-6) encodes to 0x07 instead of rounding up to 0x08
    # (src/core/numerics/quant.cpp:321-328).
    for c in range(0x7E):
        lo, hi = vals[c], vals[c + 1]
        mid = np.float32((lo + hi) / 2)
        assert float(mid) == (lo + hi) / 2
        even = c if c % 2 == 0 else c + 1
        if c == 7:
            even = 7
        assert oracle.fp32_to_fp8_e4m3(float(mid)) == even, hex(c)
        below = np.nextafter(mid, np.float32(0))
        above = np.nextafter(mid, np.float32(np.inf))
        assert oracle.fp32_to_fp8_e4m3(float(below)) == c
        assert oracle.fp32_to_fp8_e4m3(float(above)) == (7 if c == 7 else c + 1)
    assert oracle.fp32_to_fp8_e4m3(448.0) == 0x7E
    assert oracle.fp32_to_fp8_e4m3(float(np.nextafter(np.float32(448), np.float32(1e9)))) == 0x7F
    assert oracle.fp32_to_fp8_e4m3(1e30) == 0x7F and oracle.fp32_to_fp8_e4m3(-1e30) == 0xFF
    assert oracle.fp32_to_fp8_e4m3(float("inf")) == 0x7F
    assert oracle.fp32_to_fp8_e4m3(float("nan")) & 0x7F == 0x7F
    assert oracle.fp32_to_fp8_e4m3(1.0) == 0x38  # quant.hpp:564-565 names this value's code


def test_e4m3_encode_vs_torch_random():
    g = np.random.default_rng(7)
    x = np.concatenate([
        g.uniform(-448, 448, 50000), g.standard_normal(50000), g.standard_normal(50000) * 0.01,
        g.uniform(-2.0 ** -6, 2.0 ** -6, 20000)]).astype(np.float32)
    # outside the subnormal-cap interval torch's RNE cast is the same function
    keep = ~((np.abs(x) >= 7.5 * 2.0 ** -9) & (np.abs(x) < 2.0 ** -6))
    x = x[keep]
    want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([oracle.fp32_to_fp8_e4m3(float(v)) for v in x], dtype=np.uint8)
    assert np.array_equal(got, want)
    # monotone over a sorted sweep
    xs = np.sort(np.abs(x))
    codes = np.array([oracle.fp32_to_fp8_e4m3(float(v)) for v in xs[::50]])
    assert np.all(np.diff(codes.astype(int)) >= 0)


def test_e4m3_encode_every_input_vs_torch():
    """Every fp32 bit pattern with |x| <= 448 (2 x 1 138 753 537 of them, zeros and subnormals
    included) through the threaded array entry against torch's float8_e4m3fn cast, which is the
    same round-to-nearest-even function outside the reference's subnormal-cap interval
    [7.5 * 2^-9, 2^-6) (that interval is pinned by the midpoint test above); the array entry
    equals the scalar one on a sample."""
    top = int(np.float32(448.0).view(np.uint32))
    chunk = 1 << 26
    for sign in (0, 0x80000000):
        for base in range(0, top + 1, chunk):
            bits = np.arange(base, min(base + chunk, top + 1), dtype=np.uint32) | np.uint32(sign)
            x = bits.view(np.float32)
            got = oracle.fp32_to_fp8_e4m3_many(x)
            want = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
            ax = np.abs(x)
            keep = ~((ax >= 7.5 * 2.0 ** -9) & (ax < 2.0 ** -6))
            if not np.array_equal(got[keep], want[keep]):
                i = np.flatnonzero((got != want) & keep)[0]
                raise AssertionError(f"bits {int(bits[i]):#010x}: oracle {got[i]:#04x}, torch {want[i]:#04x}")
    g = np.random.default_rng(11)
    sample = g.integers(0, top + 1, 2000).astype(np.uint32).view(np.float32)
    assert np.array_equal(oracle.fp32_to_fp8_e4m3_many(sample),
                          np.array([oracle.fp32_to_fp8_e4m3(float(v)) for v in sample], np.uint8))


def test_round_bf16_vs_torch():
    g = np.random.default_rng(3)
    x = np.concatenate([g.standard_normal(100000), g.standard_normal(1000) * 1e-30,
                        g.standard_normal(1000) * 1e30]).astype(np.float32)
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(oracle.round_bf16(x).view(np.uint32), want.view(np.uint32))
    from tessera_amd import synth
    assert np.array_equal(synth.round_to_bf16(x).view(np.uint32), want.view(np.uint32))
