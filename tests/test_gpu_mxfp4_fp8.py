"""GPU parity of the MXFP4, W4A8 and FP8 paths against the CPU oracle, through the C ABI.

Bit-exact: MXFP4 dequant (every E2M1 code under every E8M0 exponent), E4M3 codes and scales
of the per-token activation quantizer.  Tolerance: GEMV outputs vs the oracle's sequential
fp32 fma, max relative error 1e-3 (tests/util.py:rel_err); the W4A8 kernels multiply exact
E4M3 x E2M1 products, so their error is summation order only and the same bound holds."""
import numpy as np
import pytest

import oracle
from tessera_amd import StatusCode, StatusError, synth
from util import norm_err, rel_err, rms_err, run, same_bits, same_bits_zero_sign_free, strict_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-3


def mx_gemm(backend, name, a, w, m, n, k):
    da, dw = backend.Upload(a), backend.Upload(w)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, name, [da, dw, dc], [m, n, k], grid=((m * n + 7) // 8, 1, 1))
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


def test_mxfp4_dequant_every_code_every_exponent(backend):
    n, k = 256, 32 * 8
    blob = np.tile(np.arange(256, dtype=np.uint8), n * k // 2 // 256 + 1)[: n * k // 2]
    scales = np.repeat(np.arange(255, dtype=np.uint8), 9)[: n * k // 32]   # 0..254, no 0xFF
    w = np.concatenate([blob, scales])
    dw = backend.Upload(w)
    out = backend.AllocateBuffer(4 * n * k)
    run(backend, "dequant_mxfp4", [dw, out], [n, k])
    backend.Synchronize()
    got = backend.CopyD2H(out, dtype=np.float32).reshape(n, k)
    assert same_bits(got, oracle.dequantize_mxfp4(w, n, k))


@pytest.mark.parametrize("k", [256, 1024, 5120])
def test_mxfp4_gemv_one_hot_reproduces_dequant(backend, k):
    g = synth.rng(300 + k)
    n = 80
    w = synth.mxfp4_weights(g, n, k, -20, 20)
    w[n * k // 2] = 0            # 2^-127, an fp32 subnormal
    deq = oracle.dequantize_mxfp4(w, n, k)
    pos = list(range(64)) + [int(t) for t in g.integers(0, k, 32)]
    for r0 in range(0, len(pos), 4):
        sel = pos[r0:r0 + 4]
        c = mx_gemm(backend, "gemm_mxfp4_rows", synth.one_hot_rows(k, sel), w, len(sel), n, k)
        for r, t in enumerate(sel):
            assert same_bits_zero_sign_free(c[r], deq[:, t]), (k, t)


MX_SHAPES = [(64, 256), (33, 512), (17, 96), (100, 1024), (129, 1280), (130, 5120), (67, 17408), (3, 32768)]


@pytest.mark.parametrize("n,k", MX_SHAPES)
@pytest.mark.parametrize("m", [1, 2, 3, 4, 7, 16])
def test_gemm_mxfp4_matches_oracle(backend, n, k, m):
    if m > 4 and k > 8192:
        pytest.skip("large-k multi-row cases are covered at m <= 4")
    g = synth.rng(2000 * m + n + k)
    w = synth.mxfp4_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_mxfp4(a, w, m, n, k)
    name = "gemm_mxfp4" if m == 1 else "gemm_mxfp4_rows"
    got = mx_gemm(backend, name, a, w, m, n, k)
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("m,n,k", [(17, 200, 1024), (20, 131, 5120), (33, 64, 2048), (64, 515, 1280), (100, 96, 4096)])
def test_gemm_mxfp4_batched_matches_oracle(backend, m, n, k):
    """The id ProjectBatch issues for MXFP4 with more than 16 rows
    (src/core/decode_internal.hpp:1494-1504): fp32 activations, no activation quantization."""
    g = synth.rng(2100 * m + n + k)
    w = synth.mxfp4_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_mxfp4(a, w, m, n, k)
    got = mx_gemm(backend, "gemm_mxfp4_batched", a, w, m, n, k)
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("n,k", [(3001, 96), (3003, 352), (2999, 768), (3001, 1280), (3005, 2560), (4099, 3072),
                                 (3002, 3584), (6007, 5120), (1027, 8192)])
@pytest.mark.parametrize("m", [1, 2, 4])
def test_mxfp4_many_output_columns(backend, n, k, m):
    """Enough weight rows that a workgroup takes several side by side, including rows shorter than
    a wavefront (lanes of one wavefront then belong to several weight rows); ragged last group."""
    g = synth.rng(37 * n + k + m)
    w = synth.mxfp4_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_mxfp4(a, w, m, n, k)
    got = mx_gemm(backend, "gemm_mxfp4" if m == 1 else "gemm_mxfp4_rows", a, w, m, n, k)
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


@pytest.mark.parametrize("n,k", [(3001, 80), (3003, 352), (2999, 768), (3001, 1280), (3005, 2560), (4099, 3072),
                                 (3002, 3584), (6007, 5120), (1027, 8192)])
@pytest.mark.parametrize("m", [1, 2, 4])
def test_fp8_many_output_columns(backend, n, k, m):
    g = synth.rng(41 * n + k + m)
    codes, scales = synth.fp8_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_fp8(a, codes, scales, m, n, k)
    da, dw, ds = backend.Upload(a), backend.Upload(codes), backend.Upload(scales)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_fp8", [da, dw, ds, dc], [m, n, k], grid=((m * n + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
    if m >= 2 and n * k >= 1 << 24 and k % 512 == 0:
        # several rows of 16 M weights or more go through the matrix cores: that path's bound
        # (tests/test_gpu_fp8_rows.py)
        assert rms_err(got, ref) <= 2e-4 and norm_err(got, ref) <= 2e-5, (rms_err(got, ref), norm_err(got, ref))
    else:
        assert rel_err(got, ref) <= TOL, rel_err(got, ref)


def quant_inputs(g, rows, cols):
    x = synth.activations_bf16_outliers(g, rows, cols)
    if rows > 2:
        x[1] = 0.0
        x[2] *= 1e-9
    return x


@pytest.mark.parametrize("rows,cols", [(1, 5120), (4, 5120), (16, 5120), (3, 100), (5, 17408), (2, 4)])
def test_quantize_fp8_pack_bit_exact(backend, rows, cols):
    g = synth.rng(rows * 131 + cols)
    x = quant_inputs(g, rows, cols)
    codes, scale = oracle.quantize_fp8_pack(x, rows, cols)
    for name in ("quantize_fp8_pack", "quantize_fp8_pack_rows"):
        dx = backend.Upload(x)
        dq = backend.AllocateBuffer(rows * cols)
        ds = backend.AllocateBuffer(4 * rows)
        run(backend, name, [dx, dq, ds], [rows, cols], grid=(rows, 1, 1), block=(1024, 1, 1))
        backend.Synchronize()
        assert np.array_equal(backend.CopyD2H(dq).reshape(rows, cols), codes)
        assert same_bits(backend.CopyD2H(ds, dtype=np.float32), scale)
    # bf16 input carries the same values
    dx16 = backend.Upload(synth.bf16_bits(x))
    dq = backend.AllocateBuffer(rows * cols)
    ds = backend.AllocateBuffer(4 * rows)
    run(backend, "quantize_fp8_pack_a16", [dx16, dq, ds], [rows, cols])
    backend.Synchronize()
    assert np.array_equal(backend.CopyD2H(dq).reshape(rows, cols), codes)
    assert same_bits(backend.CopyD2H(ds, dtype=np.float32), scale)


def test_quantize_fp8_encoder_sweep_bit_exact(backend):
    """The device E4M3 encoder against the oracle's on a dense sweep of fp32 inputs: every
    rounding boundary of every binade from 2^-12 to 448, scaled so the row scale is exactly 1
    (the row holds one 448)."""
    vals = [oracle.fp8_e4m3_to_float(c) for c in range(0x7F)]
    pts = []
    for lo, hi in zip(vals[:-1], vals[1:]):
        mid = np.float32((lo + hi) / 2)
        pts += [lo, mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(1e9)),
                np.nextafter(np.float32(hi), np.float32(0))]
    g = synth.rng(5)
    pts = np.array(pts + list(g.uniform(0, 448, 20000)) + list(g.uniform(0, 2.0 ** -5, 20000)) +
                   [448.0], dtype=np.float32)
    x = np.concatenate([pts, -pts])
    x = np.pad(x, (0, (-x.size) % 4)).reshape(1, -1)
    cols = x.shape[1]
    codes, scale = oracle.quantize_fp8_pack(x, 1, cols)
    assert scale[0] == 1.0
    dx = backend.Upload(x)
    dq, ds = backend.AllocateBuffer(cols), backend.AllocateBuffer(4)
    run(backend, "quantize_fp8_pack", [dx, dq, ds], [1, cols])
    backend.Synchronize()
    assert np.array_equal(backend.CopyD2H(dq).reshape(1, cols), codes)


def test_quantize_fp8_encoder_every_input(backend):
    """Every fp32 bit pattern the encoder can be handed under a unit row scale -- all 2 x 1 138 753 537
    values with |x| <= 448, zeros and subnormals included -- through quantize_fp8_pack on the
    device against the oracle's Fp32ToFp8E4M3Bits restatement (src/core/numerics/quant.hpp:564-565
    states its contract), in chunks of 2^24 patterns laid out as 4096 rows that each also hold a
    448, so that every row's scale is exactly 1.  Larger magnitudes never reach the encoder: the
    id clamps to +-448 first (covered by the QDQ tests below).  Stops at the first mismatch."""
    top = int(np.float32(448.0).view(np.uint32))          # 0x43E00000
    rows, per_row = 4096, 4096
    chunk = rows * per_row
    pad = np.full((rows, 4), 448.0, np.float32)
    dx = backend.AllocateBuffer(4 * rows * (per_row + 4))
    dq, ds = backend.AllocateBuffer(rows * (per_row + 4)), backend.AllocateBuffer(4 * rows)
    checked = 0
    for sign in (0, 0x80000000):
        for base in range(0, top + 1, chunk):
            bits = np.arange(base, base + chunk, dtype=np.uint64)
            bits = np.minimum(bits, top).astype(np.uint32) | np.uint32(sign)     # the last chunk repeats 448
            x = np.concatenate([bits.view(np.float32).reshape(rows, per_row), pad], axis=1)
            backend.CopyH2D(dx, x)
            run(backend, "quantize_fp8_pack", [dx, dq, ds], [rows, per_row + 4])
            backend.Synchronize()
            got = backend.CopyD2H(dq).reshape(rows, per_row + 4)
            assert np.all(backend.CopyD2H(ds, dtype=np.float32) == 1.0)
            want = oracle.fp32_to_fp8_e4m3_many(x).reshape(rows, per_row + 4)
            if not np.array_equal(got, want):
                r, c = np.argwhere(got != want)[0]
                raise AssertionError(f"input bits {int(x[r, c].view(np.uint32)):#010x}: device {got[r, c]:#04x}, oracle {want[r, c]:#04x}")
            checked += chunk
    assert checked >= 2 * (top + 1)


@pytest.mark.parametrize("rows,cols", [(1, 5120), (16, 5120), (3, 100), (4, 17408)])
def test_quantize_fp8_qdq_bit_exact(backend, rows, cols):
    g = synth.rng(rows * 17 + cols)
    x = quant_inputs(g, rows, cols)
    qdq, scale = oracle.quantize_fp8(x, rows, cols)
    dx = backend.Upload(x)
    ds = backend.AllocateBuffer(4 * rows)
    run(backend, "quantize_fp8", [dx, ds], [rows, cols], grid=(rows, 1, 1))
    backend.Synchronize()
    assert same_bits(backend.CopyD2H(dx, dtype=np.float32).reshape(rows, cols), qdq)
    assert same_bits(backend.CopyD2H(ds, dtype=np.float32), scale)


@pytest.mark.parametrize("n,k", [(64, 256), (100, 1024), (130, 5120), (33, 17408)])
@pytest.mark.parametrize("m,split", [(1, 1), (2, 1), (4, 2), (7, 1), (16, 4)])
def test_w4a8_wmma_contract(backend, n, k, m, split):
    """quantize_fp8_pack_rows -> mxfp4_row_ref -> gemm_mxfp4_wmma (-> reduce), the reference's
    verify pipeline (src/models/qwen3_5/project.cpp:92-231), against QuantizeFp8Ref +
    GemmMxFp4Ref."""
    if m > 4 and k > 8192:
        pytest.skip("large-k multi-row cases are covered at m <= 4")
    g = synth.rng(3000 * m + n + k)
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    x = synth.activations_bf16_outliers(g, m, k)
    codes, scale = oracle.quantize_fp8_pack(x, m, k)
    ref = oracle.gemm_mxfp4_w4a8(codes, scale, w, m, n, k)
    dx, dw = backend.Upload(x), backend.Upload(w)
    da8, das = backend.AllocateBuffer(m * k), backend.AllocateBuffer(4 * m)
    dref = backend.AllocateBuffer(n)
    part = backend.AllocateBuffer(4 * m * n * split)
    out = backend.AllocateBuffer(4 * m * n)
    run(backend, "quantize_fp8_pack_rows", [dx, da8, das], [m, k], grid=(m, 1, 1), block=(1024, 1, 1))
    run(backend, "mxfp4_row_ref", [dw, dref], [n, k], grid=((n + 255) // 256, 1, 1))
    run(backend, "gemm_mxfp4_wmma", [da8, dw, das, dref, part], [m, n, k, split, 0],
        grid=((n + 63) // 64, split, 1), block=(128, 1, 1))
    run(backend, "gemm_mxfp4_wmma_reduce", [part, out], [m * n, split], grid=((m * n + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(out, dtype=np.float32).reshape(m, n)
    # a single row runs on the fp32 VALU GEMV (1e-3); from two rows on the scaled MFMA takes
    # over, whose documented bound is 5e-4 of the rms output (test_gpu_gemm_mxfp4.py)
    tol = TOL if m <= 1 else 1e-2
    assert rel_err(got, ref) <= tol, rel_err(got, ref)
    assert rms_err(got, ref) <= 5e-4
    want_ref = w[n * k // 2:].reshape(n, -1).max(axis=1)
    assert np.array_equal(backend.CopyD2H(dref), want_ref)
    # and against the reference's folded arithmetic, which is exact at this exponent spread
    w8, wref = oracle.fold_mxfp4_to_fp8(w, n, k)
    folded = oracle.gemm_mxfp4_fp8(codes, scale, w8, wref, m, n, k)
    assert rel_err(got, folded) <= tol
    with pytest.raises(StatusError) as e:   # wperm is 0 or 1
        run(backend, "gemm_mxfp4_wmma", [da8, dw, das, dref, part], [m, n, k, split, 2])
    assert e.value.code == StatusCode.InvalidArgument


# rows longer than 16384 take the 32-weights-a-lane codec (17408: the dense down projection)
@pytest.mark.parametrize("n,k", [(64, 256), (100, 1008), (130, 5120), (40, 16384), (67, 17408), (9, 32768), (33, 16416)])
@pytest.mark.parametrize("m", [1, 2, 5])
def test_gemm_fp8_matches_oracle(backend, n, k, m):
    g = synth.rng(4000 * m + n + k)
    codes, scales = synth.fp8_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_fp8(a, codes, scales, m, n, k)
    da, dw, ds = backend.Upload(a), backend.Upload(codes), backend.Upload(scales)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_fp8", [da, dw, ds, dc], [m, n, k], grid=((m * n + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)


# 16 weights a lane (several rows), 32 (rows past 16384 long), 64 (one row); a row band and a K
# block boundary inside a workgroup's rows and inside a wavefront
@pytest.mark.parametrize("n,k", [(128, 128), (256, 1024), (384, 5120), (128, 17408), (128, 32768)])
@pytest.mark.parametrize("m", [1, 2, 5])
def test_gemm_fp8_block_matches_oracle(backend, n, k, m):
    """gemm_fp8_block: one scale per 128 x 128 block of W (GemmFp8BlockRef).  The device multiplies a
    lane's partial dot product by the block's scale where the reference scales every weight: same
    bound as gemm_fp8.  A one-hot row gives scale * weight bit for bit."""
    g = synth.rng(4100 * m + n + k)
    codes, scales = synth.fp8_block_weights(g, n, k)
    a = synth.activations_f32(g, m, k)
    ref = oracle.gemm_fp8_block(a, codes, scales, m, n, k)
    da, dw, ds = backend.Upload(a), backend.Upload(codes), backend.Upload(scales)
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_fp8_block", [da, dw, ds, dc], [m, n, k], grid=((m * n + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
    assert rel_err(got, ref) <= TOL, rel_err(got, ref)
    pos = sorted({min(p, k - 1) for p in (0, 127, 128, k // 2 + 3, k - 1)})[:m]
    hot = synth.one_hot_rows(k, pos)
    run(backend, "gemm_fp8_block", [backend.Upload(hot), dw, ds, dc], [len(pos), n, k])
    backend.Synchronize()
    got = backend.CopyD2H(dc, dtype=np.float32)[: len(pos) * n].reshape(len(pos), n)
    assert same_bits_zero_sign_free(got, oracle.gemm_fp8_block(hot, codes, scales, len(pos), n, k))
    with pytest.raises(StatusError) as e:   # n and k must be multiples of 128
        run(backend, "gemm_fp8_block", [da, dw, ds, dc], [m, n, k - 64])
    assert e.value.code == StatusCode.InvalidArgument


@pytest.mark.parametrize("k", [512, 17408])
def test_gemm_fp8_one_hot_bit_exact(backend, k):
    g = synth.rng(77)
    n = 50
    codes, scales = synth.fp8_weights(g, n, k)
    pos = [0, 1, 15, 16, 17, 31, 32, 255, k - 1]
    ref = oracle.gemm_fp8(synth.one_hot_rows(k, pos), codes, scales, len(pos), n, k)
    da, dw, ds = backend.Upload(synth.one_hot_rows(k, pos)), backend.Upload(codes), backend.Upload(scales)
    dc = backend.AllocateBuffer(4 * len(pos) * n)
    run(backend, "gemm_fp8", [da, dw, ds, dc], [len(pos), n, k])
    backend.Synchronize()
    assert same_bits_zero_sign_free(backend.CopyD2H(dc, dtype=np.float32).reshape(len(pos), n), ref)


@pytest.mark.parametrize("k", [64, 512, 17408])
def test_gemm_fp8_every_weight_code(backend, k):
    """All 256 E4M3 codes as weights (one per row, the code repeated along the row), a one-hot
    activation and unit row scales: the device's conversion against Fp8E4M3ToFloat, through the
    16-, 32- and 64-weights-a-lane codecs (k selects them); 0x7F and 0xFF are NaN."""
    n = 256
    codes = np.repeat(np.arange(n, dtype=np.uint8), k)
    scales = np.ones(n, np.float32)
    want = np.array([oracle.fp8_e4m3_to_float(c) for c in range(n)], np.float32)
    for m, pos in ((1, [k - 1]), (2, [0, k // 2]), (5, [1, 15, 16, 33, k - 2])):
        x = synth.one_hot_rows(k, pos)
        da, dw, ds = backend.Upload(x), backend.Upload(codes), backend.Upload(scales)
        dc = backend.AllocateBuffer(4 * m * n)
        run(backend, "gemm_fp8", [da, dw, ds, dc], [m, n, k])
        backend.Synchronize()
        got = backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)
        nan = np.isnan(want)
        for r in range(m):
            assert np.array_equal(np.isnan(got[r]), nan)
            assert same_bits_zero_sign_free(got[r][~nan], want[~nan]), (k, m, r)


def test_full_size_config2(backend):
    """BASELINE config 2 at full size: N=17408, K=5120, M in {1, 4, 16}."""
    g = synth.rng(9090)
    n, k = 17408, 5120
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    dw = backend.Upload(w)
    dref = backend.AllocateBuffer(n)
    for m in (1, 4, 16):
        x = synth.activations_bf16_outliers(g, m, k)
        codes, scale = oracle.quantize_fp8_pack(x, m, k)
        dx = backend.Upload(x)
        da8, das = backend.AllocateBuffer(m * k), backend.AllocateBuffer(4 * m)
        out = backend.AllocateBuffer(4 * m * n)
        run(backend, "quantize_fp8_pack_rows", [dx, da8, das], [m, k], grid=(m, 1, 1))
        run(backend, "gemm_mxfp4_wmma", [da8, dw, das, dref, out], [m, n, k, 1, 0], grid=((n + 63) // 64, 1, 1))
        backend.Synchronize()
        assert np.array_equal(backend.CopyD2H(da8).reshape(m, k), codes)
        got = backend.CopyD2H(out, dtype=np.float32).reshape(m, n)
        # every row, all columns: the threaded fp32-activation oracle on the quantize-dequantized rows
        # e4m3(code) * scale, which is what the W4A8 oracle multiplies (row 0 checked bit for bit)
        lut = np.array([oracle.fp8_e4m3_to_float(c) for c in range(256)], np.float32)
        qdq = (lut[codes] * scale.reshape(m, 1)).astype(np.float32)
        ref = oracle.gemm_mxfp4(qdq, w, m, n, k, threads=True)
        assert np.array_equal(ref[:1], oracle.gemm_mxfp4_w4a8(codes[:1], scale[:1], w, 1, n, k))
        print(f"configs[2] W4A8 m={m} 17408x5120: rel_err {rel_err(got, ref):.2e} (floor 0.05 rms), "
              f"{strict_rel_err(got, ref):.2e} (floor 1e-3 rms), max|d|/rms {rms_err(got, ref):.2e}")
        assert rel_err(got, ref) <= (TOL if m <= 1 else 1e-2), (m, rel_err(got, ref))
        assert rms_err(got, ref) <= 5e-4
