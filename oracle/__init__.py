"""ctypes front-end of the CPU oracle (``qmm_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
CPU-baseline leg of ``bench.py``.  The product package never imports this module.

All functions take and return numpy arrays; byte buffers are ``uint8``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

Q4K_ELEMS = 256
Q4K_BYTES = 144
Q5K_BYTES = 176
Q6K_BYTES = 210


def build(force: bool = False) -> str:
    """Compile ``qmm_oracle.c`` into ``liboracle.so`` with gcc."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    f32p, u8p, u32p = C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_uint32)
    sz = C.c_size_t
    sig = {
        "orc_fp16_to_float": (C.c_float, [C.c_uint16]),
        "orc_fp32_to_half_bits": (C.c_uint16, [C.c_float]),
        "orc_round_bf16": (None, [f32p, sz]),
        "orc_fp8_e4m3_to_float": (C.c_float, [C.c_uint8]),
        "orc_e8m0_to_float": (C.c_float, [C.c_uint8]),
        "orc_f4e2m1_to_float": (C.c_float, [C.c_uint8]),
        "orc_fp32_to_fp8_e4m3": (C.c_uint8, [C.c_float]),
        "orc_fp32_to_fp8_e4m3_many": (None, [f32p, u8p, sz]),
        "orc_get_scale_min": (None, [sz, u8p, u8p, u8p]),
        "orc_dequantize_q4k": (None, [u8p, f32p]),
        "orc_dequantize_q4k_rows": (None, [u8p, f32p, sz]),
        "orc_quantize_q4k": (None, [f32p, u8p]),
        "orc_quantize_fp8_ref": (C.c_int, [f32p, f32p, sz, sz]),
        "orc_quantize_fp8_pack_ref": (C.c_int, [f32p, u8p, f32p, sz, sz]),
        "orc_gemm_q4k_ref": (C.c_int, [f32p, u8p, f32p, sz, sz, sz]),
        "orc_gemm_q4k_ref_omp": (C.c_int, [f32p, u8p, f32p, sz, sz, sz]),
        "orc_dequantize_q5k": (None, [u8p, f32p]),
        "orc_dequantize_q5k_rows": (None, [u8p, f32p, sz]),
        "orc_gemm_q5k_ref": (C.c_int, [f32p, u8p, f32p, sz, sz, sz, C.c_int]),
        "orc_dequantize_q6k": (None, [u8p, f32p]),
        "orc_dequantize_q6k_rows": (None, [u8p, f32p, sz]),
        "orc_gemm_q6k_ref": (C.c_int, [f32p, u8p, f32p, sz, sz, sz, C.c_int]),
        "orc_gemm_mxfp4_ref": (C.c_int, [f32p, u8p, u8p, f32p, sz, sz, sz]),
        "orc_gemm_mxfp4_ref_omp": (C.c_int, [f32p, u8p, u8p, f32p, sz, sz, sz]),
        "orc_dequantize_mxfp4": (C.c_int, [u8p, f32p, sz, sz]),
        "orc_gemm_fp8_ref": (C.c_int, [f32p, u8p, f32p, f32p, sz, sz, sz]),
        "orc_gemm_fp8_block_ref": (C.c_int, [f32p, u8p, f32p, f32p, sz, sz, sz]),
        "orc_quantize_q8": (C.c_int, [f32p, u8p, f32p, sz, sz]),
        "orc_quantize_q4": (C.c_int, [f32p, u8p, f32p, sz, sz]),
        "orc_attention_quant": (C.c_int, [f32p, u8p, u8p, f32p, f32p, f32p, sz, sz, sz, sz, sz, C.c_uint64, sz, C.c_int]),
        "orc_cast_f32_f16": (None, [f32p, C.POINTER(C.c_uint16), sz]),
        "orc_attention_split": (C.c_int, [f32p, f32p, f32p, f32p, f32p, f32p, sz, sz, sz, sz, sz, C.c_uint64, sz, C.c_int, sz]),
        "orc_attention_combine": (C.c_int, [f32p, f32p, f32p, f32p, sz, sz, sz, sz]),
        "orc_permute_mxfp4_to_wmma": (C.c_int, [u8p, u8p, sz, sz]),
        "orc_permute_q4k_rowgroup": (C.c_int, [u8p, u8p, sz, sz, sz, C.c_int]),
        "orc_rope": (C.c_int, [f32p, sz, sz, sz, sz, C.c_uint64, C.c_double]),
        "orc_mrope": (C.c_int, [f32p, C.POINTER(C.c_uint64), sz, sz, sz, sz, sz, sz, sz, C.c_double]),
        "orc_attention": (C.c_int, [f32p, C.c_void_p, C.c_void_p, f32p, sz, sz, sz, sz, sz, C.c_uint64, sz, C.c_int, C.c_int]),
        "orc_qgate_split": (C.c_int, [f32p, f32p, f32p, sz, sz, sz]),
        "orc_fold_entry": (C.c_uint8, [C.c_uint, C.c_uint]),
        "orc_fold_entry_rne": (C.c_uint8, [C.c_uint, C.c_uint]),
        "orc_fold_mxfp4_to_fp8": (C.c_int, [u8p, u8p, u8p, u8p, sz, sz]),
        "orc_gemm_mxfp4_fp8_ref": (C.c_int, [u8p, f32p, u8p, u8p, f32p, sz, sz, sz]),
        "orc_gemm_mxfp4_w4a8_ref": (C.c_int, [u8p, f32p, u8p, u8p, f32p, sz, sz, sz]),
        "orc_silu_mul": (None, [f32p, f32p, f32p, sz]),
        "orc_rmsnorm": (C.c_int, [f32p, f32p, f32p, sz, sz, C.c_float]),
        "orc_embedding": (C.c_int, [C.c_int, u32p, C.c_void_p, f32p, sz, sz, sz]),
        "orc_moe_gate": (None, [f32p, f32p, sz]),
        "orc_top_k_row": (None, [f32p, sz, sz, u32p, f32p]),
        "orc_moe_expert_forward_q4k": (C.c_int, [f32p, u8p, u8p, u8p, sz, sz, f32p]),
        "orc_moe_experts_forward_q4k": (
            C.c_int, [f32p, u32p, f32p, sz, u8p, sz, u8p, sz, u8p, sz, sz, sz, f32p]),
        "orc_moe_batch_forward_q4k": (
            C.c_int, [f32p, u32p, f32p, sz, sz, u8p, sz, u8p, sz, u8p, sz, sz, sz, f32p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = _load()


class OracleError(RuntimeError):
    """A routine returned a non-zero tessera StatusCode."""

    def __init__(self, code: int):
        super().__init__(f"oracle status {code}")
        self.code = code


def _check(code: int) -> None:
    if code != 0:
        raise OracleError(code)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def _p(a: np.ndarray, ty):
    return a.ctypes.data_as(C.POINTER(ty))


# ---- scalar codecs -------------------------------------------------------
def fp16_to_float(bits: int) -> float:
    return _lib.orc_fp16_to_float(bits)


def fp32_to_half_bits(v: float) -> int:
    return _lib.orc_fp32_to_half_bits(v)


def fp8_e4m3_to_float(code: int) -> float:
    return _lib.orc_fp8_e4m3_to_float(code)


def e8m0_to_float(code: int) -> float:
    return _lib.orc_e8m0_to_float(code)


def f4e2m1_to_float(nib: int) -> float:
    return _lib.orc_f4e2m1_to_float(nib)


def fp32_to_fp8_e4m3(v: float) -> int:
    return _lib.orc_fp32_to_fp8_e4m3(v)


def fold_entry(d: int, mag: int) -> int:
    return _lib.orc_fold_entry(d, mag)


def fold_entry_rne(d: int, mag: int) -> int:
    return _lib.orc_fold_entry_rne(d, mag)


def round_bf16(x) -> np.ndarray:
    out = _f32(x).copy()
    _lib.orc_round_bf16(_p(out, C.c_float), out.size)
    return out


def get_scale_min(j: int, scales12) -> tuple[int, int]:
    s = _u8(scales12)
    assert s.size == 12
    sc, mn = C.c_uint8(), C.c_uint8()
    _lib.orc_get_scale_min(j, _p(s, C.c_uint8), C.byref(sc), C.byref(mn))
    return sc.value, mn.value


# ---- Q4_K ----------------------------------------------------------------
def dequantize_q4k(w) -> np.ndarray:
    """Any whole number of 144-byte super-blocks -> fp32, 256 values per block."""
    w = _u8(w).reshape(-1)
    assert w.size % Q4K_BYTES == 0
    nb = w.size // Q4K_BYTES
    out = np.empty(nb * Q4K_ELEMS, dtype=np.float32)
    _lib.orc_dequantize_q4k_rows(_p(w, C.c_uint8), _p(out, C.c_float), nb)
    return out


def quantize_q4k(x) -> np.ndarray:
    x = _f32(x).reshape(-1)
    assert x.size % Q4K_ELEMS == 0
    nb = x.size // Q4K_ELEMS
    out = np.zeros(nb * Q4K_BYTES, dtype=np.uint8)
    for b in range(nb):
        xb = x[b * Q4K_ELEMS:(b + 1) * Q4K_ELEMS]
        ob = out[b * Q4K_BYTES:(b + 1) * Q4K_BYTES]
        _lib.orc_quantize_q4k(_p(xb, C.c_float), _p(ob, C.c_uint8))
    return out


def gemm_q4k(a, w, m: int, n: int, k: int, threads: bool = False) -> np.ndarray:
    a, w = _f32(a), _u8(w)
    if k % Q4K_ELEMS == 0 and k and n and m:
        assert a.size == m * k and w.size == n * (k // Q4K_ELEMS) * Q4K_BYTES
    c = np.empty((m, n), dtype=np.float32)
    fn = _lib.orc_gemm_q4k_ref_omp if threads else _lib.orc_gemm_q4k_ref
    _check(fn(_p(a, C.c_float), _p(w, C.c_uint8), _p(c, C.c_float), m, n, k))
    return c


# ---- Q5_K ----------------------------------------------------------------
def dequantize_q5k(w) -> np.ndarray:
    """Any whole number of 176-byte super-blocks -> fp32, 256 values per block."""
    w = _u8(w).reshape(-1)
    assert w.size % Q5K_BYTES == 0
    nb = w.size // Q5K_BYTES
    out = np.empty(nb * Q4K_ELEMS, dtype=np.float32)
    _lib.orc_dequantize_q5k_rows(_p(w, C.c_uint8), _p(out, C.c_float), nb)
    return out


def gemm_q5k(a, w, m: int, n: int, k: int, threads: bool = False) -> np.ndarray:
    a, w = _f32(a), _u8(w)
    if k % Q4K_ELEMS == 0 and k and n and m:
        assert a.size == m * k and w.size == n * (k // Q4K_ELEMS) * Q5K_BYTES
    c = np.empty((m, n), dtype=np.float32)
    _check(_lib.orc_gemm_q5k_ref(_p(a, C.c_float), _p(w, C.c_uint8), _p(c, C.c_float), m, n, k, int(threads)))
    return c


# ---- Q6_K ----------------------------------------------------------------
def dequantize_q6k(w) -> np.ndarray:
    """Any whole number of 210-byte super-blocks -> fp32, 256 values per block."""
    w = _u8(w).reshape(-1)
    assert w.size % Q6K_BYTES == 0
    nb = w.size // Q6K_BYTES
    out = np.empty(nb * Q4K_ELEMS, dtype=np.float32)
    _lib.orc_dequantize_q6k_rows(_p(w, C.c_uint8), _p(out, C.c_float), nb)
    return out


def gemm_q6k(a, w, m: int, n: int, k: int, threads: bool = False) -> np.ndarray:
    a, w = _f32(a), _u8(w)
    if k % Q4K_ELEMS == 0 and k and n and m:
        assert a.size == m * k and w.size == n * (k // Q4K_ELEMS) * Q6K_BYTES
    c = np.empty((m, n), dtype=np.float32)
    _check(_lib.orc_gemm_q6k_ref(_p(a, C.c_float), _p(w, C.c_uint8), _p(c, C.c_float), m, n, k, int(threads)))
    return c


# ---- MXFP4 / FP8 ----------------------------------------------------------
def split_mxfp4(packed, n: int, k: int) -> tuple[np.ndarray, np.ndarray]:
    """Packed device layout -> (blob n*k/2 bytes, scales n*k/32 bytes)."""
    packed = _u8(packed).reshape(-1)
    assert packed.size == n * k // 2 + n * k // 32
    return packed[: n * k // 2], packed[n * k // 2:]


def gemm_mxfp4(a, packed, m: int, n: int, k: int, threads: bool = False) -> np.ndarray:
    a = _f32(a)
    blob, s = split_mxfp4(packed, n, k)
    c = np.empty((m, n), dtype=np.float32)
    fn = _lib.orc_gemm_mxfp4_ref_omp if threads else _lib.orc_gemm_mxfp4_ref
    _check(fn(_p(a, C.c_float), _p(blob, C.c_uint8), _p(s, C.c_uint8), _p(c, C.c_float), m, n, k))
    return c


def dequantize_mxfp4(packed, n: int, k: int) -> np.ndarray:
    packed = _u8(packed).reshape(-1)
    out = np.empty((n, k), dtype=np.float32)
    _check(_lib.orc_dequantize_mxfp4(_p(packed, C.c_uint8), _p(out, C.c_float), n, k))
    return out


def gemm_fp8(a, w, s, m: int, n: int, k: int) -> np.ndarray:
    a, w, s = _f32(a), _u8(w), _f32(s)
    assert a.size == m * k and w.size == n * k and s.size == n
    c = np.empty((m, n), dtype=np.float32)
    _check(_lib.orc_gemm_fp8_ref(_p(a, C.c_float), _p(w, C.c_uint8), _p(s, C.c_float),
                                 _p(c, C.c_float), m, n, k))
    return c


def gemm_fp8_block(a, w, s, m: int, n: int, k: int) -> np.ndarray:
    """GemmFp8BlockRef: one scale per 128 x 128 block of W (s is (n/128) x (k/128))."""
    a, w, s = _f32(a), _u8(w), _f32(s)
    assert a.size == m * k and w.size == n * k
    if n % 128 == 0 and k % 128 == 0:
        assert s.size == (n // 128) * (k // 128)
    c = np.empty((m, n), dtype=np.float32)
    _check(_lib.orc_gemm_fp8_block_ref(_p(a, C.c_float), _p(w, C.c_uint8), _p(s, C.c_float),
                                       _p(c, C.c_float), m, n, k))
    return c


def quantize_fp8(data, rows: int, cols: int) -> tuple[np.ndarray, np.ndarray]:
    """Quantize-dequantize; returns (qdq data, scales)."""
    out = _f32(data).copy().reshape(rows, cols)
    scale = np.empty(rows, dtype=np.float32)
    _check(_lib.orc_quantize_fp8_ref(_p(out, C.c_float), _p(scale, C.c_float), rows, cols))
    return out, scale


def fp32_to_fp8_e4m3_many(v) -> np.ndarray:
    """The encoder of fp32_to_fp8_e4m3 over an array (threaded)."""
    v = _f32(v).reshape(-1)
    out = np.empty(v.size, dtype=np.uint8)
    _lib.orc_fp32_to_fp8_e4m3_many(_p(v, C.c_float), _p(out, C.c_uint8), v.size)
    return out


def quantize_fp8_pack(data, rows: int, cols: int) -> tuple[np.ndarray, np.ndarray]:
    """Returns (e4m3 codes rows x cols, scales)."""
    src = _f32(data).reshape(rows, cols)
    codes = np.empty((rows, cols), dtype=np.uint8)
    scale = np.empty(rows, dtype=np.float32)
    _check(_lib.orc_quantize_fp8_pack_ref(_p(src, C.c_float), _p(codes, C.c_uint8),
                                          _p(scale, C.c_float), rows, cols))
    return codes, scale


def permute_mxfp4_to_wmma(packed, n: int, k: int) -> np.ndarray:
    """Packed MXFP4 (nibble bytes then scales) with the nibble bytes in the 16-row fragment order;
    the scales stay where they are."""
    blob, s = split_mxfp4(packed, n, k)
    out = np.empty_like(blob)
    _check(_lib.orc_permute_mxfp4_to_wmma(_p(blob, C.c_uint8), _p(out, C.c_uint8), n, k))
    return np.concatenate([out.reshape(-1), s.reshape(-1)])


def permute_q4k_rowgroup(w, n: int, k: int, rows_per_group: int = 32, inverse: bool = False) -> np.ndarray:
    """A Q4_K matrix between GGUF order and the row-group order of the gfx950 int8 decode kernel
    (same byte count; `inverse` goes back)."""
    w = _u8(w)
    out = np.empty_like(w)
    _check(_lib.orc_permute_q4k_rowgroup(_p(w, C.c_uint8), _p(out, C.c_uint8), n, k, rows_per_group, int(inverse)))
    return out


def fold_mxfp4_to_fp8(packed, n: int, k: int) -> tuple[np.ndarray, np.ndarray]:
    blob, s = split_mxfp4(packed, n, k)
    out = np.empty((n, k), dtype=np.uint8)
    wref = np.empty(n, dtype=np.uint8)
    _check(_lib.orc_fold_mxfp4_to_fp8(_p(blob, C.c_uint8), _p(s, C.c_uint8), _p(out, C.c_uint8),
                                      _p(wref, C.c_uint8), n, k))
    return out, wref


def gemm_mxfp4_fp8(a8, a_scale, w8, wref, m: int, n: int, k: int) -> np.ndarray:
    a8, a_scale, w8, wref = _u8(a8), _f32(a_scale), _u8(w8), _u8(wref)
    c = np.empty((m, n), dtype=np.float32)
    _check(_lib.orc_gemm_mxfp4_fp8_ref(_p(a8, C.c_uint8), _p(a_scale, C.c_float),
                                       _p(w8, C.c_uint8), _p(wref, C.c_uint8),
                                       _p(c, C.c_float), m, n, k))
    return c


def gemm_mxfp4_w4a8(a8, a_scale, packed, m: int, n: int, k: int) -> np.ndarray:
    a8, a_scale = _u8(a8), _f32(a_scale)
    blob, s = split_mxfp4(packed, n, k)
    c = np.empty((m, n), dtype=np.float32)
    _check(_lib.orc_gemm_mxfp4_w4a8_ref(_p(a8, C.c_uint8), _p(a_scale, C.c_float),
                                        _p(blob, C.c_uint8), _p(s, C.c_uint8),
                                        _p(c, C.c_float), m, n, k))
    return c


# ---- dense feed-forward pieces ------------------------------------------------
def silu_mul(g, u) -> np.ndarray:
    g, u = _f32(g).reshape(-1), _f32(u).reshape(-1)
    out = np.empty_like(g)
    _lib.orc_silu_mul(_p(g, C.c_float), _p(u, C.c_float), _p(out, C.c_float), g.size)
    return out


def rmsnorm(x, w, rows: int, cols: int, eps: float) -> np.ndarray:
    x, w = _f32(x).reshape(-1), _f32(w).reshape(-1)
    y = np.empty_like(x)
    _check(_lib.orc_rmsnorm(_p(x, C.c_float), _p(w, C.c_float), _p(y, C.c_float), rows, cols, eps))
    return y.reshape(rows, cols)


def embedding(kind: str, ids, table, rows: int, cols: int, vocab: int) -> np.ndarray:
    """kind: "f32", "bf16" (uint16 table) or "q4k" (uint8 blocks)."""
    ids = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
    table = np.ascontiguousarray(table)
    out = np.empty((rows, cols), dtype=np.float32)
    code = {"f32": 0, "bf16": 1, "q4k": 2}[kind]
    _check(_lib.orc_embedding(code, _p(ids, C.c_uint32), table.ctypes.data_as(C.c_void_p), _p(out, C.c_float),
                              rows, cols, vocab))
    return out


def rope(x, rows: int, heads: int, head_dim: int, rope_dim: int, pos_base: int, theta: float) -> np.ndarray:
    io = _f32(x).reshape(-1).copy()
    _check(_lib.orc_rope(_p(io, C.c_float), rows, heads, head_dim, rope_dim, pos_base, theta))
    return io.reshape(rows, heads, head_dim)


def mrope(x, pos, rows: int, heads: int, head_dim: int, rope_dim: int, sec_t: int, sec_h: int, sec_w: int,
          theta: float) -> np.ndarray:
    io = _f32(x).reshape(-1).copy()
    pos = np.ascontiguousarray(pos, dtype=np.uint64).reshape(-1)
    _check(_lib.orc_mrope(_p(io, C.c_float), _p(pos, C.c_uint64), rows, heads, head_dim, rope_dim, sec_t, sec_h, sec_w, theta))
    return io.reshape(rows, heads, head_dim)


def attention(q, k, v, m: int, n: int, heads: int, kv_heads: int, head_dim: int, q_base: int = 0, window: int = 0,
              kv_f16: bool = False, causal: bool = True) -> np.ndarray:
    """k, v: fp32 arrays, or float16 arrays when kv_f16."""
    q = _f32(q).reshape(-1)
    dt = np.float16 if kv_f16 else np.float32
    k, v = np.ascontiguousarray(k, dtype=dt).reshape(-1), np.ascontiguousarray(v, dtype=dt).reshape(-1)
    out = np.empty(m * heads * head_dim, dtype=np.float32)
    _check(_lib.orc_attention(_p(q, C.c_float), k.ctypes.data_as(C.c_void_p), v.ctypes.data_as(C.c_void_p),
                              _p(out, C.c_float), m, n, heads, kv_heads, head_dim, q_base, window, int(kv_f16), int(causal)))
    return out.reshape(m, heads * head_dim)


def quantize_kv(data, rows: int, cols: int, bits: int) -> tuple[np.ndarray, np.ndarray]:
    """QuantizeQ8Ref (bits = 8: rows x cols bytes) / QuantizeQ4Ref (bits = 4: rows x cols/2 bytes);
    returns (codes, one scale per row)."""
    data = _f32(data).reshape(-1)
    assert data.size == rows * cols and bits in (4, 8)
    out = np.empty(rows * cols * bits // 8, dtype=np.uint8)
    scale = np.empty(rows, dtype=np.float32)
    fn = _lib.orc_quantize_q8 if bits == 8 else _lib.orc_quantize_q4
    _check(fn(_p(data, C.c_float), _p(out, C.c_uint8), _p(scale, C.c_float), rows, cols))
    return out, scale


KV_KINDS = {"q8": 0, "q4": 1, "fp8": 2}


def attention_quant(q, k, v, k_scale, v_scale, m: int, n: int, heads: int, kv_heads: int, head_dim: int, kind: str,
                    q_base: int = 0, window: int = 0) -> np.ndarray:
    """AttentionQ8Ref / AttentionQ4Ref / AttentionFp8Ref: k, v hold codes, one scale per key row."""
    q, k, v, ks, vs = _f32(q).reshape(-1), _u8(k), _u8(v), _f32(k_scale), _f32(v_scale)
    out = np.empty(m * heads * head_dim, dtype=np.float32)
    _check(_lib.orc_attention_quant(_p(q, C.c_float), _p(k, C.c_uint8), _p(v, C.c_uint8), _p(ks, C.c_float),
                                    _p(vs, C.c_float), _p(out, C.c_float), m, n, heads, kv_heads, head_dim, q_base, window,
                                    KV_KINDS[kind]))
    return out.reshape(m, heads * head_dim)


def attention_split(q, k, v, m: int, n: int, heads: int, kv_heads: int, head_dim: int, split: int, q_base: int = 0,
                    window: int = 0, causal: bool = True) -> tuple[np.ndarray, np.ndarray, np.ndarray]:
    """Flash-decoding partials (pacc m*heads*split x head_dim, pmax, psum) over fp32 keys and values."""
    q, k, v = _f32(q).reshape(-1), _f32(k).reshape(-1), _f32(v).reshape(-1)
    parts = m * heads * split
    pacc = np.empty(parts * head_dim, dtype=np.float32)
    pmax, psum = np.empty(parts, dtype=np.float32), np.empty(parts, dtype=np.float32)
    _check(_lib.orc_attention_split(_p(q, C.c_float), _p(k, C.c_float), _p(v, C.c_float), _p(pacc, C.c_float),
                                    _p(pmax, C.c_float), _p(psum, C.c_float), m, n, heads, kv_heads, head_dim, q_base, window,
                                    int(causal), split))
    return pacc.reshape(parts, head_dim), pmax, psum


def attention_combine(pacc, pmax, psum, m: int, heads: int, head_dim: int, split: int) -> np.ndarray:
    pacc, pmax, psum = _f32(pacc).reshape(-1), _f32(pmax), _f32(psum)
    out = np.empty(m * heads * head_dim, dtype=np.float32)
    _check(_lib.orc_attention_combine(_p(pacc, C.c_float), _p(pmax, C.c_float), _p(psum, C.c_float), _p(out, C.c_float), m,
                                      heads, head_dim, split))
    return out.reshape(m, heads * head_dim)


def dequant_kv(codes, scale, n: int, width: int, kind: str) -> np.ndarray:
    """code * scale[key row] of a quantized cache as fp32 (n x width): the element decode of
    AttentionQ8Ref / AttentionQ4Ref / AttentionFp8Ref, for tests that feed the fp32 routines."""
    codes, scale = _u8(codes), _f32(scale)
    if kind == "q8":
        vals = codes.view(np.int8).astype(np.float32)
    elif kind == "q4":
        nib = np.stack([codes & 0xF, codes >> 4], axis=-1).reshape(-1).astype(np.int32)
        vals = np.where(nib >= 8, nib - 16, nib).astype(np.float32)
    else:
        vals = np.array([fp8_e4m3_to_float(int(c)) for c in range(256)], np.float32)[codes]
    return (vals.reshape(n, width) * scale[:, None]).astype(np.float32)


def cast_f32_f16(data) -> np.ndarray:
    """The "cast_f32_f16" built-in's conversion (significand cut toward zero); returns uint16 bits."""
    data = _f32(data).reshape(-1)
    out = np.empty(data.size, dtype=np.uint16)
    _lib.orc_cast_f32_f16(_p(data, C.c_float), out.ctypes.data_as(C.POINTER(C.c_uint16)), data.size)
    return out


def qgate_split(fused, heads: int, head_dim: int, rows: int) -> tuple[np.ndarray, np.ndarray]:
    fused = _f32(fused).reshape(-1)
    q = np.empty(rows * heads * head_dim, dtype=np.float32)
    g = np.empty_like(q)
    _check(_lib.orc_qgate_split(_p(fused, C.c_float), _p(q, C.c_float), _p(g, C.c_float), heads, head_dim, rows))
    return q, g


def ffn_gate_up_silu_q4k(x, gate, up, m: int, n: int, k: int, threads: bool = False) -> np.ndarray:
    """silu(x gate^T) * (x up^T): the two Q4_K products and silu_mul, composed as the
    reference's dense feed-forward block does (src/models/qwen3_5/trunk.cpp:294-304)."""
    g = gemm_q4k(x, gate, m, n, k, threads)
    u = gemm_q4k(x, up, m, n, k, threads)
    return silu_mul(g, u).reshape(m, n)


# ---- MoE -------------------------------------------------------------------
def moe_gate(vals) -> np.ndarray:
    v = _f32(vals).reshape(-1)
    out = np.empty_like(v)
    _lib.orc_moe_gate(_p(v, C.c_float), _p(out, C.c_float), v.size)
    return out


def top_k_row(logits, top_k: int) -> tuple[np.ndarray, np.ndarray]:
    lg = _f32(logits).reshape(-1)
    ids = np.empty(top_k, dtype=np.uint32)
    vals = np.empty(top_k, dtype=np.float32)
    _lib.orc_top_k_row(_p(lg, C.c_float), lg.size, top_k, _p(ids, C.c_uint32), _p(vals, C.c_float))
    return ids, vals


def moe_batch_forward_q4k(x, ids, wts, gate, up, down, hidden: int, inter: int) -> np.ndarray:
    """Routed-expert sum per token.  gate/up: [E][inter][hidden/256] blocks; down:
    [E][hidden][inter/256] blocks; ids/wts: rows x top_k."""
    x = _f32(x).reshape(-1, hidden)
    rows = x.shape[0]
    ids = np.ascontiguousarray(ids, dtype=np.uint32).reshape(rows, -1)
    wts = _f32(wts).reshape(rows, -1)
    top_k = ids.shape[1]
    gate, up, down = _u8(gate).reshape(-1), _u8(up).reshape(-1), _u8(down).reshape(-1)
    gs = inter * (hidden // Q4K_ELEMS) * Q4K_BYTES
    ds = hidden * (inter // Q4K_ELEMS) * Q4K_BYTES
    out = np.empty((rows, hidden), dtype=np.float32)
    _check(_lib.orc_moe_batch_forward_q4k(
        _p(x, C.c_float), _p(ids, C.c_uint32), _p(wts, C.c_float), rows, top_k,
        _p(gate, C.c_uint8), gs, _p(up, C.c_uint8), gs, _p(down, C.c_uint8), ds,
        hidden, inter, _p(out, C.c_float)))
    return out
