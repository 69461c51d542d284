"""GPU parity of the dense feed-forward ids: "silu_mul", "round_bf16" and the fused
"ffn_gate_up_silu_q4k" (gate and up products with the activation applied in the same launch)."""
import numpy as np
import pytest

import oracle
from tessera_amd import StatusCode, StatusError, synth
from util import rel_err, rms_err, run, same_bits

pytestmark = pytest.mark.gpu
TOL = 1e-3   # the GEMV's bound on each product; silu is 1-Lipschitz-ish, so the same bound holds after it


def test_round_bf16_bit_exact(backend):
    g = synth.rng(700)
    x = np.concatenate([g.standard_normal(100003), g.standard_normal(1000) * 1e-30, g.standard_normal(1000) * 1e30,
                        np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, 0.0, -0.0, np.inf, -np.inf])]).astype(np.float32)
    d = backend.Upload(x)
    run(backend, "round_bf16", [d], [x.size], grid=((x.size + 255) // 256, 1, 1))
    backend.Synchronize()
    assert same_bits(backend.CopyD2H(d, dtype=np.float32), oracle.round_bf16(x))


def test_silu_mul_matches_oracle(backend):
    g = synth.rng(701)
    n = 70001
    a = (g.standard_normal(n) * 6).astype(np.float32)
    a[:6] = [0.0, -0.0, 90.0, -90.0, 104.0, -104.0]
    u = g.standard_normal(n).astype(np.float32)
    da, du, do = backend.Upload(a), backend.Upload(u), backend.AllocateBuffer(4 * n)
    run(backend, "silu_mul", [da, du, do], [n], grid=((n + 255) // 256, 1, 1))
    backend.Synchronize()
    got, want = backend.CopyD2H(do, dtype=np.float32), oracle.silu_mul(a, u)
    # device expf and libm expf may differ in the last place: a few ulp of the result
    assert np.all(np.abs(got.astype(np.float64) - want) <= 4 * np.spacing(np.abs(want)) + 1e-36)
    # in place over the gate buffer
    run(backend, "silu_mul", [da, du, da], [n], grid=((n + 255) // 256, 1, 1))
    backend.Synchronize()
    assert same_bits(backend.CopyD2H(da, dtype=np.float32), got)


def ffn(backend, x, gate, up, m, n, k):
    dx, dg, du = backend.Upload(x), backend.Upload(gate), backend.Upload(up)
    do = backend.AllocateBuffer(4 * m * n)
    run(backend, "ffn_gate_up_silu_q4k", [dx, dg, du, do], [m, n, k], grid=((m * n + 7) // 8, 1, 1))
    backend.Synchronize()
    return backend.CopyD2H(do, dtype=np.float32).reshape(m, n)


# one row: the fused launch for 4096 <= k <= 24576 (even and odd row counts, ragged last group,
# a row count below one group), the composed path for the other k
ONE_ROW = [(512, 4096), (1027, 5120), (3, 5120), (1, 4096), (130, 8192), (67, 17408), (40, 24576),
           (96, 2048), (33, 256), (9, 32768)]


@pytest.mark.parametrize("n,k", ONE_ROW)
def test_one_row_matches_oracle(backend, n, k):
    g = synth.rng(710 + n + k)
    gate, up = synth.q4k_weights(g, n, k), synth.q4k_weights(g, n, k)
    x = synth.activations_f32(g, 1, k)
    got = ffn(backend, x, gate, up, 1, n, k)
    want = oracle.ffn_gate_up_silu_q4k(x, gate, up, 1, n, k)
    assert rel_err(got, want) < TOL


@pytest.mark.parametrize("m,n,k", [(2, 300, 5120), (5, 128, 4096), (16, 64, 2048), (17, 96, 1024), (40, 256, 512),
                                   (6, 4100, 4096), (12, 4100, 4096), (3, 2052, 8192)])   # the last three: the one-pass few-row kernel
def test_several_rows_match_oracle(backend, m, n, k):
    g = synth.rng(730 + m)
    gate, up = synth.q4k_weights(g, n, k), synth.q4k_weights(g, n, k)
    x = synth.activations_f32(g, m, k)
    got = ffn(backend, x, gate, up, m, n, k)
    want = oracle.ffn_gate_up_silu_q4k(x, gate, up, m, n, k)
    if m < 17:
        assert rel_err(got, want) < TOL
    else:
        # From 17 rows on the two products come from the fp16 MFMA GEMM, bounded by
        # max|dg| <= 4e-3 rms(g) (tests/test_gpu_gemm_q4k.py).  With |silu'| <= 1.1,
        # |d out| <= 1.1 |u| |dg| + |silu(g)| |du| <= (1.1 * 4 + 4) * 4e-3 rms(g) rms(u) for
        # operands within 4 rms, and rms(out) is about 0.7 rms(g) rms(u): 5e-2 of rms(out).
        assert rms_err(got, want) < 5e-2
    # whatever the regime, the id is exactly the library's own two products and silu_mul
    dx, dg, du = backend.Upload(x), backend.Upload(gate), backend.Upload(up)
    og, ou = backend.AllocateBuffer(4 * m * n), backend.AllocateBuffer(4 * m * n)
    run(backend, "gemm_q4k", [dx, dg, og], [m, n, k])
    run(backend, "gemm_q4k", [dx, du, ou], [m, n, k])
    run(backend, "silu_mul", [og, ou, og], [m * n])
    backend.Synchronize()
    assert same_bits(got.reshape(-1), backend.CopyD2H(og, dtype=np.float32))


def test_fused_equals_the_three_launches(backend):
    """The fused id against the library's own two GEMVs and silu_mul: the same fp32 dot products,
    with a row's chunks split over the wavefronts at other places (its slot row differs), so the
    results agree to summation-order noise, far inside the bound against the oracle."""
    g = synth.rng(750)
    n, k = 2050, 5120
    gate, up = synth.q4k_weights(g, n, k), synth.q4k_weights(g, n, k)
    x = synth.activations_f32(g, 1, k)
    dx, dg, du = backend.Upload(x), backend.Upload(gate), backend.Upload(up)
    og, ou = backend.AllocateBuffer(4 * n), backend.AllocateBuffer(4 * n)
    run(backend, "gemm_q4k", [dx, dg, og], [1, n, k])
    run(backend, "gemm_q4k", [dx, du, ou], [1, n, k])
    run(backend, "silu_mul", [og, ou, og], [n])
    backend.Synchronize()
    three = backend.CopyD2H(og, dtype=np.float32)
    assert rms_err(ffn(backend, x, gate, up, 1, n, k).reshape(-1), three) < 2e-5


def test_full_size_gate_up(backend):
    g = synth.rng(760)
    n, k = 17408, 5120
    gate, up = synth.q4k_weights(g, n, k), synth.q4k_weights(g, n, k)
    x = synth.activations_f32(g, 1, k)
    got = ffn(backend, x, gate, up, 1, n, k)
    want = oracle.ffn_gate_up_silu_q4k(x, gate, up, 1, n, k, threads=True)
    assert rel_err(got, want) < TOL


def test_argument_errors(backend):
    g = synth.rng(770)
    n, k = 64, 4096
    w = synth.q4k_weights(g, n, k)
    dx, dw = backend.Upload(synth.activations_f32(g, 1, k)), backend.Upload(w)
    out = backend.AllocateBuffer(4 * n)
    small = backend.AllocateBuffer(4 * n - 4)
    for bufs, sc in [([dx, dw, dw, small], [1, n, k]), ([dx, dw, dw, out], [1, n, k + 1]), ([dx, dw, out], [1, n, k]),
                     ([dx, dw, dw, out], [0, n, k])]:
        with pytest.raises(StatusError) as e:
            run(backend, "ffn_gate_up_silu_q4k", bufs, sc)
        assert e.value.code == StatusCode.InvalidArgument
    with pytest.raises(StatusError):
        run(backend, "silu_mul", [dx, dx, small], [n])
    with pytest.raises(StatusError):
        run(backend, "round_bf16", [small], [n])


def test_add_and_fill_bit_exact(backend):
    g = synth.rng(780)
    n = 100003
    a, b = g.standard_normal(n).astype(np.float32), (g.standard_normal(n) * 1e3).astype(np.float32)
    da, db, do = backend.Upload(a), backend.Upload(b), backend.AllocateBuffer(4 * n)
    run(backend, "add", [da, db, do], [n], grid=((n + 255) // 256, 1, 1))
    backend.Synchronize()
    assert same_bits(backend.CopyD2H(do, dtype=np.float32), a + b)
    run(backend, "fill", [do], [0xFFFFFFFF, n - 3], grid=((n + 255) // 256, 1, 1))   # value -1, all but the last 3
    backend.Synchronize()
    got = backend.CopyD2H(do, dtype=np.int32)
    assert np.all(got[:n - 3] == -1) and np.array_equal(got[n - 3:].view(np.float32), (a + b)[n - 3:])


@pytest.mark.parametrize("rows,cols", [(1, 5120), (7, 2048), (3, 100), (2, 17408), (16, 1)])
def test_rmsnorm_matches_oracle(backend, rows, cols):
    g = synth.rng(790 + cols)
    x = (g.standard_normal((rows, cols)) * 2).astype(np.float32)
    w = (1 + 0.1 * g.standard_normal(cols)).astype(np.float32)
    eps = np.float32(1e-6)
    dx, dw, dy = backend.Upload(x), backend.Upload(w), backend.AllocateBuffer(4 * rows * cols)
    run(backend, "rmsnorm", [dx, dw, dy], [rows, cols, int(eps.view(np.uint32))], grid=((rows * cols + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(dy, dtype=np.float32).reshape(rows, cols)
    want = oracle.rmsnorm(x, w, rows, cols, float(eps))
    # the sum of squares is added in another order than the oracle's sequential chain: the gain
    # differs by about sqrt(cols) * 2^-24 relative, and every output with it
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-12)) < 2e-5


@pytest.mark.parametrize("kind", ["f32", "bf16", "q4k"])
def test_embedding_bit_exact(backend, kind):
    g = synth.rng(800)
    vocab, cols = 301, 1024
    ids = np.concatenate([g.integers(0, vocab, 40), [vocab, 2 ** 32 - 1, 0, vocab - 1]]).astype(np.uint32)
    if kind == "f32":
        table = g.standard_normal((vocab, cols)).astype(np.float32)
    elif kind == "bf16":
        table = (g.standard_normal((vocab, cols)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    else:
        table = synth.q4k_weights(g, vocab, cols)
    di, dt = backend.Upload(ids), backend.Upload(table)
    do = backend.AllocateBuffer(4 * ids.size * cols)
    run(backend, f"embedding_{kind}", [di, dt, do], [ids.size, cols, vocab], grid=((ids.size * cols + 255) // 256, 1, 1))
    backend.Synchronize()
    got = backend.CopyD2H(do, dtype=np.float32).reshape(ids.size, cols)
    assert same_bits(got, oracle.embedding(kind, ids, table, ids.size, cols, vocab))
    if kind == "q4k":
        with pytest.raises(StatusError):
            run(backend, "embedding_q4k", [di, dt, do], [ids.size, cols - 1, vocab])
