"""Rows longer than the register-resident GEMV mapping holds (a row must fit one workgroup there)
take the wave-per-row kernel: any K of the format's granularity works, as in the reference."""
import numpy as np
import pytest

import oracle
from tessera_amd import synth
from util import rel_err, run

pytestmark = pytest.mark.gpu
TOL = 1e-3


def launch(backend, name, bufs, m, n, k, extra=()):
    dc = backend.AllocateBuffer(4 * m * n)
    run(backend, name, [*bufs, dc], [m, n, k, *extra])
    backend.Synchronize()
    return backend.CopyD2H(dc, dtype=np.float32).reshape(m, n)


@pytest.mark.parametrize("m", [1, 3])
def test_q4k_q5k_q6k_long_rows(backend, m):
    g = synth.rng(1200 + m)
    n = 6
    for fmt, gen, ref, k in (("q4k", synth.q4k_weights, oracle.gemm_q4k, 40960),
                             ("q5k", synth.q5k_weights, oracle.gemm_q5k, 49408),
                             ("q6k", synth.q6k_weights, oracle.gemm_q6k, 49408)):
        w = gen(g, n, k)
        a = synth.activations_f32(g, m, k)
        got = launch(backend, f"gemm_{fmt}", [backend.Upload(a), backend.Upload(w)], m, n, k)
        assert rel_err(got, ref(a, w, m, n, k)) < TOL, fmt


@pytest.mark.parametrize("m", [1, 2])
def test_mxfp4_and_fp8_long_rows(backend, m):
    g = synth.rng(1210 + m)
    n = 5
    k = 33024
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    a = synth.activations_f32(g, m, k)
    got = launch(backend, "gemm_mxfp4" if m == 1 else "gemm_mxfp4_rows", [backend.Upload(a), backend.Upload(w)], m, n, k)
    assert rel_err(got, oracle.gemm_mxfp4(a, w, m, n, k)) < TOL
    for k in (32784, 40000):            # a multiple of 16 only, and one beyond the 32-a-lane codec
        codes, scales = synth.fp8_weights(g, n, k)
        a = synth.activations_f32(g, m, k)
        got = launch(backend, "gemm_fp8", [backend.Upload(a), backend.Upload(codes), backend.Upload(scales)], m, n, k)
        assert rel_err(got, oracle.gemm_fp8(a, codes, scales, m, n, k)) < TOL, k
