"""qmm_workspace_bytes against what the launches really take: for every id that can need library
scratch and for row counts on both sides of each regime switch, a caller-owned workspace of exactly the
reported size must be accepted (and one that is a block shorter refused when the size is not zero), and
the result must equal the launch on the library's own workspace bit for bit."""
import numpy as np
import pytest
import torch

from tessera_amd import StatusCode, StatusError, synth
from util import run

pytestmark = pytest.mark.gpu


def outputs_with_exact_workspace(backend, name, scalars, make_buffers, out_index, tight=True):
    """Runs the launch on the library's workspace, then on a caller's of exactly the reported size;
    returns both outputs and the size.  `tight`: the reported size is what the launch takes, not an
    upper bound, so a block less must be refused."""
    kern = backend.LoadKernel(name)
    need = backend.WorkspaceBytes(kern, scalars)
    backend.SetWorkspace(None)
    bufs = make_buffers()
    run(backend, name, bufs, scalars)
    backend.Synchronize()
    want = backend.CopyD2H(bufs[out_index], dtype=np.float32)
    # the caller's block: exactly `need` bytes (one 256-byte block when nothing is needed: a launch that
    # wanted more than it reported would then be refused)
    size = max(need, 256)
    ws = torch.empty(size, dtype=torch.uint8, device="cuda")
    try:
        backend.SetWorkspace(backend.WrapBuffer(ws.data_ptr(), size))
        bufs = make_buffers()
        run(backend, name, bufs, scalars)
        backend.Synchronize()
        got = backend.CopyD2H(bufs[out_index], dtype=np.float32)
        if tight and need > 256:
            backend.SetWorkspace(backend.WrapBuffer(ws.data_ptr(), need - 256))
            with pytest.raises(StatusError) as e:
                run(backend, name, make_buffers(), scalars)
            assert e.value.code == StatusCode.InvalidArgument
    finally:
        backend.SetWorkspace(None)
        backend.Synchronize()
    return want, got, need


@pytest.mark.parametrize("name,extra", [("gemm_q4k", ()), ("gemm_q4k_batched", ()), ("gemm_q4k_wmma", ()),
                                        ("gemm_q4k_vec", (1,)), ("gemm_q4k_batched", (0,)), ("gemm_q4k_batched", (32,)),
                                        ("gemm_q5k_batched", ()), ("gemm_q6k", ()), ("gemm_q6k_wmma", ())])
@pytest.mark.parametrize("m", [1, 2, 5, 16, 17, 40, 63, 64, 100])
def test_block_format_gemm_ids(backend, name, extra, m):
    if name == "gemm_q4k_vec" and m > 1:
        pytest.skip("the single-row id")
    g = synth.rng(8100 + m)
    n, k = 520, 1024
    fmt = name.split("_")[1]
    w = {"q4k": synth.q4k_weights, "q5k": synth.q5k_weights, "q6k": synth.q6k_weights}[fmt](g, n, k)
    layout = extra[0] if name == "gemm_q4k_batched" and extra else 0
    if layout:
        dw, dout = backend.Upload(w), backend.AllocateBuffer(w.size)
        run(backend, "permute_q4k_rowgroup", [dw, dout], [n, k, layout, 0])
        backend.Synchronize()
        w = backend.CopyD2H(dout, dtype=np.uint8)
    a = synth.activations_bf16(g, m, k)
    make = lambda: [backend.Upload(a), backend.Upload(w), backend.AllocateBuffer(4 * m * n)]
    want, got, need = outputs_with_exact_workspace(backend, name, [m, n, k, *extra], make, 2)
    assert np.array_equal(want, got), (name, m, need)


@pytest.mark.parametrize("m", [1, 2, 16, 17, 63, 64, 130])
def test_fused_gate_up(backend, m):
    g = synth.rng(8200 + m)
    n, k = 520, 1024
    gate, up = synth.q4k_weights(g, n, k), synth.q4k_weights(g, n, k)
    x = synth.activations_bf16(g, m, k)
    make = lambda: [backend.Upload(x), backend.Upload(gate), backend.Upload(up), backend.AllocateBuffer(4 * m * n)]
    want, got, need = outputs_with_exact_workspace(backend, "ffn_gate_up_silu_q4k", [m, n, k], make, 3)
    assert np.array_equal(want, got), (m, need)


@pytest.mark.parametrize("name", ["gemm_mxfp4", "gemm_mxfp4_batched"])
@pytest.mark.parametrize("m", [1, 4, 16, 17, 100])
def test_mxfp4_fp32_rows(backend, name, m):
    g = synth.rng(8300 + m)
    n, k = 512, 1024
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    a = synth.activations_bf16(g, m, k)
    make = lambda: [backend.Upload(a), backend.Upload(w), backend.AllocateBuffer(4 * m * n)]
    want, got, need = outputs_with_exact_workspace(backend, name, [m, n, k], make, 2)
    assert np.array_equal(want, got), (name, m, need)


@pytest.mark.parametrize("m", [1, 4, 32, 33, 200])
@pytest.mark.parametrize("wperm", [0, 1])
def test_w4a8_with_and_without_the_permuted_weights(backend, m, wperm):
    g = synth.rng(8400 + m)
    n, k = 512, 1024
    w = synth.mxfp4_weights(g, n, k, -8, -4)
    if wperm:
        dw, dout = backend.Upload(w), backend.AllocateBuffer(w.size)
        run(backend, "permute_mxfp4_wmma", [dw, dout], [n, k, 0])
        backend.Synchronize()
        w = backend.CopyD2H(dout, dtype=np.uint8)
    x = synth.activations_bf16(g, m, k)
    dx, da8, das = backend.Upload(x), backend.AllocateBuffer(m * k), backend.AllocateBuffer(4 * m)
    run(backend, "quantize_fp8_pack_rows", [dx, da8, das], [m, k], grid=(m, 1, 1))
    backend.Synchronize()
    make = lambda: [da8, backend.Upload(w), das, backend.AllocateBuffer(n), backend.AllocateBuffer(4 * m * n)]
    want, got, need = outputs_with_exact_workspace(backend, "gemm_mxfp4_wmma", [m, n, k, 1, wperm], make, 4)
    assert np.array_equal(want, got), (m, wperm, need)


@pytest.mark.parametrize("rows", [1, 16, 17, 90])
def test_routed_experts(backend, rows):
    g = synth.rng(8500 + rows)
    experts, hidden, inter, top_k = 6, 256, 512, 2
    gate = np.concatenate([synth.q4k_weights(g, inter, hidden) for _ in range(experts)])
    up = np.concatenate([synth.q4k_weights(g, inter, hidden) for _ in range(experts)])
    down = np.concatenate([synth.q4k_weights(g, hidden, inter) for _ in range(experts)])
    gs, ds = gate.size // experts, down.size // experts
    x = synth.activations_bf16(g, rows, hidden)
    ids = np.stack([g.permutation(experts)[:top_k] for _ in range(rows)]).astype(np.uint32)
    wts = g.random(size=(rows, top_k)).astype(np.float32)
    make = lambda: [backend.Upload(x), backend.Upload(gate), backend.Upload(up), backend.Upload(down), backend.Upload(ids),
                    backend.Upload(wts), backend.AllocateBuffer(4 * rows * hidden)]
    want, got, need = outputs_with_exact_workspace(backend, "moe_experts_ffn_q4k_rows",
                                                   [hidden, inter, top_k, gs, gs, ds, rows, 0], make, 6, tight=False)
    assert np.array_equal(want, got), (rows, need)
    # the reference's two ids: phi from the first feeds the second
    make_gu = lambda: [backend.Upload(x), backend.Upload(gate), backend.Upload(up), backend.Upload(ids),
                       backend.AllocateBuffer(4 * rows * top_k * inter)]
    want, got, need = outputs_with_exact_workspace(backend, "moe_experts_gate_up_q4k_rows",
                                                   [hidden, inter, top_k, gs, gs, rows], make_gu, 4, tight=False)
    assert np.array_equal(want, got), (rows, need)
    phi = want
    make_dn = lambda: [backend.Upload(phi), backend.Upload(down), backend.Upload(ids), backend.Upload(wts),
                       backend.AllocateBuffer(4 * rows * hidden)]
    want, got, need = outputs_with_exact_workspace(backend, "moe_experts_down_q4k_rows",
                                                   [hidden, inter, top_k, ds, 0, rows], make_dn, 4, tight=False)
    assert np.array_equal(want, got), (rows, need)
