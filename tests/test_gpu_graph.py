"""A decode step recorded into a HIP graph: every replay must give what the eager launches give,
also after the inputs changed and after eager work (including a prefill-sized call, which grows
the library's workspace) ran between the replays.  The ids recorded here are the ones that use
library-owned scratch: the few-row Q4_K path, the fused feed-forward id, and MXFP4 / FP8 weights with four
fp32 rows (their E4M3 terms), all in the decode scratch."""
import numpy as np
import pytest
import torch

import oracle
from tessera_amd import KernelLaunch, synth
from util import rel_err

pytestmark = pytest.mark.gpu


def test_recorded_decode_step_replays_like_eager(backend):
    dev = torch.device("cuda:0")
    g = synth.rng(900)
    n, k = 4100, 4096                     # 16.8 M weights: 2..16 rows take the few-row MFMA kernels
    to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    wrap = lambda t: backend.WrapBuffer(t.data_ptr(), t.numel() * t.element_size())
    gate_h, up_h = synth.q4k_weights(g, n, k), synth.q4k_weights(g, n, k)
    gate, up = to_dev(gate_h), to_dev(up_h)
    x1, x4 = torch.empty(k, device=dev), torch.empty(4 * k, device=dev)
    y1 = torch.empty(n, device=dev)
    y4 = torch.empty(4 * n, device=dev)
    f1 = torch.empty(n, device=dev)
    f4 = torch.empty(4 * n, device=dev)
    mx = to_dev(synth.mxfp4_weights(g, n, k, -8, -4))
    codes_h, scales_h = synth.fp8_weights(g, n, k)
    codes, scales = to_dev(codes_h), to_dev(scales_h)
    m4, e4 = torch.empty(4 * n, device=dev), torch.empty(4 * n, device=dev)
    km, k8 = backend.LoadKernel("gemm_mxfp4_rows"), backend.LoadKernel("gemm_fp8")
    kq, kb, kf = backend.LoadKernel("gemm_q4k_vec"), backend.LoadKernel("gemm_q4k_batched"), backend.LoadKernel("ffn_gate_up_silu_q4k")

    def step():
        backend.LaunchKernel(kq, KernelLaunch(grid_x=(n + 7) // 8, buffers=[wrap(x1), wrap(gate), wrap(y1)], scalars=[1, n, k, 1]))
        backend.LaunchKernel(kb, KernelLaunch(grid_x=(4 * n + 7) // 8, buffers=[wrap(x4), wrap(gate), wrap(y4)], scalars=[4, n, k]))
        backend.LaunchKernel(kf, KernelLaunch(grid_x=(n + 7) // 8, buffers=[wrap(x1), wrap(gate), wrap(up), wrap(f1)], scalars=[1, n, k]))
        backend.LaunchKernel(kf, KernelLaunch(grid_x=(4 * n + 7) // 8, buffers=[wrap(x4), wrap(gate), wrap(up), wrap(f4)], scalars=[4, n, k]))
        backend.LaunchKernel(km, KernelLaunch(grid_x=(4 * n + 7) // 8, buffers=[wrap(x4), wrap(mx), wrap(m4)], scalars=[4, n, k]))
        backend.LaunchKernel(k8, KernelLaunch(grid_x=(4 * n + 255) // 256, buffers=[wrap(x4), wrap(codes), wrap(scales), wrap(e4)],
                                              scalars=[4, n, k]))

    def set_inputs(seed):
        a = synth.activations_f32(synth.rng(seed), 5, k)
        x1.copy_(to_dev(a[0]))
        x4.copy_(to_dev(a[1:].reshape(-1)))
        return a

    cur = torch.cuda.current_stream()
    backend.SetStream(cur.cuda_stream)
    a = set_inputs(1)
    step()                                # warm-up (and the eager result of the first inputs)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        backend.SetStream(torch.cuda.current_stream().cuda_stream)
        step()
    backend.SetStream(cur.cuda_stream)

    big_m = 64                            # a prefill-sized call between replays grows the other workspace
    xb = to_dev(synth.activations_f32(synth.rng(7), big_m, k))
    yb = torch.empty(big_m * n, device=dev)
    kw = backend.LoadKernel("gemm_q4k_wmma")
    for replay, seed in enumerate((1, 2, 3, 2)):
        a = set_inputs(seed)
        for t in (y1, y4, f1, f4, m4, e4):
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.cpu().numpy().copy() for t in (y1, y4, f1, f4, m4, e4)]
        for t in (y1, y4, f1, f4, m4, e4):
            t.fill_(float("nan"))
        step()                            # the same work eagerly
        torch.cuda.synchronize()
        eager = [t.cpu().numpy().copy() for t in (y1, y4, f1, f4, m4, e4)]
        for gv, ev in zip(got, eager):
            assert np.array_equal(gv.view(np.uint32), ev.view(np.uint32)), (replay, seed)
        if replay == 0:                   # and the eager result is right
            assert rel_err(eager[0], oracle.gemm_q4k(a[0], gate_h, 1, n, k)) < 1e-3
            assert rel_err(eager[1], oracle.gemm_q4k(a[1:], gate_h, 4, n, k)) < 1e-3
            assert rel_err(eager[3], oracle.ffn_gate_up_silu_q4k(a[1:], gate_h, up_h, 4, n, k)) < 1e-3
            assert rel_err(eager[5], oracle.gemm_fp8(a[1:], codes_h, scales_h, 4, n, k)) < 2e-3
        backend.LaunchKernel(kw, KernelLaunch(grid_x=n // 64 + 1, grid_y=1, buffers=[wrap(xb), wrap(gate), wrap(yb)],
                                              scalars=[big_m, n, k]))
        torch.cuda.synchronize()


def test_prefill_call_recorded_with_a_caller_owned_workspace(backend):
    """A prefill-sized Q4_K call (64 rows: fp16 MFMA path, which needs scratch) recorded into a HIP
    graph with a workspace the caller set beforehand: nothing is allocated while recording, every
    replay equals the eager result, a launch that needs more than the workspace holds is refused,
    and clearing the workspace restores the library-owned one."""
    from tessera_amd import StatusCode, StatusError
    dev = torch.device("cuda:0")
    g = synth.rng(901)
    m, n, k = 64, 1030, 4096
    to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    wrap = lambda t: backend.WrapBuffer(t.data_ptr(), t.numel() * t.element_size())
    w_h = synth.q4k_weights(g, n, k)
    w = to_dev(w_h)
    x = torch.empty(m * k, device=dev)
    y = torch.empty(m * n, device=dev)
    kern = backend.LoadKernel("gemm_q4k_wmma")
    need = backend.WorkspaceBytes(kern, [m, n, k])
    assert need >= m * k * 2                                   # the fp16 copy of the activations at least
    assert backend.WorkspaceBytes(backend.LoadKernel("gemm_q4k_vec"), [1, n, k, 1]) == 0
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    launch = KernelLaunch(grid_x=n // 64 + 1, buffers=[wrap(x), wrap(w), wrap(y)], scalars=[m, n, k])
    cur = torch.cuda.current_stream()
    backend.SetStream(cur.cuda_stream)
    backend.SetWorkspace(wrap(ws))
    try:
        a = synth.activations_f32(synth.rng(11), m, k)
        x.copy_(to_dev(a.reshape(-1)))
        backend.LaunchKernel(kern, launch)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            backend.SetStream(torch.cuda.current_stream().cuda_stream)
            backend.LaunchKernel(kern, launch)
        backend.SetStream(cur.cuda_stream)
        for seed in (11, 12, 13):
            a = synth.activations_f32(synth.rng(seed), m, k)
            x.copy_(to_dev(a.reshape(-1)))
            y.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            got = y.cpu().numpy().copy()
            y.fill_(float("nan"))
            backend.LaunchKernel(kern, launch)
            torch.cuda.synchronize()
            eager = y.cpu().numpy().copy()
            assert np.array_equal(got.view(np.uint32), eager.view(np.uint32)), seed
            if seed == 11:
                ref = oracle.gemm_q4k(a, w_h, m, n, k, threads=True)
                rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
                assert float(np.max(np.abs(eager.reshape(m, n) - ref))) <= 4e-3 * rms
        # twice the rows need twice the scratch: refused, nothing launched, nothing allocated
        xb = torch.empty(2 * m * k, device=dev)
        yb = torch.empty(2 * m * n, device=dev)
        with pytest.raises(StatusError) as err:
            backend.LaunchKernel(kern, KernelLaunch(grid_x=1, buffers=[wrap(xb), wrap(w), wrap(yb)], scalars=[2 * m, n, k]))
        assert err.value.code == StatusCode.InvalidArgument and "workspace" in str(err.value)
    finally:
        backend.SetWorkspace(None)
    backend.LaunchKernel(kern, KernelLaunch(grid_x=1, buffers=[wrap(xb), wrap(w), wrap(yb)], scalars=[2 * m, n, k]))
    torch.cuda.synchronize()


def test_recorded_prefill_survives_growth_of_the_library_workspace(backend):
    """A prefill-sized call recorded against the library-owned workspace, then a larger eager call
    that makes the library get a bigger block: the block the graph points at is retired, not freed,
    so the replays still equal eager launches.  And while a stream is being captured the library's
    block cannot grow: such a launch is refused, and works once an eager call of that size has run."""
    from tessera_amd import StatusCode, StatusError
    dev = torch.device("cuda:0")
    g = synth.rng(902)
    n, k = 1030, 4096
    to_dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    wrap = lambda t: backend.WrapBuffer(t.data_ptr(), t.numel() * t.element_size())
    w = to_dev(synth.q4k_weights(g, n, k))
    kern = backend.LoadKernel("gemm_q4k_wmma")
    cur = torch.cuda.current_stream()
    backend.SetStream(cur.cuda_stream)
    backend.SetWorkspace(None)
    # far larger than anything another test asks for (the largest is a 178 MB decode of a K-quant tensor),
    # so that this call and the next both make the block grow; inputs are made on the device
    m_small, m_big = 40000, 90000
    assert backend.WorkspaceBytes(kern, [m_big, n, k]) > 2 * backend.WorkspaceBytes(kern, [m_small, n, k]) > (512 << 20)
    gen = torch.Generator(device=dev)

    def fill(t, seed):
        gen.manual_seed(seed)
        t.normal_(generator=gen)
    x = torch.empty(m_small * k, device=dev)
    y = torch.empty(m_small * n, device=dev)
    launch = KernelLaunch(grid_x=n // 64 + 1, buffers=[wrap(x), wrap(w), wrap(y)], scalars=[m_small, n, k])
    fill(x, 21)
    # capture before any eager call of this size: the library would have to allocate, refused
    graph = torch.cuda.CUDAGraph()
    refused = False
    with torch.cuda.graph(graph):
        backend.SetStream(torch.cuda.current_stream().cuda_stream)
        try:
            backend.LaunchKernel(kern, launch)
        except StatusError as e:
            refused = e.code == StatusCode.InvalidArgument and "captured" in str(e)
    backend.SetStream(cur.cuda_stream)
    assert refused
    backend.LaunchKernel(kern, launch)          # eager: the block grows to this size
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        backend.SetStream(torch.cuda.current_stream().cuda_stream)
        backend.LaunchKernel(kern, launch)
    backend.SetStream(cur.cuda_stream)
    xb = torch.empty(m_big * k, device=dev)
    fill(xb, 22)
    yb = torch.empty(m_big * n, device=dev)
    for seed in (21, 23):
        fill(x, seed)
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = y.cpu().numpy().copy()
        # a larger eager call: the library's block is replaced (on the first pass)
        backend.LaunchKernel(kern, KernelLaunch(grid_x=1, buffers=[wrap(xb), wrap(w), wrap(yb)], scalars=[m_big, n, k]))
        torch.cuda.synchronize()
        y.fill_(float("nan"))
        backend.LaunchKernel(kern, launch)
        torch.cuda.synchronize()
        assert np.array_equal(got.view(np.uint32), y.cpu().numpy().view(np.uint32)), seed
    # and once more through the graph, now that its block is a retired one
    y.fill_(float("nan"))
    graph.replay()
    torch.cuda.synchronize()
    backend.LaunchKernel(kern, launch)
    got = y.cpu().numpy().copy()
    torch.cuda.synchronize()
    assert np.array_equal(got.view(np.uint32), y.cpu().numpy().view(np.uint32))
