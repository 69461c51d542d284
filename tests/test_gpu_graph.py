"""A decode step recorded into a HIP graph: every replay must give what the eager launches give,
also after the inputs changed and after eager work (including a prefill-sized call, which grows
the library's workspace) ran between the replays.  The ids recorded here are the ones that use
library-owned scratch: the few-row Q4_K path and the fused feed-forward id (decode scratch)."""
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
    kq, kb, kf = backend.LoadKernel("gemm_q4k_vec"), backend.LoadKernel("gemm_q4k_batched"), backend.LoadKernel("ffn_gate_up_silu_q4k")

    def step():
        backend.LaunchKernel(kq, KernelLaunch(grid_x=(n + 7) // 8, buffers=[wrap(x1), wrap(gate), wrap(y1)], scalars=[1, n, k, 1]))
        backend.LaunchKernel(kb, KernelLaunch(grid_x=(4 * n + 7) // 8, buffers=[wrap(x4), wrap(gate), wrap(y4)], scalars=[4, n, k]))
        backend.LaunchKernel(kf, KernelLaunch(grid_x=(n + 7) // 8, buffers=[wrap(x1), wrap(gate), wrap(up), wrap(f1)], scalars=[1, n, k]))
        backend.LaunchKernel(kf, KernelLaunch(grid_x=(4 * n + 7) // 8, buffers=[wrap(x4), wrap(gate), wrap(up), wrap(f4)], scalars=[4, n, k]))

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
        for t in (y1, y4, f1, f4):
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = [t.cpu().numpy().copy() for t in (y1, y4, f1, f4)]
        for t in (y1, y4, f1, f4):
            t.fill_(float("nan"))
        step()                            # the same work eagerly
        torch.cuda.synchronize()
        eager = [t.cpu().numpy().copy() for t in (y1, y4, f1, f4)]
        for gv, ev in zip(got, eager):
            assert np.array_equal(gv.view(np.uint32), ev.view(np.uint32)), (replay, seed)
        if replay == 0:                   # and the eager result is right
            assert rel_err(eager[0], oracle.gemm_q4k(a[0], gate_h, 1, n, k)) < 1e-3
            assert rel_err(eager[1], oracle.gemm_q4k(a[1:], gate_h, 4, n, k)) < 1e-3
            assert rel_err(eager[3], oracle.ffn_gate_up_silu_q4k(a[1:], gate_h, up_h, 4, n, k)) < 1e-3
        backend.LaunchKernel(kw, KernelLaunch(grid_x=n // 64 + 1, grid_y=1, buffers=[wrap(xb), wrap(gate), wrap(yb)],
                                              scalars=[big_m, n, k]))
        torch.cuda.synchronize()
