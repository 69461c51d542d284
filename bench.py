#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

Headline (BASELINE.json configs[1]): Q4_K decode GEMV, M=1, 27B FFN shapes.  One step is
one FFN's three projections -- gate and up (N=17408, K=5120) and down (N=5120, K=17408) --
on that layer's own weights; consecutive steps walk through `--layers` distinct layers
(default 8 = 1.2 GB of weights, five times the 256 MB Infinity Cache) so every launch streams
its weights from HBM, as a real decode does.  `value` is algorithmic GB/s over the timed
steps: (weights + activation + output bytes of the three launches) / time.

The JSON line also carries the roofline of the dominant kernel (gate/up GEMV) and a CPU
baseline (the oracle's restatement of the reference host GEMM on BASELINE configs[0]).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
N_FF, K_HID = 17408, 5120


def q4k_bytes(n, k):
    return n * (k // 256) * 144


def gemv_algorithmic_bytes(n, k):
    return q4k_bytes(n, k) + 4 * k + 4 * n


def cpu_baseline(seconds_budget=12.0):
    """Reference host GEMM (GemmQ4KRef restated in oracle/qmm_oracle.c) on configs[0]:
    Q4_K GEMV M=1, N=K=5120, on this host's cores.  The Vulkan-on-lavapipe baseline the
    configuration names is not available: the image has no Vulkan loader, lavapipe or glslang."""
    import numpy as np

    import oracle
    from tessera_amd import synth

    g = synth.rng(0)
    n = k = 5120
    w = synth.q4k_weights(g, n, k)
    a = synth.activations_f32(g, 1, k)
    nbytes = gemv_algorithmic_bytes(n, k)
    out = {}
    for label, threads in (("single", False), ("omp", True)):
        oracle.gemm_q4k(a, w, 1, n, k, threads=threads)
        times = []
        t_end = time.perf_counter() + seconds_budget / 2
        while len(times) < 20 or (time.perf_counter() < t_end and len(times) < 200):
            t0 = time.perf_counter()
            oracle.gemm_q4k(a, w, 1, n, k, threads=threads)
            times.append(time.perf_counter() - t0)
        times.sort()
        out[label] = (nbytes / times[len(times) // 2] / 1e9, len(times))
    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or os.cpu_count()
    return {
        "value": round(out["omp"][0], 3), "unit": "GB/s", "cores": cores, "kind": "port",
        "single_thread_GBps": round(out["single"][0], 3),
        "sample": f"Q4_K GEMV M=1 N=K=5120 (configs[0]), median of {out['omp'][1]} runs of the "
                  "oracle's GemmQ4KRef restatement, OpenMP over weight rows; lavapipe/Vulkan "
                  "absent from the image, so the reference host GEMM stands in",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--layers", type=int, default=8)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); "
                 "run with --gpus 1")

    import numpy as np
    import torch

    from tessera_amd import CreateBackend, KernelLaunch, synth

    backend = CreateBackend()
    backend.SetStream(torch.cuda.current_stream().cuda_stream)
    dev = torch.device("cuda:0")
    g = synth.rng(1)

    def to_dev(arr):
        return torch.from_numpy(np.ascontiguousarray(arr)).to(dev)

    # One layer generated on the host, the others are device copies at their own addresses
    # (caches are address-based, so identical bytes at distinct addresses still miss).
    base = [to_dev(synth.q4k_weights(g, N_FF, K_HID)), to_dev(synth.q4k_weights(g, N_FF, K_HID)),
            to_dev(synth.q4k_weights(g, K_HID, N_FF))]
    layers = [base] + [[t.clone() for t in base] for _ in range(args.layers - 1)]
    x_hid = to_dev(synth.activations_f32(g, 1, K_HID))
    x_ff = to_dev(synth.activations_f32(g, 1, N_FF))
    y_gate = torch.empty(N_FF, dtype=torch.float32, device=dev)
    y_up = torch.empty(N_FF, dtype=torch.float32, device=dev)
    y_down = torch.empty(K_HID, dtype=torch.float32, device=dev)

    def wrap(t):
        return backend.WrapBuffer(t.data_ptr(), t.numel() * t.element_size())

    kern = backend.LoadKernel("gemm_q4k_vec")
    plans = []
    for gate, up, down in layers:
        plans.append([
            KernelLaunch(grid_x=N_FF // 8, buffers=[wrap(x_hid), wrap(gate), wrap(y_gate)], scalars=[1, N_FF, K_HID, 1]),
            KernelLaunch(grid_x=N_FF // 8, buffers=[wrap(x_hid), wrap(up), wrap(y_up)], scalars=[1, N_FF, K_HID, 1]),
            KernelLaunch(grid_x=K_HID // 8, buffers=[wrap(x_ff), wrap(down), wrap(y_down)], scalars=[1, K_HID, N_FF, 1]),
        ])

    def step(i, only=None):
        for j, launch in enumerate(plans[i % len(plans)]):
            if only is None or j in only:
                backend.LaunchKernel(kern, launch)

    def timed_ms(only=None):
        """W eager warm-up steps, then exactly K steps recorded into one HIP graph (the host
        cannot issue 10-microsecond launches fast enough from Python) and timed with HIP events
        on the stream that runs them."""
        backend.SetStream(torch.cuda.current_stream().cuda_stream)
        for i in range(args.warmup):
            step(i, only)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            backend.SetStream(torch.cuda.current_stream().cuda_stream)
            for i in range(args.steps):
                step(args.warmup + i, only)
        backend.SetStream(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1)

    ms = timed_ms()
    step_bytes = 2 * gemv_algorithmic_bytes(N_FF, K_HID) + gemv_algorithmic_bytes(K_HID, N_FF)
    value = step_bytes * args.steps / (ms * 1e-3) / 1e9

    # Roofline of the dominant kernel: the gate/up GEMV alone, back to back over the layers.
    us_per_launch = timed_ms(only=(0, 1)) * 1e3 / (2 * args.steps)
    achieved = gemv_algorithmic_bytes(N_FF, K_HID) / (us_per_launch * 1e-6) / 1e9
    us_down = timed_ms(only=(2,)) * 1e3 / args.steps

    result = {
        "metric": "Q4_K/MXFP4 GEMV GB/s (% HBM peak) + prefill GEMM TFLOP/s, 27B FFN shapes",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms / args.steps, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[1]: Q4_K decode GEMV M=1, gate+up (17408x5120) and down "
                               "(5120x17408) per step, fp32 activations, fp32 accumulate",
                   "layers_rotated": args.layers, "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 1)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "gemv_kernel<Q4KPairCodec> N=17408 K=5120",
                     "us_per_launch": round(us_per_launch, 3),
                     "algorithmic_bytes_per_launch": gemv_algorithmic_bytes(N_FF, K_HID),
                     "down_us_per_launch": round(us_down, 3),
                     "down_GBps": round(gemv_algorithmic_bytes(K_HID, N_FF) / (us_down * 1e-6) / 1e9, 1)},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
