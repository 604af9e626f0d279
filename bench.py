"""Benchmark of the MoE grouped-GEMM hot path on one MI355X.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload prefill]
A step is one pass of the hot path over one batch of synthetic, HBM-resident input. The default workload is the
configuration the headline metric is quoted on: Mixtral 8x7B w1 grouped GEMM, bf16, T=4096 tokens top-2 (8192
expert-sorted rows), K=4096, N=14336, 8 experts. Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E


def cpu_baseline_prefill(c, n_experts_sample=2):
    """The reference's CPU path - a per-expert torch.matmul loop (dev/triton_groupGEMM/testing/unit_tests.py:49-55)
    in fp32 on the host cores - timed on the first `n_experts_sample` experts of the same workload."""
    import torch
    from oracle import oracle as O

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    m_sizes = c["m_sizes"].tolist()[:n_experts_sample]
    rows = sum(m_sizes)
    N = c["w"].shape[0] // len(c["m_sizes"])
    K = c["w"].shape[1]
    x = c["x_sorted"][:rows].float()
    w = c["w"][: n_experts_sample * N].float()
    O.grouped_gemm_torch_loop(x[:64], w, [64] + [0] * (n_experts_sample - 1))  # warm-up
    times = []
    for _ in range(2):
        t0 = time.perf_counter()
        O.grouped_gemm_torch_loop(x, w, m_sizes)
        times.append(time.perf_counter() - t0)
    t = min(times)
    return {
        "value": 2.0 * rows * N * K / t / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {n_experts_sample} of 8 experts ({rows} of {sum(c['m_sizes'].tolist())} rows), fp32 torch.matmul loop, best of 2",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch

    import applied_ai_amd as A
    from applied_ai_amd import configs

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    c = configs.cfg2()
    x = c["x_sorted"].to(dev)
    w = c["w"].to(dev)
    ms = c["m_sizes"].to(dev)
    G = ms.shape[0]
    N = w.shape[0] // G
    K = w.shape[1]
    rows = int(c["m_sizes"].sum())
    flop = 2.0 * rows * N * K

    for _ in range(args.warmup):
        y = A.grouped_gemm(x, w, ms)
    torch.cuda.synchronize()
    # HIP events on the stream the kernels are launched on (torch's current stream).
    start = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    stop = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        start[i].record()
        y = A.grouped_gemm(x, w, ms)
        stop[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    kern_ms = sorted(s.elapsed_time(e) for s, e in zip(start, stop))
    avg_kernel_ms = sum(kern_ms) / len(kern_ms)
    ms_per_step = wall * 1e3 / args.steps
    value = flop / (ms_per_step * 1e-3) / 1e12
    achieved = flop / (avg_kernel_ms * 1e-3) / 1e12

    out = {
        "metric": "grouped-GEMM TFLOP/s + % MFMA peak, Mixtral 8x7B bf16 T=4096 top-2",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "Mixtral 8x7B w1 grouped GEMM: T=4096 top-2 -> 8192 expert-sorted rows, K=4096, N=14336, 8 experts, bf16 in/out, fp32 accumulate",
            "m_sizes": c["m_sizes"].tolist(),
        },
        "pct_mfma_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
        "roofline": {
            "bound": "mfma",
            "kernel": "gg_bf16_persistent",
            "achieved": round(achieved, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            "traffic": None,
            "kernel_ms": {"avg": round(avg_kernel_ms, 4), "p20": round(kern_ms[len(kern_ms) // 5], 4),
                          "p50": round(kern_ms[len(kern_ms) // 2], 4), "p80": round(kern_ms[(len(kern_ms) * 4) // 5], 4)},
        },
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_prefill(c)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
