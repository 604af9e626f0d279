"""Benchmark of the MoE grouped-GEMM hot path on one MI355X.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-secondary] [--no-cpu-baseline]

A step is one pass of the hot path over one batch of synthetic, HBM-resident input. The headline workload is the
configuration the metric is quoted on: Mixtral 8x7B w1 grouped GEMM, bf16, T=4096 tokens top-2 (8192 expert-sorted
rows), K=4096, N=14336, 8 experts. Prints ONE JSON line; the other benchmark configurations (decode, W4A16, fp8)
are measured in the same run and reported under "secondary" with their own rooflines.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E

# HBM traffic per launch of the headline kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by what the
# same counters read for a plain copy of known size (profiles/gg_bf16_pingpong_mixtral_prefill_traffic.md):
# 1.94 GB fetched + 0.235 GB written.
PREFILL_TRAFFIC_BYTES = 2.18e9
# The same for the other workloads (profiles/bench_all_kernels_traffic.md): fetched + written bytes per launch.
DECODE_TRAFFIC_BYTES = {"up": 0.946e9 + 1.8e6, "down": 0.957e9 + 0.5e6}
W4A16_TRAFFIC_BYTES = {1: 32.3e6 + 0.03e6, 16: 32.3e6 + 0.46e6, 64: 44.9e6 + 1.8e6}
W4A16_GROUPED_TRAFFIC_BYTES = 254.2e6 + 1.8e6
W4A16_GROUPED_FP8OUT_TRAFFIC_BYTES = 254.4e6 + 1.15e6
FP8_BLOCK_TRAFFIC_BYTES = 9.04e9 + 0.27e9


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
        "value": round(2.0 * rows * N * K / t / 1e12, 3),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"first {n_experts_sample} of 8 experts ({rows} of {sum(c['m_sizes'].tolist())} rows), fp32 per-expert torch.matmul loop, best of 2",
    }


# After a change of load the GPU's power management overshoots and settles again: the first launch of the prefill
# GEMM after idle runs at the boost clock, launches 3-10 take 20-40 % longer than the steady state, and the
# steady state is reached after 40-50 launches (about 40 ms). Every measurement here therefore runs its workload
# untimed for SETTLE_SECONDS before its warm-up steps; the JSON line reports it as "settle_s".
SETTLE_SECONDS = 0.08


def settle(torch, fn, seconds=SETTLE_SECONDS):
    """Run fn() back to back, untimed, for at least `seconds` of wall time."""
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()


def event_time_ms(torch, fn, iters, warmup):
    """Average duration of fn() over `iters` back-to-back calls, HIP events on the current stream."""
    settle(torch, fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    s = torch.cuda.Event(enable_timing=True)
    e = torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) / iters


def secondary_workloads(torch, A, dev):
    """Decode (config 3), W4A16 (config 4) and fp8 block-scaled (config 5) shapes: HBM-bound kernels, reported as
    GB/s of algorithmic bytes against the 8 TB/s HBM peak. Weights rotate over enough distinct copies that the
    footprint exceeds the 256 MB Infinity Cache. Calls go straight through the C ABI so that the ~10 us kernels
    are not timed through Python allocation overhead."""
    from applied_ai_amd import configs

    lib = A._lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    out = []

    # ---- config 3: Mixtral decode, bf16, 64 rows over 8 experts ----
    c3 = configs.cfg3()
    m_sizes = c3["m_sizes"].tolist()
    ms_dev = c3["m_sizes"].to(dev)
    active = sum(1 for m in m_sizes if m > 0)
    for name, K, N in (("up-proj K=4096 N=14336", 4096, 14336), ("down-proj K=14336 N=4096", 14336, 4096)):
        x = torch.randn(64, K, device=dev).to(torch.bfloat16)
        ws = [(torch.randn(8 * N, K, device=dev) * 0.02).to(torch.bfloat16) for _ in range(2)]
        y = torch.empty(64, N, device=dev, dtype=torch.bfloat16)
        state = {"i": 0}

        def call():
            w = ws[state["i"] & 1]
            state["i"] += 1
            lib.moe_gg_grouped_gemm_bf16(x.data_ptr(), w.data_ptr(), y.data_ptr(), ms_dev.data_ptr(), 8, 64, N, K, N, 0, stream)

        ms = event_time_ms(torch, call, 40, 6)
        byt = active * N * K * 2 + 64 * K * 2 + 64 * N * 2
        out.append({"workload": f"Mixtral decode bf16, T=32 top-2 (64 rows, m_sizes {m_sizes}), {name}",
                    "us_per_launch": round(ms * 1e3, 2), "value": round(byt / ms / 1e6, 1), "unit": "GB/s",
                    "roofline": {"bound": "hbm", "kernel": "gg_bf16_decode", "achieved": round(byt / ms / 1e6, 1),
                                 "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(byt / ms / 1e6 / PEAK_HBM_GBS, 4),
                                 "traffic": DECODE_TRAFFIC_BYTES[name.split("-")[0]]}})
        del ws

    # ---- config 4: W4A16 split-K, K=4096, N=14336, group 128, (q - z) * s ----
    K, N, copies = 4096, 14336, 12
    qws = [torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, device=dev) for _ in range(copies)]
    sc = (torch.rand(K // 128, N, device=dev) * 0.015 + 0.005).to(torch.bfloat16)
    qz = torch.randint(-2**31, 2**31 - 1, (K // 128, N // 8), dtype=torch.int32, device=dev)
    for M in (1, 16, 64):
        a = torch.randn(M, K, device=dev).to(torch.bfloat16)
        c = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
        state = {"i": 0}

        def call():
            qw = qws[state["i"] % copies]
            state["i"] += 1
            lib.moe_gg_w4a16_splitk(a.data_ptr(), qw.data_ptr(), sc.data_ptr(), qz.data_ptr(), c.data_ptr(), M, N, K, 128, 0, 0, stream)

        ms = event_time_ms(torch, call, 120, 24)

        def call_hot():  # always the same 29 MB of weights: they stay in the 256 MB last-level cache
            lib.moe_gg_w4a16_splitk(a.data_ptr(), qws[0].data_ptr(), sc.data_ptr(), qz.data_ptr(), c.data_ptr(), M, N, K, 128, 0, 0, stream)

        ms_hot = event_time_ms(torch, call_hot, 120, 24)
        byt = K * N // 2 + (K // 128) * N * 2 + (K // 128) * N // 2 + M * K * 2 + M * N * 2
        out.append({"workload": f"W4A16 split-K M={M} K=4096 N=14336 group 128",
                    "us_per_launch": round(ms * 1e3, 2), "cache_hot_us_per_launch": round(ms_hot * 1e3, 2),
                    "value": round(byt / ms / 1e6, 1), "unit": "GB/s",
                    "roofline": {"bound": "hbm", "kernel": "w4a16_splitk_g128", "achieved": round(byt / ms / 1e6, 1),
                                 "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(byt / ms / 1e6 / PEAK_HBM_GBS, 4),
                                 "traffic": W4A16_TRAFFIC_BYTES.get(M)}})
    del qws

    # ---- W4A16 grouped (int4 experts), Mixtral decode: config 3's 64 rows over 8 experts, config 4's weight format ----
    E = 8
    qwe = [torch.randint(-2**31, 2**31 - 1, (E, K // 8, N), dtype=torch.int32, device=dev) for _ in range(2)]
    sce = (torch.rand(E, K // 128, N, device=dev) * 0.015 + 0.005).to(torch.bfloat16)
    qze = torch.randint(-2**31, 2**31 - 1, (E, K // 128, N // 8), dtype=torch.int32, device=dev)
    a = torch.randn(64, K, device=dev).to(torch.bfloat16)
    c = torch.empty(64, N, device=dev, dtype=torch.bfloat16)
    ms3 = c3["m_sizes"].to(dev)
    state = {"i": 0}

    def call():
        q = qwe[state["i"] & 1]
        state["i"] += 1
        lib.moe_gg_w4a16_grouped(a.data_ptr(), q.data_ptr(), sce.data_ptr(), qze.data_ptr(), c.data_ptr(), ms3.data_ptr(),
                                 E, 64, N, K, 128, 0, 0, stream)

    ms = event_time_ms(torch, call, 40, 6)
    act = sum(1 for m in c3["m_sizes"].tolist() if m > 0)
    byt = act * (K * N // 2 + K // 128 * N * 2 + K // 128 * N // 2) + 64 * K * 2 + 64 * N * 2
    out.append({"workload": f"W4A16 grouped GEMM (int4 experts), Mixtral decode: 64 rows over 8 experts, K={K} N={N} group 128",
                "us_per_launch": round(ms * 1e3, 2), "value": round(byt / ms / 1e6, 1), "unit": "GB/s",
                "roofline": {"bound": "hbm", "kernel": "w4a16_splitk_g128 (grid.y = experts)", "achieved": round(byt / ms / 1e6, 1),
                             "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(byt / ms / 1e6 / PEAK_HBM_GBS, 4),
                             "traffic": W4A16_GROUPED_TRAFFIC_BYTES}})

    # the same call with the 1 x 128 fp8 quantiser as its epilogue, beside the two launches it replaces
    cq = torch.empty(64, N, device=dev, dtype=torch.uint8)
    cs = torch.empty(64, N // 128, device=dev, dtype=torch.float32)

    def call_q():
        q = qwe[state["i"] & 1]
        state["i"] += 1
        lib.moe_gg_w4a16_grouped_fp8out(a.data_ptr(), q.data_ptr(), sce.data_ptr(), qze.data_ptr(), cq.data_ptr(),
                                        cs.data_ptr(), ms3.data_ptr(), E, 64, N, K, 128, 0, 0, stream)

    def call_two():
        call()
        lib.moe_gg_fp8_groupwise_quant(c.data_ptr(), 0, cq.data_ptr(), cs.data_ptr(), 64 * N, stream)

    ms_q = event_time_ms(torch, call_q, 40, 6)
    ms_two = event_time_ms(torch, call_two, 40, 6)
    byt_q = byt - 64 * N * 2 + 64 * N + 64 * (N // 128) * 4
    out.append({"workload": f"W4A16 grouped GEMM with the fp8 1x128 quantiser as epilogue, same shape (fp8 codes + scales out)",
                "us_per_launch": round(ms_q * 1e3, 2), "gemm_then_quantiser_us": round(ms_two * 1e3, 2),
                "value": round(byt_q / ms_q / 1e6, 1), "unit": "GB/s",
                "roofline": {"bound": "hbm", "kernel": "w4a16_splitk_g128 (fp8 output)", "achieved": round(byt_q / ms_q / 1e6, 1),
                             "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(byt_q / ms_q / 1e6 / PEAK_HBM_GBS, 4),
                             "traffic": W4A16_GROUPED_FP8OUT_TRAFFIC_BYTES}})
    del qwe

    # ---- config 5: DeepSeek-V3-style fp8 block-scaled, 256 experts top-8, Zipf(1.1) routing ----
    _, _, _, m5 = configs.cfg5_routing()
    G, N, K = 256, 4096, 7168
    M = int(m5.sum())
    f8 = torch.float8_e4m3fn

    def rand_fp8(rows):
        t = torch.randint(0, 256, (rows, K), dtype=torch.uint8, device=dev)
        return torch.where((t & 0x7F) == 0x7F, t & 0xF0, t)  # no NaN codes

    xq = rand_fp8(M).view(f8)
    wq = torch.empty(G * N, K, dtype=torch.uint8, device=dev)
    for g in range(G):
        wq[g * N:(g + 1) * N] = rand_fp8(N)
    wq = wq.view(f8)
    xs = torch.rand(M, K // 128, device=dev) * 0.01 + 0.001
    ws = torch.rand(G * N // 128, K // 128, device=dev) * 0.01 + 0.001
    y = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    ms_dev = m5.to(dev)

    def call():
        lib.moe_gg_grouped_gemm_fp8(xq.data_ptr(), wq.data_ptr(), y.data_ptr(), xs.data_ptr(), ws.data_ptr(), 1,
                                    ms_dev.data_ptr(), G, M, N, K, N, 0, stream)

    ms = event_time_ms(torch, call, 5, 2)
    active = int((m5 > 0).sum())
    byt = M * K + active * N * K + M * N * 2 + M * (K // 128) * 4 + active * (N // 128) * (K // 128) * 4
    flop = 2.0 * M * N * K
    out.append({"workload": "DeepSeek-V3-style fp8 e4m3 block-scaled grouped GEMM: 256 experts top-8, T=4096 (32768 rows, Zipf 1.1), K=7168, N=4096",
                "ms_per_launch": round(ms, 3), "value": round(byt / ms / 1e6, 1), "unit": "GB/s",
                "tflops": round(flop / ms / 1e9, 1),
                "roofline": {"bound": "hbm", "kernel": "gg_fp8_pingpong_block", "achieved": round(byt / ms / 1e6, 1),
                             "peak": PEAK_HBM_GBS, "unit": "GB/s", "frac": round(byt / ms / 1e6 / PEAK_HBM_GBS, 4),
                             "traffic": FP8_BLOCK_TRAFFIC_BYTES}})
    del xq, wq, xs, ws, y

    # ---- whole MoE layer (fused_moe): Mixtral 8x7B, T=4096 top-2, bf16 ----
    T, K, n, E, topk = 4096, 4096, 14336, 8, 2
    gen = torch.Generator(device=dev).manual_seed(1002)
    h = (torch.randn(T, K, device=dev, generator=gen) / 10).to(torch.bfloat16)
    w1 = torch.empty(E, 2 * n, K, device=dev, dtype=torch.bfloat16)
    w2 = torch.empty(E, K, n, device=dev, dtype=torch.bfloat16)
    for e in range(E):
        w1[e] = (torch.randn(2 * n, K, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        w2[e] = (torch.randn(K, n, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    score = torch.softmax(torch.randn(T, E, device=dev, generator=gen), dim=-1)
    tw, ids = torch.topk(score, topk)
    ids = ids.to(torch.int32)
    ms = event_time_ms(torch, lambda: A.fused_moe(h, w1, w2, tw, ids), 10, 3)
    flop = 2.0 * T * topk * (2 * n * K + K * n)
    out.append({"workload": "Mixtral 8x7B MoE layer (fused_moe: group, gather, w1 GEMM, SiLU-and-mul, w2 GEMM, top-2 combine), T=4096, bf16",
                "m_sizes": torch.bincount(ids.flatten().long(), minlength=E).tolist(),
                "ms_per_launch": round(ms, 3), "value": round(flop / ms / 1e9, 1), "unit": "TFLOP/s",
                "roofline": {"bound": "mfma", "kernel": "gg_bf16_pingpong (two launches) + glue kernels", "achieved": round(flop / ms / 1e9, 1),
                             "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                             "traffic": None}})
    del h, w1, w2

    # ---- backward of the grouped GEMM (training), Mixtral w1 shape, [M, N] gradient ----
    G, M, N, K = 8, 8192, 14336, 4096
    ms_dev = torch.tensor([1012, 1039, 1048, 1036, 998, 1023, 1040, 996], dtype=torch.int32, device=dev)  # config 2's routing
    x = (torch.randn(M, K, device=dev, generator=gen) / 8).to(torch.bfloat16)
    w = torch.empty(G * N, K, device=dev, dtype=torch.bfloat16)
    for g in range(G):
        w[g * N:(g + 1) * N] = (torch.randn(N, K, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    go = (torch.randn(M, N, device=dev, generator=gen) / 8).to(torch.bfloat16)
    gx = torch.zeros_like(x)
    gw = torch.empty_like(w)
    nbytes = lib.moe_gg_grouped_gemm_backward_workspace(G, M, N, K, 0)
    wsp = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    def call():
        lib.moe_gg_grouped_gemm_backward_bf16(go.data_ptr(), N, 0, x.data_ptr(), w.data_ptr(), ms_dev.data_ptr(), G, M, N, K,
                                              gx.data_ptr(), gw.data_ptr(), wsp.data_ptr(), nbytes, stream)

    ms = event_time_ms(torch, call, 5, 2)
    flop = 4.0 * M * N * K
    out.append({"workload": "grouped GEMM backward (grad_x and grad_w), Mixtral 8x7B w1 shape: 8192 rows, K=4096, N=14336, 8 experts, bf16",
                "ms_per_launch": round(ms, 3), "value": round(flop / ms / 1e9, 1), "unit": "TFLOP/s",
                "roofline": {"bound": "mfma", "kernel": "gg_bf16_pingpong_nt + gg_bf16_pingpong_wgrad_direct",
                             "achieved": round(flop / ms / 1e9, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                             "frac": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "traffic": None}})
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy, so that a rocprofv3 --pmc run of this command sees a kernel of known traffic")
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

    settle(torch, lambda: A.grouped_gemm(x, w, ms))
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
        "settle_s": SETTLE_SECONDS,
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
            "kernel": "gg_bf16_pingpong",
            "achieved": round(achieved, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            "traffic": PREFILL_TRAFFIC_BYTES,
            "kernel_ms": {"avg": round(avg_kernel_ms, 4), "p20": round(kern_ms[len(kern_ms) // 5], 4),
                          "p50": round(kern_ms[len(kern_ms) // 2], 4), "p80": round(kern_ms[(len(kern_ms) * 4) // 5], 4)},
        },
    }
    # Context for the roofline fraction: the vendor library's dense bf16 GEMM of the same FLOP count and data
    # (one [8192, 4096] x [4096, 14336] product through torch.matmul -> hipBLASLt), timed the same way. With
    # random operands the MFMA clock is power-limited well below the 2.5 PFLOP/s figure, for the library too.
    wd = w[:N]
    lib_ms = event_time_ms(torch, lambda: torch.matmul(x, wd.t()), 20, 5)
    out["dense_gemm_library"] = {"value": round(2.0 * x.shape[0] * N * K / lib_ms / 1e9, 1), "unit": "TFLOP/s",
                                 "what": "torch.matmul (hipBLASLt) bf16 [8192,4096]x[4096,14336], same FLOPs, no grouping"}
    del x, w, y, wd
    if args.copy_calibration:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline_prefill(c)
    if not args.no_secondary:
        out["secondary"] = secondary_workloads(torch, A, dev)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
