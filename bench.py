"""Benchmark of the MoE grouped-GEMM hot path on one MI355X.

python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-secondary] [--no-cpu-baseline] [--moe-sweep] [--budget-s S]
                [--pin OP=VARIANT ...]

A step is one pass of the hot path over one batch of synthetic, HBM-resident input. The headline workload is the
configuration the metric is quoted on: Mixtral 8x7B w1 grouped GEMM, bf16, T=4096 tokens top-2 (8192 expert-sorted
rows), K=4096, N=14336, 8 experts. Prints ONE JSON line; the other benchmark configurations (decode, W4A16, fp8)
are measured in the same run and reported under "secondary" with their own rooflines.

Order of work: every GPU measurement first (headline, the vendor library's dense GEMM, the secondary workloads), then
the CPU baselines (headline first). A wall-clock budget (--budget-s, default 300 s) is checked before every secondary
workload and every CPU baseline; what does not fit is reported as {"skipped": "time budget"}, so the line is printed
within minutes whatever the host's speed. SIGTERM / SIGINT print the line with what has been measured so far.
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

# HBM traffic per launch of the timed kernels comes from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by what
# the same counters read for a plain copy of known size. The figures live in profiles/traffic.json together with the
# commit they were measured at; the JSON line carries that commit ("traffic_measured_at") so that a figure older
# than a kernel change can be told. A missing file gives traffic = null.
def load_traffic():
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            d = json.load(f)
        return d.get("bytes_per_launch", {}), d.get("measured_at_commit")
    except (OSError, ValueError):
        return {}, None


TRAFFIC, TRAFFIC_COMMIT = load_traffic()


class Budget:
    """Wall-clock budget of the whole run, started when main() starts."""

    def __init__(self, seconds):
        self.t0 = time.perf_counter()
        self.seconds = float(seconds)

    def elapsed(self):
        return time.perf_counter() - self.t0

    def spent(self):
        return self.elapsed() >= self.seconds


SKIPPED = {"skipped": "time budget"}


def cpu_info():
    """(threads torch uses, os.cpu_count(), CPU model string)."""
    import torch

    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return torch.get_num_threads(), os.cpu_count(), model


def cpu_median_seconds(fn, reps=3):
    """1 warm-up + `reps` timed repetitions of fn(), median wall-clock seconds."""
    fn()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2]


def cpu_threads():
    import torch

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    return torch.get_num_threads()


def cpu_baseline_prefill(c):
    """The reference's CPU path - a per-expert torch.matmul loop (dev/triton_groupGEMM/testing/unit_tests.py:49-55)
    in fp32 on the host cores - timed on the whole workload (all experts, all rows): 1 warm-up + 3 repetitions,
    median."""
    from oracle import oracle as O

    threads = cpu_threads()
    m_sizes = c["m_sizes"].tolist()
    rows = sum(m_sizes)
    N = c["w"].shape[0] // len(m_sizes)
    K = c["w"].shape[1]
    x = c["x_sorted"].float()
    w = c["w"].float()
    t = cpu_median_seconds(lambda: O.grouped_gemm_torch_loop(x, w, m_sizes))
    _, ncpu, model = cpu_info()
    return {
        "value": round(2.0 * rows * N * K / t / 1e12, 3),
        "unit": "TFLOP/s",
        "cores": threads,
        "os_cpu_count": ncpu,
        "cpu_model": model,
        "kind": "port",
        "seconds": round(t, 3),
        "extrapolated": False,
        "sample": f"the whole workload ({rows} rows, {len(m_sizes)} experts), fp32 per-expert torch.matmul loop, 1 warm-up + 3 repetitions, median",
    }


def cpu_baseline_decode(m_sizes, K, N):
    """Per-expert fp32 torch.matmul loop at the decode shape (weights pre-converted to fp32, distinct per expert)."""
    import torch
    from oracle import oracle as O

    threads = cpu_threads()
    G = len(m_sizes)
    gen = torch.Generator().manual_seed(3)
    base = torch.randn(N, K, generator=gen) * 0.02
    w = torch.empty(G * N, K)
    for g in range(G):
        w[g * N:(g + 1) * N] = base * (1.0 + 0.01 * g)
    x = torch.randn(sum(m_sizes), K, generator=gen)
    t = cpu_median_seconds(lambda: O.grouped_gemm_torch_loop(x, w, m_sizes))
    active = sum(1 for m in m_sizes if m > 0)
    byt = active * N * K * 4 + sum(m_sizes) * (K + N) * 4
    return {"value": round(byt / t / 1e9, 2), "unit": "GB/s", "bytes": "fp32 operands as the CPU reads them", "cores": threads,
            "kind": "port", "seconds": round(t, 4), "extrapolated": False,
            "sample": "the whole workload, fp32 per-expert torch.matmul loop, 1 warm-up + 3 repetitions, median"}


def cpu_baseline_w4a16(M, K, N):
    """Dequantise (closed form of splitk_dequant_gemm.py:56-77) inside the timed region, then torch.matmul, fp32."""
    import torch
    from oracle import oracle as O

    threads = cpu_threads()
    gen = torch.Generator().manual_seed(4)
    qw = torch.randint(-2**31, 2**31 - 1, (K // 8, N), dtype=torch.int32, generator=gen)
    sc = torch.rand(K // 128, N, generator=gen) * 0.015 + 0.005
    qz = torch.randint(-2**31, 2**31 - 1, (K // 128, N // 8), dtype=torch.int32, generator=gen)
    a = torch.randn(M, K, generator=gen)
    t = cpu_median_seconds(lambda: O.w4a16_torch(a, qw, sc, qz, 128, 0))
    byt = K * N // 2 + (K // 128) * N * 2 + (K // 128) * N // 2 + M * K * 2 + M * N * 2
    return {"value": round(byt / t / 1e9, 3), "unit": "GB/s", "bytes": "the GPU path's algorithmic bytes", "cores": threads,
            "kind": "port", "seconds": round(t, 4), "extrapolated": False,
            "sample": "the whole workload, dequantisation inside the timed region + torch.matmul, 1 warm-up + 3 repetitions, median"}


def cpu_baseline_fp8_block(xq, wq, xs, ws, m_sizes, N, K, n_experts=32, defer=False):
    """Config 5 on the host cores: the first `n_experts` non-empty experts (the most popular ones under the Zipf
    routing come first), dequantisation with the block scales inside the timed per-expert loop, scaled to the whole
    workload by FLOPs. xq / wq / xs / ws are the GPU tensors of the timed launch; only the sample is copied. With
    defer the copy is made now and a function is returned that does the timing later (the GPU tensors can be freed)."""
    import torch
    from oracle import oracle as O

    sizes = [int(m) for m in m_sizes]
    take, seen = 0, 0
    for m in sizes:
        if seen == n_experts:
            break
        take += 1
        seen += m > 0
    sample = sizes[:take]
    rows = sum(sample)
    xq_h = xq[:rows].view(torch.uint8).cpu()
    xs_h = xs[:rows].cpu()
    wq_h = wq[:take * N].view(torch.uint8).cpu()
    ws_h = ws[:take * N // 128].cpu()

    def timed():
        threads = cpu_threads()
        t = cpu_median_seconds(lambda: O.grouped_gemm_fp8_block_torch_loop(xq_h, wq_h, xs_h, ws_h, sample, N))
        flop_sample = 2.0 * rows * N * K
        flop_all = 2.0 * sum(sizes) * N * K
        return {"value": round(flop_sample / t / 1e12, 3), "unit": "TFLOP/s", "cores": threads, "kind": "port",
                "seconds": round(t, 3), "extrapolated": True,
                "seconds_whole_workload_by_flops": round(t * flop_all / flop_sample, 3),
                "sample": f"first {seen} non-empty experts of {len(sizes)} ({rows} of {sum(sizes)} rows, {100.0 * flop_sample / flop_all:.0f} % of the FLOPs), "
                          "per-expert dequantise + torch.matmul, 1 warm-up + 3 repetitions, median"}

    return timed if defer else timed()


def cpu_baseline_w4a16_grouped(m_sizes, K, N, n_experts=2):
    """The grouped W4A16 call on the host cores: the first `n_experts` experts that have rows, dequantisation inside
    the timed per-expert loop, scaled to all experts with rows by the weight bytes they stream."""
    import torch
    from oracle import oracle as O

    threads = cpu_threads()
    sizes = [int(m) for m in m_sizes]
    take, seen = 0, 0
    for m in sizes:
        if seen == n_experts:
            break
        take += 1
        seen += m > 0
    sample = sizes[:take]
    active = sum(1 for m in sizes if m > 0)
    gen = torch.Generator().manual_seed(5)
    qw = torch.randint(-2**31, 2**31 - 1, (take, K // 8, N), dtype=torch.int32, generator=gen)
    sc = torch.rand(take, K // 128, N, generator=gen) * 0.015 + 0.005
    qz = torch.randint(-2**31, 2**31 - 1, (take, K // 128, N // 8), dtype=torch.int32, generator=gen)
    a = torch.randn(sum(sample), K, generator=gen)
    t = cpu_median_seconds(lambda: O.w4a16_grouped_torch_loop(a, qw, sc, qz, sample, 128, 0))
    per_expert = K * N // 2 + (K // 128) * N * 2 + (K // 128) * N // 2
    byt = seen * per_expert + sum(sample) * (K + N) * 2
    return {"value": round(byt / t / 1e9, 3), "unit": "GB/s", "bytes": "the GPU path's algorithmic bytes", "cores": threads,
            "kind": "port", "seconds": round(t, 4), "extrapolated": True,
            "seconds_whole_workload_by_bytes": round(t * active / max(seen, 1), 4),
            "sample": f"first {seen} of the {active} experts that have rows, per-expert dequantise + torch.matmul, "
                      "1 warm-up + 3 repetitions, median"}


def cpu_baseline_moe_layer(T, K, n, E, topk, sample_tokens=1024):
    """The MoE layer on the host cores as the reference's torch_moe states it (test_moe_gemm.py:16-30; per-expert fp32
    torch.matmul loop): the first `sample_tokens` tokens against all experts' weights, scaled to T tokens by FLOPs."""
    import torch
    from oracle import oracle as O

    threads = cpu_threads()
    Ts = min(T, sample_tokens)
    gen = torch.Generator().manual_seed(6)
    a = torch.randn(Ts, K, generator=gen) / 10
    w1 = torch.empty(E, 2 * n, K)
    w2 = torch.empty(E, K, n)
    b1 = torch.randn(2 * n, K, generator=gen) * 0.02     # one draw, a distinct scaled copy per expert: timing only
    b2 = torch.randn(K, n, generator=gen) * 0.02
    for ex in range(E):
        torch.mul(b1, 1.0 + 0.01 * ex, out=w1[ex])
        torch.mul(b2, 1.0 + 0.01 * ex, out=w2[ex])
    del b1, b2
    score = torch.softmax(torch.randn(Ts, E, generator=gen), dim=-1)
    tw, ids = torch.topk(score, topk)
    t = cpu_median_seconds(lambda: O.fused_moe_torch(a, w1, w2, tw, ids))
    flop_sample = 2.0 * Ts * topk * (2 * n * K + K * n)
    return {"value": round(flop_sample / t / 1e12, 3), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "seconds": round(t, 3), "extrapolated": Ts < T, "seconds_whole_workload_by_flops": round(t * T / Ts, 3),
            "sample": f"{Ts} of {T} tokens through all {E} experts (per-expert fp32 torch.matmul loop, SiLU-and-mul and "
                      "top-k combine in torch), 1 warm-up + 3 repetitions, median"}


def cpu_baseline_backward(m_sizes, N, K, n_experts=2):
    """Both gradients on the host cores (per-expert fp32 torch.matmul loop, pytorch_reference_backwards.py:165-197):
    the first `n_experts` experts, scaled to the whole workload by FLOPs."""
    import torch
    from oracle import oracle as O

    threads = cpu_threads()
    sizes = [int(m) for m in m_sizes]
    sample = sizes[:n_experts]
    rows = sum(sample)
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(rows, K, generator=gen) / 8
    w = torch.randn(len(sample) * N, K, generator=gen) * 0.02
    go = torch.randn(rows, N, generator=gen) / 8
    t = cpu_median_seconds(lambda: O.grouped_gemm_backward_torch_loop(go, x, w, sample))
    flop_sample = 4.0 * rows * N * K
    flop_all = 4.0 * sum(sizes) * N * K
    return {"value": round(flop_sample / t / 1e12, 3), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "seconds": round(t, 3), "extrapolated": len(sample) < len(sizes),
            "seconds_whole_workload_by_flops": round(t * flop_all / flop_sample, 3),
            "sample": f"first {len(sample)} experts of {len(sizes)} ({rows} of {sum(sizes)} rows), grad_x and grad_w by "
                      "per-expert fp32 torch.matmul, 1 warm-up + 3 repetitions, median"}


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
    return event_stats(torch, fn, iters, warmup, batches=1)["avg"]


def event_stats(torch, fn, iters, warmup, batches=5):
    """Durations of fn() in milliseconds from HIP events on the current stream: `batches` batches of
    iters // batches back-to-back calls each, one event pair per batch (an event pair per launch would cost more than
    the microsecond kernels it brackets). Returns the per-launch time of every batch as avg / p50 / p20 / p80."""
    settle(torch, fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    per = max(1, iters // batches)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(batches)]
    for s_ev, e_ev in ev:
        s_ev.record()
        for _ in range(per):
            fn()
        e_ev.record()
    torch.cuda.synchronize()
    t = sorted(s_ev.elapsed_time(e_ev) / per for s_ev, e_ev in ev)
    n = len(t)
    return {"avg": sum(t) / n, "p50": t[n // 2], "p20": t[n // 5], "p80": t[min(n - 1, (n * 4) // 5)],
            "batches": n, "launches_per_batch": per}


def timing_fields(st, unit):
    """JSON fields for an event_stats result; unit "us" or "ms" per launch."""
    k = 1e3 if unit == "us" else 1.0
    nd = 2 if unit == "us" else 3
    return {f"{unit}_per_launch": round(st["p50"] * k, nd), f"{unit}_p20": round(st["p20"] * k, nd),
            f"{unit}_p80": round(st["p80"] * k, nd), f"{unit}_avg": round(st["avg"] * k, nd),
            "timing": f"median (p20, p80) over {st['batches']} batches of {st['launches_per_batch']} back-to-back launches, HIP events"}


def hbm_roofline(kernel, byt, ms, traffic_key):
    gbs = byt / ms / 1e6
    return {"bound": "hbm", "kernel": kernel, "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": round(gbs / PEAK_HBM_GBS, 4), "traffic": TRAFFIC.get(traffic_key)}


# The secondary workloads: decode (config 3), W4A16 (config 4) and fp8 block-scaled (config 5) shapes are HBM-bound
# kernels, reported as GB/s of algorithmic bytes against the 8 TB/s HBM peak; the MoE layer and the backward pass as
# TFLOP/s. Weights rotate over enough distinct copies that the footprint exceeds the 256 MB Infinity Cache. Calls go
# straight through the C ABI so that the ~10 us kernels are not timed through Python allocation overhead. Every
# workload is a function of its own returning a list of JSON entries; one that raises is reported as an "error" entry
# and the others still run.
def wl_decode(torch, A, dev, lib, stream, cpu, shapes=((4096, 14336), (14336, 4096))):
    """shapes: (K, N) of the up- and the down-projection (the benchmark's by default; tests pass small ones)."""
    from applied_ai_amd import configs

    out = []
    c3 = configs.cfg3()
    m_sizes = c3["m_sizes"].tolist()
    ms_dev = c3["m_sizes"].to(dev)
    G, R = len(m_sizes), sum(m_sizes)
    active = sum(1 for m in m_sizes if m > 0)
    for (name, key), (K, N) in zip((("up-proj", "decode_up"), ("down-proj", "decode_down")), shapes):
        name = f"{name} K={K} N={N}"
        x = torch.randn(R, K, device=dev).to(torch.bfloat16)
        ws = [(torch.randn(G * N, K, device=dev) * 0.02).to(torch.bfloat16) for _ in range(2)]
        y = torch.empty(R, N, device=dev, dtype=torch.bfloat16)
        state = {"i": 0}

        def call():
            w = ws[state["i"] & 1]
            state["i"] += 1
            lib.moe_gg_grouped_gemm_bf16(x.data_ptr(), w.data_ptr(), y.data_ptr(), ms_dev.data_ptr(), G, R, N, K, N, 0, stream)

        st = event_stats(torch, call, 40, 6)
        ms = st["p50"]
        byt = active * N * K * 2 + R * K * 2 + R * N * 2
        e = {"workload": f"Mixtral decode bf16, T=32 top-2 ({R} rows, m_sizes {m_sizes}), {name}"}
        e.update(timing_fields(st, "us"))
        e.update({"value": round(byt / ms / 1e6, 1), "unit": "GB/s", "roofline": hbm_roofline("gg_bf16_decode", byt, ms, key)})
        del ws
        if cpu:
            e["_cpu"] = lambda m_sizes=m_sizes, K=K, N=N: cpu_baseline_decode(m_sizes, K, N)
        out.append(e)
    return out


def wl_w4a16(torch, A, dev, lib, stream, cpu, K=4096, N=14336, copies=12):
    out = []
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

        st = event_stats(torch, call, 120, 24)
        ms = st["p50"]

        def call_hot():  # always the same 29 MB of weights: they stay in the 256 MB last-level cache
            lib.moe_gg_w4a16_splitk(a.data_ptr(), qws[0].data_ptr(), sc.data_ptr(), qz.data_ptr(), c.data_ptr(), M, N, K, 128, 0, 0, stream)

        ms_hot = event_stats(torch, call_hot, 120, 24)["p50"]
        byt = K * N // 2 + (K // 128) * N * 2 + (K // 128) * N // 2 + M * K * 2 + M * N * 2
        e = {"workload": f"W4A16 split-K M={M} K={K} N={N} group 128"}
        e.update(timing_fields(st, "us"))
        e.update({"cache_hot_us_per_launch": round(ms_hot * 1e3, 2), "value": round(byt / ms / 1e6, 1), "unit": "GB/s",
                  "roofline": hbm_roofline("w4a16_splitk_g128", byt, ms, f"w4a16_m{M}")})
        if cpu:
            e["_cpu"] = lambda M=M: cpu_baseline_w4a16(M, K, N)
        out.append(e)
    return out


def wl_w4a16_grouped(torch, A, dev, lib, stream, cpu, K=4096, N=14336):
    from applied_ai_amd import configs

    out = []
    E = 8
    c3 = configs.cfg3()
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

    st = event_stats(torch, call, 40, 6)
    ms = st["p50"]
    act = sum(1 for m in c3["m_sizes"].tolist() if m > 0)
    byt = act * (K * N // 2 + K // 128 * N * 2 + K // 128 * N // 2) + 64 * K * 2 + 64 * N * 2
    e = {"workload": f"W4A16 grouped GEMM (int4 experts), Mixtral decode: 64 rows over 8 experts, K={K} N={N} group 128"}
    e.update(timing_fields(st, "us"))
    e.update({"value": round(byt / ms / 1e6, 1), "unit": "GB/s",
              "roofline": hbm_roofline("w4a16_splitk_g128 (grid.y = experts)", byt, ms, "w4a16_grouped")})
    if cpu:
        sizes3 = c3["m_sizes"].tolist()
        e["_cpu"] = lambda: cpu_baseline_w4a16_grouped(sizes3, K, N)
    out.append(e)

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

    st_q = event_stats(torch, call_q, 40, 6)
    ms_q = st_q["p50"]
    ms_two = event_stats(torch, call_two, 40, 6)["p50"]
    byt_q = byt - 64 * N * 2 + 64 * N + 64 * (N // 128) * 4
    e = {"workload": "W4A16 grouped GEMM with the fp8 1x128 quantiser as epilogue, same shape (fp8 codes + scales out)"}
    e.update(timing_fields(st_q, "us"))
    e.update({"gemm_then_quantiser_us": round(ms_two * 1e3, 2), "value": round(byt_q / ms_q / 1e6, 1), "unit": "GB/s",
              "roofline": hbm_roofline("w4a16_splitk_g128 (fp8 output)", byt_q, ms_q, "w4a16_grouped_fp8out")})
    out.append(e)
    return out


def wl_fp8_cfg5(torch, A, dev, lib, stream, cpu, m5=None, N=4096, K=7168):
    """Config 5 with the inputs its definition states: x ~ N(0, 1) through the 1 x 128 quantiser, weights ~ N(0, 0.02)
    through the 128 x 128 block quantiser (drawn and quantised expert by expert to bound memory). m5 / N / K: the
    benchmark's routing and shape by default (tests pass small ones)."""
    from applied_ai_amd import configs

    if m5 is None:
        _, _, _, m5 = configs.cfg5_routing()
    G = int(m5.shape[0])
    M = int(m5.sum())
    f8 = torch.float8_e4m3fn
    gen = torch.Generator(device=dev).manual_seed(1005)
    xq, xs = A.float8_groupwise_quantize(torch.randn(M, K, generator=gen, device=dev))
    wq = torch.empty(G * N, K, dtype=f8, device=dev)
    ws = torch.empty(G * N // 128, K // 128, dtype=torch.float32, device=dev)
    for g in range(G):
        q, sc = A.float8_blockwise_quantize_weight(torch.randn(N, K, generator=gen, device=dev) * 0.02)
        wq.view(torch.uint8)[g * N:(g + 1) * N] = q.view(torch.uint8)     # a byte copy: no fp8 copy kernel needed
        ws[g * N // 128:(g + 1) * N // 128] = sc
    y = torch.empty(M, N, device=dev, dtype=torch.bfloat16)
    ms_dev = m5.to(torch.int32).to(dev)

    def call():
        lib.moe_gg_grouped_gemm_fp8(xq.data_ptr(), wq.data_ptr(), y.data_ptr(), xs.data_ptr(), ws.data_ptr(), 1,
                                    ms_dev.data_ptr(), G, M, N, K, N, 0, stream)

    st = event_stats(torch, call, 10, 2, batches=5)
    ms = st["p50"]
    active = int((m5 > 0).sum())
    byt = M * K + active * N * K + M * N * 2 + M * (K // 128) * 4 + active * (N // 128) * (K // 128) * 4
    flop = 2.0 * M * N * K
    e = {"workload": f"DeepSeek-V3-style fp8 e4m3 block-scaled grouped GEMM: {G} experts top-8, T=4096 ({M} rows, Zipf 1.1), K={K}, N={N}; "
                     "x ~ N(0,1) through the 1x128 quantiser, w ~ N(0,0.02) through the 128x128 block quantiser"}
    e.update(timing_fields(st, "ms"))
    e.update({"value": round(byt / ms / 1e6, 1), "unit": "GB/s", "tflops": round(flop / ms / 1e9, 1),
              "roofline": hbm_roofline("gg_fp8_pingpong_block", byt, ms, "fp8_block_cfg5")})
    if cpu:
        e["_cpu"] = cpu_baseline_fp8_block(xq, wq, xs, ws, m5.tolist(), N, K, defer=True)
    return [e]


def wl_moe_layer(torch, A, dev, lib, stream, cpu, T=4096, K=4096, n=14336):
    E, topk = 8, 2
    gen = torch.Generator(device=dev).manual_seed(1002)
    h = (torch.randn(T, K, device=dev, generator=gen) / 10).to(torch.bfloat16)
    w1 = torch.empty(E, 2 * n, K, device=dev, dtype=torch.bfloat16)
    w2 = torch.empty(E, K, n, device=dev, dtype=torch.bfloat16)
    for ex in range(E):
        w1[ex] = (torch.randn(2 * n, K, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
        w2[ex] = (torch.randn(K, n, device=dev, generator=gen) * 0.02).to(torch.bfloat16)
    score = torch.softmax(torch.randn(T, E, device=dev, generator=gen), dim=-1)
    tw, ids = torch.topk(score, topk)
    ids = ids.to(torch.int32)
    st = event_stats(torch, lambda: A.fused_moe(h, w1, w2, tw, ids), 10, 3, batches=5)
    ms = st["p50"]
    flop = 2.0 * T * topk * (2 * n * K + K * n)
    e = {"workload": f"Mixtral 8x7B MoE layer (fused_moe: group, gather, w1 GEMM, SiLU-and-mul, w2 GEMM, top-2 combine), T={T}, K={K}, n={n}, bf16",
         "m_sizes": torch.bincount(ids.flatten().long(), minlength=E).tolist()}
    e.update(timing_fields(st, "ms"))
    e.update({"value": round(flop / ms / 1e9, 1), "unit": "TFLOP/s",
              "roofline": {"bound": "mfma", "kernel": "gg_bf16_pingpong (two launches) + glue kernels", "achieved": round(flop / ms / 1e9, 1),
                           "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                           "traffic": None}})
    if cpu:
        e["_cpu"] = lambda: cpu_baseline_moe_layer(T, K, n, E, topk)
    return [e]


def wl_backward(torch, A, dev, lib, stream, cpu, sizes=(1012, 1039, 1048, 1036, 998, 1023, 1040, 996), N=14336, K=4096):
    """sizes: rows per expert (config 2's routing by default; tests pass small ones)."""
    G, M = len(sizes), sum(sizes)
    gen = torch.Generator(device=dev).manual_seed(1002)
    ms_dev = torch.tensor(list(sizes), dtype=torch.int32, device=dev)
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

    st = event_stats(torch, call, 10, 2, batches=5)
    ms = st["p50"]
    flop = 4.0 * M * N * K
    e = {"workload": f"grouped GEMM backward (grad_x and grad_w), Mixtral 8x7B w1 shape: {M} rows, K={K}, N={N}, {G} experts, bf16"}
    e.update(timing_fields(st, "ms"))
    e.update({"value": round(flop / ms / 1e9, 1), "unit": "TFLOP/s",
              "roofline": {"bound": "mfma", "kernel": "gg_bf16_pingpong_nt + gg_bf16_pingpong_wgrad_direct",
                           "achieved": round(flop / ms / 1e9, 1), "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                           "frac": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "traffic": None}})
    if cpu:
        e["_cpu"] = lambda: cpu_baseline_backward(list(sizes), N, K)
    return [e]


def wl_moe_sweep(torch, A, dev, lib, stream, cpu, n=7168, k=4096, tokens=(1, 2, 4, 8, 16, 32, 64, 128, 256, 512)):
    """Context only, not a target: the sweep behind the one table of numbers the reference publishes for a
    neighbouring kernel (kernels/triton/inference/col_major_moe_gemm/test.csv:1-11): the fused MoE layer at
    m = 1 ... 512 tokens, n = 7168, k = 4096, 8 experts, top-2, fp16, reported with the reference's own formula
    2 m n k / t (perf_test_moe.py:123), which counts one m x n x k GEMM for the whole two-GEMM layer."""
    E, topk = 8, 2
    gen = torch.Generator(device=dev).manual_seed(3227)
    w1 = (torch.randn(E, 2 * n, k, device=dev, generator=gen) / 10).to(torch.float16)
    w2 = (torch.randn(E, k, n, device=dev, generator=gen) / 10).to(torch.float16)
    rows = []
    for m in tokens:
        a = (torch.randn(m, k, device=dev, generator=gen) / 10).to(torch.float16)
        score = torch.softmax(torch.randn(m, E, device=dev, generator=gen), dim=-1)
        tw, ids = torch.topk(score, topk)
        ids = ids.to(torch.int32)
        st = event_stats(torch, lambda: A.fused_moe(a, w1, w2, tw, ids), 40, 8)
        rows.append({"m": m, "us": round(st["p50"] * 1e3, 1), "tflops_reference_formula": round(2.0 * m * n * k / st["p50"] / 1e9, 3)})
    return [{"workload": f"fused_moe sweep as the reference's perf_test_moe.py runs it: n={n}, k={k}, 8 experts, top-2, fp16; "
                         "TFLOPS = 2 m n k / t (one GEMM counted for the whole layer); context for test.csv:1-11, not a target",
             "timing": "median over 5 batches of 8 back-to-back calls through the Python entry function, HIP events",
             "rows": rows}]


SECONDARY = (wl_decode, wl_w4a16, wl_w4a16_grouped, wl_fp8_cfg5, wl_moe_layer, wl_backward)
# Context entries (only with --moe-sweep).
OPTIONAL = (wl_moe_sweep,)


def secondary_workloads(torch, A, dev, cpu=True, optional=False, budget=None, out=None):
    """The GPU legs of the secondary workloads, appended to `out` as they finish. With cpu, an entry may carry its CPU
    baseline as a function under "_cpu": run_cpu_baselines() calls it once every GPU leg is done."""
    lib = A._lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    out = [] if out is None else out
    for wl in SECONDARY + (OPTIONAL if optional else ()):
        if budget is not None and budget.spent():
            out.append({"workload": wl.__name__, **SKIPPED})
            continue
        try:
            out.extend(wl(torch, A, dev, lib, stream, cpu))
        except Exception as exc:  # one workload failing must not lose the line
            out.append({"workload": wl.__name__, "error": f"{type(exc).__name__}: {exc}"})
        torch.cuda.empty_cache()
    return out


def run_cpu_baselines(entries, budget=None):
    """Replaces the "_cpu" function of every entry by its result under "cpu_baseline", in order; once the budget is
    spent the remaining ones are marked skipped."""
    for e in entries:
        fn = e.pop("_cpu", None)
        if fn is None:
            continue
        if budget is not None and budget.spent():
            e["cpu_baseline"] = dict(SKIPPED)
            continue
        try:
            e["cpu_baseline"] = fn()
        except Exception as exc:
            e["cpu_baseline"] = {"error": f"{type(exc).__name__}: {exc}"}


def printable(out):
    """The JSON line for `out`: baselines that have not run yet are marked as such."""
    def clean(e):
        if isinstance(e, dict):
            d = {k: clean(v) for k, v in e.items() if k != "_cpu"}
            if "_cpu" in e:
                d["cpu_baseline"] = {"skipped": "interrupted before it ran"}
            return d
        if isinstance(e, list):
            return [clean(v) for v in e]
        return e

    return json.dumps(clean(out))


# moe_gg_set_variant ops by name (include/moe_gg.h) and the headline kernel behind each MOE_GG_OP_GG_BF16 variant
PIN_OPS = {"gg_bf16": 0, "gg_fp8": 1, "tile_order": 2, "w4a16": 3}
HEADLINE_KERNELS = {-1: "gg_bf16_pingpong", 0: "gg_bf16_pingpong", 1: "gg_bf16_persistent<256x256>", 2: "gg_bf16_persistent<128x128>",
                    3: "gg_bf16_persistent<64x128>", 4: "gg_bf16_generic", 5: "gg_bf16_decode",
                    6: "gg_bf16_persistent<256x256, four waves>", 7: "gg_bf16_fourwave", 8: "gg_bf16_fourwave_tall"}


def parse_pins(items):
    """{"op name": variant} from --pin OP=VARIANT arguments."""
    pins = {}
    for item in items:
        op, sep, variant = item.partition("=")
        if not sep or op not in PIN_OPS:
            sys.exit(f"--pin {item}: expected OP=VARIANT with OP one of {', '.join(PIN_OPS)}")
        try:
            pins[op] = int(variant)
        except ValueError:
            sys.exit(f"--pin {item}: VARIANT must be an integer")
    return pins


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true")
    ap.add_argument("--moe-sweep", action="store_true",
                    help="also run the fused_moe sweep over m = 1 ... 512 (the shape of the reference's published sweep; context only)")
    ap.add_argument("--no-moe-sweep", action="store_true", help="accepted for compatibility: the sweep is off unless --moe-sweep is given")
    ap.add_argument("--budget-s", type=float, default=300.0,
                    help="wall-clock budget: secondary workloads and CPU baselines that would start after it are reported as skipped")
    ap.add_argument("--pin", action="append", default=[], metavar="OP=VARIANT",
                    help="pin a kernel variant for the whole run (moe_gg_set_variant): OP is gg_bf16, gg_fp8, tile_order or w4a16; "
                         "for timing and profiling the selectable kernels, e.g. --pin gg_bf16=7 --pin tile_order=1. The line says what was pinned")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy, so that a rocprofv3 --pmc run of this command sees a kernel of known traffic")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    budget = Budget(args.budget_s)
    pins = parse_pins(args.pin)
    if pins:
        TRAFFIC.clear()   # the committed traffic figures were measured on the library's automatic choice of kernels

    import signal

    import torch

    import applied_ai_amd as A
    from applied_ai_amd import configs

    out = {}

    def on_signal(signum, frame):  # a driver's time limit: print what has been measured, then leave
        if out:
            out["interrupted_by_signal"] = signum
            print(printable(out), flush=True)
        os._exit(128 + signum)

    signal.signal(signal.SIGTERM, on_signal)
    signal.signal(signal.SIGINT, on_signal)

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    for op, variant in pins.items():
        rc = A._lib.lib().moe_gg_set_variant(PIN_OPS[op], variant)
        assert rc == 0, (op, variant, rc)
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

    out.update({
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
            "kernel": HEADLINE_KERNELS.get(pins.get("gg_bf16", 0), f"gg_bf16 variant {pins.get('gg_bf16')}"),
            "achieved": round(achieved, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            "traffic": TRAFFIC.get("prefill_cfg2"),
            "kernel_ms": {"avg": round(avg_kernel_ms, 4), "p20": round(kern_ms[len(kern_ms) // 5], 4),
                          "p50": round(kern_ms[len(kern_ms) // 2], 4), "p80": round(kern_ms[(len(kern_ms) * 4) // 5], 4)},
        },
    })
    # Context for the roofline fraction: the vendor library's dense bf16 GEMM of the same FLOP count and data
    # (one [8192, 4096] x [4096, 14336] product through torch.matmul -> hipBLASLt), timed the same way. With
    # random operands the MFMA clock is power-limited well below the 2.5 PFLOP/s figure, for the library too.
    wd = w[:N]
    try:
        lib_ms = event_time_ms(torch, lambda: torch.matmul(x, wd.t()), 20, 5)
        out["dense_gemm_library"] = {"value": round(2.0 * x.shape[0] * N * K / lib_ms / 1e9, 1), "unit": "TFLOP/s",
                                     "what": "torch.matmul (hipBLASLt) bf16 [8192,4096]x[4096,14336], same FLOPs, no grouping"}
    except Exception as exc:
        out["dense_gemm_library"] = {"error": f"{type(exc).__name__}: {exc}"}
    del x, w, y, wd
    if args.copy_calibration:
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    out["traffic_measured_at"] = TRAFFIC_COMMIT
    if pins:
        # not the library's automatic choice: the figures of this line belong to the pinned kernels
        out["pinned_variants"] = pins
    cpu = not args.no_cpu_baseline
    if cpu:
        out["_cpu"] = lambda: cpu_baseline_prefill(c)
    if not args.no_secondary:
        out["secondary"] = []
        secondary_workloads(torch, A, dev, cpu=cpu, optional=args.moe_sweep, budget=budget, out=out["secondary"])
    # every GPU number is in `out` now: the CPU baselines follow, the headline's first
    run_cpu_baselines([out] + out.get("secondary", []), budget)
    out["wall_s"] = round(budget.elapsed(), 1)
    out["budget_s"] = args.budget_s
    print(printable(out))


if __name__ == "__main__":
    main()
