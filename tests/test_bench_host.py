"""Host-side pieces of bench.py that need no GPU: the batch statistics (with the device events stubbed), the JSON
fields derived from them, the traffic table, and the CPU baselines on small shapes (they are the oracle's torch forms
timed; their values are checked against the scalar oracle in tests/test_oracle.py)."""
import json
import os
import time
import types

import torch

import bench


class _Event:
    def __init__(self, enable_timing=True):
        self.t = 0.0

    def record(self):
        self.t = time.perf_counter()

    def elapsed_time(self, other):
        return (other.t - self.t) * 1e3 + 1e-3


class _Torch:
    """torch with a cuda namespace that runs on the host."""
    cuda = types.SimpleNamespace(Event=_Event, synchronize=lambda: None, empty_cache=lambda: None)

    def __getattr__(self, k):
        return getattr(torch, k)


def test_event_stats_batches_and_percentiles(monkeypatch):
    monkeypatch.setattr(bench, "SETTLE_SECONDS", 0.0)
    calls = []
    st = bench.event_stats(_Torch(), lambda: calls.append(1), 10, 3, batches=5)
    assert st["batches"] == 5 and st["launches_per_batch"] == 2
    assert st["p20"] <= st["p50"] <= st["p80"] and st["avg"] > 0
    assert len(calls) >= 10 + 3            # settle loop + warm-up + timed launches
    one = bench.event_stats(_Torch(), lambda: None, 3, 0, batches=5)      # fewer launches than batches: one per batch
    assert one["launches_per_batch"] == 1
    assert bench.event_time_ms(_Torch(), lambda: None, 20, 5) > 0          # single batch: avg = p50


def test_timing_fields_and_roofline_entries():
    st = {"avg": 0.0101, "p50": 0.01, "p20": 0.0099, "p80": 0.0103, "batches": 5, "launches_per_batch": 24}
    us = bench.timing_fields(st, "us")
    assert us["us_per_launch"] == 10.0 and us["us_p20"] == 9.9 and us["us_p80"] == 10.3 and "5 batches of 24" in us["timing"]
    ms = bench.timing_fields({**st, "p50": 1.8444}, "ms")
    assert ms["ms_per_launch"] == 1.844
    r = bench.hbm_roofline("k", 8.0e9, 2.0, "no_such_key")
    assert r["achieved"] == 4000.0 and r["frac"] == 0.5 and r["traffic"] is None and r["peak"] == 8000.0


def test_traffic_table_is_the_committed_file():
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    d = json.load(open(os.path.join(root, "profiles", "traffic.json")))
    assert bench.TRAFFIC == d["bytes_per_launch"] and bench.TRAFFIC_COMMIT == d["measured_at_commit"]
    for key in ("prefill_cfg2", "decode_up", "decode_down", "w4a16_m1", "w4a16_m16", "w4a16_m64", "w4a16_grouped",
                "w4a16_grouped_fp8out", "fp8_block_cfg5"):
        assert bench.TRAFFIC[key] > 0


def test_cpu_baselines_on_small_shapes():
    b = bench.cpu_baseline_decode([3, 0, 5], 256, 128)
    assert b["unit"] == "GB/s" and b["value"] > 0 and b["extrapolated"] is False and b["cores"] >= 1
    b = bench.cpu_baseline_w4a16(4, 256, 128)
    assert b["value"] > 0 and "dequantisation inside the timed region" in b["sample"]
    # config-5 form: the first two non-empty experts of five, scaled by FLOPs
    sizes = [6, 0, 9, 4, 2]
    N, K = 128, 256
    rows = sum(sizes)
    xq = torch.randint(0, 120, (rows, K), dtype=torch.uint8).view(torch.float8_e4m3fn)
    wq = torch.randint(0, 120, (len(sizes) * N, K), dtype=torch.uint8).view(torch.float8_e4m3fn)
    b = bench.cpu_baseline_fp8_block(xq, wq, torch.ones(rows, K // 128), torch.ones(len(sizes) * N // 128, K // 128), sizes, N, K,
                                     n_experts=2)
    assert b["extrapolated"] is True and "first 2 non-empty experts of 5 (15 of 21 rows" in b["sample"]
    assert b["seconds_whole_workload_by_flops"] >= b["seconds"]


def test_a_failing_secondary_workload_is_reported_not_raised(monkeypatch):
    def boom(*a):
        raise RuntimeError("no device")

    monkeypatch.setattr(bench, "SECONDARY", (boom,))
    fake_a = types.SimpleNamespace(_lib=types.SimpleNamespace(lib=lambda: None))
    t = _Torch()
    t.cuda.current_stream = lambda: types.SimpleNamespace(cuda_stream=0)
    out = bench.secondary_workloads(t, fake_a, torch.device("cpu"))
    assert out == [{"workload": "boom", "error": "RuntimeError: no device"}]


def test_cpu_baselines_run_after_the_gpu_legs_and_stop_at_the_budget():
    order = []
    entries = [{"workload": "a", "_cpu": lambda: order.append("a") or {"value": 1}},
               {"workload": "b"},
               {"workload": "c", "_cpu": lambda: 1 / 0},
               {"workload": "d", "_cpu": lambda: order.append("d") or {"value": 4}}]
    bench.run_cpu_baselines(entries, bench.Budget(1000.0))
    assert order == ["a", "d"] and entries[0]["cpu_baseline"] == {"value": 1} and "cpu_baseline" not in entries[1]
    assert entries[2]["cpu_baseline"]["error"].startswith("ZeroDivisionError")
    assert all("_cpu" not in e for e in entries)
    # a spent budget: nothing runs, every pending baseline is marked
    late = [{"workload": "x", "_cpu": lambda: order.append("x")}]
    bench.run_cpu_baselines(late, bench.Budget(0.0))
    assert late == [{"workload": "x", "cpu_baseline": {"skipped": "time budget"}}] and "x" not in order
    # and the secondary GPU legs are not started either
    fake_a = types.SimpleNamespace(_lib=types.SimpleNamespace(lib=lambda: None))
    t = _Torch()
    t.cuda.current_stream = lambda: types.SimpleNamespace(cuda_stream=0)
    out = bench.secondary_workloads(t, fake_a, torch.device("cpu"), budget=bench.Budget(0.0))
    assert [e["workload"] for e in out] == [w.__name__ for w in bench.SECONDARY] and all(e["skipped"] == "time budget" for e in out)


def test_the_line_printed_on_a_signal_marks_baselines_that_have_not_run():
    out = {"value": 1.0, "_cpu": lambda: None, "secondary": [{"workload": "w", "_cpu": lambda: None}, {"workload": "v", "cpu_baseline": {"value": 2}}]}
    d = json.loads(bench.printable(out))
    assert d["cpu_baseline"] == {"skipped": "interrupted before it ran"} and d["secondary"][0]["cpu_baseline"]["skipped"]
    assert d["secondary"][1]["cpu_baseline"] == {"value": 2} and "_cpu" in out      # the original is untouched


def test_new_cpu_baselines_on_small_shapes():
    b = bench.cpu_baseline_w4a16_grouped([3, 0, 5, 2], 256, 128, n_experts=2)
    assert b["unit"] == "GB/s" and b["extrapolated"] is True and "first 2 of the 3 experts" in b["sample"]
    assert b["seconds_whole_workload_by_bytes"] >= b["seconds"]
    b = bench.cpu_baseline_moe_layer(64, 128, 64, 4, 2, sample_tokens=16)
    assert b["unit"] == "TFLOP/s" and b["extrapolated"] is True and "16 of 64 tokens" in b["sample"]
    b = bench.cpu_baseline_backward([5, 0, 7, 4], 64, 128, n_experts=2)
    assert b["extrapolated"] is True and "first 2 experts of 4 (5 of 16 rows)" in b["sample"]


def test_main_prints_one_line_with_the_gpu_numbers_first(monkeypatch, capsys):
    """main() end to end with the device stubbed (CPU tensors, host-clock events, a stand-in for the GEMM): the flow of
    the run - GPU legs, then CPU baselines, one JSON line with the fields the contract names."""
    import sys

    import applied_ai_amd as A
    from applied_ai_amd import configs

    import signal

    monkeypatch.setattr(signal, "signal", lambda *a: None)       # main() installs handlers: not in the test process
    monkeypatch.setattr(bench, "SETTLE_SECONDS", 0.0)
    monkeypatch.setattr(sys, "argv", ["bench.py", "--steps", "3", "--warmup", "1"])
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    monkeypatch.setattr(torch.cuda, "set_device", lambda d: None)
    monkeypatch.setattr(torch.cuda, "synchronize", lambda *a: None)
    monkeypatch.setattr(torch.cuda, "Event", _Event)
    monkeypatch.setattr(torch.cuda, "empty_cache", lambda: None)
    monkeypatch.setattr(torch.cuda, "current_stream", lambda *a: types.SimpleNamespace(cuda_stream=0))
    real_device = torch.device
    monkeypatch.setattr(torch, "device", lambda *a: real_device("cpu"))
    G, N, K, M = 2, 64, 32, 24
    small = {"x_sorted": torch.zeros(M, K, dtype=torch.bfloat16), "w": torch.zeros(G * N, K, dtype=torch.bfloat16),
             "m_sizes": torch.tensor([10, 14], dtype=torch.int32)}
    monkeypatch.setattr(configs, "cfg2", lambda: small)
    monkeypatch.setattr(A, "grouped_gemm", lambda x, w, ms: torch.zeros(x.shape[0], w.shape[0] // ms.shape[0]))
    seen = []

    def wl(torch_, A_, dev, lib, stream, cpu):
        seen.append("gpu leg")
        return [{"workload": "w", "value": 1.0, "_cpu": lambda: seen.append("cpu leg") or {"value": 0.5}}]

    monkeypatch.setattr(bench, "SECONDARY", (wl,))
    monkeypatch.setattr(A._lib, "lib", lambda: None)
    monkeypatch.setattr(bench, "cpu_baseline_prefill", lambda c: seen.append("headline cpu") or {"value": 0.1, "cores": 1})
    bench.main()
    lines = [ln for ln in capsys.readouterr().out.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    assert seen == ["gpu leg", "headline cpu", "cpu leg"]
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "secondary", "wall_s"):
        assert key in d, key
    assert d["steps"] == 3 and d["n_gpus"] == 1 and d["vs_baseline"] is None and d["config"]["m_sizes"] == [10, 14]
    assert d["roofline"]["bound"] == "mfma" and d["cpu_baseline"] == {"value": 0.1, "cores": 1}
    assert d["secondary"] == [{"workload": "w", "value": 1.0, "cpu_baseline": {"value": 0.5}}]


def test_pin_arguments():
    assert bench.parse_pins([]) == {}
    assert bench.parse_pins(["gg_bf16=7", "tile_order=1", "w4a16=5"]) == {"gg_bf16": 7, "tile_order": 1, "w4a16": 5}
    assert bench.HEADLINE_KERNELS[7] == "gg_bf16_fourwave" and set(bench.PIN_OPS.values()) == {0, 1, 2, 3}
    for bad in (["nothing=1"], ["gg_bf16"], ["gg_bf16=x"]):
        try:
            bench.parse_pins(bad)
        except SystemExit as e:
            assert "--pin" in str(e)
        else:
            raise AssertionError(bad)
