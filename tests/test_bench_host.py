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
