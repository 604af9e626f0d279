"""A selection of the `-m gpu` tests executed on the CPU (the uncollected first-run tests, tests/wip_*.py, pass the same way):
tests/emu/gpu_tests_on_emu.py loads the emulated build of the library in place of libmoe_gg.so and turns torch's "cuda"
tensors into CPU tensors, so the GPU tests' own code - input construction, the Python entry functions, the ctypes
calls, the oracle comparisons - runs end to end without a GPU. A mistake in a GPU test or in the host layer shows up
here instead of on the GPU box. The selection is what the emulation carries in about a minute; the whole GPU suite,
the benchmark-sized cases aside, passes the same way when given the time."""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "emu"))

import build_emu  # noqa: E402

if not os.path.exists(build_emu.CXX):
    pytest.skip("host clang++ of the ROCm toolchain not found: the emulated build needs it", allow_module_level=True)

FILES = ["tests/test_gpu_routing.py", "tests/test_gpu_w4a16.py", "tests/test_gpu_w4a16_moe.py", "tests/test_gpu_decode_bf16.py",
         "tests/test_zy_validate.py", "tests/test_gpu_moe_layer.py"]
# left out: benchmark-sized cases, and the tests of argument errors that need a real device to tell host from device memory
SKIP = ("not config4 and not mixtral and not invalid and not rejects and not errors and not reference_test_shape and not 1500 "
        "and not prefill_rows and not m_sizes5 and not sizes1-1032")


SMOKE = ("import sys; sys.path.insert(0, 'tests/emu'); sys.path.insert(0, '.'); import gpu_tests_on_emu as g; g.install(); "
         "import __graft_entry__ as e; e.smoke()")


@pytest.fixture(scope="module", autouse=True)
def children():
    """The three child processes of this file, started together when its first test runs."""
    build_emu.build()
    emu = os.path.join(ROOT, "tests", "emu")
    c = {"tests": subprocess.Popen([sys.executable, os.path.join(emu, "gpu_tests_on_emu.py")] + FILES + ["-k", SKIP], cwd=ROOT,
                                   stdout=subprocess.PIPE, stderr=subprocess.STDOUT),
         "bench": subprocess.Popen([sys.executable, os.path.join(emu, "bench_on_emu.py")], cwd=ROOT, stdout=subprocess.PIPE,
                                   stderr=subprocess.PIPE),
         "smoke": subprocess.Popen([sys.executable, "-c", SMOKE], cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)}
    yield c
    for p in c.values():
        if p.poll() is None:
            p.kill()


def test_gpu_tests_pass_against_the_emulated_library(children):
    p = children["tests"]
    log = p.communicate(timeout=1500)[0].decode()
    assert p.returncode == 0, log[-3000:]
    m = re.search(r"(\d+) passed", log)
    assert m and int(m.group(1)) >= 100, log[-1000:]


def test_bench_py_runs_end_to_end_against_the_emulated_library(children):
    """bench.py's main() and every secondary workload (with CPU baselines and the optional sweep) at reduced shapes,
    through the real ctypes calls into the emulated kernels: one JSON line with the contract's fields, no workload
    ending in an "error" entry, the baselines attached after the device legs."""
    import json

    p = children["bench"]
    out, err = p.communicate(timeout=1500)
    assert p.returncode == 0, err.decode()[-3000:]
    lines = [ln for ln in out.decode().splitlines() if ln.startswith("{")]
    assert len(lines) == 1, out.decode()[-2000:]
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline", "secondary", "dense_gemm_library", "wall_s"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["unit"] == "TFLOP/s" and d["vs_baseline"] is None
    assert {"bound", "achieved", "peak", "unit", "frac", "traffic"} <= set(d["roofline"])
    assert {"value", "unit", "cores", "kind", "sample"} <= set(d["cpu_baseline"])
    sec = d["secondary"]
    assert len(sec) == 11 and not any("error" in e or "skipped" in e for e in sec), [e for e in sec if "error" in e or "skipped" in e]
    with_roofline = [e for e in sec if "roofline" in e]
    assert len(with_roofline) == 10 and all(e["roofline"]["bound"] in ("hbm", "mfma") for e in with_roofline)
    assert sum("cpu_baseline" in e for e in sec) == 9          # all but the fp8-epilogue line and the sweep
    assert sec[-1]["rows"] and sec[-1]["rows"][0]["m"] == 1


def test_smoke_entry_point_against_the_emulated_library(children):
    """__graft_entry__.smoke() (one small grouped GEMM through the Python entry function, checked against the oracle)."""
    p = children["smoke"]
    log = p.communicate(timeout=600)[0].decode()
    assert p.returncode == 0 and "smoke ok" in log, log[-2000:]
