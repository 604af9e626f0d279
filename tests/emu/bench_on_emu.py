"""bench.py executed on the CPU against the emulated library (see gpu_tests_on_emu.py), at sizes the emulation carries:
main() with a small stand-in for the headline configuration and every secondary workload function at a reduced shape,
CPU baselines included. Prints the JSON line main() printed. What it checks is bench.py's own code - tensor shapes,
ctypes argument lists, the JSON fields - not speed. Test infrastructure only.

    python tests/emu/bench_on_emu.py [further bench.py arguments, e.g. --pin gg_bf16=7 --pin w4a16=7]
"""
import functools
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, HERE):
    if p not in sys.path:
        sys.path.insert(0, p)

import gpu_tests_on_emu  # noqa: E402


def main():
    gpu_tests_on_emu.install()
    import signal

    import torch

    import bench
    from applied_ai_amd import configs

    bench.SETTLE_SECONDS = 0.0
    signal.signal = lambda *a: None          # main() installs handlers; not wanted here
    G, N, K = 3, 256, 128
    sizes = [300, 0, 70]
    gen = torch.Generator().manual_seed(1)
    small = {"x_sorted": torch.randn(sum(sizes), K, generator=gen).to(torch.bfloat16),
             "w": (torch.randn(G * N, K, generator=gen) * 0.02).to(torch.bfloat16),
             "m_sizes": torch.tensor(sizes, dtype=torch.int32)}
    configs.cfg2 = lambda: small
    m5 = torch.tensor([70, 0, 300, 5, 1, 130], dtype=torch.int64)
    bench.SECONDARY = (
        functools.partial(bench.wl_decode, shapes=((256, 128), (128, 256))),
        functools.partial(bench.wl_w4a16, K=256, N=128, copies=2),
        functools.partial(bench.wl_w4a16_grouped, K=256, N=128),
        functools.partial(bench.wl_fp8_cfg5, m5=m5, N=256, K=256),
        functools.partial(bench.wl_moe_layer, T=96, K=128, n=192),
        functools.partial(bench.wl_backward, sizes=(40, 0, 90), N=128, K=64),
    )
    bench.OPTIONAL = (functools.partial(bench.wl_moe_sweep, n=128, k=64, tokens=(1, 8)),)
    for f in bench.SECONDARY + bench.OPTIONAL:   # the error entry of a failing workload names the function
        f.__name__ = f.func.__name__
    sys.argv = ["bench.py", "--steps", "3", "--warmup", "1", "--moe-sweep"] + sys.argv[1:]   # e.g. --pin gg_bf16=7
    bench.main()


if __name__ == "__main__":
    main()
