"""The selectable kernels at the full size of benchmark config 2 (8 experts, 8192 routed rows, N = 14336, K = 4096;
256 workgroups on 8 XCDs) under the CPU emulation, on small-integer data whose fp32 sums are exact, so the expected
bf16 output is known bit for bit. About 20 minutes per grouped-GEMM case and 40 per fused first GEMM on one core; run
by tests/test_emu_kernels.py::test_config2_at_full_size when EMU_FULL_SIZE is set. Test infrastructure only.

    EMU_CUS=256 EMU_TILE_ORDER=<0|1> python tests/emu/full_size.py gemm <variant>
    EMU_CUS=256 EMU_TILE_ORDER=<0|1> python tests/emu/full_size.py swiglu <variant>   (against the default kernel's bits)
"""
import os
import sys
import time

import numpy as np
import torch

import harness as H

SIZES = [1012, 1039, 1048, 1036, 998, 1023, 1040, 996]   # config 2's routing (seed 1002): four experts end 12-24 rows past a tile edge
N, K = 14336, 4096


def main(kind, variant):
    rng = np.random.default_rng(11)
    M = sum(SIZES)
    x = rng.integers(-2, 3, (M, K)).astype(np.float32)
    t = time.time()
    if kind == "gemm":
        w = rng.integers(-2, 3, (len(SIZES) * N, K)).astype(np.float32)
        ref = np.zeros((M, N), np.float32)
        r0 = 0
        for g, m in enumerate(SIZES):
            ref[r0:r0 + m] = (torch.from_numpy(x[r0:r0 + m]) @ torch.from_numpy(w[g * N:(g + 1) * N]).T).numpy()
            r0 += m
        y = H.grouped_gemm(H.to_bf16(x), H.to_bf16(w), SIZES, N, variant=variant)
        ok = bool((y == H.to_bf16(ref)).all())
    else:
        w = rng.integers(-2, 3, (len(SIZES) * 2 * N, K)).astype(np.float32)
        x16, w16 = H.to_bf16(x / 16), H.to_bf16(w)
        y = H.grouped_gemm_swiglu(x16, w16, SIZES, N, variant=variant)
        ok = bool((y == H.grouped_gemm_swiglu(x16, w16, SIZES, N, variant=-1)).all())
    print(kind, "order", os.environ.get("EMU_TILE_ORDER"), "variant", variant, "bit-exact", ok, round(time.time() - t), "s", flush=True)
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main(sys.argv[1], int(sys.argv[2])))
