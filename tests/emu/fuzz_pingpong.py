"""Random shapes through the 256 x 256 ping-pong kernels (bf16, fp16, fused SiLU-and-mul, fp8 row-wise and block scaled) in the
emulated library, checked against the oracle: bit-exact where the data make every sum exact (small integers, scales of
one), to 1e-2 for the fused activation. Run by tests/test_emu_kernels.py in child processes, because the number of compute
units (EMU_CUS: how many workgroups share the tiles) is fixed per process; EMU_DMA and EMU_SEED pick the load-landing model
and the order in which the waves of a workgroup run.

usage: fuzz_pingpong.py SEED CASES"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import harness as H  # noqa: E402
from oracle import oracle as O  # noqa: E402

EDGE = [0, 1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 319, 320, 321, 511, 512, 513, 530, 576, 577, 640, 767, 768, 769, 832, 833]


def one_case(rng):
    G = int(rng.integers(1, 6))
    sizes = [int(rng.choice(EDGE)) if rng.random() < 0.7 else int(rng.integers(0, 900)) for _ in range(G)]
    if sum(sizes) == 0:
        sizes[0] = 1
    M = sum(sizes)
    N = int(rng.choice([64, 256, 320, 512, 768]))
    K = int(rng.choice([64, 128, 192]))
    op = str(rng.choice(["bf16", "f16", "bf16w4", "f16w4", "swiglu", "swigluw4", "gather", "fp8row", "fp8block"]))
    if op in ("bf16", "f16", "bf16w4", "f16w4"):     # ...w4: the same tiles and order on the four-wave kernel
        fp16 = op.startswith("f16")
        x = rng.integers(-4, 5, (M, K)).astype(np.float32)
        w = rng.integers(-4, 5, (G * N, K)).astype(np.float32)
        y = H.grouped_gemm(H.to16(x, fp16), H.to16(w, fp16), sizes, N, fp16=fp16, variant=7 if op.endswith("w4") else 0)
        good = (H.from16(y, fp16) == H.from16(H.to16(O.grouped_gemm(x, w, sizes), fp16), fp16)).all()
    elif op == "gather":   # the fused activation kernel reading its rows through a permutation: same bits as gather + kernel
        n, k = max(64, N // 2 // 4 * 4), int(rng.integers(1, 4))
        T = max(1, -(-M // k))
        tok = H.to_bf16(rng.integers(-2, 3, (T, K)).astype(np.float32))
        w = H.to_bf16((rng.integers(-2, 3, (G * 2 * n, K)) * 0.125).astype(np.float32))
        ids = np.repeat(np.arange(G), sizes)                      # expert of every sorted row
        flat = np.full(T * k, -1, dtype=np.int64)
        flat[rng.permutation(T * k)[:M]] = ids                    # scattered over the slots, the rest masked
        perm, ms, _ = H.route_group(flat, G)
        good = (ms == np.array(sizes)).all()
        two_step = H.grouped_gemm_swiglu(H.gather_rows(tok, perm, k, n_valid=M), w, ms, n)
        good = bool(good and (H.grouped_gemm_swiglu_gather(tok, perm, k, w, ms, n)[:M] == two_step[:M]).all())
    elif op in ("swiglu", "swigluw4"):
        n = max(64, N // 2 // 4 * 4)
        x = rng.integers(-2, 3, (M, K)).astype(np.float32)
        w = (rng.integers(-2, 3, (G * 2 * n, K)) * 0.125).astype(np.float32)
        got = H.from_bf16(H.grouped_gemm_swiglu(H.to_bf16(x), H.to_bf16(w), sizes, n, variant=7 if op == "swigluw4" else -1))
        want = O.silu_and_mul(O.grouped_gemm(x, w, sizes))
        good = not np.isnan(got).any() and np.abs(got - want).max() <= 1e-2 * max(1.0, np.abs(want).max())
    else:
        mode = 0 if op == "fp8row" else 1
        K = 128 * int(rng.integers(1, 3))
        N = max(128, N // 128 * 128)
        # magnitudes 0.5 ... 3.75: every partial sum is exact in fp32
        xq = ((0x30 + rng.integers(0, 0x18, (M, K))) | (rng.integers(0, 2, (M, K)) << 7)).astype(np.uint8)
        wq = ((0x30 + rng.integers(0, 0x18, (G * N, K))) | (rng.integers(0, 2, (G * N, K)) << 7)).astype(np.uint8)
        xs = np.ones(M if mode == 0 else (M, K // 128), np.float32)
        ws = np.ones(G * N if mode == 0 else (G * N // 128, K // 128), np.float32)
        y = H.grouped_gemm_fp8(xq, wq, xs, ws, mode, sizes, N, variant=3)
        good = (H.from_bf16(y) == O.round_bf16(O.grouped_gemm_fp8(xq, wq, xs, ws, sizes, mode))).all()
    return good, (op, sizes, N, K)


def main():
    rng = np.random.default_rng(int(sys.argv[1]))
    bad = []
    for _ in range(int(sys.argv[2])):
        good, what = one_case(rng)
        if not good:
            bad.append(what)
            print("MISMATCH", what, flush=True)
    print("cases", sys.argv[2], "bad", len(bad))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
