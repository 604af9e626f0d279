"""m_sizes that no router would produce (negative entries, sums beyond M, a huge entry) through every kernel that reads
them, in the emulated library with every tensor against a guard page (run with EMU_GUARD=end): the kernels must
behave as if each size were clamped to [0, M] and the running sum cut at M - compute exactly those rows, leave the
rest of the output alone and touch nothing outside the tensors. Run by tests/test_emu_kernels.py as a child process."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import harness as H  # noqa: E402
from oracle import oracle as O  # noqa: E402


def clamped(sizes, M):
    out, run = [], 0
    for m in sizes:
        m = min(max(int(m), 0), M)
        m = min(m, M - run)
        out.append(m)
        run += m
    return out


def ints(rng, shape, lo=-2, hi=3):
    return rng.integers(lo, hi, shape).astype(np.float32)


def exact_rows(got16, want, rows, fp16=False):
    return bool((H.from16(got16, fp16)[:rows] == H.from16(H.to16(np.nan_to_num(want), fp16), fp16)[:rows]).all())


def main():
    rng = np.random.default_rng(0)
    bad = []
    M = 200
    for sizes in ([120, -8], [150, 100], [2 ** 30, 5], [-5, -5], [0, 300, -1, 40], [64, 64, 64, 64]):
        eff = clamped(sizes, M)
        rows, G = sum(eff), len(sizes)
        for N, K in ((64, 64), (256, 128), (40, 24)):
            x, w = ints(rng, (M, K)), ints(rng, (G * N, K))
            ref = O.grouped_gemm(x, w, eff)
            for fp16 in (False, True):
                for variant in (-1, 0, 1, 2, 3, 4, 5):
                    if variant in (0, 1, 2, 3) and K % 64 or variant == 5 and K % 128:
                        continue
                    y = H.grouped_gemm(H.to16(x, fp16), H.to16(w, fp16), sizes, N, fp16=fp16, variant=variant)
                    if not (exact_rows(y, ref, rows, fp16) and (y[rows:] == H.NAN16).all()):
                        bad.append(("gemm", sizes, N, K, fp16, variant))
            if K % 64 == 0 and N % 8 == 0:
                n = N // 2
                got = H.from_bf16(H.grouped_gemm_swiglu(H.to_bf16(x), H.to_bf16(w * 0.125), sizes, n))
                want = O.silu_and_mul(O.grouped_gemm(x, w * 0.125, eff))
                close = rows == 0 or (not np.isnan(got[:rows]).any()
                                      and np.abs(got[:rows] - want[:rows]).max() <= 1e-2 * max(1.0, np.abs(want[:rows]).max()))
                if not close or not np.isnan(got[rows:]).all():
                    bad.append(("swiglu", sizes, n, K))
            if N % 4 == 0 and K % 4 == 0:
                go = ints(rng, (M, N))
                for static in (False, True):
                    gx, gw = H.backward(H.to_bf16(go), H.to_bf16(x), H.to_bf16(w), sizes, N, False, static)
                    ox, ow = O.grouped_gemm_backward(go[:rows], x[:rows], w, eff)
                    if not (exact_rows(gx, ox, rows) and exact_rows(gw, ow, G * N)):
                        bad.append(("backward", sizes, N, K, static))
        for mode in (0, 1):
            N, K = 128, 256
            xq = ((0x30 + rng.integers(0, 0x18, (M, K))) | (rng.integers(0, 2, (M, K)) << 7)).astype(np.uint8)
            wq = ((0x30 + rng.integers(0, 0x18, (G * N, K))) | (rng.integers(0, 2, (G * N, K)) << 7)).astype(np.uint8)
            xs = np.ones(M if mode == 0 else (M, K // 128), np.float32)
            ws = np.ones(G * N if mode == 0 else (G * N // 128, K // 128), np.float32)
            ref = O.grouped_gemm_fp8(xq, wq, xs, ws, eff, mode)
            for variant in (-1, 0, 1, 2, 3):
                y = H.grouped_gemm_fp8(xq, wq, xs, ws, mode, sizes, N, variant)
                if not (exact_rows(y, ref, rows) and (y[rows:] == H.NAN16).all()):
                    bad.append(("fp8", sizes, mode, variant))
        N, K = 128, 256
        qw = np.stack([O.pack_int4_along_k(rng.integers(0, 16, (K, N))) for _ in range(G)])
        qz = np.stack([O.pack_int4_along_n(rng.integers(0, 15, (K // 128, N))) for _ in range(G)])
        sc = (2.0 ** rng.integers(-3, 1, (G, K // 128, N))).astype(np.float32)
        a = ints(rng, (M, K))
        want = O.w4a16_grouped(a, qw, sc, qz, eff, 128, 1)
        c = H.w4a16(H.to_bf16(a), qw, H.to_bf16(sc), qz, 128, 1, False, sizes)
        if not (exact_rows(c, want, rows) and (c[rows:] == H.NAN16).all()):
            bad.append(("w4a16 grouped", sizes))
        cq, cs = H.w4a16(H.to_bf16(a), qw, H.to_bf16(sc), qz, 128, 1, False, sizes, fp8out=True)
        oq, os_ = O.fp8_groupwise_quant(O.round_bf16(np.nan_to_num(want)))
        if not ((cq[:rows] == oq[:rows]).all() and (cs[:rows] == os_[:rows]).all() and (cq[rows:] == 0x7F).all()):
            bad.append(("w4a16 fp8out", sizes))
        H.release()
    for b in bad:
        print("MISMATCH", b, flush=True)
    print("bad", len(bad))
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
