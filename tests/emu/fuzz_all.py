"""Random shapes through every entry point of the emulated library, checked against the oracle. With EMU_GUARD=end or
start (tests/emu/harness.py) every tensor sits against an inaccessible page, so an access outside a tensor ends the
process with a memory fault instead of passing unnoticed. Run by tests/test_emu_kernels.py in child processes.

usage: fuzz_all.py SEED CASES"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import harness as H  # noqa: E402
from oracle import oracle as O  # noqa: E402

EDGE = [0, 1, 2, 15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 272, 273, 288, 289, 320, 511, 512, 513, 530, 544]


def sizes_of(rng, gmax=6, mmax=600):
    G = int(rng.integers(1, gmax + 1))
    s = [int(rng.choice([e for e in EDGE if e <= mmax])) if rng.random() < 0.6 else int(rng.integers(0, mmax)) for _ in range(G)]
    if sum(s) == 0:
        s[int(rng.integers(0, G))] = int(rng.integers(1, 40))
    return s


def ints(rng, shape, lo=-4, hi=5):
    return rng.integers(lo, hi, shape).astype(np.float32)


def fp8_codes(rng, shape):
    """e4m3 codes of magnitude 0.5 ... 3.75 with random sign: products are multiples of 2^-8 below 2^4, so sums over a
    few hundred of them (times scales of 1 or 2) are exact in fp32 in any order."""
    return ((0x30 + rng.integers(0, 0x18, shape)) | (rng.integers(0, 2, shape) << 7)).astype(np.uint8)


def exact16(got16, want, fp16=False):
    mask = ~np.isnan(want)
    return bool((H.from16(got16, fp16)[mask] == H.from16(H.to16(np.nan_to_num(want), fp16), fp16)[mask]).all())


def c_gemm(rng):
    sizes = sizes_of(rng)
    fp16 = bool(rng.integers(0, 2))
    block = bool(rng.integers(0, 2))
    if rng.random() < 0.3:   # any shape: the generic kernel
        N, K, variant = int(rng.integers(1, 200)), int(rng.integers(1, 200)), -1
    else:
        N, K = int(rng.choice([16, 64, 100, 128, 256, 264, 512])), int(rng.choice([64, 128, 192, 256]))
        variant = int(rng.choice([-1, 0, 1, 2, 3, 4, 5, 6, 7, 7, 8, 8]))
        if variant == 5 and K % 128:
            K = 128
    G, M = len(sizes), sum(sizes)
    x, w = ints(rng, (M, K)), ints(rng, (G * N, K))
    y = H.grouped_gemm(H.to16(x, fp16), H.to16(w, fp16), sizes, N, fp16=fp16, block_layout=block, variant=variant)
    ref = O.grouped_gemm(x, w, sizes, block_layout=block)
    return exact16(y, ref, fp16) and bool((y[np.isnan(ref)] == H.NAN16).all()), ("gemm", sizes, N, K, variant, fp16, block)


def c_fp8(rng):
    sizes = sizes_of(rng)
    mode = int(rng.integers(0, 2))
    K = 128 * int(rng.integers(1, 4))
    N = 128 * int(rng.integers(1, 4)) if mode == 1 or rng.random() < 0.5 else int(rng.choice([16, 72, 200, 330]))
    variant = int(rng.choice([-1, 0, 1, 2, 3]))
    G, M = len(sizes), sum(sizes)
    xq, wq = fp8_codes(rng, (M, K)), fp8_codes(rng, (G * N, K))
    xs = (2.0 ** rng.integers(0, 2, M if mode == 0 else (M, K // 128))).astype(np.float32)
    ws = (2.0 ** rng.integers(0, 2, G * N if mode == 0 else (G * N // 128, K // 128))).astype(np.float32)
    y = H.grouped_gemm_fp8(xq, wq, xs, ws, mode, sizes, N, variant)
    return exact16(y, O.grouped_gemm_fp8(xq, wq, xs, ws, sizes, mode)), ("fp8", sizes, N, K, mode, variant)


def c_swiglu(rng):
    sizes = sizes_of(rng)
    fp16 = bool(rng.integers(0, 2))
    n, K = int(rng.choice([4, 64, 100, 128, 192, 260])), int(rng.choice([64, 128, 192]))
    G, M = len(sizes), sum(sizes)
    x = ints(rng, (M, K), -2, 3)
    w = (ints(rng, (G * 2 * n, K), -2, 3) * 0.125).astype(np.float32)
    variant = int(rng.choice([-1, -1, 7, 8]))     # the eight-wave kernel or one of its four-wave forms
    got = H.from16(H.grouped_gemm_swiglu(H.to16(x, fp16), H.to16(w, fp16), sizes, n, fp16, variant=variant), fp16)
    want = O.silu_and_mul(O.grouped_gemm(x, w, sizes))
    return bool(not np.isnan(got).any() and np.abs(got - want).max() <= 1e-2 * max(1.0, np.abs(want).max())), ("swiglu", sizes, n, K, fp16, variant)


def c_backward(rng):
    sizes = sizes_of(rng, 5, 400)
    N, K = 4 * int(rng.integers(1, 80)), 4 * int(rng.integers(1, 60))
    if rng.random() < 0.5:
        N, K = int(rng.choice([64, 128, 256, 320])), int(rng.choice([64, 128, 256]))
    block, static = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    G, M = len(sizes), sum(sizes)
    x, w = ints(rng, (M, K), -2, 3), ints(rng, (G * N, K), -2, 3)
    go = ints(rng, (M, N * G if block else N), -2, 3)
    gx, gw = H.backward(H.to_bf16(go), H.to_bf16(x), H.to_bf16(w), sizes, N, block, static)
    ox, ow = O.grouped_gemm_backward(go, x, w, sizes)
    return exact16(gx, ox) and exact16(gw, ow), ("backward", sizes, N, K, block, static)


def c_w4a16(rng):
    gs = int(rng.choice([32, 64, 128, 128]))
    K = gs * int(rng.integers(1, 9)) if gs < 128 else 128 * int(rng.integers(1, 9))
    N = 64 * int(rng.integers(1, 5))
    fp16 = bool(rng.integers(0, 2))
    zero_offset = int(rng.integers(0, 2))
    kind = str(rng.choice(["dense", "grouped", "fp8out"]))
    if kind == "fp8out":
        N = 128 * int(rng.integers(1, 3))
    sizes = None if kind == "dense" else sizes_of(rng, 5, 70)
    M = int(rng.integers(1, 80)) if sizes is None else sum(sizes)
    E = 1 if sizes is None else len(sizes)
    qv, zv = rng.integers(0, 16, (E, K, N)), rng.integers(0, 15, (E, K // gs, N))
    qw = np.stack([O.pack_int4_along_k(qv[e]) for e in range(E)])
    qz = np.stack([O.pack_int4_along_n(zv[e]) for e in range(E)])
    sc = (2.0 ** rng.integers(-3, 1, (E, K // gs, N))).astype(np.float32)
    a = ints(rng, (M, K), -2, 3)
    a16, s16 = H.to16(a, fp16), H.to16(sc, fp16)
    variant = int(rng.integers(-1, 8))              # MOE_GG_OP_W4A16: the selectable kernels too
    what = ("w4a16", kind, M if sizes is None else sizes, N, K, gs, fp16, zero_offset, variant)
    if sizes is None:
        c = H.w4a16(a16, qw[0], s16[0], qz[0], gs, zero_offset, fp16, variant=variant)
        return exact16(c, O.w4a16_gemm(a, qw[0], sc[0], qz[0], gs, zero_offset), fp16), what
    want = O.w4a16_grouped(a, qw, sc, qz, sizes, gs, zero_offset)
    if kind == "grouped":
        return exact16(H.w4a16(a16, qw, s16, qz, gs, zero_offset, fp16, sizes, variant=variant), want, fp16), what
    cq, cs = H.w4a16(a16, qw, s16, qz, gs, zero_offset, fp16, sizes, fp8out=True)
    oq, os_ = O.fp8_groupwise_quant(H.from16(H.to16(want, fp16), fp16))
    return bool((cq == oq).all() and (cs == os_).all()), what


def c_routing(rng):
    E = int(rng.choice([2, 8, 60, 256, 768]))
    k = int(rng.integers(1, min(E, 8) + 1))
    T = int(rng.integers(1, 500))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    ids, perm, ms, off = H.route_topk(logits, k)
    oi = O.topk(logits, k)
    op, om = O.route(oi, E)
    good = bool((ids == oi).all() and (perm == op).all() and (ms == om).all() and (off == O.offsets(om)).all())
    flat = rng.integers(-2, E + 2, int(rng.integers(1, 3000)))
    perm, ms, off = H.route_group(flat, E)
    op, om = O.route(flat, E)
    good = good and bool((perm == op).all() and (ms == om).all())
    nv = int(ms.sum())
    bs = int(rng.choice([1, 4, 16, 64]))
    s, e, post = H.align_block_size(perm, ms, bs)
    keep = flat[(flat >= 0) & (flat < E)]
    _, oe, opost = O.moe_align_block_size(keep, bs, E) if len(keep) else (None, e, post)
    good = good and post == opost and bool((e[:post // bs] == oe[:post // bs]).all())
    kk = int(rng.integers(1, 4))
    rows = max(1, (len(flat) + kk - 1) // kk)
    x = rng.integers(0, 60000, (rows, 8 * int(rng.integers(1, 20)))).astype(np.uint16)
    g = H.gather_rows(x, perm, kk, n_valid=nv)
    good = good and bool((g[:nv] == x[perm[:nv] // kk]).all() and (g[nv:] == 0).all())
    inv = H.invert_perm(perm, n_valid=nv)
    good = good and bool((inv[perm[:nv]] == np.arange(nv)).all())
    return good, ("routing", T, E, k, len(flat), bs, kk)


def c_quant(rng):
    rows, K = int(rng.integers(1, 40)), 128 * int(rng.integers(1, 6))
    x = (rng.standard_normal((rows, K)) * float(rng.choice([1e-3, 1.0, 300.0]))).astype(np.float32)
    bf = bool(rng.integers(0, 2))
    q, s = H.fp8_groupwise_quant(x, bf)
    oq, os_ = O.fp8_groupwise_quant(O.round_bf16(x) if bf else x)
    good = bool((q == oq).all() and (s == os_).all())
    w = (rng.standard_normal((128 * int(rng.integers(1, 4)), 128 * int(rng.integers(1, 4)))) * 0.02).astype(np.float32)
    q, s = H.fp8_block128_quant(w, bf)
    oq, os_ = O.fp8_block_quant_weight(O.round_bf16(w) if bf else w)
    return good and bool((q == oq).all() and (s == os_).all()), ("quant", rows, K, w.shape, bf)


def c_glue(rng):
    fp16 = bool(rng.integers(0, 2))
    rows, n = int(rng.integers(1, 70)), 8 * int(rng.integers(1, 40))
    x = H.to16(rng.standard_normal((rows, 2 * n)).astype(np.float32), fp16)
    got, want = H.from16(H.silu_and_mul(x, fp16), fp16), O.silu_and_mul(H.from16(x, fp16))
    good = bool((np.abs(got - want) <= 1e-2 * np.maximum(1.0, np.abs(want))).all())
    T, k, d = int(rng.integers(1, 50)), int(rng.integers(1, 5)), 8 * int(rng.integers(1, 30))
    inv = rng.permutation(T * k).astype(np.int32)
    y = ints(rng, (T * k, d))
    wts = (2.0 ** rng.integers(-2, 1, (T, k))).astype(np.float32)
    want = (wts[:, :, None] * y[inv].reshape(T, k, d)).sum(1)
    w16 = bool(rng.integers(0, 2))
    good = good and exact16(H.combine_topk(H.to16(y, fp16), inv, wts, T, k, fp16=fp16, weights_16bit=w16), want, fp16)
    return good, ("glue", rows, n, T, k, d, fp16, w16)


CASES = [c_gemm, c_gemm, c_fp8, c_swiglu, c_backward, c_w4a16, c_w4a16, c_routing, c_quant, c_glue]


def main():
    rng = np.random.default_rng(int(sys.argv[1]))
    bad = 0
    for i in range(int(sys.argv[2])):
        fn = CASES[int(rng.integers(0, len(CASES)))]
        good, what = fn(rng)
        if os.environ.get("EMU_VERBOSE"):
            print(i, what, good, flush=True)
        if not good:
            bad += 1
            print("MISMATCH", what, flush=True)
        H.release()
    print("cases", sys.argv[2], "bad", bad)
    return 1 if bad else 0


if __name__ == "__main__":
    sys.exit(main())
