"""The library's device code on the CPU: every .hip source compiled as host C++ behind a stand-in HIP header
(tests/emu) and run under a lockstep-wave emulation, called through the same C ABI as on the GPU and checked against
the oracle. This covers what the host-side tests cannot reach without a GPU: the indexing of the kernels, their tile
tables, LDS layouts, MFMA fragment layouts, wave-level exchanges, the counted waits behind the global->LDS loads, and
the dispatch in api.hip. It says nothing about speed, and rounding inside a matrix instruction may differ from the
hardware's, so products are checked bit-exactly only on data whose sums are exact (small integers, power-of-two
scales) and to the GPU tests' tolerance otherwise."""
import ctypes
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EMU = os.path.join(ROOT, "tests", "emu")
sys.path.insert(0, EMU)

import build_emu  # noqa: E402

if not os.path.exists(build_emu.CXX):
    pytest.skip("host clang++ of the ROCm toolchain not found: the emulated build needs it", allow_module_level=True)

import harness as H  # noqa: E402
from oracle import oracle as O  # noqa: E402


@pytest.fixture(scope="module", autouse=True)
def built():
    H.lib()


def ints(rng, shape, lo=-4, hi=5):
    return rng.integers(lo, hi, shape).astype(np.float32)


def exact16(got16, want, fp16=False):
    mask = ~np.isnan(want)
    got = H.from16(got16, fp16)
    return bool((got[mask] == H.from16(H.to16(np.nan_to_num(want), fp16), fp16)[mask]).all())


@pytest.fixture(params=[0, 1], ids=["two_lists", "split_tails"])
def tile_order(request):
    """Both tile orders of the ping-pong kernels (MOE_GG_OP_TILE_ORDER) for one test."""
    L = H.lib()
    assert L.moe_gg_set_variant(H.OP_TILE_ORDER, request.param) == 0
    try:
        yield request.param
    finally:
        L.moe_gg_set_variant(H.OP_TILE_ORDER, -1)


SIZES = [300, 0, 70, 530]   # a full tile + a low tile, an empty expert, a short one, a tall one whose tail is split


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7, 8, -1])
def test_bf16_every_kernel_variant(variant, tile_order):
    rng = np.random.default_rng(variant + 1)
    x, w = ints(rng, (sum(SIZES), 128)), ints(rng, (4 * 512, 128))
    y = H.grouped_gemm(H.to_bf16(x), H.to_bf16(w), SIZES, 512, variant=variant)
    assert exact16(y, O.grouped_gemm(x, w, SIZES))


@pytest.mark.parametrize("K", [64, 128, 192, 320])
@pytest.mark.parametrize("sizes,N", [([300, 0, 70, 530], 512), ([257, 1], 300), ([40], 64)])
@pytest.mark.parametrize("variant", [6, 7, 8])
def test_four_wave_kernels_over_k_steps(sizes, N, K, variant):
    """MOE_GG_GG_TILED_256_W4 and MOE_GG_GG_FOURWAVE_256 with 1, 2, 3 and 5 K steps per tile: their loops issue the
    slab loads behind the last slab too (masked to one line, into the buffer nobody reads again), and the second one
    streams slabs through tile boundaries, so the short reductions are the cases to see."""
    rng = np.random.default_rng(K + N)
    G = len(sizes)
    x, w = ints(rng, (sum(sizes), K)), ints(rng, (G * N, K))
    for fp16, block in ((False, False), (True, True)):
        y = H.grouped_gemm(H.to16(x, fp16), H.to16(w, fp16), sizes, N, fp16=fp16, block_layout=block, variant=variant)
        assert exact16(y, O.grouped_gemm(x, w, sizes, block_layout=block), fp16)


@pytest.mark.parametrize("fp16,block", [(True, False), (False, True), (True, True)])
def test_fp16_and_block_layout(fp16, block, tile_order):
    rng = np.random.default_rng(7)
    x, w = ints(rng, (sum(SIZES), 128)), ints(rng, (4 * 256, 128))
    y = H.grouped_gemm(H.to16(x, fp16), H.to16(w, fp16), SIZES, 256, fp16=fp16, block_layout=block)
    ref = O.grouped_gemm(x, w, SIZES, block_layout=block)
    assert exact16(y, ref, fp16)
    assert (y[np.isnan(ref)] == H.NAN16).all()   # the other experts' column blocks stay untouched


@pytest.mark.parametrize("sizes,N,K", [([3, 0, 7, 5], 256, 256), ([1], 64, 128), ([20, 10, 20], 33, 40), ([0, 0, 70, 0, 0], 100, 72),
                                       ([4] * 32, 16, 16)])
def test_small_and_odd_shapes_take_the_decode_and_generic_kernels(sizes, N, K):
    rng = np.random.default_rng(len(sizes))
    x, w = ints(rng, (sum(sizes), K)), ints(rng, (len(sizes) * N, K))
    for fp16 in (False, True):
        assert exact16(H.grouped_gemm(H.to16(x, fp16), H.to16(w, fp16), sizes, N, fp16=fp16), O.grouped_gemm(x, w, sizes), fp16)


@pytest.mark.parametrize("sizes", [[530], [520, 30]])
def test_low_tiles_computed_by_the_small_m_kernel(sizes, tile_order):
    """K >= 8192 with few experts: the ping-pong launch leaves the rows behind the last full tile to a launch of the
    small-M kernel (both decide it from m_sizes on the device)."""
    G, M, N, K = len(sizes), sum(sizes), 256, 8192
    ms = np.array(sizes, dtype=np.int32)
    assert H.lib().moe_gg_host_tails_apart(ms.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), G, M, N, K, 8) == 1
    rng = np.random.default_rng(1)
    x, w = ints(rng, (M, K), -2, 3), ints(rng, (G * N, K), -2, 3)
    assert exact16(H.grouped_gemm(H.to_bf16(x), H.to_bf16(w), sizes, N), O.grouped_gemm(x, w, sizes))


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("variant", [0, 1, 2, 3, -1])
def test_fp8_every_kernel_variant(mode, variant, tile_order):
    rng = np.random.default_rng(10 * mode + variant + 3)
    sizes, N, K = [300, 0, 70, 30, 530], 256, 256
    G, M = len(sizes), sum(sizes)
    # codes of magnitude 0.5 ... 3.75 and scales of 1 or 2: every partial sum is exact in fp32, whatever the order
    xq = ((0x30 + rng.integers(0, 0x18, (M, K))) | (rng.integers(0, 2, (M, K)) << 7)).astype(np.uint8)
    wq = ((0x30 + rng.integers(0, 0x18, (G * N, K))) | (rng.integers(0, 2, (G * N, K)) << 7)).astype(np.uint8)
    xs = (2.0 ** rng.integers(0, 2, M if mode == 0 else (M, K // 128))).astype(np.float32)
    ws = (2.0 ** rng.integers(0, 2, G * N if mode == 0 else (G * N // 128, K // 128))).astype(np.float32)
    y = H.grouped_gemm_fp8(xq, wq, xs, ws, mode, sizes, N, variant)
    assert exact16(y, O.grouped_gemm_fp8(xq, wq, xs, ws, sizes, mode))


@pytest.mark.parametrize("sizes,N,K", [([257, 272, 273, 288, 289], 256, 128), ([530, 1, 544, 0, 800], 300, 64), ([270], 256, 192),
                                       ([1036, 1012, 998], 512, 64), ([513] * 5, 128, 128)])
@pytest.mark.parametrize("fp16", [False, True])
def test_four_wave_kernel_with_tall_tiles(sizes, N, K, fp16):
    """MOE_GG_GG_FOURWAVE_TALL: tails of 1, 16, 17 and 32 rows ride along with the last full tile (33 do not), also when
    the tile is cut into row pieces ([270] alone: four pieces on eight compute units, the last with 64 + 14 rows)."""
    rng = np.random.default_rng(len(sizes) + N)
    x, w = ints(rng, (sum(sizes), K)), ints(rng, (len(sizes) * N, K))
    y = H.grouped_gemm(H.to16(x, fp16), H.to16(w, fp16), sizes, N, fp16=fp16, variant=8)
    assert exact16(y, O.grouped_gemm(x, w, sizes), fp16)


@pytest.mark.parametrize("fp16", [False, True])
@pytest.mark.parametrize("variant", [-1, 7, 8])
@pytest.mark.parametrize("n,K", [(192, 128), (64, 64), (328, 192)])
def test_fused_silu_and_mul_gemm(fp16, variant, n, K, tile_order):
    """The eight-wave kernel and (variants 7, 8) its four-wave forms: against the oracle, and against each other
    bit for bit (the same products in the same order, the same roundings)."""
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((sum(SIZES), K)) * 0.5).astype(np.float32)
    w = (rng.standard_normal((4 * 2 * n, K)) * 0.1).astype(np.float32)
    x16, w16 = H.to16(x, fp16), H.to16(w, fp16)
    got16 = H.grouped_gemm_swiglu(x16, w16, SIZES, n, fp16, variant=variant)
    got = H.from16(got16, fp16)
    want = O.silu_and_mul(O.grouped_gemm(H.from16(x16, fp16), H.from16(w16, fp16), SIZES))
    np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-2)
    if variant >= 7:
        assert (got16 == H.grouped_gemm_swiglu(x16, w16, SIZES, n, fp16)).all()


@pytest.mark.parametrize("fp16", [False, True])
@pytest.mark.parametrize("T,E,k,n,K", [(200, 4, 2, 128, 128), (700, 8, 2, 192, 64), (300, 3, 3, 64, 256), (33, 2, 1, 256, 128)])
def test_gather_folded_into_the_first_gemm_gives_the_same_bits(fp16, T, E, k, n, K, tile_order):
    """moe_gg_grouped_gemm_swiglu_gather on the token matrix and the permutation against moe_gg_gather_rows followed by
    moe_gg_grouped_gemm_swiglu: bit for bit, with masked slots, and rows beyond sum(m_sizes) left alone."""
    rng = np.random.default_rng(T + n)
    tok = H.to16(ints(rng, (T, K), -3, 4), fp16)
    w = H.to16(ints(rng, (E * 2 * n, K), -2, 3) * 0.125, fp16)
    ids = rng.integers(0, E, (T, k))
    ids.ravel()[rng.permutation(T * k)[:T * k // 10]] = -1
    perm, ms, _ = H.route_group(ids, E)
    nv = int(ms.sum())
    two_step = H.grouped_gemm_swiglu(H.gather_rows(tok, perm, k, n_valid=nv), w, ms, n, fp16)
    fused = H.grouped_gemm_swiglu_gather(tok, perm, k, w, ms, n, fp16)
    assert (fused[:nv] == two_step[:nv]).all() and (fused[nv:] == H.NAN16).all()


def test_gather_with_a_corrupt_permutation_stays_inside_the_token_matrix():
    """Entries of perm outside [0, T k) (a caller's mistake: route_group never writes them in the rows that are read):
    with the token matrix against guard pages on either side the call completes, and rows with valid entries are
    still right."""
    rng = np.random.default_rng(3)
    T, E, k, n, K = 150, 2, 2, 64, 128
    tok = H.to_bf16(ints(rng, (T, K), -3, 4))
    w = H.to_bf16(ints(rng, (E * 2 * n, K), -2, 3) * 0.125)
    ids = rng.integers(0, E, (T, k))
    perm, ms, _ = H.route_group(ids, E)
    want = H.grouped_gemm_swiglu(H.gather_rows(tok, perm, k), w, ms, n)
    bad = perm.copy()
    hit = rng.permutation(T * k)[:40]
    bad[hit] = rng.choice([-1, -2 ** 31, 2 ** 31 - 1, T * k, T * k + 7, 10 ** 9], 40)
    for guard in ("end", "start"):
        H.GUARD = guard
        try:
            got = H.grouped_gemm_swiglu_gather(tok, bad, k, w, ms, n).copy()
        finally:
            H.GUARD = None
            H.release()
        keep = np.setdiff1d(np.arange(T * k), hit)
        assert (got[keep] == want[keep]).all()


@pytest.mark.parametrize("sizes,N,K,block,static", [
    (SIZES, 256, 128, False, False), (SIZES, 256, 128, True, False), (SIZES, 256, 128, False, True),
    ([30, 0, 7, 53], 64, 64, False, False), ([0, 5, 0], 64, 64, False, False), ([300, 200], 68, 36, False, False)])
def test_backward(sizes, N, K, block, static, tile_order):
    rng = np.random.default_rng(N + K)
    G, M = len(sizes), sum(sizes)
    x, w = ints(rng, (M, K), -2, 3), ints(rng, (G * N, K), -2, 3)
    go = ints(rng, (M, N * G if block else N), -2, 3)
    gx, gw = H.backward(H.to_bf16(go), H.to_bf16(x), H.to_bf16(w), sizes, N, block, static)
    ox, ow = O.grouped_gemm_backward(go, x, w, sizes)
    assert exact16(gx, ox) and exact16(gw, ow)   # experts without rows: zero grad_w, written


def w4_inputs(rng, E, K, N, gs):
    qv, zv = rng.integers(0, 16, (E, K, N)), rng.integers(0, 15, (E, K // gs, N))
    qw = np.stack([O.pack_int4_along_k(qv[e]) for e in range(E)])
    qz = np.stack([O.pack_int4_along_n(zv[e]) for e in range(E)])
    return qw, qz, (2.0 ** rng.integers(-3, 1, (E, K // gs, N))).astype(np.float32)


@pytest.mark.parametrize("M,N,K,gs,fp16", [(1, 256, 512, 128, False), (5, 128, 256, 128, True), (16, 192, 256, 128, False),
                                           (33, 128, 256, 64, False), (70, 64, 256, 128, False)])
def test_w4a16_splitk(M, N, K, gs, fp16):
    rng = np.random.default_rng(M)
    qw, qz, sc = w4_inputs(rng, 1, K, N, gs)
    a = ints(rng, (M, K), -2, 3)
    c = H.w4a16(H.to16(a, fp16), qw[0], H.to16(sc[0], fp16), qz[0], gs, 1, fp16)
    assert exact16(c, O.w4a16_gemm(a, qw[0], sc[0], qz[0], gs, 1), fp16)


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6, 7])
@pytest.mark.parametrize("M,N,K,fp16", [(1, 256, 512, False), (5, 128, 1024, True), (16, 192, 256, False), (17, 64, 512, False),
                                        (33, 128, 512, False), (64, 64, 1024, True), (70, 64, 256, False), (130, 128, 512, False)])
def test_w4a16_selectable_variants(M, N, K, fp16, variant):
    """MOE_GG_OP_W4A16: 1 = passes of four activation fragments on four waves for more than 32 rows, 2 = warm-up waves
    and masked activation rows for up to 16 rows, 4 = activations staged through the wave's LDS area (every row count);
    row counts outside the range of bits 1 and 2 take the default kernels (or their staged forms)."""
    rng = np.random.default_rng(100 * variant + M)
    qw, qz, sc = w4_inputs(rng, 1, K, N, 128)
    a = ints(rng, (M, K), -2, 3)
    c = H.w4a16(H.to16(a, fp16), qw[0], H.to16(sc[0], fp16), qz[0], 128, 1, fp16, variant=variant)
    assert exact16(c, O.w4a16_gemm(a, qw[0], sc[0], qz[0], 128, 1), fp16)


@pytest.mark.parametrize("variant", [1, 2, 4, 5, 6])
def test_w4a16_grouped_selectable_variants(variant):
    rng = np.random.default_rng(40 + variant)
    sizes = [40, 0, 70, 33, 30] if variant & 1 else [3, 0, 16, 12, 1]       # average rows per expert picks the kernel
    N, K = 128, 512
    qw, qz, sc = w4_inputs(rng, len(sizes), K, N, 128)
    a = ints(rng, (sum(sizes), K), -2, 3)
    want = O.w4a16_grouped(a, qw, sc, qz, sizes, 128, 0)
    assert exact16(H.w4a16(H.to_bf16(a), qw, H.to_bf16(sc), qz, 128, 0, False, sizes, variant=variant), want)


def test_w4a16_grouped_and_its_fp8_epilogue():
    rng = np.random.default_rng(4)
    sizes, N, K = [3, 0, 9, 12], 256, 256
    qw, qz, sc = w4_inputs(rng, 4, K, N, 128)
    a = ints(rng, (sum(sizes), K), -2, 3)
    want = O.w4a16_grouped(a, qw, sc, qz, sizes, 128, 1)
    assert exact16(H.w4a16(H.to_bf16(a), qw, H.to_bf16(sc), qz, 128, 1, False, sizes), want)
    cq, cs = H.w4a16(H.to_bf16(a), qw, H.to_bf16(sc), qz, 128, 1, False, sizes, fp8out=True)
    oq, os_ = O.fp8_groupwise_quant(O.round_bf16(want))
    assert (cq == oq).all() and (cs == os_).all()


def test_routing_kernels():
    rng = np.random.default_rng(6)
    T, E, k = 300, 8, 2
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[5] = 0.25                                   # ties go to the lower expert index
    ids, perm, ms, off = H.route_topk(logits, k)
    oi = O.topk(logits, k)
    op, om = O.route(oi, E)
    assert (ids == oi).all() and (perm == op).all() and (ms == om).all() and (off == O.offsets(om)).all()
    flat = rng.integers(-1, E + 1, 1000)               # ids outside [0, E) are masked slots
    perm, ms, off = H.route_group(flat, E)
    op, om = O.route(flat, E)
    assert (perm == op).all() and (ms == om).all()
    keep = flat[(flat >= 0) & (flat < E)]
    s, e, post = H.align_block_size(perm, ms, 16)
    os_, oe, opost = O.moe_align_block_size(keep, 16, E)
    assert post == opost and (e[:post // 16] == oe[:post // 16]).all()
    # the sorted list holds positions of the unmasked list in the oracle and of the full list in the kernel: compare experts
    pad = len(flat)
    for blk in range(post // 16):
        mine = s[16 * blk:16 * blk + 16]
        assert all(flat[i] == e[blk] for i in mine if i < pad)
    nv = int(ms.sum())
    x = rng.integers(0, 60000, (500, 64)).astype(np.uint16)
    g = H.gather_rows(x, perm, 2, n_valid=nv)
    assert (g[:nv] == x[perm[:nv] // 2]).all() and (g[nv:] == 0).all()
    inv = H.invert_perm(perm, n_valid=nv)             # masked positions keep what the buffer held
    assert (inv[perm[:nv]] == np.arange(nv)).all() and (np.delete(inv, perm[:nv]) == -7).all()


def test_quantisers_bit_exact():
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((64, 512)) * 3).astype(np.float32)
    x[3, :128] = 0.0                                   # an all-zero group: scale from the 1e-12 floor
    for bf16_in in (False, True):
        q, s = H.fp8_groupwise_quant(x, bf16_in)
        oq, os_ = O.fp8_groupwise_quant(O.round_bf16(x) if bf16_in else x)
        assert (q == oq).all() and (s == os_).all()
    w = (rng.standard_normal((256, 384)) * 0.02).astype(np.float32)
    for bf16_in in (False, True):
        q, s = H.fp8_block128_quant(w, bf16_in)
        oq, os_ = O.fp8_block_quant_weight(O.round_bf16(w) if bf16_in else w)
        assert (q == oq).all() and (s == os_).all()


def test_moe_layer_as_the_sequence_of_abi_calls():
    """fused_moe's launch sequence (route, gather, w1 GEMM with SiLU-and-mul, w2 GEMM, un-permute and weighted sum)
    on numpy buffers, against the layer oracle."""
    rng = np.random.default_rng(9)
    T, E, k, K, n, d = 96, 4, 2, 128, 128, 64
    a = (rng.standard_normal((T, K)) * 0.5).astype(np.float32)
    w1 = (rng.standard_normal((E, 2 * n, K)) * 0.1).astype(np.float32)
    w2 = (rng.standard_normal((E, d, n)) * 0.1).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    a16, w1_16, w2_16 = H.to_bf16(a), H.to_bf16(w1), H.to_bf16(w2)
    ids, perm, ms, off = H.route_topk(logits, k)
    tw = np.take_along_axis(np.exp(logits) / np.exp(logits).sum(1, keepdims=True), ids, axis=1).astype(np.float32)
    xs = H.gather_rows(a16, perm, k)
    h = H.grouped_gemm_swiglu(xs, w1_16.reshape(E * 2 * n, K), ms, n)
    y = H.grouped_gemm(h, w2_16.reshape(E * d, n), ms, d)
    out = H.from_bf16(H.combine_topk(y, H.invert_perm(perm), tw, T, k))
    want = O.fused_moe(H.from_bf16(a16), H.from_bf16(w1_16), H.from_bf16(w2_16), tw, ids)
    np.testing.assert_allclose(out, want, rtol=2e-2, atol=2e-2)


def test_glue_kernels():
    rng = np.random.default_rng(11)
    x = rng.standard_normal((50, 256)).astype(np.float32)
    for fp16 in (False, True):
        x16 = H.to16(x, fp16)
        np.testing.assert_allclose(H.from16(H.silu_and_mul(x16, fp16), fp16), O.silu_and_mul(H.from16(x16, fp16)), rtol=1e-2, atol=1e-2)
    T, k, d = 32, 2, 64
    inv = rng.permutation(T * k).astype(np.int32)
    y = ints(rng, (T * k, d))
    wts = (2.0 ** rng.integers(-2, 1, (T, k))).astype(np.float32)
    want = (wts[:, :, None] * y[inv].reshape(T, k, d)).sum(1)
    for w16 in (False, True):
        assert exact16(H.combine_topk(H.to_bf16(y), inv, wts, T, k, weights_16bit=w16), want)


def test_argument_checks_reach_the_caller():
    L = H.lib()
    buf = np.zeros(64, dtype=np.uint16)
    ms = np.array([1], dtype=np.int32)
    assert L.moe_gg_grouped_gemm_bf16(None, H.P(buf), H.P(buf), H.P(ms), 1, 1, 8, 8, 8, 0, None) == -1
    assert L.moe_gg_grouped_gemm_bf16(H.P(buf), H.P(buf), H.P(buf), H.P(ms), 2000, 1, 8, 8, 8, 0, None) == -4
    assert L.moe_gg_grouped_gemm_fp8(H.P(buf), H.P(buf), H.P(buf), H.P(buf), H.P(buf), 1, H.P(ms), 1, 1, 128, 100, 128, 0, None) != 0


GOLD = os.path.join(ROOT, "tests", "golden")


def rel_fro(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def test_committed_golden_vectors():
    """The fixtures of tests/golden with the bars of the GPU tests: config 1 (routing bit-exact, GEMM to 1e-2), the
    tiny fp8 case in both scale modes and the tiny W4A16 case with both zero-point conventions (relative Frobenius
    error <= 2e-2), the moe_align_block_size known answer."""
    import json

    z = np.load(os.path.join(GOLD, "cfg1.npz"))
    ids, perm, ms, off = H.route_topk(z["logits"], 2)
    assert (ids == z["ids"]).all() and (perm == z["perm"]).all() and (ms == z["m_sizes"]).all() and (off == z["offsets"]).all()
    y = H.from_bf16(H.grouped_gemm(z["x_sorted_bf16_bits"], z["w_bf16_bits"], z["m_sizes"], 512))
    np.testing.assert_allclose(y, z["y_bf16_inputs"], rtol=1e-2, atol=1e-2)

    z = np.load(os.path.join(GOLD, "fp8_tiny.npz"))
    m = z["m_sizes"].tolist()
    tot = sum(m)
    y = H.from_bf16(H.grouped_gemm_fp8(z["xq"], z["wq"], z["xs"], z["ws"], 1, m, 256))
    assert rel_fro(y[:tot], z["y_block"][:tot]) <= 2e-2
    y = H.from_bf16(H.grouped_gemm_fp8(z["xq_row"], z["wq_row"], z["xs_row"], z["ws_row"], 0, m, 256))
    assert rel_fro(y[:tot], z["y_row"][:tot]) <= 2e-2

    z = np.load(os.path.join(GOLD, "w4a16_tiny.npz"))
    for zo in (0, 1):
        for M in (1, 16):
            c = H.from_bf16(H.w4a16(H.to_bf16(z["a"][:M]), z["qweight"], H.to_bf16(z["scales"]), z["qzeros"], 128, zo))
            assert rel_fro(c, z[f"c_zo{zo}_m{M}"]) <= 2e-2

    kat = json.load(open(os.path.join(GOLD, "moe_align_kat.json")))
    flat = np.array(kat["topk_ids"], dtype=np.int32).ravel() - 1   # the docstring numbers experts from 1
    perm, ms, off = H.route_group(flat, kat["num_experts"])
    s, e, post = H.align_block_size(perm, ms, kat["block_size"])
    assert post == 16 and s[:post].tolist() == kat["sorted_token_ids"] and e[:4].tolist() == [0, 1, 2, 3]


FUZZ = [  # (compute units, load-landing model, wave order seed): few units = long tile sequences per workgroup
    ("1", "late", "0"), ("2", "early", "0"), ("3", "late", "5"), ("8", "early", "9"), ("16", "late", "0"), ("5", "late", "77")]
GUARDED = [("end", "8", "late", "0"), ("start", "8", "early", "3"), ("end", "2", "late", "11"), ("start", "13", "late", "0")]
UBSAN_ENV = dict(EMU_UBSAN="1", EMU_OUT=os.path.join(EMU, "_build", "ubsan"), EMU_GUARD="end", EMU_TRACE="1")


def _child(script, args, **env):
    return subprocess.Popen([sys.executable, os.path.join(EMU, script)] + list(args), env=dict(os.environ, **env), stdout=subprocess.PIPE,
                            stderr=subprocess.STDOUT, cwd=ROOT)


@pytest.fixture(scope="module", autouse=True)
def children():
    """The random-launch runs of this file are child processes of their own; they are started when the first test of the
    file runs (the emulated library is built by then) and collected by the tests at its end, so that they run beside
    the tests in between instead of after them."""
    build_emu.build()
    c = {}
    for i, (cus, dma, seed) in enumerate(FUZZ):
        c["pingpong", i] = _child("fuzz_pingpong.py", [str(100 + i), "20"], EMU_CUS=cus, EMU_DMA=dma, EMU_SEED=seed, EMU_TILE_ORDER=str(i % 2))
    for i, (guard, cus, dma, seed) in enumerate(GUARDED):
        env = dict(EMU_GUARD=guard, EMU_CUS=cus, EMU_DMA=dma, EMU_SEED=seed, EMU_TRACE="1", EMU_TILE_ORDER=str(i % 2))
        if i >= 2:
            env["EMU_LDS_POISON"] = "1"      # workgroups start with NaN patterns in LDS instead of a predecessor's data
        c["guarded", i] = _child("fuzz_all.py", [str(200 + i), "40"], **env)
    for order in ("0", "1"):
        c["corrupt", order] = _child("corrupt_sizes.py", [], EMU_GUARD="end", EMU_TRACE="1", EMU_TILE_ORDER=order)
    c["ubsan build"] = _child("build_emu.py", [], **UBSAN_ENV)     # the build with trapping checks; its runs follow in the test
    yield c
    for p in c.values():
        if p.poll() is None:
            p.kill()


def test_pingpong_random_shapes_over_unit_counts_and_schedules(children):
    for i, cfg in enumerate(FUZZ):
        p = children["pingpong", i]
        log = p.communicate()[0].decode()
        assert p.returncode == 0, (cfg, log[-2000:])


def test_every_entry_point_on_random_shapes_with_tensors_against_guard_pages(children):
    """Inputs, outputs and the workspace end (or begin) at an inaccessible page: a kernel that touches memory outside a
    tensor, by one element or by one 16-byte load, ends the child process with a memory fault. Two of the four runs
    start every workgroup with LDS full of NaN patterns: a result that depends on LDS bytes its workgroup never wrote
    fails the comparison."""
    for i, cfg in enumerate(GUARDED):
        p = children["guarded", i]
        log = p.communicate()[0].decode()
        assert p.returncode == 0, (cfg, log[-2000:])


@pytest.mark.skipif(not os.environ.get("EMU_FULL_SIZE"), reason="20-40 minutes per case on one core each: set EMU_FULL_SIZE=1")
def test_config2_at_full_size():
    """Benchmark config 2 at its real size with 256 emulated CUs (tests/emu/full_size.py): the ping-pong kernel in the
    split-tail order, the four-wave kernel in both orders and its tall-tile form reproduce the exact bf16 output; the
    four-wave forms of the fused first GEMM give the default kernel's bits."""
    cases = [("gemm", "0", "1"), ("gemm", "7", "0"), ("gemm", "7", "1"), ("gemm", "8", "0"), ("swiglu", "7", "0"), ("swiglu", "8", "0")]
    procs = [subprocess.Popen([sys.executable, os.path.join(EMU, "full_size.py"), kind, variant],
                              env=dict(os.environ, EMU_CUS="256", EMU_TILE_ORDER=order), stdout=subprocess.PIPE,
                              stderr=subprocess.STDOUT, cwd=ROOT) for kind, variant, order in cases]
    for case, p in zip(cases, procs):
        log = p.communicate()[0].decode()
        assert p.returncode == 0, (case, log[-2000:])


def test_kernels_with_trapping_checks_of_alignment_shifts_overflow_and_bounds(children):
    """A second host build of the kernels in which every vector access checks its alignment, every shift its count,
    every signed operation its range and every index into a fixed-size array its bound, each ending in a trap
    (EMU_UBSAN, tests/emu/build_emu.py): 80 random calls over all entry points, against guard pages, complete
    without one. (An ordinary build would read a misaligned 16-byte LDS access without complaint; the GPU would not.)"""
    b = children["ubsan build"]
    log = b.communicate()[0].decode()
    assert b.returncode == 0, log[-2000:]
    procs = [_child("fuzz_all.py", [str(700 + i), "40"], EMU_TILE_ORDER=str(i), EMU_SEED=str(3 * i), **UBSAN_ENV) for i in range(2)]
    for i, p in enumerate(procs):
        log = p.communicate()[0].decode()
        assert p.returncode == 0, (i, log[-2000:])


def test_corrupt_m_sizes_are_clamped_by_every_kernel(children):
    """Negative sizes, sums beyond M, a size of 2^30: every kernel that reads m_sizes (all GEMM variants, fp8, SwiGLU,
    backward, W4A16 grouped) computes the rows of the clamped sizes, leaves the other rows alone and, with every tensor
    against a guard page, touches nothing outside them."""
    for order in ("0", "1"):
        p = children["corrupt", order]
        log = p.communicate()[0].decode()
        assert p.returncode == 0, (order, log[-2000:])


def test_no_data_race_between_the_waves_of_a_workgroup():
    """The kernels compiled under ThreadSanitizer with every wave as one of its fibers (tests/emu/race_check.cpp): every
    entry point runs without a report, i.e. each pair of accesses by two waves to the same LDS or global bytes is
    ordered by a barrier - also where the emulation happens to run them in a harmless order. Two control kernels
    show that the check sees a missing barrier, after ordinary stores and after a global->LDS load."""
    exe = build_emu.build_race_check()
    for kernel in ("0", "1"):
        clean = subprocess.run([exe, "selftest", kernel, "1"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
        racy = subprocess.run([exe, "selftest", kernel, "0"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
        assert clean.returncode == 0 and b"data race" not in clean.stdout, clean.stdout.decode()[-1500:]
        assert racy.returncode == 66 and b"data race" in racy.stdout, racy.stdout.decode()[-1500:]
    procs = [subprocess.Popen([exe], env=dict(os.environ, EMU_CUS=cus, EMU_SEED=seed, EMU_TILE_ORDER=order), stdout=subprocess.PIPE,
                              stderr=subprocess.STDOUT)
             for cus, seed, order in (("8", "0", "0"), ("2", "7", "1"))]
    # long tile sequences in one workgroup: split tails, row pieces of the last round, short and empty experts
    shapes = [("bf16", "512", "128", "1", "0", ["530", "300", "0", "70"]), ("swiglu", "256", "128", "2", "5", ["833", "64", "257"]),
              ("gather", "128", "128", "2", "3", ["530", "1", "300"]),
              ("fp8block", "384", "256", "1", "0", ["577", "33", "320"]), ("fp8row", "256", "128", "3", "9", ["129", "768", "1"]),
              ("f16", "384", "256", "2", "0", ["321", "511"]), ("bwd", "256", "128", "3", "4", ["300", "0", "41", "513"]),
              ("bf16w4", "512", "192", "1", "0", ["530", "300", "0", "70"]), ("f16w4", "384", "64", "2", "6", ["321", "511", "1"]),
              ("swigluw4", "192", "128", "2", "1", ["300", "70", "0", "257"]),
              ("bf16tall", "512", "192", "1", "0", ["530", "288", "0", "70", "257"]), ("swiglutall", "192", "128", "2", "1", ["270", "70", "0", "513"])]
    for i, (op, N, K, cus, seed, sizes) in enumerate(shapes):
        for order in ("0", "1"):
            procs.append(subprocess.Popen([exe, "shape", op, N, K] + sizes,
                                          env=dict(os.environ, EMU_CUS=cus, EMU_SEED=seed, EMU_TILE_ORDER=order),
                                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT))
    for p in procs:
        log = p.communicate()[0].decode()
        assert p.returncode == 0 and "data race" not in log and " rc 0" in log, log[-3000:]
        assert "calls that returned an error" not in log or "calls that returned an error: 0" in log, log[-3000:]
