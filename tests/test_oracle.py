"""Pins the CPU oracle (oracle/moe_oracle.c) against the reference's own known answers, closed forms,
independent library routines and brute force - never against a retyped copy of its own formula."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

GOLD = os.path.join(os.path.dirname(__file__), "golden")


# ---- offsets -------------------------------------------------------------------------------------
@pytest.mark.parametrize("m_sizes", [
    [25, 50, 25],          # dev/triton_groupGEMM/testing/unit_tests.py:122
    [4, 4],                # unit_tests.py:139
    [32] * 4,              # unit_tests.py:224
    [1024, 1024],          # unit_tests.py:243
    [52] * 4 + [51] * 16,  # kernels/MoE/group_GEMM/triton/testing/fast_verification.py:43-48 (M=1024, G=20)
    [0, 7, 0, 0, 3],       # empty groups (base_testing.py:106-116 produces them)
])
def test_offsets_match_cumsum(m_sizes):
    off = O.offsets(m_sizes)
    assert off.dtype == np.int32
    assert off.tolist() == [0] + np.cumsum(m_sizes).tolist()


def test_fast_verification_split_is_1024():
    assert O.offsets([52] * 4 + [51] * 16)[-1] == 1024


# ---- routing -------------------------------------------------------------------------------------
def test_moe_align_docstring_known_answer():
    # Worked example in kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:157-165
    # (experts are numbered from 1 there, 4 experts, block 4).
    kat = json.load(open(os.path.join(GOLD, "moe_align_kat.json")))
    ids = np.array(kat["topk_ids"]) - 1
    sorted_ids, expert_ids, post = O.moe_align_block_size(ids, kat["block_size"], kat["num_experts"])
    assert sorted_ids[:post].tolist() == kat["sorted_token_ids"]
    assert post == 16
    assert expert_ids[:4].tolist() == [0, 1, 2, 3]


def test_route_equals_stable_argsort_and_bincount():
    rng = np.random.default_rng(0)
    for E, n in [(8, 512), (256, 4096), (4, 1), (3, 0)]:
        flat = rng.integers(0, E, size=n).astype(np.int32)
        perm, m = O.route(flat, E)
        assert perm.tolist() == np.argsort(flat, kind="stable").tolist()
        assert m.tolist() == np.bincount(flat, minlength=E).tolist()


def test_route_drops_masked_ids_and_marks_the_tail():
    # ids outside [0, E) belong to no expert: stable argsort over the valid positions, then a tail of -1.
    rng = np.random.default_rng(5)
    E, n = 6, 200
    flat = rng.integers(0, E, size=n).astype(np.int32)
    flat[rng.permutation(n)[:37]] = -1
    flat[[3, 77]] = [E, E + 9]
    perm, m = O.route(flat, E)
    valid = np.nonzero((flat >= 0) & (flat < E))[0]
    expect = valid[np.argsort(flat[valid], kind="stable")]
    assert perm[:len(valid)].tolist() == expect.tolist()
    assert (perm[len(valid):] == -1).all() and len(valid) == n - 39
    assert m.tolist() == np.bincount(flat[valid], minlength=E).tolist()


def test_route_matches_mask_loop_grouping():
    # The reference oracle groups rows with `mask = topk_ids == i` (test_moe_gemm.py:24-29): rows of
    # expert i in increasing flat order.
    rng = np.random.default_rng(1)
    ids = rng.integers(0, 5, size=(40, 2)).astype(np.int32)
    perm, m = O.route(ids, 5)
    flat = ids.reshape(-1)
    expect = np.concatenate([np.nonzero(flat == e)[0] for e in range(5)])
    assert perm.tolist() == expect.tolist()


def test_topk_against_numpy_and_torch():
    rng = np.random.default_rng(2)
    lg = rng.standard_normal((300, 64)).astype(np.float32)
    ids = O.topk(lg, 6)
    expect = np.argsort(-lg, axis=1, kind="stable")[:, :6]
    assert np.array_equal(ids, expect)
    tk = torch.topk(torch.from_numpy(lg), 6).indices.numpy()
    assert np.array_equal(ids, tk)


def test_topk_ties_go_to_lower_index():
    lg = np.array([[1.0, 3.0, 3.0, 0.0, 3.0]], dtype=np.float32)
    assert O.topk(lg, 3).tolist() == [[1, 2, 4]]


# ---- grouped GEMM --------------------------------------------------------------------------------
def test_grouped_gemm_single_group_is_dense_matmul():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((32, 32)).astype(np.float32)
    w = rng.standard_normal((32, 32)).astype(np.float32)
    y = O.grouped_gemm(x, w, [32])  # unit_tests.py:110-116
    np.testing.assert_allclose(y, x.astype(np.float64) @ w.astype(np.float64).T, rtol=1e-6, atol=1e-6)


def test_grouped_gemm_brute_force_8x8x8():
    rng = np.random.default_rng(4)
    x = rng.integers(-3, 4, size=(8, 8)).astype(np.float32)   # integers: exact in any order
    w = rng.integers(-3, 4, size=(16, 8)).astype(np.float32)  # G=2, N=8 (unit_tests.py:136-149)
    y = O.grouped_gemm(x, w, [4, 4])
    for i in range(8):
        g = i // 4
        for n in range(8):
            assert y[i, n] == sum(x[i, k] * w[g * 8 + n, k] for k in range(8))


def test_grouped_gemm_vs_torch_loop_and_empty_groups():
    rng = np.random.default_rng(5)
    m_sizes = [0, 37, 0, 90, 1]
    x = rng.standard_normal((130, 64)).astype(np.float32)  # two trailing rows belong to no group
    w = rng.standard_normal((5 * 48, 64)).astype(np.float32)
    y = O.grouped_gemm(x, w, m_sizes)
    t = O.grouped_gemm_torch_loop(torch.from_numpy(x), torch.from_numpy(w), m_sizes).numpy()
    np.testing.assert_allclose(y[:128], t[:128], rtol=1e-5, atol=1e-5)
    assert np.isnan(y[128:]).all()  # untouched


def test_grouped_gemm_group_permutation_permutes_blocks():
    rng = np.random.default_rng(6)
    m_sizes = [10, 20, 5]
    N, K = 16, 32
    x = rng.standard_normal((35, K)).astype(np.float32)
    w = rng.standard_normal((3 * N, K)).astype(np.float32)
    y = O.grouped_gemm(x, w, m_sizes)
    order = [2, 0, 1]
    off = [0, 10, 30, 35]
    xp = np.concatenate([x[off[g]:off[g + 1]] for g in order])
    wp = np.concatenate([w[g * N:(g + 1) * N] for g in order])
    yp = O.grouped_gemm(xp, wp, [m_sizes[g] for g in order])
    expect = np.concatenate([y[off[g]:off[g + 1]] for g in order])
    assert np.array_equal(yp, expect)


def test_grouped_gemm_block_layout():
    rng = np.random.default_rng(7)
    m_sizes = [3, 0, 5]
    N, K = 8, 16
    x = rng.standard_normal((8, K)).astype(np.float32)
    w = rng.standard_normal((3 * N, K)).astype(np.float32)
    y = O.grouped_gemm(x, w, m_sizes)
    yb = O.grouped_gemm(x, w, m_sizes, block_layout=True)  # fast_verification.py:83-96
    assert yb.shape == (8, 24)
    assert np.array_equal(yb[0:3, 0:8], y[0:3])
    assert np.array_equal(yb[3:8, 16:24], y[3:8])
    assert np.isnan(yb[0:3, 8:]).all() and np.isnan(yb[3:8, :16]).all()


# ---- W4A16 ---------------------------------------------------------------------------------------
def _unpack_independent(qweight, qzeros, K, N, group):
    """Bit twiddling written independently of the C oracle: view words as bytes, split nibbles."""
    qb = qweight.view(np.uint8).reshape(K // 8, N, 4)           # little endian bytes of each word
    nib = np.stack([qb & 0xF, qb >> 4], axis=-1).reshape(K // 8, N, 8)  # nibble j = row 8*i + j
    q = nib.transpose(0, 2, 1).reshape(K, N)
    zb = qzeros.view(np.uint8).reshape(K // group, N // 8, 4)
    z = np.stack([zb & 0xF, zb >> 4], axis=-1).reshape(K // group, N)   # nibble j = column 8*i + j
    return q.astype(np.int64), z.astype(np.int64)


@pytest.mark.parametrize("zero_offset", [0, 1])
def test_w4_dequant_brute_force(zero_offset):
    rng = np.random.default_rng(8)
    K, N, group = 256, 16, 128
    qweight = rng.integers(-2**31, 2**31, size=(K // 8, N), dtype=np.int64).astype(np.int32)
    qzeros = rng.integers(-2**31, 2**31, size=(K // group, N // 8), dtype=np.int64).astype(np.int32)
    scales = rng.uniform(0.005, 0.02, size=(K // group, N)).astype(np.float32)
    w = O.w4_dequant(qweight, scales, qzeros, group, zero_offset)
    q, z = _unpack_independent(qweight, qzeros, K, N, group)
    s = np.repeat(scales, group, axis=0)
    zz = np.repeat(z, group, axis=0)
    expect = (q.astype(np.float32) * s - (zz + zero_offset).astype(np.float32) * s)
    assert np.array_equal(w, expect)


def test_w4_pack_roundtrip_and_special_cases():
    rng = np.random.default_rng(9)
    K, N = 128, 8
    q = rng.integers(0, 16, size=(K, N))
    z = rng.integers(0, 16, size=(1, N))
    s = np.full((1, N), 0.5, dtype=np.float32)
    w = O.w4_dequant(O.pack_int4_along_k(q), s, O.pack_int4_along_n(z), 128, 0)
    assert np.array_equal(w, (q - z) * 0.5)
    # q == z + 1 with the reference's (z + 1) convention gives exactly zero weights
    qq = np.tile(np.minimum(z + 1, 15), (K, 1))
    zz = qq[:1] - 1
    w0 = O.w4_dequant(O.pack_int4_along_k(qq), s, O.pack_int4_along_n(zz), 128, 1)
    assert (w0 == 0).all()
    # nibble order: only row 3 (k % 8 == 3) non-zero -> bits 12..15 of word 0
    one = np.zeros((8, 8), dtype=np.int64); one[3, :] = 0xA
    assert (O.pack_int4_along_k(one).view(np.uint32) == 0xA000).all()


def test_w4a16_gemm_is_dense_product_of_dequant():
    rng = np.random.default_rng(10)
    M, K, N = 5, 256, 24
    a = rng.standard_normal((M, K)).astype(np.float32)
    q = rng.integers(0, 16, size=(K, N)); z = rng.integers(0, 16, size=(K // 128, N))
    s = rng.uniform(0.005, 0.02, size=(K // 128, N)).astype(np.float32)
    qw, qz = O.pack_int4_along_k(q), O.pack_int4_along_n(z)
    c = O.w4a16_gemm(a, qw, s, qz, 128, 1)
    w = O.w4_dequant(qw, s, qz, 128, 1)
    np.testing.assert_allclose(c, a.astype(np.float64) @ w.astype(np.float64), rtol=1e-6, atol=1e-6)


# ---- fp8 -----------------------------------------------------------------------------------------
def test_e4m3_decode_all_codes_vs_torch():
    codes = np.arange(256, dtype=np.uint8)
    t = torch.from_numpy(codes.copy()).view(torch.float8_e4m3fn).float().numpy()
    o = O.e4m3_to_f32(codes)
    assert np.array_equal(np.isnan(t), np.isnan(o))
    assert np.array_equal(t[~np.isnan(t)], o[~np.isnan(o)])
    assert np.signbit(o[0x80]) and o[0x7E] == 448.0 and o[0x01] == 2.0 ** -9


def test_e4m3_encode_vs_torch():
    rng = np.random.default_rng(11)
    x = rng.standard_normal(20000) * rng.choice([1e-3, 0.01, 1.0, 30.0, 200.0], 20000)
    x = np.concatenate([x, [0.0, -0.0, 448.0, -448.0, 2.0**-9, 2.0**-10, 3 * 2.0**-11, 0.0175, 464.0, 1e9]])
    x = np.clip(x, -448, 448).astype(np.float32)
    t = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(O.f32_to_e4m3(x), t)
    # midpoints round to even: 1.0625 is halfway between 1.0 (0x38) and 1.125 (0x39)
    assert O.f32_to_e4m3(np.float32([1.0625, 1.1875])).tolist() == [0x38, 0x3A]


def test_fp8_groupwise_quant_closed_form():
    x = np.zeros((2, 256), dtype=np.float32)
    x[0, :128] = np.linspace(-2.0, 2.0, 128)
    x[0, 5] = 7.0        # amax of group 0
    x[1, 128:] = -3.5    # group 3: constant
    q, s = O.fp8_groupwise_quant(x, 128)
    assert s.shape == (2, 2)
    assert s[0, 0] == np.float32(7.0) / np.float32(448.0)
    assert q[0, 5] == 0x7E                                  # amax maps to +448
    assert s[0, 1] == np.float32(1e-12) / np.float32(448.0) and (q[0, 128:] == 0).all()
    assert (q[1, 128:] == 0xFE).all()                       # -448
    deq = O.e4m3_to_f32(q) * np.repeat(s, 128, axis=1)
    assert np.abs(deq - x).max() <= 7.0 / 448.0 * 16        # half a spacing at the top binade


# ---- 128 x 128 weight block quantiser ------------------------------------------------------------
# The reference takes this step from an un-vendored package, so it is pinned by what the rule fixes: constructed
# blocks with known scale and codes, the block -> (row block, K block) index order on a non-square grid of blocks,
# agreement with the pinned 1 x 128 quantiser where the two must coincide, and independent library routines
# (numpy reshape / max for the scales, torch's e4m3 cast for the codes).
def test_fp8_block_quant_weight_spikes_and_zero_block():
    rows, K = 256, 384                                       # 2 x 3 blocks: a transposed scale index would show
    w = np.zeros((rows, K), dtype=np.float32)
    spikes = {(0, 0): (5, 17, 3.0), (0, 1): (127, 128 + 0, -0.75), (0, 2): (64, 256 + 127, 1e-3),
              (1, 0): (128 + 1, 99, 448.0), (1, 2): (255, 383, -1e4)}   # block (1, 1) stays all zero
    rng = np.random.default_rng(21)
    for (bi, bj), (r, c, v) in spikes.items():
        blk = w[bi * 128:(bi + 1) * 128, bj * 128:(bj + 1) * 128]
        blk[:] = rng.uniform(-0.5, 0.5, blk.shape).astype(np.float32) * np.float32(abs(v))
        w[r, c] = v
    q, s = O.fp8_block_quant_weight(w, 128)
    assert q.shape == (rows, K) and q.dtype == np.uint8 and s.shape == (2, 3) and s.dtype == np.float32
    for (bi, bj), (r, c, v) in spikes.items():
        assert s[bi, bj] == np.float32(abs(v)) / np.float32(448.0)
        assert q[r, c] == (0x7E if v > 0 else 0xFE)          # the block's amax maps to +-448
    assert s[1, 1] == np.float32(1e-12) / np.float32(448.0)
    assert (q[128:, 128:256] == 0).all()
    # every other element of a block is below the spike, so no other code reaches the top binade's last step
    assert ((q & 0x7F) == 0x7E).sum() == len(spikes)
    deq = O.e4m3_to_f32(q) * np.kron(s, np.ones((128, 128), dtype=np.float32))
    err = np.abs(deq - w)
    bound = np.kron(s, np.ones((128, 128), dtype=np.float32)) * 16   # half a spacing of the top binade (32 / 2)
    assert (err <= bound).all()


def test_fp8_block_quant_weight_vs_numpy_and_torch_cast():
    rng = np.random.default_rng(22)
    rows, K = 384, 256
    w = (rng.standard_normal((rows, K)) * 0.02).astype(np.float32)
    w[130, 7] = 0.9                                          # one dominant block
    q, s = O.fp8_block_quant_weight(w, 128)
    amax = np.abs(w).reshape(rows // 128, 128, K // 128, 128).max(axis=(1, 3))
    s_np = np.maximum(amax, np.float32(1e-12)).astype(np.float32) / np.float32(448.0)
    assert s_np.dtype == np.float32 and np.array_equal(s, s_np)
    y = np.clip(w / np.repeat(np.repeat(s_np, 128, axis=0), 128, axis=1), -448, 448).astype(np.float32)
    codes = torch.from_numpy(y).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(q, codes)


def test_fp8_block_quant_weight_equals_groupwise_when_rows_share_amax():
    # Every row of every block holds its block's largest magnitude, so the 1 x 128 groups of the (pinned)
    # activation quantiser see the same amax as the 128 x 128 block: codes and scales must coincide.
    rng = np.random.default_rng(23)
    rows, K = 128, 256
    w = rng.uniform(-1.0, 1.0, (rows, K)).astype(np.float32)
    for bj, top in enumerate([1.5, 0.031]):
        w[:, bj * 128:(bj + 1) * 128] *= np.float32(top) * np.float32(0.99)
        w[np.arange(rows), bj * 128 + rng.integers(0, 128, rows)] = np.float32(top) * rng.choice([-1.0, 1.0], rows)
    qb, sb = O.fp8_block_quant_weight(w, 128)
    qg, sg = O.fp8_groupwise_quant(w, 128)
    assert np.array_equal(qb, qg)
    assert np.array_equal(sg, np.repeat(sb, rows, axis=0))


def test_fp8_block_quant_weight_scale_equivariance():
    # Scaling a block by a power of two scales its scale and leaves its codes alone; other blocks do not move.
    rng = np.random.default_rng(24)
    w = (rng.standard_normal((128, 256)) * 0.02).astype(np.float32)
    q0, s0 = O.fp8_block_quant_weight(w, 128)
    w2 = w.copy()
    w2[:, 128:] *= np.float32(8.0)
    q1, s1 = O.fp8_block_quant_weight(w2, 128)
    assert np.array_equal(q0, q1)
    assert s1[0, 0] == s0[0, 0] and s1[0, 1] == s0[0, 1] * np.float32(8.0)


def test_fp8_gemm_unit_scales_reduces_to_plain_gemm():
    rng = np.random.default_rng(12)
    M, N, K, G = 12, 128, 256, 2
    xq = rng.integers(0, 0x78, size=(M, K)).astype(np.uint8)
    wq = (rng.integers(0, 0x70, size=(G * N, K)) | rng.integers(0, 2, size=(G * N, K)) * 0x80).astype(np.uint8)
    m_sizes = [5, 7]
    plain = O.grouped_gemm(O.e4m3_to_f32(xq), O.e4m3_to_f32(wq), m_sizes)
    row = O.grouped_gemm_fp8(xq, wq, np.ones(M), np.ones(G * N), m_sizes, 0)
    blk = O.grouped_gemm_fp8(xq, wq, np.ones((M, K // 128)), np.ones((G * N // 128, K // 128)), m_sizes, 1)
    np.testing.assert_allclose(row, plain, rtol=1e-6)
    np.testing.assert_allclose(blk, plain, rtol=1e-6)


def test_fp8_rowwise_closed_form_of_reference_test():
    # dev/triton_groupGEMM/testing/base_testing.py:83-88
    rng = np.random.default_rng(13)
    M, N, K, G = 9, 16, 128, 3
    xq = rng.integers(0, 0x70, size=(M, K)).astype(np.uint8)
    wq = rng.integers(0, 0x70, size=(G * N, K)).astype(np.uint8)
    xs = rng.uniform(0.01, 0.1, M).astype(np.float32); ws = rng.uniform(0.01, 0.1, G * N).astype(np.float32)
    m_sizes = [2, 3, 4]
    y = O.grouped_gemm_fp8(xq, wq, xs, ws, m_sizes, 0)
    xf = torch.from_numpy(xq).view(torch.float8_e4m3fn).double(); wf = torch.from_numpy(wq).view(torch.float8_e4m3fn).double()
    start = 0
    for g, m in enumerate(m_sizes):
        e = xf[start:start + m] @ wf[g * N:(g + 1) * N].T * torch.from_numpy(xs[start:start + m]).double()[:, None] \
            * torch.from_numpy(ws[g * N:(g + 1) * N]).double()[None, :]
        np.testing.assert_allclose(y[start:start + m], e.numpy(), rtol=1e-6)
        start += m


def test_fp8_block_scales_dequantise_then_gemm():
    rng = np.random.default_rng(14)
    M, N, K, G = 6, 128, 256, 2
    x = rng.standard_normal((M, K)).astype(np.float32); w = (rng.standard_normal((G * N, K)) * 0.02).astype(np.float32)
    xq, xs = O.fp8_groupwise_quant(x); wq, ws = O.fp8_block_quant_weight(w)
    m_sizes = [4, 2]
    y = O.grouped_gemm_fp8(xq, wq, xs, ws, m_sizes, 1)
    xd = O.e4m3_to_f32(xq) * np.repeat(xs, 128, axis=1)
    wd = O.e4m3_to_f32(wq) * np.repeat(np.repeat(ws, 128, axis=0), 128, axis=1)
    np.testing.assert_allclose(y, O.grouped_gemm(xd, wd, m_sizes), rtol=1e-5, atol=1e-7)
    # and the quantised product is close to the unquantised one
    ref = O.grouped_gemm(x, w, m_sizes)
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 5e-2


def test_round_bf16_vs_torch():
    rng = np.random.default_rng(15)
    x = (rng.standard_normal(10000) * rng.choice([1e-5, 1.0, 1e5], 10000)).astype(np.float32)
    x = np.concatenate([x, np.float32([1.00390625, 1.01171875, 0.0, -0.0])])  # ties
    t = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(O.round_bf16(x), t)


def test_silu_and_mul_vs_torch_and_closed_forms():
    rng = np.random.default_rng(16)
    x = (rng.standard_normal((7, 24)) * 3).astype(np.float32)
    t = torch.from_numpy(x).double()
    e = torch.nn.functional.silu(t[:, :12]) * t[:, 12:]
    np.testing.assert_allclose(O.silu_and_mul(x), e.numpy(), rtol=1e-6, atol=1e-7)
    v = np.float32([[0.0, 2.5, -2.5, 1.0, 1.0, -1.0]])  # silu(0) = 0, silu(v) - silu(-v) = v
    o = O.silu_and_mul(v)[0]
    assert o[0] == 0.0 and abs(o[1] + o[2] - 2.5) < 1e-6


def test_fused_moe_vs_torch_float64_and_special_cases():
    """Pins orc_fused_moe: a float64 restatement with library matmuls (the structure of torch_moe,
    test_moe_gemm.py:16-30), one expert with weight 1 = that expert's MLP, and w2 = 0."""
    gen = torch.Generator().manual_seed(17)
    T, K, E, n, d, k = 9, 32, 4, 16, 24, 2
    a = torch.randn(T, K, generator=gen) / 3
    w1 = torch.randn(E, 2 * n, K, generator=gen) / 3
    w2 = torch.randn(E, d, n, generator=gen) / 3
    score = torch.softmax(torch.randn(T, E, generator=gen), dim=-1)
    tw, ids = torch.topk(score, k)
    exp = torch.zeros(T, d, dtype=torch.float64)
    for t in range(T):
        for j in range(k):
            e = int(ids[t, j])
            h = w1[e].double() @ a[t].double()
            h = torch.nn.functional.silu(h[:n]) * h[n:]
            exp[t] += tw[t, j].double() * (w2[e].double() @ h)
    got = O.fused_moe(a.numpy(), w1.numpy(), w2.numpy(), tw.numpy(), ids.numpy(), round_intermediate=False)
    np.testing.assert_allclose(got, exp.numpy(), rtol=1e-5, atol=1e-6)
    # the library-matmul form used for large sizes agrees too
    np.testing.assert_allclose(O.fused_moe_torch(a, w1, w2, tw, ids).numpy(), exp.numpy(), rtol=1e-4, atol=1e-5)
    # rounding the stored intermediates to bf16 moves the result by bf16-size errors only
    got_r = O.fused_moe(a.numpy(), w1.numpy(), w2.numpy(), tw.numpy(), ids.numpy(), round_intermediate=True)
    assert np.abs(got_r - exp.numpy()).max() < 2e-2
    # k = 1, weight 1: one expert's MLP
    one = O.fused_moe(a.numpy(), w1.numpy(), w2.numpy(), np.ones((T, 1), np.float32), np.full((T, 1), 2, np.int32), False)
    h = a.double() @ w1[2].double().T
    e1 = (torch.nn.functional.silu(h[:, :n]) * h[:, n:]) @ w2[2].double().T
    np.testing.assert_allclose(one, e1.numpy(), rtol=1e-5, atol=1e-6)
    assert np.all(O.fused_moe(a.numpy(), w1.numpy(), np.zeros_like(w2.numpy()), tw.numpy(), ids.numpy()) == 0)
    # ids outside [0, E) contribute nothing
    bad = ids.numpy().copy(); bad[:, 1] = E + 3
    only0 = O.fused_moe(a.numpy(), w1.numpy(), w2.numpy(), tw.numpy(), bad, False)
    first = O.fused_moe(a.numpy(), w1.numpy(), w2.numpy(), tw.numpy()[:, :1].copy(), ids.numpy()[:, :1].copy(), False)
    np.testing.assert_allclose(only0, first, rtol=1e-6)


def test_w4a16_grouped_and_int4_layer_compose_pinned_parts():
    """w4a16_grouped is w4a16_gemm per expert slice; dequant_gemm_moe is w4_dequant + fused_moe: check both against a
    direct numpy evaluation (dequantise, matmul in float64), including an empty expert and unweighted top-k sums."""
    rng = np.random.default_rng(19)
    E, K, N, gs = 3, 128, 16, 64
    q = rng.integers(0, 16, size=(E, K, N)); zz = rng.integers(0, 16, size=(E, K // gs, N))
    qw = np.stack([O.pack_int4_along_k(q[e]) for e in range(E)]); qz = np.stack([O.pack_int4_along_n(zz[e]) for e in range(E)])
    sc = rng.uniform(0.01, 0.02, size=(E, K // gs, N)).astype(np.float32)
    m_sizes = [2, 0, 3]
    a = rng.standard_normal((5, K)).astype(np.float32)
    got = O.w4a16_grouped(a, qw, sc, qz, m_sizes, gs, 1)
    w = (q - (np.repeat(zz, gs, axis=1) + 1)) * np.repeat(sc, gs, axis=1).astype(np.float64)      # [E, K, N]
    exp = np.concatenate([a[:2].astype(np.float64) @ w[0], a[2:].astype(np.float64) @ w[2]])
    np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-6)
    # layer: K -> 2n = N (n = 8), second weights n -> d
    n, d = N // 2, 16
    q2 = rng.integers(0, 16, size=(E, 64, d)); zz2 = rng.integers(0, 16, size=(E, 1, d))
    # the second product's K dimension is n = 8 < a quantisation group, so use a layer whose n is one group
    E2, K2, n2, d2, g2 = 2, 64, 64, 16, 64
    qa = rng.integers(0, 16, size=(E2, K2, 2 * n2)); za = rng.integers(0, 16, size=(E2, 1, 2 * n2)); sa = rng.uniform(0.01, 0.02, size=(E2, 1, 2 * n2)).astype(np.float32)
    qb = rng.integers(0, 16, size=(E2, n2, d2)); zb = rng.integers(0, 16, size=(E2, 1, d2)); sb = rng.uniform(0.01, 0.02, size=(E2, 1, d2)).astype(np.float32)
    pk = lambda t: np.stack([O.pack_int4_along_k(t[e]) for e in range(t.shape[0])])
    pn = lambda t: np.stack([O.pack_int4_along_n(t[e]) for e in range(t.shape[0])])
    x = (rng.standard_normal((4, K2)) / 4).astype(np.float32)
    ids = np.array([[0, 1], [1, 0], [0, 1], [1, 0]], dtype=np.int32)
    got = O.dequant_gemm_moe(x, pk(qa), pk(qb), sa, sb, pn(za), pn(zb), ids, None, g2, 1, round_intermediate=False)
    wa = (qa - (za + 1)) * sa.astype(np.float64); wb = (qb - (zb + 1)) * sb.astype(np.float64)
    exp = np.zeros((4, d2))
    for t in range(4):
        for e in ids[t]:
            h = x[t].astype(np.float64) @ wa[e]
            h = h[:n2] / (1 + np.exp(-h[:n2])) * h[n2:]
            exp[t] += h @ wb[e]
    np.testing.assert_allclose(got, exp, rtol=1e-4, atol=1e-5)


def test_grouped_gemm_backward_vs_autograd_and_closed_forms():
    # torch.autograd through the per-expert forward loop (fast_verification.py:83-99), float64.
    rng = np.random.default_rng(31)
    for G, sizes, N, K, pad in [(3, [5, 0, 9], 8, 12, 2), (4, [7, 7, 7, 7], 16, 8, 0), (1, [11], 4, 20, 0)]:
        M = sum(sizes) + pad
        x = rng.standard_normal((M, K)).astype(np.float32)
        w = rng.standard_normal((G * N, K)).astype(np.float32)
        go = rng.standard_normal((M, N * G)).astype(np.float32)
        gx, gw = O.grouped_gemm_backward(go, x, w, sizes)
        xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
        wt = torch.tensor(w, dtype=torch.float64, requires_grad=True)
        y = torch.zeros((M, N * G), dtype=torch.float64)
        s = 0
        for g, m in enumerate(sizes):
            if m > 0:
                y[s:s + m, g * N:(g + 1) * N] = xt[s:s + m] @ wt[g * N:(g + 1) * N].T
            s += m
        y.backward(torch.tensor(go, dtype=torch.float64))
        np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(gw, wt.grad.numpy(), rtol=1e-5, atol=1e-5)
        # rows beyond sum(m_sizes) and experts without rows get zeros
        assert not gx[sum(sizes):].any()
        for g, m in enumerate(sizes):
            if m == 0:
                assert not gw[g * N:(g + 1) * N].any()
        # adjoint identity with the pinned forward: <dY, y> = <grad_x, x> = <grad_w, w>
        yf = O.grouped_gemm(x, w, sizes, block_layout=True, fill=0.0).astype(np.float64)
        lhs = float((go.astype(np.float64) * yf).sum())
        assert abs(lhs - float((gx.astype(np.float64) * x).sum())) < 1e-3 * max(1.0, abs(lhs))
        assert abs(lhs - float((gw.astype(np.float64) * w).sum())) < 1e-3 * max(1.0, abs(lhs))
        # the [M, N] gradient layout reads the same numbers
        go_mn = np.zeros((M, N), dtype=np.float32)
        s = 0
        for g, m in enumerate(sizes):
            go_mn[s:s + m] = go[s:s + m, g * N:(g + 1) * N]
            s += m
        if G > 1:
            gx2, gw2 = O.grouped_gemm_backward(go_mn, x, w, sizes)
            np.testing.assert_array_equal(gx, gx2)
            np.testing.assert_array_equal(gw, gw2)
    # G = 1: dense products
    x = rng.standard_normal((6, 5)).astype(np.float32)
    w = rng.standard_normal((4, 5)).astype(np.float32)
    go = rng.standard_normal((6, 4)).astype(np.float32)
    gx, gw = O.grouped_gemm_backward(go, x, w, [6])
    np.testing.assert_allclose(gx, go.astype(np.float64) @ w, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(gw, go.astype(np.float64).T @ x, rtol=1e-6, atol=1e-6)


# ---- torch forms used as bench.py's CPU baselines ---------------------------------------------------
def test_w4a16_torch_form_equals_the_c_form():
    rng = np.random.default_rng(31)
    M, K, N, g = 5, 256, 64, 128
    q = rng.integers(0, 16, size=(K, N)).astype(np.uint8)
    z = rng.integers(0, 16, size=(K // g, N)).astype(np.uint8)
    sc = rng.uniform(0.005, 0.02, size=(K // g, N)).astype(np.float32)
    a = rng.standard_normal((M, K)).astype(np.float32)
    qw, qz = O.pack_int4_along_k(q), O.pack_int4_along_n(z)
    for zo in (0, 1):
        ref = O.w4a16_gemm(a, qw, sc, qz, g, zo)
        got = O.w4a16_torch(torch.from_numpy(a), torch.from_numpy(qw), torch.from_numpy(sc), torch.from_numpy(qz), g, zo)
        np.testing.assert_allclose(got.numpy(), ref, rtol=1e-4, atol=1e-4)


def test_fp8_block_torch_loop_equals_the_c_form():
    rng = np.random.default_rng(32)
    G, N, K = 3, 128, 256
    m_sizes = [4, 0, 9]
    R = sum(m_sizes)
    x = rng.standard_normal((R, K)).astype(np.float32)
    w = (rng.standard_normal((G * N, K)) * 0.02).astype(np.float32)
    xq, xs = O.fp8_groupwise_quant(x)
    wq, ws = O.fp8_block_quant_weight(w)
    ref = O.grouped_gemm_fp8(xq, wq, xs, ws, m_sizes, 1)
    got = O.grouped_gemm_fp8_block_torch_loop(torch.from_numpy(xq), torch.from_numpy(wq), torch.from_numpy(xs),
                                              torch.from_numpy(ws), m_sizes, N)
    np.testing.assert_allclose(got.numpy(), ref, rtol=1e-4, atol=1e-5)
    # a prefix of the experts only (what the bounded baseline sample does)
    got2 = O.grouped_gemm_fp8_block_torch_loop(torch.from_numpy(xq), torch.from_numpy(wq), torch.from_numpy(xs),
                                               torch.from_numpy(ws), m_sizes[:1], N)
    np.testing.assert_allclose(got2.numpy(), ref[:4], rtol=1e-4, atol=1e-5)


def test_backward_torch_loop_equals_the_c_form():
    rng = np.random.default_rng(33)
    G, N, K = 3, 24, 40
    m_sizes = [5, 0, 7]
    M = sum(m_sizes)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.standard_normal((G * N, K)).astype(np.float32)
    go = rng.standard_normal((M, N)).astype(np.float32)
    gx, gw = O.grouped_gemm_backward(go, x, w, m_sizes)
    tx, tw = O.grouped_gemm_backward_torch_loop(torch.from_numpy(go), torch.from_numpy(x), torch.from_numpy(w), m_sizes)
    np.testing.assert_allclose(tx.numpy(), gx, rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(tw.numpy(), gw, rtol=1e-4, atol=1e-4)
    # a prefix of the experts (the bounded baseline sample): their rows and weight gradients only
    tx1, tw1 = O.grouped_gemm_backward_torch_loop(torch.from_numpy(go), torch.from_numpy(x), torch.from_numpy(w), m_sizes[:1])
    np.testing.assert_allclose(tx1.numpy(), gx[:5], rtol=1e-4, atol=1e-4)
    np.testing.assert_allclose(tw1.numpy(), gw[:N], rtol=1e-4, atol=1e-4)


def test_w4a16_grouped_torch_loop_equals_the_c_form():
    rng = np.random.default_rng(34)
    E, K, N, g = 3, 256, 64, 128
    m_sizes = [4, 0, 3]
    q = rng.integers(0, 16, size=(E, K, N)).astype(np.uint8)
    z = rng.integers(0, 16, size=(E, K // g, N)).astype(np.uint8)
    sc = rng.uniform(0.005, 0.02, size=(E, K // g, N)).astype(np.float32)
    a = rng.standard_normal((sum(m_sizes), K)).astype(np.float32)
    qw = np.stack([O.pack_int4_along_k(q[e]) for e in range(E)])
    qz = np.stack([O.pack_int4_along_n(z[e]) for e in range(E)])
    ref = O.w4a16_grouped(a, qw, sc, qz, m_sizes, g, 0)
    got = O.w4a16_grouped_torch_loop(torch.from_numpy(a), torch.from_numpy(qw), torch.from_numpy(sc), torch.from_numpy(qz), m_sizes, g, 0)
    np.testing.assert_allclose(got.numpy(), ref, rtol=1e-4, atol=1e-4)
