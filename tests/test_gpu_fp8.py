"""GPU parity of the fp8 grouped GEMM (row-wise and block scales) and of the 1x128 quantiser.
GEMM: relative Frobenius error <= 2e-2 against the dequantise-then-matmul oracle; quantiser: bit-exact."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import rel_fro, to_np

pytestmark = pytest.mark.gpu
TOL = 2e-2
F8 = torch.float8_e4m3fn
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def f8(codes):
    return torch.from_numpy(np.ascontiguousarray(codes)).view(F8)


def run(xq, wq, xs, ws, m_sizes, mode):
    import applied_ai_amd as A

    fn = A.grouped_gemm_fp8_blockwise if mode == 1 else A.grouped_gemm_fp8_rowwise
    y = fn(f8(xq).cuda(), f8(wq).cuda(), torch.tensor(m_sizes, dtype=torch.int32, device="cuda"),
           torch.from_numpy(np.ascontiguousarray(xs, dtype=np.float32)).cuda(), torch.from_numpy(np.ascontiguousarray(ws, dtype=np.float32)).cuda())
    torch.cuda.synchronize()
    return y


def test_golden_fixture_block_and_rowwise():
    z = np.load(os.path.join(GOLD, "fp8_tiny.npz"))
    m = z["m_sizes"].tolist()
    tot = sum(m)
    y = run(z["xq"], z["wq"], z["xs"], z["ws"], m, 1)
    assert rel_fro(to_np(y)[:tot], z["y_block"][:tot]) <= TOL
    y = run(z["xq_row"], z["wq_row"], z["xs_row"], z["ws_row"], m, 0)
    assert rel_fro(to_np(y)[:tot], z["y_row"][:tot]) <= TOL


@pytest.mark.parametrize("mode", [0, 1])
@pytest.mark.parametrize("G,N,K,m_sizes", [
    (1, 128, 128, [16]),
    (2, 128, 256, [100, 28]),
    (4, 256, 512, [0, 300, 1, 83]),
    (8, 512, 1024, [7, 130, 64, 0, 255, 129, 33, 2]),
    (3, 384, 7168, [5, 200, 60]),
])
def test_against_oracle(mode, G, N, K, m_sizes):
    print(f"case mode={mode} G={G} N={N} K={K} m_sizes={m_sizes}", flush=True)
    rng = np.random.default_rng(G + N + K)
    M = sum(m_sizes)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((G * N, K)) * 0.05).astype(np.float32)
    if mode == 1:
        xq, xs = O.fp8_groupwise_quant(x); wq, ws = O.fp8_block_quant_weight(w)
    else:
        xs = np.abs(x).max(axis=1) / 448.0; ws = np.abs(w).max(axis=1) / 448.0
        xq = torch.from_numpy(np.clip(x / xs[:, None], -448, 448)).to(F8).view(torch.uint8).numpy()
        wq = torch.from_numpy(np.clip(w / ws[:, None], -448, 448)).to(F8).view(torch.uint8).numpy()
    y = run(xq, wq, xs, ws, m_sizes, mode)
    ref = O.grouped_gemm_fp8(xq, wq, xs, ws, m_sizes, mode)
    assert rel_fro(to_np(y), ref) <= TOL


def test_unit_scales_equal_plain_fp8_product():
    """All scales = 1: block-scaled and row-wise kernels must agree bit for bit with each other
    (same MFMA sums, scaling by 1.0 is exact) - the invariant that ties the block extension to the reference's
    row-wise kernel (dev/triton_groupGEMM/groupgemm.py:374-384)."""
    rng = np.random.default_rng(21)
    G, N, K = 2, 256, 512
    m_sizes = [37, 91]
    M = sum(m_sizes)
    xq = rng.integers(0, 0x60, size=(M, K)).astype(np.uint8) | (rng.integers(0, 2, size=(M, K)) * 0x80).astype(np.uint8)
    wq = rng.integers(0, 0x50, size=(G * N, K)).astype(np.uint8) | (rng.integers(0, 2, size=(G * N, K)) * 0x80).astype(np.uint8)
    yb = run(xq, wq, np.ones((M, K // 128)), np.ones((G * N // 128, K // 128)), m_sizes, 1)
    yr = run(xq, wq, np.ones(M), np.ones(G * N), m_sizes, 0)
    ref = O.grouped_gemm(O.e4m3_to_f32(xq), O.e4m3_to_f32(wq), m_sizes)
    assert rel_fro(to_np(yr), ref) <= 4e-3
    assert rel_fro(to_np(yb), ref) <= 4e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_quantiser_bit_exact(dtype):
    import applied_ai_amd as A

    gen = torch.Generator().manual_seed(4)
    x = (torch.randn(300, 1024, generator=gen) * torch.rand(300, 1, generator=gen) * 5).to(dtype)
    x[0, :128] = 0          # all-zero group: scale 1e-12 / 448, codes 0
    x[1, 5] = 1000.0        # outlier dominates its group
    q, s = A.float8_groupwise_quantize(x.cuda())
    torch.cuda.synchronize()
    oq, os_ = O.fp8_groupwise_quant(x.float().numpy())
    assert q.dtype == F8 and s.shape == (300, 8)
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), oq)
    assert np.array_equal(s.cpu().numpy(), os_)
    with pytest.raises(ValueError):
        A.float8_groupwise_quantize(torch.zeros(4, 100, device="cuda"))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_quantiser_bit_exact(dtype):
    """float8_blockwise_quantize_weight (128 x 128 blocks) against the oracle: codes and scales bit for bit, on a
    3 x 5 grid of blocks with an all-zero block, a dominant outlier and a block of tiny values; also a [G, N, K]
    stack, which is quantised as [G*N, K]."""
    import applied_ai_amd as A

    gen = torch.Generator().manual_seed(44)
    w = (torch.randn(384, 640, generator=gen) * 0.02).to(dtype)
    w[128:256, 256:384] = 0          # all-zero block: scale 1e-12 / 448, codes 0
    w[300, 17] = 50.0                # outlier dominates block (2, 0)
    w[0:128, 512:640] *= 1e-6        # tiny block
    q, s = A.float8_blockwise_quantize_weight(w.cuda())
    torch.cuda.synchronize()
    oq, os_ = O.fp8_block_quant_weight(w.float().numpy())
    assert q.dtype == F8 and q.shape == w.shape and s.shape == (3, 5) and s.dtype == torch.float32
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), oq)
    assert np.array_equal(s.cpu().numpy(), os_)
    q3, s3 = A.float8_blockwise_quantize_weight(w.reshape(3, 128, 640).cuda())
    assert q3.shape == (3, 128, 640) and torch.equal(q3.view(torch.uint8).reshape(384, 640), q.view(torch.uint8))
    assert torch.equal(s3, s)
    with pytest.raises(ValueError):
        A.float8_blockwise_quantize_weight(torch.zeros(100, 128, device="cuda"))


def test_config5_full_size():
    """benchmark config 5 as one launch: 256 experts, T = 4096 tokens top-8 -> 32768 rows with Zipf(1.1) routing,
    x ~ N(0,1) [32768, 7168] through the 1 x 128 quantiser, fused gate+up weights ~ N(0, 0.02) [256, 4096, 7168]
    through the 128 x 128 block quantiser (drawn and quantised expert by expert to bound memory), bf16 out.
    Checked against the dequantise-then-matmul oracle (the recipe of dev/triton_groupGEMM/testing/
    base_testing.py:83-90 with block scales) on rows of the largest expert, a mid-sized one, eight experts with at
    most 16 rows, expert 0 and the last expert, at the first, a middle and the last 128 columns; plus bitwise
    determinism, and rows at or beyond sum(m_sizes) staying untouched."""
    import applied_ai_amd as A
    from applied_ai_amd import configs

    _, _, _, m_all = configs.cfg5_routing()
    m_np = m_all.numpy()
    G, N, K = 256, 4096, 7168
    R = int(m_np.sum())
    assert R == 32768 and len(m_np) == G
    PAD = 64                                        # rows beyond sum(m_sizes): must stay as they were
    M = R + PAD
    gen = torch.Generator(device="cuda").manual_seed(1005)
    x = torch.randn(M, K, generator=gen, device="cuda")
    xq, xs = A.float8_groupwise_quantize(x)
    del x
    wq = torch.empty(G * N, K, dtype=F8, device="cuda")
    ws = torch.empty(G * N // 128, K // 128, dtype=torch.float32, device="cuda")
    for g in range(G):
        wg = torch.randn(N, K, generator=gen, device="cuda") * 0.02
        q, s = A.float8_blockwise_quantize_weight(wg)
        wq[g * N:(g + 1) * N] = q
        ws[g * N // 128:(g + 1) * N // 128] = s
    m_dev = m_all.to(torch.int32).cuda()
    SENT = 12345.0
    lib = A._lib.lib()

    def launch():
        y = torch.full((M, N), SENT, dtype=torch.bfloat16, device="cuda")
        rc = lib.moe_gg_grouped_gemm_fp8(xq.data_ptr(), wq.data_ptr(), y.data_ptr(), xs.data_ptr(), ws.data_ptr(), 1,
                                         m_dev.data_ptr(), G, M, N, K, N, 0, torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        torch.cuda.synchronize()
        return y

    print(f"cfg5 full size: G={G} rows={R} (+{PAD} pad) N={N} K={K} max m={m_np.max()} empty={(m_np == 0).sum()}", flush=True)
    y = launch()
    y2 = launch()
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))
    assert bool((y[R:] == SENT).all())
    assert not bool((y[:R] == SENT).all(dim=1).any())   # every routed row was written

    order = np.argsort(-m_np, kind="stable")
    small = [int(g) for g in np.nonzero((m_np > 0) & (m_np <= 16))[0]]
    step = max(1, len(small) // 8)
    pick = [int(order[0]), int(order[G // 4]), 0, G - 1] + small[::step][:8]
    pick = [g for g in dict.fromkeys(pick) if m_np[g] > 0]
    off = O.offsets(m_np)
    for g in pick:
        m = int(m_np[g])
        idx = sorted(set(list(range(min(m, 24))) + list(range(max(0, m - 24), m)) + [m // 2]))
        rows = torch.tensor([int(off[g]) + i for i in idx], device="cuda")
        xq_h = xq.view(torch.uint8)[rows].cpu().numpy(); xs_h = xs[rows].cpu().numpy()
        for c0 in (0, 1920, N - 128):
            wr = slice(g * N + c0, g * N + c0 + 128)
            ref = O.grouped_gemm_fp8(xq_h, wq.view(torch.uint8)[wr].cpu().numpy(), xs_h,
                                     ws[(g * N + c0) // 128:(g * N + c0) // 128 + 1].cpu().numpy(), [len(idx)], 1)
            got = to_np(y[rows, c0:c0 + 128])
            err = rel_fro(got, ref)
            assert err <= TOL, f"expert {g} ({m} rows) columns {c0}: {err}"
    print(f"cfg5 full size: checked experts {pick}", flush=True)


def test_config5_shape_sampled_experts():
    """benchmark config 5 at full K and N (7168, 4096) with its Zipf routing, on a sample of experts (largest,
    smallest, two in between): activations quantised by the GPU quantiser, weights by the block quantiser,
    oracle on a 256-column slice."""
    import applied_ai_amd as A
    from applied_ai_amd import configs

    _, _, _, m_all = configs.cfg5_routing()
    order = np.argsort(-m_all.numpy())
    pick = [int(order[0]), int(order[40]), int(order[128]), int(order[-1])]
    m_sizes = [min(int(m_all[g]), 700) for g in pick]
    print(f"cfg5 sample experts {pick} rows {m_sizes}", flush=True)
    G, N, K = len(pick), 4096, 7168
    gen = torch.Generator().manual_seed(1005)
    x = torch.randn(sum(m_sizes), K, generator=gen)
    w = torch.randn(G * N, K, generator=gen) * 0.02
    xq, xs = A.float8_groupwise_quantize(x.cuda())
    wq, ws = A.float8_blockwise_quantize_weight(w.cuda())
    y = A.grouped_gemm_fp8_blockwise(xq, wq, torch.tensor(m_sizes, dtype=torch.int32, device="cuda"), xs, ws)
    torch.cuda.synchronize()
    off = O.offsets(m_sizes)
    xq_h = xq.view(torch.uint8).cpu().numpy(); xs_h = xs.cpu().numpy()
    wq_h = wq.view(torch.uint8).cpu().numpy(); ws_h = ws.cpu().numpy()
    for gi in range(G):
        rows = slice(off[gi], min(off[gi + 1], off[gi] + 64))
        wr = slice(gi * N + 1024, gi * N + 1280)
        ref = O.grouped_gemm_fp8(xq_h[rows], wq_h[wr], xs_h[rows], ws_h[(gi * N + 1024) // 128:(gi * N + 1280) // 128],
                                 [rows.stop - rows.start], 1)
        assert rel_fro(to_np(y[rows, 1024:1280]), ref) <= TOL
    # quantised result is close to the unquantised product too
    g0 = slice(off[0], off[0] + 32)
    exact = x[g0].double() @ w[1024:1280].double().T
    assert rel_fro(to_np(y[g0, 1024:1280]), exact.numpy()) <= 6e-2


@pytest.mark.parametrize("variant", [0, 1, 2, 3])  # MOE_GG_FP8_TILED_128, _STREAM_PINGPONG, _STREAM_TILED, _PINGPONG
@pytest.mark.parametrize("mode", [0, 1])
def test_every_kernel_variant_against_oracle(variant, mode):
    """Experts of 0, 1, 64 (streaming kernel's largest), 65 (tiled kernels' smallest), 300 and 17 rows through each
    of the four kernel combinations of moe_gg_set_variant(MOE_GG_OP_GG_FP8, ...)."""
    import applied_ai_amd as A

    G, N, K = 6, 256, 512
    m_sizes = [0, 1, 64, 65, 300, 17]
    rng = np.random.default_rng(77)
    M = sum(m_sizes)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((G * N, K)) * 0.05).astype(np.float32)
    if mode == 1:
        xq, xs = O.fp8_groupwise_quant(x); wq, ws = O.fp8_block_quant_weight(w)
    else:
        xs = np.abs(x).max(axis=1) / 448.0; ws = np.abs(w).max(axis=1) / 448.0
        xq = torch.from_numpy(np.clip(x / xs[:, None], -448, 448)).to(F8).view(torch.uint8).numpy()
        wq = torch.from_numpy(np.clip(w / ws[:, None], -448, 448)).to(F8).view(torch.uint8).numpy()
    lib = A._lib.lib()
    assert lib.moe_gg_set_variant(1, variant) == 0
    try:
        y = run(xq, wq, xs, ws, m_sizes, mode)
    finally:
        lib.moe_gg_set_variant(1, -1)
    ref = O.grouped_gemm_fp8(xq, wq, xs, ws, m_sizes, mode)
    assert rel_fro(to_np(y), ref) <= TOL


@pytest.mark.parametrize("variant", [-1, 1, 2])
def test_many_experts_most_of_them_empty(variant):
    """200 experts, most without rows, a few beyond the streaming kernel's 64 rows: its grid rows are taken by the
    n-th expert within its row range, found by one wave over more experts than it has lanes."""
    import applied_ai_amd as A

    G, N, K = 200, 128, 256
    rng = np.random.default_rng(200)
    m_sizes = rng.integers(1, 9, size=G)
    m_sizes[rng.permutation(G)[:140]] = 0
    m_sizes[[0, 77, 199]] = [70, 130, 5]
    m_sizes = [int(v) for v in m_sizes]
    M = sum(m_sizes)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((G * N, K)) * 0.05).astype(np.float32)
    xq, xs = O.fp8_groupwise_quant(x); wq, ws = O.fp8_block_quant_weight(w)
    lib = A._lib.lib()
    assert lib.moe_gg_set_variant(1, variant) == 0
    try:
        y = run(xq, wq, xs, ws, m_sizes, 1)
    finally:
        lib.moe_gg_set_variant(1, -1)
    ref = O.grouped_gemm_fp8(xq, wq, xs, ws, m_sizes, 1)
    assert rel_fro(to_np(y), ref) <= TOL


def test_rowwise_block_layout_of_the_training_copy():
    """grouped_gemm_fp8_rowwise_forward writes [M, N*G]: expert g's rows in columns [g*N, (g+1)*N), the same values
    as the [M, N] entry point (kernels/MoE/group_GEMM/triton/tgroup_gemm_forward.py:468-480)."""
    import applied_ai_amd as A

    G, N, K, m_sizes = 4, 256, 512, [0, 300, 1, 83]
    rng = np.random.default_rng(9)
    M = sum(m_sizes)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((G * N, K)) * 0.05).astype(np.float32)
    xs = np.abs(x).max(axis=1) / 448.0; ws = np.abs(w).max(axis=1) / 448.0
    xq = torch.from_numpy(np.clip(x / xs[:, None], -448, 448)).to(F8).cuda()
    wq = torch.from_numpy(np.clip(w / ws[:, None], -448, 448)).to(F8).cuda()
    args = (xq, wq, torch.tensor(m_sizes, dtype=torch.int32, device="cuda"),
            torch.from_numpy(xs.astype(np.float32)).cuda(), torch.from_numpy(ws.astype(np.float32)).cuda())
    plain = A.grouped_gemm_fp8_rowwise(*args)
    wide = A.grouped_gemm_fp8_rowwise_forward(*args)
    assert wide.shape == (M, N * G)
    row = 0
    for g, m in enumerate(m_sizes):
        assert torch.equal(wide[row:row + m, g * N:(g + 1) * N], plain[row:row + m])
        row += m
    ref = O.grouped_gemm_fp8(xq.view(torch.uint8).cpu().numpy(), wq.view(torch.uint8).cpu().numpy(), xs, ws, m_sizes, 0)
    assert rel_fro(to_np(plain), ref) <= TOL
