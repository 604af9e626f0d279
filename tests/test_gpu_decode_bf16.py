"""GPU parity of the small-M (decode) bf16 grouped GEMM path against the CPU oracle (rtol = atol = 1e-2)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import to_np

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2
DECODE = 5  # MOE_GG_GG_DECODE


def run(x, w, m_sizes, variant):
    import applied_ai_amd as A

    lib = A._lib.lib()
    lib.moe_gg_set_variant(0, variant)
    try:
        y = A.grouped_gemm(x.cuda(), w.cuda(), torch.tensor(m_sizes, dtype=torch.int32, device="cuda"))
        torch.cuda.synchronize()
    finally:
        lib.moe_gg_set_variant(0, -1)
    return y


@pytest.mark.parametrize("G,N,K,m_sizes", [
    (8, 512, 256, [3, 0, 0, 9, 16, 0, 11, 25]),   # empties, a 16-row expert, one above 16 rows (two passes)
    (8, 1024, 1024, [8] * 8),
    (4, 328, 384, [0, 30, 1, 70]),                # N not a multiple of the 64-column block
    (2, 256, 128, [40, 3]),
    (1, 64, 128, [1]),
])
@pytest.mark.parametrize("variant", [DECODE, -1])
def test_decode_small(G, N, K, m_sizes, variant):
    print(f"case G={G} N={N} K={K} m_sizes={m_sizes} variant={variant}", flush=True)
    gen = torch.Generator().manual_seed(G * 100 + N + K)
    M = sum(m_sizes)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    w = (torch.randn(G * N, K, generator=gen) * 0.05).to(torch.bfloat16)
    y = to_np(run(x, w, m_sizes, variant))
    ref = O.grouped_gemm(to_np(x), to_np(w), m_sizes)
    np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("down", [False, True])
def test_mixtral_decode_shapes(down):
    """benchmark config 3: T=32 top-2 over 8 experts (64 rows); up-proj K=4096, N=14336 and down-proj K=14336,
    N=4096. Oracle on every row for a 512-column slice per expert; bitwise determinism; and the auto-dispatch picks
    the same result as the pinned decode variant."""
    from applied_ai_amd import configs

    c = configs.cfg3(down)
    m_sizes = c["m_sizes"].tolist()
    K, N = (14336, 4096) if down else (4096, 14336)
    print(f"cfg3 down={down} m_sizes={m_sizes}", flush=True)
    y = run(c["x_sorted"], c["w"], m_sizes, DECODE)
    y2 = run(c["x_sorted"], c["w"], m_sizes, -1)
    assert torch.equal(y, y2)
    off = O.offsets(m_sizes)
    cols = slice(1024, 1536)
    for g in range(8):
        if m_sizes[g] == 0:
            continue
        xr = c["x_sorted"][off[g]:off[g + 1]].float().numpy()
        wr = c["w"][g * N:(g + 1) * N][cols].float().numpy()
        ref = O.grouped_gemm(xr, wr, [m_sizes[g]])
        np.testing.assert_allclose(to_np(y[off[g]:off[g + 1], cols]), ref, rtol=RTOL, atol=ATOL)


def test_forced_empty_experts_leave_rows_untouched():
    """Config 3 with two experts forced empty: their weights are skipped and rows beyond sum(m_sizes) stay as they were."""
    import applied_ai_amd as A

    G, N, K = 8, 256, 512
    m_sizes = [7, 0, 12, 16, 0, 5, 9, 3]
    M = sum(m_sizes) + 4
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16).cuda()
    w = (torch.randn(G * N, K, generator=gen) * 0.05).to(torch.bfloat16).cuda()
    y = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
    lib = A._lib.lib()
    lib.moe_gg_set_variant(0, DECODE)
    try:
        ms = torch.tensor(m_sizes, dtype=torch.int32, device="cuda")   # bound to a name: it must outlive the launch
        rc = lib.moe_gg_grouped_gemm_bf16(x.data_ptr(), w.data_ptr(), y.data_ptr(), ms.data_ptr(), G, M, N, K, N, 0,
                                          torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
    finally:
        lib.moe_gg_set_variant(0, -1)
    assert rc == 0
    ref = O.grouped_gemm(to_np(x), to_np(w), m_sizes)
    tot = sum(m_sizes)
    np.testing.assert_allclose(to_np(y)[:tot], ref[:tot], rtol=RTOL, atol=ATOL)
    assert (to_np(y)[tot:] == 3.0).all()
