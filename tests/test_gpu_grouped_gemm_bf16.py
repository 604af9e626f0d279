"""GPU parity of the bf16 grouped GEMM (through the C ABI) against the CPU oracle.
Tolerance: rtol 1e-2 / atol 1e-2 against the fp32 per-expert product (the bar of
kernels/MoE/group_GEMM/triton/testing/fast_verification.py:111-122)."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import bf16_inputs, random_m_sizes, to_np

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def run(x, w, m_sizes, fn=None):
    import applied_ai_amd as A

    fn = fn or A.grouped_gemm
    ms = torch.tensor(m_sizes, dtype=torch.int32, device="cuda")
    y = fn(x.cuda(), w.cuda(), ms)
    torch.cuda.synchronize()
    return y


def check(x, w, m_sizes):
    print(f"case G={len(m_sizes)} M={x.shape[0]} K={x.shape[1]} N={w.shape[0] // len(m_sizes)} m_sizes={m_sizes[:16]}", flush=True)
    y = to_np(run(x, w, m_sizes))
    ref = O.grouped_gemm(to_np(x), to_np(w), m_sizes)
    tot = sum(m_sizes)
    np.testing.assert_allclose(y[:tot], ref[:tot], rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("G", [1, 4, 16])
@pytest.mark.parametrize("M", [64, 512])
def test_reference_base_shapes(G, M):
    # dev/triton_groupGEMM/testing/base_testing.py:135-138: N = K = 256
    x, w, gen = bf16_inputs(G, M, 256, 256, seed=G * 1000 + M)
    check(x, w, random_m_sizes(G, M, gen))


@pytest.mark.parametrize("G", [4, 8])
@pytest.mark.parametrize("M", [128, 256])
@pytest.mark.parametrize("N,K", [(128, 256), (256, 128), (64, 64)])
def test_reference_various_dimensions(G, M, N, K):
    # dev/triton_groupGEMM/testing/unit_tests.py:99-103
    x, w, gen = bf16_inputs(G, M, N, K, seed=7 + G + M + N)
    check(x, w, random_m_sizes(G, M, gen))


@pytest.mark.parametrize("G,M,N,K,m_sizes", [
    (1, 32, 32, 32, [32]),              # unit_tests.py:110-116
    (3, 100, 32, 32, [25, 50, 25]),     # unit_tests.py:119-134
    (2, 8, 8, 8, [4, 4]),               # unit_tests.py:136-149
    (32, 32 * 4, 16, 16, [4] * 32),     # unit_tests.py:151-166 (G=32, N=K=16)
    (4, 128, 64, 128, [32] * 4),        # unit_tests.py:224
    (4, 700, 328, 192, [0, 300, 1, 399]),
    (5, 70, 100, 72, [0, 0, 70, 0, 0]),  # K not a multiple of 64: generic kernel
    (3, 50, 33, 40, [20, 10, 20]),       # odd N
])
def test_edge_cases(G, M, N, K, m_sizes):
    x, w, _ = bf16_inputs(G, M, N, K, seed=11)
    check(x, w, m_sizes)


@pytest.mark.parametrize("K,dtype", [(8192, torch.bfloat16), (8320, torch.bfloat16), (8192, torch.float16)])
@pytest.mark.parametrize("m_sizes", [
    [1012, 1039, 1048, 1036, 998, 1023, 1040, 996],   # the Mixtral routing of the benchmark: tails of 12-24 rows
    [1025, 1055, 1056, 1057, 1000, 1000, 1000, 1000],  # tails of 1, 31, 32, 33 rows (one and two passes)
    [40, 2008, 2000, 2000, 2048, 0, 48, 48],           # experts that are one low tile, an empty one
    [1151, 1024, 1024, 1024, 1024, 1024, 1024, 897],   # a tail of 127 rows (four passes)
])
def test_low_tiles_left_to_the_small_m_kernel(m_sizes, K, dtype):
    """One full round of 256 x 256 tiles on 256 workgroups plus a few low tiles: the automatic choice computes the
    low tiles with the small-M kernel behind the ping-pong kernel (moe_gg_host_tails_apart mirrors the decision)."""
    import ctypes

    import applied_ai_amd as A

    G, N = len(m_sizes), 2048
    M = sum(m_sizes)
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    arr = (ctypes.c_int32 * G)(*m_sizes)
    assert A._lib.lib().moe_gg_host_tails_apart(arr, G, M, N, K, cus - cus % 8) == (1 if cus == 256 else 0)
    x, w, _ = bf16_inputs(G, M, N, K, seed=21, w_std=0.05)
    check(x.to(dtype), w.to(dtype), m_sizes)


def test_large_two_groups():
    # unit_tests.py:235-256: (G, M, N, K) = (2, 2048, 512, 1024), m_sizes [1024, 1024]
    x, w, _ = bf16_inputs(2, 2048, 512, 1024, seed=12)
    check(x, w, [1024, 1024])


def test_fast_verification_shape_and_block_layout():
    # kernels/MoE/group_GEMM/triton/testing/fast_verification.py:31-48,83-96: G=20, M=1024, N=512, K=256
    import applied_ai_amd as A

    G, M, N, K = 20, 1024, 512, 256
    m_sizes = [52] * 4 + [51] * 16
    x, w, _ = bf16_inputs(G, M, N, K, seed=13)
    check(x, w, m_sizes)
    ms = torch.tensor(m_sizes, dtype=torch.int32, device="cuda")
    yb = torch.full((M, N * G), float("nan"), dtype=torch.bfloat16, device="cuda")
    xd, wd = x.cuda(), w.cuda()     # bound to names: the device copies must outlive the launch
    rc = A._lib.lib().moe_gg_grouped_gemm_bf16(xd.data_ptr(), wd.data_ptr(), yb.data_ptr(), ms.data_ptr(),
                                               G, M, N, K, N * G, 1, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    ref = O.grouped_gemm(to_np(x), to_np(w), m_sizes, block_layout=True)
    got = to_np(yb)
    written = ~np.isnan(ref)
    np.testing.assert_allclose(got[written], ref[written], rtol=RTOL, atol=ATOL)
    assert np.isnan(got[~written]).all()  # other experts' column blocks are not touched
    yf = A.grouped_gemm_forward(x.cuda(), w.cuda(), ms)
    assert yf.shape == (M, N * G)
    np.testing.assert_allclose(to_np(yf)[written], ref[written], rtol=RTOL, atol=ATOL)


def test_rows_beyond_sum_are_untouched():
    import applied_ai_amd as A

    G, M, N, K = 3, 96, 64, 64
    x, w, _ = bf16_inputs(G, M, N, K, seed=14)
    ms = torch.tensor([10, 0, 30], dtype=torch.int32, device="cuda")
    y = torch.full((M, N), 7.0, dtype=torch.bfloat16, device="cuda")
    xd, wd = x.cuda(), w.cuda()     # bound to names: the device copies must outlive the launch
    rc = A._lib.lib().moe_gg_grouped_gemm_bf16(xd.data_ptr(), wd.data_ptr(), y.data_ptr(), ms.data_ptr(),
                                               G, M, N, K, N, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert (to_np(y)[40:] == 7.0).all()


def test_bitwise_deterministic():
    # unit_tests.py:214-233
    x, w, _ = bf16_inputs(4, 128, 64, 128, seed=15)
    a = run(x, w, [32] * 4)
    b = run(x, w, [32] * 4)
    assert torch.equal(a, b)


def test_config1_plumbing_from_golden_fixture():
    # benchmark config 1 (8 experts, K=256, N=512, 256 tokens top-2) run in bf16 against the committed vectors
    import os

    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "cfg1.npz"))
    x = torch.from_numpy(z["x_sorted_bf16_bits"].astype(np.int16)).view(torch.bfloat16)
    w = torch.from_numpy(z["w_bf16_bits"].astype(np.int16)).view(torch.bfloat16)
    y = to_np(run(x, w, z["m_sizes"].tolist()))
    np.testing.assert_allclose(y, z["y_bf16_inputs"], rtol=RTOL, atol=ATOL)


def test_invalid_inputs_raise():
    import applied_ai_amd as A

    x = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(16, 32, dtype=torch.bfloat16, device="cuda")
    ms = torch.tensor([4, 4], dtype=torch.int32, device="cuda")
    with pytest.raises(AssertionError):       # K mismatch: dev/triton_groupGEMM/groupgemm.py:425
        A.grouped_gemm(x, w, ms)
    with pytest.raises(ValueError):
        A.grouped_gemm(x, torch.zeros(15, 64, dtype=torch.bfloat16, device="cuda"), ms)
    with pytest.raises(RuntimeError):         # host tensors: no CPU path
        A.grouped_gemm(x.cpu(), torch.zeros(16, 64, dtype=torch.bfloat16), ms.cpu())


def test_mixtral_prefill_shape_sampled_rows():
    """benchmark config 2 at full size (T=4096 top-2, K=4096, N=14336, 8 experts); the oracle checks 8 sampled rows
    per expert over all columns, and linearity checks the rest: y(2x) == 2 y(x) exactly in bf16."""
    from applied_ai_amd import configs

    c = configs.cfg2()
    m_sizes = c["m_sizes"].tolist()
    xs = c["x_sorted"].cuda(); wd = c["w"].cuda()
    ms = c["m_sizes"].cuda()
    import applied_ai_amd as A
    y = A.grouped_gemm(xs, wd, ms)
    y2 = A.grouped_gemm(xs * 2, wd, ms)
    torch.cuda.synchronize()
    assert torch.equal(y2, y * 2)
    off = O.offsets(m_sizes)
    rng = np.random.default_rng(0)
    N = 14336
    for g in range(8):
        rows = np.unique(np.concatenate([[off[g], off[g + 1] - 1], rng.integers(off[g], off[g + 1], 6)]))
        xr = c["x_sorted"][rows].float().numpy()
        ref = O.grouped_gemm(xr, c["w"][g * N:(g + 1) * N].float().numpy(), [len(rows)])
        np.testing.assert_allclose(to_np(y[rows]), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 3, 4, 5])
def test_fp16_every_kernel_family(variant):
    """IEEE half data through every kernel family (ping-pong, tiled 256 / 128 / 64, generic, small-M) and through the
    automatic choice, against the oracle on the same half-rounded inputs."""
    import applied_ai_amd as A

    L = A._lib.lib()
    cases = [(8, [300, 0, 517, 64, 1, 255, 256, 700], 512, 256), (4, [5, 0, 17, 9], 256, 512), (3, [20, 10, 20], 40, 72)]
    try:
        for G, ms, N, K in cases:
            if variant == 5 and (K % 128 or sum(ms) > 24 * G):
                continue
            if variant in (0, 1, 2, 3) and K % 64:
                continue
            x, w, _ = bf16_inputs(G, sum(ms), N, K, seed=41, w_std=0.25)
            x, w = x.half(), w.half()
            L.moe_gg_set_variant(0, variant)
            y = A.grouped_gemm(x.cuda(), w.cuda(), torch.tensor(ms, dtype=torch.int32, device="cuda"))
            assert y.dtype == torch.float16
            ref = O.grouped_gemm(to_np(x), to_np(w), ms)
            np.testing.assert_allclose(to_np(y), ref, rtol=RTOL, atol=ATOL)
            yb = A.grouped_gemm_forward(x.cuda(), w.cuda(), torch.tensor(ms, dtype=torch.int32, device="cuda"))
            row = 0
            for g, m in enumerate(ms):
                assert torch.equal(yb[row:row + m, g * N:(g + 1) * N], y[row:row + m])
                row += m
    finally:
        L.moe_gg_set_variant(0, -1)


@pytest.mark.parametrize("variant", [-1, 0, 2, 4, 5])
def test_largest_expert_count(variant):
    """G = 1024, the largest expert count the grouped kernels take (their in-LDS offset tables): many empty experts,
    a few rows each otherwise; every kernel family against the oracle."""
    import applied_ai_amd as A

    L = A._lib.lib()
    G, N, K = 1024, 128, 128
    rng = np.random.default_rng(5)
    ms = rng.integers(0, 9, size=G)
    ms[rng.integers(0, G, size=300)] = 0
    ms[[0, 511, 1023]] = [300, 260, 17]   # some row tiles at the first, a middle and the last expert
    ms = [int(v) for v in ms]
    x, w, _ = bf16_inputs(G, sum(ms), N, K, seed=6, w_std=0.25)
    try:
        L.moe_gg_set_variant(0, variant)
        y = A.grouped_gemm(x.cuda(), w.cuda(), torch.tensor(ms, dtype=torch.int32, device="cuda"))
    finally:
        L.moe_gg_set_variant(0, -1)
    ref = O.grouped_gemm(to_np(x), to_np(w), ms)
    np.testing.assert_allclose(to_np(y), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("which", ["y", "x", "w"])
def test_tensors_beyond_two_to_the_31_elements(which):
    """Each operand in turn is larger than 2^31 elements (4 GB of bf16), so every row, column and expert offset of
    that operand is exercised beyond 32 bits; sampled rows (the last ones among them) against an fp32 product."""
    import applied_ai_amd as A

    L = A._lib.lib()
    if which == "y":      # output [70000, 32768]
        G, ms, N, K, variants = 2, [35000, 35000], 32768, 64, (-1, 2)
    elif which == "x":    # activations [40000, 65536]
        G, ms, N, K, variants = 1, [40000], 64, 65536, (-1, 0)
    else:                 # weights [64 * 1024, 32768 + 128]
        G, ms, N, K, variants = 64, [4] * 64, 1024, 32768 + 128, (-1, 0)
    M = sum(ms)
    assert max(M * N, M * K, G * N * K) > 2 ** 31
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.empty((M, K), dtype=torch.bfloat16, device="cuda").normal_(generator=gen)
    w = torch.empty((G * N, K), dtype=torch.bfloat16, device="cuda").normal_(std=0.05, generator=gen)
    m = torch.tensor(ms, dtype=torch.int32, device="cuda")
    rows = sorted(set([0, 1, M // 2, M - 2, M - 1] + torch.randint(0, M, (40,), generator=torch.Generator().manual_seed(4)).tolist()))
    bounds = np.cumsum([0] + ms)
    try:
        for variant in variants:
            L.moe_gg_set_variant(0, variant)
            y = A.grouped_gemm(x, w, m)
            torch.cuda.synchronize()
            for r in rows:
                g = int(np.searchsorted(bounds, r, side="right") - 1)
                ref = x[r].float() @ w[g * N:(g + 1) * N].float().t()
                assert torch.allclose(y[r].float(), ref, rtol=RTOL, atol=ATOL * 4), (which, variant, r)
            del y
    finally:
        L.moe_gg_set_variant(0, -1)
