"""GPU parity of the W4A16 split-K dequant GEMM against the CPU oracle (relative Frobenius error <= 2e-2)."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import rel_fro, to_np

pytestmark = pytest.mark.gpu
TOL = 2e-2
GOLD = os.path.join(os.path.dirname(__file__), "golden")


def run(a, qw, scales, qz, zo, gs=None):
    import applied_ai_amd as A

    c = A.matmul_split_k(a.cuda(), torch.from_numpy(qw).cuda(), scales.cuda(), torch.from_numpy(qz).cuda(), zero_offset=zo,
                         groupsize=gs)
    torch.cuda.synchronize()
    return c


@pytest.mark.parametrize("zo", [0, 1])
@pytest.mark.parametrize("M", [1, 16])
def test_golden_fixture(zo, M):
    z = np.load(os.path.join(GOLD, "w4a16_tiny.npz"))
    a = torch.from_numpy(z["a"][:M]).to(torch.bfloat16)
    c = run(a, z["qweight"], torch.from_numpy(z["scales"]).to(torch.bfloat16), z["qzeros"], zo)
    assert rel_fro(to_np(c), z[f"c_zo{zo}_m{M}"]) <= TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N,gs,zo", [
    (1, 256, 128, 128, 1), (16, 256, 128, 128, 0), (64, 256, 128, 128, 1), (5, 1152, 256, 128, 1),
    (33, 512, 64, 128, 0), (16, 512, 64, 64, 0), (8, 256, 64, 32, 1), (17, 4096, 192, 128, 1), (100, 512, 128, 128, 1),
])
def test_against_oracle(dtype, M, K, N, gs, zo):
    print(f"case {dtype} M={M} K={K} N={N} group={gs} zero_offset={zo}", flush=True)
    rng = np.random.default_rng(M * 7 + K + N)
    q = rng.integers(0, 16, size=(K, N)); zz = rng.integers(0, 16, size=(K // gs, N))
    scales = torch.from_numpy(rng.uniform(0.005, 0.02, size=(K // gs, N)).astype(np.float32)).to(dtype)
    a = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dtype)
    qw, qz = O.pack_int4_along_k(q), O.pack_int4_along_n(zz)
    c = run(a, qw, scales, qz, zo, gs)
    assert c.dtype == dtype and c.shape == (M, N)
    ref = O.w4a16_gemm(to_np(a), qw, to_np(scales), qz, gs, zo)
    assert rel_fro(to_np(c), ref) <= TOL


def test_full_int32_range_words_and_determinism():
    # the reference's own driver draws qweight / zeros over the full int32 range (splitk_dequant_gemm.py:143-151)
    rng = np.random.default_rng(3)
    M, K, N = 16, 1024, 256
    qw = rng.integers(-2**31, 2**31, size=(K // 8, N), dtype=np.int64).astype(np.int32)
    qz = rng.integers(-2**31, 2**31, size=(K // 128, N // 8), dtype=np.int64).astype(np.int32)
    scales = torch.from_numpy(rng.uniform(0.005, 0.02, size=(K // 128, N)).astype(np.float32)).to(torch.float16)
    a = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.float16)
    c1 = run(a, qw, scales, qz, 1)
    c2 = run(a, qw, scales, qz, 1)
    assert torch.equal(c1, c2)  # no atomics: bit-identical run to run
    assert rel_fro(to_np(c1), O.w4a16_gemm(to_np(a), qw, to_np(scales), qz, 128, 1)) <= TOL


@pytest.mark.parametrize("M", [1, 16, 64])
def test_config4_full_size(M):
    """benchmark config 4: K=4096, N=14336, group 128, (q - z) * s. Oracle on all rows for a 256-column slice, plus
    linearity in the activations over the whole output: c(a1 + a2) ~= c(a1) + c(a2)."""
    from applied_ai_amd import configs

    c4 = configs.cfg4(M)
    qw = configs.pack_int4_along_k(c4["q"]).numpy(); qz = configs.pack_int4_along_n(c4["z"]).numpy()
    c = run(c4["a"], qw, c4["scales"], qz, 0)
    cols = slice(4096, 4352)
    ref = O.w4a16_gemm(to_np(c4["a"]), np.ascontiguousarray(qw[:, cols]), to_np(c4["scales"][:, cols]),
                       np.ascontiguousarray(qz[:, 512:544]), 128, 0)
    assert rel_fro(to_np(c[:, cols]), ref) <= TOL
    a2 = torch.randn(M, 4096, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    s = run((c4["a"].float() + a2.float()).to(torch.bfloat16), qw, c4["scales"], qz, 0)
    t = run(a2, qw, c4["scales"], qz, 0)
    assert rel_fro(to_np(s), to_np(c) + to_np(t)) <= 3e-2


def test_invalid_arguments():
    import applied_ai_amd as A

    a = torch.zeros(4, 256, dtype=torch.bfloat16, device="cuda")
    b = torch.zeros(32, 64, dtype=torch.int32, device="cuda")
    s = torch.zeros(2, 64, dtype=torch.bfloat16, device="cuda")
    z = torch.zeros(2, 8, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        A.matmul_split_k(a, b[:31], s, z)
    with pytest.raises(ValueError):
        A.matmul_split_k(a, b, s.to(torch.float16), z)
    with pytest.raises(ValueError):
        A.matmul_split_k(a, b, s, z, zero_offset=2)
    with pytest.raises(RuntimeError):
        A.matmul_split_k(a.cpu(), b.cpu(), s.cpu(), z.cpu())


def test_qlinear_entry_points_of_the_reference():
    """a100_qlinear / h100_qlinear / small_qlinear (the reference's data-parallel W4A16 layers) share packing,
    group size 128 and the (q - (z + 1)) * s formula with matmul_split_k: same result, in a's dtype."""
    import applied_ai_amd as A

    M, K, N = 16, 512, 128
    rng = np.random.default_rng(3)
    q = rng.integers(0, 16, size=(K, N)); zz = rng.integers(0, 16, size=(K // 128, N))
    scales = torch.from_numpy(rng.uniform(0.005, 0.02, size=(K // 128, N)).astype(np.float32)).to(torch.float16)
    a = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(torch.float16)
    qw, qz = O.pack_int4_along_k(q), O.pack_int4_along_n(zz)
    args = (a.cuda(), torch.from_numpy(qw).cuda(), scales.cuda(), torch.from_numpy(qz).cuda())
    want = A.matmul_split_k(*args)
    for fn in (A.a100_qlinear, A.h100_qlinear, A.small_qlinear):
        got = fn(*args)
        assert got.dtype == torch.float16 and torch.equal(got, want)
    ref = O.w4a16_gemm(to_np(a), qw, to_np(scales), qz, 128, 1)
    assert rel_fro(to_np(want), ref) <= TOL
