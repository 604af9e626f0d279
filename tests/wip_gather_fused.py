"""GPU parity of the first MoE GEMM with the row gather folded into its loads (moe_gg_grouped_gemm_swiglu_gather,
fused_moe(..., fuse_gather=True)): bit-identical to the gathered copy followed by the plain fused kernel, and the
layer against the oracle. Not collected by pytest under this name (run it by naming the file): the kernel has run under the CPU emulation only
(tests/test_emu_kernels.py); it joins the collected GPU tests once it has passed on a GPU."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def make(T, E, k, n, K, dtype, seed, masked=0.0):
    gen = torch.Generator().manual_seed(seed)
    tok = (torch.randn(T, K, generator=gen) / 4).to(dtype)
    w1 = (torch.randn(E, 2 * n, K, generator=gen) / 8).to(dtype)
    ids = torch.randint(0, E, (T, k), generator=gen, dtype=torch.int32)
    if masked:
        drop = torch.rand(T, k, generator=gen) < masked
        ids[drop] = -1
    return tok, w1, ids


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("T,E,k,n,K,masked", [
    (700, 8, 2, 192, 128, 0.0), (1500, 4, 2, 256, 256, 0.1), (300, 3, 3, 64, 64, 0.0), (2100, 16, 4, 128, 512, 0.05)])
def test_same_bits_as_gather_then_gemm(dtype, T, E, k, n, K, masked):
    import applied_ai_amd as A

    print(f"case {dtype} T={T} E={E} k={k} n={n} K={K} masked={masked}", flush=True)
    tok, w1, ids = make(T, E, k, n, K, dtype, seed=T + n, masked=masked)
    tok, w1, ids = tok.cuda(), w1.cuda(), ids.cuda()
    perm, m_sizes, offsets = A.route_group(ids, E)
    nv = int(offsets[-1])
    two_step = A.grouped_gemm_swiglu(A.gather_sorted(tok, perm, k, offsets), w1.view(E * 2 * n, K), m_sizes)
    fused = A.grouped_gemm_swiglu_gathered(tok, perm, k, w1.view(E * 2 * n, K), m_sizes)
    torch.cuda.synchronize()
    assert fused.dtype == dtype and fused.shape == two_step.shape
    assert torch.equal(fused[:nv].view(torch.int16), two_step[:nv].view(torch.int16))


def test_mixtral_layer_shape_same_bits_and_layer_option():
    """The benchmark's layer (T = 4096, K = 4096, n = 14336, 8 experts, top-2): first GEMM bit-identical on all 8192 rows;
    fused_moe with fuse_gather=True equals the default path bit for bit."""
    import applied_ai_amd as A

    T, E, k, n, K = 4096, 8, 2, 14336, 4096
    gen = torch.Generator(device="cuda").manual_seed(77)
    tok = (torch.randn(T, K, device="cuda", generator=gen) / 10).to(torch.bfloat16)
    w1 = torch.empty(E, 2 * n, K, device="cuda", dtype=torch.bfloat16)
    w2 = torch.empty(E, K, n, device="cuda", dtype=torch.bfloat16)
    for e in range(E):
        w1[e] = (torch.randn(2 * n, K, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
        w2[e] = (torch.randn(K, n, device="cuda", generator=gen) * 0.02).to(torch.bfloat16)
    score = torch.softmax(torch.randn(T, E, device="cuda", generator=gen), dim=-1)
    tw, ids = torch.topk(score, k)
    ids = ids.to(torch.int32)
    perm, m_sizes, offsets = A.route_group(ids, E)
    two_step = A.grouped_gemm_swiglu(A.gather_sorted(tok, perm, k, offsets), w1.view(E * 2 * n, K), m_sizes)
    fused = A.grouped_gemm_swiglu_gathered(tok, perm, k, w1.view(E * 2 * n, K), m_sizes)
    torch.cuda.synchronize()
    assert torch.equal(fused.view(torch.int16), two_step.view(torch.int16))
    del two_step, fused
    a = A.fused_moe(tok, w1, w2, tw, ids)
    b = A.fused_moe(tok, w1, w2, tw, ids, fuse_gather=True)
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_argument_errors():
    import applied_ai_amd as A

    tok = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(2 * 2 * 8, 64, dtype=torch.bfloat16, device="cuda")
    ms = torch.tensor([8, 8], dtype=torch.int32, device="cuda")
    perm = torch.arange(16, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        A.grouped_gemm_swiglu_gathered(tok, perm.long(), 2, w, ms)
    with pytest.raises(ValueError):
        A.grouped_gemm_swiglu_gathered(tok, perm, 0, w, ms)
    with pytest.raises(AssertionError):
        A.grouped_gemm_swiglu_gathered(tok, perm, 2, torch.zeros(32, 32, dtype=torch.bfloat16, device="cuda"), ms)
    y = A.grouped_gemm_swiglu_gathered(tok, perm, 2, w, ms)
    torch.cuda.synchronize()
    assert y.shape == (16, 8) and float(y.float().abs().max()) == 0.0
