"""GPU parity of the MoE layer (fused_moe and its glue kernels) against the oracle.
Layer: |y - ref| <= 1e-2 + 1e-2 |ref| against the double-precision oracle that rounds the stored intermediates
to bf16 (the reference's bar is atol 1e-2 on fp16 data, test_moe_gemm.py:78-79; bf16 has three mantissa bits
fewer, hence the relative term). silu_and_mul / combine: one bf16 rounding of the exact value."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import to_np

pytestmark = pytest.mark.gpu


def bf(t):
    return t.to(torch.bfloat16)


def make(m, n, k, e, topk, seed=3227):
    gen = torch.Generator().manual_seed(seed)
    a = bf(torch.randn(m, k, generator=gen) / 10)
    w1 = bf(torch.randn(e, 2 * n, k, generator=gen) / 10)
    w2 = bf(torch.randn(e, k, n, generator=gen) / 10)
    score = torch.softmax(torch.randn(m, e, generator=gen), dim=-1)
    tw, ids = torch.topk(score, topk)
    return a, w1, w2, tw, ids


def close(y, ref):
    d = np.abs(y - ref)
    return bool(np.all(d <= 1e-2 + 1e-2 * np.abs(ref))), float(d.max())


def test_silu_and_mul_is_correctly_rounded():
    import applied_ai_amd as A

    gen = torch.Generator().manual_seed(5)
    x = bf(torch.randn(37, 2 * 264, generator=gen) * 4)
    x[0, :8] = torch.tensor([0.0, -0.0, 30.0, -30.0, 88.0, -88.0, 1e-3, -1e-3]).to(torch.bfloat16)
    y = to_np(A.silu_and_mul(x.cuda()))
    exact = O.silu_and_mul(x.float().numpy()).astype(np.float64)
    ref = O.round_bf16(exact.astype(np.float32))
    # the kernel evaluates in fp32 with the hardware exponential: allow one bf16 ulp around the exact value
    ulp = np.maximum(np.abs(ref) * 2.0 ** -7, 1e-30)
    assert np.all(np.abs(y - exact) <= ulp)
    assert np.mean(y == ref) > 0.99


def test_combine_topk_matches_weighted_sum():
    import applied_ai_amd as A

    gen = torch.Generator().manual_seed(6)
    T, k, E, d = 50, 3, 6, 136
    ids = torch.stack([torch.randperm(E, generator=gen)[:k] for _ in range(T)]).to(torch.int32)
    w = torch.rand(T, k, generator=gen)
    perm, m_sizes, offsets = A.route_group(ids.cuda(), E)
    y = bf(torch.randn(T * k, d, generator=gen))
    for wt in (w, bf(w)):
        out = to_np(A.combine_topk(y.cuda(), perm, offsets, wt.cuda()))
        p = perm.cpu().numpy()
        inv = np.empty(T * k, dtype=np.int64); inv[p] = np.arange(T * k)
        exp = (y.float().numpy()[inv].reshape(T, k, d).astype(np.float64) * wt.float().numpy().astype(np.float64)[:, :, None]).sum(1)
        assert np.all(np.abs(out - exp) <= np.abs(exp) * 2.0 ** -7 + 1e-6)


@pytest.mark.parametrize("m", [1, 2, 16, 33, 200])
def test_fused_moe_small_against_c_oracle(m):
    import applied_ai_amd as A

    n, k, e, topk = 128, 256, 8, 2
    a, w1, w2, tw, ids = make(m, n, k, e, topk, seed=100 + m)
    print(f"fused_moe m={m} n={n} k={k} e={e}", flush=True)
    y = to_np(A.fused_moe(a.cuda(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda()))
    ref = O.fused_moe(a.float().numpy(), w1.float().numpy(), w2.float().numpy(), tw.numpy(), ids.numpy())
    ok, worst = close(y, ref)
    assert ok, worst
    assert y.shape == (m, k)


def test_fused_moe_top1_and_many_experts_with_empty_ones():
    import applied_ai_amd as A

    a, w1, w2, tw, ids = make(40, 64, 128, 32, 1, seed=7)   # most of the 32 experts get one row or none
    y = to_np(A.fused_moe(a.cuda(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda()))
    ref = O.fused_moe(a.float().numpy(), w1.float().numpy(), w2.float().numpy(), tw.numpy(), ids.numpy())
    ok, worst = close(y, ref)
    assert ok, worst


@pytest.mark.parametrize("m,frac", [(40, 0.3), (700, 0.1), (8, 1.0)])
def test_fused_moe_with_masked_slots(m, frac):
    """Slots whose expert id is -1 (or beyond the last expert) contribute nothing, as in the reference's torch_moe
    (test_moe_gemm.py:24-29: no mask matches them, their rows stay zero); frac = 1: every slot masked, result zero."""
    import applied_ai_amd as A

    n, k, e, topk = 128, 256, 8, 2
    a, w1, w2, tw, ids = make(m, n, k, e, topk, seed=500 + m)
    gen = torch.Generator().manual_seed(m)
    drop = torch.rand(ids.shape, generator=gen) < frac
    ids = torch.where(drop, torch.full_like(ids, -1), ids)
    if m > 8:
        ids[0, 0] = e + 3
    print(f"fused_moe masked m={m} dropped={int(drop.sum())}", flush=True)
    y = to_np(A.fused_moe(a.cuda(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda()))
    ref = O.fused_moe(a.float().numpy(), w1.float().numpy(), w2.float().numpy(), tw.numpy(), ids.numpy())
    ok, worst = close(y, ref)
    assert ok, worst
    if frac == 1.0:
        assert not y.any()
    out = torch.full((m, topk, 2 * n), 7.0, dtype=torch.bfloat16, device="cuda")
    A.invoke_fused_moe_kernel(a.cuda(), w1.cuda(), out, tw.cuda(), ids.cuda(), top_k=topk)
    flat = ids.reshape(-1)
    ref1 = np.zeros((m * topk, 2 * n), dtype=np.float32)
    for p in range(m * topk):
        ex = int(flat[p])
        if 0 <= ex < e:
            ref1[p] = a[p // topk].float().numpy() @ w1[ex].float().numpy().T
    ok, worst = close(to_np(out).reshape(m * topk, 2 * n), ref1)
    assert ok, worst


def test_fused_moe_inplace_and_int32_ids_and_bf16_weights():
    import applied_ai_amd as A

    a, w1, w2, tw, ids = make(24, 64, 128, 4, 2, seed=8)
    ref = O.fused_moe(a.float().numpy(), w1.float().numpy(), w2.float().numpy(), bf(tw).float().numpy(), ids.numpy())
    h = a.cuda().clone()
    out = A.fused_moe(h, w1.cuda(), w2.cuda(), bf(tw).cuda(), ids.to(torch.int32).cuda(), inplace=True)
    assert out.data_ptr() == h.data_ptr()
    ok, worst = close(to_np(h), ref)
    assert ok, worst


def test_fused_moe_reference_test_shape():
    """The reference's own case (test_moe_gemm.py:33-57): n = 14336 // 2, k = 4096, e = 8, top-2, here with
    m = 64 and bf16; checked against the per-expert fp32 torch.matmul form of the oracle."""
    import applied_ai_amd as A

    a, w1, w2, tw, ids = make(64, 14336 // 2, 4096, 8, 2)
    y = to_np(A.fused_moe(a.cuda(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda()))
    ref = O.fused_moe_torch(a, w1, w2, tw, ids).numpy()
    d = np.abs(y - ref)
    # no intermediate rounding in this form of the oracle: add the bf16 storage error of three roundings
    assert np.all(d <= 2e-2 + 2e-2 * np.abs(ref)), float(d.max())
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) < 1e-2


def test_fused_moe_prefill_rows_take_the_fused_activation_path():
    """768 tokens, top-2 -> 1536 expert-sorted rows: the first GEMM runs with SiLU-and-mul in its epilogue.
    Same oracle, same bar; and the result equals the layer built from the separate kernels bit for bit."""
    import applied_ai_amd as A
    from applied_ai_amd import moe

    assert 768 * 2 >= moe.FUSED_SWIGLU_MIN_ROWS
    a, w1, w2, tw, ids = make(768, 192, 256, 8, 2, seed=21)
    args = (a.cuda(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda())
    y = A.fused_moe(*args)
    ref = O.fused_moe(a.float().numpy(), w1.float().numpy(), w2.float().numpy(), tw.numpy(), ids.numpy())
    ok, worst = close(to_np(y), ref)
    assert ok, worst
    saved = moe.FUSED_SWIGLU_MIN_ROWS
    try:
        moe.FUSED_SWIGLU_MIN_ROWS = 1 << 40
        y2 = A.fused_moe(*args)
    finally:
        moe.FUSED_SWIGLU_MIN_ROWS = saved
    assert torch.equal(y.view(torch.int16), y2.view(torch.int16))


def test_fused_moe_rejects_bad_arguments():
    import applied_ai_amd as A

    a, w1, w2, tw, ids = make(4, 64, 128, 4, 2)
    with pytest.raises(AssertionError):
        A.fused_moe(a.cuda()[:, :64].contiguous(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda())
    with pytest.raises(AssertionError):
        A.fused_moe(a.cuda().half(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda())
    with pytest.raises(RuntimeError):
        A.fused_moe(a, w1, w2, tw, ids)


@pytest.mark.parametrize("sizes,n,K", [
    ([300, 0, 41, 700], 256, 128),        # ragged, an empty expert
    ([256, 256], 128, 64),                # one K step
    ([100, 37], 200, 192),                # n not a multiple of the 128-column tile
    ([513, 64, 1], 1032, 256),            # several column tiles and a partial one
])
def test_swiglu_gemm_equals_gemm_then_silu_and_mul(sizes, n, K):
    """The fused kernel rounds both products to bf16 before the activation: bit-identical to the two-kernel path,
    and within the GEMM bar of the double-precision oracle."""
    import applied_ai_amd as A

    G, M = len(sizes), sum(sizes) + 5
    gen = torch.Generator().manual_seed(77)
    x = bf(torch.randn(M, K, generator=gen))
    w = bf(torch.randn(G * 2 * n, K, generator=gen) / 8)
    m = torch.tensor(sizes, dtype=torch.int32)
    fused = A.grouped_gemm_swiglu(x.cuda(), w.cuda(), m.cuda())
    two = A.silu_and_mul(A.grouped_gemm(x.cuda(), w.cuda(), m.cuda()))
    R = sum(sizes)
    assert fused.shape == (M, n)
    assert torch.equal(fused[:R].view(torch.int16), two[:R].view(torch.int16))
    h1 = O.round_bf16(O.grouped_gemm(x.float().numpy(), w.float().numpy(), sizes, fill=0.0))
    ref = O.silu_and_mul(h1)[:R]
    ok, worst = close(to_np(fused)[:R], ref)
    assert ok, worst


def test_swiglu_errors(lib=None):
    import applied_ai_amd as A

    x = torch.zeros(8, 96, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(2 * 2 * 64, 96, dtype=torch.bfloat16, device="cuda")
    m = torch.tensor([4, 4], dtype=torch.int32, device="cuda")
    with pytest.raises(RuntimeError):      # K % 64 != 0: unsupported
        A.grouped_gemm_swiglu(x, w, m)
    with pytest.raises(AssertionError):    # K mismatch
        A.grouped_gemm_swiglu(x[:, :64].contiguous(), w, m)


@pytest.mark.parametrize("M,k,E,N,K", [(33, 2, 8, 256, 128), (700, 2, 8, 512, 256), (5, 4, 16, 64, 64)])
def test_invoke_fused_moe_kernel_both_gemms_of_the_layer(M, k, E, N, K):
    """The reference's GEMM-level entry (v0_moe_fused.py:183-220) as fused_moe uses it (:271-289): first GEMM with
    top_k = k on [M, K] rows, second with top_k = 1 on [M * k, N] rows and the routed weights; against a per-row
    fp32 product, atol = rtol = 1e-2 (test_moe_gemm.py:78-79 uses atol 1e-2)."""
    import applied_ai_amd as A

    gen = torch.Generator().manual_seed(M + E)
    x = (torch.randn(M, K, generator=gen) / 4).bfloat16()
    w1 = (torch.randn(E, N, K, generator=gen) / 4).bfloat16()
    w2 = (torch.randn(E, K, N, generator=gen) / 4).bfloat16()
    score = torch.softmax(torch.randn(M, E, generator=gen), dim=-1)
    tw, ids = torch.topk(score, k)
    sorted_ids, expert_ids, post = A.moe_align_block_size(ids.cuda(), 16, E)
    c1 = torch.empty((M, k, N), dtype=torch.bfloat16, device="cuda")
    A.invoke_fused_moe_kernel(x.cuda(), w1.cuda(), c1, tw.cuda(), ids.cuda(), sorted_ids, expert_ids, post, False, k, {})
    ref1 = torch.einsum("mk,mjnk->mjn", x.float(), w1.float()[ids])
    assert torch.allclose(c1.float().cpu(), ref1, rtol=1e-2, atol=1e-2)
    h = c1.view(M * k, N)
    c2 = torch.empty((M, k, K), dtype=torch.bfloat16, device="cuda")
    A.invoke_fused_moe_kernel(h, w2.cuda(), c2, tw.cuda(), ids.cuda(), sorted_ids, expert_ids, post, True, 1, {})
    ref2 = torch.einsum("mjn,mjkn->mjk", c1.float().cpu(), w2.float()[ids]) * tw[:, :, None]
    assert torch.allclose(c2.float().cpu(), ref2, rtol=1e-2, atol=1e-2)


def test_fp16_forms_of_silu_and_mul_and_combine():
    """The glue kernels on IEEE half data (the int4 layer runs in it): SiLU-and-mul within one fp16 ulp of the fp32
    formula (the exponential is the fast one), the combine within the bar of the layer."""
    import applied_ai_amd as A

    gen = torch.Generator().manual_seed(5)
    x = (torch.randn(37, 2 * 64, generator=gen) * 3).half()
    got = A.silu_and_mul(x.cuda()).cpu()
    want = (torch.nn.functional.silu(x[:, :64].float()) * x[:, 64:].float())
    assert got.dtype == torch.float16
    ulp = torch.maximum(want.abs(), torch.tensor(2.0 ** -14)) * 2.0 ** -10
    assert bool(((got.float() - want).abs() <= ulp).all())

    T, k, E, d = 50, 3, 8, 64
    ids = torch.stack([torch.randperm(E, generator=gen)[:k] for _ in range(T)]).to(torch.int32)
    perm, m_sizes, offsets = A.route_group(ids.cuda(), E)
    y = torch.randn(T * k, d, generator=gen).half()
    for w in (torch.rand(T, k, generator=gen), torch.rand(T, k, generator=gen).half()):
        out = A.combine_topk(y.cuda(), perm, offsets, w.cuda()).cpu()
        inv = torch.empty(T * k, dtype=torch.long)
        inv[perm.cpu().long()] = torch.arange(T * k)
        want = (w.float()[:, :, None] * y.float()[inv].view(T, k, d)).sum(1)
        assert out.dtype == torch.float16 and torch.allclose(out.float(), want, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("m", [2, 33, 200, 1500])
def test_fused_moe_fp16_as_the_reference_test_runs_it(m):
    """fp16 data (kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:33-60) against torch_moe restated in
    fp32 (:16-30); the reference's bar: atol 1e-2, rtol 0 (:78-79)."""
    import applied_ai_amd as A

    n, k, e, topk = 128, 256, 8, 2
    a, w1, w2, tw, ids = make(m, n, k, e, topk, seed=300 + m)
    a, w1, w2 = a.half(), w1.half(), w2.half()
    y = A.fused_moe(a.cuda(), w1.cuda(), w2.cuda(), tw.cuda(), ids.cuda())
    assert y.dtype == torch.float16 and y.shape == (m, k)
    ref = torch.zeros(m, k)
    for t in range(m):
        for j in range(topk):
            ex = int(ids[t, j])
            h = a[t].float() @ w1[ex].float().t()
            h = torch.nn.functional.silu(h[:n]) * h[n:]
            ref[t] += tw[t, j] * (h @ w2[ex].float().t())
    assert torch.allclose(y.float().cpu(), ref, atol=1e-2, rtol=0), float((y.float().cpu() - ref).abs().max())


@pytest.mark.parametrize("sizes,n,K", [([300, 0, 41, 700], 256, 128), ([513, 64, 1], 1032, 256)])
def test_swiglu_gemm_fp16_equals_gemm_then_silu_and_mul(sizes, n, K):
    """The fp16 form of the fused kernel: bit-identical to the fp16 GEMM followed by the fp16 activation kernel."""
    import applied_ai_amd as A

    G, M = len(sizes), sum(sizes) + 5
    gen = torch.Generator().manual_seed(78)
    x = torch.randn(M, K, generator=gen).half()
    w = (torch.randn(G * 2 * n, K, generator=gen) / 8).half()
    m = torch.tensor(sizes, dtype=torch.int32)
    fused = A.grouped_gemm_swiglu(x.cuda(), w.cuda(), m.cuda())
    two = A.silu_and_mul(A.grouped_gemm(x.cuda(), w.cuda(), m.cuda()))
    R = sum(sizes)
    assert fused.dtype == torch.float16 and fused.shape == (M, n)
    assert torch.equal(fused[:R].view(torch.int16), two[:R].view(torch.int16))
