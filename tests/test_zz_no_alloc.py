"""The backward entry point that allocates nothing (moe_gg_grouped_gemm_backward_bf16_static): its transposed copies
live in an array inside the library's device image instead of a caller workspace. Checked through the C ABI against
moe_gg_grouped_gemm_backward_bf16 bit for bit, on two calls in a row, the second with a smaller input (the array
keeps the first call's contents), and against the double-precision oracle to the bar of the backward tests
(rtol = atol = 1e-2, kernels/MoE/group_GEMM/triton/testing/fast_verification.py:110-122). Collected last on purpose."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import to_np

pytestmark = pytest.mark.gpu

STATIC_BYTES = 32 << 20


def _inputs(sizes, M, N, K, block_layout, seed):
    G = len(sizes)
    gen = torch.Generator().manual_seed(seed)
    x = (torch.randn(M, K, generator=gen) * 0.5).to(torch.bfloat16)
    w = (torch.randn(G * N, K, generator=gen) * 0.5).to(torch.bfloat16)
    go = (torch.randn(M, N * G if block_layout else N, generator=gen) * 0.5).to(torch.bfloat16)
    return x, w, go, torch.tensor(sizes, dtype=torch.int32)


def _both(lib, sizes, M, N, K, block_layout, seed, beyond_static=False):
    """(grad_x, grad_w) of the workspace entry point and of the static one; untouched memory is NaN in both.
    beyond_static: the call's workspace size exceeds the library's array (it must then be a call that needs no
    copies); the reference is the oracle's per-expert torch loop instead of its scalar C loop (size)."""
    G = len(sizes)
    x, w, go, m = _inputs(sizes, M, N, K, block_layout, seed)
    xd, wd, god, md = x.cuda(), w.cuda(), go.cuda(), m.cuda()
    layout = 1 if block_layout else 0
    stream = torch.cuda.current_stream().cuda_stream
    nbytes = lib.moe_gg_grouped_gemm_backward_workspace(G, max(M, 1), N, K, layout)
    assert nbytes > STATIC_BYTES if beyond_static else 0 < nbytes <= STATIC_BYTES
    ws = torch.full((nbytes // 2,), float("nan"), dtype=torch.bfloat16, device="cuda")
    out = []
    for static in (False, True):
        gx = torch.full((M, K), float("nan"), dtype=torch.bfloat16, device="cuda")
        gw = torch.full((G * N, K), float("nan"), dtype=torch.bfloat16, device="cuda")
        print(f"backward static={static} sizes={sizes} M={M} N={N} K={K} block_layout={block_layout}", flush=True)
        if static:
            args = (god.data_ptr(), go.shape[1], layout, xd.data_ptr(), wd.data_ptr(), md.data_ptr(), G, M, N, K, gx.data_ptr(),
                    gw.data_ptr(), stream)
            # once untimed (the first launch of a kernel loads its code object, which takes device memory), then
            # with the device's free memory and torch's own count read on both sides: the call allocates nothing
            assert lib.moe_gg_grouped_gemm_backward_bf16_static(*args) == 0
            torch.cuda.synchronize()
            free0, alloc0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
            rc = lib.moe_gg_grouped_gemm_backward_bf16_static(*args)
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() == alloc0
        else:
            rc = lib.moe_gg_grouped_gemm_backward_bf16(god.data_ptr(), go.shape[1], layout, xd.data_ptr(), wd.data_ptr(),
                                                       md.data_ptr(), G, M, N, K, gx.data_ptr(), gw.data_ptr(), ws.data_ptr(),
                                                       nbytes, stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        out.append((gx, gw))
    (gx0, gw0), (gx1, gw1) = out
    assert torch.equal(gx0.view(torch.int16), gx1.view(torch.int16))
    assert torch.equal(gw0.view(torch.int16), gw1.view(torch.int16))
    R = sum(sizes)
    if beyond_static:
        rx, rw = (t.numpy() for t in O.grouped_gemm_backward_torch_loop(go.float(), x.float(), w.float(), sizes))
    else:
        rx, rw = O.grouped_gemm_backward(go.float().numpy(), x.float().numpy(), w.float().numpy(), sizes)
    for got, ref in ((to_np(gx1)[:R], rx[:R]), (to_np(gw1), rw)):
        assert np.all(np.abs(got - ref) <= 1e-2 + 1e-2 * np.abs(ref))
    assert bool(gx1[R:].isnan().all())      # rows beyond sum(m_sizes) are not written by the C ABI


def test_static_scratch_backward_two_calls_in_a_row():
    import applied_ai_amd as A

    lib = A._lib.lib()
    _both(lib, [37, 90, 200, 3, 0, 70], 448, 256, 320, True, seed=31)   # 1.2 MB of transposed copies
    _both(lib, [17, 5], 24, 72, 40, True, seed=32)                      # smaller: the array still holds the first call's
    _both(lib, [100, 0, 27, 1], 128, 64, 192, False, seed=33)           # [M, N] gradient layout


def test_static_scratch_backward_limit_and_large_calls():
    import applied_ai_amd as A

    lib = A._lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    # Needs transposed copies (N % 64 != 0) of 16 * 1032 * 1024 * 2 bytes > 32 MiB: refused before any launch.
    G, M, N, K = 16, 64, 1032, 1024
    assert lib.moe_gg_grouped_gemm_backward_workspace(G, M, N, K, 0) > STATIC_BYTES
    x = torch.zeros(M, K, dtype=torch.bfloat16, device="cuda"); w = torch.zeros(G * N, K, dtype=torch.bfloat16, device="cuda")
    go = torch.zeros(M, N, dtype=torch.bfloat16, device="cuda"); m = torch.full((G,), 4, dtype=torch.int32, device="cuda")
    gx = torch.zeros_like(x); gw = torch.ones_like(w)
    rc = lib.moe_gg_grouped_gemm_backward_bf16_static(go.data_ptr(), N, 0, x.data_ptr(), w.data_ptr(), m.data_ptr(), G, M, N, K,
                                                      gx.data_ptr(), gw.data_ptr(), stream)
    assert rc == -4     # MOE_GG_EUNSUPPORTED
    torch.cuda.synchronize()
    assert bool((gw == 1).all())
    # A call large enough to read its operands as stored needs no copies and is not limited: 8 x 300 rows, 512 x 512.
    sizes = [300] * 8
    G, M, N, K = 8, 2400, 512, 512
    assert lib.moe_gg_grouped_gemm_backward_workspace(G, M, N, K, 1) <= STATIC_BYTES
    _both(lib, sizes, M, N, K, True, seed=34)
    # The same with 2048 x 2048 weights: the workspace form would want 64 MiB for w^T alone, twice the array, but both
    # gradients are computed from the operands as stored, so the static form runs (and touches no scratch).
    _both(lib, sizes, M, 2048, 2048, False, seed=35, beyond_static=True)
