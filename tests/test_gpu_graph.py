"""HIP-graph capture of the library's launches: every entry point only enqueues kernels on the given stream, so a
captured sequence must replay with the same results as eager calls (checked on several replays with new inputs
and eager work in between)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_grouped_gemm_and_layer_replay_like_eager():
    import applied_ai_amd as A

    gen = torch.Generator().manual_seed(11)
    T, K, n, E, k = 64, 256, 128, 8, 2
    h = (torch.randn(T, K, generator=gen) / 4).to(torch.bfloat16).cuda()
    w1 = (torch.randn(E, 2 * n, K, generator=gen) / 8).to(torch.bfloat16).cuda()
    w2 = (torch.randn(E, K, n, generator=gen) / 8).to(torch.bfloat16).cuda()
    logits = torch.randn(T, E, generator=gen).cuda()

    def run():
        ids, perm, m_sizes, offsets = A.route_topk(logits, k)
        xs = A.gather_sorted(h, perm, k)
        y = A.grouped_gemm(xs, w1.view(E * 2 * n, K), m_sizes)
        tw = torch.full((T, k), 0.5, device="cuda")
        out = A.fused_moe(h, w1, w2, tw, ids)
        return y, out

    run()  # warm-up outside the capture (library and allocator initialisation)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            gy, gout = run()
    for rep in range(3):
        h.copy_((torch.randn(T, K, generator=gen) / 4).to(torch.bfloat16))
        logits.copy_(torch.randn(T, E, generator=gen))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        ey, eout = run()
        torch.cuda.synchronize()
        R = T * k
        assert torch.equal(gy[:R], ey[:R]), f"replay {rep}: grouped_gemm differs"
        assert torch.equal(gout, eout), f"replay {rep}: fused_moe differs"
