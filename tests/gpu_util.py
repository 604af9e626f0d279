"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def random_m_sizes(G, M, gen):
    """Sorted random cut points, as the reference tests draw them (empty groups occur):
    dev/triton_groupGEMM/testing/base_testing.py:106-116."""
    cuts = torch.sort(torch.randint(0, M, (G - 1,), generator=gen)).values.tolist() if G > 1 else []
    starts = [0] + cuts
    ends = cuts + [M]
    return [ends[i] - starts[i] for i in range(G)]


def bf16_inputs(G, M, N, K, seed, w_std=1.0):
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    w = (torch.randn(G * N, K, generator=gen) * w_std).to(torch.bfloat16)
    return x, w, gen


def to_np(t):
    return t.detach().float().cpu().numpy()


def rel_fro(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
