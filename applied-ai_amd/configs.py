"""Synthetic workloads of the five benchmark configurations (seeded, drawn on the CPU generator so the
CPU checker and the GPU path see identical bits). Draw order per config: x, router logits, weights,
then scales / zeros. Seeds are 1000 + config number."""
import math
from typing import Dict

import torch


def route_reference(logits: torch.Tensor, k: int):
    """Routing recipe of the reference's MoE tests on the host: top-k ids
    (kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:54-57), rows grouped by ascending
    expert with a stable sort (v0_moe_fused.py:141-166), per-expert counts.
    Returns (ids [T,k] int32, perm [T*k] int32, m_sizes [E] int32)."""
    E = logits.shape[1]
    ids = torch.topk(logits, k).indices
    flat = ids.reshape(-1)
    perm = torch.argsort(flat, stable=True)
    m_sizes = torch.bincount(flat, minlength=E).to(torch.int32)
    return ids.to(torch.int32), perm.to(torch.int32), m_sizes


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def cfg1() -> Dict[str, torch.Tensor]:
    """CPU plumbing: 8 experts, K=256, N=512, fp32, 256 tokens top-2 -> 512 sorted rows."""
    g = _gen(1001)
    x = torch.randn(256, 256, generator=g)
    logits = torch.randn(256, 8, generator=g)
    w = torch.randn(8, 512, 256, generator=g) * 0.02
    ids, perm, m_sizes = route_reference(logits, 2)
    return dict(x=x, logits=logits, w=w.reshape(8 * 512, 256), ids=ids, perm=perm, m_sizes=m_sizes,
                x_sorted=x[(perm // 2).long()], k=2)


def moe_bf16(T: int, E: int, k: int, K: int, N: int, seed: int, w_std: float = 0.02) -> Dict[str, torch.Tensor]:
    g = _gen(seed)
    x = torch.randn(T, K, generator=g).to(torch.bfloat16)
    logits = torch.randn(T, E, generator=g)
    w = torch.empty(E * N, K, dtype=torch.bfloat16)
    for e in range(E):  # per expert, to bound host memory
        w[e * N:(e + 1) * N] = (torch.randn(N, K, generator=g) * w_std).to(torch.bfloat16)
    ids, perm, m_sizes = route_reference(logits, k)
    return dict(x=x, logits=logits, w=w, ids=ids, perm=perm, m_sizes=m_sizes, x_sorted=x[(perm // k).long()], k=k)


def cfg2() -> Dict[str, torch.Tensor]:
    """Mixtral 8x7B w1, bf16: T=4096 top-2 -> 8192 rows, K=4096, N=14336."""
    return moe_bf16(4096, 8, 2, 4096, 14336, 1002)


def cfg3(down: bool = False) -> Dict[str, torch.Tensor]:
    """Mixtral decode: T=32 top-2 -> 64 rows; up-proj K=4096,N=14336 or down-proj K=14336,N=4096."""
    K, N = (14336, 4096) if down else (4096, 14336)
    return moe_bf16(32, 8, 2, K, N, 1003)


def cfg4(M: int, K: int = 4096, N: int = 14336, group: int = 128) -> Dict[str, torch.Tensor]:
    """W4A16: bf16 a [M,K]; int4 weights [K,N] uniform 0..15 (unpacked here as uint8 `q`), bf16 scales
    U(0.005, 0.02) [K/group, N], int4 zeros [K/group, N] (unpacked uint8 `z`)."""
    g = _gen(1004)
    a = torch.randn(M, K, generator=g).to(torch.bfloat16)
    q = torch.randint(0, 16, (K, N), generator=g, dtype=torch.uint8)
    scales = (torch.rand(K // group, N, generator=g) * 0.015 + 0.005).to(torch.bfloat16)
    z = torch.randint(0, 16, (K // group, N), generator=g, dtype=torch.uint8)
    return dict(a=a, q=q, scales=scales, z=z)


def pack_int4_along_k(q: torch.Tensor) -> torch.Tensor:
    """[K, N] uint8 0..15 -> int32 [K/8, N]; nibble j of a word holds row 8*i + j
    (kernels/triton/inference/gptq/splitk_dequant_gemm.py:56,76)."""
    K, N = q.shape
    v = q.to(torch.int64).reshape(K // 8, 8, N)
    out = torch.zeros(K // 8, N, dtype=torch.int64)
    for j in range(8):
        out |= v[:, j, :] << (4 * j)
    out = torch.where(out >= 2 ** 31, out - 2 ** 32, out)
    return out.to(torch.int32)


def pack_int4_along_n(z: torch.Tensor) -> torch.Tensor:
    """[G, N] uint8 0..15 -> int32 [G, N/8]; nibble j of a word holds column 8*i + j
    (splitk_dequant_gemm.py:57,70)."""
    G, N = z.shape
    v = z.to(torch.int64).reshape(G, N // 8, 8)
    out = torch.zeros(G, N // 8, dtype=torch.int64)
    for j in range(8):
        out |= v[:, :, j] << (4 * j)
    out = torch.where(out >= 2 ** 31, out - 2 ** 32, out)
    return out.to(torch.int32)


def zipf_logits(T: int, E: int, alpha: float, gen: torch.Generator) -> torch.Tensor:
    """Router logits whose top-k follows a Zipf(alpha)-skewed expert popularity: log p_e + Gumbel(0,1)."""
    p = torch.arange(1, E + 1, dtype=torch.float64) ** (-alpha)
    logp = torch.log(p / p.sum()).to(torch.float32)
    u = torch.rand(T, E, generator=gen).clamp_(1e-20, 1.0 - 1e-7)
    gumbel = -torch.log(-torch.log(u))
    return logp[None, :] + gumbel


def cfg5_routing(T: int = 4096, E: int = 256, k: int = 8, seed: int = 1005):
    g = _gen(seed)
    logits = zipf_logits(T, E, 1.1, g)
    return (logits,) + route_reference(logits, k)


def flops(m_sizes, N: int, K: int) -> float:
    return 2.0 * float(sum(int(m) for m in m_sizes)) * N * K
