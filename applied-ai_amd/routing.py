"""Routing in front of the grouped GEMM: top-k expert choice, expert-sorted permutation, m_sizes, offsets.

The host-side mirror of what the reference's MoE tests do with torch.topk
(kernels/triton/inference/col_major_moe_gemm/test_moe_gemm.py:54-57) plus the grouping of the external
moe_align_block_size op (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:141-166, without its
padding); the work runs in the HIP kernels behind include/moe_gg.h."""
from typing import Tuple

import torch

from . import _lib
from .ops import _require_cuda, _stream_ptr


def route_topk(logits: torch.Tensor, k: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """logits [T, E] fp32 -> (ids [T, k] int32, perm [T*k] int32, m_sizes [E] int32, offsets [E+1] int32).

    ids are the k best experts per token in descending score (ties to the lower id); perm lists the flat
    positions token*k + j grouped by ascending expert, stable, so sorted row i comes from token perm[i] // k;
    m_sizes / offsets are what grouped_gemm consumes."""
    if logits.dim() != 2 or logits.dtype != torch.float32:
        raise ValueError("logits must be fp32 [T, E]")
    dev = _require_cuda(logits)
    logits = logits.contiguous()
    T, E = logits.shape
    ids = torch.empty((T, k), dtype=torch.int32, device=dev)
    perm = torch.empty((T * k,), dtype=torch.int32, device=dev)
    m_sizes = torch.empty((E,), dtype=torch.int32, device=dev)
    offsets = torch.empty((E + 1,), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_route_topk(logits.data_ptr(), T, E, k, ids.data_ptr(), perm.data_ptr(),
                                          m_sizes.data_ptr(), offsets.data_ptr(), _stream_ptr(dev))
    _lib.check(rc, "moe_gg_route_topk")
    return ids, perm, m_sizes, offsets


def route_group(topk_ids: torch.Tensor, num_experts: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Grouping only, for expert ids chosen elsewhere: topk_ids int32 [T, k] -> (perm, m_sizes, offsets)."""
    if topk_ids.dtype != torch.int32:
        raise ValueError("topk_ids must be int32")
    dev = _require_cuda(topk_ids)
    flat = topk_ids.contiguous().reshape(-1)
    n = flat.shape[0]
    perm = torch.empty((n,), dtype=torch.int32, device=dev)
    m_sizes = torch.empty((num_experts,), dtype=torch.int32, device=dev)
    offsets = torch.empty((num_experts + 1,), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_route_group(flat.data_ptr(), n, num_experts, perm.data_ptr(), m_sizes.data_ptr(),
                                           offsets.data_ptr(), _stream_ptr(dev))
    _lib.check(rc, "moe_gg_route_group")
    return perm, m_sizes, offsets


def moe_align_block_size(topk_ids: torch.Tensor, block_size: int,
                         num_experts: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Drop-in for the reference's moe_align_block_size (kernels/triton/inference/col_major_moe_gemm/
    v0_moe_fused.py:138-180), which wraps an external op: topk_ids [T, k] -> (sorted_token_ids
    [T*k + E*(block_size-1)] int32, expert_ids [T*k + E] int32, num_tokens_post_padded [1] int32). The flat positions
    token*k + j are grouped by ascending expert, stable, each expert's run padded with the value T*k up to a multiple
    of block_size (worked example :157-165); expert_ids holds the expert of every block (-1 beyond the last one,
    where the reference leaves the buffer uninitialised)."""
    ids = topk_ids if topk_ids.dtype == torch.int32 else topk_ids.to(torch.int32)
    perm, m_sizes, _ = route_group(ids, num_experts)
    dev = perm.device
    n = perm.shape[0]
    sorted_ids = torch.empty((n + num_experts * (block_size - 1),), dtype=torch.int32, device=dev)
    expert_ids = torch.empty((n + num_experts,), dtype=torch.int32, device=dev)
    num_post_pad = torch.empty((1,), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_align_block_size(perm.data_ptr(), m_sizes.data_ptr(), num_experts, n, block_size,
                                                sorted_ids.data_ptr(), expert_ids.data_ptr(), num_post_pad.data_ptr(),
                                                _stream_ptr(dev))
    _lib.check(rc, "moe_gg_align_block_size")
    return sorted_ids, expert_ids, num_post_pad


def gather_sorted(x: torch.Tensor, perm: torch.Tensor, k: int, offsets: torch.Tensor = None) -> torch.Tensor:
    """x_sorted[i] = x[perm[i] // k]: the token rows in expert-sorted order. With offsets (the [E + 1] table of
    route_group / route_topk) only its last entry's worth of perm is in use (ids outside [0, E) were dropped); the
    rows behind it, and rows whose perm entry names no row of x, come back as zeros."""
    if x.dim() != 2 or perm.dtype != torch.int32:
        raise ValueError("x must be 2-D and perm int32")
    dev = _require_cuda(x, perm)
    if offsets is not None and (offsets.dtype != torch.int32 or offsets.device != dev or not offsets.is_contiguous()):
        raise ValueError("offsets must be a contiguous int32 tensor on x's device")
    x = x.contiguous()
    n = perm.shape[0]
    out = torch.empty((n, x.shape[1]), dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_gather_rows(x.data_ptr(), perm.data_ptr(), k, out.data_ptr(), n,
                                           x.shape[1] * x.element_size(), x.shape[0],
                                           offsets[-1:].data_ptr() if offsets is not None else None, _stream_ptr(dev))
    _lib.check(rc, "moe_gg_gather_rows")
    return out
