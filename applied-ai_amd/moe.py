"""A whole MoE layer on top of the grouped GEMM, with the reference's fused_moe signature
(kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:222-296).

The reference pads every expert's token list to a block multiple (moe_align_block_size) and runs a gather-style
GEMM twice; here the rows are gathered once into expert-sorted order and the two products are plain grouped GEMMs
over m_sizes, so no padding rows are computed:

    perm, m_sizes, offsets = group topk_ids by expert (stable)            moe_gg_route_group
    xs  = hidden_states[perm // k]                                        moe_gg_gather_rows
    h1  = grouped_gemm(xs, w1, m_sizes)            [R, 2n]                moe_gg_grouped_gemm_bf16
    h2  = silu(h1[:, :n]) * h1[:, n:]              [R, n]                 moe_gg_silu_and_mul
          (both in one kernel without h1 when there are many rows: moe_gg_grouped_gemm_swiglu_bf16, same bits)
    y2  = grouped_gemm(h2, w2, m_sizes)            [R, d]                 moe_gg_grouped_gemm_bf16
    out[t] = sum_j topk_weights[t, j] * y2[inv[t * k + j]]                moe_gg_invert_perm, moe_gg_combine_topk

Everything runs in the HIP kernels behind include/moe_gg.h; torch only provides the buffers."""
import torch

from . import _lib
from .ops import (_require_cuda, _stream_ptr, grouped_gemm, grouped_gemm_swiglu, grouped_gemm_swiglu_gathered,
                  matmul_split_k_grouped)
from .routing import gather_sorted, route_group

# fused_moe folds SiLU-and-mul into the first GEMM from this many expert-sorted rows on (the fused kernel is the
# 256 x 256 ping-pong kernel; below, the small-M kernels of grouped_gemm are faster than it).
FUSED_SWIGLU_MIN_ROWS = 1024


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """out = silu(x[:, :n]) * x[:, n:] for bf16 or fp16 x [rows, 2n] (ops.silu_and_mul, v0_moe_fused.py:284)."""
    if x.dim() != 2 or x.dtype not in (torch.bfloat16, torch.float16) or x.shape[1] % 2:
        raise ValueError("x must be bf16 or fp16 [rows, 2n]")
    dev = _require_cuda(x)
    x = x.contiguous()
    rows, n = x.shape[0], x.shape[1] // 2
    out = torch.empty((rows, n), dtype=x.dtype, device=dev)
    with torch.cuda.device(dev):
        L = _lib.lib()
        fn = L.moe_gg_silu_and_mul_f16 if x.dtype == torch.float16 else L.moe_gg_silu_and_mul
        rc = fn(x.data_ptr(), out.data_ptr(), rows, n, _stream_ptr(dev))
    _lib.check(rc, "moe_gg_silu_and_mul")
    return out


def combine_topk(y: torch.Tensor, perm: torch.Tensor, offsets: torch.Tensor, topk_weights: torch.Tensor,
                 out: torch.Tensor = None) -> torch.Tensor:
    """out[t] = sum_j topk_weights[t, j] * y[row of (t, j)], y in expert-sorted row order (perm as from
    route_group / route_topk, offsets its [E + 1] prefix table); fp32 accumulation, result in y's dtype (bf16 or
    fp16; the weights are fp32 or have y's dtype)."""
    if y.dim() != 2 or y.dtype not in (torch.bfloat16, torch.float16):
        raise ValueError("y must be bf16 or fp16 [rows, d]")
    if topk_weights.dim() != 2 or topk_weights.dtype not in (torch.float32, y.dtype):
        raise ValueError("topk_weights must be [T, k] in fp32 or in y's dtype")
    dev = _require_cuda(y, perm, offsets, topk_weights)
    y = y.contiguous()
    topk_weights = topk_weights.contiguous()
    T, k = topk_weights.shape
    if perm.shape[0] != T * k:
        raise ValueError("perm must have T * k entries")
    inv = torch.full((T * k,), -1, dtype=torch.int32, device=dev)
    if out is None:
        out = torch.empty((T, y.shape[1]), dtype=y.dtype, device=dev)
    elif out.shape != (T, y.shape[1]) or out.dtype != y.dtype or not out.is_contiguous():
        raise ValueError("out must be a contiguous [T, d] tensor of y's dtype")
    fp16 = y.dtype == torch.float16
    wdt = 2 if topk_weights.dtype == torch.float32 else (1 if fp16 else 0)  # MOE_GG_DTYPE_FP32 / _FP16 / _BF16
    with torch.cuda.device(dev):
        L = _lib.lib()
        rc = L.moe_gg_invert_perm(perm.data_ptr(), inv.data_ptr(), T * k, offsets[-1:].data_ptr(), _stream_ptr(dev))
        _lib.check(rc, "moe_gg_invert_perm")
        fn = L.moe_gg_combine_topk_f16 if fp16 else L.moe_gg_combine_topk
        rc = fn(y.data_ptr(), inv.data_ptr(), topk_weights.data_ptr(), wdt, out.data_ptr(), T, k,
                y.shape[1], y.shape[0], _stream_ptr(dev))
    _lib.check(rc, "moe_gg_combine_topk")
    return out


def invoke_fused_moe_kernel(A: torch.Tensor, B: torch.Tensor, C: torch.Tensor, topk_weights: torch.Tensor,
                            topk_ids: torch.Tensor, sorted_token_ids: torch.Tensor = None,
                            expert_ids: torch.Tensor = None, num_tokens_post_padded: torch.Tensor = None,
                            mul_routed_weight: bool = False, top_k: int = 1, config: dict = None) -> None:
    """One gather-style expert GEMM of the reference's fused MoE with its call signature
    (kernels/triton/inference/col_major_moe_gemm/v0_moe_fused.py:183-220, kernel :17-135): for every flat
    position p = token * k + j of topk_ids, C.view(-1, N)[p] = A[p // top_k] @ B[topk_ids[p]].T, times
    topk_weights.view(-1)[p] if mul_routed_weight (:122-126). A is [M, K] with top_k = k for the first GEMM and
    [M * k, K] with top_k = 1 for the second; B [E, N, K]; C [M, k, N], written in place. bf16 or fp16.

    The rows are grouped by expert from topk_ids itself (the grouping that sorted_token_ids / expert_ids /
    num_tokens_post_padded encode with padding; those arguments and config are accepted and not needed), gathered,
    multiplied by the grouped GEMM and scattered back; the routed weight multiplies the bf16 product."""
    assert A.is_contiguous() and B.is_contiguous() and C.is_contiguous(), "A, B and C must be contiguous"
    assert A.dtype in (torch.bfloat16, torch.float16) and B.dtype == A.dtype and C.dtype == A.dtype, "bf16 or fp16"
    E, N, K = B.shape
    assert A.shape[1] == K, "Incompatible dimensions"
    n = topk_ids.numel()
    assert C.numel() == n * N and A.shape[0] * top_k == n, "C must be [M, k, N] and A [M * k / top_k, K]"
    _require_cuda(A, B, C, topk_ids)
    ids = topk_ids if topk_ids.dtype == torch.int32 else topk_ids.to(torch.int32)
    perm, m_sizes, offsets = route_group(ids, E)
    xs = gather_sorted(A, perm, top_k, offsets)
    y = grouped_gemm(xs, B.view(E * N, K), m_sizes)
    if mul_routed_weight:
        w = topk_weights if topk_weights.dtype in (torch.float32, A.dtype) else topk_weights.float()
        w = w.contiguous().view(n, 1)
    else:
        w = torch.ones((n, 1), dtype=torch.float32, device=A.device)
    combine_topk(y, perm, offsets, w, out=C.view(n, N))


def fused_moe(hidden_states: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, topk_weights: torch.Tensor,
              topk_ids: torch.Tensor, inplace: bool = False, fuse_gather: bool = False) -> torch.Tensor:
    """Mixture-of-experts layer with top-k gating; arguments as the reference's fused_moe
    (v0_moe_fused.py:222-227): hidden_states [M, K], w1 [E, 2n, K], w2 [E, d, n], topk_weights / topk_ids [M, k].
    bf16 or fp16 (:216). With inplace=True the result is written into hidden_states (d must equal K), as the
    reference does (:291-294). fuse_gather=True lets the first GEMM read the token rows through the permutation
    (as the reference's kernel does through sorted_token_ids, :75-80) instead of from a gathered copy, where the
    fused first GEMM runs at all; the result has the same bits."""
    assert hidden_states.shape[1] == w1.shape[2], "Incompatible dimensions"
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert w1.is_contiguous(), "Expert weights1 must be contiguous"
    assert w2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype in (torch.bfloat16, torch.float16), "Only float16 and bfloat16 are supported"
    assert w1.dtype == hidden_states.dtype and w2.dtype == hidden_states.dtype, "weights must have the activations' dtype"
    _require_cuda(hidden_states, w1, w2, topk_weights, topk_ids)
    E, two_n, K = w1.shape
    assert two_n % 2 == 0 and w2.shape[0] == E and w2.shape[2] == two_n // 2, "Incompatible expert weights"
    k = topk_ids.shape[1]
    ids = topk_ids if topk_ids.dtype == torch.int32 else topk_ids.to(torch.int32)
    tw = topk_weights if topk_weights.dtype in (torch.float32, hidden_states.dtype) else topk_weights.float()

    perm, m_sizes, offsets = route_group(ids, E)
    rows = perm.shape[0]
    swiglu_tiles = (rows // 256 + E) * ((two_n // 2 + 127) // 128)   # bound of the fused kernel's tile table
    fused_act = (rows >= FUSED_SWIGLU_MIN_ROWS and K % 64 == 0 and two_n % 8 == 0 and two_n * K < 2 ** 31
                 and swiglu_tiles <= 1023 * 256)
    if fused_act and fuse_gather and hidden_states.shape[0] * K * 2 < 2 ** 31:
        h2 = grouped_gemm_swiglu_gathered(hidden_states, perm, k, w1.view(E * two_n, K), m_sizes)
    else:
        xs = gather_sorted(hidden_states, perm, k, offsets)
        if fused_act:
            h2 = grouped_gemm_swiglu(xs, w1.view(E * two_n, K), m_sizes)
        else:
            h2 = silu_and_mul(grouped_gemm(xs, w1.view(E * two_n, K), m_sizes))
    y2 = grouped_gemm(h2, w2.view(E * w2.shape[1], w2.shape[2]), m_sizes)
    return combine_topk(y2, perm, offsets, tw, out=hidden_states if inplace else None)


def dequant_gemm_moe(hidden_states: torch.Tensor, qw1: torch.Tensor, qw2: torch.Tensor, scales_qw1: torch.Tensor,
                     scales_qw2: torch.Tensor, zeros_qw1: torch.Tensor, zeros_qw2: torch.Tensor, topk_ids: torch.Tensor,
                     topk_weights: torch.Tensor = None, zero_offset: int = 1) -> torch.Tensor:
    """MoE layer with int4 (GPTQ) expert weights; arguments as the reference's dequant_gemm_moe
    (kernels/triton/inference/gptq/mixtral/w4a16_fused_dequant_gemm.py:255-318): hidden_states [M, K] bf16 or fp16,
    qw1 [E, K/8, 2n] / qw2 [E, n/8, d] int32, scales [E, K/g, 2n] / [E, n/g, d] in that dtype, zeros [E, K/g, 2n/8] /
    [E, n/g, d/8] int32, topk_ids [M, k]. Like the reference, the k rows of a token are summed without routed
    weights (:316-317) unless topk_weights is given. Same pipeline as fused_moe with the two products done by
    the grouped W4A16 kernel (moe_gg_w4a16_grouped)."""
    assert hidden_states.is_contiguous(), "Hidden_states must be contiguous"
    assert qw1.is_contiguous(), "Expert weights1 must be contiguous"
    assert qw2.is_contiguous(), "Expert weights2 must be contiguous"
    assert hidden_states.dtype in (torch.bfloat16, torch.float16), "bf16 or fp16"
    _require_cuda(hidden_states, qw1, qw2, scales_qw1, scales_qw2, zeros_qw1, zeros_qw2, topk_ids)
    E = qw1.shape[0]
    assert hidden_states.shape[1] == qw1.shape[1] * 8, "Incompatible dimensions"
    assert qw2.shape[0] == E and qw2.shape[1] * 8 * 2 == qw1.shape[2], "Incompatible expert weights"
    T, k = topk_ids.shape
    ids = topk_ids if topk_ids.dtype == torch.int32 else topk_ids.to(torch.int32)
    if topk_weights is None:
        tw = torch.ones((T, k), dtype=torch.float32, device=hidden_states.device)
    else:
        tw = topk_weights if topk_weights.dtype in (torch.float32, hidden_states.dtype) else topk_weights.float()

    perm, m_sizes, offsets = route_group(ids, E)
    xs = gather_sorted(hidden_states, perm, k, offsets)
    h1 = matmul_split_k_grouped(xs, qw1, scales_qw1, zeros_qw1, m_sizes, zero_offset=zero_offset)
    h2 = silu_and_mul(h1)
    y2 = matmul_split_k_grouped(h2, qw2, scales_qw2, zeros_qw2, m_sizes, zero_offset=zero_offset)
    return combine_topk(y2, perm, offsets, tw)
