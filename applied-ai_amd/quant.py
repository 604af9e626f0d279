"""fp8 quantisers used to prepare inputs of the block-scaled fp8 grouped GEMM."""
from typing import Tuple

import torch

from . import _lib
from .ops import _require_cuda, _stream_ptr


def float8_groupwise_quantize(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """1 x 128 group-wise quantisation to torch.float8_e4m3fn; returns (q like x, scales [..., K/128] fp32).
    Drop-in for float8_groupwise_quantize (kernels/triton/inference/fp8/float8_groupwise_quant.py:53-91)."""
    if block_size != 128:
        raise ValueError("only block_size = 128 is implemented")
    if x.size(-1) % block_size != 0:
        raise ValueError(f"Input tensor must have a last dimension that is a multiple of {block_size}")
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("x must be fp32 or bf16")
    dev = _require_cuda(x)
    x = x.contiguous()
    out = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    scales = x.new_empty(*x.size()[:-1], x.size(-1) // block_size, dtype=torch.float32)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_fp8_groupwise_quant(x.data_ptr(), 0 if x.dtype == torch.bfloat16 else 2, out.data_ptr(),
                                                   scales.data_ptr(), x.numel(), _stream_ptr(dev))
    _lib.check(rc, "moe_gg_fp8_groupwise_quant")
    return out, scales


def float8_blockwise_quantize_weight(w: torch.Tensor, block: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """128 x 128 block quantisation of a [rows, K] weight matrix (or a stack [G, N, K], taken as [G*N, K]) with the
    scale and clamp rule of the 1 x 128 quantiser, one scale per block: returns (q like w as float8_e4m3fn, scales
    [rows/128, K/128] fp32), the w / w_scale of grouped_gemm_fp8_blockwise. The reference takes this step from an
    un-vendored package (quantize_fp8_block, kernels/needs_perf_help/fp8_gemm_bench.py:16-21)."""
    if block != 128:
        raise ValueError("only block = 128 is implemented")
    if w.dim() not in (2, 3) or w.size(-1) % block != 0 or w.size(-2) % block != 0:
        raise ValueError(f"w must be [rows, K] or [G, N, K] with N (rows) and K multiples of {block}")
    if w.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("w must be fp32 or bf16")
    dev = _require_cuda(w)
    w = w.contiguous()
    K = w.size(-1)
    rows = w.numel() // K
    out = torch.empty_like(w, dtype=torch.float8_e4m3fn)
    scales = torch.empty(rows // block, K // block, dtype=torch.float32, device=w.device)
    with torch.cuda.device(dev):
        rc = _lib.lib().moe_gg_fp8_block128_quant(w.data_ptr(), 0 if w.dtype == torch.bfloat16 else 2, out.data_ptr(),
                                                  scales.data_ptr(), rows, K, _stream_ptr(dev))
    _lib.check(rc, "moe_gg_fp8_block128_quant")
    return out, scales
