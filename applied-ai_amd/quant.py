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
    """128 x 128 block quantisation of a [rows, K] weight matrix with the same scale and clamp rule as the
    1 x 128 quantiser (one scale per block). Weight preparation, off the hot path: plain torch ops on whatever
    device w lives on. The reference has no in-tree definition of this quantiser (it calls an un-vendored
    FBGEMM routine, kernels/needs_perf_help/fp8_gemm_bench.py:16-21)."""
    rows, K = w.shape
    t = w.float().reshape(rows // block, block, K // block, block)
    s = t.abs().amax(dim=(1, 3)).clamp_min(1e-12) / 448.0
    q = (t / s[:, None, :, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).reshape(rows, K)
    return q, s.contiguous()
