"""MI355X-native MoE grouped-GEMM inference path (gfx950 HIP kernels behind a C ABI)."""
from . import _lib
from .quant import float8_blockwise_quantize_weight, float8_groupwise_quantize
from .moe import combine_topk, dequant_gemm_moe, fused_moe, invoke_fused_moe_kernel, silu_and_mul
from .routing import gather_sorted, moe_align_block_size, route_group, route_topk
from .ops import (a100_qlinear, h100_qlinear, small_qlinear, grouped_gemm, grouped_gemm_backward, grouped_gemm_forward, grouped_gemm_fp8_blockwise, grouped_gemm_fp8_rowwise, grouped_gemm_fp8_rowwise_forward, grouped_gemm_swiglu, grouped_gemm_swiglu_gathered,
                  matmul_split_k, matmul_split_k_grouped)

__all__ = ["grouped_gemm", "grouped_gemm_forward", "grouped_gemm_backward", "grouped_gemm_fp8_rowwise", "grouped_gemm_fp8_blockwise",
           "matmul_split_k", "route_topk", "route_group", "gather_sorted", "float8_groupwise_quantize",
           "float8_blockwise_quantize_weight", "fused_moe", "silu_and_mul", "combine_topk", "matmul_split_k_grouped",
           "dequant_gemm_moe", "grouped_gemm_swiglu", "grouped_gemm_swiglu_gathered", "grouped_gemm_fp8_rowwise_forward", "moe_align_block_size", "invoke_fused_moe_kernel", "a100_qlinear", "h100_qlinear", "small_qlinear", "_lib"]
