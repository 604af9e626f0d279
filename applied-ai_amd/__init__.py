"""MI355X-native MoE grouped-GEMM inference path (gfx950 HIP kernels behind a C ABI)."""
from . import _lib
from .ops import grouped_gemm, grouped_gemm_forward, matmul_split_k

__all__ = ["grouped_gemm", "grouped_gemm_forward", "matmul_split_k", "_lib"]
