"""The forward ping-pong kernels in the split-tail tile order (MOE_GG_OP_TILE_ORDER = MOE_GG_ORDER_SPLIT_TAILS) on the
GPU: the collected parity tests of the kernels that take the order (bf16 / fp16 forward, fp8 row-wise and block-scaled,
the fused SiLU-and-mul GEMM, grad_x of the backward pass), run again with the order pinned. Not collected by pytest
under this name (run it by naming the file): the order has run under the CPU emulation only
(tests/test_emu_kernels.py, tests/test_pingpong_prologue_on_host.py); its tests join the collected ones, and the order
may become the default, once this file has passed on a GPU and a timed run has shown what the order is worth."""
import pytest

from tests.test_gpu_backward import (test_adjoint_identity_at_training_size, test_fast_verification_case,  # noqa: F401
                                     test_gradients_from_operands_as_stored_equal_the_transposed_copy_paths, test_ragged_shapes)
from tests.test_gpu_fp8 import (test_against_oracle as test_fp8_against_oracle, test_config5_full_size,  # noqa: F401
                                test_unit_scales_equal_plain_fp8_product)
from tests.test_gpu_grouped_gemm_bf16 import (test_bitwise_deterministic, test_edge_cases,  # noqa: F401
                                              test_fast_verification_shape_and_block_layout, test_large_two_groups,
                                              test_low_tiles_left_to_the_small_m_kernel,
                                              test_mixtral_prefill_shape_sampled_rows, test_rows_beyond_sum_are_untouched)
from tests.test_gpu_moe_layer import (test_fused_moe_prefill_rows_take_the_fused_activation_path,  # noqa: F401
                                      test_swiglu_gemm_equals_gemm_then_silu_and_mul,
                                      test_swiglu_gemm_fp16_equals_gemm_then_silu_and_mul)
from tests.test_gpu_random_shapes import *  # noqa: F401,F403

pytestmark = pytest.mark.gpu
OP_TILE_ORDER, ORDER_SPLIT_TAILS = 2, 1


@pytest.fixture(autouse=True)
def split_tails():
    import applied_ai_amd as A

    lib = A._lib.lib()
    assert lib.moe_gg_set_variant(OP_TILE_ORDER, ORDER_SPLIT_TAILS) == 0
    try:
        yield
    finally:
        lib.moe_gg_set_variant(OP_TILE_ORDER, -1)
