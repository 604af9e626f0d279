"""The two four-wave forms of the 256 x 256 kernel on the GPU: MOE_GG_GG_TILED_256_W4 (the lock-step tiled kernel on
four waves of 128 x 128 outputs) and MOE_GG_GG_FOURWAVE_256 (the ping-pong kernel's tiles, tile order and slab stream on
four waves, reads and loads placed behind single MFMAs). Neither is ever chosen automatically. The collected parity
tests of the bf16 / fp16 grouped GEMM run again with each variant pinned (shapes a variant cannot take, K % 64 != 0
or unaligned pointers, fall through to the generic kernel as they do for every pinned variant), and with
MOE_GG_GG_FOURWAVE_256 pinned the fused SiLU-and-mul GEMM runs its four-wave form in the layer tests. Not collected by
pytest under this name (run it by naming the file): the kernels have run under the CPU emulation only
(tests/test_emu_kernels.py); they join the collected tests once this file has passed on a GPU."""
import pytest

from tests.test_gpu_grouped_gemm_bf16 import (test_bitwise_deterministic, test_config1_plumbing_from_golden_fixture,  # noqa: F401
                                              test_edge_cases, test_fast_verification_shape_and_block_layout,
                                              test_large_two_groups, test_mixtral_prefill_shape_sampled_rows,
                                              test_reference_base_shapes, test_reference_various_dimensions,
                                              test_rows_beyond_sum_are_untouched)

from tests.test_gpu_moe_layer import (test_fused_moe_prefill_rows_take_the_fused_activation_path,  # noqa: F401,E402
                                      test_swiglu_gemm_equals_gemm_then_silu_and_mul,
                                      test_swiglu_gemm_fp16_equals_gemm_then_silu_and_mul)

pytestmark = pytest.mark.gpu
OP_GG_BF16 = 0


@pytest.fixture(autouse=True, params=[6, 7], ids=["tiled_256_w4", "fourwave_256"])
def four_wave_variant(request):
    import applied_ai_amd as A

    lib = A._lib.lib()
    assert lib.moe_gg_set_variant(OP_GG_BF16, request.param) == 0
    try:
        yield request.param
    finally:
        lib.moe_gg_set_variant(OP_GG_BF16, -1)
