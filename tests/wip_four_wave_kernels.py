"""The four-wave forms of the 256 x 256 kernel on the GPU: MOE_GG_GG_TILED_256_W4 (the lock-step tiled kernel on
four waves of 128 x 128 outputs), MOE_GG_GG_FOURWAVE_256 (the ping-pong kernel's tiles, tile order and slab stream on
four waves, reads and loads placed behind single MFMAs) and MOE_GG_GG_FOURWAVE_TALL (the same with tiles of up to
256 + 32 rows; its ninth fragment's MFMAs are written out in assembly with VGPR accumulators, so this run is also the
first check of their wait states: a wrong result here, not a fault, is what a missing one would look like). None is
ever chosen automatically. The collected parity
tests of the bf16 / fp16 grouped GEMM run again with each variant pinned (shapes a variant cannot take, K % 64 != 0
or unaligned pointers, fall through to the generic kernel as they do for every pinned variant), and with
MOE_GG_GG_FOURWAVE_256 / _TALL pinned the fused SiLU-and-mul GEMM runs its four-wave form in the layer tests. Not collected by
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


@pytest.fixture(autouse=True, params=[6, 7, 8], ids=["tiled_256_w4", "fourwave_256", "fourwave_tall"])
def four_wave_variant(request):
    import applied_ai_amd as A

    lib = A._lib.lib()
    assert lib.moe_gg_set_variant(OP_GG_BF16, request.param) == 0
    try:
        yield request.param
    finally:
        lib.moe_gg_set_variant(OP_GG_BF16, -1)


@pytest.mark.parametrize("sizes", [[257, 272, 273, 288, 289, 0, 544, 1036], [1012, 1039, 1048, 1036, 998, 1023, 1040, 996]])
def test_tails_around_the_tall_tile_limit(sizes, four_wave_variant):
    """Tails of 1, 16, 17 and 32 rows (taken along by the last full tile when MOE_GG_GG_FOURWAVE_TALL is pinned) and 33
    (a tile of their own), and the benchmark's expert sizes; every row against the oracle's fp32 per-expert matmul loop
    (dev/triton_groupGEMM/testing/unit_tests.py:49-55; bar of the grouped-GEMM parity tests: 1e-2 + 1e-2 |ref|)."""
    import torch

    import applied_ai_amd as A
    from oracle import oracle as O

    N, K = 1024, 512
    gen = torch.Generator().manual_seed(77)
    x = (torch.randn(sum(sizes), K, generator=gen) * 0.5).to(torch.bfloat16)
    w = (torch.randn(len(sizes) * N, K, generator=gen) * 0.1).to(torch.bfloat16)
    xd, wd, md = x.cuda(), w.cuda(), torch.tensor(sizes, dtype=torch.int32).cuda()
    y = A.grouped_gemm(xd, wd, md).float().cpu()
    ref = O.grouped_gemm_torch_loop(x.float(), w.float(), sizes)
    assert bool(((y - ref).abs() <= 1e-2 + 1e-2 * ref.abs()).all())
