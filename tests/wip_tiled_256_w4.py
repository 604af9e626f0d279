"""The 256 x 256 tiled kernel on four waves of 128 x 128 outputs each (MOE_GG_GG_TILED_256_W4, never chosen
automatically) on the GPU, against the oracle. Not collected by pytest under this name (run it by naming the file):
the variant has run under the CPU emulation only; it joins the collected tests once it has passed on a GPU."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import bf16_inputs, to_np

pytestmark = pytest.mark.gpu
OP_GG_BF16, TILED_256_W4 = 0, 6


@pytest.mark.parametrize("sizes,N,K", [([300, 0, 70, 530], 512, 256), ([1024, 1024], 1024, 512)])
def test_four_wave_tiled_kernel_against_oracle(sizes, N, K):
    import applied_ai_amd as A

    lib = A._lib.lib()
    G, M = len(sizes), sum(sizes)
    x, w, _ = bf16_inputs(G, M, N, K, seed=61)
    print(f"four-wave 256x256 tiled kernel sizes={sizes} N={N} K={K}", flush=True)
    assert lib.moe_gg_set_variant(OP_GG_BF16, TILED_256_W4) == 0
    try:
        y = A.grouped_gemm(x.cuda(), w.cuda(), torch.tensor(sizes, dtype=torch.int32).cuda())
        torch.cuda.synchronize()
    finally:
        lib.moe_gg_set_variant(OP_GG_BF16, -1)
    ref = O.grouped_gemm(to_np(x), to_np(w), sizes)
    np.testing.assert_allclose(to_np(y), ref, rtol=1e-2, atol=1e-2)
