"""GPU side of the opt-in m_sizes validation of the Python mirror (the host logic itself is covered without a GPU in
tests/test_host_checks.py). Collected late on purpose, so that a failure here cannot hide the parity tests before it."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.gpu_util import to_np

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def test_validate_option_on_device_tensors():
    """validate=True: the two cases the reference's tests expect an exception for (sum(m_sizes) > M, a negative
    size; dev/triton_groupGEMM/testing/unit_tests.py:191-212) raise ValueError; valid sizes give the same result as
    without the check; without it the kernels clamp the sizes and nothing is touched out of bounds."""
    import applied_ai_amd as A

    x = torch.randn(64, 32).to(torch.bfloat16).cuda()
    w = torch.randn(64, 32).to(torch.bfloat16).cuda()
    good = torch.tensor([32, 32], dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        A.grouped_gemm(x, w, torch.tensor([32, 40], dtype=torch.int32, device="cuda"), validate=True)
    with pytest.raises(ValueError):
        A.grouped_gemm(x, w, torch.tensor([40, -8], dtype=torch.int32, device="cuda"), validate=True)
    assert torch.equal(A.grouped_gemm(x, w, good, validate=True), A.grouped_gemm(x, w, good))
    y = A.grouped_gemm(x, w, torch.tensor([40, -8], dtype=torch.int32, device="cuda"))   # clamped: 40 rows, then none
    torch.cuda.synchronize()
    ref = O.grouped_gemm(to_np(x), to_np(w), [40, 0])
    np.testing.assert_allclose(to_np(y[:40]), ref[:40], rtol=RTOL, atol=ATOL)
