"""Host-side argument checks of the Python mirror that need no GPU: the opt-in m_sizes validation
(dev/triton_groupGEMM/testing/unit_tests.py:191-212 expects an exception for sum(m_sizes) > M and for negative sizes)."""
import pytest
import torch

import applied_ai_amd as A
from applied_ai_amd.ops import check_m_sizes


def test_check_m_sizes_accepts_valid_and_rejects_bad():
    check_m_sizes(torch.tensor([32, 32], dtype=torch.int32), 64)
    check_m_sizes(torch.tensor([0, 0, 7], dtype=torch.int32), 64)       # fewer rows than M is fine
    check_m_sizes(torch.zeros(0, dtype=torch.int32), 0)
    with pytest.raises(ValueError, match="exceeds"):
        check_m_sizes(torch.tensor([32, 40], dtype=torch.int32), 64)    # unit_tests.py:195-201
    with pytest.raises(ValueError, match="negative"):
        check_m_sizes(torch.tensor([40, -8], dtype=torch.int32), 64)    # unit_tests.py:203-212
    with pytest.raises(ValueError, match="exceeds"):
        check_m_sizes(torch.tensor([2**31 - 1, 2**31 - 1], dtype=torch.int32), 64)   # no int32 wrap-around in the sum


@pytest.mark.parametrize("fn", ["grouped_gemm", "grouped_gemm_forward"])
def test_validate_runs_before_the_launch(fn):
    """With validate=True a bad m_sizes raises ValueError before anything touches a device (here: host tensors, which
    would otherwise be refused with RuntimeError because there is no CPU path); off by default."""
    x = torch.zeros(64, 32, dtype=torch.bfloat16)
    w = torch.zeros(64, 32, dtype=torch.bfloat16)
    bad = torch.tensor([32, 40], dtype=torch.int32)
    with pytest.raises(ValueError):
        getattr(A, fn)(x, w, bad, validate=True)
    with pytest.raises(RuntimeError, match="no CPU path"):
        getattr(A, fn)(x, w, bad)
    with pytest.raises(RuntimeError, match="no CPU path"):
        getattr(A, fn)(x, w, torch.tensor([32, 32], dtype=torch.int32), validate=True)


def test_validate_on_the_fp8_entry_points():
    f8 = torch.float8_e4m3fn
    x = torch.zeros(64, 128, dtype=torch.uint8).view(f8)
    w = torch.zeros(256, 128, dtype=torch.uint8).view(f8)
    neg = torch.tensor([40, -8], dtype=torch.int32)
    with pytest.raises(ValueError, match="negative"):
        A.grouped_gemm_fp8_rowwise(x, w, neg, torch.ones(64), torch.ones(256), validate=True)
    with pytest.raises(ValueError, match="negative"):
        A.grouped_gemm_fp8_rowwise_forward(x, w, neg, torch.ones(64), torch.ones(256), validate=True)
    with pytest.raises(ValueError, match="negative"):
        A.grouped_gemm_fp8_blockwise(x, w, neg, torch.ones(64, 1), torch.ones(2, 1), validate=True)
