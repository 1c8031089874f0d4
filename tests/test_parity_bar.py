"""The comparison the GPU parity tests use (gpu_harness.assert_parity), tried on the oracle's own
output for the bench shape: small V over thousands of keys gives outputs of about 2e-3, far below
the absolute tolerance, so the bar must also be relative to the expected values."""
import numpy as np
import pytest

import workloads as W
from gpu_harness import assert_parity, MAX_ABS


def test_the_bar_rejects_zeros_a_scaled_output_and_one_wrong_row(orc):
    case = W.c2(16)
    want = orc.attention_bf16(case["buf"], case["ldi"], 0, case["q_dim"], case["q_dim"] + case["kv_dim"], case["seq"],
                              case["seq"], case["heads"], case["kv_heads"], 128, case["scale"], False, None)
    assert np.abs(want).max() < MAX_ABS          # the absolute bar alone cannot see anything here
    assert_parity(want.astype(np.float32), want, "identity")
    one_row = want.copy()
    one_row[17] = -one_row[17]
    for wrong in (np.zeros_like(want), 0.9 * want, one_row):
        with pytest.raises(AssertionError):
            assert_parity(wrong, want, "must fail")
    with pytest.raises(AssertionError):
        assert_parity(np.zeros_like(want), np.zeros_like(want), "zero reference")
    assert_parity(np.zeros_like(want), np.zeros_like(want), "zero reference allowed", zero_reference_ok=True)
    bad = want.copy()
    bad[0, 0] = np.nan
    with pytest.raises(AssertionError):
        assert_parity(bad, want, "nan")
