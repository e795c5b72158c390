"""Parity proper: every reference golden case through the HIP C ABI."""
import numpy as np
import pytest

import tvx_case as TC

pytestmark = pytest.mark.gpu
# the layout-inference fixtures are source graphs for the C++ API's transform: tests/test_cpp_api.py runs them
CASES = [c for c in TC.all_cases() if not c[1].get("layout_inference")]


@pytest.mark.parametrize("item", CASES, ids=TC.case_id)
def test_hip_matches_reference_golden(item, oracle):
    _, case = item
    out = TC.run_case_gpu(case)
    assert TC.matches(case, out), (out[:16], TC.golden_of(case)[:16])
    # and bit-for-bit the oracle on integer outputs
    ref = oracle.run_case(case)
    if out.dtype in (np.uint8, np.int8):
        assert np.array_equal(out, ref)
    else:
        assert np.allclose(out.astype(np.float32), ref.astype(np.float32), rtol=1e-2, atol=1e-3)
