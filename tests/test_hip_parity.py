"""GPU parity: the HIP path, called through the reference's plugin signature, against the golden
vectors written from the reference's compiled dp_core and against the C oracle."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

SMALL = ([f"ties_{i}" for i in range(10)] + [f"rand_{i}" for i in range(10)] +
         [f"infeasible_{i}" for i in range(10)] + [f"cfg3_smallV_{i}" for i in range(8)] +
         ["cfg2_small", "cfg4_small", "galvatron_like", "cfg0", "cfg0_other_time"])


@pytest.mark.parametrize("name", SMALL)
def test_golden_small_full_arrays(golden, name):
    """results AND the full f / mark arrays (reference layouts) are bit-identical"""
    rec = golden[name]
    inst = H.build_case(rec)
    total, res, rem, f, mark = H.hip_solve(inst, export=True)
    H.assert_same_results((total, res, rem), H.golden_results(rec), name)
    assert H.sha(f) == rec["f_sha256"], f"{name}: final f differs"
    assert H.sha(mark) == rec["mark_sha256"], f"{name}: argmin table differs"


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg4"])
def test_golden_full_size(golden, name):
    if name not in golden:
        pytest.skip("fixture not generated")
    rec = golden[name]
    inst = H.build_case(rec)
    H.assert_same_results(H.hip_solve(inst), H.golden_results(rec), name)
