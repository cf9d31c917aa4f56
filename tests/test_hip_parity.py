"""GPU parity: the HIP path, called through the reference's plugin signature, against the golden
vectors written from the reference's compiled dp_core and against the C oracle."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

SMALL = ([f"ties_{i}" for i in range(10)] + [f"rand_{i}" for i in range(10)] +
         [f"infeasible_{i}" for i in range(10)] + [f"cfg3_smallV_{i}" for i in range(8)] +
         ["cfg2_small", "cfg4_small", "galvatron_like", "cfg0", "cfg0_other_time"] +
         [f"zeromem_{i}" for i in range(8)] + [f"initf_{i}" for i in range(8)] + ["initf_galvatron_like"])


@pytest.mark.parametrize("name", SMALL)
def test_golden_small_full_arrays(golden, name):
    """results AND the full f / mark arrays (reference layouts) are bit-identical"""
    rec = golden[name]
    inst = H.build_case(rec)
    total, res, rem, f, mark = H.hip_solve(inst, export=True)
    H.assert_same_results((total, res, rem), H.golden_results(rec), name)
    assert H.sha(f) == rec["f_sha256"], f"{name}: final f differs"
    assert H.sha(mark) == rec["mark_sha256"], f"{name}: argmin table differs"


def test_golden_covers_every_benchmark_config_on_the_gpu_box(golden):
    """The same guard as the CPU suite's: every benchmark configuration has its vectors here too."""
    for name in ["cfg0", "cfg1", "cfg2", "cfg4"] + [f"cfg3_{i:03d}" for i in range(256)]:
        assert name in golden, name


@pytest.mark.parametrize("name", ["cfg1", "cfg2", "cfg4"] + [f"zeromem_{i}" for i in range(8)] +
                         [f"initf_{i}" for i in range(8)] + ["initf_galvatron_like"])
def test_golden_full_size(golden, name):
    assert name in golden, f"the committed vectors have no case {name}: a lost fixture is a failure, not a skip"
    rec = golden[name]
    inst = H.build_case(rec)
    H.assert_same_results(H.hip_solve(inst), H.golden_results(rec), name)
