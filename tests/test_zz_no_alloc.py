"""gdp_solve_static -- the entry point that obtains no memory -- against gdp_solve, through the C ABI.

Collected last on purpose (file name): it works in the library's one static device array, twice in a
row, the second time on a smaller instance, so that anything a call wrongly kept from the one before
would show."""
import numpy as np
import pytest

import helpers as H
from galvatron_dp import _lib, workloads as W

pytestmark = pytest.mark.gpu


def _problem(inst, **kw):
    keys = sorted(inst.other_mem)
    return _lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                        [inst.other_time[k] for k in keys], inter_index=inst.inter_index, **kw)


def _same(a, b, ctx):
    assert a.total.tobytes() == b.total.tobytes(), f"{ctx}: totals differ {a.total} {b.total}"
    assert np.array_equal(a.remaining, b.remaining), f"{ctx}: remaining differs"
    assert np.array_equal(a.res, b.res), f"{ctx}: strategy lists differ"


def test_static_entry_point_matches_gdp_solve_twice_in_a_row(golden):
    """Two calls in a row, the second on a smaller instance (fewer layers, strategies and rows: every
    table of the second call lies inside memory the first one used)."""
    rng = np.random.Generator(np.random.PCG64(77))
    big = W.random_instance(rng, 12, 44, 9000, mem_hi=900, inf_frac=0.1)
    small = W.random_instance(rng, 5, 22, 1500, integer_costs=True, mem_hi=300, inf_frac=0.05)
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")

    def free_bytes():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    for n, inst in enumerate((big, small)):
        want = _problem(inst)
        _lib.solve_batch([want])                       # gdp_solve_batch of one instance is gdp_solve
        got = _problem(inst)
        before = free_bytes()
        _lib.solve_static(got)
        assert n == 0 or free_bytes() == before, "the second call changed the free device memory"
        _same(got, want, f"call {n}")
        assert np.isfinite(want.total).any(), "the case should have feasible keys"


@pytest.mark.parametrize("name", ["cfg0", "galvatron_like", "ties_3", "infeasible_2", "cfg4_small", "zeromem_3", "zeromem_6"])
def test_static_entry_point_on_golden_cases(golden, name):
    """... and against the reference's results for recorded cases, the Galvatron-like shape included."""
    rec = golden[name]
    inst = H.build_case(rec)
    prob = _problem(inst)
    _lib.solve_static(prob)
    keys = rec["keys"]
    got = ({k: prob.total[i] for i, k in enumerate(keys)},
           {k: [int(x) if prob.remaining[i] != -1 else -1 for x in prob.res[i]] for i, k in enumerate(keys)},
           {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
    H.assert_same_results(got, H.golden_results(rec), name)
