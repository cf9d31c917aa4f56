"""Pins for the CPU oracle (oracle/dp_oracle.c) that need neither the reference nor a GPU:
a hand-derived known answer, brute-force path enumeration, closed forms and invariants.
Each is chosen so that a plausible mistake (dropped term, wrong association, wrong tie-break,
transposed inter, off-by-one in the start row) fails at least one of them."""
import itertools
import math

import numpy as np
import pytest

from oracle import dp_oracle as O


def test_hand_derived_known_answer():
    # L=2, S=2, V=5; every value exactly representable; derived by hand from csrc/dp_core.cpp:57-117
    mem = np.array([[1, 2], [2, 1]], np.int32)
    intra = np.array([[3, 1], [2, 5]], float)
    inter = np.zeros((2, 2, 2))
    inter[1] = [[0, 1], [4, 0]]           # row = source, column = target: a transposed read changes f[2]
    om = {0: 0, 1: 1, 2: 2, 3: 3, 5: 5}
    ot = {k: 0.5 for k in om}
    total, res, rem, f, mark = O.solve(mem, intra, inter, 5, om, ot, keep=True)
    inf = math.inf
    assert f.tolist() == [[inf, inf], [inf, inf], [inf, 9.0], [5.0, 6.0], [5.0, 6.0]]
    assert mark[0].tolist() == [[-1, -1], [0, -1], [0, 0], [0, 0], [0, 0]]
    assert mark[1].tolist() == [[-1, -1], [-1, 0], [0, 0], [0, 1], [0, 1]]   # [2]: all-inf candidates -> 0
    assert total == {0: 5.5, 1: 5.5, 2: 9.5, 3: inf, 5: inf}
    assert res == {0: [0, 0], 1: [0, 0], 2: [0, 1], 3: [-1, -1], 5: [-1, -1]}
    assert rem == {0: 1, 1: 0, 2: 0, 3: -1, 5: -1}


def test_duplicate_strategy_never_wins():
    # duplicate strategy 0 as a new last column/row: ties must go to the lower index
    mem = np.array([[1, 2, 1], [2, 1, 2]], np.int32)
    intra = np.array([[3, 1, 3], [2, 5, 2]], float)
    inter = np.zeros((2, 3, 3))
    inter[1] = [[0, 1, 0], [4, 0, 4], [0, 1, 0]]
    om = {0: 0, 1: 1, 2: 2}
    ot = {k: 0.5 for k in om}
    total, res, rem, f, mark = O.solve(mem, intra, inter, 5, om, ot, keep=True)
    assert total == {0: 5.5, 1: 5.5, 2: 9.5}
    assert all(2 not in r for r in res.values())
    assert not (mark == 2).any()


def _brute(mem, intra, inter, V, other_mem, other_time):
    """Enumerate all S^L assignments; path cost summed in the DP's association order
    ((((0 + inter0) + intra0) + inter1) + intra1)...; the minimum over feasible paths equals the DP
    value bit for bit because rounding is monotone.  Among equal-cost paths the DP's backtrack picks
    the lexicographically smallest when compared from the LAST layer backwards."""
    L, S = mem.shape
    out = {}
    for k in sorted(other_mem):
        budget = V - 1 - other_mem[k]
        best = None
        for path in itertools.product(range(S), repeat=L):
            m = sum(int(mem[l, path[l]]) for l in range(L))
            if m > budget:
                continue
            c = 0.0
            for l in range(L):
                prev = path[l - 1] if l > 0 else None
                # layer 0: every source gives (0 + inter[0][si][s]) + intra; the DP takes the min over si
                if l == 0:
                    c = min((0.0 + inter[0, si, path[0]]) + intra[0, path[0]] for si in range(S))
                else:
                    c = (c + inter[l, prev, path[l]]) + intra[l, path[l]]
            if best is None or c < best:
                best = c
        out[k] = math.inf if best is None or not best < math.inf else best + other_time[k]
    return out


@pytest.mark.parametrize("seed", range(12))
def test_brute_force_tiny(seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    L, S = int(rng.integers(1, 5)), int(rng.integers(1, 4))
    V = int(rng.integers(8, 40))
    mem = rng.integers(1, 10, size=(L, S)).astype(np.int32)
    if seed % 3 == 0:      # integer costs: exact ties
        intra = rng.integers(0, 4, size=(L, S)).astype(float)
        inter = rng.integers(0, 3, size=(L, S, S)).astype(float)
    else:
        intra = rng.uniform(0.1, 10, size=(L, S))
        inter = rng.uniform(0, 3, size=(L, S, S))
    om = {1: 0, 2: int(rng.integers(0, V // 2)), 3: int(rng.integers(0, V + 2))}
    ot = {k: float(rng.uniform(0, 2)) for k in om}
    total, res, rem = O.solve(mem, intra, inter, V, om, ot)
    want = _brute(mem, intra, inter, V, om, ot)
    for k in om:
        assert np.float64(total[k]).tobytes() == np.float64(want[k]).tobytes(), (k, total[k], want[k])
        if total[k] < math.inf:
            # the returned path is feasible and reproduces the cost and the remaining memory
            used = sum(int(mem[l, res[k][l]]) for l in range(L))
            assert used + rem[k] == V - 1 - om[k] and rem[k] >= 0
            c = min((0.0 + inter[0, si, res[k][0]]) + intra[0, res[k][0]] for si in range(S))
            for l in range(1, L):
                c = (c + inter[l, res[k][l - 1], res[k][l]]) + intra[l, res[k][l]]
            assert c + ot[k] == total[k]
        else:
            assert rem[k] == -1 and res[k] == [-1] * L


def test_single_strategy_closed_form():
    # S=1: total = left-to-right sum, remaining = V-1-other_mem-sum(mem)
    rng = np.random.Generator(np.random.PCG64(3))
    L, V = 9, 500
    mem = rng.integers(1, 40, size=(L, 1)).astype(np.int32)
    intra = rng.uniform(0, 7, size=(L, 1))
    inter = rng.uniform(0, 2, size=(L, 1, 1))
    om = {1: 0, 4: 100, 8: V - int(mem.sum())}        # the last one leaves remaining = -1 + ... infeasible by one
    ot = {1: 0.25, 4: 1.5, 8: 0.0}
    total, res, rem = O.solve(mem, intra, inter, V, om, ot)
    c = 0.0
    for l in range(L):
        c = (c + inter[l, 0, 0]) + intra[l, 0]
    assert total[1] == c + 0.25 and rem[1] == V - 1 - int(mem.sum())
    assert total[4] == c + 1.5 and rem[4] == V - 1 - 100 - int(mem.sum())
    assert total[8] == math.inf and rem[8] == -1 and res[8] == [-1] * L
    assert res[1] == [0] * L


def test_budget_exactly_enough_and_one_short():
    mem = np.full((4, 2), 5, np.int32)
    intra = np.ones((4, 2))
    inter = np.zeros((4, 2, 2))
    total, res, rem = O.solve(mem, intra, inter, 21, {1: 0, 2: 1}, {1: 0.0, 2: 0.0})
    assert total[1] == 4.0 and rem[1] == 0 and res[1] == [0, 0, 0, 0]
    assert total[2] == math.inf and rem[2] == -1


def test_infinite_intra_column_and_oversize_mem():
    rng = np.random.Generator(np.random.PCG64(11))
    L, S, V = 4, 5, 120
    mem = rng.integers(1, 20, size=(L, S)).astype(np.int32)
    intra = rng.uniform(1, 5, size=(L, S))
    inter = rng.uniform(0, 1, size=(L, S, S))
    intra[:, 2] = np.inf                 # never selectable, f = inf but mark = 0 (all-inf candidates)
    mem[1, 4] = V + 7                    # whole column infeasible at layer 1: mark = -1 everywhere
    total, res, rem, f, mark = O.solve(mem, intra, inter, V, {1: 0}, {1: 0.0}, keep=True)
    assert np.isinf(f[:, 2]).all()
    assert (mark[1, :, 4] == -1).all()
    for l in range(L):
        for s in range(S):
            assert ((mark[l, :, s] == -1) == (np.arange(V) < mem[l, s])).all()
    # layer 0 with f0 = 0: argmin over sources of inter[0][si][s]; the +inf column has all-inf candidates -> 0
    want0 = inter[0].argmin(axis=0)
    want0[2] = 0
    for s in range(S):
        col = mark[0, :, s]
        assert (col[col >= 0] == want0[s]).all()
    assert 2 not in res[1] and total[1] < math.inf


def test_invariants_medium():
    rng = np.random.Generator(np.random.PCG64(21))
    L, S, V = 6, 7, 400
    mem = rng.integers(1, 60, size=(L, S)).astype(np.int32)
    intra = rng.uniform(1, 9, size=(L, S))
    inter = rng.uniform(0, 2, size=(L, S, S))
    om = {1: 0, 2: 30, 4: 90, 8: 200}
    ot = {k: 0.0 for k in om}
    total, res, rem, f, mark = O.solve(mem, intra, inter, V, om, ot, keep=True)
    # f is non-increasing in v (more budget never costs more)
    fin = np.where(np.isinf(f), 1e300, f)
    assert (np.diff(fin, axis=0) <= 0).all()
    # more reserved memory never lowers the cost
    t = [total[k] for k in sorted(om)]
    assert all(a <= b for a, b in zip(t, t[1:]))
    # result independent of V beyond the sum of the largest memories
    big = V + int(mem.max(axis=1).sum())
    t2, r2, m2 = O.solve(mem, intra, inter, big, {1: 0}, {1: 0.0})
    t3, r3, m3 = O.solve(mem, intra, inter, big + 50, {1: 0}, {1: 0.0})
    assert t2 == t3 and r2 == r3 and m3[1] == m2[1] + 50
    # first layer: f = min_si inter[0][si][s] + intra[0][s] (f0 = 0)
    t1, r1, m1, f1, mk1 = O.solve(mem[:1], intra[:1], inter[:1], V, {1: 0}, {1: 0.0}, keep=True)
    want = (0.0 + inter[0]).min(axis=0) + intra[0]
    assert np.array_equal(f1[V - 1], want)
    assert np.array_equal(mk1[0, V - 1], inter[0].argmin(axis=0))


def test_association_order_matters_and_is_left_to_right():
    # (f + inter) + intra, not f + (inter + intra): pick numbers where the two differ
    f0 = 0.0
    inter = np.array([[[1e16]], [[1.0]]])
    intra = np.array([[1.0], [1.0]])
    mem = np.ones((2, 1), np.int32)
    total, res, rem = O.solve(mem, intra, inter, 10, {1: 0}, {1: 0.0})
    c = ((((f0 + 1e16) + 1.0) + 1.0) + 1.0)
    assert total[1] == c
    assert c != (1e16 + (1.0 + 1.0)) + 1.0 or c != 1e16 + 3.0


def test_coarse_branch_closed_form():
    rng = np.random.Generator(np.random.PCG64(8))
    L, S, V = 5, 6, 300
    mem = rng.integers(1, 40, size=(L, S)).astype(np.int32)
    intra = rng.uniform(1, 9, size=(L, S))
    inter = rng.uniform(0, 2, size=(L, S, S))
    tp = np.array([1, 1, 2, 2, 4, 4], np.int32)
    om = {1: 10, 2: 20, 4: 280}
    ot = {1: 0.5, 2: 0.25, 4: 0.0}
    total, res, rem = O.coarse(mem, intra, inter, V, tp, om, ot)
    for k in om:
        best, arg = math.inf, -1
        for i in range(S):
            if tp[i] != k:
                continue
            t = sum(intra[:, i]) + sum(inter[:, i, i]) + ot[k]      # dynamic_programming.py:70
            m = sum(int(x) for x in mem[:, i]) + om[k]
            if V - 1 - m >= 0 and best > t:
                best, arg = t, i
        assert total[k] == best
        if arg >= 0:
            assert list(res[k]) == [arg] * L and rem[k] == V - 1 - (int(mem[:, arg].sum()) + om[k])
        else:
            assert rem[k] == -1


@pytest.mark.parametrize("name", ["flush_coarse", "flush_coarse_tight"])
def test_coarse_branch_against_the_reference_scenarios(name, monkeypatch):
    """What pins ``dp_oracle_coarse``: the two coarse-mode scenarios whose return tuples were written from
    the reference's own ``DpOnModel`` (tests/golden/dp_on_model_golden.json).  Every coarse instance of
    such a run is also handed to the C function, which must give what the host class gives -- and the
    run as a whole must give the reference's recorded tuples.  (Coarse mode never reaches the plugin:
    no device is needed.)"""
    import json
    import os

    import dp_on_model_stubs as stubs
    from galvatron_dp.dynamic_programming import DPAlg, DpOnModel

    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "golden", "dp_on_model_golden.json")) as fh:
        want = json.load(fh)[name]
    seen = []
    plain = DPAlg._fit_coarse

    def checked(self):
        total, res, rem = plain(self)
        wt, wr, wm = O.coarse(self.v_data, self.intra_cost, np.asarray(self.inter_cost), self.max_mem,
                              [s[1] for s in self.strategy_set], self.other_mem_cost, self.other_time_cost)
        for k in self.other_mem_cost:
            assert np.float64(total[k]).tobytes() == np.float64(wt[k]).tobytes(), (k, total[k], wt[k])
            assert int(rem[k]) == int(wm[k]) and [int(x) for x in res[k]] == [int(x) for x in wr[k]]
        seen.append(len(self.other_mem_cost))
        return total, res, rem

    monkeypatch.setattr(DPAlg, "_fit_coarse", checked)
    cfg = stubs.scenario(name)
    dpm = stubs.build(DpOnModel, cfg, other_timecost_model=stubs.StubOther, pipeline_costmodel=stubs.stub_pipeline_costmodel)
    assert stubs.run(dpm, cfg) == want
    assert len(seen) >= 3, "the scenario should have gone through the coarse branch for every stage"


def test_the_reference_walk_can_leave_the_table_with_memory_costs_of_zero():
    """A cell whose memory cost is 0 takes candidates from its own layer (the update is in place), but the
    walk back follows its argmin as if it pointed into the layer before; under a budget of a few bins it then
    arrives at a negative row, with which the reference indexes its argmin table (csrc/dp_core.cpp:105-113):
    undefined behaviour.  The restatement says which keys those are, and agrees with the reference's build on
    all the others."""
    from galvatron_dp import workloads as W
    flagged = 0
    for seed, (L, S, V) in enumerate([(8, 17, 1), (12, 31, 65), (9, 8, 5), (6, 40, 64), (13, 5, 3), (10, 22, 7)]):
        inst = W.zero_memory_tiny_budget(seed, L, S, V)
        undefined = set()
        total, res, rem = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time,
                                  undefined=undefined)
        flagged += len(undefined)
        for k in undefined:
            assert total[k] < math.inf            # the cost itself is what the in-place update computed
        if O.ref_available():
            rt, rr, rm = O.ref_solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time)
            for k in total:
                assert np.float64(total[k]).tobytes() == np.float64(rt[k]).tobytes()
                if k not in undefined:
                    assert rem[k] == rm[k] and (rm[k] == -1 or res[k] == rr[k]), (seed, k)
    assert flagged >= 3, "the cases should include keys whose walk leaves the table"
