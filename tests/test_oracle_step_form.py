"""The step form of the DP (oracle/dp_steps.py: one evaluation per step of the cost columns instead of one
per budget bin) against the vectors written from the reference's compiled dp_core and against the dense C
restatement.  It is an independent way to the same bits: a mistake in the dense restatement that the step
form does not share (or the other way round) shows up here."""
import numpy as np
import pytest

import helpers as H
from galvatron_dp import workloads as W
from oracle import dp_oracle as O
from oracle import dp_steps as St

SMALL = ([f"ties_{i}" for i in range(10)] + [f"rand_{i}" for i in range(10)] + [f"infeasible_{i}" for i in range(10)] +
         [f"initf_{i}" for i in range(6)])
LARGER = [f"cfg3_smallV_{i}" for i in range(8)] + ["galvatron_like", "cfg0", "cfg0_other_time", "cfg2_small", "cfg4_small",
                                                   "initf_galvatron_like"]


@pytest.mark.parametrize("name", SMALL)
def test_step_form_gives_the_reference_arrays(golden, name):
    rec = golden[name]
    inst = H.build_case(rec)
    total, res, rem, _ = St.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0)
    H.assert_same_results((total, res, rem), H.golden_results(rec), name)
    layers, _ = St.relax(inst.mem, inst.intra, inst.inter, inst.V, f0=inst.f0)
    f, mark = St.dense(layers, inst.V)
    assert H.sha(f) == rec["f_sha256"] and H.sha(mark) == rec["mark_sha256"]


@pytest.mark.parametrize("name", LARGER)
def test_step_form_gives_the_reference_results(golden, name):
    rec = golden[name]
    inst = H.build_case(rec)
    total, res, rem, stats = St.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0)
    H.assert_same_results((total, res, rem), H.golden_results(rec), name)
    dense = inst.L * inst.V * inst.S * inst.S
    assert sum(s["relaxations"] for s in stats) <= dense


@pytest.mark.parametrize("seed", range(8))
def test_step_form_against_the_dense_restatement(seed):
    rng = np.random.Generator(np.random.PCG64(3100 + seed))
    L, S, V = int(rng.integers(1, 9)), int(rng.integers(1, 50)), int(rng.integers(30, 1500))
    inst = W.random_instance(rng, L, S, V, integer_costs=bool(seed % 2), mem_hi=max(1, V // (L + 1)),
                             inf_frac=0.15 * (seed % 3 == 0), over_frac=0.1 * (seed % 4 == 0), n_keys=4)
    want = O.solve(inst.mem, inst.intra, inst.inter, V, inst.other_mem, inst.other_time, keep=True)
    total, res, rem, _ = St.solve(inst.mem, inst.intra, inst.inter, V, inst.other_mem, inst.other_time)
    H.assert_same_results((total, res, rem), want[:3], f"seed {seed}")
    layers, _ = St.relax(inst.mem, inst.intra, inst.inter, V)
    f, mark = St.dense(layers, V)
    assert f.tobytes() == want[3].tobytes() and np.array_equal(mark, want[4])
