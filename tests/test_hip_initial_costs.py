"""GPU: the contents of ``_f`` on entry are the initial costs, as in the reference, which relaxes in
place from whatever the caller's array holds (csrc/dp_core.cpp:46-47,67; DPAlg hands in zeros,
dynamic_programming.py:16).  Through the plugin signature and the C ABI, in every launch scheme, against
the C oracle and the vectors written from the reference's compiled dp_core (``initf_*``)."""
import numpy as np
import pytest

import galvatron_dp_core as shim
import helpers as H
from galvatron_dp import _lib, workloads as W
from oracle import dp_oracle as O

pytestmark = pytest.mark.gpu


def _problem(inst, **kw):
    keys = sorted(inst.other_mem)
    return _lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                        [inst.other_time[k] for k in keys], inter_index=inst.inter_index, f0=inst.f0, **kw)


def _results(prob, inst):
    keys = sorted(inst.other_mem)
    return ({k: prob.total[i] for i, k in enumerate(keys)},
            {k: [int(x) if prob.remaining[i] != -1 else -1 for x in prob.res[i]] for i, k in enumerate(keys)},
            {k: int(prob.remaining[i]) for i, k in enumerate(keys)})


def _case(seed, L, S, V, **kw):
    rng = np.random.Generator(np.random.PCG64(seed))
    inst = W.random_instance(rng, L, S, V, mem_hi=max(2, V // (L + 1)), integer_costs=bool(seed % 2), n_keys=4, **kw)
    return W.with_initial_costs(inst, rng, integer=bool(seed % 2), inf_frac=0.05 * (seed % 3 == 0))


@pytest.mark.parametrize("seed", range(6))
def test_plugin_call_with_random_initial_costs_equals_the_oracle(seed):
    inst = _case(600 + seed, L=3 + seed, S=[5, 22, 40, 44, 64, 88][seed], V=700 + 411 * seed)
    want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0, keep=True)
    if seed % 2 == 0:     # (integer initial costs can leave the minima at what zeros give)
        zero = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time)
        assert zero[0] != want[0], "the initial costs should matter in this case"
    got = H.hip_solve(inst)                       # as a caller makes the call: nothing exported
    H.assert_same_results(got, want[:3], f"seed {seed}")
    total, res, rem, f, mark = H.hip_solve(inst, export=True)
    H.assert_same_results((total, res, rem), want[:3], f"seed {seed}, exported")
    assert f.tobytes() == want[3].tobytes() and np.array_equal(mark, want[4])


@pytest.mark.parametrize("kw", [dict(launch="fused"), dict(launch="per_layer"), dict(launch="per_layer", keep_marks=True),
                                dict(launch="fused", keep_marks=True), dict(compute_all=True), dict()])
def test_every_launch_scheme_starts_from_the_initial_costs(kw):
    inst = _case(611, L=9, S=44, V=6000, inf_frac=0.1)
    want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0)
    prob = _problem(inst, **kw)
    with _lib.Plan([prob]) as plan:
        plan.set_option(_lib.GDP_OPT_POISON, 1)
        for run in range(3):          # a plan with two cost buffers writes over buffer 0 in every run
            plan.run()
            plan.fetch()
            H.assert_same_results(_results(prob, inst), want, f"{kw}, run {run}")


def test_memory_costs_of_zero_read_the_initial_costs_in_place():
    inst = _case(620, L=5, S=22, V=900, mem_lo=0)
    assert (inst.mem == 0).any()
    want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0, keep=True)
    total, res, rem, f, mark = H.hip_solve(inst, export=True)
    H.assert_same_results((total, res, rem), want[:3], "zero memory costs")
    assert f.tobytes() == want[3].tobytes() and np.array_equal(mark, want[4])
    H.assert_same_results(H.hip_solve(inst), want[:3], "zero memory costs, nothing exported")


def test_batch_mixes_instances_with_and_without_initial_costs():
    insts = [_case(630 + i, L=4 + i % 3, S=[22, 44][i % 2], V=1500 + 300 * i) for i in range(6)]
    for i in (1, 4):
        insts[i].f0 = None
    insts[2].f0 = np.zeros_like(insts[2].f0)             # zeros are what every caller of the reference passes
    probs = [_problem(i) for i in insts]
    _lib.solve_batch(probs)
    for n, (inst, prob) in enumerate(zip(insts, probs)):
        want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0)
        H.assert_same_results(_results(prob, inst), want, f"instance {n}")


def test_batch_entry_of_the_plugin_passes_the_initial_costs():
    insts = [_case(640 + i, L=5, S=22, V=1200) for i in range(3)]
    calls = []
    for inst in insts:
        res = {k: np.full(inst.L, -1, dtype=np.int32) for k in inst.other_mem}
        calls.append((inst.L, inst.V, inst.S, inst.mem, None, inst.f0.copy(), inst.inter, inst.intra, inst.other_mem,
                      inst.other_time, res))
    for inst, call, (total, rem) in zip(insts, calls, shim.dynamic_programming_core_batch(calls)):
        want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0)
        H.assert_same_results((total, {k: [int(x) for x in v] for k, v in call[10].items()}, rem), want, "batch entry")


def test_static_entry_point_starts_from_the_initial_costs():
    for seed, (L, S, V) in enumerate([(6, 44, 5000), (4, 22, 1200)]):
        inst = _case(650 + seed, L=L, S=S, V=V)
        want = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, f0=inst.f0)
        prob = _problem(inst)
        _lib.solve_static(prob)
        H.assert_same_results(_results(prob, inst), want, f"static, call {seed}")


def test_rejected_initial_costs_raise_before_any_device_work():
    inst = _case(660, L=3, S=5, V=200)
    for bad in (np.nan, -np.inf, -0.0):
        f = inst.f0.copy()
        f[17, 3] = bad
        res = {k: np.full(inst.L, -1, dtype=np.int32) for k in inst.other_mem}
        with pytest.raises(ValueError):
            shim.dynamic_programming_core(inst.L, inst.V, inst.S, inst.mem, None, f, inst.inter, inst.intra,
                                          inst.other_mem, inst.other_time, res)
        assert all((r == -1).all() for r in res.values())
