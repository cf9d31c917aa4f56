"""GPU tests of the flow launch: all layers of a small plan in one launch whose tasks wait on the cost
cells themselves (NaN = not written yet), through the C ABI.  Same bits as the oracle and as the
reference-built goldens are required, as for every other launch scheme."""
import os

import numpy as np
import pytest

import helpers as H
from galvatron_dp import _lib, workloads as W

pytestmark = pytest.mark.gpu

_PRESETS = ("GALVATRON_DP_KEEP_MARKS", "GALVATRON_DP_TILE_TS", "GALVATRON_DP_TILE_R", "GALVATRON_DP_FUSED",
            "GALVATRON_DP_LATENCY_VARIANT", "GALVATRON_DP_FLOW")


def _problem(inst, **kw):
    keys = sorted(inst.other_mem)
    return _lib.Problem(inst.mem, inst.intra, inst.inter_tables, inst.V, [inst.other_mem[k] for k in keys],
                        [inst.other_time[k] for k in keys], inter_index=inst.inter_index, **kw)


def _results(prob, keys):
    return ({k: prob.total[i] for i, k in enumerate(keys)}, {k: [int(x) for x in prob.res[i]] for i, k in enumerate(keys)},
            {k: int(prob.remaining[i]) for i, k in enumerate(keys)})


def _check_against_golden(prob, rec, name):
    keys = rec["keys"]
    got = ({k: prob.total[i] for i, k in enumerate(keys)},
           {k: [int(x) if prob.remaining[i] != -1 else -1 for x in prob.res[i]] for i, k in enumerate(keys)},
           {k: int(prob.remaining[i]) for i, k in enumerate(keys)})
    H.assert_same_results(got, H.golden_results(rec), name)


@pytest.mark.parametrize("S", [1, 7, 8, 9, 12, 13, 22, 24, 25, 29, 33, 40, 44, 48, 49, 63, 65, 96, 97, 128])
def test_flow_launch_matches_the_oracle(S, monkeypatch):
    """Small instances run as one flow launch by default; sources on 1, 2 and 4 waves per task where S
    allows (S on both sides of every sources-per-wave step); f of the last layer compared too, and the
    run repeated on the same plan (the cells are reset behind every run)."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    from oracle import dp_oracle as O
    rng = np.random.Generator(np.random.PCG64([11, S]))
    inst = W.random_instance(rng, 6, S, 900 + S, mem_hi=150, inf_frac=0.1, per_layer_inter=bool(S % 2), n_keys=3)
    wt, wr, wm, wf, _ = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, keep=True)
    keys = sorted(inst.other_mem)
    seen = []
    for preset in (None, "1", "2", "4"):
        if preset is not None:
            monkeypatch.setenv("GALVATRON_DP_LATENCY_VARIANT", preset)
        for export_f in (False, True):
            prob = _problem(inst, export_f=export_f)
            with _lib.Plan([prob]) as plan:
                for rep in range(3):
                    if rep == 2:
                        plan.set_option(_lib.GDP_OPT_POISON, 1)
                    t = plan.run(1)
                    plan.fetch()
                    assert t.flow == 1 and t.fused == 0 and t.relax_launches == 1, (t.flow, t.fused, t.relax_launches)
                    H.assert_same_results(_results(prob, keys), (wt, wr, wm), f"S={S} preset={preset} run {rep}")
                    if export_f:
                        assert prob.f_out.tobytes() == wf.tobytes()
            seen.append(t.latency_variant)
    for preset, k in zip(("1", "2", "4"), seen[2::2]):
        if S <= 32 * int(preset):
            assert k == int(preset), (preset, seen)


def test_flow_launch_on_the_goldens(golden):
    """cfg0 and the Galvatron-like instance at full size, with and without row skipping."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    for name in ("cfg0", "galvatron_like", "ties_6", "infeasible_9", "rand_5"):
        rec = golden[name]
        inst = H.build_case(rec)
        for compute_all in (False, True):
            prob = _problem(inst, compute_all=compute_all)
            with _lib.Plan([prob]) as plan:
                t = plan.run(1)
                plan.fetch()
                if name == "cfg0" or (name == "galvatron_like" and not compute_all):
                    assert t.flow == 1
                _check_against_golden(prob, rec, f"{name} compute_all={compute_all}")
                t = plan.run(1)
                plan.fetch()
                _check_against_golden(prob, rec, f"{name} compute_all={compute_all} again")
        prob = _problem(inst)
        _lib.solve_batch([prob])
        _check_against_golden(prob, rec, f"{name} solve")


def test_flow_launch_batch_of_small_instances(golden, monkeypatch):
    """Several small instances of different depth and S in one plan: one flow launch per group of equal S."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    monkeypatch.setenv("GALVATRON_DP_FLOW", "1")
    names = ["ties_1", "rand_2", "cfg3_smallV_0", "infeasible_3", "rand_5", "cfg3_smallV_3", "ties_6", "rand_7"]
    probs = [_problem(H.build_case(golden[n])) for n in names]
    with _lib.Plan(probs) as plan:
        for rep in range(2):
            t = plan.run(1)
            plan.fetch()
            for n, prob in zip(names, probs):
                _check_against_golden(prob, golden[n], f"{n} run {rep}")


def test_flow_switched_off_and_on_again(golden):
    """A plan laid out for the flow launch runs per layer when told to, and flows again afterwards (the
    cells are reset first); a plan laid out for something else refuses the option."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    rec = golden["galvatron_like"]
    inst = H.build_case(rec)
    prob = _problem(inst)
    with _lib.Plan([prob]) as plan:
        for flow in (1, 0, 1, 1, 0, 0, 1):
            plan.set_option(_lib.GDP_OPT_FLOW, flow)
            t = plan.run(1)
            plan.fetch()
            assert t.flow == flow and t.fused == 0
            assert t.relax_launches == (1 if flow else inst.L)
            _check_against_golden(prob, rec, f"flow={flow}")
    prob = _problem(inst, launch="per_layer")
    with _lib.Plan([prob]) as plan:
        t = plan.run(1)
        assert t.flow == 0
        with pytest.raises(ValueError):
            plan.set_option(_lib.GDP_OPT_FLOW, 1)


def test_abandoned_flow_launch_falls_back_or_reports(golden):
    """A spin limit of 1 makes waiting wavefronts give up at once (forced from the host; every kernel
    still runs to completion).  With the fallback the plan switches to per-layer launches and returns
    the right answer; without it the run reports an error.  Either way the next plan works."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    rec = golden["cfg0"]
    inst = H.build_case(rec)
    prob = _problem(inst)
    with _lib.Plan([prob]) as plan:
        plan.set_option(_lib.GDP_OPT_SPIN_LIMIT, 1)
        t = plan.run(1)
        plan.fetch()
        _check_against_golden(prob, rec, "fallback")
        assert t.flow == 0 and t.relax_launches == inst.L       # it did give up: 24 layers do not fit on the device at once
        t = plan.run(1)
        plan.fetch()
        _check_against_golden(prob, rec, "after the fallback")
    prob2 = _problem(inst)
    with _lib.Plan([prob2]) as plan:
        plan.set_option(_lib.GDP_OPT_SPIN_LIMIT, 1)
        plan.set_option(_lib.GDP_OPT_NO_FALLBACK, 1)
        with pytest.raises(RuntimeError, match="bounded wait"):
            plan.run()
    prob3 = _problem(inst)
    _lib.solve_batch([prob3])
    _check_against_golden(prob3, rec, "after")


def test_a_flow_wait_that_cannot_end_costs_milliseconds(golden, monkeypatch):
    """The tasks of the first layer leave their stores out (forced from the host; every kernel still ends
    normally), so the second layer waits for cells that stay unwritten until the bound of the wait -- 5 ms for
    a plan of this size -- runs out; the solve is then repeated with one launch per layer, and after the
    back-off the plan flows again."""
    import time
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    rec = golden["cfg0"]
    inst = H.build_case(rec)
    monkeypatch.setenv("GALVATRON_DP_SHARED_BACKOFF_MS", "150")
    prob = _problem(inst)
    try:
        with _lib.Plan([prob]) as plan:
            assert plan.run(1).flow == 1
            plan.set_option(_lib.GDP_OPT_DEBUG_STALL, 1)
            t0 = time.perf_counter()
            t = plan.run(1)
            dt = time.perf_counter() - t0
            plan.fetch()
            _check_against_golden(prob, rec, "after the bounded wait ran out")
            assert t.flow == 0 and t.relax_launches == inst.L
            assert dt < 0.25, f"give-up and repeated solve took {dt * 1e3:.0f} ms"
            plan.set_option(_lib.GDP_OPT_DEBUG_STALL, 0)
            time.sleep(0.3)
            t = plan.run(1)
            plan.fetch()
            assert t.flow == 1, "the plan was not armed again after the back-off"
            _check_against_golden(prob, rec, "armed again")
    finally:
        _lib.debug_shared_device(False)


def test_flow_plans_from_several_threads(golden):
    """Threads that call the plugin side by side (as the reference's parallel search does): one flow
    launch runs at a time, a plan that finds the turn taken solves with one launch per layer beside
    it.  Every result equals the reference's, whichever way a call ran."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    import threading
    names = ["cfg0", "galvatron_like", "rand_5", "ties_6"]
    errors, flowed = [], []

    def work(tid):
        try:
            for it in range(12):
                name = names[(tid + it) % len(names)]
                rec = golden[name]
                prob = _problem(H.build_case(rec))
                if it % 2:
                    _lib.solve_batch([prob])
                else:
                    with _lib.Plan([prob]) as plan:
                        for _ in range(3):
                            flowed.append(plan.run(1).flow)
                            plan.fetch()
                            _check_against_golden(prob, rec, f"thread {tid} {name}")
                _check_against_golden(prob, rec, f"thread {tid} {name}")
        except Exception as e:       # noqa: BLE001
            errors.append((tid, repr(e)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(6)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    assert any(flowed)


def test_flow_alternating_problems_in_the_same_memory():
    """Two different problems of one shape solved in turn: the library hands the second the device
    memory the first has just left (same layout, same addresses), so a cost cell or cache line that
    survived from the other problem's run would show up as a wrong result."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    from oracle import dp_oracle as O
    rng = np.random.Generator(np.random.PCG64(77))
    L, S, V = 12, 22, 6000
    a = W.random_instance(rng, L, S, V, mem_hi=300, inf_frac=0.05, n_keys=3)
    # same memory costs (same bands, same layout), other times: every cell differs
    b = W.Instance("b", a.mem.copy(), a.intra * 1.7 + 0.25, a.inter * 0.6, a.V, dict(a.other_mem), dict(a.other_time),
                   None if a.inter_tables is None else a.inter_tables * 0.6, a.inter_index)
    want = {}
    for name, inst in (("a", a), ("b", b)):
        wt, wr, wm, _, _ = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, keep=True)
        want[name] = (wt, wr, wm)
    assert want["a"][0] != want["b"][0]
    keys = sorted(a.other_mem)
    for it in range(40):
        name, inst = (("a", a), ("b", b))[it % 2]
        prob = _problem(inst)
        if it % 8 < 6:
            _lib.solve_batch([prob])
        else:
            with _lib.Plan([prob]) as plan:
                for _ in range(2):
                    t = plan.run(1)
                    assert t.flow == 1
                    plan.fetch()
        H.assert_same_results(_results(prob, keys), want[name], f"iteration {it} problem {name}")


def test_launches_that_never_wait_on_a_device_that_seems_shared(golden):
    """After a waiting launch was given up with the default spin limit the library takes the device to
    be shared and chooses one launch per layer where the choice is its own; an explicit request still
    counts; the state ends by itself (here: is ended by the test aid)."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    rec = golden["cfg0"]
    inst = H.build_case(rec)
    big = golden["cfg2_small"]
    big_inst = H.build_case(big)
    try:
        _lib.debug_shared_device(True)
        for r, i in ((rec, inst), (big, big_inst)):
            prob = _problem(i)
            with _lib.Plan([prob]) as plan:
                t = plan.run(1)
                plan.fetch()
                assert t.flow == 0 and t.fused == 0 and t.relax_launches == i.L
                _check_against_golden(prob, r, "seems shared")
        prob = _problem(big_inst, launch="fused")
        with _lib.Plan([prob]) as plan:
            assert plan.run(1).fused == 1
            plan.fetch()
            _check_against_golden(prob, big, "explicit request")
    finally:
        _lib.debug_shared_device(False)
    prob = _problem(inst)
    with _lib.Plan([prob]) as plan:
        assert plan.run(1).flow == 1
        plan.fetch()
        _check_against_golden(prob, rec, "afterwards")


def test_flow_launch_on_the_fuzz_shapes_without_exports():
    """The shapes of the differential test (V from 1 to 4099, S around every tile and wave width), run as
    callers run them: nothing exported, so only the bands are computed (closed under reading) and rows
    below them are filled where something reads them.  Results against the oracle; memory costs small,
    large, beyond the budget; +inf costs; ties."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    from oracle import dp_oracle as O
    from test_hip_fuzz import SHAPES
    flowed = 0
    for n, (L, S, V) in enumerate(SHAPES):
        for variant in range(4):
            rng = np.random.Generator(np.random.PCG64([91, n, variant]))
            hi = [max(1, V // (L + 1)), max(1, V // 2), V + 3, 3][variant]
            inst = W.random_instance(rng, L, S, V, integer_costs=variant in (1, 3), mem_hi=hi,
                                     per_layer_inter=bool(variant % 2), inf_frac=0.2 if variant >= 2 else 0.0,
                                     over_frac=0.1 if variant == 3 else 0.0, n_keys=min(4, 1 + variant))
            wt, wr, wm, _, _ = O.solve(inst.mem, inst.intra, inst.inter, inst.V, inst.other_mem, inst.other_time, keep=True)
            keys = sorted(inst.other_mem)
            prob = _problem(inst)
            with _lib.Plan([prob]) as plan:
                for rep in range(2):
                    t = plan.run(1)
                    plan.fetch()
                    flowed += t.flow
                    H.assert_same_results(_results(prob, keys), (wt, wr, wm), f"shape {(L, S, V)} variant {variant} run {rep}")
    assert flowed > len(SHAPES)


def test_small_plans_on_both_sides_of_the_early_preparation():
    """Up to 16 instances with up to 224 layers in all get their cost buffers prepared by a kernel that is
    fed with its arguments and starts before the plan's tables are uploaded; one more instance or layer
    takes the ordinary way.  One-shot solves (gdp_solve_batch) on both sides of both limits, twice each
    (the second lands in the memory the first left behind), against the oracle."""
    if any(k in os.environ for k in _PRESETS):
        pytest.skip("the environment presets the layout")
    from oracle import dp_oracle as O
    rng = np.random.Generator(np.random.PCG64(5))

    def batch(shapes):
        insts = [W.random_instance(rng, L, S, V, mem_hi=max(2, V // (L + 2)), inf_frac=0.05, n_keys=2) for (L, S, V) in shapes]
        wants = [O.solve(i.mem, i.intra, i.inter, i.V, i.other_mem, i.other_time) for i in insts]
        for rep in range(2):
            probs = [_problem(i) for i in insts]
            _lib.solve_batch(probs)
            for n, (i, prob, want) in enumerate(zip(insts, probs, wants)):
                H.assert_same_results(_results(prob, sorted(i.other_mem)), want, f"{len(shapes)} instances, #{n}, run {rep}")

    batch([(224, 5, 700)])
    batch([(225, 5, 700)])
    batch([(14, 9, 400)] * 16)                      # 16 instances, 224 layers
    batch([(14, 9, 400)] * 15 + [(15, 9, 400)])     # 225 layers
    batch([(6, 12, 300)] * 17)
    batch([(3, 22, 900), (40, 8, 500), (1, 13, 200), (28, 40, 2000)])
