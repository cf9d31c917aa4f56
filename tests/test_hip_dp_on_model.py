"""GPU test of the host-side counterpart of the reference's DPAlg / DpOnModel: same constructor
arguments, same return tuples, compared with what the REFERENCE's classes returned for the same
stub cost models (tests/golden/dp_on_model_golden.json, written by
tests/golden/make_dp_on_model_golden.py from the reference's code and its compiled dp_core)."""
import json
import os

import numpy as np
import pytest

import dp_on_model_stubs as stubs
import helpers as H

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def want():
    with open(os.path.join(HERE, "golden", "dp_on_model_golden.json")) as fh:
        return json.load(fh)


@pytest.mark.parametrize("name", stubs.SCENARIOS)
def test_dp_on_model_matches_reference(want, name):
    from galvatron_dp.dynamic_programming import DpOnModel
    cfg = stubs.scenario(name)
    dpm = stubs.build(DpOnModel, cfg, other_timecost_model=stubs.StubOther,
                      pipeline_costmodel=stubs.stub_pipeline_costmodel)
    got = stubs.run(dpm, cfg)
    assert got == want[name]


@pytest.mark.parametrize("name", stubs.REAL_SCENARIOS)
def test_cost_models_dp_and_pipeline_model_together_match_reference(want, name):
    """Producer -> DP -> pipeline model: this repository's cost models, DpOnModel and HIP core against
    the reference's cost models, DpOnModel and compiled dp_core on the same synthetic profile."""
    from galvatron_dp import cost_models
    from galvatron_dp.dynamic_programming import DpOnModel
    cfg = stubs.real_scenario(name)
    dpm = stubs.build_real(DpOnModel, cost_models, cost_models, cfg)
    got = stubs.run(dpm, cfg)
    assert got == want[name]


def test_dpalg_fit_matches_plugin_semantics(golden):
    from galvatron_dp.dynamic_programming import DPAlg
    rec = golden["galvatron_like"]
    inst = H.build_case(rec)
    dp = DPAlg(inst.V - 1, inst.other_mem, inst.other_time, inst.L, inst.S, None, True)
    dp.set_v_and_cost(inst.mem, inst.intra, np.asarray(inst.inter))
    total, res, rem = dp.fit()
    H.assert_same_results((total, res, rem), H.golden_results(rec), "DPAlg.fit")
    assert isinstance(res[1], list)
    many = DPAlg.fit_many([dp, dp])
    for out in many:
        H.assert_same_results(out, H.golden_results(rec), "DPAlg.fit_many")


def test_dpalg_coarse_mode_needs_no_device():
    from galvatron_dp.dynamic_programming import DPAlg
    from oracle import dp_oracle as O
    rng = np.random.Generator(np.random.PCG64(12))
    L, S, V = 6, 8, 400
    mem = rng.integers(1, 50, size=(L, S)).astype(np.int32)
    intra = rng.uniform(1, 9, size=(L, S))
    inter = rng.uniform(0, 2, size=(L, S, S))
    strategy_set = [[1, [1, 2, 4, 8][i % 4], 8, {}] for i in range(S)]
    om, ot = {1: 10, 2: 20, 4: 300, 8: 0}, {1: 0.5, 2: 0.25, 4: 0.0, 8: 1.0}
    dp = DPAlg(V - 1, om, ot, L, S, strategy_set, False)
    dp.set_v_and_cost(mem, intra, inter)
    total, res, rem = dp.fit()
    wt, wr, wm = O.coarse(mem, intra, inter, V, [s[1] for s in strategy_set], om, ot)
    for k in om:
        assert total[k] == wt[k] and rem[k] == wm[k] and list(res[k]) == list(wr[k])
