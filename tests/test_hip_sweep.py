"""GPU test of the sweep driver: the DP instances of ALL tasks of a sweep solved in one device
batch, against what the reference's engine (its own DpOnModel, cost models and compiled dp_core,
task by task) produced: best throughput, the text of the result file, and the throughput, pipeline
degree and vocabulary tp of every (task, sp_search)."""
import json
import os

import pytest

import sweep_cases as S
from galvatron_dp import cost_models
from galvatron_dp.search import SearchEngine

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def want():
    with open(os.path.join(HERE, "golden", "sweep_golden.json")) as fh:
        return json.load(fh)


@pytest.mark.parametrize("name", list(S.SWEEPS))
def test_sweep_matches_reference(want, name):
    got = S.run(SearchEngine, cost_models, name)
    ref = want["sweeps"][name]
    assert got["throughput"] == ref["throughput"]
    assert got["files"] == ref["files"]
    assert got["table"] == ref["table"]


def test_task_by_task_schedule_gives_the_same(want, tmp_path):
    engine = S.build(SearchEngine, cost_models, "two_types_tp", str(tmp_path))
    t = engine.parallelism_optimization(one_batch=False)
    assert S.summarize(engine, t, str(tmp_path))["table"] == want["sweeps"]["two_types_tp"]["table"]
    assert engine.solved_instances > 0 and engine.optimal["bsz"] == 64


def test_one_task_on_its_own_gives_its_entry_of_the_sweep(want, tmp_path):
    """SearchEngine.dynamic_programming -- one (task, sp_search), as the reference's method of that name
    solves it (search_engine.py:601-638) -- against the same task's entry in the reference's sweep."""
    engine = S.build(SearchEngine, cost_models, "bsz_range", str(tmp_path))
    engine.set_searching_bsz()
    ref = want["sweeps"]["bsz_range"]["table"]
    seen = 0
    for task in engine.tasks():
        bsz, chunk, min_tp, max_tp, vsp, embed_sdp = task
        for sp_search in engine._spaces()[4]:
            key = '%d/%d/%d/%d/%d/%d/%d' % (bsz, chunk, min_tp, max_tp, vsp, embed_sdp, sp_search)
            picked = engine._task_strategies(bsz, chunk, min_tp, max_tp, sp_search)
            if key not in ref or picked is None:
                continue
            cand, mbsz, stage = picked
            r = engine.dynamic_programming(cand, bsz, chunk, mbsz, stage, min_tp, max_tp, vsp, embed_sdp, sp_search)
            assert [S.C.hexf(r['throughput']), int(r['min_pp_deg']), S.C.jsonable(r['vtp'])] == ref[key], key
            assert set(r) == {'min_cost', 'min_res_list', 'min_pp_deg', 'mem_remain', 'mem_cost', 'throughput', 'vtp'}
            seen += 1
    assert seen == len(ref)
