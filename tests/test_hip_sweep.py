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
