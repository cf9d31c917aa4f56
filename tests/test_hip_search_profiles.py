"""GPU test of whole searches that start from the profilers' files: the two cases of the reference's
own end-to-end test (tests/search_engine/test_parallelsim_optimization.py:9-128 of the reference),
with its profile data, through SearchEngine and the HIP dynamic program.

Checked against (1) what that test asserts -- the predicted throughput to 1e-6 and the fields of the
written configuration, e.g. "the first 8 of 28 layers checkpointed" -- and (2) what the reference's
engine produced on this image (tests/golden/search_profile_golden.json): throughput bit for bit, the
text of the result file, and the throughput, pipeline degree and vocabulary tp of every task."""
import json
import os

import pytest

import profile_cases as P
import sweep_cases as S
from galvatron_dp.search import SearchEngine

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def want():
    with open(os.path.join(HERE, "golden", "search_profile_golden.json")) as fh:
        return json.load(fh)


@pytest.mark.parametrize("name", list(P.E2E_CASES))
def test_whole_search_from_profile_files(want, tmp_path, name):
    case, known, ref = P.E2E_CASES[name], P.E2E_KNOWN[name], want["e2e"][name]
    engine = P.build(SearchEngine, P.profiles(), str(tmp_path), case["modes"], seqlen_list=case["seqlen_list"],
                     **case["args"])
    throughput = engine.parallelism_optimization()
    # (1) the reference's own assertions
    assert abs(throughput - known["throughput"]) < 1e-6
    output_dir = os.path.join(str(tmp_path), "output")
    files = [f for f in os.listdir(output_dir) if f.endswith(".json")]
    assert len(files) == 1 and files[0].startswith("galvatron_config_")
    with open(os.path.join(output_dir, files[0])) as fh:
        config = json.load(fh)
    for field, value in known["config"].items():
        assert config[field] == value, field
    # (2) the reference's engine on this image
    got = S.summarize(engine, throughput, output_dir)
    assert got["throughput"] == ref["throughput"]
    assert got["files"] == ref["files"]
    assert got["table"] == ref["table"]
