"""Host logic of the sweep driver (galvatron_dp/search.py) against what the reference's
GalvatronSearchEngine produced (tests/golden/sweep_golden.json, written by
tests/golden/make_sweep_golden.py): strategy generation and batch-size ranges here (no device
needed), whole sweeps in test_hip_sweep.py."""
import json
import os

import pytest

import sweep_cases as S
from galvatron_dp.search import SearchEngine, array2str, strategy2config

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def want():
    with open(os.path.join(HERE, "golden", "sweep_golden.json")) as fh:
        return json.load(fh)


def test_generated_strategies_match_the_reference(want):
    assert len(want["strategies"]) == len(S.STRATEGY_CASES) >= 200
    seen = set()
    for rec in want["strategies"]:
        e = SearchEngine(S.search_args(**rec["case"]))
        try:
            got = e.generate_strategies()
        except AssertionError:
            got = "AssertionError"
        assert got == rec["want"], rec["case"]
        assert [e.args.disable_sdp, e.args.disable_pp, e.args.disable_tp, e.args.disable_ckpt] == rec["flags"]
        seen.add(len(got) if isinstance(got, list) else got)
    assert max(x for x in seen if isinstance(x, int)) > 50 and 1 in seen


def test_batch_size_ranges_match_the_reference(want):
    for rec in want["bsz"]:
        e = SearchEngine(S.search_args(**rec["case"]))
        try:
            e.set_searching_bsz()
            got = [e.min_bsz, e.max_bsz, e.bsz_scale, e.BSZs]
        except IndexError:
            got = "IndexError"
        assert got == rec["want"], rec["case"]


def test_known_strategy_lists():
    # 8 GPUs, everything allowed, tensor parallel only: pp x tp grid with the dp remainder; both
    # layouts of the tp group where tp and dp are both above 1; ZeRO-3 twin where dp > 1; then the
    # checkpointed twins of all of them
    e = SearchEngine(S.search_args(sp_space='tp'))
    got = e.generate_strategies()
    plain = [s for s in got if 'cpt' not in s[-1]]
    assert len(got) == 2 * len(plain)
    assert [1, 1, 8, {'fsdp': 0}] in plain and [1, 1, 8, {'fsdp': 1}] in plain and [8, 1, 1, {}] in plain
    assert [1, 2, 4, {'tp': 0, 'fsdp': 1, 'sp': 0}] in plain and [1, 8, 1, {'sp': 0}] in plain
    assert all(s[0] * s[1] * s[2] == 8 for s in got)
    one = SearchEngine(S.search_args(search_space='3d', num_gpus_per_node=16, sp_space='sp')).generate_strategies()
    assert one == [[2, 2, 4, {'tp': 1, 'fsdp': 0, 'sp': 1}]]


def test_result_file_fields():
    layers = [[2, 2, 2, {'tp': 1, 'fsdp': 0, 'sp': 0}], [2, 4, 1, {'sp': 1, 'cpt': 1}], [2, 1, 4, {'fsdp': 1}]]
    assert strategy2config(layers) == {"pp_deg": 2, "tp_sizes_enc": "2,4,1", "tp_consecutive_flags": "1,1,1",
                                       "dp_types_enc": "0,0,1", "use_sp": "0,1,0"}
    assert strategy2config([]) == {} and array2str([3, 1]) == "3,1"
    e = SearchEngine(S.search_args(settle_bsz=32, disable_ckpt=1, disable_tp_consec=1, output_config_path="/x"))
    e.set_model("m", [dict(layer_num=3, hidden_size=8, seq_len=4)])
    assert e.result_path() == "/x/galvatron_config_m_1nodes_8gpus_per_node_8GB_bf16_bsz32_[ckpt_tpconsec_off].json"
    re = dict(min_pp_deg=2, min_res_list=[layers[:2], layers[2:]], vtp=2, vsp=0, embed_sdp=1)
    cfg = e.result_config(re, 32, 4, {2: [2, 1]})
    assert cfg["checkpoint"] == "0,1,0" and cfg["pp_division"] == "2,1" and cfg["global_bsz"] == 32
    assert cfg["chunks"] == 4 and cfg["vtp"] == 2 and cfg["embed_sdp"] == 1 and cfg["pipeline_type"] == "pipedream_flush"
    assert e.result_config(dict(min_pp_deg=-1, min_res_list=None), 32, 4, {}) is None


def test_a_failure_while_tasks_are_prepared_leaves_the_engine_as_it_was(tmp_path):
    """``parallelism_optimization`` works on a copy of the strategy list and hands parts of the batch to a
    worker thread: whatever goes wrong while the tasks are prepared, the engine holds its own list again
    afterwards and no worker is left behind (no device is needed: the failure comes before the first part)."""
    import threading

    from galvatron_dp import cost_models
    engine = S.build(SearchEngine, cost_models, "llama_like", str(tmp_path))
    mine = engine.strategies
    before = threading.active_count()

    def boom(*a, **k):
        raise RuntimeError("cost model failed")

    engine._task_strategies = boom
    with pytest.raises(RuntimeError, match="cost model failed"):
        engine.parallelism_optimization()
    assert engine.strategies is mine
    assert threading.active_count() == before
