"""Reading the profilers' files into the cost-model argument records
(galvatron_dp/profile_configs.py, SearchEngine.initialize_search_engine) against

* the values the reference's own tests assert after loading the same files
  (tests/search_engine/test_get_configs.py:60-118, test_initialize.py:31-33 of the reference), and
* everything the reference's GalvatronSearchEngine held after ``initialize_search_engine`` on them
  (tests/golden/search_profile_golden.json, written by tests/golden/make_search_profile_golden.py),
  float for float.

No device needed; the whole searches from these files are in test_hip_search_profiles.py."""
import json
import os

import numpy as np
import pytest

import profile_cases as P
from galvatron_dp import profile_configs
from galvatron_dp.search import SearchEngine

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def want():
    with open(os.path.join(HERE, "golden", "search_profile_golden.json")) as fh:
        return json.load(fh)


@pytest.fixture(scope="module")
def data():
    return P.profiles()


@pytest.mark.parametrize("modes", P.LOADING_CASES, ids=lambda m: "-".join(map(str, m)))
def test_loaded_state_matches_the_reference(want, data, tmp_path, modes):
    engine = P.build(SearchEngine, data, str(tmp_path), modes)
    ref = next(r["want"] for r in want["loading"] if tuple(r["modes"]) == modes)
    got = P.loaded_state(engine)
    assert sorted(got) == sorted(ref)
    for key in ref:
        assert got[key] == ref[key], key


@pytest.mark.parametrize("modes", P.LOADING_CASES, ids=lambda m: "-".join(map(str, m)))
def test_values_the_reference_tests_assert(data, tmp_path, modes):
    time_mode, memory_mode, sp = modes
    engine = P.build(SearchEngine, data, str(tmp_path), modes)
    tc, mc = engine.time_config, engine.memory_config
    key, val = {"static": ("layertype_0_bsz8_seq4096", 11.219752883911134),
                "batch": ("layertype_0_bsz4_seq4096", 11.152996063232425),
                "sequence": ("layertype_0_bsz1_seq32768", 123.1998901367187)}[time_mode]
    assert abs(tc[key] - val) < 1e-6
    layer = "layertype_0_sp" if sp else "layertype_0"
    assert layer in mc
    if memory_mode == "sequence":
        assert 512 in mc[layer] and 2048 in mc[layer]
    assert 4096 in mc[layer]
    act8 = mc[layer][4096]["tp_activation_per_bsz_dict"][8]
    expect = (79.5704345703125 if memory_mode == "static" else 130.5587158203125) if sp else 191.6251220703125
    assert abs(act8 - expect) < 1e-6
    # hardware (test_get_configs.py:112-118)
    assert abs(engine.allreduce_bandwidth['2_0'] - 153.933) < 1e-3
    assert abs(engine.allreduce_bandwidth['4_1'] - 164.272) < 1e-3
    assert abs(engine.p2p_bandwidth[2] - 147.32) < 1e-3
    assert abs(engine.overlap_coe - 1.1534195950157762) < 1e-6
    assert abs(engine.sp_allreduce[8][8 * 1024 * 1024] - 0.1827 / 2) < 1e-4
    assert abs(engine.sp_allreduce[8][16 * 1024 * 1024] - 0.29410000000000003 / 2) < 1e-4
    assert abs(engine.sp_all2all[4][8 * 1024 * 1024] - 0.1255) < 1e-4
    # records (test_initialize.py:19-33)
    for name in ("model_args_list", "train_args_list", "parallel_args_list", "profile_model_args_list",
                 "profile_hardware_args_list"):
        assert len(getattr(engine, name)) == engine.num_layertype == 1
    assert engine.model_args_list[0].seq_length == 4096
    assert engine.train_args_list[0].mixed_precision is True
    assert engine.parallel_args_list[0].sequence_parallel == sp


@pytest.mark.parametrize("name", list(P.E2E_CASES))
def test_state_before_the_whole_searches(want, data, tmp_path, name):
    case = P.E2E_CASES[name]
    engine = P.build(SearchEngine, data, str(tmp_path), case["modes"], seqlen_list=case["seqlen_list"], **case["args"])
    assert P.loaded_state(engine) == want["e2e"][name]["state"]


def test_fits_are_what_the_mathematics_fixes():
    """Points that lie exactly on a line / parabola give that line / parabola back."""
    seqs = [1024 * k for k in range(1, 9)]
    tc = {"layertype_0_bsz1_seq%d" % s: 2e-7 * s * s + 3e-3 * s + 1.5 for s in seqs}
    tc.update({"layertype_other_bsz1_seq%d" % s: 5e-3 * s + 4.0 for s in seqs})
    layers, other = profile_configs.fit_layer_times(tc, "sequence", 1, [6000])
    assert layers[0] == pytest.approx(2e-7 * 6000 * 6000 + 3e-3 * 6000 + 1.5, rel=1e-9)
    assert other[0] == pytest.approx(5e-3 * 6000 + 4.0, rel=1e-9)
    tb = {"layertype_0_bsz%d_seq512" % b: (7.0 * b + 2.0) / b for b in range(1, 11)}
    tb.update({"layertype_other_bsz%d_seq512" % b: (3.0 * b + 1.0) / b for b in range(1, 11)})
    tb["layertype_0_bsz4_seq1024"] = 1e9                      # another sequence length: not part of the fit
    layers, other = profile_configs.fit_layer_times(tb, "batch", 1, [512])
    np.testing.assert_allclose(layers[0], [7.0, 2.0], rtol=1e-8)
    np.testing.assert_allclose(other[0], [3.0, 1.0], rtol=1e-8)
    with pytest.raises(AssertionError):
        profile_configs.fit_layer_times({k: v for k, v in list(tb.items())[:5]}, "batch", 1, [512])
    sp = {"allreduce_size_4_%dMB_time" % m: 2 * (0.01 * m + 0.05) for m in (1, 2, 4, 8, 16, 32, 64, 128)}
    sp.update({"all2all_size_4_%dMB_time" % m: 0.02 * m + 0.03 for m in (1, 2, 4, 8, 16, 32, 64, 128)})
    ar, a2a = profile_configs.remap_config(sp, "allreduce"), profile_configs.remap_config(sp, "all2all")
    np.testing.assert_allclose(ar[4]["popt"], [0.01, 0.05], rtol=1e-7)
    np.testing.assert_allclose(a2a[4]["popt"], [0.02, 0.03], rtol=1e-7)
    assert ar[4][8 * 1024 * 1024] == (2 * (0.01 * 8 + 0.05)) / 2 and a2a[4][8 * 1024 * 1024] == 0.02 * 8 + 0.03


def test_bandwidth_tables_and_names():
    env = {"allreduce_size_8_consec_1": 160.0, "allreduce_size_4_consec_0": 100.0, "allreduce_size_4_consec_1": 125.0,
           "allreduce_size_2_consec_0": 80.0, "allreduce_size_2_consec_1": 50.0}
    bw, coe = profile_configs.read_allreduce_bandwidth_config(env, gpu_num=8)
    assert bw == {'8': 160.0, '4_0': 100.0, '4_1': 125.0, '2_0': 80.0, '2_1': 50.0, '1': np.inf}
    assert coe == {'8': 1 / 160.0, '4_0': 0.01, '4_1': 0.008, '2_0': 0.0125, '2_1': 0.02, '1': 0}
    assert profile_configs.read_allreduce_bandwidth_config(env, gpu_num=1) == ({'1': np.inf}, {'1': 0})
    bw, coe = profile_configs.read_p2p_bandwidth_config({"pp_size_2": 40.0, "pp_size_4": 20.0, "note": 1})
    assert bw == {2: 40.0, 4: 20.0} and coe == {2: 0.025, 4: 0.05}
    assert profile_configs.num2str([4096], 'seq') == 'seq4096'
    assert profile_configs.num2str([4096, 512], 'seq') == 'seq[4096,512]'
    assert profile_configs.int_keys({"8": {"x": {"12": 1}}, "a1": 2}) == {8: {"x": {12: 1}}, "a1": 2}
    with pytest.raises(FileNotFoundError):
        profile_configs.read_json_config("/nonexistent/file.json")


def test_default_locations(tmp_path):
    """Without path arguments the profiles are looked for under <model dir>/configs and the hardware
    files under <model dir>/../../profile_hardware/hardware_configs (search_engine.py:59-84,250-284)."""
    e = SearchEngine(P.reference_test_args(num_nodes=2, num_gpus_per_node=4, mixed_precision="fp16"))
    e.set_search_engine_info("/m/llama", P.LAYER_CONFIGS, "llama-7b")
    assert e.time_profiling_path() == "/m/llama/configs/computation_profiling_fp16_llama-7b.json"
    assert e.memory_profiling_path() == "/m/llama/configs/memory_profiling_fp16_llama-7b.json"
    got = profile_configs.hardware_paths(e.args, e.path)
    base = "/m/llama/../../profile_hardware/hardware_configs/"
    assert got == (base + "allreduce_bandwidth_2nodes_4gpus_per_node.json", base + "p2p_bandwidth_2nodes_4gpus_per_node.json",
                   base + "overlap_coefficient.json", base + "sp_time_2nodes_4gpus_per_node.json")


def test_search_info_is_printed_on_initialisation(data, tmp_path, capsys):
    """initialize_search_engine ends with the summary of what the search will work with
    (search_engine.py:101-106,916-969 of the reference): its section titles and a few of its lines."""
    engine = P.build(SearchEngine, data, str(tmp_path), P.LOADING_CASES[0])
    text = capsys.readouterr().out
    for title in ("--- Optimization Configs ----", "---- Environment Configs ----", "------- Model Configs -------",
                  "--- Model Computation Configs ---", "--- Model Memory Configs ---", "Model Args List:",
                  "Profile Hardware Args List:"):
        assert title in text, title
    assert "Memory constraint: %d GB" % engine.args.memory_constraint in text
    assert "Model Name: %s" % engine.model_name in text
    assert "Layer_num: %s" % engine.layernum_list in text


def test_model_type_and_microbatch_function(data, tmp_path):
    """The two optional setters of the reference's scripts (search_dist.py of every model: set_model_type,
    set_microbatch_func).  The chunk function they install is called with four arguments everywhere
    (cost_model.py:79, dynamic_programming.py:224, search_engine.py:1103 of the reference)."""
    from galvatron_dp.pp_utils import optimal_chunk_func_default
    engine = P.build(SearchEngine, data, str(tmp_path), P.LOADING_CASES[0])
    assert engine.model_type == "gpt"
    engine.set_model_type("bert")
    assert engine.model_type == "bert"
    engine.set_microbatch_func(microbatch_size=4, max_chunk=8)
    strategy = [2, 2, 2, {"fsdp": 0}]
    for local_bsz, mbsz, min_tp in ((32, 1, 1), (32, 16, 2), (6, 3, 1), (0, 1, 1)):
        assert engine.optimal_chunk_func(local_bsz, strategy, mbsz, min_tp) == \
            optimal_chunk_func_default(local_bsz, strategy, 4, min_tp)
    engine.set_cost_models()
    assert all(p.optimal_chunk_func is engine.optimal_chunk_func for p in engine.parallel_args_list)
