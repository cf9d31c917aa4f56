"""Scenarios that start from the profilers' files, shared by tests/golden/make_search_profile_golden.py
(which runs them through the reference's GalvatronSearchEngine) and the tests
(galvatron_dp.search.SearchEngine).

The profile data is what the reference's own search-engine tests write to disk
(tests/utils/search_configs.py:9-547 of the reference), kept here as the data file
tests/golden/search_profiles.json; the scenarios restate the parameters of those tests
(tests/search_engine/test_get_configs.py:14-118, test_initialize.py:6-13,
test_parallelsim_optimization.py:9-26 and the argument defaults of tests/utils/search_args.py:5-76).
"""
import json
import os
from types import SimpleNamespace

import numpy as np

import cost_model_cases as C

HERE = os.path.dirname(os.path.abspath(__file__))
PROFILES = os.path.join(HERE, "golden", "search_profiles.json")

# the "llama_search" model of the reference's tests (tests/models/configs/llama.py:48-56; one layer type)
LAYER_CONFIGS = [dict(hidden_size=3584, layer_num=28, seq_len=4096)]
MODEL_NAME = "llama_search"


def reference_test_args(**over):
    """The argument defaults the reference's tests use (tests/utils/search_args.py:5-76)."""
    a = dict(set_model_config_manually=0, set_layernum_manually=0, set_seqlen_manually=0, num_nodes=1,
             num_gpus_per_node=8, memory_constraint=24, min_bsz=8, max_bsz=10240, recommend_min_bsz=0, settle_bsz=-1,
             settle_chunk=-1, bsz_scale=8, search_space="full", sp_space="tp", disable_dp=0, disable_tp=0,
             disable_vtp=0, disable_pp=0, disable_sdp=0, disable_ckpt=0, disable_tp_consec=0, max_tp_deg=8,
             max_pp_deg=8, default_dp_type="ddp", embed_sdp=0, mixed_precision="bf16", pipeline_type="gpipe",
             use_pipeline_costmodel=1, costmodel_coe=1.0, sequence_parallel=False, global_memory_buffer=True,
             async_grad_reduce=True, make_vocab_size_divisible_by=128, fine_grained_mode=1,
             time_profile_mode="static", memory_profile_mode="static", memory_profiling_path=None,
             time_profiling_path=None, allreduce_bandwidth_config_path=None, p2p_bandwidth_config_path=None,
             overlap_coe_path=None, sp_time_path=None, output_config_path=None, log_dir="logs",
             parallel_search=False, local_rank=0,
             # what the reference's model set-up copies from the model into the arguments and the search
             # reads back (galvatron/models/llama_hf/meta_configs/config_utils.py:83-95)
             hidden_size=LAYER_CONFIGS[0]["hidden_size"], seq_length=LAYER_CONFIGS[0]["seq_len"])
    a.update(over)
    return SimpleNamespace(**a)


# (time mode, memory mode, sequence parallel): test_get_configs.py:17-27
LOADING_CASES = [("static", "static", False), ("batch", "static", False), ("sequence", "static", False),
                 ("static", "static", True), ("batch", "static", True), ("sequence", "static", True),
                 ("static", "sequence", True), ("batch", "sequence", True), ("sequence", "sequence", True)]

# whole searches: test_parallelsim_optimization.py:10-13 with the keyword arguments of :16-26
_E2E_COMMON = dict(settle_bsz=64, sp_space="tp+sp", memory_constraint=36, default_dp_type="zero2",
                   pipeline_type="pipedream_flush", async_grad_reduce=False, sequence_parallel=True)
E2E_CASES = {
    "fine_grained": dict(modes=("sequence", "sequence", True), seqlen_list=[8192],
                         args=dict(_E2E_COMMON, settle_chunk=32, fine_grained_mode=1)),
    "coarse": dict(modes=("sequence", "sequence", True), seqlen_list=[8192],
                   args=dict(_E2E_COMMON, settle_chunk=8, fine_grained_mode=0)),
}
# what the reference's test asserts for them (test_parallelsim_optimization.py:35,58-83,85,108-128)
E2E_KNOWN = {
    "fine_grained": dict(throughput=2.8074257503114315,
                         config=dict(pp_deg=1, global_bsz=64, chunks=32, pp_division="28",
                                     pipeline_type="pipedream_flush", default_dp_type="zero2", vtp=8, vsp=0,
                                     embed_sdp=0, tp_sizes_enc=",".join(["8"] * 28),
                                     tp_consecutive_flags=",".join(["1"] * 28), dp_types_enc=",".join(["0"] * 28),
                                     use_sp=",".join(["0"] * 28), checkpoint=",".join(["1"] * 8 + ["0"] * 20))),
    "coarse": dict(throughput=2.5234175303522344,
                   config=dict(pp_deg=1, global_bsz=64, chunks=8, pp_division="28", pipeline_type="pipedream_flush",
                               default_dp_type="zero2", vtp=1, vsp=0, embed_sdp=1, tp_sizes_enc=",".join(["1"] * 28),
                               tp_consecutive_flags=",".join(["1"] * 28), dp_types_enc=",".join(["1"] * 28),
                               use_sp=",".join(["0"] * 28), checkpoint=",".join(["1"] * 28))),
}


def profiles():
    with open(PROFILES) as fh:
        return json.load(fh)


def write_files(data, configs_dir, hardware_dir, time_mode, memory_mode, sp, model_name=MODEL_NAME, precision="bf16",
                num_nodes=1, gpus_per_node=8):
    """The files the profilers would have left, under the names the engine looks for
    (tests/utils/search_configs.py:549-609)."""
    os.makedirs(configs_dir, exist_ok=True)
    os.makedirs(hardware_dir, exist_ok=True)
    memory_kind = "sequence_sp" if memory_mode == "sequence" else ("static_sp" if sp else "static")

    def dump(obj, folder, name):
        with open(os.path.join(folder, name), "w") as fh:
            json.dump(obj, fh)

    dump(data["time"][time_mode], configs_dir, "computation_profiling_%s_%s.json" % (precision, model_name))
    dump(data["memory"][memory_kind], configs_dir, "memory_profiling_%s_%s.json" % (precision, model_name))
    shape = "%dnodes_%dgpus_per_node.json" % (num_nodes, gpus_per_node)
    dump(data["hardware"]["allreduce"], hardware_dir, "allreduce_bandwidth_" + shape)
    dump(data["hardware"]["p2p"], hardware_dir, "p2p_bandwidth_" + shape)
    dump(data["hardware"]["overlap"], hardware_dir, "overlap_coefficient.json")
    dump(data["hardware"]["sp"], hardware_dir, "sp_time_" + shape)


def build(engine_cls, data, workdir, modes, seqlen_list=None, **arg_over):
    """An initialised engine reading its profiles from ``workdir``, the way the reference's tests set
    one up (tests/utils/search_configs.py:611-653)."""
    time_mode, memory_mode, sp = modes
    configs_dir, hardware_dir = os.path.join(workdir, "configs"), os.path.join(workdir, "hardware_configs")
    output_dir, log_dir = os.path.join(workdir, "output"), os.path.join(workdir, "logs")
    os.makedirs(output_dir, exist_ok=True)
    os.makedirs(log_dir, exist_ok=True)
    over = dict(time_profiling_path=configs_dir, memory_profiling_path=configs_dir,
                allreduce_bandwidth_config_path=hardware_dir, p2p_bandwidth_config_path=hardware_dir,
                overlap_coe_path=hardware_dir, sp_time_path=hardware_dir, output_config_path=output_dir,
                log_dir=log_dir, time_profile_mode=time_mode, memory_profile_mode=memory_mode, sequence_parallel=sp)
    over.update(arg_over)
    engine = engine_cls(reference_test_args(**over))
    engine.set_search_engine_info(configs_dir, [dict(c) for c in LAYER_CONFIGS], MODEL_NAME)
    if seqlen_list is not None:
        engine.seqlen_list = list(seqlen_list)
    write_files(data, configs_dir, hardware_dir, time_mode, memory_mode, sp)
    engine.initialize_search_engine()
    return engine


def _plain(x):
    """numpy arrays as lists, then cost_model_cases.jsonable (floats as hex strings)."""
    if isinstance(x, np.ndarray):
        return [_plain(v) for v in x.tolist()]
    if isinstance(x, dict):
        return {k: _plain(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [_plain(v) for v in x]
    return x


def loaded_state(engine):
    """Everything the engine holds after reading its profiles, JSON-able with exact floats."""
    records = []
    for i in range(engine.num_layertype):
        rec = {}
        for name in ("model_args_list", "train_args_list", "parallel_args_list", "profile_model_args_list",
                     "profile_hardware_args_list"):
            fields = dict(vars(getattr(engine, name)[i]))
            fields.pop("optimal_chunk_func", None)
            rec[name] = fields
        records.append(rec)
    state = dict(time_profiled_list=engine.time_profiled_list, other_time_profiled_list=engine.other_time_profiled_list,
                 param_sizes=engine.param_sizes, act_sizes=engine.act_sizes,
                 other_memory_pp_off=engine.other_memory_pp_off, other_memory_pp_on=engine.other_memory_pp_on,
                 allreduce_bandwidth=engine.allreduce_bandwidth, allreduce_comm_coe=engine.allreduce_comm_coe,
                 p2p_bandwidth=engine.p2p_bandwidth, p2p_comm_coe=engine.p2p_comm_coe, overlap_coe=engine.overlap_coe,
                 sp_allreduce=engine.sp_allreduce, sp_all2all=engine.sp_all2all, memory_config=engine.memory_config,
                 time_config=engine.time_config, records=records,
                 strategies=engine.strategies,
                 paths=[os.path.basename(engine.time_profiling_path()), os.path.basename(engine.memory_profiling_path()),
                        os.path.basename(engine.args.allreduce_bandwidth_config_path),
                        os.path.basename(engine.args.p2p_bandwidth_config_path),
                        os.path.basename(engine.args.overlap_coe_path), os.path.basename(engine.args.sp_time_path)])
    return C.jsonable(_plain(state))
