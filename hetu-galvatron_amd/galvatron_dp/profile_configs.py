"""From the profilers' JSON files to the cost-model argument records of a sweep.

Counterpart of the loading half of the reference's search engine
(``galvatron/core/search_engine/search_engine.py:45-84,99-337``) and of the file helpers it uses
(``galvatron/utils/config_utils.py:14-16,59-91,93-101,108-138``): same file names, same keys, same
fits (``scipy.optimize.curve_fit`` on the same points in the same order), same records.  The
functions here take plain values; ``SearchEngine`` (search.py) holds the state and calls them.

Files (``<P>`` = mixed precision, ``<M>`` = model name, ``<N>`` nodes of ``<G>`` GPUs):
  computation_profiling_<P>_<M>.json   {"layertype_<i|other>_bsz<B>_seq<S>": ms}
  memory_profiling_<P>_<M>.json        {"layertype_<i>[_sp]": {seq: {"parameter_size", "tp_activation_per_bsz_dict"}},
                                        "other_memory_pp_off[_sp]" / "other_memory_pp_on_first[_sp]" /
                                        "other_memory_pp_on_last[_sp]": {seq: {"model_states": {tp: MB}, "activation": {tp: MB}}}}
  allreduce_bandwidth_<N>nodes_<G>gpus_per_node.json   {"allreduce_size_<k>_consec_<0|1>": GB/s}
  p2p_bandwidth_<N>nodes_<G>gpus_per_node.json         {"pp_size_<k>": GB/s}
  overlap_coefficient.json                             {"overlap_coe": x}
  sp_time_<N>nodes_<G>gpus_per_node.json               {"allreduce_size_<k>_<MB>MB_time": ms, "all2all_size_...": ms}
"""
from __future__ import annotations

import json
import os

import numpy as np
from scipy.optimize import curve_fit

from .cost_models import ModelArgs, ParallelArgs, ProfileHardwareArgs, ProfileModelArgs, TrainArgs

__all__ = ["read_json_config", "write_json_config", "num2str", "read_allreduce_bandwidth_config",
           "read_p2p_bandwidth_config", "remap_config", "int_keys", "fit_layer_times", "layer_memory",
           "hardware_paths", "cost_model_args"]

HARDWARE_DIR = '../../profile_hardware/hardware_configs/'     # relative to the model's directory


def read_json_config(path):
    """config_utils.py:14-16.  A missing file raises FileNotFoundError."""
    with open(path, 'r', encoding="utf-8") as fh:
        return json.load(fh)


def write_json_config(config, path):
    """config_utils.py:18-20."""
    with open(path, 'w') as fh:
        json.dump(config, fh, indent=4)


def num2str(num, name):
    """'seq4096' for one value, 'seq[a,b]' for several (config_utils.py:93-101)."""
    if name == 'seq' and len(num) == 1:
        num = num[0]
    if isinstance(num, list):
        return '%s[%s]' % (name, ",".join(map(str, num)))
    return '%s%d' % (name, num)


def int_keys(tree):
    """The same nested dicts with every all-digit string key turned into an int
    (search_engine.py:107-117)."""
    if not isinstance(tree, dict):
        return tree
    return {(int(k) if isinstance(k, str) and k.isdigit() else k): int_keys(v) for k, v in tree.items()}


def _line(x, m, c):
    return m * x + c


def _parabola(x, a, b, c):
    return a * x * x + b * x + c


def read_allreduce_bandwidth_config(config_path, gpu_num):
    """({group: GB/s}, {group: 1 / (GB/s)}) with the groups 'world', 'k_0' (strided) and 'k_1'
    (consecutive) for k = world/2, world/4 ... 2, and '1' (config_utils.py:59-78)."""
    env = read_json_config(config_path) if isinstance(config_path, str) else config_path
    bandwidth, coe = {}, {}
    if gpu_num >= 2:
        bandwidth['%d' % gpu_num] = env['allreduce_size_%d_consec_1' % gpu_num]
        coe['%d' % gpu_num] = 1.0 / bandwidth['%d' % gpu_num]
    k = gpu_num // 2
    while k >= 2:
        for consec in (0, 1):
            name = '%d_%d' % (k, consec)
            bandwidth[name] = env['allreduce_size_%d_consec_%d' % (k, consec)]
            coe[name] = 1.0 / bandwidth[name]
        k //= 2
    bandwidth['1'] = np.inf
    coe['1'] = 0
    return bandwidth, coe


def read_p2p_bandwidth_config(config_path):
    """({pp degree: GB/s}, {pp degree: 1 / (GB/s)}) (config_utils.py:80-91)."""
    env = read_json_config(config_path) if isinstance(config_path, str) else config_path
    bandwidth, coe = {}, {}
    for key, val in env.items():
        if 'pp_size_' in key:
            deg = int(key.split('_')[-1])
            bandwidth[deg] = val
            coe[deg] = 1.0 / val
    return bandwidth, coe


def remap_config(config, op):
    """{group size: {message bytes: ms, ..., 'popt': [slope per MB, offset]}} from the entries
    '<op>_size_<k>_<n>MB_time' of the sequence-parallel profile; all-reduce times are halved (one
    all-gather or reduce-scatter) (config_utils.py:108-138)."""
    out = {}
    for key, val in config.items():
        if not key.startswith(op):
            continue
        if op == "allreduce":
            val = val / 2
        parts = key.split("_")
        group, mb = int(parts[-3]), int(parts[-2][:-2])
        out.setdefault(group, {})[mb * 1024 * 1024] = val
    for group, times in out.items():
        x = [size // 1024 // 1024 for size in times]
        y = list(times.values())
        assert len(x) >= 8, f"Different size in communication profile of {op} should not be lower than 8."
        times["popt"] = curve_fit(_line, x, y)[0]
    return out


def fit_layer_times(time_config, mode, num_layertype, seqlen_list):
    """(forward time per layer type, forward time of the non-layer parts per layer type) from the
    computation profile (search_engine.py:123-194).

    static:   the profiled ms of every matching entry, as they come (the non-layer entries once per
              layer type);
    batch:    [m, c] of ms·bsz = m·bsz + c over the entries of the type's sequence length;
    sequence: the value at the type's sequence length of a parabola (layers) or a line (the rest)
              through the bsz = 1 entries."""
    layers, other = [], []
    if mode == 'static':
        for i in range(num_layertype):
            for key, ms in time_config.items():
                if key.startswith('layertype_%d_' % i):
                    layers.append(ms)
                if key.startswith('layertype_other_'):
                    other.append(ms)
    elif mode == 'batch':
        for kind, out in (('%d', layers), ('other', other)):
            for i in range(num_layertype):
                prefix = 'layertype_%s_' % (kind % i if kind == '%d' else kind)
                x, y = [], []
                for key, ms in time_config.items():
                    if key.startswith(prefix) and '_seq%d' % seqlen_list[i] in key:
                        x.append(int(key.split('_')[-2][3:]))
                        y.append(ms * x[-1])
                assert len(x) >= 8, "Different bsz in computation profile of %s should not be lower than 8." % prefix[:-1]
                out.append(curve_fit(_line, x, y)[0])
    elif mode == 'sequence':
        for kind, out, curve in (('%d', layers, _parabola), ('other', other, _line)):
            for i in range(num_layertype):
                prefix = 'layertype_%s_' % (kind % i if kind == '%d' else kind)
                x, y = [], []
                for key, ms in time_config.items():
                    if key.startswith(prefix) and "_bsz1_" in key:
                        x.append(int(key.split('seq')[-1]))
                        y.append(ms)
                out.append(curve(seqlen_list[i], *curve_fit(curve, x, y)[0]))
    else:
        return None, None
    return layers, other


def layer_memory(memory_config, mode, sequence_parallel, num_layertype, seqlen_list):
    """(parameter MB per layer type, {tp: activation MB per sample} per layer type, non-layer memory
    without pipeline, {'first_stage', 'last_stage'} non-layer memory with pipeline) from the memory
    profile whose digit keys are ints already (search_engine.py:195-247).

    static:   the entries at the model's sequence length(s);
    sequence: parameters from the shortest profiled sequence, activations from the longest, scaled
              linearly to the model's length.  The scaling of the non-layer activations is written
              into ``memory_config`` itself, as the reference does."""
    params = [0] * num_layertype
    acts = [{} for _ in range(num_layertype)]
    if mode == "sequence":
        assert sequence_parallel, "Sequence parallel is required for sequence memory profiling."
        assert num_layertype == 1, "Only support num(layertype) == 1 for sequence memory profiling."
        longest = []
        for i in range(num_layertype):
            table = memory_config['layertype_%d_sp' % i]
            lengths = [int(s) for s in table.keys()]
            hi, lo = max(lengths), min(lengths)
            longest.append(hi)
            params[i] = table[lo]['parameter_size']
            acts[i] = table[hi]['tp_activation_per_bsz_dict'].copy()
            for tp in acts[i]:
                acts[i][tp] = acts[i][tp] / hi * seqlen_list[i]
        off = memory_config['other_memory_pp_off_sp'][longest[0]]
        on = {'first_stage': memory_config['other_memory_pp_on_first_sp'][longest[0]],
              'last_stage': memory_config['other_memory_pp_on_last_sp'][longest[-1]]}
        for tp in off['activation']:
            off['activation'][tp] = off['activation'][tp] / longest[0] * seqlen_list[0]
            on['first_stage']['activation'][tp] = on['first_stage']['activation'][tp] / longest[0] * seqlen_list[0]
            on['last_stage']['activation'][tp] = on['last_stage']['activation'][tp] / longest[-1] * seqlen_list[-1]
        return params, acts, off, on
    if mode == "static":
        tail = '_sp' if sequence_parallel else ''
        for i in range(num_layertype):
            entry = memory_config['layertype_%d%s' % (i, tail)][seqlen_list[i]]
            params[i] = entry['parameter_size']
            acts[i] = entry['tp_activation_per_bsz_dict'].copy()
        seq = num2str(seqlen_list, 'seq')[3:]
        if seq.isdigit():
            seq = int(seq)
        off = memory_config['other_memory_pp_off' + tail][int(seq) if sequence_parallel else seq]
        on = {'first_stage': memory_config['other_memory_pp_on_first' + tail][seq],
              'last_stage': memory_config['other_memory_pp_on_last' + tail][seq]}
        return params, acts, off, on
    return params, acts, None, None


def hardware_paths(args, model_path):
    """Where the four hardware files lie: the directory an argument names, or
    ``<model_path>/../../profile_hardware/hardware_configs/``; the file names carry the cluster's
    shape (search_engine.py:250-284).  Returns (allreduce, p2p, overlap, sp)."""
    def place(given, name):
        base = os.path.join(model_path, HARDWARE_DIR) if given is None else given
        return os.path.join(base, name)

    shape = '%dnodes_%dgpus_per_node.json' % (args.num_nodes, args.num_gpus_per_node)
    return (place(args.allreduce_bandwidth_config_path, 'allreduce_bandwidth_' + shape),
            place(args.p2p_bandwidth_config_path, 'p2p_bandwidth_' + shape),
            place(args.overlap_coe_path, 'overlap_coefficient.json'),
            place(args.sp_time_path, 'sp_time_' + shape))


def cost_model_args(args, layer, optimal_chunk_func, parameter_size, tp_activation_per_bsz_dict, other_memory_pp_off,
                    other_memory_pp_on, forward_time, other_time, allreduce_comm_coe, p2p_comm_coe, overlap_coe,
                    sp_allreduce, sp_all2all):
    """The five argument records of one layer type (search_engine.py:293-336).  ``layer`` is
    (hidden size, layer count, sequence length)."""
    hidden, count, seq = layer
    return (ModelArgs(parameter_size=parameter_size, seq_length=seq, hidden_size=hidden, layer_num=count),
            TrainArgs(mixed_precision=args.mixed_precision != 'fp32', async_grad_reduce=args.async_grad_reduce),
            ParallelArgs(use_zero2_for_dp=args.default_dp_type == 'zero2', disable_vtp=args.disable_vtp,
                         sequence_parallel=args.sequence_parallel, sp_space=args.sp_space,
                         pipeline_type=args.pipeline_type, optimal_chunk_func=optimal_chunk_func),
            ProfileModelArgs(tp_activation_per_bsz_dict=tp_activation_per_bsz_dict,
                             other_memory_pp_off=other_memory_pp_off, other_memory_pp_on=other_memory_pp_on,
                             forward_computation_time=forward_time, other_time_profiled=other_time),
            ProfileHardwareArgs(bct_fct_coe=2, extra_overhead=0, comm_coe_dict=allreduce_comm_coe,
                                dp_overlap_coe=overlap_coe, bct_overlap_coe=overlap_coe,
                                p2p_comm_coe_dict=p2p_comm_coe, costmodel_coe=args.costmodel_coe,
                                allreduce_dict=sp_allreduce, all2all_dict=sp_all2all))
