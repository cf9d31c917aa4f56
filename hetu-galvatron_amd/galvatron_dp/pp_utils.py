"""How the layers of a model are dealt out to pipeline stages before the DP runs, and the chunk
(micro-batch count) helpers of the sweep.

Counterpart of the pipeline-division utilities of the reference's search engine
(``galvatron/core/search_engine/search_engine.py:972-1104``): same function names, arguments and
returned values; the tests compare against values recorded from the reference's functions.
"""
from __future__ import annotations

import copy

import numpy as np

from .cost_models import MemoryCostModel

__all__ = ["pp_division_even", "pp_division_memory_balanced", "get_pp_stage_for_bsz", "get_cost_all_stages",
           "get_layer_costs", "optimal_chunk_func_default", "check_optimal_chunks"]


def pp_division_even(layernum_list, pp_deg):
    """floor(total / pp) layers per stage, the remainder on the last one (search_engine.py:1083-1088)."""
    total = np.sum(layernum_list)
    share = int(total // pp_deg)
    return [share] * (pp_deg - 1) + [total - share * (pp_deg - 1)]


def get_layer_costs(layernum_list, layer_costs):
    """One entry per layer from one entry per layer type (search_engine.py:1077-1081)."""
    out = []
    for count, cost in zip(layernum_list, layer_costs):
        out += [cost] * count
    return out


def get_cost_all_stages(layer_memcosts, pp_stage_division):
    """Per-stage sums of a per-layer list that may carry one extra leading entry (the non-layer
    memory, counted on the first stage) or one leading and one trailing entry
    (search_engine.py:1060-1075)."""
    division = copy.deepcopy(pp_stage_division)
    extra = len(layer_memcosts) - np.sum(division)
    if extra == 1:
        division[0] += 1
    elif extra == 2:
        division[0] += 1
        division[-1] += 1
    assert np.sum(division) == len(layer_memcosts)
    bounds = [int(np.sum(division[:i])) for i in range(len(division) + 1)]
    return [np.sum(layer_memcosts[a:b]) for a, b in zip(bounds[:-1], bounds[1:])]


def optimal_chunk_func_default(local_bsz, strategy, microbatch_size, min_tp):
    """ceil(samples of one pipeline lane / micro-batch size), at least 1 (search_engine.py:1090-1098)."""
    assert strategy[1] % min_tp == 0
    lane = local_bsz // (strategy[1] // min_tp)
    chunk = np.ceil(lane / microbatch_size)
    return 1 if chunk == 0 else chunk


def check_optimal_chunks(world_size, strategies, optimal_chunk_func, bsz, mbsz_dict, min_tp):
    """{pp degree: chunks of the pure data-parallel strategy at tp = min_tp} (search_engine.py:1100-1104)."""
    out = {}
    for pp in sorted(set(s[0] for s in strategies)):
        out[pp] = optimal_chunk_func(bsz / (world_size // pp // min_tp),
                                     [pp, min_tp, world_size // pp, {'fsdp': 0, 'cpt': 0}], mbsz_dict[pp], min_tp)
    return out


def pp_division_memory_balanced(model_args_list, train_args_list, parallel_args_list, profile_model_args_list,
                                layer_num, pp_deg, bsz, mbsz, strategies):
    """Stage sizes that even out the memory of the cheapest (pure data-parallel, gpipe) placement of
    every layer plus the non-layer memory of the first and last stage; returns (layers per stage,
    MB per stage) (search_engine.py:972-1046).

    Greedy fill up to the average, a stage taking a layer while less than half of it would overshoot;
    then stages more than 30 % above the average hand layers on, and no stage stays empty."""
    n_types = len(layer_num)
    assert n_types == len(model_args_list) == len(train_args_list) == len(parallel_args_list) == len(profile_model_args_list)
    if pp_deg == 1:
        return [np.sum(layer_num)], None
    candidates = [s for s in strategies if s[0] == pp_deg]
    if not candidates:
        return None, None
    records = []
    for i in range(n_types):
        parallel = copy.deepcopy(parallel_args_list[i])
        parallel.pipeline_type = 'gpipe'
        records.append(dict(model_args=copy.deepcopy(model_args_list[i]), train_args=copy.deepcopy(train_args_list[i]),
                            parallel_args=parallel, profile_model_args=copy.deepcopy(profile_model_args_list[i])))
    world = candidates[0][0] * candidates[0][1] * candidates[0][2]
    per_layer = []
    for i in range(n_types):
        cost = MemoryCostModel([pp_deg, 1, world // pp_deg, {}], global_batch_size=bsz, mbsz=mbsz, min_tp=1, max_tp=1,
                               **records[i]).get_memory_cost()['enc_total']
        per_layer += [np.min(cost)] * layer_num[i]
    other = MemoryCostModel(candidates[0], global_batch_size=bsz, mbsz=mbsz, min_tp=1, max_tp=1,
                            **records[0]).get_memory_cost()['other'][1]
    average = (np.sum(per_layer) + np.sum(other)) / pp_deg

    division = [0] * pp_deg
    filled = other.copy()
    nxt = 0
    for stage in range(pp_deg):
        while nxt < len(per_layer):
            if stage < pp_deg - 1 and average - filled[stage] < 0.5 * per_layer[nxt]:
                break
            filled[stage] += per_layer[nxt]
            nxt += 1
            division[stage] += 1

    for stage in range(pp_deg - 1):                       # too much on an early stage: pass layers on
        first, last = int(np.sum(division[:stage])), int(np.sum(division[:stage + 1]))
        load = np.sum(per_layer[first:last]) + other[stage]
        while load > average * 1.3:
            division[stage] -= 1
            division[stage + 1] += 1
            last -= 1
            load -= per_layer[last]
    for stage in range(pp_deg - 1):                       # no empty stage, front to back ...
        while division[stage] <= 0:
            division[stage] += 1
            division[stage + 1] -= 1
    for stage in range(pp_deg - 1, 0, -1):                # ... and back to front
        while division[stage] <= 0:
            division[stage] += 1
            division[stage - 1] -= 1

    per_stage = other.copy()
    for stage in range(pp_deg):
        first, last = int(np.sum(division[:stage])), int(np.sum(division[:stage + 1]))
        per_stage[stage] += np.sum(per_layer[first:last])
    return division, per_stage


def get_pp_stage_for_bsz(strategies, model_args_list, train_args_list, parallel_args_list, profile_model_args_list,
                         layer_num_list, bsz, mbsz_dict, single_layer_even=True):
    """{pp degree: layers per stage}: even for a single layer type (unless asked otherwise), memory
    balanced for several (search_engine.py:1048-1058)."""
    out = {}
    for pp in sorted(set(s[0] for s in strategies)):
        if single_layer_even and len(layer_num_list) == 1:
            out[pp] = pp_division_even(layer_num_list, pp)
        else:
            out[pp] = pp_division_memory_balanced(model_args_list, train_args_list, parallel_args_list,
                                                  profile_model_args_list, layer_num_list, pp, bsz, mbsz_dict[pp],
                                                  strategies)[0]
    return out
