"""The sweep of the search engine: which (batch size, chunks, min_tp, max_tp, vsp, embed_sdp,
sp_search) tasks exist, which strategies each may use, one ``DpOnModel.fit`` per task, the choice
of the best throughput and the result file.

Counterpart of ``GalvatronSearchEngine.parallelism_optimization`` / ``set_searching_bsz`` /
``dynamic_programming`` / ``save_results`` / ``generate_strategies``
(``galvatron/core/search_engine/search_engine.py:339-688,783-914``): same task order, same strategy
filters, same tie-breaking (first strictly better throughput wins) and the same
``galvatron_config_*.json``.  What differs is where the DPs run: the reference solves them task by
task (optionally on a thread pool); here the DP instances of ALL tasks of a sweep are collected
first and solved in one device batch, then every task is finished from its share of the results.

The cost-model argument records come either from the profilers' files
(``set_search_engine_info`` + ``initialize_search_engine``, search_engine.py:45-337; the reading
itself is in profile_configs.py) or directly from the caller (``set_model`` +
``set_cost_model_args``).
"""
from __future__ import annotations

import copy
import json
import os

import numpy as np

from . import _lib, cost_models, profile_configs
from .dynamic_programming import DPAlg, DpOnModel
from .pp_utils import check_optimal_chunks, get_pp_stage_for_bsz, optimal_chunk_func_default

__all__ = ["SearchEngine", "strategy2config", "array2str"]


def array2str(values):
    """'a,b,c' (galvatron/utils/config_utils.py:11-12)."""
    return ",".join(map(str, values))


def strategy2config(strategy_list):
    """Per-layer strategies as the comma-separated fields of the result file
    (galvatron/utils/config_utils.py:46-57)."""
    if len(strategy_list) == 0:
        return {}
    return {"pp_deg": strategy_list[0][0],
            "tp_sizes_enc": array2str([s[1] for s in strategy_list]),
            "tp_consecutive_flags": array2str([0 if 'tp' in s[-1] and not s[-1]['tp'] else 1 for s in strategy_list]),
            "dp_types_enc": array2str([1 if s[-1].get('fsdp') else 0 for s in strategy_list]),
            "use_sp": array2str([1 if s[-1].get('sp') else 0 for s in strategy_list])}


def _powers_of_two(limit):
    out, k = [], 1
    while k <= limit:
        out.append(k)
        k *= 2
    return out


class SearchEngine:
    """``args`` is a namespace with the reference's search flags (galvatron/core/search_engine/
    arguments.py): num_nodes, num_gpus_per_node, memory_constraint (GB), search_space, sp_space,
    max_tp_deg, max_pp_deg, disable_dp/sdp/tp/pp/ckpt/tp_consec/vtp, global_memory_buffer,
    settle_bsz, settle_chunk, bsz_scale, min_bsz, max_bsz, recommend_min_bsz, use_pipeline_costmodel,
    pipeline_type, default_dp_type, mixed_precision, sequence_parallel, hidden_size,
    fine_grained_mode, output_config_path."""

    def __init__(self, args):
        self.args = args
        args.gpu_num = args.num_nodes * args.num_gpus_per_node
        self.memory_constraint = args.memory_constraint * 1024
        self.optimal_chunk_func = optimal_chunk_func_default
        self.model_type = 'gpt'
        self.model_name = None
        self.path = None
        self.mem_path = None
        self.time_path = None
        self.strategies = None
        self.results = None
        self.optimal = None
        self.solved_instances = 0
        self.keep_device_cache = False      # True: a sweep leaves the library's cached device allocations in place
        self.overlap_part = 512             # DP instances per part handed to the device while later tasks are still
                                            # being prepared on the host; 0: one batch when everything is prepared

    # ---- model, paths (search_engine.py:45-97) ---------------------------------------------------------
    def set_model(self, model_name, model_layer_configs, path=None):
        self.model_name = model_name
        self.path = path
        self.set_model_layer_configs(model_layer_configs)

    def set_search_engine_info(self, path, model_layer_configs, model_name):
        """``path``: the model's directory (profiles in ``<path>/configs`` unless the arguments name
        another place); ``model_layer_configs``: one {'hidden_size', 'layer_num', 'seq_len'} per layer
        type."""
        self.set_model_layer_configs(model_layer_configs)
        self.path = path
        self.model_name = model_name
        self.memory_profiling_path()
        self.time_profiling_path()

    def set_path(self, path):
        self.path = path

    def set_model_name(self, name):
        self.model_name = name

    def set_model_type(self, model_type):
        """Kept for the scripts that call it (search_engine.py:55-56); nothing in a search reads it."""
        self.model_type = model_type

    def set_microbatch_func(self, microbatch_size, max_chunk):
        """Chunk counts from a fixed micro-batch size instead of the one each task implies
        (search_engine.py:88-89); to be called before the cost-model records are built.  The reference
        installs a callable of two arguments here while every call site passes four (cost_model.py:79,
        dynamic_programming.py:224, search_engine.py:1103), so its own searches raise TypeError after this
        call; this one takes the four arguments.  ``max_chunk`` is not used, as in the reference."""
        self.optimal_chunk_func = lambda local_bsz, strategy, mbsz=None, min_tp=1: optimal_chunk_func_default(
            local_bsz, strategy, microbatch_size, min_tp)

    def set_model_layer_configs(self, model_layer_configs):
        if model_layer_configs is None:
            return
        self.hiddensize_list = [c['hidden_size'] for c in model_layer_configs]
        self.layernum_list = [c['layer_num'] for c in model_layer_configs]
        self.seqlen_list = [c['seq_len'] for c in model_layer_configs]
        self.num_layertype = len(self.layernum_list)

    def _profile_path(self, given, stem):
        assert self.model_name is not None, 'Should specify the model name!'
        base = os.path.join(self.path, 'configs') if given is None else given
        return os.path.join(base, '%s_%s_%s.json' % (stem, self.args.mixed_precision, self.model_name))

    def memory_profiling_path(self):
        if self.mem_path is None:
            self.mem_path = self._profile_path(self.args.memory_profiling_path, 'memory_profiling')
        return self.mem_path

    def time_profiling_path(self):
        if self.time_path is None:
            self.time_path = self._profile_path(self.args.time_profiling_path, 'computation_profiling')
        return self.time_path

    # ---- profiles -> argument records (search_engine.py:99-337) ---------------------------------------
    def initialize_search_engine(self):
        self.generate_strategies()
        self.get_profiled_model_configs()
        self.get_profiled_hardware_configs()
        self.set_cost_models()
        self.show_search_info()

    def show_search_info(self):
        """What the search will work with, printed (search_engine.py:916-969)."""
        args, bar = self.args, '=' * 80
        sections = [
            ('--- Optimization Configs ----',
             [('Memory constraint: %d GB' % args.memory_constraint,), ('Pipeline Type:', args.pipeline_type),
              ('Default DP Type:', args.default_dp_type), ('Mixed Precision:', args.mixed_precision), ('Search Space:',),
              (', '.join(cost_models.form_strategy(s) for s in self.strategies or []),)]),
            ('---- Environment Configs ----',
             [('Allreduce Bandwidth (GB/s):', getattr(self, 'allreduce_bandwidth', None)),
              ('Allreduce Communication Coefficient (ms/MB):', getattr(self, 'allreduce_comm_coe', None)),
              ('P2P Bandwidth (GB/s):', getattr(self, 'p2p_bandwidth', None)),
              ('P2P Communication Coefficient (ms/MB):', getattr(self, 'p2p_comm_coe', None)),
              ('Overlap coefficient:', getattr(self, 'overlap_coe', None))]),
            ('------- Model Configs -------',
             [('Model Name:', self.model_name), ('Num layertype:', self.num_layertype), ('Layer_num:', self.layernum_list),
              ('Hidden_size:', self.hiddensize_list), ('Seq_len:', self.seqlen_list)]),
            ('--- Model Computation Configs ---',
             [('Forward computation time:', getattr(self, 'time_profiled_list', None))]),
            ('--- Model Memory Configs ---',
             [('Parameter Memory Cost:', getattr(self, 'param_sizes', None)),
              ('Activation Memory Cost of Different TP degree (per bsz):',), (getattr(self, 'act_sizes', None),),
              ('Other Memory Cost (pp = 1):',), (getattr(self, 'other_memory_pp_off', None),),
              ('Other Memory Cost (pp > 1):',), (getattr(self, 'other_memory_pp_on', None),)]),
            ('Model Args List:', [(self.model_args_list,)]), ('Train Args List:', [(self.train_args_list,)]),
            ('Parallel Args List:', [(self.parallel_args_list,)]),
            ('Profile Model Args List:', [(self.profile_model_args_list,)]),
            ('Profile Hardware Args List:', [(self.profile_hardware_args_list,)])]
        for title, lines in sections:
            print(bar)
            print(title)
            for line in lines:
                print(*line)
        print(bar)

    def get_profiled_model_configs(self):
        args = self.args
        self.time_config = profile_configs.read_json_config(self.time_profiling_path())
        self.memory_config = profile_configs.int_keys(profile_configs.read_json_config(self.memory_profiling_path()))
        self.time_profiled_list, self.other_time_profiled_list = profile_configs.fit_layer_times(
            self.time_config, args.time_profile_mode, self.num_layertype, self.seqlen_list)
        (self.param_sizes, self.act_sizes, self.other_memory_pp_off,
         self.other_memory_pp_on) = profile_configs.layer_memory(
            self.memory_config, args.memory_profile_mode, args.sequence_parallel, self.num_layertype, self.seqlen_list)
        return self.time_config, self.memory_config

    def get_profiled_hardware_configs(self):
        """Also rewrites the four path arguments to the files' full names, as the reference does."""
        args = self.args
        (args.allreduce_bandwidth_config_path, args.p2p_bandwidth_config_path, args.overlap_coe_path,
         args.sp_time_path) = profile_configs.hardware_paths(args, self.path)
        self.allreduce_bandwidth, self.allreduce_comm_coe = profile_configs.read_allreduce_bandwidth_config(
            args.allreduce_bandwidth_config_path, gpu_num=args.gpu_num)
        self.p2p_bandwidth, self.p2p_comm_coe = profile_configs.read_p2p_bandwidth_config(args.p2p_bandwidth_config_path)
        self.overlap_coe = profile_configs.read_json_config(args.overlap_coe_path)['overlap_coe']
        sp_config = profile_configs.read_json_config(args.sp_time_path)
        self.sp_allreduce = profile_configs.remap_config(sp_config, "allreduce")
        self.sp_all2all = profile_configs.remap_config(sp_config, "all2all")
        return self.allreduce_bandwidth, self.p2p_bandwidth, self.overlap_coe, self.sp_allreduce, self.sp_all2all

    def set_cost_models(self):
        records = [profile_configs.cost_model_args(
            self.args, (self.hiddensize_list[i], self.layernum_list[i], self.seqlen_list[i]), self.optimal_chunk_func,
            self.param_sizes[i], self.act_sizes[i], self.other_memory_pp_off, self.other_memory_pp_on,
            self.time_profiled_list[i], self.other_time_profiled_list[0], self.allreduce_comm_coe, self.p2p_comm_coe,
            self.overlap_coe, self.sp_allreduce, self.sp_all2all) for i in range(self.num_layertype)]
        (self.model_args_list, self.train_args_list, self.parallel_args_list, self.profile_model_args_list,
         self.profile_hardware_args_list) = [list(column) for column in zip(*records)]

    def set_cost_model_args(self, model_args_list, train_args_list, parallel_args_list, profile_model_args_list,
                            profile_hardware_args_list, allreduce_comm_coe):
        self.model_args_list, self.train_args_list = model_args_list, train_args_list
        self.parallel_args_list, self.profile_model_args_list = parallel_args_list, profile_model_args_list
        self.profile_hardware_args_list = profile_hardware_args_list
        self.allreduce_comm_coe = allreduce_comm_coe

    # ---- strategies (search_engine.py:783-914) -------------------------------------------------------
    def generate_dp_tp_pp_sdp(self, gpu_num=None, search_space=None):
        args = self.args
        world = args.gpu_num if gpu_num is None else gpu_num
        space = args.search_space                      # as the reference: the argument is not consulted
        sizes = _powers_of_two(world)

        def placements(pp, tp, with_sdp):
            dp = world // (pp * tp)
            kinds = (0, 1) if with_sdp else (0,)
            if tp == 1 or tp == world / pp:
                return [[pp, tp, dp, {}]] if dp == 1 else [[pp, tp, dp, {'fsdp': f}] for f in kinds]
            return [[pp, tp, dp, {'tp': c, 'fsdp': f}] for c in (0, 1) for f in kinds]

        if space == 'full':
            out = [s for pp in sizes for tp in sizes if pp * tp <= world for s in placements(pp, tp, True)]
        elif space == 'dp+tp':
            out = [s for tp in sizes if tp <= world for s in placements(1, tp, False)]
        elif space == 'dp+pp':
            out = [s for pp in sizes if pp <= world for s in placements(pp, 1, False)]
        elif space == '3d':
            out = [[2, 2, world // 4, {'tp': 1, 'fsdp': 0}]]
        elif space == 'dp':
            out = [[1, 1, world, {'fsdp': 0}]]
        elif space == 'sdp':
            out = [[1, 1, world, {'fsdp': 1}]]
        elif space == 'tp':
            out = [[1, args.max_tp_deg, world // args.max_tp_deg, {'fsdp': 0}]]
            if out[0][2] > 1:
                out[0][-1]['tp'] = 1
        elif space == 'pp':
            out = [[args.max_pp_deg, 1, world // args.max_pp_deg, {'fsdp': 0}]]

        if args.sp_space in ('tp', 'sp'):
            for s in out:
                if s[1] > 1:
                    s[-1]['sp'] = 0 if args.sp_space == 'tp' else 1
            return out
        if args.sp_space == 'tp+sp':
            both = []
            for s in out:
                if s[1] > 1:
                    for sp in (0, 1):
                        twin = copy.deepcopy(s)
                        twin[-1]['sp'] = sp
                        both.append(twin)
                else:
                    both.append(copy.deepcopy(s))
            return both
        return out

    def generate_strategies(self):
        args = self.args
        strategies = self.generate_dp_tp_pp_sdp()
        if args.search_space == 'dp+tp':
            args.disable_sdp = args.disable_pp = 1
        elif args.search_space == 'dp+pp':
            args.disable_sdp = args.disable_tp = 1
        elif args.search_space == '3d':
            args.disable_sdp = 1
        if args.search_space in ['3d', 'dp', 'tp', 'pp', 'sdp']:
            args.disable_ckpt = 1
            self.strategies = strategies
            return strategies
        assert not (args.disable_sdp and args.disable_dp)

        def allowed(s):
            flags = s[-1]
            if s[2] > 1 and 'fsdp' in flags:
                if (args.disable_dp and flags['fsdp'] == 0) or (args.disable_sdp and flags['fsdp'] == 1):
                    return False
            if (args.disable_tp and s[1] > 1) or (args.disable_pp and s[0] > 1):
                return False
            if args.disable_tp_consec and 'tp' in flags and flags['tp'] == 0:
                return False
            return s[1] <= args.max_tp_deg and s[0] <= args.max_pp_deg

        strategies = [s for s in strategies if allowed(s)]
        if not args.disable_ckpt:
            with_cpt = []
            for s in strategies:
                twin = copy.deepcopy(s)
                twin[-1]['cpt'] = 1
                with_cpt.append(twin)
            strategies += with_cpt
        self.strategies = strategies
        return strategies

    # ---- batch sizes (search_engine.py:539-599) ------------------------------------------------------
    def set_searching_bsz(self):
        args = self.args
        if args.settle_bsz is not None and args.settle_bsz > 0:
            self.min_bsz = self.max_bsz = args.settle_bsz
            self.bsz_scale = 0
            self.BSZs = [args.settle_bsz]
            return
        scale = self.bsz_scale = args.bsz_scale
        if args.recommend_min_bsz:
            recommended = self.recommend_min_bsz(scale)
            args.min_bsz = recommended if recommended > 0 else args.min_bsz
        self.min_bsz = max(args.min_bsz, scale) // scale * scale
        self.max_bsz = int(np.ceil(args.max_bsz / scale) * scale) if args.max_bsz % scale else (args.max_bsz + scale)
        self.BSZs = list(range(self.min_bsz, self.max_bsz, scale))
        self.max_bsz = self.BSZs[-1]

    def recommend_min_bsz(self, scale):
        """A start of the batch-size range from the largest batches the pure dp / sdp / tp baselines
        hold: 35 % of the way down from the largest to the smallest of them."""
        args, world = self.args, self.args.gpu_num
        if args.search_space not in ['full', 'dp+pp', 'dp+tp']:
            return -1
        baselines = []
        if not args.disable_dp:
            baselines.append([1, 1, world, {'fsdp': 0}])
        if not args.disable_sdp:
            baselines.append([1, 1, world, {'fsdp': 1}])
        if not args.disable_tp:
            baselines.append([1, world, 1, {'fsdp': 0}])
        limits = [self.estimate_strategy_max_bsz([s], scale) for s in baselines]
        hi, lo = np.max(limits), np.min(limits)
        start = int((lo * (1 - 0.65) + hi * 0.65) // scale * scale)
        return start if start > scale else scale

    def estimate_strategy_max_bsz(self, strategies, scale):
        bsz = scale
        while True:
            stage = get_pp_stage_for_bsz(strategies, self.model_args_list, self.train_args_list, self.parallel_args_list,
                                         self.profile_model_args_list, self.layernum_list, bsz, {1: bsz})
            fit = self._dp_on_model(strategies, stage, history=False).fit(bsz, 1, 1, 0, 1, print_=False,
                                                                          mbsz_dict={1: bsz})
            if fit[2] == -1:
                return bsz - scale
            bsz += scale

    # ---- the sweep (search_engine.py:339-537,601-638) ------------------------------------------------
    def _dp_on_model(self, strategies, pp_stage_dict, history=True, logger=None):
        args = self.args
        extra = dict(model_microbatch_after_dp=args.use_pipeline_costmodel, pipeline_type=args.pipeline_type,
                     logger=logger) if history else {}
        return DpOnModel(strategies, cost_models.MemoryCostModel, cost_models.TimeCostModel,
                         model_args_list=self.model_args_list, train_args_list=self.train_args_list,
                         parallel_args_list=self.parallel_args_list,
                         profile_model_args_list=self.profile_model_args_list,
                         profile_hardware_args_list=self.profile_hardware_args_list, max_mem=self.memory_constraint,
                         layer_num=self.layernum_list, sequence_len=self.seqlen_list, multi_layer_type=True,
                         pp_stage_dict=pp_stage_dict, comm_coe_dict=self.allreduce_comm_coe, gpu_num=args.gpu_num,
                         config=args, **extra)

    def dynamic_programming(self, strategies, bsz, chunk, mbsz_dict, pp_stage_dict, min_tp, max_tp, vsp, embed_sdp,
                            sp_search, logger=None):
        """One (task, sp_search) on its own: the ``DpOnModel.fit`` of that task and what the sweep keeps of it
        (search_engine.py:601-638).  The sweep itself does not go through here: it prepares all tasks first
        and solves their DP instances together."""
        model = self._dp_on_model(strategies, pp_stage_dict, logger=logger)
        check_optimal_chunks(self.args.gpu_num, strategies, self.optimal_chunk_func, bsz, mbsz_dict, min_tp)
        cost, res_list, pp_deg, remain, mem_cost, vtp = model.fit(bsz, min_tp, max_tp, vsp, embed_sdp, sp_search,
                                                                  print_=False, mbsz_dict=mbsz_dict)
        return {'min_cost': cost, 'min_res_list': res_list, 'min_pp_deg': pp_deg, 'mem_remain': remain,
                'mem_cost': mem_cost, 'throughput': bsz / cost, 'vtp': vtp}

    def _spaces(self):
        """(min_tp values, max_tp values, vsp values, embed_sdp values, sp_search values)."""
        args = self.args
        min_tps = [1] if args.disable_vtp else [k for k in _powers_of_two(args.gpu_num) if k <= args.max_tp_deg]
        if not args.global_memory_buffer:
            max_tps, sp_searches = [args.max_tp_deg], [1, 3]
        else:
            max_tps, sp_searches = min_tps, [1, 2, 3]          # 1: tp, 2: sp, 3: both
        if args.sp_space == 'tp+sp':
            vsps = [0, 1]
        elif args.sp_space == 'tp':
            vsps, sp_searches = [0], [1]
        else:
            raise AssertionError("Only sp mode unsupport now.")
        embed_sdps = [0] if args.disable_sdp else [0, 1]
        return min_tps, max_tps, vsps, embed_sdps, sp_searches

    def tasks(self):
        """(bsz, chunk, min_tp, max_tp, vsp, embed_sdp) in the reference's order of visiting them."""
        min_tps, max_tps, vsps, embed_sdps, _ = self._spaces()
        out = []
        for bsz in self.BSZs:
            chunks = [self.args.settle_chunk] if self.args.settle_chunk != -1 else range(1, bsz + 1)
            for chunk in chunks:
                if bsz % chunk != 0:
                    continue
                for min_tp in min_tps:
                    for max_tp in max_tps:
                        if min_tp > max_tp:
                            continue
                        for vsp in vsps:
                            for embed_sdp in embed_sdps:
                                out.append((bsz, chunk, min_tp, max_tp, vsp, embed_sdp))
        return out

    def _task_strategies(self, bsz, chunk, min_tp, max_tp, sp_search):
        """The strategies one (task, sp_search) may use, its micro-batch sizes per pipeline degree and
        its stage division; None when nothing is left (search_engine.py:393-426)."""
        world = self.args.gpu_num
        lane = lambda pp: bsz // (world // pp // min_tp)          # noqa: E731  samples per pipeline lane at tp = min_tp
        cand = [s for s in self.strategies if min_tp <= s[1] <= max_tp]
        cand = [s for s in cand if chunk <= lane(s[0])]
        if sp_search == 1:
            cand = [s for s in cand if s[-1].get('sp', 0) == 0]
        if sp_search == 2:
            cand = [s for s in cand if 'sp' not in s[-1] or s[-1]['sp'] == 1]
        if not cand:
            return None
        pps = [pp for pp in sorted(set(s[0] for s in cand))
               if pp * min_tp <= world and bsz % (world // pp // min_tp) == 0]
        if not pps:
            return None
        cand = [s for s in cand if s[0] in pps]
        mbsz = {pp: (lane(pp) + chunk - 1) // chunk for pp in pps}
        # strict: the chunk count searched must be the one these micro-batch sizes really give
        cand = [s for s in cand if chunk == (lane(s[0]) + mbsz[s[0]] - 1) // mbsz[s[0]]]
        if not cand:
            return None
        stage = get_pp_stage_for_bsz(cand, self.model_args_list, self.train_args_list, self.parallel_args_list,
                                     self.profile_model_args_list, self.layernum_list, bsz, mbsz)
        return cand, mbsz, stage

    def parallelism_optimization(self, one_batch=True, print_=False):
        """Runs the sweep; returns the best throughput (samples/s), -1 when nothing fits.  The nested
        ``results[bsz][chunk][min_tp][max_tp][vsp][embed_sdp][sp_search]`` dict of the reference is kept
        in ``self.results``, the winner in ``self.optimal``; the result file is written when there is
        a winner.  ``one_batch=False`` solves task by task (the reference's schedule)."""
        self.set_searching_bsz()
        sp_searches = self._spaces()[4]
        strategies_backup = self.strategies
        self.strategies = copy.deepcopy(self.strategies)
        pending = []               # (task, sp_search, DpOnModel, ticket, first instance, number of instances, stage)
        all_dps = []
        row_cache = {}             # intra-layer time rows, shared by the DpOnModel objects of this sweep
        # The device solves what has been prepared so far while the next tasks are being prepared: the
        # instances go to a worker thread in parts of at least `part` (the library call releases the
        # interpreter lock while the device works).
        part = self.overlap_part if one_batch else 0
        solved, sent = [], 0       # futures of the parts, instances handed over so far
        pool = None
        if part:
            from concurrent.futures import ThreadPoolExecutor
            pool = ThreadPoolExecutor(1)
        try:
            for task in self.tasks():
                bsz, chunk, min_tp, max_tp, vsp, embed_sdp = task
                for sp_search in sp_searches:
                    if (sp_search == 1 and vsp == 1) or (sp_search == 2 and vsp == 0):
                        continue
                    picked = self._task_strategies(bsz, chunk, min_tp, max_tp, sp_search)
                    if picked is None:
                        continue
                    cand, mbsz, stage = picked
                    model = self._dp_on_model(cand, stage)
                    model.row_cache = row_cache
                    check_optimal_chunks(self.args.gpu_num, cand, self.optimal_chunk_func, bsz, mbsz, min_tp)
                    ticket, dps = model.fit_begin(bsz, min_tp, max_tp, vsp, embed_sdp, sp_search, mbsz_dict=mbsz)
                    pending.append((task, sp_search, model, ticket, len(all_dps), len(dps), stage))
                    all_dps += dps
                    if pool is not None and len(all_dps) - sent >= part:
                        solved.append(pool.submit(DPAlg.fit_many, all_dps[sent:]))
                        sent = len(all_dps)
            self.solved_instances = len(all_dps)
            if pool is not None:
                if sent < len(all_dps):
                    solved.append(pool.submit(DPAlg.fit_many, all_dps[sent:]))
                fits = []
                for f in solved:
                    fits += f.result()
            elif one_batch:
                fits = DPAlg.fit_many(all_dps)
            else:
                fits = []
                for _, _, _, _, first, count, _ in pending:
                    fits += DPAlg.fit_many(all_dps[first:first + count])
        finally:
            # whatever happened while the tasks were prepared or solved: no worker is left solving on the
            # device, and the engine holds its own strategy list again
            if pool is not None:
                pool.shutdown(wait=True, cancel_futures=True)
            self.strategies = strategies_backup
        if not self.keep_device_cache:
            # the library keeps the device allocations of finished batches for the next one; a search is
            # usually the last thing its process asks of the device, so they are handed back here
            _lib.cache_trim()

        results = {}
        for bsz, chunk, min_tp, max_tp, vsp, embed_sdp in self.tasks():        # the reference's empty levels
            results.setdefault(bsz, {}).setdefault(chunk, {}).setdefault(min_tp, {}).setdefault(max_tp, {}) \
                .setdefault(vsp, {}).setdefault(embed_sdp, {})
        for task, sp_search, model, ticket, first, count, stage in pending:
            bsz, chunk, min_tp, max_tp, vsp, embed_sdp = task
            cost, res_list, pp_deg, remain, mem_cost, vtp = model.fit_end(ticket, fits[first:first + count], print_)
            results[bsz][chunk][min_tp][max_tp][vsp][embed_sdp][sp_search] = {
                'min_cost': cost, 'min_res_list': res_list, 'min_pp_deg': pp_deg, 'mem_remain': remain,
                'mem_cost': mem_cost, 'throughput': bsz / cost, 'vtp': vtp, 'pp_stage_dict': copy.deepcopy(stage)}
        self.results = results

        best, where = -1, None
        for bsz, by_chunk in results.items():
            for chunk, by_min in by_chunk.items():
                for min_tp, by_max in by_min.items():
                    for max_tp, by_vsp in by_max.items():
                        for vsp, by_sdp in by_vsp.items():
                            for embed_sdp, by_sp in by_sdp.items():
                                for sp_search, entry in by_sp.items():
                                    if entry['throughput'] > best:
                                        best = entry['throughput']
                                        where = (bsz, chunk, min_tp, max_tp, vsp, embed_sdp, sp_search)
        self.optimal = None
        if best > 0:
            bsz, chunk, min_tp, max_tp, vsp, embed_sdp, sp_search = where
            entry = results[bsz][chunk][min_tp][max_tp][vsp][embed_sdp][sp_search]
            entry['vsp'], entry['embed_sdp'] = vsp, embed_sdp
            self.optimal = dict(bsz=bsz, chunk=chunk, min_tp=min_tp, max_tp=max_tp, vsp=vsp, embed_sdp=embed_sdp,
                                sp_search=sp_search, result=entry)
            self.save_results(entry, bsz, chunk, entry['pp_stage_dict'])
        return best

    # ---- result file (search_engine.py:640-688) --------------------------------------------------------
    def result_config(self, re, bsz, chunk, pp_stage_dict):
        """The dict that goes into galvatron_config_*.json, or None when there is no valid result."""
        if not (re['min_pp_deg'] > 0 and re['min_res_list'] is not None):
            return None
        layers = re['min_res_list']
        if isinstance(layers, list) and isinstance(layers[0], list) and isinstance(layers[0][0], list):
            layers = [s for stage in layers for s in stage]
        config = strategy2config(layers)
        config['checkpoint'] = array2str([1 if s[-1].get('cpt') else 0 for s in layers])
        config['global_bsz'] = bsz
        config['chunks'] = chunk
        config['pp_division'] = array2str(pp_stage_dict[config['pp_deg']])
        config['pipeline_type'] = self.args.pipeline_type
        config['default_dp_type'] = self.args.default_dp_type
        config['vtp'] = re['vtp']
        config['vsp'] = re['vsp']
        config['embed_sdp'] = re['embed_sdp']
        return config

    def result_path(self):
        args = self.args
        off = [name for name, flag in (('dp', args.disable_dp), ('tp', args.disable_tp), ('pp', args.disable_pp),
                                       ('sdp', args.disable_sdp), ('ckpt', args.disable_ckpt),
                                       ('tpconsec', args.disable_tp_consec)) if flag]
        name = 'galvatron_config_%s_%dnodes_%dgpus_per_node_%dGB' % (self.model_name, args.num_nodes,
                                                                     args.num_gpus_per_node,
                                                                     self.memory_constraint // 1024)
        name += '_%s' % args.mixed_precision
        name += '_bsz%d' % args.settle_bsz if args.settle_bsz > 0 else ''
        name += '_[%s_off]' % '_'.join(off) if off else ''
        folder = args.output_config_path
        if folder is None:
            folder = os.path.join(self.path, 'configs/')
        return os.path.join(folder, name + '.json')

    def save_results(self, results, bsz, chunk, pp_stage_dict):
        config = self.result_config(results, bsz, chunk, pp_stage_dict)
        if config is None:
            return None
        path = self.result_path()
        with open(path, 'w') as fp:
            json.dump(config, fp, indent=4)
        return path
