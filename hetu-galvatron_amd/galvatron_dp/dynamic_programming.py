"""Host-side counterpart of the reference's ``dynamic_programming.py``
(galvatron/core/search_engine/dynamic_programming.py): ``DPAlg`` and ``DpOnModel`` with the
reference's constructor arguments, call signatures and return values, running the layer-wise DP
on the MI355X.

What differs is where the work goes.  The reference builds one ``DPAlg`` per pipeline stage and
calls the plugin once per stage; here every stage of every pipeline degree that one
``DpOnModel.fit`` looks at is collected first and solved in ONE device batch
(``galvatron_dp_core.dynamic_programming_core_batch``), and the O(S^2) pairwise inter-layer cost
table is built once per (pp_deg, layer type) from per-strategy feature vectors.

``memcost_model`` / ``timecost_model`` are passed in exactly as the reference passes them
(dynamic_programming.py:129-150); ``OtherTimeCostModel`` and ``pipeline_costmodel`` (which the
reference imports from its own cost_model.py, :3-4) are taken from the ``other_timecost_model`` /
``pipeline_costmodel`` keyword arguments and default to ``galvatron_dp.cost_models``.
"""
from __future__ import annotations

import numpy as np

import galvatron_dp_core
from . import cost_models

__all__ = ["DPAlg", "DpOnModel"]


class DPAlg:
    """One DP instance.  Same arguments, attributes and ``fit`` return value
    ``(total_cost, res_list, remaining_mem)`` -- three dicts keyed like ``other_mem_cost`` -- as the
    reference class (dynamic_programming.py:7-94).  ``_f`` / ``_mark`` are only materialised when the
    plugin is asked to export them (``galvatron_dp_core.set_export(True)``)."""

    def __init__(self, max_mem=8200, other_mem_cost=None, other_time_cost=None, layer_num=24, strategy_num=4,
                 strategy_set=None, fine_grained_mode=True, use_cpp_core=True) -> None:
        assert other_mem_cost is not None
        self.max_mem = max_mem + 1                      # number of budget bins (dynamic_programming.py:10)
        self.layer_num = layer_num
        self.strategy_num = strategy_num
        self.other_mem_cost = other_mem_cost
        self.other_time_cost = other_time_cost
        self.v_data = None
        self.inter_cost = None
        self.intra_cost = None
        self.use_cpp_core = use_cpp_core
        self.strategy_set = strategy_set
        self.fine_grained_mode = fine_grained_mode
        self._f = None
        self._mark = None

    def set_v_and_cost(self, v: np.ndarray, intra_layer_cost: np.ndarray, inter_layer_cost: np.ndarray):
        assert v.ndim == 2 and intra_layer_cost.ndim == 2 and inter_layer_cost.ndim == 3
        assert v.shape == (self.layer_num, self.strategy_num)
        assert intra_layer_cost.shape == (self.layer_num, self.strategy_num)
        assert inter_layer_cost.shape == (self.layer_num, self.strategy_num, self.strategy_num)
        self.v_data = v.astype(np.int32)
        self.inter_cost = inter_layer_cost
        self.intra_cost = intra_layer_cost

    def set_v_and_cost_shared(self, v: np.ndarray, intra_layer_cost: np.ndarray, inter_tables: np.ndarray,
                              inter_index: np.ndarray):
        """``set_v_and_cost`` for layers that share a few transition matrices: ``inter_tables`` [T,S,S]
        and ``inter_index`` [L] instead of the dense [L,S,S] array (which would repeat each matrix once
        per layer on the host, in the upload and in device memory).  Fine-grained mode only."""
        assert self.fine_grained_mode
        assert v.shape == (self.layer_num, self.strategy_num) and intra_layer_cost.shape == v.shape
        assert inter_tables.ndim == 3 and inter_tables.shape[1:] == (self.strategy_num, self.strategy_num)
        assert inter_index.shape == (self.layer_num,)
        self.v_data = v.astype(np.int32)
        self.inter_cost = galvatron_dp_core.SharedInter(inter_tables, inter_index)
        self.intra_cost = intra_layer_cost

    # -- coarse mode: one strategy for the whole stage, closed form (dynamic_programming.py:62-75) ----
    def _fit_coarse(self):
        keys = list(self.other_mem_cost)
        res_list = {k: np.full(self.layer_num, -1, dtype=np.int32) for k in keys}
        total_cost = {k: np.inf for k in keys}
        remaining_mem = {k: -1 for k in keys}
        for k in keys:
            for i in range(self.strategy_num):
                if self.strategy_set[i][1] != k:
                    continue
                # plain left-to-right sums, as the builtin sum() over array elements gives
                time_cost = sum(self.intra_cost[:, i]) + sum(self.inter_cost[:, i, i]) + self.other_time_cost[k]
                mem_cost = sum(self.v_data[:, i]) + self.other_mem_cost[k]
                if self.max_mem - 1 - mem_cost >= 0 and total_cost[k] > time_cost:
                    remaining_mem[k] = self.max_mem - 1 - mem_cost
                    total_cost[k] = time_cost
                    res_list[k] = np.full(self.layer_num, i, dtype=np.int32)
        return total_cost, res_list, remaining_mem

    def plugin_call(self):
        """The eleven positional arguments of the plugin call for this instance
        (dynamic_programming.py:79-91), with a fresh ``res_list``."""
        res_list = {k: np.full(self.layer_num, -1, dtype=np.int32) for k in self.other_mem_cost}
        if galvatron_dp_core.export_enabled():
            self._f = np.full((self.max_mem, self.strategy_num), 0, dtype=np.float64)
            self._mark = np.full((self.layer_num, self.max_mem, self.strategy_num), -1, dtype=np.int32)
        return (self.layer_num, self.max_mem, self.strategy_num, self.v_data, self._mark, self._f, self.inter_cost,
                self.intra_cost, self.other_mem_cost, self.other_time_cost, res_list)

    @staticmethod
    def _wrap(call, out):
        total_cost, remaining_mem = out
        return total_cost, {k: list(v) for k, v in call[10].items()}, remaining_mem

    def fit(self):
        if not self.fine_grained_mode:
            return self._fit_coarse()
        call = self.plugin_call()
        return self._wrap(call, galvatron_dp_core.dynamic_programming_core(*call))

    @classmethod
    def fit_many(cls, dps):
        """``[dp.fit() for dp in dps]`` with all fine-grained instances in one device batch."""
        out = [None] * len(dps)
        idx, calls = [], []
        for n, dp in enumerate(dps):
            if dp.fine_grained_mode:
                idx.append(n)
                calls.append(dp.plugin_call())
            else:
                out[n] = dp._fit_coarse()
        if calls:
            for n, call, res in zip(idx, calls, galvatron_dp_core.dynamic_programming_core_batch(calls)):
                out[n] = cls._wrap(call, res)
        return out


def _same_strategy(a, b, ignore=()):
    """Equal (pp, tp, dp) and equal option dictionaries apart from the keys in ``ignore``
    (the reference's ``match_strategy``, dynamic_programming.py:196-210)."""
    if not np.array_equal(a[:3], b[:3]):
        return False
    da, db = a[-1], b[-1]
    for key in set(da) | set(db):
        if key in ignore:
            continue
        if key not in da or key not in db or da[key] != db[key]:
            return False
    return True


_INTER_STRUCTURES = {}


def _inter_structure(strategy_set, sequence_parallel):
    """What the pairwise inter-layer cost of a strategy set owes to the strategies alone
    (dynamic_programming.py:292-367): ``big`` max(tp_i, tp_j); ``redistribute`` the pairs whose
    activations have to be re-laid out; ``coe_picks`` [(group size, layout flag or None, mask)] naming the
    collective coefficient each pair takes; ``bias`` / ``has_bias`` the tiny ordering biases between
    strategies that differ only in sp / fsdp / cpt, later rules overriding earlier ones as in the
    reference.  Kept per strategy set (a sweep builds the same few sets hundreds of times)."""
    key = (tuple((int(st[0]), int(st[1]), int(st[2]), tuple(sorted(st[-1].items()))) for st in strategy_set),
           sequence_parallel)
    hit = _INTER_STRUCTURES.get(key)
    if hit is not None:
        return hit
    S = len(strategy_set)
    tp = np.array([s[1] for s in strategy_set], dtype=np.int64)
    dp = np.array([s[2] for s in strategy_set], dtype=np.int64)
    has_tp = np.array(['tp' in s[-1] for s in strategy_set])
    tp_flag = np.array([s[-1].get('tp', -1) for s in strategy_set], dtype=np.int64)
    tp_i, tp_j = tp[:, None], tp[None, :]
    both = has_tp[:, None] & has_tp[None, :]
    differ = tp_flag[:, None] != tp_flag[None, :]
    redistribute = tp_j > tp_i
    redistribute |= both & (tp_j == tp_i) & differ
    redistribute |= both & ((tp * dp)[:, None] == 8) & (tp_i == 4) & (tp_j == 2) & differ
    if sequence_parallel:
        redistribute |= tp_j != tp_i
    big = np.maximum(tp_i, tp_j)
    # communication coefficient of the wider of the two tensor-parallel groups: the plain one when
    # that group is everything (or there is no data parallelism beside it), else by the layout
    # flag of the strategy that owns the wider group
    small_dp = np.minimum(dp[:, None], dp[None, :])
    plain = (big == 1) | (small_dp == 1)
    owner_flag = np.where(tp_j > tp_i, tp_flag[None, :], tp_flag[:, None])
    assert np.isin(owner_flag[~plain], (0, 1)).all()
    coe_picks = []
    for t in np.unique(big):
        t = int(t)
        here = big == t
        if (here & plain).any():
            coe_picks.append((t, None, here & plain))
        for flag in (0, 1):
            pick = here & ~plain & (owner_flag == flag)
            if pick.any():
                coe_picks.append((t, flag, pick))

    # "Same apart from key k" (the reference's match_strategy, dynamic_programming.py:196-210) is
    # equality of (pp, tp, dp) and of the option dictionaries with k removed.
    def same_apart_from(*ignore):
        ids, seen = [], {}
        for st in strategy_set:
            k = (tuple(int(x) for x in st[:3]), frozenset((a, b) for a, b in st[-1].items() if a not in ignore))
            ids.append(seen.setdefault(k, len(seen)))
        ids = np.array(ids)
        return ids[:, None] == ids[None, :]

    on = lambda name: np.array([bool(st[-1].get(name)) for st in strategy_set])       # noqa: E731
    sp_j, fsdp_j, cpt_j, fsdp_i = on('sp')[None, :], on('fsdp')[None, :], on('cpt')[None, :], on('fsdp')[:, None]
    off_diagonal = ~np.eye(S, dtype=bool)
    only_fsdp, only_cpt, both_keys = same_apart_from('fsdp'), same_apart_from('cpt'), same_apart_from('fsdp', 'cpt')
    bias = np.full((S, S), np.nan)
    bias[off_diagonal & same_apart_from('sp') & sp_j] = 1e-10
    bias[off_diagonal & only_fsdp & fsdp_j] = 1e-9
    bias[off_diagonal & only_cpt & cpt_j] = 2e-9
    bias[off_diagonal & both_keys & fsdp_j & cpt_j] = 3e-9
    bias[off_diagonal & both_keys & ~only_fsdp & ~only_cpt & fsdp_i & cpt_j] = 1e-9
    hit = {"big": big, "redistribute": redistribute, "coe_picks": coe_picks, "has_bias": ~np.isnan(bias),
           "bias": np.nan_to_num(bias)}
    if len(_INTER_STRUCTURES) > 4096:
        _INTER_STRUCTURES.clear()
    _INTER_STRUCTURES[key] = hit
    return hit


class _Prepared:
    """Everything one pipeline degree contributes to the batch: the DP instances of its stages and
    what is needed to turn their results into the reference's return tuple."""
    __slots__ = ("pp_deg", "bsz", "mbsz", "min_tp", "strategy_set", "min_cost_strategy_ids", "other_mem_cost",
                 "other_time_cost", "pp_stage_list", "dps", "local_sets", "chunks", "coarse")


class DpOnModel:
    """Same constructor arguments as the reference (dynamic_programming.py:129-150) plus the two
    callables the reference imports from its cost_model.py (default: this package's)."""

    def __init__(self, strategies_set, memcost_model, timecost_model, model_args_list=None, train_args_list=None,
                 parallel_args_list=None, profile_model_args_list=None, profile_hardware_args_list=None,
                 max_mem=8192, layer_num=24, sequence_len=[512], multi_layer_type=False, pp_stage_dict=None,
                 search_history=None, comm_coe_dict={}, gpu_num=8, mem_cache=True, model_microbatch_after_dp=False,
                 pipeline_type='gpipe', config=None, logger=None, other_timecost_model=None,
                 pipeline_costmodel=None):
        self.strategies_set = strategies_set
        self.memcost_model = memcost_model
        self.timecost_model = timecost_model
        self.other_timecost_model = other_timecost_model or cost_models.OtherTimeCostModel
        self.pipeline_costmodel = pipeline_costmodel or cost_models.pipeline_costmodel
        self.model_args_list = model_args_list
        self.train_args_list = train_args_list
        self.parallel_args_list = parallel_args_list
        self.profile_model_args_list = profile_model_args_list
        self.profile_hardware_args_list = profile_hardware_args_list
        self.max_mem = max_mem
        self.layer_num = layer_num
        self.sequence_len = sequence_len
        self.n_gpu = strategies_set[0][0] * strategies_set[0][1] * strategies_set[0][2]
        self.ppdeg_set = np.unique(np.array([s[0] for s in strategies_set], dtype=np.int32))
        self.multi_layer_type = multi_layer_type
        self.search_history = search_history
        self.comm_coe_dict = comm_coe_dict
        self.gpu_num = gpu_num
        self.config = config
        self.logger = logger
        if multi_layer_type:
            lists = (model_args_list, train_args_list, parallel_args_list, profile_model_args_list,
                     profile_hardware_args_list)
            assert isinstance(layer_num, list)
            self.total_layer_num = sum(layer_num)
            assert all(isinstance(x, list) and len(x) == len(layer_num) for x in lists)
            assert isinstance(pp_stage_dict, dict)
            for ppdeg in self.ppdeg_set:
                if ppdeg > 1:
                    assert ppdeg in pp_stage_dict and sum(pp_stage_dict[ppdeg]) == self.total_layer_num
            self.pp_stage_dict = pp_stage_dict
            if 1 not in self.pp_stage_dict:
                self.pp_stage_dict[1] = [self.total_layer_num]
        self.mem_cache = 0
        if max_mem // 1024 > 20 and mem_cache:
            self.mem_cache = int(max_mem * 0.2)          # reserved for the framework's allocator cache (:190-193)
            self.max_mem -= self.mem_cache
        self.model_microbatch_after_dp = model_microbatch_after_dp
        self.pipeline_type = pipeline_type
        # Optional (no counterpart in the reference): a dict shared by the DpOnModel objects of one sweep,
        # which all hold the SAME strategy lists and argument records.  Rows of intra-layer times are
        # then computed once per (strategies, batch size, layer type) instead of once per task.
        self.row_cache = None

    def match_strategy(self, s1, s2, except_keys=[]):
        return _same_strategy(s1, s2, tuple(except_keys))

    # ---- inputs of the DP -------------------------------------------------------------------------
    def _model_kwargs(self, i):
        return dict(model_args=self.model_args_list[i], train_args=self.train_args_list[i],
                    parallel_args=self.parallel_args_list[i], profile_model_args=self.profile_model_args_list[i])

    def _intra_cost(self, strategy_set, bsz, chunks):
        """[L,S] time of a layer under each strategy (dynamic_programming.py:228-245).  With this
        package's own time model the S values of a layer type come out of one array evaluation
        (``cost_models.time_cost_rows``, the same bits); any other model is called per strategy."""
        blocks = []
        for i, n in enumerate(self.layer_num):
            b = bsz / chunks[i] if self.model_microbatch_after_dp else bsz
            row = None
            key = None
            if self.row_cache is not None:
                # the strategy lists and records are the sweep's own objects (kept alive by the entry)
                key = ("time", tuple(map(id, strategy_set)), b, i, id(self.timecost_model),
                       id(self.profile_hardware_args_list[i]), id(self.model_args_list[i]), id(self.train_args_list[i]),
                       id(self.parallel_args_list[i]), id(self.profile_model_args_list[i]))
                hit = self.row_cache.get(key)
                if hit is not None:
                    blocks.append(hit[0].reshape(1, -1).repeat(n, axis=0))
                    continue
            if self.timecost_model is cost_models.TimeCostModel:
                try:
                    row = cost_models.time_cost_rows(strategy_set, b,
                                                     profile_hardware_args=self.profile_hardware_args_list[i],
                                                     **self._model_kwargs(i))
                except cost_models.NotVectorisable:
                    row = None
            if row is None:
                row = [self.timecost_model(s, b, profile_hardware_args=self.profile_hardware_args_list[i],
                                           logger=self.logger, **self._model_kwargs(i)).gen_result() for s in strategy_set]
            row = np.array(row, dtype=np.float64)
            if key is not None:
                self.row_cache[key] = (row, list(strategy_set), self.profile_hardware_args_list[i], self.model_args_list[i],
                                       self.train_args_list[i], self.parallel_args_list[i], self.profile_model_args_list[i])
            blocks.append(row.reshape(1, -1).repeat(n, axis=0))
        return np.concatenate(blocks, axis=0)

    def _memory_rows(self, strategy_set, i, bsz, mbsz, min_tp, max_tp, vsp, embed_sdp, stage_ids):
        """(enc_total [stages, S], 'other' of the first strategy on the first stage) for layer type
        ``i``: one array evaluation with this package's own memory model, one object per strategy and
        stage otherwise.  ``stage_ids`` is ``[None]`` where the stage does not matter (gpipe)."""
        if self.memcost_model is cost_models.MemoryCostModel:
            key = None
            if self.row_cache is not None:
                # the rows depend on neither max_tp nor vsp nor embed_sdp: a sweep that walks through those
                # keeps them and recomputes the 'other' entry alone
                key = ("mem", tuple(map(id, strategy_set)), bsz, mbsz, min_tp, tuple(stage_ids), i,
                       id(self.model_args_list[i]), id(self.train_args_list[i]), id(self.parallel_args_list[i]),
                       id(self.profile_model_args_list[i]))
                hit = self.row_cache.get(key)
                if hit is not None:
                    other = cost_models.memory_cost_other(strategy_set, bsz, mbsz, min_tp, max_tp, vsp=vsp,
                                                          embed_sdp=embed_sdp, **self._model_kwargs(i)) if i == 0 else None
                    return hit[0], other
            try:
                rows, other = cost_models.memory_cost_rows(
                    strategy_set, bsz, mbsz, min_tp, max_tp, vsp=vsp, embed_sdp=embed_sdp,
                    stage_idx=[0 if x is None else x for x in stage_ids], **self._model_kwargs(i))
                if key is not None:
                    self.row_cache[key] = (rows, list(strategy_set), self.model_args_list[i], self.train_args_list[i],
                                           self.parallel_args_list[i], self.profile_model_args_list[i])
                return rows, other
            except cost_models.NotVectorisable:
                pass
        rows, other = [], None
        for stage_idx in stage_ids:
            extra = {} if stage_idx is None else {"stage_idx": stage_idx}
            costs = [self.memcost_model(s, bsz, mbsz=mbsz, min_tp=min_tp, max_tp=max_tp, vsp=vsp, embed_sdp=embed_sdp,
                                        logger=self.logger, **extra, **self._model_kwargs(i)).get_memory_cost()
                     for s in strategy_set]
            rows.append([c['enc_total'] for c in costs])
            if other is None:
                other = costs[0]['other']
        return np.array(rows), other

    def _memory_cost(self, strategy_set, pp_deg, bsz, mbsz, min_tp, max_tp, vsp, embed_sdp):
        """Per-stage [L,S] memory tables (ceil MB, int32) and the ``other`` memory of the first layer
        type (dynamic_programming.py:254-288)."""
        other_mem_cost = {}
        stage_ids = [None] if self.pipeline_type == "gpipe" else list(range(pp_deg))
        per_type = []
        for i, n in enumerate(self.layer_num):
            enc_total, other = self._memory_rows(strategy_set, i, bsz, mbsz, min_tp, max_tp, vsp, embed_sdp, stage_ids)
            if i == 0:
                for k, val in other.items():
                    other_mem_cost[k] = np.ceil(val).astype(int)
            per_type.append(np.ceil(enc_total).astype(np.int32))          # [stages, S]
        tables = [np.concatenate([rows[j].reshape(1, -1).repeat(n, axis=0) for rows, n in zip(per_type, self.layer_num)],
                                 axis=0) for j in range(len(stage_ids))]
        if self.pipeline_type == "gpipe":
            return [tables[0]] * pp_deg, other_mem_cost
        return tables, other_mem_cost

    def _inter_matrix(self, strategy_set, idx, mbsz, min_tp):
        """[S,S] cost of switching from strategy i (row) to strategy j (column) between two layers
        of type ``idx`` (dynamic_programming.py:292-367).  What depends on the strategies alone --
        which pairs redistribute, which collective coefficient a pair takes, which pairs get one of
        the tiny ordering biases -- is worked out once per strategy set (``_inter_structure``, kept
        for the whole sweep); a call adds the volumes and coefficients."""
        st = _inter_structure(strategy_set, bool(self.config.sequence_parallel))
        big = st["big"]
        sample_num = self.sequence_len[idx] * self.config.hidden_size * (4 if self.config.mixed_precision == "fp32" else 2)
        volume = (big - 1) / big * mbsz * (big // min_tp) * sample_num      # same order of operations
        cost = np.where(st["redistribute"], volume, 0.0)
        coe = np.empty(big.shape, dtype=np.float64)
        table = self.comm_coe_dict
        for t, flag, pick in st["coe_picks"]:
            if flag is None:
                coe[pick] = table['%d' % t] if '%d' % t in table else table['%d_1' % t]
            else:
                coe[pick] = table['%d_%d' % (t, flag)]
        cost = cost * coe * 1e-7
        return np.where(st["has_bias"], st["bias"], cost)

    def _inter_tables(self, strategy_set, mbsz, min_tp):
        """The transition matrices of one pipeline degree as the device takes them: ``tables``
        [1 + layer types, S, S] -- matrix 0 is all zeros, for the first layer of the model, which has no
        switch before it (dynamic_programming.py:372) -- and ``index`` [L] naming every layer's matrix."""
        S = len(strategy_set)
        key = None
        if self.row_cache is not None:
            key = ("inter", tuple(map(id, strategy_set)), mbsz, min_tp, id(self.comm_coe_dict), id(self.config),
                   tuple(self.sequence_len), tuple(self.layer_num))
            hit = self.row_cache.get(key)
            if hit is not None:
                return hit[0], hit[1]
        tables = np.zeros((1 + len(self.layer_num), S, S), dtype=np.float64)
        index = []
        for idx, n in enumerate(self.layer_num):
            tables[1 + idx] = self._inter_matrix(strategy_set, idx, mbsz, min_tp)
            index += [1 + idx] * n
        index = np.array(index, dtype=np.int32)
        index[0] = 0
        if key is not None:
            self.row_cache[key] = (tables, index, list(strategy_set), self.comm_coe_dict, self.config)
        return tables, index

    def _inter_cost(self, strategy_set, mbsz, min_tp):
        """The same as one dense [L,S,S] array, the reference's layout (dynamic_programming.py:289-372)."""
        tables, index = self._inter_tables(strategy_set, mbsz, min_tp)
        return tables[index]

    def _global_memory(self, mbsz, min_tp, max_tp, sp_search, coarse):
        cfg = self.config
        use = cfg.sequence_parallel if coarse else (cfg.sequence_parallel and cfg.global_memory_buffer and sp_search != 2)
        if not use:
            return 0
        g = mbsz / min_tp * max_tp * cfg.hidden_size * max(self.sequence_len) * 4 / 1024 / 1024
        if cfg.mixed_precision:
            g = g / 2
        return g

    def _prepare(self, pp_deg, bsz, mbsz, min_tp, max_tp, vsp, embed_sdp, sp_search):
        P = _Prepared()
        P.pp_deg, P.bsz, P.mbsz, P.min_tp = pp_deg, bsz, mbsz, min_tp
        P.chunks = None
        if self.model_microbatch_after_dp:
            dp_size = self.gpu_num // pp_deg
            P.chunks = [pa.optimal_chunk_func(bsz * min_tp // dp_size, [pp_deg, min_tp, dp_size], mbsz, min_tp)
                        for pa in self.parallel_args_list]
        strategy_set = [s for s in self.strategies_set if s[0] == pp_deg]
        P.strategy_set = strategy_set
        S = len(strategy_set)
        intra = self._intra_cost(strategy_set, bsz, P.chunks)
        P.min_cost_strategy_ids = np.argmin(intra, axis=1)
        P.other_time_cost = self.other_timecost_model(
            mbsz, pp_deg, self.n_gpu, vsp, embed_sdp, min_tp, max_tp, self.sequence_len,
            model_args=self.model_args_list[0], train_args=self.train_args_list[0],
            parallel_args=self.parallel_args_list[0], profile_model_args=self.profile_model_args_list[0],
            profile_hardware_args=self.profile_hardware_args_list[0], logger=self.logger).gen_result()
        v_stage, P.other_mem_cost = self._memory_cost(strategy_set, pp_deg, bsz, mbsz, min_tp, max_tp, vsp, embed_sdp)
        tables, index = self._inter_tables(strategy_set, mbsz, min_tp)
        P.pp_stage_list = self.pp_stage_dict[pp_deg]
        P.coarse = self.config.fine_grained_mode == 0
        gmem = int(self._global_memory(mbsz, min_tp, max_tp, sp_search, P.coarse))
        P.dps, P.local_sets = [], []
        columns = [[si] for si in range(S)] if P.coarse else [list(range(S))]
        inter = tables[index] if P.coarse else None      # dense only where single columns are cut out of it
        for cols in columns:                             # coarse mode: one single-strategy DP per strategy
            start = 0
            local = [strategy_set[c] for c in cols]
            for i in range(pp_deg):
                n = P.pp_stage_list[i]
                other_mem = {k: v[i] + gmem for k, v in P.other_mem_cost.items()}
                other_time = {k: v[i] for k, v in P.other_time_cost[0].items()}
                dp = DPAlg(self.max_mem, other_mem, other_time, n, len(cols), local, self.config.fine_grained_mode)
                rows = slice(start, start + n)
                if P.coarse:
                    dp.set_v_and_cost(v_stage[i][rows][:, cols], intra[rows][:, cols],
                                      inter[rows][:, cols][:, :, cols])
                else:                                    # every stage of the pipeline degree shares the tables
                    dp.set_v_and_cost_shared(v_stage[i][rows], intra[rows], tables, index[rows])
                P.dps.append(dp)
                start += n
            P.local_sets.append(local)
        return P

    # ---- from DP results to the reference's return tuple ------------------------------------------
    def _stage_results(self, P, fits, local_set):
        comm_cost_list, res_list_list, mem_remain_list, mem_cost_list = [], [], [], []
        best_strategy_flag = {}
        start = 0
        for i, (comm_cost, res_list, mem_remain) in enumerate(fits):
            n = P.pp_stage_list[i]
            mem_cost = {k: 0 for k in P.other_time_cost[0]}
            for k in comm_cost:
                if mem_remain[k] == -1:
                    res_list[k] = None
                flag = res_list[k] is not None and \
                    (np.array(res_list[k]) == P.min_cost_strategy_ids[start:start + n]).all()
                best_strategy_flag.setdefault(k, [False] * P.pp_deg)[i] = flag
                if res_list[k] is not None:
                    res_list[k] = [local_set[x] for x in res_list[k]]
                mem_cost[k] = self.max_mem - mem_remain[k] if mem_remain[k] >= 0 else np.inf
            comm_cost_list.append(comm_cost)
            res_list_list.append(res_list)
            mem_remain_list.append(mem_remain)
            mem_cost_list.append(mem_cost)
            start += n
        return comm_cost_list, res_list_list, mem_remain_list, mem_cost_list, best_strategy_flag

    def _pipeline_cost(self, P, per_stage_res, k):
        flat = []
        for r in per_stage_res:
            flat += r
        extra = {}
        if self.row_cache is not None and self.pipeline_costmodel is cost_models.pipeline_costmodel:
            extra["cache"] = self.row_cache       # this package's own model: per-strategy times kept across the sweep
        return self.pipeline_costmodel(self.timecost_model, self.layer_num, self.model_args_list, self.train_args_list,
                                       self.parallel_args_list, self.profile_model_args_list,
                                       self.profile_hardware_args_list, flat, P.pp_stage_list, P.chunks, P.bsz,
                                       P.min_tp, P.other_time_cost[1][k], self.logger, **extra)

    def _finish(self, P, fits):
        pp_deg = P.pp_deg
        from_history = None
        best_strategy_flag = {k: [False] * pp_deg for k in P.other_mem_cost}
        if P.coarse:                                    # dynamic_programming.py:379-444
            final_cost, vtp = np.inf, -1
            final_res, final_remain, final_memcost = [], [], []
            for si, local in enumerate(P.local_sets):
                stage_fits = fits[si * pp_deg:(si + 1) * pp_deg]
                comm, res, remain, memcost, flags = self._stage_results(P, stage_fits, local)
                for k, f in flags.items():
                    best_strategy_flag[k] = f
                for k in P.other_time_cost[0]:
                    per_stage = [r[k] for r in res]
                    if self.model_microbatch_after_dp:
                        if None not in per_stage:
                            cost = self._pipeline_cost(P, per_stage, k)
                            if final_cost > cost:
                                final_cost, vtp = cost, k
                                final_res = [r[vtp] for r in res]
                                final_remain = [r[vtp] for r in remain]
                                final_memcost = [r[vtp] for r in memcost]
                    else:
                        final_cost = sum(c[k] for c in comm)
            return final_cost, final_res, final_remain, final_memcost, vtp, best_strategy_flag, from_history
        comm, res, remain, memcost, flags = self._stage_results(P, fits, P.strategy_set)
        best_strategy_flag.update(flags)
        comm_cost, vtp = np.inf, -1
        for k in P.other_time_cost[0]:                  # dynamic_programming.py:489-506
            per_stage = [r[k] for r in res]
            if self.model_microbatch_after_dp:
                if None not in per_stage:
                    cost = self._pipeline_cost(P, per_stage, k)
                    if comm_cost > cost:
                        comm_cost, vtp = cost, k
            else:
                comm_cost = sum(c[k] for c in comm)
        if vtp != -1:
            res = [r[vtp] for r in res]
            remain = [r[vtp] for r in remain]
            memcost = [r[vtp] for r in memcost]
        else:
            res, remain, memcost = None, [-1 for _ in remain], [-1 for _ in memcost]
        return comm_cost, res, remain, memcost, vtp, best_strategy_flag, from_history

    def _build_dp_and_run_multi_layer_type(self, pp_deg, bsz, mbsz, min_tp, max_tp, vsp, embed_sdp, sp_search):
        """Same arguments and return tuple as the reference method (dynamic_programming.py:212,513):
        ``(comm_cost, res_list_list, mem_remain_list, mem_cost_list, vtp, best_strategy_flag, from_history)``."""
        P = self._prepare(pp_deg, bsz, mbsz, min_tp, max_tp, vsp, embed_sdp, sp_search)
        return self._finish(P, DPAlg.fit_many(P.dps))

    def _say(self, print_, *lines):
        if not print_:
            return
        for line in lines:
            if self.logger is not None:
                self.logger.info(line)
            else:
                print(line, flush=True)

    def fit_begin(self, bsz, min_tp, max_tp, vsp, embed_sdp, sp_search, mbsz_dict=None):
        """First half of ``fit``: prepares every pipeline degree and returns ``(ticket, dps)``.  The
        caller solves ``dps`` (``DPAlg.fit_many``, alone or together with the instances of other
        ``fit_begin`` calls: a whole sweep in one device batch) and hands the results to ``fit_end``."""
        if mbsz_dict is None:
            mbsz_dict = {pp_deg: 8 for pp_deg in self.ppdeg_set}
        todo = []
        for pp_deg in self.ppdeg_set:
            if pp_deg * min_tp > self.gpu_num:
                continue
            divisible = not (bsz % (self.gpu_num // (pp_deg * min_tp)))
            if divisible:
                assert self.multi_layer_type
            todo.append((pp_deg, self._prepare(pp_deg, bsz, mbsz_dict[pp_deg], min_tp, max_tp, vsp, embed_sdp,
                                               sp_search) if divisible else None))
        ticket = (todo, (bsz, min_tp, max_tp, vsp, embed_sdp, sp_search))
        return ticket, [dp for _, P in todo if P is not None for dp in P.dps]

    def fit_end(self, ticket, fits, print_=True):
        """Second half of ``fit``: ``fits`` are the results of the instances ``fit_begin`` returned, in
        the same order."""
        todo, (bsz, min_tp, max_tp, vsp, embed_sdp, sp_search) = ticket
        best = (np.inf, None, -1, -1, -1, -1)
        pos = 0
        for pp_deg, P in todo:
            self._say(print_, f'bsz={bsz}, pp_deg={pp_deg}, min_tp={min_tp}, max_tp={max_tp}, vsp={vsp}, '
                              f'embed_sdp={embed_sdp}, sp_search={sp_search}:')
            if P is None:
                if best[1] is None:
                    best = (best[0], '[current bsz is not divisible by bsz_scale]') + best[2:]
                self._say(print_, f'Best strategy: {False} \nFrom history: {False}',
                          f'time cost: {np.inf}, memory remaining: {-1}, memory cost: {np.inf}')
                continue
            mine = fits[pos:pos + len(P.dps)]
            pos += len(P.dps)
            comm_cost, res_list, mem_remain, mem_cost, vtp, best_strategy_flag, from_history = self._finish(P, mine)
            mem_cost = [m + self.mem_cache for m in mem_cost] if isinstance(mem_cost, list) else mem_cost + self.mem_cache
            self._say(print_, f'Best strategy: {best_strategy_flag} \nFrom history: {from_history}',
                      f'time cost: {comm_cost}, memory remaining: {mem_remain}, memory cost: {mem_cost}')
            if best[0] > comm_cost:
                best = (comm_cost, res_list, pp_deg, mem_remain, mem_cost, vtp)
        return best

    def fit(self, bsz, min_tp, max_tp, vsp, embed_sdp, sp_search, print_=True, mbsz_dict=None):
        """Same arguments and return value as the reference (dynamic_programming.py:515-565):
        ``(min_comm_cost, min_res_list, min_pp_deg, min_mem_remain, min_mem_cost, min_vtp)``.
        All pipeline degrees are prepared first and their DP instances solved in one device batch."""
        ticket, dps = self.fit_begin(bsz, min_tp, max_tp, vsp, embed_sdp, sp_search, mbsz_dict)
        return self.fit_end(ticket, DPAlg.fit_many(dps), print_)
