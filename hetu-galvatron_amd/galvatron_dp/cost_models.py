"""Per-layer memory / time cost models of the search engine: the producers of the DP's inputs
(``v``, ``intra``, ``other_mem_cost``, ``other_time_cost``) and the pipeline time model that picks
among the DP's results.

Counterpart of the reference's ``galvatron/core/search_engine/cost_model.py:10-767`` and
``cost_model_args.py:6-49``: same class names, constructor arguments, argument dataclasses and
returned values, so that ``DpOnModel`` (the reference's or ``galvatron_dp.dynamic_programming``'s)
can be handed these classes unchanged.  Every number is produced with the reference's order of
floating-point operations (the tests compare bit for bit against values recorded from the
reference).  Unlike the reference's classes, these do not copy the argument records into a
namespace and compute in stages: each constructor computes its terms straight from the records.

A strategy is ``[pp, tp, dp, flags]`` with flags ``fsdp`` (ZeRO-3), ``cpt`` (activation
checkpointing), ``sp`` (Ulysses sequence parallelism instead of tensor parallelism) and ``tp``
(whether the tensor-parallel group is made of consecutive ranks).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Optional, Union

import numpy as np

__all__ = ["ModelArgs", "TrainArgs", "ParallelArgs", "ProfileModelArgs", "ProfileHardwareArgs",
           "MemoryCostModel", "TimeCostModel", "OtherTimeCostModel", "pipeline_costmodel",
           "memory_cost_rows", "time_cost_rows", "NotVectorisable",
           "chunk_like_torch", "get_real_chunk", "get_time_cost_all_stages", "form_strategy",
           "strategy_str2list"]


# ---- argument records (cost_model_args.py:6-49: same fields, same defaults) ---------------------
@dataclass
class ModelArgs:
    parameter_size: int = 48
    seq_length: int = 1024
    hidden_size: int = 4096
    layer_num: int = 16


@dataclass
class TrainArgs:
    mixed_precision: bool = False
    checkpoint: bool = False
    async_grad_reduce: bool = True
    pytorch_context_mem: int = 1024


@dataclass
class ParallelArgs:
    use_zero2_for_dp: bool = False
    disable_vtp: bool = False
    sequence_parallel: bool = False
    sp_space: str = 'sp+tp'
    pipeline_type: str = 'gpipe'
    optimal_chunk_func: Optional[Callable] = None
    chunks: Optional[int] = None


@dataclass
class ProfileModelArgs:
    tp_activation_per_bsz_dict: dict = field(default_factory=lambda: {1: 85, 2: 47, 4: 28, 8: 18.5})
    other_memory_pp_off: dict = field(default_factory=lambda: {'model_states': 640, 'activation': 320})
    other_memory_pp_on: dict = field(default_factory=lambda: {
        'first_stage': {'model_states': 640, 'activation': 320},
        'last_stage': {'model_states': 640, 'activation': 320}})
    forward_computation_time: Optional[Union[float, np.ndarray]] = 35 / 24
    other_time_profiled: Optional[Union[float, np.ndarray]] = 0


@dataclass
class ProfileHardwareArgs:
    bct_fct_coe: float = 2
    extra_overhead: float = 0
    comm_coe_dict: dict = field(default_factory=lambda: {
        '8': 0.0062326653993580354, '4_0': 0.006042551648710218, '4_1': 0.006087464692704782,
        '2_0': 0.006496332820123041, '2_1': 0.006424794567193714, '1': 0})
    dp_overlap_coe: float = 1.3
    bct_overlap_coe: float = 1.3
    p2p_comm_coe_dict: dict = field(default_factory=lambda: {
        2: 0.006787944610371979, 4: 0.0074923765069042254, 8: 0.00920674670398468})
    allreduce_dict: dict = field(default_factory=lambda: {})
    all2all_dict: dict = field(default_factory=lambda: {})
    costmodel_coe: float = 1.0


# ---- small helpers --------------------------------------------------------------------------------
def _flag(strategy, name) -> bool:
    """A flag of the strategy's last element; absent means off."""
    return bool(strategy[-1].get(name, 0))


def _is_ulysses(strategy) -> bool:
    return strategy[-1].get('sp', 0) == 1


def _line(x, coefficients):
    """A profiled straight line ``m*x + c`` given as (m, c) (cost_model.py:303-305)."""
    m, c = coefficients
    return m * x + c


def _group_coe(table, size, consecutive=None):
    """Coefficient of a collective over ``size`` ranks from the profiled table, whose keys are
    '<size>' when there is one placement and '<size>_<0|1>' when the group can be laid out in two
    ways (cost_model.py:328-340)."""
    if consecutive is None:
        key = '%d' % size
        return table[key] if key in table else table['%d_1' % size]
    return table['%d_%d' % (size, consecutive)]


def chunk_like_torch(size, chunks):
    """The pieces ``torch.arange(size).chunk(chunks)`` would give, as index arrays
    (cost_model.py:661-678): pieces of ceil(size/chunks) until the range is used up."""
    if chunks <= 0:
        raise ValueError("chunks must be positive")
    step = (size + chunks - 1) // chunks
    pieces = []
    for i in range(chunks):
        lo = i * step
        if lo >= size:
            break
        pieces.append(np.arange(lo, min(lo + step, size)))
    return pieces


def get_real_chunk(local_bsz, chunk):
    """Number of micro-batches that asking for ``chunk`` of them really gives (cost_model.py:680-685)."""
    if chunk == 1:
        return 1
    return len(chunk_like_torch(int(local_bsz), int(chunk)))


def sum_like_numpy(values):
    """``np.sum`` of a short list of numbers, bit for bit, without the cost of turning it into an array
    (a sweep makes tens of thousands of such sums, a few microseconds each).  Up to seven elements numpy adds
    them from left to right; from eight on it adds in blocks, and the list goes through numpy itself."""
    n = len(values)
    if n > 7:
        return np.add.reduce(values)
    if n == 0:
        return np.float64(0.0)
    acc = 0                      # numpy starts from the identity: a lone -0.0 comes out as +0.0
    for x in values:
        acc = acc + x
    return acc if isinstance(acc, np.generic) else (np.int64(acc) if isinstance(acc, int) else np.float64(acc))


def get_time_cost_all_stages(layer_timecosts, pp_stage_division):
    """Sum of the layers' times per pipeline stage (cost_model.py:687-693)."""
    assert sum(int(x) for x in pp_stage_division) == len(layer_timecosts)
    out, first = [], 0
    for count in pp_stage_division:
        last = first + int(count)
        out.append(sum_like_numpy(layer_timecosts[first:last]))
        first = last
    return out


def form_strategy(strategy):
    """'pp-tp-dp' text of a strategy with its flags (galvatron/utils/strategy_utils.py:3-26):
    'f' after dp for fsdp, '*' after the consecutive one of tp / dp, then '-c', '-sp'."""
    assert len(strategy) == 4
    flags = strategy[-1]
    tp, dp = '%d' % strategy[1], '%d' % strategy[2]
    if flags.get('fsdp'):
        dp += 'f'
    if 'tp' in flags:
        if flags['tp']:
            tp += '*'
        else:
            dp += '*'
    if flags.get('cpt'):
        dp += '-c'
    if flags.get('sp'):
        dp += '-sp'
    return '%d-%s-%s' % (strategy[0], tp, dp)


def strategy_str2list(text):
    """Inverse of form_strategy (galvatron/utils/strategy_utils.py:28-59)."""
    part = text.split('-')
    consecutive = None
    if '*' in part[1]:
        consecutive, part[1] = 1, part[1][:-1]
    elif '*' in part[2]:
        consecutive, part[2] = 0, part[2][:-1]
    fsdp = 0
    if 'f' in part[2]:
        fsdp, part[2] = 1, part[2][:-1]
    cpt = 1 if len(part) >= 4 and part[3] == 'c' else 0
    sp = 1 if (len(part) >= 4 and part[3] == 'sp') or (len(part) >= 5 and part[4] == 'sp') else 0
    pp, tp, dp = int(part[0]), int(part[1]), int(part[2])
    flags = {}
    if tp > 1 and dp > 1:
        flags['tp'] = consecutive
    if dp > 1:
        flags['fsdp'] = fsdp
    if cpt:
        flags['cpt'] = 1
    if sp:
        flags['sp'] = 1
    return [pp, tp, dp, flags]


def _zero_ratios(chunks, mixed_precision, async_grad_reduce):
    """(zero2, zero3): share of the model states a rank keeps under ZeRO-2 / ZeRO-3 as functions of
    the sharding degree d (cost_model.py:99-110).  0.003 is the reference's safety margin; with
    gradient accumulation (chunks > 1) the gradients (and, synchronously, an fp32 copy: x5/4) stay
    whole."""
    shard = lambda d: 1 / d + 0.003                                  # noqa: E731
    if chunks == 1:
        zero2 = (lambda d: 7 / 8 * shard(d) + 1 / 8) if mixed_precision else (lambda d: 3 / 4 * shard(d) + 1 / 4)
        return zero2, shard
    if async_grad_reduce:
        zero2 = (lambda d: 6 / 8 * shard(d) + 2 / 8) if mixed_precision else (lambda d: 2 / 4 * shard(d) + 2 / 4)
        zero3 = (lambda d: 7 / 8 * shard(d) + 1 / 8) if mixed_precision else (lambda d: 3 / 4 * shard(d) + 1 / 4)
        return zero2, zero3
    zero2 = (lambda d: (7 / 8 * shard(d) + 1 / 8) * 5 / 4) if mixed_precision else (lambda d: 3 / 4 * shard(d) + 1 / 4)
    return zero2, (lambda d: shard(d) * 5 / 4)


# ---- memory -----------------------------------------------------------------------------------------
def _other_memory(strategy, chunks, zero2_ratio, zero3_ratio, global_batch_size, min_tp, max_tp, vsp, embed_sdp, train_args,
                  parallel_args, profile):
    """{vocab tp degree: [MB per pipeline stage]} of embedding / head / context
    (cost_model.py:140-210)."""
    pp, tp, dp = strategy[0], strategy[1], strategy[2]
    off, on = profile.other_memory_pp_off, profile.other_memory_pp_on
    if parallel_args.disable_vtp:
        degrees = [1]
    else:
        degrees, k = [], min_tp
        while k * pp <= strategy[0] * strategy[1] * strategy[2] and k <= max_tp:
            degrees.append(k)
            k *= 2
    degrees = [k for k in degrees if k in off['model_states'].keys()
               and k in on['first_stage']['model_states'] and k in on['last_stage']['model_states']]
    out = {}
    for k in degrees:
        per_stage = [0] * pp
        samples = global_batch_size * k / tp / dp
        samples /= chunks
        if vsp:
            states_key, shard = 1, tp * dp
        else:
            states_key, shard = k, tp * dp // k
        if embed_sdp:
            ratio = zero3_ratio(shard)
        else:
            ratio = zero2_ratio(shard) if parallel_args.use_zero2_for_dp else 1.0
        if pp == 1:
            per_stage[0] += off['model_states'][states_key] * ratio + off['activation'][k] * samples
        else:
            if parallel_args.pipeline_type == 'pipedream_flush':
                first, last = samples * pp, samples * 1
            else:
                first = last = samples
            per_stage[0] += (on['first_stage']['model_states'][states_key] * ratio
                             + on['first_stage']['activation'][k] * first)
            per_stage[-1] += (on['last_stage']['model_states'][states_key] * ratio
                              + on['last_stage']['activation'][k] * last)
        for i in range(len(per_stage)):
            per_stage[i] += train_args.pytorch_context_mem
        out[k] = per_stage
    return out


class MemoryCostModel:
    """Memory (MB) of one layer under one strategy, and of the non-layer parts of the model per
    pipeline stage and vocabulary-tensor-parallel degree (cost_model.py:10-219)."""

    def __init__(self, strategy, global_batch_size: int = 8, mbsz: int = -1, min_tp: int = -1, max_tp: int = -1,
                 stage_idx: int = 0, vsp: int = 0, embed_sdp: bool = False, model_args: ModelArgs = None,
                 train_args: TrainArgs = None, parallel_args: ParallelArgs = None,
                 profile_model_args: ProfileModelArgs = None, logger=None):
        assert mbsz > -1, f'Invalid mbsz: {mbsz}'
        assert min_tp > -1, f'Invalid min_tp: {min_tp}'
        assert None not in (model_args, train_args, parallel_args, profile_model_args), "One or more variables are None"
        self.logger = logger
        pp, tp, dp = strategy[0], strategy[1], strategy[2]
        self.pp_size, self.tp_size, self.dp_size = pp, tp, dp
        ulysses = _is_ulysses(strategy)
        self.sdp_size = tp * dp if ulysses else dp

        # micro-batches: what was asked for (or the chunk function's choice), capped by the samples
        # a pipeline lane has (cost_model.py:77-83)
        chunks = parallel_args.chunks
        if chunks is None:
            chunks = parallel_args.optimal_chunk_func(global_batch_size // dp, strategy, mbsz, min_tp)
        cap = global_batch_size // (tp * dp // min_tp)
        cap = 1 if cap == 0 else cap
        self.chunks = int(cap if chunks > cap else chunks)

        # samples whose activations are alive at once on this stage (cost_model.py:85-97)
        sizes = [len(c) for c in chunk_like_torch(int(global_batch_size / dp / (tp // min_tp)), self.chunks)]
        self.bsz = global_batch_size / dp
        if pp == 1 or parallel_args.pipeline_type == 'pipedream_flush':
            assert self.chunks == len(sizes)
            in_flight = pp - stage_idx if pp - stage_idx <= self.chunks else self.chunks
            self.act_1f1b_ratio = np.sum(sizes[:in_flight]) / np.sum(sizes)
            self.act_1f1b_ratio_first = np.sum(sizes[:min(pp, self.chunks)]) / np.sum(sizes)
            self.act_1f1b_ratio_last = sizes[0] / np.sum(sizes)
            self.bsz = self.act_1f1b_ratio * self.bsz
        else:
            self.bsz = sizes[0]

        self.zero2_ratio, self.zero3_ratio = _zero_ratios(self.chunks, train_args.mixed_precision,
                                                          train_args.async_grad_reduce)

        # parameters and model states of the layer (cost_model.py:112-128)
        self.parameter_size = model_args.parameter_size if ulysses else model_args.parameter_size / tp
        self.model_states_size = 4 * self.parameter_size
        flags = strategy[-1]
        if flags.get('fsdp'):
            self.model_states_size *= self.zero3_ratio(self.sdp_size)
        elif 'fsdp' in flags and flags['fsdp'] == 0 and parallel_args.use_zero2_for_dp:
            self.model_states_size *= self.zero2_ratio(self.sdp_size)

        # activations (cost_model.py:130-138)
        per_sample = profile_model_args.tp_activation_per_bsz_dict
        if flags.get('cpt'):
            assert per_sample['checkpoint'] is not None
            self.activation_size = per_sample['checkpoint'] * self.bsz
            if parallel_args.sequence_parallel:
                self.activation_size /= tp
        else:
            self.activation_size = per_sample[tp] * self.bsz

        self.other_memory_cost = self._other_memory(strategy, global_batch_size, min_tp, max_tp, vsp, embed_sdp,
                                                    train_args, parallel_args, profile_model_args)

    def _other_memory(self, strategy, global_batch_size, min_tp, max_tp, vsp, embed_sdp, train_args, parallel_args,
                      profile):
        return _other_memory(strategy, self.chunks, self.zero2_ratio, self.zero3_ratio, global_batch_size, min_tp,
                             max_tp, vsp, embed_sdp, train_args, parallel_args, profile)

    def get_memory_cost(self):
        return {'parameter': self.parameter_size, 'model_states': self.model_states_size,
                'activation': self.activation_size, 'enc_total': self.model_states_size + self.activation_size,
                'other': self.other_memory_cost}


# ---- memory of a whole strategy set at once ---------------------------------------------------------
class NotVectorisable(Exception):
    """The array forms below cover the inputs the search engine produces; anything else (a lane
    without samples, a micro-batch split that does not give the asked count, a tensor-parallel degree
    the profile has no entry for ...) is left to the per-strategy classes, which then compute or
    raise exactly as the reference does."""


_STRATEGY_ARRAYS = {}


def _strategy_arrays(strategies):
    """pp / tp / dp and the flags of a strategy list as arrays, kept per list (a sweep evaluates the
    same few lists thousands of times)."""
    key = tuple((int(s[0]), int(s[1]), int(s[2]), tuple(sorted(s[-1].items()))) for s in strategies)
    hit = _STRATEGY_ARRAYS.get(key)
    if hit is None:
        flags = [s[-1] for s in strategies]
        tp = np.array([s[1] for s in strategies], dtype=np.int64)
        dp = np.array([s[2] for s in strategies], dtype=np.int64)
        ulysses = np.array([f.get('sp', 0) == 1 for f in flags], dtype=bool)
        hit = {"pp": np.array([s[0] for s in strategies], dtype=np.int64), "tp": tp, "dp": dp, "ulysses": ulysses,
               "sdp": np.where(ulysses, tp * dp, dp),
               "fsdp": np.array([bool(f.get('fsdp', 0)) for f in flags], dtype=bool),
               "fsdp_off": np.array([('fsdp' in f and f['fsdp'] == 0) for f in flags], dtype=bool),
               "cpt": np.array([bool(f.get('cpt', 0)) for f in flags], dtype=bool)}
        if len(_STRATEGY_ARRAYS) > 4096:
            _STRATEGY_ARRAYS.clear()
        _STRATEGY_ARRAYS[key] = hit
    return hit


def _zero_ratio_arrays(chunks, d, mixed_precision, async_grad_reduce):
    """(zero2, zero3) of ``_zero_ratios`` for arrays of micro-batch counts and sharding degrees, the
    same expressions term by term."""
    shard = 1 / d + 0.003
    if mixed_precision:
        one = (7 / 8 * shard + 1 / 8, shard)
        many = (6 / 8 * shard + 2 / 8, 7 / 8 * shard + 1 / 8) if async_grad_reduce else \
            ((7 / 8 * shard + 1 / 8) * 5 / 4, shard * 5 / 4)
    else:
        one = (3 / 4 * shard + 1 / 4, shard)
        many = (2 / 4 * shard + 2 / 4, 3 / 4 * shard + 1 / 4) if async_grad_reduce else \
            (3 / 4 * shard + 1 / 4, shard * 5 / 4)
    single = chunks == 1
    return np.where(single, one[0], many[0]), np.where(single, one[1], many[1])


def memory_cost_rows(strategies, global_batch_size, mbsz, min_tp, max_tp, stage_idx=0, vsp=0, embed_sdp=False,
                     model_args=None, train_args=None, parallel_args=None, profile_model_args=None):
    """``MemoryCostModel(s, ...).get_memory_cost()`` for every strategy of a list in array
    arithmetic: returns ``(enc_total float64 [S], other)`` with ``other`` the first strategy's
    ``'other'`` entry (all that DpOnModel reads, dynamic_programming.py:254-288).  ``stage_idx`` may
    be a sequence of pipeline stages: ``enc_total`` is then [stages, S] (``other`` is taken with the
    first of them).  Each element is
    produced by the same operations in the same order as the class (cost_model.py:10-219), hence the
    same bits; raises ``NotVectorisable`` where the class would take a path this form does not cover."""
    S = len(strategies)
    if S == 0:
        raise NotVectorisable
    A = _strategy_arrays(strategies)
    pp, tp, dp, ulysses, sdp = A["pp"], A["tp"], A["dp"], A["ulysses"], A["sdp"]
    if mbsz <= -1 or min_tp <= 0 or (tp // min_tp < 1).any() or (tp * dp // min_tp < 1).any():
        raise NotVectorisable

    asked = parallel_args.chunks
    if asked is None:
        asked = np.array([parallel_args.optimal_chunk_func(global_batch_size // s[2], s, mbsz, min_tp)
                          for s in strategies], dtype=np.float64)
    else:
        asked = np.full(S, asked, dtype=np.float64)
    cap = global_batch_size // (tp * dp // min_tp)
    cap = np.where(cap == 0, 1, cap)
    chunks = np.where(asked > cap, cap, asked).astype(np.int64)           # int() of the class: towards zero
    if (chunks < 1).any():
        raise NotVectorisable

    # the split torch.arange(size).chunk(chunks) gives: pieces of `step` until the range is used up
    size = (global_batch_size / dp / (tp // min_tp)).astype(np.int64)
    if (size < 1).any():
        raise NotVectorisable
    step = (size + chunks - 1) // chunks
    pieces = (size + step - 1) // step
    first_piece = np.minimum(step, size)
    bsz = global_batch_size / dp
    one_f_one_b = (pp == 1) | (parallel_args.pipeline_type == 'pipedream_flush')
    if one_f_one_b.any():
        if (pieces != chunks)[one_f_one_b].any():
            raise NotVectorisable                                          # the class asserts here
        stage = np.asarray(stage_idx, dtype=np.int64)
        left = pp - (stage[:, None] if stage.ndim == 1 else stage)
        in_flight = np.where(left <= chunks, left, chunks)
        if (in_flight < 1)[..., one_f_one_b].any():
            raise NotVectorisable
        ratio = np.minimum(in_flight * step, size) / size                   # sum of the first pieces / sum of all
        bsz = np.where(one_f_one_b, ratio * bsz, first_piece)
    else:
        bsz = first_piece.astype(np.float64)
        if np.ndim(stage_idx) == 1:
            bsz = np.broadcast_to(bsz, (len(stage_idx), S))

    zero2, zero3 = _zero_ratio_arrays(chunks, sdp, train_args.mixed_precision, train_args.async_grad_reduce)
    parameter = np.where(ulysses, model_args.parameter_size, model_args.parameter_size / tp)
    states = 4 * parameter
    if parallel_args.use_zero2_for_dp:
        states = np.where(A["fsdp"], states * zero3, np.where(A["fsdp_off"], states * zero2, states))
    else:
        states = np.where(A["fsdp"], states * zero3, states)

    per_sample = profile_model_args.tp_activation_per_bsz_dict
    cpt = A["cpt"]
    if cpt.any() and per_sample.get('checkpoint') is None:
        raise NotVectorisable
    if any(int(t) not in per_sample for t in tp[~cpt]):
        raise NotVectorisable
    plain = np.array([per_sample[int(t)] if not c else 0.0 for t, c in zip(tp, cpt)], dtype=np.float64) * bsz
    if cpt.any():
        kept = per_sample['checkpoint'] * bsz
        if parallel_args.sequence_parallel:
            kept = kept / tp
        activation = np.where(cpt, kept, plain)
    else:
        activation = plain

    other = memory_cost_other(strategies, global_batch_size, mbsz, min_tp, max_tp, vsp=vsp, embed_sdp=embed_sdp,
                              model_args=model_args, train_args=train_args, parallel_args=parallel_args,
                              profile_model_args=profile_model_args)
    return states + activation, other


def memory_cost_other(strategies, global_batch_size, mbsz, min_tp, max_tp, vsp=0, embed_sdp=False, model_args=None,
                      train_args=None, parallel_args=None, profile_model_args=None):
    """The ``'other'`` entry of ``MemoryCostModel(strategies[0], ...).get_memory_cost()`` alone -- the one
    part of ``memory_cost_rows`` that depends on ``max_tp``, ``vsp`` and ``embed_sdp`` (the per-layer
    rows do not, so a sweep can keep them while it walks through those).  For inputs that
    ``memory_cost_rows`` accepts."""
    s0 = strategies[0]
    asked = parallel_args.chunks
    if asked is None:
        asked = float(parallel_args.optimal_chunk_func(global_batch_size // s0[2], s0, mbsz, min_tp))
    cap = global_batch_size // (int(s0[1]) * int(s0[2]) // min_tp)
    if cap == 0:
        cap = 1
    chunks0 = int(cap if asked > cap else asked)                           # int() of the class: towards zero
    z2, z3 = _zero_ratios(chunks0, train_args.mixed_precision, train_args.async_grad_reduce)
    return _other_memory(s0, chunks0, z2, z3, global_batch_size, min_tp, max_tp, vsp, embed_sdp, train_args,
                         parallel_args, profile_model_args)


# ---- time -------------------------------------------------------------------------------------------
class TimeCostModel:
    """Time (s) of one layer under one strategy for one pass over ``global_batch_size`` samples
    (cost_model.py:221-466)."""

    def __init__(self, strategy, global_batch_size: int = 8, no_comm: bool = False, model_args: ModelArgs = None,
                 train_args: TrainArgs = None, parallel_args: ParallelArgs = None,
                 profile_model_args: ProfileModelArgs = None, profile_hardware_args: ProfileHardwareArgs = None,
                 logger=None):
        assert None not in (model_args, train_args, parallel_args, profile_hardware_args), "One or more variables are None"
        if model_args.layer_num is None:
            model_args.layer_num = 24              # as the reference: written back into the caller's record
        hw = profile_hardware_args
        self.logger = logger
        self.hw, self.no_comm, self.strategy = hw, no_comm, strategy
        self.mixed_precision = train_args.mixed_precision
        self.pp_size, self.tp_size, self.dp_size = strategy[0], strategy[1], strategy[2]
        pp, tp, dp = self.pp_size, self.tp_size, self.dp_size
        self.sp_space = parallel_args.sp_space
        self.fsdp = _flag(strategy, 'fsdp')
        self.checkpoint = _flag(strategy, 'cpt')
        ulysses = _is_ulysses(strategy)
        self.sdp_size = tp * dp if ulysses else dp
        if tp == 1:
            self.sp_dict = np.inf
        else:
            self.sp_dict = (hw.all2all_dict if ulysses else hw.allreduce_dict)[tp]
        self.seq_len, self.hidden_size, self.layer_num = model_args.seq_length, model_args.hidden_size, model_args.layer_num
        self.bsz = global_batch_size / dp
        self.optimal_microbatch = 1
        self.parameter_size = model_args.parameter_size if ulysses else model_args.parameter_size / tp

        # computation of the whole (dummy) model: forward profiled, backward = coefficient x forward,
        # plus one more forward when activations are recomputed (cost_model.py:299-311)
        per_layer = profile_model_args.forward_computation_time
        if isinstance(per_layer, np.ndarray):
            self.fct = _line(self.bsz / tp, per_layer) * self.layer_num
        else:
            self.fct = per_layer * self.bsz / tp * self.layer_num
        self.bct = self.fct * hw.bct_fct_coe
        if self.checkpoint:
            self.bct += self.fct

        # gradient all-reduce volume and its coefficient (cost_model.py:313-343)
        self.dp_message_size = (2 * (dp - 1) / dp * self.parameter_size) * self.layer_num
        if train_args.mixed_precision:
            self.dp_message_size /= 2
        self.fsdp_allgather_message_size = self.dp_message_size * 0.5
        if no_comm:
            self.dp_message_size = 0
        if ulysses:
            self.dc = _group_coe(hw.comm_coe_dict, self.sdp_size)
        elif tp == 1 or dp == 1:
            self.dc = _group_coe(hw.comm_coe_dict, dp)
        else:
            consecutive_tp = strategy[-1]['tp']
            assert consecutive_tp in [0, 1]
            self.dc = _group_coe(hw.comm_coe_dict, dp, 0 if consecutive_tp else 1)
        self.dc_overlap = self.dc * hw.dp_overlap_coe

        self._tensor_parallel_time(train_args)

        # pipeline send/recv (cost_model.py:405-412)
        self.p2p_comm_coe = None
        if pp > 1 and hw.p2p_comm_coe_dict is not None:
            self.p2p_comm_coe = hw.p2p_comm_coe_dict[pp]
            self.p2p_message_size = pp * 2 * self.bsz * self.seq_len * self.hidden_size * 4 / 1024 / 1024
            if train_args.mixed_precision:
                self.p2p_message_size = self.p2p_message_size / 2

    def _tensor_parallel_time(self, train_args):
        """Activation collectives of tensor / sequence parallelism (cost_model.py:345-403): either
        from profiled message times ('tp+sp' search space) or from volume x coefficient."""
        tp, dp, hw = self.tp_size, self.dp_size, self.hw
        if self.sp_space == 'tp+sp':
            self.tp_comm_num = 4 * self.layer_num
            if self.checkpoint:
                self.tp_comm_num *= 1.5
            if tp == 1:
                per_message = 0
            else:
                self.per_tp_message_size = self.bsz * self.seq_len * self.hidden_size * (2 if train_args.mixed_precision else 4)
                if self.per_tp_message_size in self.sp_dict:
                    per_message = self.sp_dict[self.per_tp_message_size]
                else:
                    per_message = _line(1 / 1024 / 1024 * self.per_tp_message_size, self.sp_dict["popt"])
            self.tp_communication_time = self.tp_comm_num * per_message
            return
        collectives = 4
        self.tp_message_size = 2 * (tp - 1) / tp * (self.bsz * self.seq_len * self.hidden_size * collectives * 4 / 1024 / 1024) * self.layer_num
        if self.checkpoint:
            self.tp_message_size *= 1.5
        if train_args.mixed_precision:
            self.tp_message_size /= 2
        if tp == 1 or dp == 1:
            tc = _group_coe(hw.comm_coe_dict, tp)
        else:
            consecutive_tp = self.strategy[-1]['tp']
            assert consecutive_tp in [0, 1]
            tc = _group_coe(hw.comm_coe_dict, tp, 1 if consecutive_tp else 0)
        self.tp_communication_time = self.tp_message_size * tc

    def bct_dp_overlap(self, dp_message_size, bct):
        """Backward computation against the gradient all-reduce running under it: the overlapped
        part is slowed down by the overlap coefficients, the rest of the longer one runs alone
        (cost_model.py:414-431)."""
        comm = dp_message_size * self.dc_overlap
        comp = bct * self.hw.bct_overlap_coe
        if comm > comp:
            return comp, (dp_message_size - comp / self.dc_overlap) * self.dc, False
        if comm < comp:
            return comm, bct - comm / self.hw.bct_overlap_coe, False
        return comp, 0, False

    def gen_result(self):
        tp, dp, hw = self.tp_size, self.dp_size, self.hw
        if tp == 1 and dp > 1:
            overlapped, rest, _ = self.bct_dp_overlap(self.dp_message_size, self.bct)
            result = self.fct + overlapped + rest + hw.extra_overhead
        elif dp == 1 and tp > 1:
            result = self.fct + self.bct + self.tp_communication_time
        elif dp == 1 and tp == 1:
            result = self.fct + self.bct
        elif tp < tp * dp // 2:
            overlapped, rest, _ = self.bct_dp_overlap(self.dp_message_size, self.bct)
            result = self.fct + overlapped + rest + self.tp_communication_time + hw.extra_overhead
        else:
            overlapped, rest, _ = self.bct_dp_overlap(self.dp_message_size, self.bct * 1 / 2)
            result = self.fct + 1 / 2 * self.bct + overlapped + rest + self.tp_communication_time + hw.extra_overhead
        if self.fsdp:                                       # parameter all-gather of the forward pass
            result = result + self.fsdp_allgather_message_size * self.dc * self.optimal_microbatch
        if self.pp_size > 1 and self.p2p_comm_coe is not None:
            result = result + self.p2p_message_size * self.p2p_comm_coe
        result = result * (0.001 * hw.costmodel_coe)        # ms -> s, calibrated
        return result / self.layer_num


def time_cost_rows(strategies, global_batch_size, no_comm=False, model_args=None, train_args=None, parallel_args=None,
                   profile_model_args=None, profile_hardware_args=None):
    """``TimeCostModel(s, global_batch_size, ...).gen_result()`` for every strategy of a list in
    array arithmetic (float64 [S]); the same operations in the same order as the class
    (cost_model.py:221-466), table look-ups per strategy, everything else elementwise.  Raises
    ``NotVectorisable`` where the class would raise or take a path not covered here."""
    S = len(strategies)
    if S == 0:
        raise NotVectorisable
    if model_args.layer_num is None:
        model_args.layer_num = 24                       # as the class: written back into the caller's record
    hw = profile_hardware_args
    mixed = train_args.mixed_precision
    layer_num, seq_len, hidden = model_args.layer_num, model_args.seq_length, model_args.hidden_size
    A = _strategy_arrays(strategies)
    pp, tp, dp, ulysses, sdp, fsdp, cpt = A["pp"], A["tp"], A["dp"], A["ulysses"], A["sdp"], A["fsdp"], A["cpt"]
    bsz = global_batch_size / dp
    parameter = np.where(ulysses, model_args.parameter_size, model_args.parameter_size / tp)

    per_layer = profile_model_args.forward_computation_time
    if isinstance(per_layer, np.ndarray):
        fct = _line(bsz / tp, per_layer) * layer_num
    else:
        fct = per_layer * bsz / tp * layer_num
    bct = fct * hw.bct_fct_coe
    bct = np.where(cpt, bct + fct, bct)

    dp_message = (2 * (dp - 1) / dp * parameter) * layer_num
    if mixed:
        dp_message = dp_message / 2
    allgather = dp_message * 0.5
    if no_comm:
        dp_message = np.zeros(S)

    # per-strategy look-ups: coefficients of the gradient and activation collectives
    dc, tc, per_message = np.empty(S), np.zeros(S), np.zeros(S)
    tp_sp = parallel_args.sp_space == 'tp+sp'
    word = 2 if mixed else 4
    try:
        for i, st in enumerate(strategies):
            t, d = int(tp[i]), int(dp[i])
            both = not (t == 1 or d == 1)
            if both and not ulysses[i] or (both and not tp_sp):
                consecutive = st[-1]['tp']
                if consecutive not in (0, 1):
                    raise NotVectorisable
            if ulysses[i]:
                dc[i] = _group_coe(hw.comm_coe_dict, int(sdp[i]))
            elif not both:
                dc[i] = _group_coe(hw.comm_coe_dict, d)
            else:
                dc[i] = _group_coe(hw.comm_coe_dict, d, 0 if consecutive else 1)
            if tp_sp:
                if t > 1:
                    table = (hw.all2all_dict if ulysses[i] else hw.allreduce_dict)[t]
                    size = bsz[i] * seq_len * hidden * word
                    per_message[i] = table[size] if size in table else _line(1 / 1024 / 1024 * size, table["popt"])
            elif not both:
                tc[i] = _group_coe(hw.comm_coe_dict, t)
            else:
                tc[i] = _group_coe(hw.comm_coe_dict, t, 1 if consecutive else 0)
    except (KeyError, TypeError):
        raise NotVectorisable from None
    dc_overlap = dc * hw.dp_overlap_coe

    if tp_sp:
        comm_num = np.where(cpt, 4 * layer_num * 1.5, 4 * layer_num)
        tp_time = comm_num * per_message
    else:
        volume = 2 * (tp - 1) / tp * (bsz * seq_len * hidden * 4 * 4 / 1024 / 1024) * layer_num
        volume = np.where(cpt, volume * 1.5, volume)
        if mixed:
            volume = volume / 2
        tp_time = volume * tc

    def overlap(message, backward):
        """bct_dp_overlap of the class, both of its return values."""
        comm = message * dc_overlap
        comp = backward * hw.bct_overlap_coe
        with np.errstate(divide='ignore', invalid='ignore'):
            more_comm = (message - comp / dc_overlap) * dc
            more_comp = backward - comm / hw.bct_overlap_coe
        first = np.where(comm > comp, comp, np.where(comm < comp, comm, comp))
        rest = np.where(comm > comp, more_comm, np.where(comm < comp, more_comp, 0.0))
        return first, rest

    o_full, r_full = overlap(dp_message, bct)
    o_half, r_half = overlap(dp_message, bct * 1 / 2)
    extra = hw.extra_overhead
    only_dp = (tp == 1) & (dp > 1)
    only_tp = (dp == 1) & (tp > 1)
    neither = (dp == 1) & (tp == 1)
    narrow_tp = tp < tp * dp // 2
    result = np.where(only_dp, fct + o_full + r_full + extra,
             np.where(only_tp, fct + bct + tp_time,
             np.where(neither, fct + bct,
             np.where(narrow_tp, fct + o_full + r_full + tp_time + extra,
                      fct + 1 / 2 * bct + o_half + r_half + tp_time + extra))))
    result = np.where(fsdp, result + allgather * dc * 1, result)
    if hw.p2p_comm_coe_dict is not None and (pp > 1).any():
        try:
            coe = np.array([hw.p2p_comm_coe_dict[int(x)] if x > 1 else 0.0 for x in pp])
        except KeyError:
            raise NotVectorisable from None
        message = pp * 2 * bsz * seq_len * hidden * 4 / 1024 / 1024
        if mixed:
            message = message / 2
        result = np.where(pp > 1, result + message * coe, result)
    result = result * (0.001 * hw.costmodel_coe)
    return result / layer_num


class OtherTimeCostModel:
    """Time (s) of the non-layer parts of the model (embedding, head) per pipeline stage and vocabulary
    tensor-parallel degree, with and without the gradient all-reduce (cost_model.py:468-658)."""

    def __init__(self, mbsz: int = 1, pp_deg: int = 2, world_size: int = 8, vsp: bool = False, embed_sdp: bool = False,
                 min_tp: int = 1, max_tp: int = 8, sequence_length_list: list = [512], model_args: ModelArgs = None,
                 train_args: TrainArgs = None, parallel_args: ParallelArgs = None,
                 profile_model_args: ProfileModelArgs = None, profile_hardware_args: ProfileHardwareArgs = None,
                 logger=None):
        assert None not in (model_args, train_args, parallel_args, profile_model_args, profile_hardware_args), \
            "One or more variables are None"
        self.logger = logger
        hw, prof = profile_hardware_args, profile_model_args
        self.hw = hw
        self.pp_deg = pp_deg
        self.sequence_length_list = sequence_length_list
        self.hidden_size = model_args.hidden_size
        self.sp_space = parallel_args.sp_space
        self.dp_coe, self.fct, self.tp_time, self.sp_size, self.dp_size, self.comm_factor = {}, {}, {}, {}, {}, {}
        word = 2 if train_args.mixed_precision else 4

        degrees, k = [], min_tp
        while k <= max_tp and world_size // pp_deg >= k:
            degrees.append(k)
            k *= 2

        for k in degrees:
            # activation collectives of the embedding / head, one per sequence length (cost_model.py:533-570)
            times = []
            # message sizes of the largest degree stay readable on the object, as in the reference
            self.per_tp_message_size, self.tp_message_size = [], []
            for seq_len in sequence_length_list:
                if vsp != 0:
                    times.append(0)
                elif self.sp_space == 'tp+sp':
                    size = mbsz * seq_len * model_args.hidden_size * word
                    self.per_tp_message_size.append(size)
                    if k == 1:
                        times.append(0)
                    elif size in hw.allreduce_dict:
                        times.append(hw.allreduce_dict[size])
                    else:
                        times.append(_line(1 / 1024 / 1024 * size, hw.allreduce_dict[k]["popt"]))
                else:
                    dp = world_size // pp_deg // k
                    coe = _group_coe(hw.comm_coe_dict, k) if (k == 1 or dp == 1) else _group_coe(hw.comm_coe_dict, k, 0)
                    size = (k - 1) / k * (mbsz * seq_len * self.hidden_size / 1024 / 1024) * word
                    self.tp_message_size.append(size)
                    times.append(size * coe)
            self.tp_time[k] = (sum(times) + times[-1]) if pp_deg == 1 else (times[0], times[-1])

            # computation (cost_model.py:572-591)
            profiled = prof.other_time_profiled
            if isinstance(profiled, np.ndarray):
                compute = _line(mbsz / min_tp, profiled)
            else:
                compute = mbsz / min_tp * profiled
            self.fct[k] = compute if pp_deg == 1 else (compute / 2, compute / 2)

            # gradient all-reduce of the embedding / head (cost_model.py:593-619)
            if vsp == 0:
                dp = world_size // pp_deg // k
                coe = _group_coe(hw.comm_coe_dict, dp) if (k == 1 or dp == 1) else _group_coe(hw.comm_coe_dict, dp, 0)
            else:
                dp = world_size // pp_deg
                coe = _group_coe(hw.comm_coe_dict, dp)
            self.dp_coe[k] = coe * ((dp - 1) / dp)          # bus -> algorithm bandwidth
            states_key = k if vsp == 0 else 1
            if pp_deg == 1:
                self.dp_size[k] = prof.other_memory_pp_off['model_states'][states_key] / 4
            else:
                stage = 'first_stage' if vsp == 0 else 'last_stage'
                size = prof.other_memory_pp_on[stage]['model_states'][states_key] / 4
                self.dp_size[k] = (size, size)

        # share of the volume moved in the forward / backward pass (cost_model.py:621-626)
        self.fwd_factor, self.bwd_factor = (0.5, 1.0) if embed_sdp else (0.0, 0.5)

    def get_overlap_time(self, forward_comm_time, forward_comp_time, backward_comm_time, backward_comp_time, tp_time):
        """Computation slowed down while communication runs under it (cost_model.py:629-640)."""
        slow = self.hw.dp_overlap_coe

        def one_pass(comm, comp):
            comp = comp * slow
            return comm + (comp - comm) / slow if comp > comm else comm

        return one_pass(forward_comm_time, forward_comp_time) + one_pass(backward_comm_time, backward_comp_time) + tp_time

    def gen_result(self):
        with_comm, without_comm = {}, {}
        ratio = self.hw.bct_fct_coe
        for k in self.dp_size.keys():
            with_comm[k], without_comm[k] = [0] * self.pp_deg, [0] * self.pp_deg
            if self.pp_deg == 1:
                stages = [(0, self.dp_size[k], self.fct[k], self.tp_time[k])]
            else:
                stages = [(0, self.dp_size[k][0], self.fct[k][0], self.tp_time[k][0]),
                          (-1, self.dp_size[k][-1], self.fct[k][-1], self.tp_time[k][-1])]
            for where, volume, compute, tp_time in stages:
                with_comm[k][where] = 0.001 * self.get_overlap_time(
                    volume * self.dp_coe[k] * self.fwd_factor, compute,
                    volume * self.dp_coe[k] * self.bwd_factor, compute * ratio, tp_time)
                without_comm[k][where] = 0.001 * self.get_overlap_time(
                    volume * self.dp_coe[k] * self.fwd_factor, compute,
                    volume * self.dp_coe[k] * (self.bwd_factor - 0.5), compute * ratio, tp_time)
        return with_comm, without_comm


# ---- pipeline -----------------------------------------------------------------------------------------
def pipeline_costmodel(timecostmodel, layer_num_list, model_args_list, train_args_list, parallel_args_list,
                       profile_model_args_list, profile_hardware_args_list, strategies, partition, chunks, bsz, min_tp,
                       other_time_cost, logger=None, return_stage_cost=False, cache=None):
    """Time of one iteration of a pipeline whose layers run the given strategies, split into stages
    by ``partition`` (cost_model.py:695-767): steady state = every stage's computation once plus
    (micro-batches - 1) times the last stage's, bounded below by the 1F1B warm-up / cool-down
    estimate, plus the gradient synchronisation that is not hidden.
    ``cache`` (no counterpart in the reference): a dict a caller keeps across calls -- a sweep asks for the
    time of the same (layer type, strategy, micro-batch size) hundreds of times.  Entries are keyed by the
    identity of the objects involved and keep those objects alive, so that an identity is never reused."""
    if strategies is None:
        return ([np.inf] * len(partition), np.inf) if return_stage_cost else np.inf
    type_of_layer = []
    for t, count in enumerate(layer_num_list):
        type_of_layer += [t] * count
    lane = int(bsz / (strategies[0][1] * strategies[0][2] // min_tp))
    if isinstance(chunks, list):
        chunks = [get_real_chunk(lane, c) for c in chunks]
        bsz_per_chunk = [bsz / c for c in chunks]
        max_chunk = np.max(chunks)
    else:
        chunks = get_real_chunk(lane, chunks)
        bsz_per_chunk = [bsz / chunks] * len(layer_num_list)
        max_chunk = chunks
    pp_deg = len(partition)

    if cache is None:
        names = [form_strategy(s) for s in strategies]
    else:
        names = []
        for s in strategies:
            hit = cache.get(("form", id(s)))
            if hit is None:
                hit = cache[("form", id(s))] = (form_strategy(s), s)
            names.append(hit[0])
    all_texts = list(set(names))
    full, compute_only = {}, {}
    for t in range(len(layer_num_list)):
        common = dict(model_args=model_args_list[t], train_args=train_args_list[t], parallel_args=parallel_args_list[t],
                      profile_model_args=profile_model_args_list[t],
                      profile_hardware_args=profile_hardware_args_list[t])
        texts = all_texts
        if cache is not None:
            base = ("ptime", id(timecostmodel), bsz_per_chunk[t]) + tuple(id(v) for v in common.values())
            texts = []
            for text in all_texts:
                hit = cache.get(base + (text,))
                if hit is None:
                    texts.append(text)
                else:
                    full[t, text], compute_only[t, text] = hit[0], hit[1]
        rows = None
        # this package's own model: all strategies at once -- where there are enough of them for one array
        # evaluation (some sixty array operations) to be cheaper than an object per strategy
        if timecostmodel is TimeCostModel and len(texts) >= 8:
            try:
                parsed = [strategy_str2list(text) for text in texts]
                rows = (time_cost_rows(parsed, bsz_per_chunk[t], **common),
                        time_cost_rows(parsed, bsz_per_chunk[t], no_comm=True, **common))
            except NotVectorisable:
                rows = None
        for n, text in enumerate(texts):
            if rows is not None:
                full[t, text], compute_only[t, text] = rows[0][n], rows[1][n]
                continue
            full[t, text] = timecostmodel(strategy_str2list(text), bsz_per_chunk[t], logger=logger, **common).gen_result()
            compute_only[t, text] = timecostmodel(strategy_str2list(text), bsz_per_chunk[t], no_comm=True, logger=logger,
                                                  **common).gen_result()
        if cache is not None:
            for text in texts:
                cache[base + (text,)] = (full[t, text], compute_only[t, text], timecostmodel, tuple(common.values()))
    per_layer_full = [full[type_of_layer[i], name] for i, name in enumerate(names)]
    per_layer_compute = [compute_only[type_of_layer[i], name] for i, name in enumerate(names)]
    stage_full = get_time_cost_all_stages(per_layer_full, partition)
    stage_compute = get_time_cost_all_stages(per_layer_compute, partition)
    assert len(other_time_cost) == len(stage_compute)
    for i in range(len(other_time_cost)):
        stage_compute[i] += other_time_cost[i]

    result = sum_like_numpy(stage_compute) + stage_compute[-1] * (max_chunk - 1)
    ramp = min(pp_deg - 1, max_chunk - 1) * stage_compute[0]
    tail = sum_like_numpy(stage_compute[1:])
    result = max(result,
                 max(ramp * 1 / 3, tail * 1 / 3) + max(ramp * 2 / 3, tail * 2 / 3)
                 + stage_compute[0] * max(0, max_chunk + 1 - pp_deg))
    exposed = [stage_full[i] - sum_like_numpy(stage_compute[:i + 1]) for i in range(pp_deg)]
    reduce_time = np.max(exposed)
    result += reduce_time if reduce_time > 0 else 0
    if return_stage_cost:
        return stage_full, result
    return result
