"""Seeded scenarios for the cost models, shared by tests/golden/make_cost_model_golden.py (which
runs them through the reference's classes) and tests/test_cost_models.py (which runs them through
galvatron_dp.cost_models): a case is rebuilt from its seed on both sides, the fixture holds only the
numbers that came out.  Profiles are synthetic, of the shape of the reference's mock profiles
(tests/utils/search_configs.py:9-547): activation per sample and tp degree, model states and
activation of the non-layer parts per vocabulary tp degree and pipeline position, collective
coefficients keyed '<size>' or '<size>_<0|1>', fitted lines ('popt') for sequence-parallel
collectives."""
import numpy as np

N_MEMORY, N_TIME, N_OTHER, N_PIPELINE, N_PP = 400, 400, 200, 120, 150


def _rng(kind, seed):
    return np.random.Generator(np.random.PCG64([{"memory": 1, "time": 2, "other": 3, "pipeline": 4, "pp": 5}[kind], seed]))


def hexf(x):
    return float(x).hex()


def jsonable(x):
    if isinstance(x, dict):
        return {str(k): jsonable(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [jsonable(v) for v in x]
    if isinstance(x, (bool, np.bool_)):
        return bool(x)
    if isinstance(x, (int, np.integer)):
        return int(x)
    if isinstance(x, (float, np.floating)):
        return hexf(x)
    if x is None or isinstance(x, str):
        return x
    raise TypeError(type(x))


def chunk_func(local_bsz, strategy, microbatch_size, min_tp):
    """Micro-batch count for a local batch: ceil(samples of one pipeline lane / micro-batch size), at
    least 1 (what the search engine passes as ``optimal_chunk_func``, search_engine.py:1090-1098)."""
    assert strategy[1] % min_tp == 0
    lane = local_bsz // (strategy[1] // min_tp)
    chunk = np.ceil(lane / microbatch_size)
    return 1 if chunk == 0 else chunk


def _pieces(size, chunks):
    step = (size + chunks - 1) // chunks
    return len(range(0, size, step)) if size > 0 else 0


def profile(rng):
    """One synthetic hardware + model profile."""
    act = {k: float(rng.uniform(10, 90)) / (k ** 0.7) for k in (1, 2, 4, 8)}
    act['checkpoint'] = float(rng.uniform(2, 12))
    tab = lambda lo, hi: {k: float(rng.uniform(lo, hi)) / k for k in (1, 2, 4, 8)}  # noqa: E731
    p = {
        'tp_activation_per_bsz_dict': act,
        'other_memory_pp_off': {'model_states': tab(500, 3000), 'activation': tab(100, 800)},
        'other_memory_pp_on': {'first_stage': {'model_states': tab(300, 2000), 'activation': tab(50, 500)},
                               'last_stage': {'model_states': tab(300, 2000), 'activation': tab(50, 500)}},
        'forward_computation_time': (np.array([rng.uniform(0.5, 3.0), rng.uniform(0.0, 1.0)])
                                     if rng.random() < 0.5 else float(rng.uniform(0.5, 3.0))),
        'other_time_profiled': (np.array([rng.uniform(0.5, 5.0), rng.uniform(0.0, 2.0)])
                                if rng.random() < 0.5 else float(rng.uniform(0.5, 5.0))),
        'comm_coe_dict': {'8': float(rng.uniform(0.004, 0.009)), '4_0': float(rng.uniform(0.004, 0.009)),
                          '4_1': float(rng.uniform(0.004, 0.009)), '2_0': float(rng.uniform(0.004, 0.009)),
                          '2_1': float(rng.uniform(0.004, 0.009)), '1': 0},
        'p2p_comm_coe_dict': ({k: float(rng.uniform(0.005, 0.01)) for k in (2, 4, 8)} if rng.random() < 0.85 else None),
        'allreduce_dict': {k: {'popt': [float(rng.uniform(0.01, 0.1)), float(rng.uniform(0.0, 0.5))]} for k in (2, 4, 8)},
        'all2all_dict': {k: {'popt': [float(rng.uniform(0.01, 0.1)), float(rng.uniform(0.0, 0.5))]} for k in (2, 4, 8)},
        'dp_overlap_coe': float(rng.uniform(1.0, 1.6)), 'bct_overlap_coe': float(rng.uniform(1.0, 1.6)),
        'bct_fct_coe': float(rng.choice([2.0, 2.0, 1.8, 2.3])), 'extra_overhead': float(rng.choice([0.0, 0.0, 3.5])),
        'costmodel_coe': float(rng.choice([1.0, 1.0, 1.07])),
    }
    # a few exactly profiled message sizes next to the fitted lines
    for table in (p['allreduce_dict'], p['all2all_dict']):
        for k in (2, 4, 8):
            for size in (2 ** 22, 2 ** 24, 2 ** 25):
                if rng.random() < 0.5:
                    table[k][size] = float(rng.uniform(0.05, 2.0))
    return p


def strategy(rng, world=8, pp=None):
    pp = int(rng.choice([1, 2, 4, 8])) if pp is None else pp
    rest = world // pp
    tp = int(rng.choice([t for t in (1, 2, 4, 8) if t <= rest]))
    dp = rest // tp
    flags = {}
    if dp > 1 or rng.random() < 0.3:
        flags['fsdp'] = int(rng.integers(0, 2)) if dp > 1 else 0
    if tp > 1 and dp > 1:
        flags['tp'] = int(rng.integers(0, 2))
    if rng.random() < 0.5:
        flags['cpt'] = int(rng.integers(0, 2))
    if tp > 1 and rng.random() < 0.5:
        flags['sp'] = int(rng.integers(0, 2))
    return [pp, tp, dp, flags]


def all_strategies():
    out = []
    for pp in (1, 2, 4, 8):
        rest = 8 // pp
        for tp in (1, 2, 4, 8):
            if tp > rest:
                continue
            dp = rest // tp
            for fsdp in (0, 1):
                for cpt in (0, 1):
                    for sp in (0, 1):
                        for consec in (0, 1):
                            flags = {}
                            if dp > 1:
                                flags['fsdp'] = fsdp
                            if tp > 1 and dp > 1:
                                flags['tp'] = consec
                            if cpt:
                                flags['cpt'] = 1
                            if sp:
                                flags['sp'] = 1
                            s = [pp, tp, dp, flags]
                            if s not in out:
                                out.append(s)
    return out


def _records(args_mod, prof, model, train, parallel):
    return (args_mod.ModelArgs(**model), args_mod.TrainArgs(**train), args_mod.ParallelArgs(**parallel),
            args_mod.ProfileModelArgs(tp_activation_per_bsz_dict=prof['tp_activation_per_bsz_dict'],
                                      other_memory_pp_off=prof['other_memory_pp_off'],
                                      other_memory_pp_on=prof['other_memory_pp_on'],
                                      forward_computation_time=prof['forward_computation_time'],
                                      other_time_profiled=prof['other_time_profiled']),
            args_mod.ProfileHardwareArgs(bct_fct_coe=prof['bct_fct_coe'], extra_overhead=prof['extra_overhead'],
                                         comm_coe_dict=prof['comm_coe_dict'], dp_overlap_coe=prof['dp_overlap_coe'],
                                         bct_overlap_coe=prof['bct_overlap_coe'],
                                         p2p_comm_coe_dict=prof['p2p_comm_coe_dict'],
                                         allreduce_dict=prof['allreduce_dict'], all2all_dict=prof['all2all_dict'],
                                         costmodel_coe=prof['costmodel_coe']))


def _common(rng):
    model = dict(parameter_size=float(rng.uniform(20, 800)), seq_length=int(rng.choice([512, 2048, 4096])),
                 hidden_size=int(rng.choice([1024, 4096, 5120])), layer_num=int(rng.choice([8, 24, 32])))
    train = dict(mixed_precision=bool(rng.integers(0, 2)), async_grad_reduce=bool(rng.integers(0, 2)),
                 pytorch_context_mem=int(rng.choice([0, 1024])))
    parallel = dict(use_zero2_for_dp=bool(rng.integers(0, 2)), disable_vtp=bool(rng.random() < 0.2),
                    sequence_parallel=bool(rng.integers(0, 2)), sp_space=str(rng.choice(['tp', 'tp+sp'])),
                    pipeline_type=str(rng.choice(['gpipe', 'pipedream_flush'])), optimal_chunk_func=chunk_func,
                    chunks=None)
    return model, train, parallel


# ---- memory -----------------------------------------------------------------------------------------
def memory_case(seed):
    rng = _rng("memory", seed)
    while True:
        prof = profile(rng)
        s = strategy(rng)
        model, train, parallel = _common(rng)
        min_tp = int(rng.choice([m for m in (1, 2, 4) if s[1] % m == 0 and m <= s[1]]))
        gbsz = int(rng.choice([8, 16, 24, 32, 64, 128]))
        mbsz = int(rng.choice([1, 2, 4, 8]))
        if rng.random() < 0.4:
            parallel['chunks'] = int(rng.choice([1, 2, 3, 4, 8, 16]))
        kw = dict(global_batch_size=gbsz, mbsz=mbsz, min_tp=min_tp, max_tp=int(rng.choice([2, 4, 8])),
                  stage_idx=int(rng.integers(0, s[0])), vsp=int(rng.integers(0, 2)), embed_sdp=bool(rng.integers(0, 2)))
        # the reference asserts that the asked number of micro-batches comes out of the split
        lane = int(gbsz / s[2] / (s[1] // min_tp))
        chunks = parallel['chunks'] if parallel['chunks'] is not None else chunk_func(gbsz // s[2], s, mbsz, min_tp)
        cap = gbsz // (s[1] * s[2] // min_tp)
        chunks = int(min(chunks, cap if cap else 1))
        if lane > 0 and _pieces(lane, chunks) == chunks:
            return dict(prof=prof, strategy=s, model=model, train=train, parallel=parallel, kw=kw)


def memory_cases():
    return list(range(N_MEMORY))


def run_memory(mod, args_mod, seed):
    c = memory_case(seed)
    m, t, p, pm, _ = _records(args_mod, c['prof'], c['model'], c['train'], c['parallel'])
    obj = mod.MemoryCostModel(c['strategy'], model_args=m, train_args=t, parallel_args=p, profile_model_args=pm, **c['kw'])
    return jsonable({'cost': obj.get_memory_cost(), 'chunks': obj.chunks, 'bsz': obj.bsz, 'sdp_size': obj.sdp_size})


# ---- time -------------------------------------------------------------------------------------------
def time_case(seed):
    rng = _rng("time", seed)
    prof = profile(rng)
    s = strategy(rng)
    model, train, parallel = _common(rng)
    if rng.random() < 0.1:
        model['layer_num'] = None
    return dict(prof=prof, strategy=s, model=model, train=train, parallel=parallel,
                gbsz=float(rng.choice([8, 16, 32, 64, 2.5, 10.0 / 3])), no_comm=bool(rng.random() < 0.3))


def time_cases():
    return list(range(N_TIME))


def run_time(mod, args_mod, seed):
    c = time_case(seed)
    m, t, p, pm, hw = _records(args_mod, c['prof'], c['model'], c['train'], c['parallel'])
    obj = mod.TimeCostModel(c['strategy'], c['gbsz'], no_comm=c['no_comm'], model_args=m, train_args=t,
                            parallel_args=p, profile_model_args=pm, profile_hardware_args=hw)
    out = {'result': obj.gen_result(), 'fct': obj.fct, 'bct': obj.bct, 'dp_message_size': obj.dp_message_size,
           'fsdp_allgather_message_size': obj.fsdp_allgather_message_size, 'dc': obj.dc,
           'tp_communication_time': obj.tp_communication_time, 'layer_num_after': m.layer_num}
    overlapped, rest, flag = obj.bct_dp_overlap(obj.dp_message_size, obj.bct)
    out['overlap'] = [overlapped, rest, bool(flag)]
    return jsonable(out)


# ---- other time -------------------------------------------------------------------------------------
def other_case(seed):
    rng = _rng("other", seed)
    prof = profile(rng)
    model, train, parallel = _common(rng)
    pp = int(rng.choice([1, 2, 4, 8]))
    return dict(prof=prof, model=model, train=train, parallel=parallel,
                kw=dict(mbsz=int(rng.choice([1, 2, 4, 8])), pp_deg=pp, world_size=8, vsp=int(rng.integers(0, 2)),
                        embed_sdp=bool(rng.integers(0, 2)), min_tp=int(rng.choice([1, 2])),
                        max_tp=int(rng.choice([2, 4, 8])),
                        sequence_length_list=[int(x) for x in rng.choice([512, 1024, 2048], size=int(rng.integers(1, 3)))]))


def other_cases():
    return list(range(N_OTHER))


def run_other(mod, args_mod, seed):
    c = other_case(seed)
    m, t, p, pm, hw = _records(args_mod, c['prof'], c['model'], c['train'], c['parallel'])
    obj = mod.OtherTimeCostModel(model_args=m, train_args=t, parallel_args=p, profile_model_args=pm,
                                 profile_hardware_args=hw, **c['kw'])
    with_comm, without = obj.gen_result()
    return jsonable({'with': with_comm, 'without': without})


# ---- pipeline ---------------------------------------------------------------------------------------
def pipeline_case(seed):
    rng = _rng("pipeline", seed)
    n_types = int(rng.integers(1, 3))
    pp = int(rng.choice([1, 2, 4]))
    layer_num_list = [int(rng.integers(pp, 9)) for _ in range(n_types)]
    total = sum(layer_num_list)
    cuts = sorted(rng.choice(np.arange(1, total), size=pp - 1, replace=False)) if pp > 1 else []
    partition = [int(b - a) for a, b in zip([0] + list(cuts), list(cuts) + [total])]
    # every layer of one candidate shares tp*dp; the first strategy fixes the lane width
    first = strategy(rng, pp=pp)
    strategies = [first] + [strategy(rng, pp=pp) for _ in range(total - 1)]
    profs, records = [], []
    for _ in range(n_types):
        profs.append(profile(rng))
        records.append(_common(rng))
    min_tp = int(rng.choice([m for m in (1, 2) if all(s[1] % m == 0 for s in strategies)]))
    chunks = [int(rng.choice([1, 2, 4, 8])) for _ in range(n_types)] if rng.random() < 0.4 else int(rng.choice([1, 2, 4, 8]))
    return dict(layer_num_list=layer_num_list, partition=partition, strategies=strategies, profs=profs,
                records=records, chunks=chunks, bsz=int(rng.choice([16, 32, 64])), min_tp=min_tp,
                other_time_cost=[float(rng.uniform(0.0, 0.05)) for _ in range(pp)],
                none=bool(rng.random() < 0.05))


def pipeline_cases():
    return list(range(N_PIPELINE))


def run_pipeline(mod, args_mod, seed):
    c = pipeline_case(seed)
    lists = [[], [], [], [], []]
    for prof, (model, train, parallel) in zip(c['profs'], c['records']):
        for lst, rec in zip(lists, _records(args_mod, prof, model, train, parallel)):
            lst.append(rec)
    strategies = None if c['none'] else c['strategies']
    stage, total = mod.pipeline_costmodel(mod.TimeCostModel, c['layer_num_list'], *lists, strategies, c['partition'],
                                          c['chunks'], c['bsz'], c['min_tp'], c['other_time_cost'],
                                          return_stage_cost=True)
    only = mod.pipeline_costmodel(mod.TimeCostModel, c['layer_num_list'], *lists, strategies, c['partition'],
                                  c['chunks'], c['bsz'], c['min_tp'], c['other_time_cost'])
    return jsonable({'stage': list(stage), 'total': total, 'only': only})


# ---- pipeline division ------------------------------------------------------------------------------
def pp_case(seed):
    rng = _rng("pp", seed)
    n_types = int(rng.integers(1, 3))
    layer_num = [int(rng.integers(4, 33)) for _ in range(n_types)]
    pp = int(rng.choice([1, 2, 4, 8]))
    strategies = [s for s in all_strategies() if rng.random() < 0.6 or s[0] == pp]
    if rng.random() < 0.1:
        strategies = [s for s in strategies if s[0] != pp]           # nothing to choose from -> (None, None)
    rng.shuffle(strategies)
    profs = [profile(rng) for _ in range(n_types)]
    records = [_common(rng) for _ in range(n_types)]
    mbsz = {1: int(rng.choice([4, 8])), 2: int(rng.choice([2, 4])), 4: int(rng.choice([1, 2])), 8: 1}
    return dict(layer_num=layer_num, pp=pp, strategies=[list(s) for s in strategies], profs=profs, records=records,
                bsz=int(rng.choice([32, 64, 128])), mbsz=mbsz, even=bool(rng.integers(0, 2)))


def pp_cases():
    return list(range(N_PP))


def run_pp(pp_mod, args_mod, seed):
    """``pp_mod`` holds the division functions (the reference's search_engine module or
    galvatron_dp.pp_utils)."""
    c = pp_case(seed)
    lists = [[], [], [], [], []]
    for prof, (model, train, parallel) in zip(c['profs'], c['records']):
        for lst, rec in zip(lists, _records(args_mod, prof, model, train, parallel)):
            lst.append(rec)
    m, t, p, pm, _ = lists
    division, per_stage = pp_mod.pp_division_memory_balanced(m, t, p, pm, c['layer_num'], c['pp'], c['bsz'],
                                                             c['mbsz'][c['pp']], c['strategies'])
    out = {'division': None if division is None else [int(x) for x in division],
           'per_stage': None if per_stage is None else list(per_stage),
           'types_untouched': [x.pipeline_type for x in p]}
    if any(s[0] == c['pp'] for s in c['strategies']):
        stage = pp_mod.get_pp_stage_for_bsz([s for s in c['strategies'] if s[0] <= 4], m, t, p, pm, c['layer_num'],
                                            c['bsz'], c['mbsz'], single_layer_even=c['even'])
        out['stage_dict'] = {k: None if v is None else [int(x) for x in v] for k, v in stage.items()}
        world = 8
        out['chunks'] = pp_mod.check_optimal_chunks(world, [s for s in c['strategies'] if s[0] <= 4],
                                                    pp_mod.optimal_chunk_func_default, c['bsz'], c['mbsz'], 1)
    costs = [float(i) * 1.5 + 0.25 for i in range(sum(c['layer_num']) + seed % 3)]
    even = pp_mod.pp_division_even(c['layer_num'], c['pp'])
    out['even'] = [int(x) for x in even]
    out['stage_sums'] = pp_mod.get_cost_all_stages(costs, even if c['pp'] > 1 or seed % 3 < 2 else [sum(c['layer_num'])])
    out['layer_costs'] = pp_mod.get_layer_costs(c['layer_num'], [1.5, 2.5][:len(c['layer_num'])])
    return jsonable(out)
