"""Deterministic stand-ins for the search engine's cost models, with the call signatures
``DpOnModel`` uses (galvatron/core/search_engine/dynamic_programming.py:232-288,248-253,489-500).
They are NOT the reference's cost models (those are a later row of the scope table): they only give
``DpOnModel`` -- the reference's and this repository's -- the same numbers to work with, so that
the two can be compared.  Shared by tests/golden/make_dp_on_model_golden.py and the tests."""
from types import SimpleNamespace

import numpy as np


def strategies(n_gpu=8, pps=(1, 2, 4)):
    out = []
    for pp in pps:
        world = n_gpu // pp
        tp = 1
        while tp <= world:
            dp = world // tp
            for fsdp in (0, 1):
                for cpt in (0, 1):
                    variants = [{}]
                    if tp > 1 and dp > 1:
                        variants = [{'tp': 0}, {'tp': 1}]
                    elif tp > 1:
                        variants = [{'tp': 1}]
                    for v in variants:
                        sps = (0, 1) if tp > 1 else (None,)
                        for sp in sps:
                            info = dict(v)
                            info['fsdp'] = fsdp
                            info['cpt'] = cpt
                            if sp is not None:
                                info['sp'] = sp
                            out.append([pp, tp, dp, info])
            tp *= 2
    return out


def _flags(strategy):
    o = strategy[-1]
    return o.get('fsdp', 0), o.get('cpt', 0), o.get('tp', 1), o.get('sp', 0)


class StubTime:
    def __init__(self, strategy, bsz, no_comm=False, model_args=None, train_args=None, parallel_args=None,
                 profile_model_args=None, profile_hardware_args=None, logger=None):
        self.s, self.bsz, self.no_comm, self.scale = strategy, bsz, no_comm, model_args.scale

    def gen_result(self):
        pp, tp, dp = self.s[:3]
        fsdp, cpt, consec, sp = _flags(self.s)
        compute = self.scale * self.bsz / (tp * dp) * (1.0 + 0.33 * cpt)
        comm = 0.0 if self.no_comm else self.scale * (0.11 * (tp - 1) / tp * (1.3 - 0.2 * consec) * (1 - 0.15 * sp)
                                                      + 0.07 * (dp - 1) / dp * (1 + 0.5 * fsdp))
        return compute + comm


class StubMem:
    def __init__(self, strategy, bsz, mbsz=1, min_tp=1, max_tp=8, stage_idx=0, vsp=0, embed_sdp=0, model_args=None,
                 train_args=None, parallel_args=None, profile_model_args=None, logger=None):
        self.s, self.bsz, self.mbsz, self.stage_idx, self.vsp, self.embed_sdp = strategy, bsz, mbsz, stage_idx, vsp, embed_sdp
        self.scale = model_args.mem_scale
        self.max_tp = max_tp

    def get_memory_cost(self):
        pp, tp, dp = self.s[:3]
        fsdp, cpt, consec, sp = _flags(self.s)
        states = 420.0 * self.scale / tp / (dp if fsdp else 1)
        act = 95.3 * self.scale * self.mbsz / tp * (0.25 if cpt else 1.0) * (0.8 if sp else 1.0) * (pp - self.stage_idx)
        other = {}
        t = 1
        while t <= self.max_tp:
            other[t] = np.array([1800.5 / t + (350.25 if i == 0 else 0.0) + 40.0 * self.embed_sdp for i in range(pp)])
            t *= 2
        return {'enc_total': states + act, 'other': other}


class StubOther:
    def __init__(self, mbsz, pp_deg, n_gpu, vsp, embed_sdp, min_tp, max_tp, sequence_len, model_args=None,
                 train_args=None, parallel_args=None, profile_model_args=None, profile_hardware_args=None, logger=None):
        self.mbsz, self.pp, self.max_tp, self.vsp = mbsz, pp_deg, max_tp, vsp

    def gen_result(self):
        with_comm, no_comm = {}, {}
        t = 1
        while t <= self.max_tp:
            with_comm[t] = [3.5 * self.mbsz / t + 0.6 * (t - 1) + (1.25 if i in (0, self.pp - 1) else 0.0)
                            for i in range(self.pp)]
            no_comm[t] = [3.5 * self.mbsz / t + (1.25 if i in (0, self.pp - 1) else 0.0) for i in range(self.pp)]
            t *= 2
        return with_comm, no_comm


def stub_pipeline_costmodel(timecostmodel, layer_num_list, model_args_list, train_args_list, parallel_args_list,
                            profile_model_args_list, profile_hardware_args_list, strategies, partition, chunks, bsz,
                            min_tp, other_time_cost, logger=None, return_stage_cost=False):
    if strategies is None:
        return np.inf
    type_of = []
    for t, n in enumerate(layer_num_list):
        type_of += [t] * n
    ch = max(chunks) if isinstance(chunks, list) else chunks
    per_layer = [timecostmodel(s, bsz / ch, model_args=model_args_list[type_of[i]], train_args=None, parallel_args=None,
                               profile_model_args=None, profile_hardware_args=None).gen_result()
                 for i, s in enumerate(strategies)]
    stage, pos = [], 0
    for i, n in enumerate(partition):
        stage.append(sum(per_layer[pos:pos + n]) + other_time_cost[i])
        pos += n
    return sum(stage) + max(stage) * (ch - 1)


class StubParallelArgs:
    def optimal_chunk_func(self, local_bsz, strategy, mbsz, min_tp):
        return max(1, int(local_bsz // max(1, mbsz)))


def scenario(name):
    """Constructor keyword arguments and ``fit`` arguments of one comparison case."""
    base = dict(layer_num=[12], pipeline_type='pipedream_flush', micro=True, sp=True, fine=1, max_mem=9000,
                bsz=64, min_tp=1, max_tp=8, vsp=0, embed_sdp=0, sp_search=1, mbsz={1: 8, 2: 4, 4: 2}, scales=[1.0],
                mem_scales=[1.0], pps=(1, 2, 4), stage={1: [12], 2: [7, 5], 4: [4, 3, 3, 2]}, seq=[2048])
    table = {
        'flush_fine': {},
        'flush_fine_tight': {'max_mem': 5000, 'mem_scales': [3.0]},
        'flush_fine_mix': {'max_mem': 8000, 'mem_scales': [5.0]},
        'flush_fine_mix7': {'max_mem': 7000, 'mem_scales': [5.0], 'bsz': 128},
        'flush_fine_loose': {'max_mem': 30000},
        'gpipe_two_types': {'layer_num': [6, 6], 'pipeline_type': 'gpipe', 'sp': False, 'scales': [1.0, 1.7],
                            'mem_scales': [3.0, 4.5], 'seq': [2048, 512], 'max_mem': 9000},
        'flush_coarse': {'fine': 0, 'max_mem': 14000},
        'flush_coarse_tight': {'fine': 0, 'max_mem': 6000, 'mem_scales': [3.0]},
        'no_microbatch_after_dp': {'micro': False},
        'odd_batch': {'bsz': 36, 'max_mem': 12000},
        'min_tp2': {'min_tp': 2, 'max_mem': 11000, 'sp_search': 2},
        'infeasible': {'max_mem': 1500},
    }
    cfg = dict(base)
    cfg.update(table[name])
    return cfg


SCENARIOS = ['flush_fine', 'flush_fine_tight', 'flush_fine_mix', 'flush_fine_mix7', 'flush_fine_loose',
             'gpipe_two_types', 'flush_coarse', 'flush_coarse_tight',
             'no_microbatch_after_dp', 'odd_batch', 'min_tp2', 'infeasible']


def build(DpOnModel, cfg, **extra):
    n = len(cfg['layer_num'])
    margs = [SimpleNamespace(scale=cfg['scales'][i], mem_scale=cfg['mem_scales'][i]) for i in range(n)]
    config = SimpleNamespace(hidden_size=4096, mixed_precision='bf16', sequence_parallel=cfg['sp'],
                             global_memory_buffer=True, fine_grained_mode=cfg['fine'])
    comm = {'1': 0.0, '2': 0.021, '2_0': 0.027, '2_1': 0.021, '4': 0.034, '4_0': 0.041, '4_1': 0.034, '8': 0.05,
            '8_1': 0.05}
    return DpOnModel(strategies(8, cfg['pps']), StubMem, StubTime, model_args_list=margs, train_args_list=[None] * n,
                     parallel_args_list=[StubParallelArgs() for _ in range(n)], profile_model_args_list=[None] * n,
                     profile_hardware_args_list=[None] * n, max_mem=cfg['max_mem'], layer_num=list(cfg['layer_num']),
                     sequence_len=list(cfg['seq']), multi_layer_type=True,
                     pp_stage_dict={k: list(v) for k, v in cfg['stage'].items()}, comm_coe_dict=comm, gpu_num=8,
                     model_microbatch_after_dp=cfg['micro'], pipeline_type=cfg['pipeline_type'], config=config,
                     **extra)


# ---- scenarios with the real cost models ------------------------------------------------------------
# The whole producer -> DP -> pipeline-model chain: the reference's DpOnModel fed by the reference's
# MemoryCostModel / TimeCostModel / OtherTimeCostModel / pipeline_costmodel on one side, this
# repository's classes on the other, over a synthetic profile (tests/cost_model_cases.py).
REAL_SCENARIOS = ['real_flush', 'real_gpipe_two_types', 'real_tight_zero2', 'real_vsp_embed_sdp']


def real_scenario(name):
    base = dict(layer_num=[12], pipeline_type='pipedream_flush', micro=True, sp=True, fine=1, max_mem=24000,
                bsz=64, min_tp=1, max_tp=8, vsp=0, embed_sdp=0, sp_search=1, mbsz={1: 8, 2: 4, 4: 2},
                pps=(1, 2, 4), stage={1: [12], 2: [7, 5], 4: [4, 3, 3, 2]}, seq=[2048], profile_seeds=[11],
                params=[120.0], zero2=False, sp_space='tp+sp', mixed=True)
    table = {
        'real_flush': {},
        'real_gpipe_two_types': {'layer_num': [6, 6], 'pipeline_type': 'gpipe', 'seq': [2048, 512],
                                 'profile_seeds': [5, 6], 'params': [150.0, 60.0], 'sp_space': 'tp', 'max_mem': 30000},
        'real_tight_zero2': {'max_mem': 9000, 'zero2': True, 'params': [220.0], 'profile_seeds': [23], 'mixed': False},
        'real_vsp_embed_sdp': {'vsp': 1, 'embed_sdp': 1, 'profile_seeds': [31], 'bsz': 32, 'max_mem': 16000},
    }
    cfg = dict(base)
    cfg.update(table[name])
    return cfg


def build_real(DpOnModel, cost_mod, args_mod, cfg, **extra):
    """DpOnModel over ``cost_mod``'s MemoryCostModel / TimeCostModel and ``args_mod``'s argument
    records (the reference's modules or galvatron_dp.cost_models for both)."""
    import cost_model_cases as C
    n = len(cfg['layer_num'])
    lists = [[], [], [], [], []]
    for i in range(n):
        prof = C.profile(np.random.Generator(np.random.PCG64([99, cfg['profile_seeds'][i]])))
        model = dict(parameter_size=cfg['params'][i], seq_length=cfg['seq'][i], hidden_size=4096, layer_num=24)
        train = dict(mixed_precision=cfg['mixed'], async_grad_reduce=True, pytorch_context_mem=1024)
        parallel = dict(use_zero2_for_dp=cfg['zero2'], disable_vtp=False, sequence_parallel=cfg['sp'],
                        sp_space=cfg['sp_space'], pipeline_type=cfg['pipeline_type'],
                        optimal_chunk_func=C.chunk_func, chunks=None)
        for lst, rec in zip(lists, C._records(args_mod, prof, model, train, parallel)):
            lst.append(rec)
    config = SimpleNamespace(hidden_size=4096, mixed_precision='bf16' if cfg['mixed'] else 'fp32',
                             sequence_parallel=cfg['sp'], global_memory_buffer=True, fine_grained_mode=cfg['fine'])
    return DpOnModel(strategies(8, cfg['pps']), cost_mod.MemoryCostModel, cost_mod.TimeCostModel,
                     model_args_list=lists[0], train_args_list=lists[1], parallel_args_list=lists[2],
                     profile_model_args_list=lists[3], profile_hardware_args_list=lists[4], max_mem=cfg['max_mem'],
                     layer_num=list(cfg['layer_num']), sequence_len=list(cfg['seq']), multi_layer_type=True,
                     pp_stage_dict={k: list(v) for k, v in cfg['stage'].items()},
                     comm_coe_dict=lists[4][0].comm_coe_dict, gpu_num=8, model_microbatch_after_dp=cfg['micro'],
                     pipeline_type=cfg['pipeline_type'], config=config, **extra)


def run(dpm, cfg):
    fit = dpm.fit(cfg['bsz'], cfg['min_tp'], cfg['max_tp'], cfg['vsp'], cfg['embed_sdp'], cfg['sp_search'],
                  print_=False, mbsz_dict=dict(cfg['mbsz']))
    per_pp = {}
    for pp in cfg['pps']:
        if pp * cfg['min_tp'] > 8 or cfg['bsz'] % (8 // (pp * cfg['min_tp'])):
            continue
        per_pp[str(pp)] = dpm._build_dp_and_run_multi_layer_type(pp, cfg['bsz'], cfg['mbsz'][pp], cfg['min_tp'],
                                                                 cfg['max_tp'], cfg['vsp'], cfg['embed_sdp'],
                                                                 cfg['sp_search'])
    return canon({'fit': fit, 'per_pp': per_pp})


def canon(x):
    """JSON-able, bit-exact form: floats as hex strings, numpy scalars as Python numbers."""
    if isinstance(x, (bool, np.bool_)):
        return bool(x)
    if isinstance(x, (float, np.floating)):
        return float(x).hex()
    if isinstance(x, (int, np.integer)):
        return int(x)
    if isinstance(x, dict):
        return {str(k): canon(v) for k, v in x.items()}
    if isinstance(x, (list, tuple)):
        return [canon(v) for v in x]
    if isinstance(x, np.ndarray):
        return [canon(v) for v in x.tolist()]
    return x
