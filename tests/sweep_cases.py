"""Scenarios for the sweep driver, shared by tests/golden/make_sweep_golden.py (which runs them through
the reference's GalvatronSearchEngine: search_engine.py:339-688,783-914, fed with the argument
records directly instead of profile files) and the tests (galvatron_dp.search.SearchEngine)."""
import os
import tempfile
from types import SimpleNamespace

import numpy as np

import cost_model_cases as C


def search_args(**over):
    """The search flags with the reference's defaults where a sweep reads them
    (galvatron/core/search_engine/arguments.py)."""
    a = dict(num_nodes=1, num_gpus_per_node=8, memory_constraint=8, use_pipeline_costmodel=1, max_tp_deg=8,
             max_pp_deg=8, disable_vtp=0, global_memory_buffer=1, sp_space='tp+sp', disable_dp=0, disable_sdp=0,
             disable_tp=0, disable_pp=0, disable_ckpt=0, disable_tp_consec=0, parallel_search=False, settle_bsz=-1,
             settle_chunk=-1, bsz_scale=8, min_bsz=8, max_bsz=64, recommend_min_bsz=0, search_space='full',
             pipeline_type='pipedream_flush', default_dp_type='ddp', mixed_precision='bf16', sequence_parallel=True,
             hidden_size=4096, fine_grained_mode=1, output_config_path=None, log_dir=None,
             memory_profiling_path=None, time_profiling_path=None, embed_sdp=0, async_grad_reduce=True,
             costmodel_coe=1.0, worker=0)
    a.update(over)
    return SimpleNamespace(**a)


STRATEGY_CASES = [dict(search_space=space, sp_space=sp, num_gpus_per_node=gpus, max_tp_deg=mtp, max_pp_deg=mpp, **off)
                  for space in ('full', 'dp+tp', 'dp+pp', '3d', 'dp', 'sdp', 'tp', 'pp')
                  for sp in ('tp', 'tp+sp', 'sp')
                  for gpus, mtp, mpp in ((8, 8, 8), (16, 4, 2), (4, 2, 4))
                  for off in ({}, {'disable_ckpt': 1, 'disable_tp_consec': 1}, {'disable_sdp': 1, 'disable_pp': 1},
                              {'disable_dp': 1})]

BSZ_CASES = [dict(settle_bsz=20), dict(min_bsz=16, max_bsz=64, bsz_scale=8), dict(min_bsz=20, max_bsz=50, bsz_scale=10),
             dict(min_bsz=15, max_bsz=45, bsz_scale=15), dict(min_bsz=32, max_bsz=96, bsz_scale=32),
             dict(min_bsz=3, max_bsz=70, bsz_scale=16), dict(min_bsz=100, max_bsz=64, bsz_scale=8)]

SWEEPS = {
    # one layer type, both sequence-parallel search spaces, every chunk count that divides the batch
    'llama_like': dict(args=dict(settle_bsz=32, max_tp_deg=4, memory_constraint=8), layers=[(12, 4096, 2048)],
                       params=[96.0], profile_seeds=[41]),
    # two layer types (memory-balanced stage division), tensor parallel only, no vocabulary tp sweep
    'two_types_tp': dict(args=dict(settle_bsz=64, settle_chunk=4, sp_space='tp', disable_vtp=1, memory_constraint=10,
                                   pipeline_type='gpipe', mixed_precision='fp32', disable_ckpt=1),
                         layers=[(6, 4096, 2048), (8, 4096, 512)], params=[140.0, 70.0], profile_seeds=[42, 43]),
    # nothing fits
    'no_room': dict(args=dict(settle_bsz=64, settle_chunk=1, max_tp_deg=2, memory_constraint=1, disable_vtp=1,
                              sp_space='tp'), layers=[(12, 4096, 2048)], params=[300.0], profile_seeds=[44]),
    # a range of batch sizes
    'bsz_range': dict(args=dict(min_bsz=16, max_bsz=32, bsz_scale=16, settle_chunk=2, max_tp_deg=2, sp_space='tp',
                                global_memory_buffer=0, memory_constraint=12, disable_sdp=1),
                      layers=[(10, 4096, 1024)], params=[80.0], profile_seeds=[45]),
    # one strategy for all layers of a stage (the coarse branch of DPAlg.fit, dynamic_programming.py:62-75)
    'coarse': dict(args=dict(settle_bsz=32, settle_chunk=2, max_tp_deg=4, memory_constraint=8, fine_grained_mode=0),
                   layers=[(12, 4096, 2048)], params=[96.0], profile_seeds=[46]),
    # no pipeline cost model behind the DP, ZeRO-2 as the data-parallel default, gradients reduced synchronously
    'flat_zero2': dict(args=dict(settle_bsz=48, max_tp_deg=4, memory_constraint=10, use_pipeline_costmodel=0,
                                 default_dp_type='zero2', sp_space='tp'),
                       layers=[(8, 4096, 2048)], params=[120.0], profile_seeds=[47],
                       train=dict(async_grad_reduce=False), parallel=dict(use_zero2_for_dp=True)),
    # no pipeline parallelism at all, two layer types, checkpointing and consecutive-tp variants off
    'no_pp': dict(args=dict(settle_bsz=16, search_space='dp+tp', disable_ckpt=1, disable_tp_consec=1,
                            memory_constraint=14, max_tp_deg=8),
                  layers=[(4, 4096, 1024), (6, 4096, 2048)], params=[60.0, 110.0], profile_seeds=[48, 49]),
}


def build(engine_cls, args_mod, name, workdir):
    """An engine of ``engine_cls`` (the reference's GalvatronSearchEngine or galvatron_dp.search.SearchEngine)
    set up for sweep ``name``, writing into ``workdir``."""
    cfg = SWEEPS[name]
    args = search_args(output_config_path=workdir, log_dir=os.path.join(workdir, 'logs'), **cfg['args'])
    engine = engine_cls(args)
    layer_configs = [dict(layer_num=n, hidden_size=h, seq_len=s) for n, h, s in cfg['layers']]
    lists = [[], [], [], [], []]
    for i, (n, h, s) in enumerate(cfg['layers']):
        prof = C.profile(np.random.Generator(np.random.PCG64([77, cfg['profile_seeds'][i]])))
        model = dict(parameter_size=cfg['params'][i], seq_length=s, hidden_size=h, layer_num=24)
        train = dict(mixed_precision=args.mixed_precision != 'fp32', async_grad_reduce=True, pytorch_context_mem=1024)
        train.update(cfg.get('train', {}))
        parallel = dict(use_zero2_for_dp=False, disable_vtp=bool(args.disable_vtp), sequence_parallel=True,
                        sp_space=args.sp_space, pipeline_type=args.pipeline_type, optimal_chunk_func=C.chunk_func,
                        chunks=None)
        parallel.update(cfg.get('parallel', {}))
        for lst, rec in zip(lists, C._records(args_mod, prof, model, train, parallel)):
            lst.append(rec)
    if hasattr(engine, 'set_model'):
        engine.set_model('sweep_' + name, layer_configs, path=workdir)
        engine.set_cost_model_args(*lists, allreduce_comm_coe=lists[4][0].comm_coe_dict)
    else:                                              # the reference's engine: the same state, set by hand
        engine.set_model_layer_configs(layer_configs)
        engine.set_path(workdir)
        engine.set_model_name('sweep_' + name)
        (engine.model_args_list, engine.train_args_list, engine.parallel_args_list, engine.profile_model_args_list,
         engine.profile_hardware_args_list) = lists
        engine.allreduce_comm_coe = lists[4][0].comm_coe_dict
    engine.generate_strategies()
    return engine


def summarize(engine, throughput, workdir):
    """What a sweep produced, JSON-able: best throughput, the result file's name and text, and the
    throughput of every (task, sp_search)."""
    files = sorted(f for f in os.listdir(workdir) if f.endswith('.json'))
    texts = {f: open(os.path.join(workdir, f)).read() for f in files}
    table = {}
    results = getattr(engine, 'results', None)
    if results is not None:
        for bsz, a in results.items():
            for chunk, b in a.items():
                for min_tp, c in b.items():
                    for max_tp, d in c.items():
                        for vsp, e in d.items():
                            for embed_sdp, f in e.items():
                                for sp_search, entry in f.items():
                                    key = '%d/%d/%d/%d/%d/%d/%d' % (bsz, chunk, min_tp, max_tp, vsp, embed_sdp, sp_search)
                                    table[key] = [C.hexf(entry['throughput']), int(entry['min_pp_deg']),
                                                  C.jsonable(entry['vtp'])]
    return {'throughput': C.hexf(throughput), 'files': texts, 'table': table}


def run(engine_cls, args_mod, name):
    with tempfile.TemporaryDirectory() as workdir:
        engine = build(engine_cls, args_mod, name, workdir)
        throughput = engine.parallelism_optimization()
        return summarize(engine, throughput, workdir)
