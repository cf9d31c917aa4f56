"""The checks of the reference's own cost-model tests (tests/search_engine/test_cost_model.py:18-630 of
the reference) applied to galvatron_dp.cost_models: the same strategies and settings, the same mock
profile (tests/utils/cost_args.py:13-121, from the profile data in tests/golden/search_profiles.json),
the same attributes read back from the model objects and the same expected relations."""
import pytest

import profile_cases as P
from galvatron_dp import cost_models as M
from galvatron_dp import profile_configs
from galvatron_dp.pp_utils import optimal_chunk_func_default

RECORD_FIELDS = {
    M.ModelArgs: ['parameter_size', 'seq_length', 'hidden_size', 'layer_num'],
    M.TrainArgs: ['mixed_precision', 'checkpoint', 'async_grad_reduce', 'pytorch_context_mem'],
    M.ParallelArgs: ['use_zero2_for_dp', 'disable_vtp', 'sequence_parallel', 'sp_space', 'pipeline_type',
                     'optimal_chunk_func', 'chunks'],
    M.ProfileModelArgs: ['tp_activation_per_bsz_dict', 'other_memory_pp_off', 'other_memory_pp_on',
                         'forward_computation_time', 'other_time_profiled'],
    M.ProfileHardwareArgs: ['bct_fct_coe', 'extra_overhead', 'comm_coe_dict', 'dp_overlap_coe', 'bct_overlap_coe',
                            'p2p_comm_coe_dict', 'allreduce_dict', 'all2all_dict', 'costmodel_coe'],
}


def records(settings):
    """The five records with their defaults, every setting written into the record that has a field
    of that name (tests/utils/cost_args.py:123-168)."""
    out = []
    for cls, fields in RECORD_FIELDS.items():
        rec = cls()
        for k, v in settings.items():
            if k in fields:
                setattr(rec, k, v)
        out.append(rec)
    return out


def memory_settings():
    mc = profile_configs.int_keys(P.profiles()["memory"]["static"])
    pick = lambda table: {k: mc[table][4096][k] for k in ('model_states', 'activation')}
    return dict(parameter_size=mc['layertype_0'][4096]['parameter_size'],
                tp_activation_per_bsz_dict=mc['layertype_0'][4096]['tp_activation_per_bsz_dict'],
                other_memory_pp_off=pick('other_memory_pp_off'),
                other_memory_pp_on={'first_stage': pick('other_memory_pp_on_first'),
                                    'last_stage': pick('other_memory_pp_on_last')},
                pipeline_type='gpipe', mixed_precision=True, use_zero2_for_dp=0, use_zero3_for_embed=0, disable_vtp=0,
                max_tp_deg=8, gpu_num=8, vsp=0, optimal_chunk_func=optimal_chunk_func_default)


def time_settings():
    data = P.profiles()
    hw = data["hardware"]
    return dict(parameter_size=48, microbatch=False, optimal_chunk_func=optimal_chunk_func_default, sequence_length=512,
                hidden_size=1024, forward_computation_time=data["time"]["static"]['layertype_0_bsz8_seq4096'],
                bct_fct_coe=2, extra_overhead=0,
                comm_coe_dict=profile_configs.read_allreduce_bandwidth_config(hw['allreduce'], 8)[1],
                dp_overlap_coe=hw['overlap']['overlap_coe'], bct_overlap_coe=hw['overlap']['overlap_coe'],
                p2p_comm_coe_dict=profile_configs.read_p2p_bandwidth_config(hw['p2p'])[1], layer_num=None,
                use_zero2_for_dp=0, mixed_precision=False, no_comm=False, costmodel_coe=1.0, async_grad_reduce=True,
                allreduce_dict=profile_configs.remap_config(hw['sp'], 'allreduce'),
                all2all_dict=profile_configs.remap_config(hw['sp'], 'all2all'), sp_space='tp')


CPT_ACT = {1: 85, 2: 47, 4: 28, 8: 18.5, 'checkpoint': 10.0}

MEMORY_CASES = [  # test_cost_model.py:19-118
    ([1, 1, 8, {'fsdp': 0}],
     dict(global_batch_size=32, pipeline_type='gpipe', sequence_parallel=True, use_zero2_for_dp=0),
     dict(sdp_size=8, pp_stages=1, check_activation=True)),
    ([1, 2, 4, {'fsdp': 0, 'cpt': 1}],
     dict(global_batch_size=32, tp_activation_per_bsz_dict=CPT_ACT, sequence_parallel=True),
     dict(sdp_size=4, has_checkpoint=True, check_tp_division=True)),
    ([1, 4, 2, {'sp': 1, 'cpt': 1}],
     dict(global_batch_size=32, parameter_size=48, sequence_parallel=True, tp_activation_per_bsz_dict=CPT_ACT,
          mixed_precision=True, async_grad_reduce=True),
     dict(sdp_size=8, check_sp=True, has_checkpoint=True)),
    ([2, 1, 4, {'fsdp': 1}],
     dict(global_batch_size=32, pipeline_type='pipedream_flush', mixed_precision=True, async_grad_reduce=True),
     dict(pp_stages=2, has_fsdp=True, check_pipeline=True)),
    ([2, 2, 2, {'fsdp': 0}],
     dict(global_batch_size=32, use_zero2_for_dp=1, mixed_precision=True, vsp=1, disable_vtp=0, async_grad_reduce=True),
     dict(pp_stages=2, has_zero2=True, has_vsp=True, check_hybrid=True)),
    ([1, 4, 2, {'fsdp': 1}],
     dict(global_batch_size=16, vsp=1, async_grad_reduce=False, mixed_precision=True),
     dict(has_vsp=True, has_fsdp=True, check_async_grad=True)),
]


@pytest.mark.parametrize("strategy,updates,expected", MEMORY_CASES)
def test_memory_cost_model(strategy, updates, expected):
    a = memory_settings()
    a.update(updates, mbsz=2, min_tp=1, max_tp=8)
    model_args, train_args, parallel_args, profile_model_args, _ = records(a)
    model = M.MemoryCostModel(strategy=strategy, global_batch_size=a.get('global_batch_size', 8), mbsz=a['mbsz'],
                              min_tp=a['min_tp'], max_tp=a['max_tp'], stage_idx=a.get('stage_idx', 0),
                              vsp=a.get('vsp', 0), embed_sdp=a.get('embed_sdp', False), model_args=model_args,
                              train_args=train_args, parallel_args=parallel_args, profile_model_args=profile_model_args)
    costs = model.get_memory_cost()
    assert isinstance(costs, dict)
    assert all(k in costs for k in ['parameter', 'model_states', 'activation', 'enc_total', 'other'])
    if 'sdp_size' in expected:
        assert model.sdp_size == expected['sdp_size']
    if 'pp_stages' in expected:
        assert len(costs['other'][1]) == expected['pp_stages']
    act, mixed, async_ = a['tp_activation_per_bsz_dict'], a['mixed_precision'], a.get('async_grad_reduce', True)
    if expected.get('has_checkpoint'):
        if a['sequence_parallel']:
            assert model.activation_size == act['checkpoint'] * model.bsz / model.tp_size
        else:
            assert model.activation_size == act['checkpoint'] * model.bsz
    if expected.get('has_fsdp'):
        if model.chunks == 1:
            ratio = lambda d: 1 / d + 0.003
        elif async_:
            ratio = (lambda d: 7 / 8 * (1 / d + 0.003) + 1 / 8) if mixed else (lambda d: 3 / 4 * (1 / d + 0.003) + 1 / 4)
        else:
            ratio = lambda d: (1 / d + 0.003) * 5 / 4
        assert model.model_states_size == 4 * costs['parameter'] * ratio(model.sdp_size)
    if expected.get('has_zero2'):
        if model.chunks == 1:
            ratio = (lambda d: 7 / 8 * (1 / d + 0.003) + 1 / 8) if mixed else (lambda d: 3 / 4 * (1 / d + 0.003) + 1 / 4)
        elif async_:
            ratio = (lambda d: 6 / 8 * (1 / d + 0.003) + 2 / 8) if mixed else (lambda d: 2 / 4 * (1 / d + 0.003) + 2 / 4)
        else:
            ratio = (lambda d: (7 / 8 * (1 / d + 0.003) + 1 / 8) * 5 / 4) if mixed else (lambda d: 3 / 4 * (1 / d + 0.003) + 1 / 4)
        assert abs(model.model_states_size - costs['parameter'] * 4 * ratio(model.sdp_size)) < 1e-6
    if expected.get('has_vsp'):
        if strategy[-1].get('sp') == 1:
            assert model.parameter_size == a['parameter_size']
        else:
            assert model.parameter_size == a['parameter_size'] / model.tp_size
    if expected.get('check_activation'):
        assert model.activation_size == act[model.tp_size] * model.bsz
    if expected.get('check_tp_division'):
        assert costs['parameter'] == a['parameter_size'] / model.tp_size
    if expected.get('check_pipeline') and a['pipeline_type'] == 'pipedream_flush':
        assert model.bsz != updates['global_batch_size'] / model.dp_size
    if expected.get('check_hybrid'):
        assert model.tp_size > 1 and model.pp_size > 1
        assert model.parameter_size == a['parameter_size'] / model.tp_size
    if expected.get('check_async_grad') and not async_:
        assert model.model_states_size > costs['parameter'] * 4 / model.tp_size
    if expected.get('check_sp'):
        assert model.sdp_size == model.tp_size * model.dp_size


TIME_CASES = [  # test_cost_model.py:224-300
    ([1, 1, 8, {'fsdp': 0, 'tp': 1}],
     dict(global_batch_size=32, microbatch=False, comm_coe_dict={'8': 1.0, '8_1': 0.8, '1': 1.0, '1_1': 1.0},
          allreduce_dict={1: 1.0}, all2all_dict={1: 1.0}),
     dict(check_dp=True, has_overlap=True)),
    ([1, 4, 2, {'fsdp': 0, 'tp': 1, 'cpt': 1}],
     dict(global_batch_size=32, microbatch=False, sequence_length=1024, hidden_size=2048, sp_space='tp'),
     dict(check_tp=True, has_checkpoint=True)),
    ([2, 1, 4, {'fsdp': 1, 'tp': 1}],
     dict(global_batch_size=32, microbatch=False, p2p_comm_coe_dict={2: 1.0, 4: 0.8, 8: 0.6}, mixed_precision=True),
     dict(check_pp=True, has_fsdp=True)),
    ([1, 4, 2, {'sp': 1, 'tp': 1}],
     dict(global_batch_size=32, microbatch=False, sp_space='tp+sp', sequence_length=1024, hidden_size=2048),
     dict(check_sp=True, check_tp_comm=True)),
    ([2, 2, 2, {'fsdp': 0, 'tp': 0}],
     dict(global_batch_size=32, microbatch=False, no_comm=True),
     dict(check_hybrid=True, check_no_comm=True)),
]


@pytest.mark.parametrize("strategy,updates,expected", TIME_CASES)
def test_time_cost_model(strategy, updates, expected):
    a = time_settings()
    a.update(updates)
    model_args, train_args, parallel_args, profile_model_args, profile_hardware_args = records(a)
    model = M.TimeCostModel(strategy=strategy, global_batch_size=a.get('global_batch_size', 8),
                            no_comm=a.get('no_comm', False), model_args=model_args, train_args=train_args,
                            parallel_args=parallel_args, profile_model_args=profile_model_args,
                            profile_hardware_args=profile_hardware_args)
    result = model.gen_result()
    assert isinstance(result, float) and result >= 0
    assert (model.pp_size, model.tp_size, model.dp_size) == tuple(strategy[:3])
    mixed = a['mixed_precision']
    if expected.get('check_dp'):
        size = (2 * (model.dp_size - 1) / model.dp_size * model.parameter_size) * model.layer_num
        if mixed:
            size /= 2
        assert model.dp_message_size == size
        if expected.get('has_overlap'):
            overlap_part, _, _ = model.bct_dp_overlap(model.dp_message_size, model.bct)
            assert overlap_part > 0
    want_tp = None
    if expected.get('check_tp') and a['sp_space'] == 'tp':
        want_tp = 2 * (model.tp_size - 1) / model.tp_size * \
            (model.bsz * model.seq_len * model.hidden_size * 4 * 4 / 1024 / 1024) * model.layer_num
        if mixed:
            want_tp /= 2
        if not model.checkpoint:
            assert abs(model.tp_message_size - want_tp) < 1e-6
    if expected.get('check_pp') and model.p2p_comm_coe is not None:
        size = model.pp_size * 2 * model.bsz * model.seq_len * model.hidden_size * 4 / 1024 / 1024
        if mixed:
            size /= 2
        assert model.p2p_message_size == size
    if expected.get('check_sp'):
        assert model.sdp_size == model.tp_size * model.dp_size
        assert model.parameter_size == a['parameter_size']
        if expected.get('check_tp_comm'):
            assert model.per_tp_message_size == model.bsz * model.seq_len * model.hidden_size * (2 if mixed else 4)
            assert model.tp_comm_num == 4 * model.layer_num
    if expected.get('has_checkpoint'):
        assert model.checkpoint and model.bct > model.fct
        if a['sp_space'] == 'tp+sp':
            assert model.tp_comm_num == 6 * model.layer_num
        else:
            assert model.tp_message_size == 1.5 * want_tp
    if expected.get('has_fsdp'):
        assert model.fsdp
        assert model.fsdp_allgather_message_size == model.dp_message_size * 0.5
    if expected.get('check_hybrid'):
        assert model.pp_size > 1 and model.tp_size > 1 and model.dp_size > 1
    if expected.get('check_no_comm'):
        assert model.dp_message_size == 0


def other_settings():  # test_cost_model.py:431-483
    table = {n: {1024: 0.1, 2048: 0.2, 4096: 0.4, 'popt': [0.0001, 0.1]} for n in (2, 4, 8)}
    states = {1: 640, 2: 320, 4: 160, 8: 80}
    return dict(mbsz=4, pp_deg=1, world_size=8, sequence_length=[1024], hidden_size=1024, mixed_precision=False,
                comm_coe_dict={'1': 1.0, '1_1': 1.0, '2': 0.8, '2_1': 0.8, '2_0': 0.9, '4': 0.6, '4_1': 0.6, '4_0': 0.7,
                               '8': 0.5, '8_1': 0.5, '8_0': 0.6},
                allreduce_dict=table, sp_space='tp', vsp=0, min_tp=1, max_tp=8,
                other_memory_pp_on={'first_stage': {'model_states': dict(states)},
                                    'last_stage': {'model_states': dict(states)}},
                other_memory_pp_off={'model_states': dict(states)}, other_time_profiled_list=35.0)


OTHER_CASES = [  # test_cost_model.py:486-553
    (dict(pp_deg=1, world_size=8, min_tp=1, max_tp=4), dict(tp_sizes=[1, 2, 4], has_pp=False)),
    (dict(pp_deg=4, world_size=8, min_tp=1, max_tp=4), dict(tp_sizes=[1, 2], has_pp=True)),
    (dict(pp_deg=1, world_size=8, vsp=1, min_tp=1, max_tp=4), dict(tp_sizes=[1, 2, 4], check_vsp=True)),
    (dict(pp_deg=1, world_size=8, mixed_precision=True, min_tp=1, max_tp=4),
     dict(tp_sizes=[1, 2, 4], check_precision=True)),
    (dict(pp_deg=1, world_size=8, sp_space='tp+sp', min_tp=1, max_tp=4), dict(tp_sizes=[1, 2, 4], check_sp_tp=True)),
]


@pytest.mark.parametrize("updates,expected", OTHER_CASES)
def test_other_time_cost_model(updates, expected):
    a = other_settings()
    a.update(updates)
    model_args, train_args, parallel_args, profile_model_args, profile_hardware_args = records(a)
    profile_model_args.other_time_profiled = a['other_time_profiled_list']
    model = M.OtherTimeCostModel(mbsz=a['mbsz'], pp_deg=a['pp_deg'], world_size=a['world_size'], vsp=a.get('vsp', False),
                                 embed_sdp=a.get('embed_sdp', False), min_tp=a['min_tp'], max_tp=a['max_tp'],
                                 sequence_length_list=a['sequence_length'], model_args=model_args,
                                 train_args=train_args, parallel_args=parallel_args,
                                 profile_model_args=profile_model_args, profile_hardware_args=profile_hardware_args)
    result, _ = model.gen_result()
    assert isinstance(result, dict) and set(result) == set(expected['tp_sizes'])
    for tp in expected['tp_sizes']:
        assert len(result[tp]) == a['pp_deg'] and all(v >= 0 for v in result[tp])
        if expected.get('has_pp'):
            assert abs(result[tp][0] - result[tp][-1]) < 1e-6
        else:
            assert len(result[tp]) == 1
        if expected.get('check_vsp'):
            assert model.dp_size[tp] == a['other_memory_pp_off']['model_states'][1] / 4
        if expected.get('check_sp_tp') and tp > 1:
            assert model.per_tp_message_size[0] == a['mbsz'] * a['sequence_length'][0] * a['hidden_size'] * \
                (2 if a['mixed_precision'] else 4)
    if expected.get('check_precision'):
        last = expected['tp_sizes'][-1]
        assert model.tp_message_size[0] == (last - 1) / last * \
            (a['mbsz'] * a['sequence_length'][0] * a['hidden_size'] / 1024 / 1024) * 2
