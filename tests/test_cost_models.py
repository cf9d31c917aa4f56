"""The cost models (galvatron_dp/cost_models.py) against numbers recorded from the reference's
classes (tests/golden/cost_model_golden.json, written by tests/golden/make_cost_model_golden.py)
on seeded scenarios, bit for bit (floats as hex), plus closed forms that pin single terms
independently of the fixture."""
import json
import os

import numpy as np
import pytest

import cost_model_cases as C
from galvatron_dp import cost_models as M
from galvatron_dp import pp_utils as PP

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def golden():
    with open(os.path.join(HERE, "golden", "cost_model_golden.json")) as fh:
        return json.load(fh)


@pytest.mark.parametrize("kind,runner", [("memory", C.run_memory), ("time", C.run_time), ("other", C.run_other),
                                         ("pipeline", C.run_pipeline)])
def test_bit_identical_to_recorded_reference_outputs(golden, kind, runner):
    assert len(golden[kind]) >= 100
    for rec in golden[kind]:
        got = runner(M, M, rec["case"])
        assert got == rec["want"], f"{kind} case {rec['case']}"


def test_pipeline_division_bit_identical_to_recorded_reference_outputs(golden):
    assert len(golden["pp"]) >= 100
    kinds = set()
    for rec in golden["pp"]:
        got = C.run_pp(PP, M, rec["case"])
        assert got == rec["want"], f"pp case {rec['case']}"
        kinds.add("none" if rec["want"]["division"] is None else len(rec["want"]["division"]))
    assert {"none", 1, 2, 4, 8} <= kinds          # every pipeline degree and the no-candidate case occur


def test_pipeline_division_closed_forms():
    assert PP.pp_division_even([10], 4) == [2, 2, 2, 4] and PP.pp_division_even([6, 6], 1) == [12]
    assert PP.get_layer_costs([2, 3], [1.0, 5.0]) == [1.0, 1.0, 5.0, 5.0, 5.0]
    # a leading entry for the non-layer memory goes to the first stage, a trailing one to the last
    assert PP.get_cost_all_stages([1, 2, 3, 4], [2, 2]) == [3, 7]
    assert PP.get_cost_all_stages([10, 1, 2, 3, 4], [2, 2]) == [13, 7]
    assert PP.get_cost_all_stages([10, 1, 2, 3, 4, 20], [2, 2]) == [13, 27]
    assert PP.optimal_chunk_func_default(16, [2, 2, 2, {}], 3, 1) == 3.0      # ceil((16 // 2) / 3)
    assert PP.optimal_chunk_func_default(0, [1, 1, 8, {}], 4, 1) == 1
    assert PP.check_optimal_chunks(8, [[1, 1, 8, {}], [2, 1, 4, {}]], PP.optimal_chunk_func_default, 64,
                                   {1: 4, 2: 2}, 1) == {1: 2.0, 2: 8.0}


def test_strategy_text_round_trip(golden):
    for rec in golden["strings"]:
        assert M.form_strategy(rec["strategy"]) == rec["text"]
        assert M.strategy_str2list(rec["text"]) == rec["back"]


def test_micro_batch_split_is_torch_chunk():
    # torch.arange(10).chunk(4) -> sizes 3,3,3,1; .chunk(6) of 9 gives 5 pieces of 2,2,2,2,1
    assert [len(p) for p in M.chunk_like_torch(10, 4)] == [3, 3, 3, 1]
    assert [len(p) for p in M.chunk_like_torch(9, 6)] == [2, 2, 2, 2, 1]
    assert M.get_real_chunk(9, 6) == 5 and M.get_real_chunk(9, 1) == 1
    with pytest.raises(ValueError):
        M.chunk_like_torch(4, 0)
    assert M.get_time_cost_all_stages([1.0, 2.0, 4.0, 8.0], [1, 3]) == [1.0, 14.0]


def _args(**over):
    line = {"popt": [0.02, 0.1]}
    hw = M.ProfileHardwareArgs(allreduce_dict={2: line, 4: line, 8: line}, all2all_dict={2: line, 4: line, 8: line})
    return dict(model_args=M.ModelArgs(parameter_size=48, seq_length=512, hidden_size=1024, layer_num=24),
                train_args=M.TrainArgs(mixed_precision=over.get("mixed", False)),
                parallel_args=M.ParallelArgs(sp_space="tp"), profile_model_args=M.ProfileModelArgs(),
                profile_hardware_args=hw)


def test_time_model_closed_forms():
    # pure data parallel, 8 ranks: ring all-reduce volume 2(d-1)/d * parameters per layer
    t = M.TimeCostModel([1, 1, 8, {"fsdp": 0}], 64, **_args())
    assert t.dp_message_size == (2 * 7 / 8 * 48) * 24
    assert t.fct == 35 / 24 * 8 / 1 * 24 and t.bct == t.fct * 2
    assert t.dc == M.ProfileHardwareArgs().comm_coe_dict["8"]
    # mixed precision halves it; ZeRO-3 gathers half of the volume once more in the forward pass
    t16 = M.TimeCostModel([1, 1, 8, {"fsdp": 1}], 64, **_args(mixed=True))
    assert t16.dp_message_size == t.dp_message_size / 2
    assert t16.fsdp_allgather_message_size == t16.dp_message_size * 0.5
    plain = M.TimeCostModel([1, 1, 8, {"fsdp": 0}], 64, **_args(mixed=True))
    assert t16.gen_result() > plain.gen_result()
    # no parallelism at all: forward + backward, per layer, in seconds
    one = M.TimeCostModel([1, 1, 1, {}], 8, **_args())
    assert one.gen_result() == (one.fct + one.bct) * 0.001 / 24
    # tensor parallel over consecutive ranks uses the '<tp>_1' coefficient, the other layout '<tp>_0'
    a = M.TimeCostModel([1, 2, 4, {"tp": 1, "fsdp": 0}], 64, **_args())
    b = M.TimeCostModel([1, 2, 4, {"tp": 0, "fsdp": 0}], 64, **_args())
    coe = M.ProfileHardwareArgs().comm_coe_dict
    assert a.tp_communication_time == a.tp_message_size * coe["2_1"]
    assert b.tp_communication_time == b.tp_message_size * coe["2_0"]
    assert a.dc == coe["4_0"] and b.dc == coe["4_1"]
    # checkpointing: one more forward in the backward pass, half again as many activation collectives
    c = M.TimeCostModel([1, 2, 4, {"tp": 1, "fsdp": 0, "cpt": 1}], 64, **_args())
    assert c.bct == a.bct + a.fct and c.tp_message_size == a.tp_message_size * 1.5
    # the overlap model: whichever of all-reduce and backward is longer keeps running alone afterwards
    over, rest, flag = a.bct_dp_overlap(a.dp_message_size, a.bct)
    assert flag is False and over <= a.bct * 1.3 and rest >= 0


def test_memory_model_closed_forms():
    prof = M.ProfileModelArgs(tp_activation_per_bsz_dict={1: 85, 2: 47, 4: 28, 8: 18.5, "checkpoint": 10.0},
                              other_memory_pp_off={"model_states": {1: 640, 2: 320, 4: 160, 8: 80},
                                                   "activation": {1: 320, 2: 160, 4: 80, 8: 40}},
                              other_memory_pp_on={s: {"model_states": {1: 640, 2: 320, 4: 160, 8: 80},
                                                      "activation": {1: 320, 2: 160, 4: 80, 8: 40}}
                                                  for s in ("first_stage", "last_stage")})
    kw = dict(global_batch_size=32, mbsz=4, min_tp=1, max_tp=8, model_args=M.ModelArgs(parameter_size=48),
              train_args=M.TrainArgs(mixed_precision=True), profile_model_args=prof)
    par = lambda **o: M.ParallelArgs(optimal_chunk_func=C.chunk_func, **o)          # noqa: E731
    dp = M.MemoryCostModel([1, 1, 8, {"fsdp": 0}], parallel_args=par(), **kw)
    assert dp.chunks == 1 and dp.bsz == 4.0 and dp.sdp_size == 8
    cost = dp.get_memory_cost()
    assert cost["parameter"] == 48 and cost["model_states"] == 4 * 48 and cost["activation"] == 85 * 4.0
    assert cost["enc_total"] == cost["model_states"] + cost["activation"]
    assert sorted(cost["other"]) == [1, 2, 4, 8]
    assert cost["other"][1] == [640 * 1.0 + 320 * (32 * 1 / 1 / 8 / 1) + 1024]
    # ZeRO-3 over 8 ranks, one micro-batch: states shrink to 1/8 (+ the 0.003 margin)
    z3 = M.MemoryCostModel([1, 1, 8, {"fsdp": 1}], parallel_args=par(), **kw)
    assert z3.get_memory_cost()["model_states"] == 4 * 48 * (1 / 8 + 0.003)
    # tensor parallel divides the parameters, Ulysses does not and shards over tp*dp instead
    tp = M.MemoryCostModel([1, 4, 2, {"fsdp": 1, "tp": 1}], parallel_args=par(), **kw)
    ul = M.MemoryCostModel([1, 4, 2, {"fsdp": 1, "tp": 1, "sp": 1}], parallel_args=par(), **kw)
    assert tp.parameter_size == 12 and ul.parameter_size == 48 and tp.sdp_size == 2 and ul.sdp_size == 8
    # checkpointed activations, divided over tp only with sequence parallelism
    ck = M.MemoryCostModel([1, 2, 4, {"fsdp": 0, "tp": 1, "cpt": 1}], parallel_args=par(sequence_parallel=True), **kw)
    ck0 = M.MemoryCostModel([1, 2, 4, {"fsdp": 0, "tp": 1, "cpt": 1}], parallel_args=par(), **kw)
    assert ck.activation_size == 10.0 * ck.bsz / 2 and ck0.activation_size == 10.0 * ck0.bsz
    # 1F1B: stage 0 of 4 holds min(4, chunks) micro-batches, the last stage one
    f = [M.MemoryCostModel([4, 1, 2, {"fsdp": 0}], stage_idx=i, parallel_args=par(pipeline_type="pipedream_flush"), **kw)
         for i in range(4)]
    assert [m.chunks for m in f] == [4] * 4
    assert [m.act_1f1b_ratio for m in f] == [1.0, 0.75, 0.5, 0.25]
    g = M.MemoryCostModel([4, 1, 2, {"fsdp": 0}], parallel_args=par(pipeline_type="gpipe"), **kw)
    assert g.bsz == 4                                        # one micro-batch of 16/4 samples
    with pytest.raises(AssertionError):
        M.MemoryCostModel([1, 1, 8, {}], parallel_args=par(), global_batch_size=8, min_tp=1, model_args=M.ModelArgs(),
                          train_args=M.TrainArgs(), profile_model_args=prof)       # mbsz missing


def test_pipeline_model_degenerate_cases():
    assert M.pipeline_costmodel(M.TimeCostModel, [4], [], [], [], [], [], None, [2, 2], 4, 32, 1, [0, 0]) == np.inf
    stage, total = M.pipeline_costmodel(M.TimeCostModel, [4], [], [], [], [], [], None, [2, 2], 4, 32, 1, [0, 0],
                                        return_stage_cost=True)
    assert stage == [np.inf, np.inf] and total == np.inf
    # one stage, one micro-batch, nothing else: the sum of the layers' times
    a = _args()
    lists = [[a["model_args"]], [a["train_args"]], [a["parallel_args"]], [a["profile_model_args"]],
             [a["profile_hardware_args"]]]
    s = [1, 1, 8, {"fsdp": 0}]
    total = M.pipeline_costmodel(M.TimeCostModel, [3], *lists, [s, s, s], [3], 1, 64, 1, [0.0])
    one = M.TimeCostModel(s, 64, **a).gen_result()
    compute = M.TimeCostModel(s, 64, no_comm=True, **a).gen_result()
    assert total == np.sum([compute] * 3) + max(np.sum([one] * 3) - np.sum([compute] * 3), 0)


# ---- array forms over a whole strategy list ---------------------------------------------------------
def _hex(x):
    return float(x).hex()


def test_memory_rows_equal_the_class_strategy_by_strategy():
    """``memory_cost_rows`` (one array evaluation per strategy list, all pipeline stages at once) gives
    the bits of ``MemoryCostModel`` -- which the recorded reference outputs pin -- for every strategy,
    stage and the first strategy's 'other' entry, on the seeded memory scenarios."""
    compared = 0
    for seed in range(0, C.N_MEMORY, 2):
        c = C.memory_case(seed)
        m, t, p, pm, _ = C._records(M, c['prof'], c['model'], c['train'], c['parallel'])
        rng = np.random.Generator(np.random.PCG64([77, seed]))
        pp = c['strategy'][0]
        strs = [c['strategy']] + [s for s in C.all_strategies()
                                  if s[0] == pp and s[1] % c['kw']['min_tp'] == 0 and rng.random() < 0.5]
        kw = dict(c['kw'])
        stages = list(range(pp)) if p.pipeline_type == 'pipedream_flush' else [kw['stage_idx']]
        kw.pop('stage_idx')
        rows, other = M.memory_cost_rows(strs, stage_idx=stages, model_args=m, train_args=t, parallel_args=p,
                                         profile_model_args=pm, **kw)
        assert rows.shape == (len(stages), len(strs))
        for j, stage in enumerate(stages):
            for i, s in enumerate(strs):
                want = M.MemoryCostModel(s, stage_idx=stage, model_args=m, train_args=t, parallel_args=p,
                                         profile_model_args=pm, **kw).get_memory_cost()
                assert _hex(want['enc_total']) == _hex(rows[j, i]), (seed, stage, s)
                if i == 0 and j == 0:
                    assert C.jsonable(want['other']) == C.jsonable(other), (seed, s)
                compared += 1
        one, _ = M.memory_cost_rows(strs, stage_idx=stages[0], model_args=m, train_args=t, parallel_args=p,
                                    profile_model_args=pm, **kw)
        assert one.shape == (len(strs),) and [_hex(x) for x in one] == [_hex(x) for x in rows[0]]
    assert compared > 2000


def test_time_rows_equal_the_class_strategy_by_strategy():
    compared = 0
    for seed in range(0, C.N_TIME, 2):
        c = C.time_case(seed)
        rng = np.random.Generator(np.random.PCG64([78, seed]))
        strs = [c['strategy']] + [s for s in C.all_strategies() if rng.random() < 0.3]
        m, t, p, pm, hw = C._records(M, c['prof'], c['model'], c['train'], c['parallel'])
        rows = M.time_cost_rows(strs, c['gbsz'], no_comm=c['no_comm'], model_args=m, train_args=t, parallel_args=p,
                                profile_model_args=pm, profile_hardware_args=hw)
        assert m.layer_num is not None                    # written back as the class does
        for i, s in enumerate(strs):
            m2, t2, p2, pm2, hw2 = C._records(M, c['prof'], c['model'], c['train'], c['parallel'])
            want = M.TimeCostModel(s, c['gbsz'], no_comm=c['no_comm'], model_args=m2, train_args=t2, parallel_args=p2,
                                   profile_model_args=pm2, profile_hardware_args=hw2).gen_result()
            assert _hex(want) == _hex(rows[i]), (seed, s)
            compared += 1
    assert compared > 4000


def test_array_forms_decline_what_they_do_not_cover():
    """Inputs on which the class asserts, raises or takes a rare path make the array form raise
    NotVectorisable (its callers then go strategy by strategy), never return something else."""
    a = _args()
    mem = dict(model_args=a['model_args'], train_args=a['train_args'], parallel_args=a['parallel_args'],
               profile_model_args=a['profile_model_args'])
    mem['parallel_args'].chunks = 2
    with pytest.raises(M.NotVectorisable):                # a lane without samples
        M.memory_cost_rows([[1, 8, 1, {}]], 4, 1, 1, 8, **mem)
    with pytest.raises(M.NotVectorisable):                # tensor-parallel degree without an activation entry
        M.memory_cost_rows([[1, 16, 1, {}]], 64, 1, 1, 8, **mem)
    with pytest.raises(M.NotVectorisable):                # min_tp above the strategy's tp
        M.memory_cost_rows([[1, 2, 4, {'fsdp': 0, 'tp': 1}]], 64, 1, 4, 8, **mem)
    with pytest.raises(M.NotVectorisable):                # no layout flag although both tp and dp are above 1
        M.time_cost_rows([[1, 2, 4, {'fsdp': 0}]], 64, **a)
    with pytest.raises(M.NotVectorisable):
        M.time_cost_rows([], 64, **a)


def test_sum_like_numpy_is_numpy_sum_bit_for_bit():
    """Short lists are added without numpy (a sweep makes tens of thousands of such sums); the result must be
    what ``np.sum`` gives, in value, bits and type, for every length on either side of the switch to numpy."""
    import random
    from galvatron_dp.cost_models import sum_like_numpy
    rng = random.Random(5)
    for n in range(0, 13):
        for _ in range(300):
            xs = [rng.choice([1.0, -1.0]) * rng.random() * 10 ** rng.randint(-8, 16) for _ in range(n)]
            if n and rng.random() < 0.3:
                xs = [np.float64(x) for x in xs]
            got, want = sum_like_numpy(xs), np.sum(xs)
            assert np.float64(got).tobytes() == np.float64(want).tobytes() and type(got) is type(want), (xs, got, want)
    assert sum_like_numpy([np.float64(-0.0)]).tobytes() == np.sum([np.float64(-0.0)]).tobytes()
    assert sum_like_numpy([3, 4, 5]) == 12 and type(sum_like_numpy([3, 4, 5])) is type(np.sum([3, 4, 5]))
    assert sum_like_numpy([1e16, 1.0, 1.0]) == (1e16 + 1.0) + 1.0
