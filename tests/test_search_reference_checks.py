"""The checks of the reference's own host-side search tests (tests/search_engine/test_pp_utils.py:17-155,
test_bsz_utils.py:7-98, test_generate_strategies.py:10-46 of the reference) applied to
galvatron_dp.pp_utils and galvatron_dp.search: the same inputs, the same expected values."""
import copy

import numpy as np
import pytest

import profile_cases as P
from galvatron_dp.cost_models import form_strategy
from galvatron_dp.pp_utils import (check_optimal_chunks, get_pp_stage_for_bsz, optimal_chunk_func_default,
                                   pp_division_memory_balanced)
from galvatron_dp.search import SearchEngine
from test_cost_models_reference_checks import memory_settings, records

STRATEGIES_PP4 = [[4, 1, 8, {}], [4, 2, 4, {}], [4, 4, 2, {}]]


def two_layer_types():
    lists = [[], [], [], [], []]
    for _ in range(2):
        for lst, rec in zip(lists, records(copy.deepcopy(memory_settings()))):
            lst.append(rec)
    return lists


def test_pp_division_memory_balanced():
    model, train, parallel, profile, _ = two_layer_types()
    layer_num, pp_deg = [16, 16], 4
    division, per_stage = pp_division_memory_balanced(model, train, parallel, profile, layer_num, pp_deg, 32, 8,
                                                      STRATEGIES_PP4)
    assert division is not None and len(division) == pp_deg
    assert sum(division) == sum(layer_num) and all(n > 0 for n in division)
    assert (max(per_stage) - min(per_stage)) / max(per_stage) < 0.3


@pytest.mark.parametrize("single_layer_even", [True, False])
def test_get_pp_stage_for_bsz(single_layer_even):
    model, train, parallel, profile, _ = two_layer_types()
    stages = get_pp_stage_for_bsz(STRATEGIES_PP4, model, train, parallel, profile, [16, 16], 32, {1: 8, 2: 8, 4: 8},
                                  single_layer_even)
    assert isinstance(stages, dict) and 4 in stages and sum(stages[4]) == 32


@pytest.mark.parametrize("world_size,bsz,min_tp", [(8, 32, 1), (16, 64, 2), (32, 128, 4)])
def test_check_optimal_chunks(world_size, bsz, min_tp):
    strategies = [[pp, min_tp, world_size // (pp * min_tp), {'fsdp': 0, 'cpt': 0}] for pp in (2, 4)]
    mbsz = {2: 8, 4: 4}
    chunks = check_optimal_chunks(world_size, strategies, optimal_chunk_func_default, bsz, mbsz, min_tp)
    assert set(chunks) == {2, 4}
    for pp, n in chunks.items():
        assert isinstance(n, (int, float)) and n > 0
        assert n == np.ceil(bsz / (world_size // pp // min_tp) / mbsz[pp])


def bsz_engine(**over):
    return SearchEngine(P.reference_test_args(gpu_num=8, min_bsz=16, max_bsz=64, bsz_scale=8, recommend_min_bsz=False,
                                              **over))


def test_settle_bsz():
    e = bsz_engine(settle_bsz=20)
    e.set_searching_bsz()
    assert (e.min_bsz, e.max_bsz, e.bsz_scale, e.BSZs) == (20, 20, 0, [20])


def test_normal_bsz_range():
    e = bsz_engine()
    e.set_searching_bsz()
    assert (e.min_bsz, e.max_bsz, e.bsz_scale, e.BSZs) == (16, 64, 8, [16, 24, 32, 40, 48, 56, 64])


@pytest.mark.parametrize("lo,hi,scale,expected", [(20, 50, 10, [20, 30, 40, 50]), (15, 45, 15, [15, 30, 45]),
                                                  (32, 96, 32, [32, 64, 96])])
def test_bsz_range_with_different_scales(lo, hi, scale, expected):
    e = bsz_engine()
    e.args.min_bsz, e.args.max_bsz, e.args.bsz_scale = lo, hi, scale
    e.set_searching_bsz()
    assert e.BSZs == expected and e.min_bsz == expected[0] and e.max_bsz == expected[-1]


@pytest.mark.parametrize("recommended,expected", [(24, 24), (-1, 16)])
def test_recommended_min_bsz(monkeypatch, recommended, expected):
    e = bsz_engine()
    monkeypatch.setattr(e, 'recommend_min_bsz', lambda scale: recommended)
    e.args.recommend_min_bsz = True
    e.set_searching_bsz()
    assert e.min_bsz == expected


def test_bsz_edges():
    e = bsz_engine()
    e.args.max_bsz, e.args.bsz_scale = 50, 16
    e.set_searching_bsz()
    assert e.max_bsz == int(np.ceil(50 / 16) * 16) - 16
    e = bsz_engine()
    e.args.min_bsz, e.args.bsz_scale = 4, 8
    e.set_searching_bsz()
    assert e.min_bsz == 8


FULL_TP_SP = ("1-1-8, 1-1-8f, 1-2-4*, 1-2-4*-sp, 1-2-4f*, 1-2-4f*-sp, 1-2*-4, 1-2*-4-sp, 1-2*-4f, 1-2*-4f-sp, 1-4-2*, "
              "1-4-2*-sp, 1-4-2f*, 1-4-2f*-sp, 1-4*-2, 1-4*-2-sp, 1-4*-2f, 1-4*-2f-sp, 1-8-1, 1-8-1-sp, 2-1-4, 2-1-4f, "
              "2-2-2*, 2-2-2*-sp, 2-2-2f*, 2-2-2f*-sp, 2-2*-2, 2-2*-2-sp, 2-2*-2f, 2-2*-2f-sp, 2-4-1, 2-4-1-sp, 4-1-2, "
              "4-1-2f, 4-2-1, 4-2-1-sp, 8-1-1, 1-1-8-c, 1-1-8f-c, 1-2-4*-c, 1-2-4*-c-sp, 1-2-4f*-c, 1-2-4f*-c-sp, "
              "1-2*-4-c, 1-2*-4-c-sp, 1-2*-4f-c, 1-2*-4f-c-sp, 1-4-2*-c, 1-4-2*-c-sp, 1-4-2f*-c, 1-4-2f*-c-sp, 1-4*-2-c, "
              "1-4*-2-c-sp, 1-4*-2f-c, 1-4*-2f-c-sp, 1-8-1-c, 1-8-1-c-sp, 2-1-4-c, 2-1-4f-c, 2-2-2*-c, 2-2-2*-c-sp, "
              "2-2-2f*-c, 2-2-2f*-c-sp, 2-2*-2-c, 2-2*-2-c-sp, 2-2*-2f-c, 2-2*-2f-c-sp, 2-4-1-c, 2-4-1-c-sp, 4-1-2-c, "
              "4-1-2f-c, 4-2-1-c, 4-2-1-c-sp, 8-1-1-c")


@pytest.mark.parametrize("search_space", ["dp+tp", "dp+pp", "3d", "dp", "tp", "pp", "sdp", "full"])
@pytest.mark.parametrize("sp_space", ["tp", "sp", "tp+sp"])
def test_generate_strategies(tmp_path, search_space, sp_space):
    e = SearchEngine(P.reference_test_args(search_space=search_space, sp_space=sp_space))
    e.set_search_engine_info(str(tmp_path), P.LAYER_CONFIGS, P.MODEL_NAME)
    e.generate_strategies()
    if search_space == "full" and sp_space == "tp+sp":
        assert len(e.strategies) == 74
        assert ", ".join(form_strategy(s) for s in e.strategies) == FULL_TP_SP
    else:
        assert len(e.strategies) > 0
