"""Writes tests/golden/sweep_golden.json: what the REFERENCE's GalvatronSearchEngine
(galvatron/core/search_engine/search_engine.py) produces for the scenarios of tests/sweep_cases.py:
the strategy lists of generate_strategies (:783-914), the batch-size ranges of set_searching_bsz
(:539-559), and for whole sweeps (parallelism_optimization :339-537 with its own DpOnModel, cost
models and compiled dp_core from oracle/_ref) the best throughput, the text of the
galvatron_config_*.json it writes (:640-688) and the throughput of every task.  Run in the build
container only:

    python oracle/build.py && python tests/golden/make_sweep_golden.py

The reference modules are loaded from where they lie; package __init__ files are not executed
(galvatron.utils is served as its two plain modules, see make_cost_model_golden.py).  The engine's
per-task result table is captured by wrapping its ``dynamic_programming`` method.  The fixture
holds data only.
"""
import contextlib
import importlib
import io
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, HERE)

import cost_model_cases as C  # noqa: E402
import sweep_cases as S  # noqa: E402
from make_cost_model_golden import reference_module  # noqa: E402
from oracle import dp_oracle as O  # noqa: E402


def main():
    _, args_mod, _ = reference_module()
    sys.modules["galvatron_dp_core"] = O.ref_module()
    engine_mod = importlib.import_module("_ref_search_engine.search_engine")
    Engine = engine_mod.GalvatronSearchEngine
    out = {"strategies": [], "bsz": [], "sweeps": {}}
    for case in S.STRATEGY_CASES:
        e = Engine(S.search_args(**case))
        try:
            got = e.generate_strategies()
        except AssertionError:
            got = "AssertionError"
        out["strategies"].append({"case": case, "want": got,
                                  "flags": [e.args.disable_sdp, e.args.disable_pp, e.args.disable_tp, e.args.disable_ckpt]})
    for case in S.BSZ_CASES:
        e = Engine(S.search_args(**case))
        with contextlib.redirect_stdout(io.StringIO()):
            try:
                e.set_searching_bsz()
                got = [e.min_bsz, e.max_bsz, e.bsz_scale, e.BSZs]
            except IndexError:
                got = "IndexError"
        out["bsz"].append({"case": case, "want": got})
    for name in S.SWEEPS:
        # keep what dynamic_programming returns for every task: the engine itself only keeps a local dict
        table = {}
        original = Engine.dynamic_programming

        def spy(self, strategies, bsz, chunk, mbsz_dict, pp_stage_dict, min_tp, max_tp, vsp, embed_sdp, sp_search, logger):
            r = original(self, strategies, bsz, chunk, mbsz_dict, pp_stage_dict, min_tp, max_tp, vsp, embed_sdp, sp_search, logger)
            table['%d/%d/%d/%d/%d/%d/%d' % (bsz, chunk, min_tp, max_tp, vsp, embed_sdp, sp_search)] = [
                C.hexf(r['throughput']), int(r['min_pp_deg']), C.jsonable(r['vtp'])]
            return r

        Engine.dynamic_programming = spy
        try:
            with contextlib.redirect_stdout(io.StringIO()):
                got = S.run(Engine, args_mod, name)
        finally:
            Engine.dynamic_programming = original
        got['table'] = table
        out["sweeps"][name] = got
        print(name, got['throughput'], len(table), list(got['files']), flush=True)
    with open(os.path.join(HERE, "sweep_golden.json"), "w") as fh:
        json.dump(out, fh, separators=(",", ":"))


if __name__ == "__main__":
    main()
