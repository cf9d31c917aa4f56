"""Writes two fixtures for the part of the search engine that starts from the profilers' files
(galvatron/core/search_engine/search_engine.py:45-337) and for whole searches from them:

tests/golden/search_profiles.json -- the profile DATA the reference's own tests hold
  (tests/utils/search_configs.py:9-547: the dict literals returned by its ``create_*`` functions), read
  out of that file's syntax tree with ``ast.literal_eval``; nothing of the file is executed.

tests/golden/search_profile_golden.json -- what the REFERENCE's GalvatronSearchEngine holds after
  ``initialize_search_engine`` for the nine loading scenarios of tests/profile_cases.py, and what
  ``parallelism_optimization`` returns and writes for the two whole searches (its own DpOnModel, cost
  models and the compiled dp_core from oracle/_ref), together with the throughput of every task.

Run in the build container only:

    python oracle/build.py && python tests/golden/make_search_profile_golden.py

The reference modules are loaded from where they lie; package __init__ files are not executed (see
make_cost_model_golden.py).  The fixtures hold data only.
"""
import ast
import contextlib
import importlib
import io
import json
import os
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, HERE)

import cost_model_cases as C  # noqa: E402
import profile_cases as P  # noqa: E402
import sweep_cases as S  # noqa: E402
from make_cost_model_golden import reference_module  # noqa: E402
from oracle import dp_oracle as O  # noqa: E402

REF_FIXTURES = "/root/reference/tests/utils/search_configs.py"


def returned_literals(path):
    """{function name: the dict literal it returns} for the zero-argument ``create_*`` functions."""
    tree = ast.parse(open(path).read())
    out = {}
    for node in tree.body:
        if isinstance(node, ast.FunctionDef) and node.name.startswith("create_"):
            ret = [n for n in node.body if isinstance(n, ast.Return)]
            assert len(ret) == 1, node.name
            out[node.name] = ast.literal_eval(ret[0].value)
    return out


def profile_data():
    lit = returned_literals(REF_FIXTURES)
    return {"time": {"static": lit["create_static_time_config"], "batch": lit["create_batch_time_config"],
                     "sequence": lit["create_sequence_time_config"]},
            "memory": {"static": lit["create_static_memory_config"], "static_sp": lit["create_static_memory_config_sp"],
                       "sequence_sp": lit["create_sequence_memory_config_sp"]},
            "hardware": lit["create_hardware_configs"]}


def main():
    data = profile_data()
    with open(P.PROFILES, "w") as fh:
        json.dump(data, fh, separators=(",", ":"))
    _, args_mod, _ = reference_module()
    sys.modules["galvatron_dp_core"] = O.ref_module()
    Engine = importlib.import_module("_ref_search_engine.search_engine").GalvatronSearchEngine
    out = {"loading": [], "e2e": {}}
    for modes in P.LOADING_CASES:
        with tempfile.TemporaryDirectory() as workdir, contextlib.redirect_stdout(io.StringIO()):
            engine = P.build(Engine, data, workdir, modes)
            out["loading"].append({"modes": list(modes), "want": P.loaded_state(engine)})
    for name, case in P.E2E_CASES.items():
        table = {}
        original = Engine.dynamic_programming

        def spy(self, strategies, bsz, chunk, mbsz_dict, pp_stage_dict, min_tp, max_tp, vsp, embed_sdp, sp_search, logger):
            r = original(self, strategies, bsz, chunk, mbsz_dict, pp_stage_dict, min_tp, max_tp, vsp, embed_sdp, sp_search, logger)
            table['%d/%d/%d/%d/%d/%d/%d' % (bsz, chunk, min_tp, max_tp, vsp, embed_sdp, sp_search)] = [
                C.hexf(r['throughput']), int(r['min_pp_deg']), C.jsonable(r['vtp'])]
            return r

        Engine.dynamic_programming = spy
        try:
            with tempfile.TemporaryDirectory() as workdir, contextlib.redirect_stdout(io.StringIO()):
                engine = P.build(Engine, data, workdir, case["modes"], seqlen_list=case["seqlen_list"], **case["args"])
                state = P.loaded_state(engine)
                throughput = engine.parallelism_optimization()
                got = S.summarize(engine, throughput, os.path.join(workdir, "output"))
        finally:
            Engine.dynamic_programming = original
        got["table"] = table
        got["state"] = state
        out["e2e"][name] = got
        print(name, float.fromhex(got["throughput"]), "reference's test expects", P.E2E_KNOWN[name]["throughput"],
              len(table), list(got["files"]), flush=True)
    with open(os.path.join(HERE, "search_profile_golden.json"), "w") as fh:
        json.dump(out, fh, separators=(",", ":"))


if __name__ == "__main__":
    main()
