"""Writes tests/golden/cost_model_golden.json: what the REFERENCE's cost models
(galvatron/core/search_engine/cost_model.py: MemoryCostModel :10-219, TimeCostModel :221-466,
OtherTimeCostModel :468-658, pipeline_costmodel :695-767) and its pipeline-division utilities
(search_engine.py:972-1104) return for seeded random scenarios over
synthetic profiles of the shape the reference's mock profiles have (tests/utils/search_configs.py:
per-tp activation tables, model-state tables per vocabulary tp degree, collective coefficients keyed
'<size>' / '<size>_<0|1>', fitted lines for the sequence-parallel collectives).  Run in the build
container only:

    python tests/golden/make_cost_model_golden.py

The reference module is loaded from where it lies (it imports numpy and dataclasses only); its
package __init__ files are not executed, and the two string helpers it imports lazily from
galvatron.utils are served from galvatron/utils/strategy_utils.py through a stand-in package entry.
The fixture holds data only: the scenario inputs (tests/cost_model_cases.py rebuilds the argument
records from them) and the returned numbers, floats as hex strings.
"""
import importlib
import importlib.util
import json
import os
import sys
import types

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "tests"))

import cost_model_cases as C  # noqa: E402

REF_DIR = "/root/reference/galvatron/core/search_engine"


def reference_module():
    pkg = types.ModuleType("_ref_search_engine")
    pkg.__path__ = [REF_DIR]
    sys.modules["_ref_search_engine"] = pkg
    spec = importlib.util.spec_from_file_location("_ref_strategy_utils", "/root/reference/galvatron/utils/strategy_utils.py")
    su = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(su)
    g = types.ModuleType("galvatron")
    g.__path__ = []
    # galvatron.utils without its __init__ (which pulls torch-based training helpers): the two plain
    # modules the search engine needs, their public names gathered on the stand-in package
    gu = types.ModuleType("galvatron.utils")
    gu.__path__ = ["/root/reference/galvatron/utils"]
    sys.modules["galvatron"], sys.modules["galvatron.utils"] = g, gu
    for name in ("strategy_utils", "config_utils"):
        sub = importlib.import_module("galvatron.utils." + name)
        for k, v in vars(sub).items():
            if not k.startswith("_"):
                setattr(gu, k, v)
    mod = importlib.import_module("_ref_search_engine.cost_model")
    args = importlib.import_module("_ref_search_engine.cost_model_args")
    return mod, args, su


def main():
    mod, args, su = reference_module()
    out = {"memory": [], "time": [], "other": [], "pipeline": [], "strings": [], "pp": []}
    engine = importlib.import_module("_ref_search_engine.search_engine")      # pipeline-division utilities, :972-1104
    for case in C.pp_cases():
        out["pp"].append({"case": case, "want": C.run_pp(engine, args, case)})
    for case in C.memory_cases():
        out["memory"].append({"case": case, "want": C.run_memory(mod, args, case)})
    for case in C.time_cases():
        out["time"].append({"case": case, "want": C.run_time(mod, args, case)})
    for case in C.other_cases():
        out["other"].append({"case": case, "want": C.run_other(mod, args, case)})
    for case in C.pipeline_cases():
        out["pipeline"].append({"case": case, "want": C.run_pipeline(mod, args, case)})
    for s in C.all_strategies():
        text = su.form_strategy(s)
        out["strings"].append({"strategy": s, "text": text, "back": su.strategy_str2list(text)})
    with open(os.path.join(HERE, "cost_model_golden.json"), "w") as fh:
        json.dump(out, fh, separators=(",", ":"))
    print({k: len(v) for k, v in out.items()})


if __name__ == "__main__":
    main()
