"""Writes tests/golden/dp_on_model_golden.json: what the REFERENCE's ``DpOnModel``
(galvatron/core/search_engine/dynamic_programming.py:128-565) returns for the scenarios of
tests/dp_on_model_stubs.py when it is given the stub cost models and the reference's own compiled
dp_core (oracle/_ref).  Run in the build container only:

    python oracle/build.py && python tests/golden/make_dp_on_model_golden.py

The reference module is loaded from where it lies (its three files import only numpy, tqdm and
dataclasses); its package __init__ files, which pull in the training runtime, are not executed.
For the stub scenarios ``OtherTimeCostModel`` and ``pipeline_costmodel``, which the reference module
imports from its own cost_model.py, are replaced by the stubs (the comparison is about DpOnModel
alone); the ``real_*`` scenarios run the reference's DpOnModel on the reference's own cost models.
The fixture holds data only (the returned tuples, floats as hex strings).
"""
import importlib
import json
import os
import sys
import types

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import dp_on_model_stubs as stubs  # noqa: E402
from oracle import dp_oracle as O  # noqa: E402

REF_DIR = "/root/reference/galvatron/core/search_engine"


def reference_module():
    pkg = types.ModuleType("_ref_search_engine")
    pkg.__path__ = [REF_DIR]
    sys.modules["_ref_search_engine"] = pkg
    sys.modules["galvatron_dp_core"] = O.ref_module()          # what `import galvatron_dp_core` finds in DPAlg.fit
    mod = importlib.import_module("_ref_search_engine.dynamic_programming")
    return mod


def serve_strategy_helpers():
    """pipeline_costmodel imports form_strategy / strategy_str2list from galvatron.utils when called;
    serve them from galvatron/utils/strategy_utils.py without running the package's __init__."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("_ref_strategy_utils",
                                                  "/root/reference/galvatron/utils/strategy_utils.py")
    su = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(su)
    g = types.ModuleType("galvatron")
    g.__path__ = []
    gu = types.ModuleType("galvatron.utils")
    gu.form_strategy, gu.strategy_str2list = su.form_strategy, su.strategy_str2list
    sys.modules["galvatron"], sys.modules["galvatron.utils"] = g, gu


def main():
    mod = reference_module()
    real_other, real_pipeline = mod.OtherTimeCostModel, mod.pipeline_costmodel
    out = {}
    mod.OtherTimeCostModel = stubs.StubOther
    mod.pipeline_costmodel = stubs.stub_pipeline_costmodel
    for name in stubs.SCENARIOS:
        cfg = stubs.scenario(name)
        dpm = stubs.build(mod.DpOnModel, cfg)
        out[name] = stubs.run(dpm, cfg)
        print(name, out[name]['fit'][0], out[name]['fit'][2], out[name]['fit'][5], flush=True)
    # the same class fed by the reference's own cost models
    mod.OtherTimeCostModel, mod.pipeline_costmodel = real_other, real_pipeline
    serve_strategy_helpers()
    cost_mod = importlib.import_module("_ref_search_engine.cost_model")
    args_mod = importlib.import_module("_ref_search_engine.cost_model_args")
    for name in stubs.REAL_SCENARIOS:
        cfg = stubs.real_scenario(name)
        dpm = stubs.build_real(mod.DpOnModel, cost_mod, args_mod, cfg)
        out[name] = stubs.run(dpm, cfg)
        print(name, out[name]['fit'][0], out[name]['fit'][2], out[name]['fit'][5], flush=True)
    with open(os.path.join(HERE, "dp_on_model_golden.json"), "w") as fh:
        json.dump(out, fh, separators=(",", ":"))
    print("wrote", len(out), "scenarios")


if __name__ == "__main__":
    main()
