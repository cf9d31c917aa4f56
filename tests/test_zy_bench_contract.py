"""bench.py as the driver runs it: its command line, the one JSON line it prints, and that the traffic
figures it quotes from profiles/ were measured on the kernel sources that are in the tree."""
import importlib.util
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def _bench_module():
    spec = importlib.util.spec_from_file_location("bench_under_test", BENCH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert out.returncode != 0
    assert "ONE GPU" in (out.stderr + out.stdout), out.stderr[-400:]


def test_quoted_traffic_belongs_to_the_kernel_sources_in_the_tree():
    """Every measured byte count carries the hash of the kernel sources it was measured on; bench.py reports
    null instead of a stale figure, and this test says so before a run does."""
    b = _bench_module()
    now = b._kernel_sources_hash()
    stale = {k: v[3] for k, v in b.MEASURED_TRAFFIC.items() if v[1] != now}
    assert not stale, f"re-measure (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE) and update bench.py: {stale}"
    for key, (nbytes, _, tile, profile) in b.MEASURED_TRAFFIC.items():
        assert os.path.exists(os.path.join(ROOT, profile)), profile
        assert b._traffic(key, tile)[0] == nbytes


@pytest.mark.gpu
def test_the_line_the_driver_parses():
    out = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--also", "cfg0"],
                         capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert out.returncode == 0, out.stderr[-800:]
    lines = [ln for ln in out.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1, out.stdout[-800:]
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 5 and d["warmup"] == 2 and d["dtype"] == "f64" and d["vs_baseline"] is None
    assert d["config"]["workload"] == "cfg2" and d["config"]["bit_exact"] is True
    r = d["roofline"]
    assert 0.0 < r["frac"] <= 1.0 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9
    assert r["traffic"] is not None and r["traffic"] >= 16 * 80 * 131072 * 64      # no less than the algorithmic bytes
    assert abs(d["value"] - d["config"]["relaxations_per_step"] / (d["ms_per_step"] * 1e-3)) / d["value"] < 1e-6
    c = d["cpu_baseline"]
    assert c["kind"] in ("reference", "port") and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
    assert d["also"]["cfg0"]["bit_exact"] is True
