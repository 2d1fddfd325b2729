"""bench.py's contract: more than one GPU is refused with a message (this build runs on one GPU); on a GPU a short
run prints exactly one JSON line with the fields the driver reads, the roofline and cpu_baseline objects and the
figures of the neighbouring operators."""

import json
import os
import subprocess
import sys

import pytest

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_BENCH = os.path.join(_ROOT, "bench.py")


def test_more_than_one_gpu_is_refused():
    res = subprocess.run([sys.executable, _BENCH, "--gpus", "2", "--steps", "1", "--warmup", "0"], capture_output=True,
                         text=True, timeout=300)  # fmt: skip
    assert res.returncode != 0
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


@pytest.mark.gpu
def test_one_json_line_with_the_contract_fields():
    res = subprocess.run([sys.executable, _BENCH, "--gpus", "1", "--steps", "20", "--warmup", "3"], capture_output=True,
                         text=True, timeout=600)  # fmt: skip
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [l for l in res.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    r = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):  # fmt: skip
        assert key in r, key
    assert r["n_gpus"] == 1 and r["steps"] == 20 and r["warmup"] == 3 and r["vs_baseline"] is None
    assert r["dtype"] == "bf16" and r["data"] == "synthetic" and "workload" in r["config"] and "model" not in r["config"]
    roof = r["roofline"]
    assert roof["bound"] == "mfma" and roof["peak"] == 2500.0 and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert 0.02 < roof["frac"] < 1.0
    # measured HBM traffic comes from a committed profile of this very kernel source, or is null with the reason
    assert (roof["traffic"] or 0) > 0 or "stale" in roof["traffic_source"] or "not measured" in roof["traffic_source"]
    # C2's working set fits the memory-side cache: the line also carries the time with cold caches, which cannot be
    # meaningfully faster than the replay of one set
    assert r["ms_per_step_cold"] > 0.9 * r["ms_per_step_events"] and r["value_cold"] > 0 and "sets" in r["cold_note"]
    cpu = r["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    # the value and the time per step are two views of the same measurement
    flops = r["config"]["flops_per_step"]
    assert abs(r["value"] - flops / (r["ms_per_step"] * 1e-3) / 1e12) / r["value"] < 1e-3
    for leg in ("backward", "ln_mul", "in_linear_silu"):
        assert leg in r and "error" not in r[leg], (leg, r.get(leg))
    assert all(c["roofline"]["bound"] == "hbm" for c in r["ln_mul"]["cases"])
