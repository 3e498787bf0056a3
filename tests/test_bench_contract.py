"""bench.py's command-line contract: one JSON line with the agreed keys, one GPU only."""
from __future__ import annotations

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
REQUIRED = ["metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
            "dtype", "data", "config", "roofline", "cpu_baseline"]


def test_more_than_one_gpu_is_refused():
    """This build measures one GPU; asking for more ends with a message that says so, before any device is touched."""
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in (proc.stderr + proc.stdout) or "1 GPU" in (proc.stderr + proc.stdout)


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_contract_keys():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--steps", "2", "--warmup", "1", "--legs", "step"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in REQUIRED:
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 2 and rec["warmup"] == 1 and rec["unit"] == "ms"
    assert rec["higher_is_better"] is False and rec["vs_baseline"] is None and rec["dtype"] == "f32"
    assert "workload" in rec["config"] and "model" not in rec["config"]
    roof = rec["roofline"]
    assert roof["bound"] in ("hbm", "mfma") and roof["unit"] in ("GB/s", "TFLOP/s")
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3 and 0.0 < roof["frac"] < 1.0
    cpu = rec["cpu_baseline"]
    assert cpu["kind"] in ("reference", "port") and cpu["cores"] >= 1 and cpu["value"] > rec["value"]
    assert abs(rec["value"] - rec["ms_per_step"]) < 1e-9
