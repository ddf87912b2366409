"""The programs at the repository root keep their contracts: bench.py refuses more than one GPU
with one line and exit status 2, and prints one JSON line with the fields the measurement needs;
the smoke entry point generates the plain implementation's tokens."""

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert proc.returncode == 2
    lines = [l for l in proc.stdout.splitlines() if l.strip()]
    assert len(lines) == 1 and "--gpus 2" in lines[0]


@pytest.mark.gpu
def test_bench_line_has_the_contract_fields():
    """A short run on two layers of the default shape (the line says so: layers and
    layers_of_full_model)."""
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--layers", "2", "--steps", "8", "--warmup", "2"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [l for l in proc.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 8 and rec["warmup"] == 2 and rec["higher_is_better"] is True
    assert len(rec["config"]) <= 20 and all(not isinstance(v, (dict, list)) for v in rec["config"].values())
    assert rec["config"]["layers"] == 2 and rec["config"]["layers_of_full_model"] == 36
    assert set(rec["prefill"]) == {"value", "tokens", "ms", "frac"} and rec["prefill"]["tokens"] == 2048
    assert rec["roofline"]["bound"] == "hbm" and rec["roofline"]["peak"] == 8000.0
    assert abs(rec["roofline"]["frac"] - rec["roofline"]["achieved"] / rec["roofline"]["peak"]) < 1e-3
    assert set(rec["points"]) == {"decode_b1", "decode_b64"}
    assert abs(rec["value"] - 8 * 1000.0 / rec["ms_per_step"]) / rec["value"] < 0.01


@pytest.mark.gpu
def test_smoke_entry_point():
    sys.path.insert(0, str(ROOT))
    import __graft_entry__

    __graft_entry__.smoke()
