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
    assert rec["config"]["num_hidden_layers"] == 2 and rec["config"]["layers_of_full_model"] == 36
    assert {"value", "tokens", "ms", "frac"} <= set(rec["prefill"]) and rec["prefill"]["tokens"] == 2048
    assert rec["roofline"]["bound"] == "hbm" and rec["roofline"]["peak"] == 8000.0
    assert abs(rec["roofline"]["frac"] - rec["roofline"]["achieved"] / rec["roofline"]["peak"]) < 1e-3
    assert set(rec["points"]) == {"decode_b1", "decode_b64"}
    assert all(isinstance(v, float) for v in rec["points"].values())
    assert abs(rec["value"] - 8 * 1000.0 / rec["ms_per_step"]) / rec["value"] < 0.01

    # the arithmetic behind the fractions (which bench.py takes from the model's parts and the cache
    # manager), recomputed here from the sizes the line names, with the architecture's own formulas
    c = rec["config"]
    h, d, i, v, layers = c["hidden_size"], c["head_dim"], c["intermediate_size"], c["vocab_size"], c["num_hidden_layers"]
    q, kv = c["num_attention_heads"] * d, c["num_key_value_heads"] * d
    assert c["tie_word_embeddings"] is True
    per_layer = h * (q + 2 * kv) + q * h + 3 * h * i + 2 * h + 2 * d       # matrices, two norms, q/k norms
    weight_bytes = 2 * (v * h + layers * per_layer + h)                    # tied table once, final norm
    kv_per_token = 2 * layers * kv * 2
    step_s = rec["ms_per_step"] * 1e-3
    # each of the 8 requests holds its 2,048-token prompt and between 1 and ~100 decoded tokens
    low = (weight_bytes + 8 * 2049 * kv_per_token) / step_s / 1e9
    high = (weight_bytes + 8 * 2150 * kv_per_token) / step_s / 1e9
    assert low * 0.999 <= rec["roofline"]["achieved"] <= high * 1.001, (low, rec["roofline"]["achieved"], high)
    flop = 2048 * 2 * layers * (h * (q + 2 * kv) + q * h + 3 * h * i) + 2 * q * 2048 * 2048 * layers + 2 * v * h
    assert abs(rec["prefill"]["frac"] - flop / (rec["prefill"]["ms"] * 1e-3) / 2.5e15) < 2e-4
    assert abs(rec["prefill"]["value"] - 2048 / (rec["prefill"]["ms"] * 1e-3)) / rec["prefill"]["value"] < 1e-3
    for b, point in rec["point_rooflines"].items():
        batch = int(b.rsplit("b", 1)[1])
        assert abs(rec["points"][b] - batch * 1000.0 / point["ms_per_step"]) / rec["points"][b] < 0.01
        floor = (weight_bytes + batch * 2049 * kv_per_token) / (point["ms_per_step"] * 1e-3) / 1e9 / 8000.0
        assert floor * 0.999 <= point["frac"] <= floor * 1.06
    # the device's own peaks stand beside the published ones, and are plausible for this part
    assert 2000 < rec["measured_peak"]["hbm_gbs"] < 8000 and 500 < rec["measured_peak"]["mfma_bf16_tflops"] < 2600
    assert rec["roofline"]["measured_peak"] == rec["measured_peak"]["hbm_gbs"]
    assert rec["trials"]["windows"] == 3 and len(rec["trials"]["ms_per_step"]) == 3
    assert min(rec["trials"]["ms_per_step"]) <= rec["ms_per_step"] <= max(rec["trials"]["ms_per_step"])


@pytest.mark.gpu
def test_smoke_entry_point():
    sys.path.insert(0, str(ROOT))
    import __graft_entry__

    __graft_entry__.smoke()
