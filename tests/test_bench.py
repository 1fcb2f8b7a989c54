"""The measurement script keeps its contract: one JSON line with the agreed fields at one GPU, one line and exit
status 2 for more."""

import json
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_in_one_line():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode == 2
    lines = [line for line in run.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


@pytest.mark.gpu
def test_the_line_of_a_short_run():
    """Two layers of the default shape, a few steps: every field of the contract is there, `config` is flat with at
    most 20 keys and names both numbers of layers, the fractions are what their parts give."""
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--layers", "2", "--steps", "4", "--warmup", "2",
                          "--no-tune"], capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [line for line in run.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 4 and record["warmup"] == 2 and record["higher_is_better"]
    assert record["dtype"] == "bf16" and record["unit"] == "tok/s" and "synthetic" in record["data"]
    config = record["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["layers"] == 28 and config["layers_run"] == 2 and config["global_batch"] == 8
    assert record["value"] == pytest.approx(8 / (record["ms_per_step"] * 1e-3), rel=1e-3)
    prefill, roofline = record["prefill"], record["roofline"]
    assert set(prefill) == {"value", "tokens", "ms", "frac"} and prefill["tokens"] == 2048
    assert prefill["value"] == pytest.approx(2048 / (prefill["ms"] * 1e-3), rel=1e-3) and 0 < prefill["frac"] < 1
    assert set(roofline) == {"bound", "achieved", "peak", "unit", "frac"} and roofline["bound"] == "hbm"
    assert roofline["peak"] == 8000.0 and roofline["frac"] == pytest.approx(roofline["achieved"] / 8000.0, abs=1e-3)
    assert set(record["points"]) == {"decode_b1", "decode_b64"}
