"""bench.py's line: one JSON object with the fields its readers take, for one GPU; more GPUs are
refused in one line with exit code 2."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=600)


def test_more_than_one_gpu_is_refused_in_one_line():
    r = _bench("--gpus", "2", "--steps", "3", "--warmup", "1")
    assert r.returncode == 2
    lines = [line for line in r.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


@pytest.mark.gpu
def test_the_line_of_a_short_run():
    """One layer of the default shape (the line then names both layer counts), a few steps."""
    r = _bench("--layers", "1", "--steps", "3", "--warmup", "1", "--points", "1", "--prefill-tokens", "256")
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [line for line in r.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 3 and out["warmup"] == 1 and out["higher_is_better"] is True
    assert out["dtype"] == "bf16" and out["unit"] == "tokens/s" and "synthetic" in out["data"]
    assert abs(out["value"] - out["config"]["global_batch"] / out["ms_per_step"] * 1e3) < 1e-2 * out["value"]
    config = out["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["layers"] == 1 and config["layers_full"] == 32 and config["hidden_size"] == 4096
    assert set(out["prefill"]) >= {"value", "tokens", "ms", "frac"} and out["prefill"]["tokens"] == 256
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert "decode_b1" in out["points"]
