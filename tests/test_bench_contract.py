"""The benchmark script's contract, on a tiny model of the same kind: one JSON line on standard
output with the keys that the record needs, a flat `config` of at most twenty keys, the prefill,
roofline and points blocks; for more than one GPU a line that says so and exit status 2."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=600)


def test_more_than_one_gpu_is_refused_with_status_2():
    p = run("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert p.returncode == 2 and "one GPU" in p.stdout + p.stderr


@pytest.mark.gpu
def test_the_default_run_of_a_tiny_model_prints_the_record():
    p = run("--tiny", "--steps", "4", "--warmup", "1", "--runs", "2", "--context", "256", "--prefill-tokens", "128", "--no-peaks")
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, lines
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 4 and rec["warmup"] == 1 and rec["higher_is_better"] is True
    assert rec["unit"] == "tok/s" and rec["value"] > 0 and abs(rec["value"] - rec["config"]["global_batch"] / rec["ms_per_step"] * 1e3) < 1e-2 * rec["value"]
    assert len(rec["config"]) <= 20 and all(not isinstance(v, (dict, list)) for v in rec["config"].values())
    assert set(rec["prefill"]) >= {"value", "tokens", "ms", "frac"} and rec["prefill"]["tokens"] == 128
    assert rec["roofline"]["bound"] == "hbm" and rec["roofline"]["unit"] == "GB/s" and rec["roofline"]["peak"] == 8000.0
    assert abs(rec["roofline"]["frac"] - rec["roofline"]["achieved"] / rec["roofline"]["peak"]) < 1e-3
    assert set(rec["points"]) == {"decode_b1", "decode_b64"} and all(v > 0 for v in rec["points"].values())
