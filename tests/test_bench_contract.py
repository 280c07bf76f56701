"""bench.py's contract with whoever runs it: one GPU only (anything else is said in one line, exit status 2), and one
JSON line with the agreed keys."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args, timeout=600):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], cwd=ROOT, capture_output=True,
                          text=True, timeout=timeout)


def test_more_than_one_gpu_is_refused_in_one_line():
    done = run_bench("--gpus", "2", "--steps", "3", "--warmup", "1", timeout=120)
    assert done.returncode == 2
    lines = [line for line in done.stdout.splitlines() if line.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


@pytest.mark.gpu
def test_the_line_of_a_short_run():
    """Two layers of the 2B sizes, a short context: the line's keys, not its figures."""
    done = run_bench("--layers", "2", "--steps", "3", "--warmup", "1", "--context", "512", "--batch", "4",
                     "--prefill-tokens", "256", "--latency-steps", "4", "--no-points")
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [line for line in done.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 3 and out["warmup"] == 1 and out["higher_is_better"] is True
    assert out["dtype"] == "bf16" and out["unit"] == "tokens/s" and out["value"] > 0
    config = out["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert config["layers"] == 2 and config["layers_of_full_model"] == 26 and config["global_batch"] == 4
    assert set(out["prefill"]) == {"value", "tokens", "ms", "frac"} and out["prefill"]["tokens"] == 256
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert abs(out["value"] - 4 / (out["ms_per_step"] * 1e-3)) / out["value"] < 1e-3
    check = out["self_check"]
    assert check["same_token"] == check["of"] == 4
    ceilings = out["measured_ceilings"]
    assert "error" not in ceilings and 1000 < ceilings["hbm_read_8k_pieces_gbps"] < 8000
