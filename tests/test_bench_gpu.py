"""bench.py keeps its contract: one JSON line with the fields the driver reads, and exit code 2 for more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=600)


def test_more_than_one_gpu_is_refused():
    p = run_bench("--gpus", "2")
    assert p.returncode == 2 and "one GPU" in p.stdout and len(p.stdout.strip().splitlines()) == 1


@pytest.mark.gpu
def test_bench_line(gpu):
    p = run_bench("--layers", "2", "--steps", "4", "--warmup", "2", "--context", "512", "--prefill-tokens", "256")
    assert p.returncode == 0, p.stderr[-2000:]
    rec = json.loads(p.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 4 and rec["warmup"] == 2 and rec["dtype"] == "bf16"
    cfg = rec["config"]
    assert len(cfg) <= 20 and all(not isinstance(v, (dict, list)) for v in cfg.values())
    assert cfg["layers"] == 2 and cfg["layers_full"] == 36 and cfg["hidden"] == 2560 and cfg["global_batch"] == 8
    assert rec["value"] > 0 and abs(rec["value"] - 8 / (rec["ms_per_step"] / 1e3)) < 1e-2 * rec["value"]
    assert set(rec["prefill"]) == {"value", "tokens", "ms", "frac"} and rec["prefill"]["tokens"] == 256
    assert set(rec["roofline"]) == {"bound", "achieved", "peak", "unit", "frac"} and rec["roofline"]["peak"] == 8000.0
    assert abs(rec["roofline"]["frac"] - rec["roofline"]["achieved"] / 8000.0) < 1e-3
    # the points away from the default context are left out when the context is not the default one
    assert set(rec["points"]) == {"decode_b1", "decode_b32", "decode_b64"} and all(v > 0 for v in rec["points"].values())


@pytest.mark.gpu
def test_other_workloads_run(gpu):
    p = run_bench("--layers", "2", "--mixed", "--context", "1024", "--prefill-tokens", "256", "--steps", "16")
    assert p.returncode == 0, p.stderr[-2000:]
    assert json.loads(p.stdout.strip().splitlines()[-1])["ms"] > 0
    p = run_bench("--layers", "2", "--requests", "6", "--concurrency", "3", "--prompt-len", "100", "--new-tokens", "3")
    assert p.returncode == 0, p.stderr[-2000:]
    assert json.loads(p.stdout.strip().splitlines()[-1])["req_per_s"] > 0
