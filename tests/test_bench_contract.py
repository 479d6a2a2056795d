"""bench.py's command line: the options parse without a GPU, more than one GPU is refused with a message, and
(on a GPU) one small run prints exactly one JSON line with the fields the contract names."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_options_parse_without_a_gpu():
    out = subprocess.run([sys.executable, BENCH, "--help"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0
    for opt in ("--gpus", "--steps", "--warmup", "--config", "--kernel", "--api", "--alloc", "--flags"):
        assert opt in out.stdout


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode != 0
    assert "one GPU" in (out.stdout + out.stderr)


@pytest.mark.gpu
@pytest.mark.parametrize("extra", [[], ["--api", "object"], ["--api", "functional"], ["--kernel", "adam8_ema"],
                                   ["--grad-dtype", "f32"], ["--alloc", "tensor"], ["--alloc", "arena"]])
def test_one_small_run_prints_the_contract_line(extra):
    cmd = [sys.executable, BENCH, "--config", "c1_flat_fp32" if not extra or extra[0] == "--alloc" else "c2_sdxl_lora_r16",
           "--steps", "3", "--warmup", "1", "--cpu-sample", "1048576"] + extra
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["vs_baseline"] is None
    assert d["unit"] == "params/s" and d["higher_is_better"] is True and d["data"] == "synthetic"
    assert "workload" in d["config"] and "model" not in d["config"]
    # the placement the run really used: the lane pool unless another was asked for (or the pool did not fit)
    want = extra[1] if extra and extra[0] == "--alloc" else "pool"
    assert d["config"]["alloc"] == want or (want == "pool" and d["config"]["alloc"] == "arena" and "lane pool" in out.stderr)
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9 and 0 < r["frac"] < 1
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
