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
    for opt in ("--gpus", "--steps", "--warmup", "--config", "--kernel", "--api", "--alloc", "--flags", "--rows"):
        assert opt in out.stdout


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert out.returncode != 0
    assert "one GPU" in (out.stdout + out.stderr)


def _load_bench():
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench_under_test", BENCH)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_the_rows_of_the_default_run_cover_every_configuration_and_entry_point():
    """What the default command times after the headline: all five configurations through the table, the two LoRA
    sets through the functional update at the 100 steps the configurations name, the bit-exact flag, the functional
    arithmetic and one allocation per tensor on the largest set."""
    b = _load_bench()
    from eridiffusion_amd import workloads as W
    rows = [dict(b.HEADLINE, **change) for change, _, _ in b.ROWS]
    for r in rows:
        assert r["config"] in W.CONFIGS and r["api"] in ("table", "functional", "object") and r["alloc"] in ("pool", "tensor")
    table = {r["config"] for r in rows if r["api"] == "table" and r["flags"] == 0 and r["alloc"] == "pool" and r["mode"] == "eri"}
    assert table | {b.HEADLINE["config"]} == set(W.CONFIGS)
    assert {r["config"] for r in rows if r["api"] == "functional"} == {"c2_sdxl_lora_r16", "c3_flux_lora_r32"}
    assert any(r["config"] == "c5_flux12b_full" and r["flags"] == 2 and r["api"] == "table" for r in rows)
    assert any(r["config"] == "c5_flux12b_full" and r["flags"] == 2 and r["api"] == "object" for r in rows)
    assert any(r["config"] == "c5_flux12b_full" and r["alloc"] == "tensor" for r in rows)
    assert any(r["config"] == "c5_flux12b_full" and r["mode"] == "l2" for r in rows)
    for change, steps, warmup in b.ROWS:
        if change["config"] in ("c2_sdxl_lora_r16", "c3_flux_lora_r32"):
            assert steps == 100
        assert warmup >= 1
    # every kernel widens to fp32 and rounds each operation to fp32; the traffic probe only moves bytes
    assert {k: v for k, v in b.ARITHMETIC.items() if v != "f32"} == {"traffic": "u8"}
    assert any(r["config"] == "c5_flux12b_full" and r["kernel"] == "traffic" for r in rows)


@pytest.mark.gpu
def test_the_rows_of_the_small_configurations_carry_their_keys():
    cmd = [sys.executable, BENCH, "--config", "c1_flat_fp32", "--steps", "3", "--warmup", "1", "--cpu-sample", "1048576",
           "--rows", "all", "--rows-max-params", str(200_000_000)]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    rows = d["configs"]
    assert [(r["workload"], r["kernel"], r["api"]) for r in rows] == [
        ("c1_flat_fp32", "adam8", "table"),
        ("c2_sdxl_lora_r16", "adam8", "table"), ("c2_sdxl_lora_r16", "adam8", "functional"), ("c2_sdxl_lora_r16", "traffic", "table"),
        ("c3_flux_lora_r32", "adam8", "table"), ("c3_flux_lora_r32", "adam8", "functional"), ("c3_flux_lora_r32", "traffic", "table")]
    for r in rows:
        assert "error" not in r, r
        for key in ("workload", "kernel", "api", "mode", "flags", "alloc", "param_dtype", "params", "tensors", "steps", "warmup",
                    "ms_per_step", "params_per_s", "kernel_ms", "kernel_ms_min", "frac", "frac_of_step"):
            assert key in r, key
        assert r["steps"] == 100 and r["ms_per_step"] > 0 and 0 < r["frac"] < 1 and 0 < r["frac_of_step"] < 1
        assert r["mode"] == ("l2" if r["api"] == "functional" else "eri")
        assert r["alloc"] in ("pool", "arena")
        if r["api"] == "table" and r["kernel"] == "adam8":
            assert r["cpu_params_per_s"] > 0 and "whole workload" in r["cpu_sample"]


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
    assert d["dtype"] == "f32" and "configs" not in d  # the rows belong to the default command line
    assert "workload" in d["config"] and "model" not in d["config"]
    # the placement the run really used: the lane pool unless another was asked for (or the pool did not fit)
    want = extra[1] if extra and extra[0] == "--alloc" else "pool"
    assert d["config"]["alloc"] == want or (want == "pool" and d["config"]["alloc"] == "arena" and "lane pool" in out.stderr)
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["peak"] == 8000.0 and r["unit"] == "GB/s"
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9 and 0 < r["frac"] < 1
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and c["sample"]
