"""bench.py's contract with its caller: one JSON line on stdout with the agreed keys, one GPU only, and the workload
constants it is quoted on (attention forward B=2 H=16 S=8192 D=128 bf16 causal; Lion over 1.3 B
parameters; the GPT-2-small sets of the reference's own benchmarks, benchmarks/benchmark_lion.py:10-16 and
benchmarks/benchmark_flash_attention.py:195-209)."""
import json
import math
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_workload_constants():
    sys.path.insert(0, ROOT)
    import bench

    n = lambda shapes: sum(math.prod(s) for s in shapes)
    assert n(bench.GPT2_SMALL_SHAPES) == 124_439_808 and len(bench.GPT2_SMALL_SHAPES) == 148
    assert n(bench.LION_LARGE_SHAPES) == 1_308_622_848
    assert bench.LION_HP["lr"] == 1e-4 and tuple(bench.LION_HP["betas"]) == (0.9, 0.99)


@pytest.mark.gpu
def test_default_run_prints_one_json_line_with_the_agreed_keys():
    r = subprocess.run([sys.executable, BENCH, "--steps", "3", "--warmup", "1", "--settle", "10"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["unit"] == "TFLOP/s" and d["dtype"] == "bf16" and d["data"].startswith("synthetic") and "workload" in d["config"]
    assert "model" not in d["config"]
    # the headline value is the algorithmic FLOPs of the causal forward over the whole-step time
    flops = 2.0 * 2 * 16 * 8192 * 8192 * 128
    assert d["value"] == pytest.approx(flops / (d["ms_per_step"] * 1e-3) / 1e12, rel=1e-6)
    rf = d["roofline"]
    assert rf["bound"] == "mfma" and rf["peak"] == 2500.0 and rf["unit"] == "TFLOP/s"
    assert rf["frac"] == pytest.approx(rf["achieved"] / rf["peak"], rel=1e-9)
    assert rf["achieved"] == pytest.approx(flops / (rf["kernel_ms_avg"] * 1e-3) / 1e12, rel=1e-6)
    assert rf["kernel_ms_avg"] <= d["ms_per_step"] * 1.001, "a launch cannot take longer than the step that contains it"
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["cores"] >= 1 and cb["value"] > 0 and cb["sample"]
    lion = d["lion"]
    assert lion["unit"] == "GB/s" and lion["roofline"]["bound"] == "hbm" and lion["roofline"]["peak"] == 8000.0
    assert lion["roofline"]["achieved"] == pytest.approx(16.0 * 1_308_622_848 / (lion["roofline"]["kernel_ms_avg"] * 1e-3) / 1e9, rel=1e-6)
    assert lion["cpu_baseline"]["kind"] == "port"
    assert set(d["configs"]) >= {"2_attn_fwd_gpt2_small", "3_lion_gpt2_small", "5a_attn_fwd_throughput"}
    # the headline launch varied one thing at a time (mask, operand bits, head_dim), and the ratio the causal form pays
    hv = d["headline_variants"]
    assert set(hv) >= {"causal", "noncausal", "zero_operands", "zero_operands_noncausal", "head_dim_64", "causal_over_half_noncausal", "causal_one_item_per_workgroup",
                       "config_5a_one_item_per_workgroup"}
    assert hv["causal_over_half_noncausal"] == pytest.approx(hv["causal"]["kernel_ms_avg"] / (0.5 * hv["noncausal"]["kernel_ms_avg"]), rel=1e-9)
    assert "bwd" in d["configs"]["2_attn_fwd_gpt2_small"] and "training_loop" in d["configs"]["3_lion_gpt2_small"]
