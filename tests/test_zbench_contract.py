"""bench.py's command-line contract, as far as it can be checked without a GPU, and the
shape of its one JSON line on a GPU (a short run of the headline workload)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_no_steps_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--steps", "0"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "--steps" in r.stderr and r.stdout.strip() == ""


def test_workloads_named_by_the_bench_exist():
    from flash_tree_attn_amd.synthetic import CONFIGS, algorithmic_bytes
    import torch
    for name in ("cfg1_plumbing_fp32", "cfg2_medusa_7b_fp16", "cfg3_gqa_8b_bf16", "cfg4_long_ctx_bf16", "cfg5_ragged_70b_bf16",
                 "decode1_mha_fp16", "decode1_gqa4_bf16", "reftest_mha_fp16", "d256_gqa2_bf16"):
        assert CONFIGS[name].name == name
    # the headline's algorithmic bytes: K+V 268.44 MB, tree k/v 2.10, q and out 4.19 each, mask, lengths
    cfg = CONFIGS["cfg3_gqa_8b_bf16"]
    lens = torch.full((cfg.bsz,), cfg.cache_len, dtype=torch.int64)
    mask = torch.zeros(cfg.q_len, cfg.q_len)
    assert algorithmic_bytes(cfg, lens, mask) == 268435456 + 2097152 + 2 * 4194304 + 64 * 64 * 4 + 8 * 8


@pytest.mark.gpu
def test_json_line_of_a_short_run():
    r = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "5", "--settle-ms", "0", "--cpu-seconds", "2"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["unit"] == "GB/s" and d["vs_baseline"] is None and d["dtype"] == "bf16"
    assert d["config"]["workload"] == "cfg3_gqa_8b_bf16"
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3 and 0.05 < rf["frac"] < 1.0
    cb = d["cpu_baseline"]
    assert cb["kind"] == "port" and cb["unit"] == "GB/s" and cb["cores"] >= 1 and cb["value"] > 0 and "sample" in cb
    assert abs(d["value"] - d["config"]["algorithmic_bytes"] / (d["ms_per_step"] * 1e-3) / 1e9) < 1.0
    # 20 steps are four batches of five calls, and the line says so
    bt = d["us_per_call_batches"]
    assert bt["batches"] == 4 and bt["calls_per_batch"] == 5 and bt["calls_in_last_batch"] == 5 and "median" in d["ms_per_step_is"]
    assert bt["min"] <= bt["median"] <= bt["max"]
