"""bench.py contract checks that need no GPU."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and r.stdout.strip() == ""
    assert "one GPU only" in r.stderr


def test_workload_tables_match_the_configurations():
    sys.path.insert(0, ROOT)
    import bench
    from nabla_amd import workloads as W

    sizes = {name: W.n_params(bench.workload(name)["shapes"]) for name in
             ("mlp-sgd-f32", "gpt2-small-f32", "llama-1.1b", "llama3-8b")}
    assert sizes == {"mlp-sgd-f32": 235_146, "gpt2-small-f32": 124_439_808,
                     "llama-1.1b": 1_100_046_336, "llama3-8b": 8_030_257_152}
    assert len(bench.workload("ragged-4096")["shapes"]) == 4096
    cfg = bench.workload("llama3-8b")
    assert (cfg["lr"], cfg["wd"], cfg["betas"], cfg["clip"], cfg["scaler"]) == (2e-4, 0.1, (0.9, 0.95), 1.0, True)
    assert bench.bytes_per_param(cfg) == (28, 2)
    assert bench.bytes_per_param(bench.workload("gpt2-small-f32")) == (28, 0)
    assert bench.bytes_per_param(bench.workload("mlp-sgd-f32")) == (12, 0)


def test_traffic_file_is_consistent_with_the_profile_summary():
    with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
        t = json.load(f)
    total = t["llama3-8b:nbo_update_bf16_adamw"]
    algorithmic = 8_030_257_152 * 28
    assert 0.99 < total / algorithmic < 1.02
    d = t["_detail"]["per_launch_bytes"]["nbo_update_bf16_adamw"]
    assert d["fetch_bytes"] + d["write_bytes"] == total
