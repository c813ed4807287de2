"""bench.py contract checks: the ones that need no GPU, and two real runs of the measurement
scripts on their smallest inputs."""
import json
import os
import subprocess
import sys

import pytest

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
    det = t["_detail"].get("llama3-8b", t["_detail"])  # per-workload layout; single-workload in older files
    d = det["per_launch_bytes"]["nbo_update_bf16_adamw"]
    assert d["fetch_bytes"] + d["write_bytes"] == total
    # the counters were collected for the kernels as they are now: the file carries a hash of the
    # kernel source of its profile run, and a change to the kernels asks for a new run
    from nabla_amd.profile_summary import kernel_source_hash

    for workload in ("llama3-8b", "llama-1.1b"):
        assert t["_detail"][workload].get("kernel_source_sha256") == kernel_source_hash(), (
            f"profiles/traffic.json [{workload}] was collected for other kernel source: run the commands at the top "
            "of profiles/adamw_fused_step_*.md again and `python -m nabla_amd.kernel_bench --summarize`")


@pytest.mark.gpu
def test_small_mlp_bench_line_has_the_contract_fields(gpu):
    """One real `bench.py` run on the smallest workload: one JSON line with the fields the
    driver reads, the roofline block and the CPU baseline."""
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "mlp-sgd-f32", "--steps", "20",
                        "--warmup", "3", "--cpu-seconds", "1"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [x for x in r.stdout.splitlines() if x.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 3 and d["config"]["workload"] == "mlp-sgd-f32"
    assert d["roofline"]["bound"] == "hbm" and d["roofline"]["peak"] == 8000.0 and d["roofline"]["kernel"] == "nbo_update_f32_sgd"
    assert abs(d["roofline"]["frac"] - d["roofline"]["achieved"] / d["roofline"]["peak"]) < 1e-3
    assert d["cpu_baseline"]["kind"] == "port" and d["cpu_baseline"]["cores"] >= 1 and d["value"] > 0


@pytest.mark.gpu
def test_kernel_bench_prints_a_row_for_every_measurement(gpu):
    """`python -m nabla_amd.kernel_bench` on one tensor: every row has a positive time."""
    r = subprocess.run([sys.executable, "-m", "nabla_amd.kernel_bench", "--elements", "1e6", "--reps", "1"],
                       capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    rows = [x for x in r.stdout.splitlines() if x.startswith("| ") and "`nbo_" in x]
    assert len(rows) >= 45
    for row in rows:
        cells = [c.strip() for c in row.strip("|").split("|")]
        assert float(cells[2]) > 0.0 and float(cells[4]) > 0.0, row


@pytest.mark.gpu
def test_kernel_bench_flow_compares_the_four_calls_with_the_fused_one(gpu):
    """`python -m nabla_amd.kernel_bench --flow` on one tensor: both rows with a positive time."""
    r = subprocess.run([sys.executable, "-m", "nabla_amd.kernel_bench", "--flow", "--elements", "1e6", "--reps", "2"],
                       capture_output=True, text=True, timeout=300, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    rows = [x for x in r.stdout.splitlines() if x.startswith("| ") and ("four calls" in x or "fused" in x)]
    assert len(rows) == 2
    for row in rows:
        cells = [c.strip() for c in row.strip("|").split("|")]
        assert float(cells[3]) > 0.0 and float(cells[4]) > 0.0, row


@pytest.mark.gpu
def test_every_ceiling_probe_runs_and_reports_a_rate(gpu):
    """`nbo_hbm_ceiling` for every access pattern, in one plain allocation and across the HBM's
    regions, on streams of 192 MiB: a finite positive rate, best >= mean, and the argument checks
    of the entry point.  (No bounds on the rate itself: 192 MiB fits the last-level cache, and a
    shared or throttled GPU may be slow; rates are what `kernel_bench --ceilings` reports.)"""
    import ctypes as C
    import math

    from nabla_amd import _lib
    from nabla_amd import kernel_bench as KB

    L = _lib.load()
    nbytes = 192 << 20
    for pat, (name, ro, rmw, wo) in enumerate(KB.PATTERNS):
        for spread in (0, 1):
            best, mean, regions = C.c_double(), C.c_double(), C.c_int(-1)
            _lib.check(L.nbo_hbm_ceiling(pat, spread, nbytes, 3, 5, C.byref(best), C.byref(mean), C.byref(regions)))
            assert math.isfinite(best.value) and 0.0 < mean.value <= best.value, (name, spread, best.value, mean.value)
            assert regions.value in ((0, 2, 3) if spread else (0,)), (name, spread, regions.value)
    best, mean = C.c_double(), C.c_double()
    for bad in (lambda: L.nbo_hbm_ceiling(len(KB.PATTERNS), 0, nbytes, 3, 0, C.byref(best), C.byref(mean), None),
                lambda: L.nbo_hbm_ceiling(0, 0, nbytes + 4096, 3, 0, C.byref(best), C.byref(mean), None),
                lambda: L.nbo_hbm_ceiling(0, 0, nbytes, 0, 0, C.byref(best), C.byref(mean), None),
                lambda: L.nbo_hbm_ceiling(0, 0, nbytes, 3, 0, None, C.byref(mean), None)):
        assert bad() == _lib.ERR_ARG


@pytest.mark.gpu
def test_every_probe_shape_touches_each_vector_exactly_once_per_launch(gpu):
    """`nbo_hbm_ceiling_shape`: every access shape (register rows, LDS-direct loads, both at once,
    loading and storing waves apart, software-pipelined) over the four 1:1 read/write patterns.
    The in-place streams start at zero and every launch adds 1.0 to each element, so after the
    run every element must equal the number of launches: a window that was skipped, done twice
    or written to the wrong place shows as a mismatch."""
    import ctypes as C
    import math

    from nabla_amd import _lib
    from nabla_amd import kernel_bench as KB

    L = _lib.load()
    nbytes = 48 << 20
    for shape in range(len(KB.SHAPES)):
        for pat in KB.FULL_PATTERNS:
            print(f"probe shape {shape} pattern {pat}", flush=True)
            best, mean, regions, bad = C.c_double(), C.c_double(), C.c_int(-1), C.c_uint64(1 << 60)
            _lib.check(L.nbo_hbm_ceiling_shape(pat, shape, 0, nbytes, 2, 0, C.byref(best), C.byref(mean),
                                               C.byref(regions), C.byref(bad)))
            assert bad.value == 0, (shape, pat, bad.value)
            assert math.isfinite(best.value) and 0.0 < mean.value <= best.value, (shape, pat)
    best, mean = C.c_double(), C.c_double()
    for bad_call in (lambda: L.nbo_hbm_ceiling_shape(0, 3, 0, nbytes, 2, 0, C.byref(best), C.byref(mean), None, None),
                     lambda: L.nbo_hbm_ceiling_shape(9, len(KB.SHAPES), 0, nbytes, 2, 0, C.byref(best), C.byref(mean), None, None),
                     lambda: L.nbo_hbm_ceiling_shape(9, 6, 0, 32768, 2, 0, C.byref(best), C.byref(mean), None, None)):
        assert bad_call() == _lib.ERR_ARG


@pytest.mark.gpu
def test_placed_buffers_are_usable_memory_in_the_regions_asked_for(gpu):
    """`nbo_alloc_placed` (measurement entry point): two buffers in different regions, then the
    rotation the optimizer's state gets; the memory is ordinary device memory (torch reads and
    writes it, the engine steps over tensors carved from it), and the argument checks hold."""
    import ctypes as C

    import numpy as np
    import torch

    import oracle as O
    from nabla_amd import _lib
    from nabla_amd import optim as nb
    from nabla_amd.placed import PlacedBuffers, carved_bytes
    from tests import helpers as H

    shapes = [(4096, 8192), (1, 4097), (3, 5)]
    nbytes = carved_bytes(shapes, 4)
    for regions in ((0, 1), (-1, -1)):
        bufs = PlacedBuffers(nbytes, regions)
        assert "2 regions" in bufs.note() or "3 regions" in bufs.note(), bufs.note()
        p_t, g_t = bufs.carve(0, shapes, torch.float32), bufs.carve(1, shapes, torch.float32)
        p0, g0 = H.randn_list(shapes[1:], 5, 0.02), H.randn_list(shapes[1:], 6, 1e-2)
        p_t[0].zero_(), g_t[0].fill_(1.0)
        for t, a in zip(p_t[1:], p0):
            t.copy_(torch.from_numpy(a).reshape(t.shape))
        for t, a in zip(g_t[1:], g0):
            t.copy_(torch.from_numpy(a).reshape(t.shape))
        opt = nb.Sgd.new(0.5, shapes)
        opt.step(p_t, g_t)
        ref, vel = H.copy_list(p0), H.zeros_like_list(p0)
        O.sgd_step(O.sgd_meta(0.5), ref, g0, vel)
        H.assert_bits_equal(H.host_list(p_t[1:]), ref, f"SGD step over placed buffers, regions {regions}")
        assert bool((p_t[0] == -0.5).all())
        del p_t, g_t, opt
        bufs.close()
    L = _lib.load()
    h, ptrs = C.c_void_p(), (C.c_void_p * 3)()
    for n, reg in ((1, [0]), (4, [0, 1, 2, 0]), (2, [0, 3]), (2, [0, -1])):
        assert L.nbo_alloc_placed(n, 1 << 30, (C.c_int * len(reg))(*reg), ptrs, C.byref(h)) == _lib.ERR_ARG
    assert L.nbo_alloc_placed(2, 1 << 20, (C.c_int * 2)(0, 1), ptrs, C.byref(h)) == _lib.ERR_TOO_LARGE  # below 128 MiB
    assert L.nbo_free_placed(None) == 0
