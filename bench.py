#!/usr/bin/env python3
"""Benchmark of the fused optimizer step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama3-8b]

One "step" is one Trainer tail over the whole synthetic parameter set, with
gradients already resident in HBM: unscale + found-inf check, global-norm clip to
1.0, mixed-precision AdamW update (bf16 params/grads, f32 master/m/v).  Prints one
JSON line: whole-step algorithmic HBM throughput (30 B/param/step) from a timed pass
that records no events, the spread over the steps and the roofline figure of the
dominant kernel from two further passes with HIP events on the launch stream, the CPU
restatement of the reference timed on this host's cores on a bounded sample, and the
device path's parity with it on that sample.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E peak
BYTES_UPDATE = 28       # per param: R g2 + master4 + m4 + v4, W master4 + m4 + v4 + p2
BYTES_NORM = 2          # per param: R g2
ROOT = os.path.dirname(os.path.abspath(__file__))

# The driver clears device memory that has been freed, in the background, and that competes with
# the step for HBM bandwidth until it is done (measured: the 1.1B set runs 5.20 instead of 5.13 ms
# per step for 3.7 s after its placement search released 91 GiB; the free-memory figure does not
# show it).  The benchmark therefore keeps count of what it -- and the state placement on its
# behalf -- has released, and idles in proportion before it times anything.
CLEARING_GIB_PER_S = 20.0  # cautious: 24-25 GiB/s was observed, with the GPU busy or idle
_released_gib = 0.0
WAKE_UP_S = 0.05


def note_released(gib):
    global _released_gib
    _released_gib += max(0.0, gib)


def wait_for_clearing(base_s):
    """Idles base_s plus the time the driver needs for what has been released so far; returns
    the seconds waited."""
    global _released_gib
    wait = base_s + (_released_gib / CLEARING_GIB_PER_S if base_s > 0 else 0.0)
    _released_gib = 0.0
    time.sleep(wait)
    return round(wait, 2)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="llama3-8b",
                    choices=["llama3-8b", "llama-1.1b", "gpt2-small-f32", "mlp-sgd-f32", "ragged-4096", "ragged-4096-packed",
                             "llama-1.1b-bf16", "llama-1.1b-f16", "llama-1.1b-f16-mixed"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-ceiling", action="store_true",
                    help="skip the micro-kernel measurement of the memory system's read-modify-write ceiling")
    ap.add_argument("--zero-grads", choices=["off", "fused", "separate"], default="off",
                    help="also clear the gradients every step (trainer.rs:285-290): inside the update "
                         "kernel, or as a separate pass; +2 B/param of writes, reported in the config")
    ap.add_argument("--primary-only", action="store_true",
                    help="with the default workload, skip the additional llama-1.1b measurement")
    ap.add_argument("--calibrate-copy", type=float, default=0.0, metavar="GiB",
                    help="instead of the benchmark, run the library's plain copy kernel over "
                         "this many GiB (--steps times); a transfer of known size against which "
                         "rocprofv3's FETCH_SIZE / WRITE_SIZE counters are scaled")
    ap.add_argument("--table", action="store_true",
                    help="instead of one JSON line, measure every workload (--steps / --warmup each, --cpu-seconds of "
                         "CPU baseline each) and print a markdown table")
    ap.add_argument("--settle-seconds", type=float, default=2.0,
                    help="idle time between setup and the warm-up steps, for the driver's background clearing of "
                         "the device memory that setup freed to finish; one second per 20 GiB released is added "
                         "(0: no waiting at all)")
    ap.add_argument("--cpu-seconds", type=float, default=20.0,
                    help="rough budget for the CPU baseline sample")
    return ap.parse_args()


def workload(name):
    from nabla_amd import workloads as W

    if name == "llama3-8b":
        return dict(shapes=W.llama_8b_shapes(), mixed=True, kind="adamw", lr=2e-4, wd=0.1,
                    betas=(0.9, 0.95), scaler=True, clip=1.0, p_sigma=0.02, g_sigma=1e-3)
    if name == "llama-1.1b":
        return dict(shapes=W.llama_1b_shapes(), mixed=True, kind="adamw", lr=2e-4, wd=0.1,
                    betas=(0.9, 0.95), scaler=True, clip=1.0, p_sigma=0.02, g_sigma=1e-3)
    if name in ("llama-1.1b-bf16", "llama-1.1b-f16"):  # Optimizer<bf16> / Optimizer<f16>: all in 16 bits
        return dict(shapes=W.llama_1b_shapes(), mixed=False, pure=True, half=name[-4:].lstrip("-"), kind="adamw",
                    lr=2e-4, wd=0.1, betas=(0.9, 0.95), eps=1e-8 if name.endswith("bf16") else 1e-4,
                    scaler=True, clip=1.0, p_sigma=0.02, g_sigma=1e-3)
    if name == "llama-1.1b-f16-mixed":  # f16 tensors over f32 master weights and moments
        return dict(shapes=W.llama_1b_shapes(), mixed=True, half="f16", kind="adamw", lr=2e-4, wd=0.1,
                    betas=(0.9, 0.95), scaler=True, clip=1.0, p_sigma=0.02, g_sigma=1e-3)
    if name in ("ragged-4096", "ragged-4096-packed"):  # packed: tensors back to back in two flat buffers
        return dict(packed=name.endswith("packed"), shapes=[(1, n) for n in W.ragged_sizes()], mixed=True, kind="adamw", lr=2e-4,
                    wd=0.1, betas=(0.9, 0.95), scaler=True, clip=1.0, p_sigma=0.02, g_sigma=1e-3)
    if name == "gpt2-small-f32":
        return dict(shapes=W.gpt2_small_shapes(), mixed=False, kind="adam", lr=3e-4, wd=0.0,
                    betas=(0.9, 0.999), scaler=False, clip=0.0, p_sigma=0.02, g_sigma=1e-3)
    return dict(shapes=W.MLP_SHAPES, mixed=False, kind="sgd", lr=0.01, wd=0.0, betas=(0.0, 0.0),
                scaler=False, clip=0.0, p_sigma=0.05, g_sigma=1e-2)


def bytes_per_param(cfg):
    if cfg.get("pure"):
        return 14, 2  # R p, g, m, v + W p, m, v at 2 B each; norm pass R g
    if cfg["kind"] == "sgd":
        return 12, 0
    if cfg["mixed"]:
        return BYTES_UPDATE, BYTES_NORM
    return 28, 0


def baseline_sample(cfg):
    """The tensors the CPU baseline and the parity check run on: the workload's own tensors in
    list order until the sample holds ~24 M params (a tensor that would take it past 64 M is
    left out), but at least one tensor."""
    sample, n = [], 0
    for s in cfg["shapes"]:
        if n and n + s[0] * s[1] > 64_000_000:
            continue
        sample.append(s)
        n += s[0] * s[1]
        if n >= 24_000_000:
            break
    return sample, n


def _oracle_meta(cfg):
    import oracle as O

    if cfg["kind"] == "sgd":
        return O.sgd_meta(cfg["lr"])
    if cfg["kind"] == "adam":
        return O.adam_meta(cfg["lr"], *cfg["betas"])
    return O.adamw_meta(cfg["lr"], *cfg["betas"], eps=cfg.get("eps", 1e-8), weight_decay=cfg["wd"])


def cpu_baseline(cfg, budget_s):
    """The oracle ("port" of the reference's CPU backend) on this host: every Backend
    primitive a separate pass with a fresh output, element-parallel passes on all
    cores, the reference's serial passes serial.  Timed on a sample of the workload's
    own tensors sized to roughly `budget_s` seconds."""
    import numpy as np

    import oracle as O

    cores = len(os.sched_getaffinity(0))
    O.set_threads(cores)
    sample, n = baseline_sample(cfg)
    rng = np.random.default_rng(0)
    f32 = np.float32
    master = [(rng.standard_normal(r * c, dtype=f32) * f32(cfg["p_sigma"])) for r, c in sample]
    m = [np.zeros_like(a) for a in master]
    v = [np.zeros_like(a) for a in master]
    scale = 65536.0 if cfg["scaler"] else 1.0
    g32 = [(rng.standard_normal(r * c, dtype=f32) * f32(cfg["g_sigma"] * scale)) for r, c in sample]
    meta = _oracle_meta(cfg)
    scaler = O.default_scaler() if cfg["scaler"] else None
    narrow = (lambda a: O.cast(a, np.float16)) if cfg.get("half") == "f16" else O.bf16_from_f32
    if cfg.get("pure"):
        p = [narrow(a) for a in master]
        m, v = [np.zeros_like(a) for a in p], [np.zeros_like(a) for a in p]
        g16 = [narrow(a) for a in g32]

        def run():  # trainer.rs:230-283 with T = bf16 / f16
            gg = [a.copy() for a in g16]
            if O.scaler_unscale_and_update(scaler, gg):
                O.clip_grad_norm(gg, cfg["clip"])
                O.adam_step(meta, p, gg, m, v)
    elif cfg["mixed"]:
        g = [narrow(a) for a in g32]
        p = [narrow(a) for a in master]
        run = lambda: O.mixed_step(meta, scaler, cfg["clip"], p, g, master, m, v)  # noqa: E731
    elif cfg["kind"] == "sgd":
        run = lambda: O.sgd_step(meta, master, g32, m)  # noqa: E731
    else:
        def run():
            gg = [a.copy() for a in g32]
            return O.f32_step(meta, scaler, cfg["clip"], master, gg, m, v)
    run()  # warm (page faults, thread pool)
    steps, t0 = 0, time.perf_counter()
    while True:
        run()
        steps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or steps >= 50:
            break
    upd, nrm = bytes_per_param(cfg)
    pps = n * steps / el
    return {
        "value": round(pps * (upd + nrm) / 1e9, 3),
        "unit": "GB/s",
        "cores": cores,
        "kind": "port",
        "params_per_s": round(pps, 1),
        "ms_per_step_sample": round(el / steps * 1e3, 2),
        "sample": f"first {len(sample)} tensors of the workload ({n} params), {steps} steps; "
                  "reference-faithful pass chain (12 passes/tensor for AdamW, fresh output each), "
                  f"rayon-parallel passes on {cores} threads, map/scan/clip passes serial",
    }


def parity_check(cfg, steps=3):
    """Part of the CPU-baseline leg: the device path and the oracle on the same seeded inputs
    (the reference's xorshift64 + Box-Muller generator), `steps` steps over the CPU baseline's
    sample of the workload, compared after the last step against both variants of the oracle
    (denominator by correctly rounded sqrt, as the device computes it, and by libm powf as the
    reference's source reads).  Reports, per state array, the largest distance in units of the
    last place, the number of elements beyond 2 ulp (f32) / 1 ulp (16-bit), and whether every
    step's decisions (found_inf, clipped, scale, step_count) agree bit for bit."""
    import numpy as np
    import torch

    import oracle as O
    from nabla_amd import optim as nb

    sample, n = baseline_sample(cfg)
    pure, half = bool(cfg.get("pure")), cfg.get("half", "bf16")
    mixed = cfg["mixed"]
    scale = 65536.0 if cfg["scaler"] else 1.0
    master0 = [O.randn_f32(r * c, 1000 + i, cfg["p_sigma"]) for i, (r, c) in enumerate(sample)]
    g32 = [O.randn_f32(r * c, 5000 + i, cfg["g_sigma"] * scale) for i, (r, c) in enumerate(sample)]
    narrow = (lambda a: O.cast(a, np.float16)) if half == "f16" else O.bf16_from_f32
    hdt = torch.float16 if half == "f16" else torch.bfloat16

    def dev(a, shape):
        if a.dtype == np.uint16:
            return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to("cuda:0").reshape(shape)
        return torch.from_numpy(a.copy()).to("cuda:0").reshape(shape)

    def host(t):
        t = t.detach().reshape(-1).cpu()
        if t.dtype == torch.bfloat16:
            return t.view(torch.int16).numpy().view(np.uint16).copy()
        return t.numpy().copy()

    if pure or mixed:
        p0, g0 = [narrow(a) for a in master0], [narrow(a) for a in g32]
    else:
        p0, g0 = [a.copy() for a in master0], g32
    # ---- device ----
    if cfg["kind"] == "sgd":
        opt = nb.Sgd.new(cfg["lr"], sample)
    elif cfg["kind"] == "adam":
        opt = nb.Adam.new(cfg["lr"], sample).beta1(cfg["betas"][0]).beta2(cfg["betas"][1])
    else:
        opt = nb.AdamW.new(cfg["lr"], sample, master=mixed, dtype=half if pure else "f32") \
            .beta1(cfg["betas"][0]).beta2(cfg["betas"][1]).eps(cfg.get("eps", 1e-8)).weight_decay(cfg["wd"])
    p_dev = [dev(a, s) for a, s in zip(p0, sample)]
    g_dev = [dev(a, s) for a, s in zip(g0, sample)]
    if mixed:
        for i, a in enumerate(master0):
            opt.write_state(f"w{i}", dev(a, sample[i]))
    scaler_dev = nb.GradScaler.new() if cfg["scaler"] else None
    fused = cfg["scaler"] or cfg["clip"] > 0
    dev_decisions = []
    for _ in range(steps):
        if fused:
            opt.fused_step(p_dev, g_dev, scaler=scaler_dev, max_norm=cfg["clip"])
            i = opt.last_step()
            dev_decisions.append((i.found_inf, i.clipped, i.scale, i.step_count))
        else:
            opt.step(p_dev, g_dev)
    got = {"params": [host(t) for t in p_dev]}
    if cfg["kind"] != "sgd":
        got["m"] = [host(opt.read_state(f"m{i}")) for i in range(len(sample))]
        got["v"] = [host(opt.read_state(f"v{i}")) for i in range(len(sample))]
    if mixed:
        got["master"] = [host(opt.read_state(f"w{i}")) for i in range(len(sample))]
    del opt, p_dev, g_dev

    # ---- oracle, both variants of the denominator ----
    def oracle_run(mode):
        O.set_pow_mode(mode)
        try:
            meta = _oracle_meta(cfg)
            sc = O.default_scaler() if cfg["scaler"] else None
            p = [a.copy() for a in p0]
            master = [a.copy() for a in master0]
            zeros = (lambda: [np.zeros_like(a) for a in p]) if pure else (lambda: [np.zeros_like(a) for a in master0])
            m, v = zeros(), zeros()
            decisions = []
            for _ in range(steps):
                if pure:
                    gg = [a.copy() for a in g0]
                    ok = O.scaler_unscale_and_update(sc, gg)
                    norm = O.clip_grad_norm(gg, cfg["clip"]) if ok else 0.0
                    if ok:
                        O.adam_step(meta, p, gg, m, v)
                    decisions.append((0 if ok else 1, int(ok and norm > cfg["clip"] > 0), sc.scale, meta.step_count))
                elif mixed:
                    ok, norm = O.mixed_step(meta, sc, cfg["clip"], p, g0, master, m, v)
                    decisions.append((0 if ok else 1, int(ok and norm > cfg["clip"] > 0), sc.scale, meta.step_count))
                elif cfg["kind"] == "sgd":
                    O.sgd_step(meta, p, g0, m)
                else:
                    gg = [a.copy() for a in g0]
                    O.f32_step(meta, sc, cfg["clip"], p, gg, m, v)
            ref = {"params": p}
            if cfg["kind"] != "sgd":
                ref["m"], ref["v"] = m, v
            if mixed:
                ref["master"] = master
            return ref, decisions
        finally:
            O.set_pow_mode(O.POW_LIBM)

    # Two ways in which one ulp of the update (the reference's powf(x, 0.5) against the correctly
    # rounded sqrt: 0.06 % of inputs) becomes more than 2 ulp of an f32 parameter:
    # (a) parameter and update nearly cancel, so the ulp of the update is many ulps of the tiny
    #     result: |difference| <= steps * 8 * lr * 2^-23 and magnitude < 16 * lr * steps;
    # (b) p - update lies next to a rounding tie, so the ulp of the update turns p's rounding:
    #     one ulp of p per step at most, and with the same gradient in every step, as here, the
    #     same element ties again in every step: |difference| <= steps ulps of the larger of the
    #     parameter's first and last value.
    bound, small = steps * 8 * cfg["lr"] * 2.0 ** -23, 16.0 * cfg["lr"] * steps
    start = {"params": p0, "master": master0}

    def compare(ref):
        out = {}
        for key, arrs in got.items():
            sixteen = arrs[0].dtype in (np.uint16, np.float16)
            worst = beyond = cancel = flips = 0
            for i, (a, b) in enumerate(zip(arrs, ref[key])):
                if not a.size:
                    continue
                d = O.ulp_distance_bf16(a.view(np.uint16), b.view(np.uint16)) if sixteen else O.ulp_distance_f32(a, b)
                worst = max(worst, int(d.max()))
                far = d > (1 if sixteen else 2)
                beyond += int(far.sum())
                if far.any() and not sixteen and key in start:
                    x, y = a[far].astype(np.float64), b[far].astype(np.float64)
                    diff, big = np.abs(x - y), np.maximum(np.abs(x), np.abs(y))
                    in_a = (diff <= bound) & (big < small)
                    ulp_p = np.spacing(np.maximum(np.abs(start[key][i][far]), big.astype(np.float32)).astype(np.float32))
                    in_b = ~in_a & (diff <= steps * ulp_p.astype(np.float64))
                    cancel += int(in_a.sum())
                    flips += int(in_b.sum())
            out[key] = {"max_ulp": worst, "beyond_bar": beyond, "near_cancellation": cancel, "rounding_ties": flips,
                        "unexplained": beyond - cancel - flips}
        return out

    ref_sqrt, dec_sqrt = oracle_run(O.POW_SQRT)
    ref_libm, dec_libm = oracle_run(O.POW_LIBM)
    return {
        "sample": f"first {len(sample)} tensors of the workload ({n} params), {steps} steps, inputs from the "
                  "reference's xorshift64 + Box-Muller generator",
        "bar": "f32 states within 2 ulp, 16-bit params within 1 ulp, decisions bit-exact; an f32 parameter beyond 2 ulp "
               f"must either differ by at most steps * 8 * lr * 2^-23 = {bound:.3e} and be smaller than 16 * lr * steps = "
               f"{small:.3e} (near_cancellation of parameter and update) or differ by at most {steps} ulps of its "
               "larger end (rounding_ties: p - update next to a tie in every step, the gradient being the same in "
               "every step); `unexplained` must be 0",
        "decisions_bit_exact": (not fused) or (dev_decisions == dec_sqrt == dec_libm),
        "vs_oracle_sqrt": compare(ref_sqrt),
        "vs_oracle_libm_powf": compare(ref_libm),
    }


def measured_ceiling(achieved_gbps):
    """What this GPU's memory system gives an in-place read-modify-write over three streams
    placed across the HBM's regions like optimizer state, and the update's own stream shape
    (1 read, 3 in place, 1 written), measured now with the library's probe kernels
    (`nbo_hbm_ceiling`; `python -m nabla_amd.kernel_bench --ceilings` has the whole table):
    the yardstick next to the nominal 8 TB/s."""
    from nabla_amd import kernel_bench as KB

    wait_for_clearing(1.0)  # the workloads measured before have just been torn down
    rows = KB.measure_ceilings(gib=2.0, reps=10, patterns=(6, 7, 9), spreads=(1,))
    name, spread, best, mean, regions, rw = max(rows, key=lambda r: r[3])
    return {"ceiling_measured": round(mean, 1),
            "ceiling_kernel": f"nbo_hbm_ceiling: {name}, 2 GiB per stream, "
                              f"{'placed across ' + str(regions) + ' HBM regions' if spread else 'one plain allocation'}, "
                              "mean of 10 launches",
            "frac_of_ceiling_measured": round(achieved_gbps / mean, 4) if mean > 0 else None}


def measure(name, steps, warmup, zero_grads="off", settle_s=2.0):
    """Builds the workload on the device, runs `warmup` + `steps` steps, returns the
    result record (without the CPU baseline)."""
    import ctypes as C

    import torch

    from nabla_amd import _lib
    from nabla_amd import optim as nb

    L = _lib.load()
    cfg = workload(name)
    shapes = cfg["shapes"]
    n = sum(r * c for r, c in shapes)
    dev = torch.device("cuda:0")
    torch.manual_seed(0)

    pure, half = bool(cfg.get("pure")), cfg.get("half", "bf16")
    hdt = torch.float16 if half == "f16" else torch.bfloat16
    pdt = hdt if (cfg["mixed"] or pure) else torch.float32
    if cfg.get("packed"):
        # most tensors then start at addresses that are only element-aligned
        flat_p, flat_g = torch.empty(n, dtype=pdt, device=dev), torch.empty(n, dtype=pdt, device=dev)
        offs = [0]
        for r, c in shapes:
            offs.append(offs[-1] + r * c)
        params = [flat_p[offs[i]:offs[i + 1]].view(shapes[i]) for i in range(len(shapes))]
        grads = [flat_g[offs[i]:offs[i + 1]].view(shapes[i]) for i in range(len(shapes))]
    else:
        params = [torch.empty(s, dtype=pdt, device=dev) for s in shapes]
        grads = [torch.empty(s, dtype=pdt, device=dev) for s in shapes]
    free_before_state = torch.cuda.mem_get_info()[0]
    if cfg["kind"] == "sgd":
        opt = nb.Sgd.new(cfg["lr"], shapes)
    elif cfg["kind"] == "adam":
        opt = nb.Adam.new(cfg["lr"], shapes).beta1(cfg["betas"][0]).beta2(cfg["betas"][1])
    else:
        opt = nb.AdamW.new(cfg["lr"], shapes, master=cfg["mixed"], dtype=half if pure else "f32") \
            .beta1(cfg["betas"][0]).beta2(cfg["betas"][1]).eps(cfg.get("eps", 1e-8)).weight_decay(cfg["wd"])
    # what the placement search created beyond what the state keeps has been released again
    searched = re.search(r"chunks of (\d+) MiB; (\d+) chunks created", opt.state_placement_note())
    if searched:
        kept_gib = (free_before_state - torch.cuda.mem_get_info()[0]) / 2**30
        note_released(int(searched.group(1)) * int(searched.group(2)) / 1024 - kept_gib)
    scale = 65536.0 if cfg["scaler"] else 1.0
    for i, s in enumerate(shapes):  # synthetic, random-init
        w = torch.randn(s, dtype=torch.float32, device=dev) * cfg["p_sigma"]
        if cfg["mixed"]:
            opt.write_state(f"w{i}", w)
        else:
            params[i].copy_(w)
        grads[i].copy_((torch.randn(s, dtype=torch.float32, device=dev) * (cfg["g_sigma"] * scale)).to(pdt))
        del w
    plist, glist = nb.TensorList(params), nb.TensorList(grads)
    if cfg["mixed"]:
        opt.params_from_master(plist)
    scaler = nb.GradScaler.new() if cfg["scaler"] else None
    reserved = torch.cuda.memory_reserved()
    torch.cuda.empty_cache()
    note_released((reserved - torch.cuda.memory_reserved()) / 2**30)  # the temporaries of the fill above

    fused = cfg["scaler"] or cfg["clip"] > 0

    def step():
        if fused:
            opt.fused_step(plist, glist, scaler=scaler, max_norm=cfg["clip"], zero_grads=zero_grads == "fused")
        else:
            opt.step(plist, glist)
        if zero_grads == "separate" or (zero_grads == "fused" and not fused):
            nb.zero_grad(glist)

    upd_b, nrm_b = bytes_per_param(cfg)
    zero_b = 0 if zero_grads == "off" else (2 if (cfg["mixed"] or pure) else 4)
    fam = ("pf16" if half == "f16" else "pbf16") if pure else half if cfg["mixed"] else "f32"
    # The update kernel comes in three forms: one workgroup per chunk, the same preparing its own
    # scalars ("_self": the unfused Adam / AdamW step in one launch) and one workgroup per row of a
    # chunk ("_rows": lists of middle size; unfused, behind the scalar-preparation launch).  The
    # library chooses; the third pass below sees which one ran.
    base = f"nbo_update_{fam}_{cfg['kind']}"
    candidates = [base] + ([] if cfg["kind"] == "sgd" else [base + "_self", base + "_rows"])
    names = candidates + ([f"nbo_norm_{fam}", "nbo_finalize"] if fused else ["nbo_prep"])
    # Setup has just freed tens of GiB (the placement search's spare chunks, torch's temporaries,
    # the previous workload), and the driver clears freed device memory in the background
    # (measured: 37.9 instead of 37.3 ms per step on the 8B set while it does).  It is the
    # benchmark's own setup, not the step, so it is given time to finish.
    torch.cuda.synchronize()
    _lib.check(L.nbo_sync())
    settled_s = wait_for_clearing(settle_s)
    # After an idle wait the GPU takes some 20 ms of work to clock up again; a workload whose
    # warm-up steps are shorter than that is given 50 ms of untimed steps first.
    wake_t0 = time.perf_counter()
    while settled_s > 0 and n < 2_000_000_000 and time.perf_counter() - wake_t0 < WAKE_UP_S:
        for _ in range(10):
            step()
        _lib.check(L.nbo_sync())
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    _lib.check(L.nbo_sync())
    # The timed region holds the steps and nothing else: no event is recorded inside it.
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    _lib.check(L.nbo_sync())
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    # Second pass, untimed: every step between one pair of events on the stream the library
    # launches on (the null stream, which is torch's current one), for the spread over the steps.
    assert torch.cuda.current_stream().cuda_stream == 0, "the library launches on the null stream"
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for e0, e1 in pairs:
        e0.record()
        step()
        e1.record()
    torch.cuda.synchronize()
    per_step = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
    # Third pass, untimed: the library brackets each of its launches with events on its launch
    # stream; the dominant kernel's average duration is the roofline figure.
    _lib.check(L.nbo_profile_enable(1))
    for _ in range(steps):
        step()
    per_kernel = {}
    for kname in names:
        cnt, ms = C.c_uint64(0), C.c_double(0.0)
        if L.nbo_profile_read(kname.encode(), C.byref(cnt), C.byref(ms)) != 0:
            if kname == base:
                raise RuntimeError(f"the library has no kernel {kname}")
            cnt.value, ms.value = 0, 0.0  # a form this element type does not have (16-bit state has no "_rows")
        per_kernel[kname] = (cnt.value, ms.value)
    _lib.check(L.nbo_profile_enable(0))
    dom = max(candidates, key=lambda k: per_kernel[k][0])
    per_kernel = {k: v for k, v in per_kernel.items() if v[0] > 0 or k == dom}

    ms_step = (t1 - t0) / steps * 1e3
    gbps = n * (upd_b + nrm_b + zero_b) / (ms_step * 1e-3) / 1e9
    dom_ms = per_kernel[dom][1] / max(per_kernel[dom][0], 1)
    dom_b = upd_b + (zero_b if zero_grads == "fused" and fused else 0)  # fused zeroing: the update kernel writes g too
    dom_gbps = n * dom_b / (dom_ms * 1e-3) / 1e9 if dom_ms > 0 else 0.0
    info = opt.last_step() if fused else None

    # HBM bytes per launch by rocprofv3's counters: they cannot be read from inside this process,
    # so the figure is the one a counter run of this same command left in profiles/traffic.json
    # (see nabla_amd/profile_summary.py) and the line says so
    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            table = json.load(f)
        traffic = table.get(f"{name}:{dom}")
        det = table.get("_detail", {}).get(name, {})
        if traffic is not None:
            from nabla_amd.profile_summary import kernel_source_hash

            same = det.get("kernel_source_sha256") == kernel_source_hash()
            traffic_source = (f"profiles/traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE run of this command at "
                              f"commit {det.get('commit', '?')} on {det.get('date', '?')}; not measured in this run; the "
                              f"kernel source is {'the one' if same else 'NOT the one'} those counters were collected for)")

    out = {
        "metric": "AdamW step HBM GB/s (% of peak) + params/s, bf16-mixed, whole step "
                  "(unscale + found_inf + clip + update)"
        if cfg["kind"] == "adamw" else f"{cfg['kind']} step HBM GB/s",
        "value": round(gbps, 1),
        "unit": "GB/s",
        "pct_of_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "params_per_s": round(n / (ms_step * 1e-3), 1),
        "n_gpus": 1,
        "steps": steps,
        "warmup": warmup,
        "ms_per_step": round(ms_step, 4),
        "ms_per_step_spread": {"min": round(per_step[0], 4), "median": round(per_step[len(per_step) // 2], 4),
                               "max": round(per_step[-1], 4),
                               "how": "a second pass of the same number of steps, each between one pair of HIP "
                                      "events on the launch stream; `ms_per_step` and `value` are the mean of the "
                                      "timed pass (wall clock around all steps, no events inside)"},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": half if pure else "f32",
        "storage": (f"{half} params/grads/m/v" if pure else
                    f"{half} params/grads, f32 master/m/v" if cfg["mixed"] else "f32 params/grads/m/v"),
        "data": "synthetic (random-init parameters and gradients of the named shapes, resident in HBM)",
        "config": {"workload": name, "tensors": len(shapes), "params": n,
                   "bytes_per_param_step": upd_b + nrm_b + zero_b, "zero_grads": zero_grads,
                   "optimizer": cfg["kind"],
                   "loss_scale": scale if cfg["scaler"] else None, "clip_max_norm": cfg["clip"] or None,
                   "state_hbm_regions": opt.state_regions(), "state_placement": opt.state_placement_note(),
                   "settle_s_after_setup": settled_s,
                   "wake_up_s_after_idle": WAKE_UP_S if (settled_s > 0 and n < 2_000_000_000) else 0.0},
        "roofline": {
            "kernel": dom,
            "bound": "hbm",
            "achieved": round(dom_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dom_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "algorithmic_bytes_per_launch": n * dom_b,
            "avg_launch_ms": round(dom_ms, 4),
            "launches": per_kernel[dom][0],
            "how": "HIP events around each launch on the library's launch stream, in a pass of its own after the "
                   "timed one",
        },
        "kernels_ms": {k: round(v[1] / max(v[0], 1), 4) for k, v in per_kernel.items()},
    }
    if info is not None:
        out["last_step"] = {"found_inf": info.found_inf, "clipped": info.clipped,
                            "norm": info.norm, "scale": info.scale, "step_count": info.step_count}
    free_before_teardown = torch.cuda.mem_get_info()[0]
    del opt, plist, glist, params, grads
    torch.cuda.empty_cache()
    note_released((torch.cuda.mem_get_info()[0] - free_before_teardown) / 2**30)
    return out, cfg


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build measures one GPU only (got --gpus {args.gpus}); "
              "the optimizer step has no multi-GPU path here", file=sys.stderr)
        sys.exit(2)
    sys.path.insert(0, ROOT)
    import ctypes as C

    import torch

    from nabla_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the engine has no CPU path", file=sys.stderr)
        sys.exit(3)
    _lib.init()
    L = _lib.load()
    if args.calibrate_copy > 0:
        dev = torch.device("cuda:0")
        nbytes = int(args.calibrate_copy * (1 << 30)) // 16 * 16
        src = torch.ones(nbytes // 4, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        _lib.check(L.nbo_profile_enable(1))
        for _ in range(args.steps):
            _lib.check(L.nbo_copy_bytes(src.data_ptr(), dst.data_ptr(), nbytes))
        cnt, ms = C.c_uint64(0), C.c_double(0.0)
        _lib.check(L.nbo_profile_read(b"nbo_copy_f32x4", C.byref(cnt), C.byref(ms)))
        print(json.dumps({"calibrate": "nbo_copy_f32x4", "bytes_read": nbytes, "bytes_written": nbytes,
                          "launches": cnt.value, "avg_launch_ms": round(ms.value / max(cnt.value, 1), 4),
                          "GBps": round(2 * nbytes / (ms.value / max(cnt.value, 1)) / 1e6, 1)}))
        return
    if args.table:
        names = ["mlp-sgd-f32", "gpt2-small-f32", "llama-1.1b", "llama-1.1b-bf16", "llama-1.1b-f16", "llama-1.1b-f16-mixed",
                 "ragged-4096", "ragged-4096-packed", "llama3-8b"]
        print(f"`python bench.py --table --steps {args.steps} --warmup {args.warmup} --cpu-seconds {args.cpu_seconds}` on one "
              "MI355X: `value` is whole-step algorithmic HBM throughput, `kernel` the dominant kernel's (HIP events on the "
              "launch stream), `CPU` the oracle in reference-faithful form on the host's cores on a sample of the same "
              "workload.\n")
        print("| workload | params | ms/step (min / median / max) | value GB/s | % of 8 TB/s | params/s | dominant kernel "
              "GB/s | HBM regions of state | CPU params/s (cores) | GPU/CPU | parity vs sqrt oracle: max ulp m / v / "
              "master / params | parity vs libm-powf oracle: max ulp m / v / master / params (elements beyond 2 ulp, or 1 ulp of a 16-bit type; of those, neither near-cancellation nor a rounding tie in every step) | "
              "decisions |")
        print("|---|---|---|---|---|---|---|---|---|---|---|---|---|")

        def ulps(cmp):
            return " / ".join(str(cmp[k]["max_ulp"]) if k in cmp else "-" for k in ("m", "v", "master", "params"))

        for name in names:
            d, cfg = measure(name, args.steps, args.warmup, "off", args.settle_seconds)
            c = cpu_baseline(cfg, args.cpu_seconds)
            par = parity_check(cfg)
            beyond = sum(x["beyond_bar"] for x in par["vs_oracle_libm_powf"].values())
            unexplained = sum(x["unexplained"] for x in par["vs_oracle_libm_powf"].values())
            sp = d["ms_per_step_spread"]
            print(f"| {name} | {d['config']['params']:,} | {d['ms_per_step']} ({sp['min']} / {sp['median']} / {sp['max']}) | "
                  f"{d['value']} | {d['pct_of_peak']} | "
                  f"{d['params_per_s']:.3e} | {d['roofline']['achieved']} ({d['roofline']['kernel']}) | "
                  f"{d['config']['state_hbm_regions']} | {c['params_per_s']:.3e} ({c['cores']}) | "
                  f"{d['params_per_s'] / c['params_per_s']:.0f}x | {ulps(par['vs_oracle_sqrt'])} | "
                  f"{ulps(par['vs_oracle_libm_powf'])} ({beyond}; unexplained: {unexplained}) | "
                  f"{'bit-exact' if par['decisions_bit_exact'] else 'DIFFER'} |", flush=True)
        return
    out, cfg = measure(args.workload, args.steps, args.warmup, args.zero_grads, args.settle_seconds)
    if args.workload == "llama3-8b" and not args.primary_only:
        # the metric is quoted on the 1.1B and the 8B shapes: the smaller one rides along
        # (ten warm-up steps: after the idle wait the GPU takes some 20 ms of work to clock up again)
        try:
            small, _ = measure("llama-1.1b", 20, 10, settle_s=args.settle_seconds)
            out["also"] = {"llama-1.1b": {k: small[k] for k in ("value", "unit", "pct_of_peak", "params_per_s",
                                                                "ms_per_step", "ms_per_step_spread", "steps", "warmup",
                                                                "config", "roofline", "kernels_ms")}}
        except Exception as e:  # the ride-along must not cost the headline measurement
            out["also"] = {"llama-1.1b": {"error": str(e)}}
    if not args.no_ceiling and out["roofline"]["achieved"] > 0:
        try:
            out["roofline"].update(measured_ceiling(out["roofline"]["achieved"]))
        except Exception as e:  # the yardstick must not cost the measurement
            out["roofline"].update({"ceiling_measured": None, "ceiling_kernel": f"not measured: {e}"})
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, args.cpu_seconds)
        out["cpu_baseline"]["gpu_over_cpu"] = round(out["value"] / max(out["cpu_baseline"]["value"], 1e-9), 1)
        try:
            out["parity"] = parity_check(cfg)
        except Exception as e:  # the check must not cost the measurement
            out["parity"] = {"error": f"{type(e).__name__}: {e}"}
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
