#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/ with the CPU oracle.

    python tests/golden/make_golden.py

The reference is a Rust workspace and no Rust toolchain exists here, so no vector
can come from running it; these fixtures freeze the oracle's output (after the
oracle itself has been pinned by tests/test_oracle_pinning.py) as plain data:
inputs and expected bit patterns, small enough to read in a diff.  They guard the
oracle against drifting with the host's libm and give the device tests a second,
host-independent target.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
import oracle as O  # noqa: E402

SHAPES = [(1, 1), (3, 5), (1, 1000), (2, 4100)]


def sgd_case():
    p = [O.randn_f32(r * c, 100 + i, 0.05) for i, (r, c) in enumerate(SHAPES)]
    out = {f"p0_{i}": a.copy() for i, a in enumerate(p)}
    vel = [np.zeros_like(a) for a in p]
    meta = O.sgd_meta(0.01)
    for step in range(3):
        g = [O.randn_f32(r * c, 200 + 10 * step + i, 1e-2) for i, (r, c) in enumerate(SHAPES)]
        for i, a in enumerate(g):
            out[f"g{step}_{i}"] = a
        O.sgd_step(meta, p, g, vel)
    for i, a in enumerate(p):
        out[f"p_{i}"] = a
    return out


def adam_case(kind):
    p = {m: [O.randn_f32(r * c, 300 + i, 0.02) for i, (r, c) in enumerate(SHAPES)] for m in (0, 1)}
    out = {f"p0_{i}": a.copy() for i, a in enumerate(p[0])}
    st = {m: ([np.zeros_like(a) for a in p[m]], [np.zeros_like(a) for a in p[m]]) for m in (0, 1)}
    mk = (lambda: O.adam_meta(3e-4)) if kind == "adam" else \
        (lambda: O.adamw_meta(2e-4, 0.9, 0.95, 1e-8, 0.1))
    metas = {0: mk(), 1: mk()}
    for step in range(3):
        g = [O.randn_f32(r * c, 400 + 10 * step + i, 1e-3) for i, (r, c) in enumerate(SHAPES)]
        for i, a in enumerate(g):
            out[f"g{step}_{i}"] = a
        for mode in (0, 1):
            O.set_pow_mode(mode)
            O.adam_step(metas[mode], p[mode], g, st[mode][0], st[mode][1])
        O.set_pow_mode(0)
    for i in range(len(SHAPES)):
        out[f"p_libm_{i}"] = p[0][i]
        out[f"p_sqrt_{i}"] = p[1][i]
        out[f"m_{i}"] = st[0][0][i]
        out[f"v_{i}"] = st[0][1][i]
        assert np.array_equal(st[0][0][i], st[1][0][i]) and np.array_equal(st[0][1][i], st[1][1][i])
    return out


def mixed_case(half="bf16"):
    """bf16 (uint16 patterns) or f16 (float16) params/grads, f32 master/m/v, scaler (growth
    every 2 clean steps), clip 1.0, 6 steps, +inf injected at step 3."""
    narrow = O.bf16_from_f32 if half == "bf16" else (lambda a: O.cast(a, np.float16))
    master = {m: [O.randn_f32(r * c, 500 + i, 0.02) for i, (r, c) in enumerate(SHAPES)] for m in (0, 1)}
    out = {f"w0_{i}": a.copy() for i, a in enumerate(master[0])}
    pb = {m: [narrow(a) for a in master[m]] for m in (0, 1)}
    st = {m: ([np.zeros_like(a) for a in master[m]], [np.zeros_like(a) for a in master[m]]) for m in (0, 1)}
    metas = {m: O.adamw_meta(2e-4, 0.9, 0.95, 1e-8, 0.1) for m in (0, 1)}
    scal = {m: O.ScalerState(65536.0, 2.0, 0.5, 2, 0) for m in (0, 1)}
    trace = []
    for step in range(6):
        scale = scal[0].scale
        g = [narrow(O.randn_f32(r * c, 600 + 10 * step + i, 1e-3 * scale))
             for i, (r, c) in enumerate(SHAPES)]
        if step == 3:
            g[2][77] = 0x7F80 if half == "bf16" else np.inf
        for i, a in enumerate(g):
            out[f"g{step}_{i}"] = a
        for mode in (0, 1):
            O.set_pow_mode(mode)
            ran, norm = O.mixed_step(metas[mode], scal[mode], 1.0, pb[mode], g, master[mode],
                                     st[mode][0], st[mode][1])
        O.set_pow_mode(0)
        trace.append([0.0 if ran else 1.0, scal[0].scale, float(metas[0].step_count), norm])
    out["trace"] = np.array(trace, dtype=np.float64)  # found_inf, scale, step_count, norm
    for i in range(len(SHAPES)):
        out[f"p_libm_{i}"], out[f"p_sqrt_{i}"] = pb[0][i], pb[1][i]
        out[f"w_libm_{i}"], out[f"w_sqrt_{i}"] = master[0][i], master[1][i]
        out[f"m_{i}"], out[f"v_{i}"] = st[0][0][i], st[0][1][i]
    return out


def main():
    np.savez_compressed(os.path.join(HERE, "sgd_f32.npz"), **sgd_case())
    np.savez_compressed(os.path.join(HERE, "adam_f32.npz"), **adam_case("adam"))
    np.savez_compressed(os.path.join(HERE, "adamw_f32.npz"), **adam_case("adamw"))
    np.savez_compressed(os.path.join(HERE, "mixed_adamw_bf16.npz"), **mixed_case())
    np.savez_compressed(os.path.join(HERE, "mixed_adamw_f16.npz"), **mixed_case("f16"))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
