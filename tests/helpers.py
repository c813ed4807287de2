"""Shared helpers for the parity tests: seeded inputs, oracle <-> device plumbing,
ulp comparisons.  The oracle is the checker only; the device path under test is
always libnabla_optim.so through nabla_amd.optim."""
from __future__ import annotations

import numpy as np

import oracle as O

from nabla_amd.workloads import (MLP_SHAPES, gpt2_small_shapes, llama_1b_shapes,  # noqa: F401,E402
                                 llama_8b_shapes, llama_shapes, ragged_sizes)

# ---- seeded tensors (the reference's xorshift64 + Box-Muller stream) ----------------

def randn_list(shapes, seed0, sigma, dtype=np.float32):
    out = []
    for i, (r, c) in enumerate(shapes):
        n = r * c
        a = O.randn_f64(n, seed0 + i) * sigma
        out.append(a.astype(dtype))
    return out


def zeros_like_list(arrs):
    return [np.zeros_like(a) for a in arrs]


def copy_list(arrs):
    return [a.copy() for a in arrs]


# ---- numpy <-> torch (device) -----------------------------------------------------------

def to_dev(arr, shape=None):
    import torch

    if arr.dtype == np.uint16:  # bf16 bit patterns
        t = torch.from_numpy(arr.view(np.int16).copy()).view(torch.bfloat16)
    else:
        t = torch.from_numpy(arr.copy())
    t = t.to("cuda:0")
    if shape is not None:
        t = t.reshape(shape)
    return t


def to_host(t):
    import torch

    t = t.detach().reshape(-1).cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def dev_list(arrs, shapes):
    return [to_dev(a, s) for a, s in zip(arrs, shapes)]


def host_list(tensors):
    return [to_host(t) for t in tensors]


# ---- comparisons ---------------------------------------------------------------------------

def max_ulp_f32(a_list, b_list):
    worst = 0
    for a, b in zip(a_list, b_list):
        if a.size:
            worst = max(worst, int(O.ulp_distance_f32(a, b).max()))
    return worst


def narrow_list(arrs, half):
    """f32 arrays -> the oracle's representation of `half` ("bf16": uint16 bit patterns,
    "f16": np.float16), rounded as T::from_f32 does."""
    return [O.bf16_from_f32(a) if half == "bf16" else O.cast(np.ascontiguousarray(a, dtype=np.float32), np.float16)
            for a in arrs]


def widen_list(arrs):
    """bf16 patterns / float16 arrays -> f32 (exact)."""
    return [O.bf16_to_f32(a) if a.dtype == np.uint16 else O.cast(a, np.float32) for a in arrs]


def max_ulp_half(a_list, b_list):
    """Largest distance in units of the last place between 16-bit patterns (bf16 or f16)."""
    worst = 0
    for a, b in zip(a_list, b_list):
        if a.size:
            worst = max(worst, int(O.ulp_distance_bf16(a.view(np.uint16), b.view(np.uint16)).max()))
    return worst


def max_ulp_bf16(a_list, b_list):
    worst = 0
    for a, b in zip(a_list, b_list):
        if a.size:
            worst = max(worst, int(O.ulp_distance_bf16(a, b).max()))
    return worst


def assert_bits_equal(a_list, b_list, what):
    for i, (a, b) in enumerate(zip(a_list, b_list)):
        assert a.dtype == b.dtype, f"{what}: tensor {i}: {a.dtype} vs {b.dtype}"
        bits = {np.dtype(np.float16): np.uint16, np.dtype(np.float32): np.uint32, np.dtype(np.float64): np.uint64}
        av = a.view(bits[a.dtype]) if a.dtype in bits else a
        bv = b.view(bits[b.dtype]) if b.dtype in bits else b
        if not np.array_equal(av, bv):
            bad = np.nonzero(av != bv)[0]
            raise AssertionError(
                f"{what}: tensor {i} differs in {bad.size}/{a.size} elements, first at {bad[0]}: "
                f"{a[bad[0]]!r} vs {b[bad[0]]!r}")


def count_beyond_ulp_f32(a_list, b_list, tol):
    """(#elements beyond tol ulp, total) over a list."""
    n_bad = 0
    total = 0
    for a, b in zip(a_list, b_list):
        if a.size:
            n_bad += int((O.ulp_distance_f32(a, b) > tol).sum())
            total += a.size
    return n_bad, total


# ---- what the tests report beyond pass / fail ---------------------------------------------------

# Lines for pytest's terminal summary (tests/conftest.py prints them whether or not output is
# captured): every use of the tolerance clause below, every oracle step that had to follow the
# device's norm.
REPORT_LINES = []


def report(line):
    REPORT_LINES.append(line)
    print(line, flush=True)


# ---- the one legitimate difference between the device's norm and the reference's ---------------

NORM_FOLLOWED = {"steps": 0, "events": 0}


def oracle_step_with_device_norm(step_fn, state_lists, scalars, max_norm, dev_info, what):
    """Runs one oracle step, `step_fn() -> (ran, norm)`, next to a device step whose outcome is
    `dev_info` (nbo_step_info).  The reference adds the squares of the gradients serially, the
    device in a fixed tree: the two f64 norms agree to ~1e-13 relative but not always in the last
    bit, and T(max_norm / norm) -- the factor every gradient is multiplied by -- can then differ
    (about once in 10^4 clipped steps of a long list).  That difference is within the tolerance,
    but everything after it stops being bit-comparable, so: if the factor (or the decision to
    clip) differs, the oracle's state is put back and the step repeated with the device's norm in
    the place of the serial one, and the caller can go on demanding equal bits.  The norms
    themselves are always held to 1e-12 relative.  `state_lists` are the lists of arrays and
    `scalars` the ctypes structures (meta, scaler state) the step changes."""
    import copy

    if max_norm <= 0 or dev_info is None:
        return step_fn()
    snap_lists = [[a.copy() for a in lst] for lst in state_lists]
    snap_scalars = [copy.copy(x) if x is not None else None for x in scalars]
    ran, norm = step_fn()
    NORM_FOLLOWED["steps"] += 1
    if not ran or dev_info.found_inf:
        return ran, norm
    assert abs(dev_info.norm - norm) <= 1e-12 * norm, f"{what}: device norm {dev_info.norm!r} vs serial {norm!r}"

    def factor(n):  # None: not clipped (trainer.rs:515)
        return np.float32(max_norm / n).tobytes() if (n > max_norm and n > 0.0) else None

    if factor(dev_info.norm) != factor(norm):
        for lst, snap in zip(state_lists, snap_lists):
            for a, b in zip(lst, snap):
                a[...] = b
        for x, sx in zip(scalars, snap_scalars):
            if x is not None:
                C = type(x)
                import ctypes

                ctypes.memmove(ctypes.byref(x), ctypes.byref(sx), ctypes.sizeof(C))
        O.set_clip_norm_override(dev_info.norm)
        try:
            ran, _ = step_fn()
        finally:
            O.set_clip_norm_override(-1.0)
        NORM_FOLLOWED["events"] += 1
        report(f"[norm-follow] {what}: clip factor from the device's norm {dev_info.norm!r} differs from the serial "
               f"norm's {norm!r}; the oracle step was repeated with the device's norm")
    return ran, norm


# ---- the 2-ulp bar for parameters and its one documented escape ------------------------------

# No test may leave more than this many elements per 10^9 element-steps beyond 2 ulp (each of
# them inside the cancellation bound).  The mechanism: the reference's powf(x, 0.5) and the
# correctly rounded sqrt differ by 1 ulp for 0.06 % of inputs, which moves the update by 1 ulp;
# where p * (1 - wd * lr) and the update nearly cancel, that is more than 2 ulp of the tiny
# result.  Measured on this suite: 0.3 to 3 elements per 10^6 element-steps (the printed reports
# give each test's count), so the cap below leaves a factor of three.
ESCAPES_PER_1E9_ELEMENT_STEPS = 10000


def tolerance_report(dev_list, ref_list, lr, steps, what, element_steps=None):
    """f32 parameters against the libm-powf oracle: every element must be within 2 ulp or,
    failing that, within |delta| <= steps * 8 * lr * 2^-23 (a 1-ulp change of the update
    against a result that nearly cancelled).  Counts, prints and returns how often the second
    clause was needed: (n_beyond_2ulp, n_total, worst_ulp, worst_abs, first locations)."""
    n_total = n_beyond = worst_ulp = 0
    worst_abs = 0.0
    first = []
    bound = steps * 8 * lr * 2.0 ** -23
    for i, (a, b) in enumerate(zip(dev_list, ref_list)):
        if not a.size:
            continue
        ulp = O.ulp_distance_f32(a, b)
        absd = np.abs(a.astype(np.float64) - b.astype(np.float64))
        beyond = ulp > 2
        n_total += a.size
        worst_ulp = max(worst_ulp, int(ulp.max()))
        if beyond.any():
            idx = np.nonzero(beyond)[0]
            n_beyond += idx.size
            worst_abs = max(worst_abs, float(absd[idx].max()))
            for e in idx[:max(0, 5 - len(first))]:
                first.append((i, int(e), float(a[e]), float(b[e]), int(ulp[e])))
            outside = beyond & ~(absd <= bound)
            assert not outside.any(), (
                f"{what}: tensor {i}: {int(outside.sum())} params beyond 2 ulp and beyond the cancellation "
                f"bound {bound:.3e}; worst ulp {int(ulp.max())}, worst |d| {absd.max():.3e}")
            # the mechanism itself: a difference of a few ulps of the update can only be many
            # ulps of the parameter where the parameter is no larger than a few updates
            big = np.maximum(np.abs(a[idx]), np.abs(b[idx])).astype(np.float64)
            assert (big < 16.0 * lr * steps).all(), (
                f"{what}: tensor {i}: an element beyond 2 ulp has magnitude {big.max():.3e}, not below "
                f"16 * lr * steps = {16.0 * lr * steps:.3e}: this is not the near-cancellation the clause is for")
    es = element_steps if element_steps is not None else n_total * steps
    report(f"[tolerance] {what}: {n_beyond} of {n_total} elements ({es} element-steps) beyond 2 ulp of the "
           f"libm-powf oracle, all within |d| <= {bound:.3e} and of magnitude < 16 * lr * steps; worst {worst_ulp} ulp, "
           f"worst |d| {worst_abs:.3e}; first (tensor, index, device, oracle, ulp): {first}")
    ceiling = max(5, int(ESCAPES_PER_1E9_ELEMENT_STEPS * es / 1e9))
    assert n_beyond <= ceiling, f"{what}: {n_beyond} elements beyond 2 ulp, more than the ceiling of {ceiling}"
    return n_beyond, n_total, worst_ulp, worst_abs, first
