"""Learning-rate schedules of nabla-train (`optim/core.rs:81-252`): host-side f64
scalar math that feeds `Optimizer::set_lr`.  Every formula keeps the reference's
operation order, so the produced f64 values are the same bits."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

from .optim import OptimStateError, rust_f64_str


def powi(a: float, n: int) -> float:
    """f64::powi as compiler-rt's __powidf2 (used by the Step schedule, core.rs:170)."""
    recip = n < 0
    b = -n if recip else n
    r = 1.0
    while True:
        if b & 1:
            r *= a
        b >>= 1
        if b == 0:
            break
        a *= a
    return 1.0 / r if recip else r


@dataclass(frozen=True)
class Cosine:
    warmup_steps: int
    total_steps: int
    min_lr: float


@dataclass(frozen=True)
class Linear:
    warmup_steps: int
    total_steps: int


@dataclass(frozen=True)
class OneCycle:
    max_lr: float
    total_steps: int
    pct_start: float


@dataclass(frozen=True)
class Step:
    step_size: int
    gamma: float


LrSchedule = object  # any of the four classes above (enum LrSchedule, core.rs:101-121)


@dataclass
class ScheduleState:
    """core.rs:123-127."""

    base_lr: float
    schedule: object


_USIZE_MASK = (1 << 64) - 1


def _f64_as_usize(x: float) -> int:
    """Rust's `x as usize`: truncation toward zero, saturating at both ends, NaN -> 0."""
    if x != x or x <= 0.0:
        return 0
    if x >= 18446744073709551616.0:
        return _USIZE_MASK
    return int(x)


def _as_i32(k: int) -> int:
    """Rust's `k as i32` for a usize k: the low 32 bits, reinterpreted as signed."""
    k &= 0xFFFFFFFF
    return k - (1 << 32) if k & 0x80000000 else k


def _warmup_lr(base_lr, step, warmup_steps):  # core.rs:81-84
    return base_lr * float(step) / float(max(warmup_steps, 1))


def _decay_progress(step, start, total):  # core.rs:86-89
    # usize subtractions: where total < start (a schedule shorter than its warm-up) the
    # reference's release build wraps around instead of going negative, and so does this
    return float((step - start) & _USIZE_MASK) / float(max((total - start) & _USIZE_MASK, 1))


def _cosine_decay(high, low, progress):  # core.rs:96-99
    return low + 0.5 * (high - low) * (1.0 + math.cos(math.pi * progress))


def lr_at_step(schedule, base_lr: float, step: int) -> float:
    """core.rs:129-173."""
    if isinstance(schedule, Cosine):
        if step < schedule.warmup_steps:
            return _warmup_lr(base_lr, step, schedule.warmup_steps)
        return _cosine_decay(base_lr, schedule.min_lr,
                             _decay_progress(step, schedule.warmup_steps, schedule.total_steps))
    if isinstance(schedule, Linear):
        if step < schedule.warmup_steps:
            return _warmup_lr(base_lr, step, schedule.warmup_steps)
        progress = _decay_progress(step, schedule.warmup_steps, schedule.total_steps)
        return base_lr * max(1.0 - progress, 0.0)
    if isinstance(schedule, OneCycle):
        up_steps = _f64_as_usize(float(schedule.total_steps) * schedule.pct_start)
        if step < up_steps:
            return base_lr + (schedule.max_lr - base_lr) * float(step) / float(max(up_steps, 1))
        return _cosine_decay(schedule.max_lr, base_lr,
                             _decay_progress(step, up_steps, schedule.total_steps))
    if isinstance(schedule, Step):
        k = step // max(schedule.step_size, 1)
        return base_lr * powi(schedule.gamma, _as_i32(k))
    raise TypeError(f"not an LrSchedule: {schedule!r}")


def schedule_pairs(state: ScheduleState) -> List[Tuple[str, str]]:
    """core.rs:175-216."""
    s = state.schedule
    out = [("schedule.enabled", "1"), ("schedule.base_lr", rust_f64_str(state.base_lr))]
    if isinstance(s, Cosine):
        out += [("schedule.kind", "cosine"), ("schedule.warmup_steps", str(s.warmup_steps)),
                ("schedule.total_steps", str(s.total_steps)), ("schedule.min_lr", rust_f64_str(s.min_lr))]
    elif isinstance(s, Linear):
        out += [("schedule.kind", "linear"), ("schedule.warmup_steps", str(s.warmup_steps)),
                ("schedule.total_steps", str(s.total_steps))]
    elif isinstance(s, OneCycle):
        out += [("schedule.kind", "onecycle"), ("schedule.max_lr", rust_f64_str(s.max_lr)),
                ("schedule.total_steps", str(s.total_steps)), ("schedule.pct_start", rust_f64_str(s.pct_start))]
    elif isinstance(s, Step):
        out += [("schedule.kind", "step"), ("schedule.step_size", str(s.step_size)),
                ("schedule.gamma", rust_f64_str(s.gamma))]
    else:
        raise TypeError(f"not an LrSchedule: {s!r}")
    return out


def _get(m, key):
    if key not in m:
        raise OptimStateError(f"missing {key}")
    return m[key]


def _f64(m, key):
    v = _get(m, key)
    try:
        if v.strip() != v or not v:
            raise ValueError
        return float(v)
    except ValueError:
        raise OptimStateError(f"bad {key}: {v}") from None


def _usize(m, key):
    v = _get(m, key)
    body = v[1:] if v.startswith("+") else v
    if not body.isascii() or not body.isdigit():
        raise OptimStateError(f"bad {key}: {v}")
    return int(body)


def parse_schedule_state(m: Dict[str, str]) -> Optional[ScheduleState]:
    """core.rs:218-252."""
    if m.get("schedule.enabled", "0") != "1":
        return None
    base_lr = _f64(m, "schedule.base_lr")
    kind = _get(m, "schedule.kind")
    if kind == "cosine":
        s = Cosine(_usize(m, "schedule.warmup_steps"), _usize(m, "schedule.total_steps"),
                   _f64(m, "schedule.min_lr"))
    elif kind == "linear":
        s = Linear(_usize(m, "schedule.warmup_steps"), _usize(m, "schedule.total_steps"))
    elif kind == "onecycle":
        s = OneCycle(_f64(m, "schedule.max_lr"), _usize(m, "schedule.total_steps"),
                     _f64(m, "schedule.pct_start"))
    elif kind == "step":
        s = Step(_usize(m, "schedule.step_size"), _f64(m, "schedule.gamma"))
    else:
        raise OptimStateError(f"bad schedule.kind: {kind}")
    return ScheduleState(base_lr, s)
