"""ctypes bindings for the CPU oracle -- TEST INFRASTRUCTURE ONLY.

The oracle (``oracle/nabla_cpu_oracle.c``) restates the arithmetic of nabla's CPU
backend on the optimizer-step path.  Only tests, the smoke check and the
benchmark's ``cpu_baseline`` leg may import this module; the shipped package
``nabla_amd`` never does.

All tensors are numpy arrays (float32 / float64 / uint16-for-bf16), C-contiguous,
modified in place exactly where the reference modifies its tensors.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass, field

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnabla_oracle.so")

POW_LIBM = 0
POW_SQRT = 1

KIND_ADAMW, KIND_ADAM, KIND_SGD = 0, 1, 2


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


class Meta(C.Structure):
    """OptimMeta (optim/core.rs:53-62)."""

    _fields_ = [
        ("kind", C.c_int32),
        ("lr", C.c_double),
        ("beta1", C.c_double),
        ("beta2", C.c_double),
        ("eps", C.c_double),
        ("weight_decay", C.c_double),
        ("momentum", C.c_double),
        ("step_count", C.c_uint64),
    ]


class ScalerState(C.Structure):
    """GradScalerState (optim/core.rs:326-332)."""

    _fields_ = [
        ("scale", C.c_double),
        ("growth_factor", C.c_double),
        ("backoff_factor", C.c_double),
        ("growth_interval", C.c_uint64),
        ("consecutive_ok", C.c_uint64),
    ]


class Schedule(C.Structure):
    _fields_ = [
        ("kind", C.c_int32),
        ("warmup_steps", C.c_uint64),
        ("total_steps", C.c_uint64),
        ("a", C.c_double),
        ("b", C.c_double),
    ]


def adamw_meta(lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01, step_count=0):
    """AdamW::new defaults (alg.rs:29-38)."""
    return Meta(KIND_ADAMW, lr, beta1, beta2, eps, weight_decay, 0.0, step_count)


def adam_meta(lr, beta1=0.9, beta2=0.999, eps=1e-8, step_count=0):
    """Adam::new defaults (alg.rs:190-198)."""
    return Meta(KIND_ADAM, lr, beta1, beta2, eps, 0.0, 0.0, step_count)


def sgd_meta(lr, momentum=0.0, weight_decay=0.0):
    """Sgd::new defaults (alg.rs:324-329)."""
    return Meta(KIND_SGD, lr, 0.0, 0.0, 0.0, weight_decay, momentum, 0)


def default_scaler():
    s = ScalerState()
    lib().orc_scaler_default(C.byref(s))
    return s


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


def _declare(L):
    L.orc_powi.restype = C.c_double
    L.orc_powi.argtypes = [C.c_double, C.c_int]
    L.orc_bf16_from_f32.restype = C.c_uint16
    L.orc_bf16_from_f32.argtypes = [C.c_float]
    L.orc_bf16_from_f64.restype = C.c_uint16
    L.orc_bf16_from_f64.argtypes = [C.c_double]
    L.orc_f16_from_f64.restype = C.c_uint16
    L.orc_f16_from_f64.argtypes = [C.c_double]
    L.orc_bf16_to_f32.restype = C.c_float
    L.orc_bf16_to_f32.argtypes = [C.c_uint16]
    L.orc_lr_at_step.restype = C.c_double
    L.orc_lr_at_step.argtypes = [C.POINTER(Schedule), C.c_double, C.c_uint64]
    L.orc_get_pow_mode.restype = C.c_int
    L.orc_get_threads.restype = C.c_int
    for suf in ("f32", "f64", "bf16", "f16"):
        getattr(L, f"orc_clip_grad_norm_{suf}").restype = C.c_double
        getattr(L, f"orc_clip_grad_norm_{suf}").argtypes = [
            C.c_size_t, C.c_void_p, C.c_void_p, C.c_double]
        getattr(L, f"orc_scaler_unscale_and_update_{suf}").restype = C.c_int


def set_pow_mode(mode: int) -> None:
    lib().orc_set_pow_mode(int(mode))


def set_clip_norm_override(norm: float) -> None:
    """Test hook: norm >= 0 makes clip_grad_norm decide and scale with `norm` (its return value
    stays the square root of its own serial sum); negative switches it off."""
    L = lib()
    L.orc_set_clip_norm_override.argtypes = [C.c_double]
    L.orc_set_clip_norm_override(float(norm))


def set_threads(n: int) -> None:
    lib().orc_set_threads(int(n))


def powi(a: float, n: int) -> float:
    return lib().orc_powi(a, n)


def _suffix(arr: np.ndarray) -> str:
    if arr.dtype == np.float32:
        return "f32"
    if arr.dtype == np.float64:
        return "f64"
    if arr.dtype == np.uint16:  # bf16 bit patterns
        return "bf16"
    if arr.dtype == np.float16:
        return "f16"
    raise TypeError(f"oracle: unsupported dtype {arr.dtype}")


def _ptrs(arrs):
    for a in arrs:
        if not (isinstance(a, np.ndarray) and a.flags.c_contiguous):
            raise TypeError("oracle: tensors must be C-contiguous numpy arrays")
    return (C.c_void_p * max(len(arrs), 1))(*[a.ctypes.data for a in arrs])


def _sizes(arrs):
    return (C.c_uint64 * max(len(arrs), 1))(*[a.size for a in arrs])


def _ctype(arr):
    """Constructor of the C scalar that goes with `arr`'s element type; for bf16 (uint16
    patterns) the Python float is narrowed with bf16::from_f64 first."""
    if arr.dtype == np.uint16:
        return lambda s: C.c_uint16(lib().orc_bf16_from_f64(C.c_double(s)))
    if arr.dtype == np.float16:
        return lambda s: C.c_uint16(lib().orc_f16_from_f64(C.c_double(s)))
    return C.c_float if arr.dtype == np.float32 else C.c_double


# ---- casts / generators ------------------------------------------------------

def bf16_from_f32(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_cast_f32_to_bf16(C.c_void_p(x.ctypes.data), C.c_void_p(out.ctypes.data),
                               C.c_size_t(x.size))
    return out


def bf16_to_f32(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().orc_cast_bf16_to_f32(C.c_void_p(h.ctypes.data), C.c_void_p(out.ctypes.data),
                               C.c_size_t(h.size))
    return out


def randn_f64(n: int, seed: int) -> np.ndarray:
    out = np.empty(n, dtype=np.float64)
    lib().orc_randn_f64(C.c_void_p(out.ctypes.data), C.c_size_t(n), C.c_uint64(seed))
    return out


def randn_f32(n: int, seed: int, sigma: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    lib().orc_randn_scaled_f32(C.c_void_p(out.ctypes.data), C.c_size_t(n), C.c_uint64(seed),
                               C.c_double(sigma))
    return out


def bench_rand_f32(n: int, state: int = 42):
    """benchmarks/src/lib.rs:7-22; returns (values, next state)."""
    out = np.empty(n, dtype=np.float32)
    st = C.c_uint64(state)
    lib().orc_bench_rand_f32(C.c_void_p(out.ctypes.data), C.c_size_t(n), C.byref(st))
    return out, st.value


def lr_at_step(sched: Schedule, base_lr: float, step: int) -> float:
    return lib().orc_lr_at_step(C.byref(sched), base_lr, step)


# ---- primitives ----------------------------------------------------------------

def scale(a, s):
    out = np.empty_like(a)
    getattr(lib(), f"orc_scale_{_suffix(a)}")(C.c_void_p(a.ctypes.data), _ctype(a)(s),
                                              C.c_void_p(out.ctypes.data), C.c_size_t(a.size))
    return out


def axpy_inplace(y, alpha, x):
    getattr(lib(), f"orc_axpy_inplace_{_suffix(y)}")(C.c_void_p(y.ctypes.data), _ctype(y)(alpha),
                                                     C.c_void_p(x.ctypes.data), C.c_size_t(y.size))


def powf(a, p):
    out = np.empty_like(a)
    getattr(lib(), f"orc_powf_{_suffix(a)}")(C.c_void_p(a.ctypes.data), _ctype(a)(p),
                                             C.c_void_p(out.ctypes.data), C.c_size_t(a.size))
    return out


def map_add(a, c):
    """Tensor::map(|x| x + c)."""
    out = np.empty_like(a)
    getattr(lib(), f"orc_map_add_{_suffix(a)}")(C.c_void_p(a.ctypes.data), _ctype(a)(c),
                                                C.c_void_p(out.ctypes.data), C.c_size_t(a.size))
    return out


_CAST_TYPE = {np.dtype(np.float32): 0, np.dtype(np.uint16): 1, np.dtype(np.float64): 2, np.dtype(np.float16): 3}


def cast(src: np.ndarray, dst_dtype) -> np.ndarray:
    """B::cast default (backend/mod.rs:157-160); np.uint16 stands for bf16 patterns,
    np.float16 is f16."""
    src = np.ascontiguousarray(src)
    out = np.empty(src.shape, dtype=dst_dtype)
    lib().orc_cast(C.c_void_p(src.ctypes.data), C.c_int(_CAST_TYPE[src.dtype]),
                   C.c_void_p(out.ctypes.data), C.c_int(_CAST_TYPE[out.dtype]), C.c_size_t(src.size))
    return out


def _binary(name, a, b):
    out = np.empty_like(a)
    getattr(lib(), f"orc_{name}_{_suffix(a)}")(C.c_void_p(a.ctypes.data), C.c_void_p(b.ctypes.data),
                                               C.c_void_p(out.ctypes.data), C.c_size_t(a.size))
    return out


def emul(a, b):
    return _binary("emul", a, b)


def ediv(a, b):
    return _binary("ediv", a, b)


def add(a, b):
    return _binary("add", a, b)


# ---- optimizers ------------------------------------------------------------------

def sgd_step(meta: Meta, params, grads, velocity):
    """Sgd::step (alg.rs:382-416)."""
    suf = _suffix(params[0]) if params else "f32"
    getattr(lib(), f"orc_sgd_step_{suf}")(C.byref(meta), C.c_size_t(len(params)), _sizes(params),
                                          _ptrs(params), _ptrs(grads), _ptrs(velocity))


def adam_step(meta: Meta, params, grads, m, v):
    """Adam::step / AdamW::step (alg.rs:254-291 / 109-150); meta.kind selects."""
    suf = _suffix(params[0]) if params else "f32"
    getattr(lib(), f"orc_adam_step_{suf}")(C.byref(meta), C.c_size_t(len(params)), _sizes(params),
                                           _ptrs(params), _ptrs(grads), _ptrs(m), _ptrs(v))


def adamw_step_single(param, grad, m, v, lr, beta1, beta2, eps, weight_decay, step):
    """adamw_step free function (alg.rs:431-469)."""
    suf = _suffix(param)
    getattr(lib(), f"orc_adamw_step_single_{suf}")(
        C.c_void_p(param.ctypes.data), C.c_void_p(grad.ctypes.data), C.c_void_p(m.ctypes.data),
        C.c_void_p(v.ctypes.data), C.c_size_t(param.size), C.c_double(lr), C.c_double(beta1),
        C.c_double(beta2), C.c_double(eps), C.c_double(weight_decay), C.c_uint64(step))


def scaler_unscale_and_update(state: ScalerState, grads) -> bool:
    """GradScaler::unscale_and_update (core.rs:351-388)."""
    suf = _suffix(grads[0]) if grads else "f32"
    ok = getattr(lib(), f"orc_scaler_unscale_and_update_{suf}")(
        C.byref(state), C.c_size_t(len(grads)), _sizes(grads), _ptrs(grads))
    return bool(ok)


def clip_grad_norm(grads, max_norm: float) -> float:
    """clip_grad_norm (trainer.rs:500-523)."""
    suf = _suffix(grads[0]) if grads else "f32"
    return getattr(lib(), f"orc_clip_grad_norm_{suf}")(
        C.c_size_t(len(grads)), _sizes(grads), _ptrs(grads), C.c_double(max_norm))


def zero_grad(grads):
    suf = _suffix(grads[0]) if grads else "f32"
    getattr(lib(), f"orc_zero_grad_{suf}")(C.c_size_t(len(grads)), _sizes(grads), _ptrs(grads))


def scale_grad(grads, factor):
    suf = _suffix(grads[0]) if grads else "f32"
    getattr(lib(), f"orc_scale_grad_{suf}")(C.c_size_t(len(grads)), _sizes(grads), _ptrs(grads),
                                            _ctype(grads[0])(factor))


def f32_step(meta, scaler, max_norm, params, grads, m, v):
    """Trainer tail for T=f32 (trainer.rs:230-283). Returns (ran, norm)."""
    norm = C.c_double(0.0)
    L = lib()
    L.orc_f32_step.restype = C.c_int
    ran = L.orc_f32_step(C.byref(meta), C.byref(scaler) if scaler is not None else None,
                         C.c_double(max_norm), C.c_size_t(len(params)), _sizes(params),
                         _ptrs(params), _ptrs(grads), _ptrs(m), _ptrs(v), C.byref(norm))
    return bool(ran), norm.value


def mixed_step(meta, scaler, max_norm, params_half, grads_half, master, m, v):
    """Trainer tail for bf16 (np.uint16 patterns) or f16 (np.float16) params/grads with f32
    master/m/v. Returns (ran, norm)."""
    kinds = {a.dtype for a in list(params_half) + list(grads_half)}
    if kinds - {np.dtype(np.uint16)} and kinds - {np.dtype(np.float16)}:
        raise TypeError("oracle.mixed_step: tensors are bf16 bit patterns (uint16) or float16, not a mix")
    half_type = 3 if np.dtype(np.float16) in kinds else 1
    norm = C.c_double(0.0)
    L = lib()
    L.orc_mixed_step_half.restype = C.c_int
    ran = L.orc_mixed_step_half(C.byref(meta), C.byref(scaler) if scaler is not None else None,
                                C.c_double(max_norm), C.c_size_t(len(master)), _sizes(master),
                                _ptrs(params_half), _ptrs(grads_half), C.c_int(half_type), _ptrs(master),
                                _ptrs(m), _ptrs(v), C.byref(norm))
    return bool(ran), norm.value


# ---- ulp helpers used by the parity tests ------------------------------------------

def f32_ordered(a: np.ndarray) -> np.ndarray:
    """Map f32 bit patterns to a monotone int64 line (sign-magnitude -> signed)."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.int64)
    return np.where(u & 0x80000000, -(u & 0x7FFFFFFF), u)


def bf16_ordered(h: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(h, dtype=np.uint16).astype(np.int64)
    return np.where(u & 0x8000, -(u & 0x7FFF), u)


def ulp_distance_f32(a, b) -> np.ndarray:
    return np.abs(f32_ordered(a) - f32_ordered(b))


def ulp_distance_bf16(a, b) -> np.ndarray:
    return np.abs(bf16_ordered(a) - bf16_ordered(b))
