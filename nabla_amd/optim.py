"""Host-side mirror of nabla-train's optimizer interface over the C ABI.

Names, argument meaning and error behaviour follow
``nabla-train/src/optim/{core,alg}.rs`` and ``nabla-train/src/trainer.rs`` of the
reference, so that a test written against the reference reads the same here:

    opt = AdamW.new(2e-4, shapes).beta2(0.95).weight_decay(0.1)
    opt.step(params, grads)

Tensors are anything that exposes ``data_ptr()``, ``shape`` and ``dtype`` for
memory resident on GPU 0 (torch tensors in the tests).  All arithmetic happens in
the gfx950 kernels of libnabla_optim.so; this module only marshals pointers.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

from . import _lib
from ._lib import (DT_BF16, DT_F16, DT_F32, DT_F64, KIND_ADAM, KIND_ADAMW, KIND_SGD, STEP_SKIP_NONFINITE,
                   STEP_ZERO_GRADS, STEP_ZERO_ON_SKIP, NablaOptimError)


class NablaPanic(AssertionError):
    """Where the reference panics (assert_eq! in alg.rs:110-119, shape asserts)."""


class OptimStateError(ValueError):
    """Where the reference returns Err(String) (optim/core.rs:67-69)."""


_PANIC = {_lib.ERR_LEN_MISMATCH, _lib.ERR_COUNT_MISMATCH, _lib.ERR_SHAPE}
_STATE = {_lib.ERR_STATE_KEY, _lib.ERR_STATE_INDEX, _lib.ERR_KIND}


def _call(status: int) -> None:
    try:
        _lib.check(status)
    except NablaOptimError as e:
        if e.status in _PANIC:
            raise NablaPanic(e.message) from None
        if e.status in _STATE:
            raise OptimStateError(e.message) from None
        raise


def _dtype_code(t) -> int:
    name = str(t.dtype)
    if name.endswith("float32"):
        return DT_F32
    if name.endswith("bfloat16"):
        return DT_BF16
    if name.endswith("float64"):
        return DT_F64
    if name.endswith("float16"):  # after bfloat16, which ends the same way
        return DT_F16
    raise TypeError(f"unsupported tensor dtype {name}")


def _shape2(t) -> Tuple[int, int]:
    """(rows, cols) of a tensor; the reference's tensors are always 2-D."""
    s = tuple(int(x) for x in t.shape)
    if len(s) == 2:
        return s
    if len(s) == 1:
        return (1, s[0])
    if len(s) == 0:
        return (1, 1)
    rows = 1
    for x in s[:-1]:
        rows *= x
    return (rows, s[-1])


def _u64_array(values):
    return (C.c_uint64 * max(len(values), 1))(*values)


class TensorList:
    """A ``&[&Tensor<T, B>]`` argument: same-dtype device tensors, described once."""

    def __init__(self, tensors: Sequence, dtype: Optional[int] = None):
        self.tensors = list(tensors)
        for t in self.tensors:
            if hasattr(t, "is_contiguous") and not t.is_contiguous():
                raise ValueError("tensors must be contiguous (row-major, as in the reference)")
        self.shapes = [_shape2(t) for t in self.tensors]
        if dtype is None:
            dtype = _dtype_code(self.tensors[0]) if self.tensors else DT_F32
        for t in self.tensors:
            if _dtype_code(t) != dtype:
                raise TypeError("all tensors of a list share one dtype")
        self.dtype = dtype
        n = len(self.tensors)
        rows = _u64_array([s[0] for s in self.shapes])
        cols = _u64_array([s[1] for s in self.shapes])
        self.ptrs = [t.data_ptr() for t in self.tensors]  # as described to the device
        ptrs = (C.c_void_p * max(n, 1))(*self.ptrs)
        self._h = C.c_void_p()
        _call(_lib.load().nbo_list_create(n, rows, cols, dtype, ptrs, C.byref(self._h)))

    def key(self):
        return tuple((t.data_ptr(), s) for t, s in zip(self.tensors, self.shapes))

    def rebind(self, tensors: Sequence) -> None:
        """Point the list at other tensors of the same shapes and dtype: only the address
        table is uploaded again (nbo_list_set_ptrs), the descriptor stays."""
        tensors = list(tensors)
        if [_shape2(t) for t in tensors] != self.shapes or any(_dtype_code(t) != self.dtype for t in tensors):
            raise ValueError("rebind needs tensors of the list's shapes and dtype")
        for t in tensors:
            if hasattr(t, "is_contiguous") and not t.is_contiguous():
                raise ValueError("tensors must be contiguous (row-major, as in the reference)")
        new_ptrs = [t.data_ptr() for t in tensors]
        ptrs = (C.c_void_p * max(len(tensors), 1))(*new_ptrs)
        _call(_lib.load().nbo_list_set_ptrs(self._h, ptrs))
        self.tensors, self.ptrs = tensors, new_ptrs

    def __len__(self):
        return len(self.tensors)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                _lib.load().nbo_list_destroy(h)
            except Exception:
                pass


class _ListCache:
    """Reuse the device descriptor while the caller passes the same tensors."""

    def __init__(self):
        self._last: Dict[str, TensorList] = {}

    def get(self, slot: str, tensors) -> TensorList:
        if isinstance(tensors, TensorList):
            return tensors
        tensors = list(tensors)
        cur = self._last.get(slot)
        # compared with what the list was built from, not with its tensor objects as they are
        # now: the same object may have been resized or given other storage since
        if cur is not None and len(cur) == len(tensors) and all(
                s == _shape2(b) and _dtype_code(b) == cur.dtype for s, b in zip(cur.shapes, tensors)):
            if all(p == b.data_ptr() for p, b in zip(cur.ptrs, tensors)):
                return cur
            cur.rebind(tensors)  # same layout, new addresses (fresh gradient tensors every step)
            return cur
        cur = TensorList(tensors)
        self._last[slot] = cur
        return cur


_free_cache = _ListCache()


@dataclass
class OptimMeta:
    """optim/core.rs:53-62; kind is 'adamw' | 'adam' | 'sgd' (core.rs:293-299)."""

    kind: str
    lr: float
    beta1: float
    beta2: float
    eps: float
    weight_decay: float
    momentum: float
    step_count: int


_KIND_STR = {KIND_ADAMW: "adamw", KIND_ADAM: "adam", KIND_SGD: "sgd"}
_KIND_CODE = {v: k for k, v in _KIND_STR.items()}


def rust_f64_str(x: float) -> str:
    """Rust's `f64::to_string()` (Display): shortest round-trip digits, never
    scientific notation, integers printed without a fraction."""
    if x != x:
        return "NaN"
    if x in (float("inf"), float("-inf")):
        return "inf" if x > 0 else "-inf"
    r = repr(float(x))
    if "e" not in r and "E" not in r:
        return r[:-2] if r.endswith(".0") else r
    mant, exp = r.lower().split("e")
    exp = int(exp)
    sign = ""
    if mant.startswith("-"):
        sign, mant = "-", mant[1:]
    if "." in mant:
        ip, fp = mant.split(".")
    else:
        ip, fp = mant, ""
    digits = ip + fp
    point = len(ip) + exp
    if point <= 0:
        s = "0." + "0" * (-point) + digits
    elif point >= len(digits):
        s = digits + "0" * (point - len(digits))
    else:
        s = digits[:point] + "." + digits[point:]
    if "." in s:
        s = s.rstrip("0").rstrip(".")
    return sign + s


def optim_meta_pairs(meta: OptimMeta) -> List[Tuple[str, str]]:
    """optim/core.rs:263-277."""
    return [
        ("optim.kind", meta.kind),
        ("optim.lr", rust_f64_str(meta.lr)),
        ("optim.beta1", rust_f64_str(meta.beta1)),
        ("optim.beta2", rust_f64_str(meta.beta2)),
        ("optim.eps", rust_f64_str(meta.eps)),
        ("optim.weight_decay", rust_f64_str(meta.weight_decay)),
        ("optim.momentum", rust_f64_str(meta.momentum)),
        ("optim.step_count", str(int(meta.step_count))),
    ]


def _parse_str(m: Dict[str, str], key: str) -> str:
    if key not in m:
        raise OptimStateError(f"missing {key}")
    return m[key]


def _parse_f64(m, key) -> float:
    v = _parse_str(m, key)
    try:
        if v.strip() != v or v == "":
            raise ValueError
        return float(v)
    except ValueError:
        raise OptimStateError(f"bad {key}: {v}") from None


def _parse_usize(m, key) -> int:
    v = _parse_str(m, key)
    body = v[1:] if v.startswith("+") else v
    if not body.isascii() or not body.isdigit():
        raise OptimStateError(f"bad {key}: {v}")
    return int(body)


def parse_optim_meta(m: Dict[str, str]) -> OptimMeta:
    """optim/core.rs:279-308."""
    kind = _parse_str(m, "optim.kind")
    if kind not in _KIND_CODE:
        raise OptimStateError(f"bad optim.kind: {kind}")
    return OptimMeta(kind, _parse_f64(m, "optim.lr"), _parse_f64(m, "optim.beta1"),
                     _parse_f64(m, "optim.beta2"), _parse_f64(m, "optim.eps"),
                     _parse_f64(m, "optim.weight_decay"), _parse_f64(m, "optim.momentum"),
                     _parse_usize(m, "optim.step_count"))


class _Optimizer:
    """Common part of Sgd / Adam / AdamW: trait Optimizer + trait OptimState."""

    KIND = KIND_ADAMW
    NAME = "AdamW"

    def __init__(self, lr: float, param_shapes: Sequence[Tuple[int, int]], *, dtype: str = "f32",
                 master: bool = False):
        self._shapes = [(int(r), int(c)) for r, c in param_shapes]
        # "bf16" / "f16" are the reference's Optimizer<bf16> / Optimizer<f16>: tensors, state and
        # arithmetic all of that type
        self._state_dtype = {"f32": DT_F32, "f64": DT_F64, "bf16": DT_BF16, "f16": DT_F16}[dtype]
        if master and dtype != "f32":
            raise ValueError("master weights are f32: master=True goes with dtype='f32'")
        self._master = bool(master)
        self._meta = _lib.Meta(self.KIND, 0, float(lr), 0.0, 0.0, 0.0, 0.0, 0.0, 0)
        self._h = None
        self._cache = _ListCache()

    # -- construction ---------------------------------------------------------------
    @classmethod
    def new(cls, lr, param_shapes, **kw):
        return cls(lr, param_shapes, **kw)

    @classmethod
    def from_params(cls, lr, params, **kw):
        return cls(lr, [_shape2(p) for p in params], **kw)

    def _set(self, field, value):
        if self._h is not None:
            raise RuntimeError("builder setters apply before the first use; use set_state after")
        setattr(self._meta, field, float(value))
        return self

    def _handle(self):
        if self._h is None:
            n = len(self._shapes)
            h = C.c_void_p()
            _call(_lib.load().nbo_optim_create(
                C.byref(self._meta), n, _u64_array([s[0] for s in self._shapes]),
                _u64_array([s[1] for s in self._shapes]), self._state_dtype, int(self._master),
                C.byref(h)))
            self._h = h
        return self._h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                _lib.load().nbo_optim_destroy(h)
            except Exception:
                pass

    # -- trait Optimizer (optim/core.rs:9-44) ------------------------------------------
    def step(self, params, grads) -> None:
        p = self._cache.get("p", params)
        g = self._cache.get("g", grads)
        _call(_lib.load().nbo_optim_step(self._handle(), p._h, g._h))

    step_slices = step

    def step_with_vars(self, module, param_vars) -> None:
        """optim/core.rs:18-39: parameters from `module.parameters_mut()`, gradients from
        each variable's `grad()` (None, or an exception, means "no gradient")."""
        params = list(module.parameters_mut())
        if len(params) != len(param_vars):
            raise NablaPanic(f"nabla-train: step_with_vars param_vars length ({len(param_vars)}) doesn't "
                             f"match module parameters count ({len(params)})")
        grads = []
        for i, v in enumerate(param_vars):
            try:
                g = v.grad()
            except Exception:
                g = None
            if g is None:
                raise NablaPanic(f"nabla-train: step_with_vars: param_vars[{i}] has no gradient "
                                 "(call backward first)")
            grads.append(g)
        self.step(params, grads)

    def reset(self) -> None:
        _call(_lib.load().nbo_optim_reset(self._handle()))

    def set_lr(self, lr: float) -> None:
        self._meta.lr = float(lr)
        if self._h is not None:
            _call(_lib.load().nbo_optim_set_lr(self._h, float(lr)))

    # -- accessors ---------------------------------------------------------------------
    def lr(self) -> float:
        return self._meta.lr

    def step_count(self) -> int:
        return self.meta().step_count

    # -- the fused Trainer tail (trainer.rs:230-291) --------------------------------------
    def fused_step(self, params, grads, scaler: Optional["GradScaler"] = None,
                   max_norm: float = 0.0, zero_grads: bool = False,
                   skip_nonfinite: bool = False, no_alloc: bool = False, zero_on_skip: bool = False) -> None:
        """`zero_on_skip=True`: a skipped step leaves zeros in the gradients, as the reference's
        `unscale_and_update` does when it finds inf / NaN (optim/core.rs:372-375).
        `no_alloc=True` goes through nbo_fused_step_noalloc: same results, the norm pass's
        scratch comes from the library's statically allocated device array (pass TensorLists,
        or the same tensors as in an earlier call, so that no descriptor is built either)."""
        p = self._cache.get("p", params)
        g = self._cache.get("g", grads)
        flags = ((STEP_ZERO_GRADS if zero_grads else 0) | (STEP_SKIP_NONFINITE if skip_nonfinite else 0)
                 | (STEP_ZERO_ON_SKIP if zero_on_skip else 0))
        lib = _lib.load()
        fn = lib.nbo_fused_step_noalloc if no_alloc else lib.nbo_fused_step
        _call(fn(self._handle(), scaler._handle() if scaler else None, p._h, g._h, float(max_norm), flags))

    def fused_step_norm(self, params, grads, sumsq: float, max_norm: float = 0.0,
                        zero_grads: bool = False) -> None:
        """clip_grad_norm + step (+ zeroing) over gradients whose sum of squares is already
        known (from `unscale_accumulate`), without another norm pass (trainer.rs:274-290)."""
        p = self._cache.get("p", params)
        g = self._cache.get("g", grads)
        _call(_lib.load().nbo_fused_step_norm(self._handle(), p._h, g._h, float(max_norm), float(sumsq),
                                              STEP_ZERO_GRADS if zero_grads else 0))

    def last_step(self) -> _lib.StepInfo:
        info = _lib.StepInfo()
        _call(_lib.load().nbo_optim_last_step(self._handle(), C.byref(info)))
        return info

    def trace(self, max_entries: int = 1024) -> List[_lib.StepInfo]:
        buf = (_lib.StepInfo * max(max_entries, 1))()
        n = C.c_uint64(0)
        total = C.c_uint64(0)
        _call(_lib.load().nbo_optim_trace_read(self._handle(), buf, max_entries, C.byref(n),
                                               C.byref(total)))
        return [buf[i] for i in range(n.value)]

    def state_regions(self) -> int:
        """0: state arrays are plain allocations; n: spread over n HBM regions."""
        n = C.c_int(0)
        _call(_lib.load().nbo_optim_state_regions(self._handle(), C.byref(n)))
        return n.value

    def state_placement_note(self) -> str:
        """What the placement of the state arrays found, or why it fell back to plain allocations."""
        buf = C.create_string_buffer(512)
        _call(_lib.load().nbo_optim_state_placement_note(self._handle(), buf, 512))
        return buf.value.decode("utf-8", "replace")

    # -- master weights (mixed precision) -----------------------------------------------
    def master_from_params(self, params) -> None:
        p = self._cache.get("p", params)
        _call(_lib.load().nbo_optim_master_from_params(self._handle(), p._h))

    def params_from_master(self, params) -> None:
        p = self._cache.get("p", params)
        _call(_lib.load().nbo_optim_params_from_master(self._handle(), p._h))

    # -- trait OptimState (optim/core.rs:64-79) --------------------------------------------
    def kind(self) -> str:
        return _KIND_STR[self.KIND]

    def _state_names(self) -> List[str]:
        n = len(self._shapes)
        if self.KIND == KIND_SGD:
            return [f"v{i}" for i in range(n)]
        return [f"m{i}" for i in range(n)] + [f"v{i}" for i in range(n)]

    def _torch_dtype(self):
        import torch
        return {DT_F64: torch.float64, DT_BF16: torch.bfloat16,
                DT_F16: torch.float16}.get(self._state_dtype, torch.float32)

    def read_state(self, name: str):
        """One state tensor as a new device tensor (a clone, like state_tensors())."""
        import torch
        idx = int(name[1:]) if name[1:].isdigit() and int(name[1:]) < len(self._shapes) else 0
        r, c = self._shapes[idx] if self._shapes else (0, 0)
        dt = torch.float32 if name.startswith("w") else self._torch_dtype()
        out = torch.empty((r, c), dtype=dt, device="cuda:0")
        _call(_lib.load().nbo_optim_state_read(self._handle(), name.encode(), out.data_ptr(),
                                               out.numel(), 1))
        return out

    def write_state(self, name: str, tensor) -> None:
        import torch
        dt = torch.float32 if name.startswith("w") else self._torch_dtype()
        t = tensor.to(device="cuda:0", dtype=dt).contiguous()
        _call(_lib.load().nbo_optim_state_write(self._handle(), name.encode(), t.data_ptr(),
                                                t.numel(), 1))
        _call(_lib.load().nbo_sync())

    def state_tensors(self) -> List[Tuple[str, object]]:
        return [(n, self.read_state(n)) for n in self._state_names()]

    def load_state_tensors(self, tensors: Sequence[Tuple[str, object]]) -> None:
        """alg.rs:487-516 / 564-593 / 631-648: unknown prefixes are ignored, every
        expected tensor must be present, nothing is changed unless all are."""
        n = len(self._shapes)
        prefixes = ("v",) if self.KIND == KIND_SGD else ("m", "v")
        found: Dict[str, object] = {}
        for name, t in tensors:
            pref = name[:1]
            if pref not in prefixes:
                continue
            body = name[1:]
            digits = body[1:] if body.startswith("+") else body
            if not digits.isascii() or not digits.isdigit():
                raise OptimStateError(f"bad tensor key: {name}")
            i = int(digits)
            if i >= n:
                raise OptimStateError(f"{pref} index out of range: {i}")
            found[f"{pref}{i}"] = t
        for pref in prefixes:
            for i in range(n):
                if f"{pref}{i}" not in found:
                    raise OptimStateError(f"missing {pref}{i}")
        for key, t in found.items():
            self.write_state(key, t)

    def meta(self) -> OptimMeta:
        if self._h is None:
            m = self._meta
            sgd = self.KIND == KIND_SGD
            return OptimMeta(self.kind(), m.lr, 0.0 if sgd else m.beta1, 0.0 if sgd else m.beta2,
                             0.0 if sgd else m.eps,
                             0.0 if self.KIND == KIND_ADAM else m.weight_decay,
                             m.momentum if sgd else 0.0, 0 if sgd else m.step_count)
        out = _lib.Meta()
        _call(_lib.load().nbo_optim_get_meta(self._h, C.byref(out)))
        return OptimMeta(_KIND_STR[out.kind], out.lr, out.beta1, out.beta2, out.eps,
                         out.weight_decay, out.momentum, out.step_count)

    def load_meta(self, meta: OptimMeta) -> None:
        if meta.kind != self.kind():
            raise OptimStateError("optim kind mismatch")
        m = _lib.Meta(_KIND_CODE[meta.kind], 0, meta.lr, meta.beta1, meta.beta2, meta.eps,
                      meta.weight_decay, meta.momentum, int(meta.step_count))
        if self._h is not None:  # otherwise the engine is created from the updated meta
            _call(_lib.load().nbo_optim_load_meta(self._h, C.byref(m)))
        self._meta.lr = meta.lr
        if self.KIND == KIND_SGD:
            self._meta.momentum, self._meta.weight_decay = meta.momentum, meta.weight_decay
        else:
            self._meta.beta1, self._meta.beta2, self._meta.eps = meta.beta1, meta.beta2, meta.eps
            if self.KIND == KIND_ADAMW:
                self._meta.weight_decay = meta.weight_decay
            self._meta.step_count = int(meta.step_count)

    def meta_pairs(self) -> List[Tuple[str, str]]:
        return optim_meta_pairs(self.meta())

    def load_meta_pairs(self, m: Dict[str, str]) -> None:
        self.load_meta(parse_optim_meta(m))


class AdamW(_Optimizer):
    """alg.rs:7-167; defaults beta1 0.9, beta2 0.999, eps 1e-8, weight_decay 0.01."""

    KIND, NAME = KIND_ADAMW, "AdamW"

    def __init__(self, lr, param_shapes, **kw):
        super().__init__(lr, param_shapes, **kw)
        self._meta.beta1, self._meta.beta2, self._meta.eps = 0.9, 0.999, 1e-8
        self._meta.weight_decay = 0.01

    def beta1(self, x):
        return self._set("beta1", x)

    def beta2(self, x):
        return self._set("beta2", x)

    def eps(self, x):
        return self._set("eps", x)

    def weight_decay(self, x):
        return self._set("weight_decay", x)

    def moments(self):
        n = len(self._shapes)
        return ([self.read_state(f"m{i}") for i in range(n)],
                [self.read_state(f"v{i}") for i in range(n)])

    def set_state(self, step_count, beta1, beta2, eps, weight_decay, lr):
        self.load_meta(OptimMeta(self.kind(), lr, beta1, beta2, eps, weight_decay, 0.0, step_count))


class Adam(_Optimizer):
    """alg.rs:169-308; defaults beta1 0.9, beta2 0.999, eps 1e-8."""

    KIND, NAME = KIND_ADAM, "Adam"

    def __init__(self, lr, param_shapes, **kw):
        super().__init__(lr, param_shapes, **kw)
        self._meta.beta1, self._meta.beta2, self._meta.eps = 0.9, 0.999, 1e-8

    beta1 = AdamW.beta1
    beta2 = AdamW.beta2
    eps = AdamW.eps
    moments = AdamW.moments

    def set_state(self, step_count, beta1, beta2, eps, lr):
        self.load_meta(OptimMeta(self.kind(), lr, beta1, beta2, eps, 0.0, 0.0, step_count))


class Sgd(_Optimizer):
    """alg.rs:310-428; defaults momentum 0, weight_decay 0."""

    KIND, NAME = KIND_SGD, "SGD"

    def momentum(self, x):
        return self._set("momentum", x)

    def weight_decay(self, x):
        return self._set("weight_decay", x)

    def momentum_value(self):
        return self._meta.momentum

    def weight_decay_value(self):
        return self._meta.weight_decay

    def velocity(self):
        return [self.read_state(f"v{i}") for i in range(len(self._shapes))]

    def set_state(self, lr, momentum, weight_decay):
        self.load_meta(OptimMeta(self.kind(), lr, 0.0, 0.0, 0.0, weight_decay, momentum, 0))


@dataclass
class GradScalerState:
    """optim/core.rs:326-332."""

    scale: float = 65536.0
    growth_factor: float = 2.0
    backoff_factor: float = 0.5
    growth_interval: int = 2000
    consecutive_ok: int = 0


class GradScaler:
    """optim/core.rs:254-260, 334-413."""

    def __init__(self):
        self._h = None
        self._init = GradScalerState()

    @classmethod
    def new(cls):
        return cls()

    def _handle(self):
        if self._h is None:
            s = self._init
            st = _lib.ScalerState(s.scale, s.growth_factor, s.backoff_factor, s.growth_interval,
                                  s.consecutive_ok)
            h = C.c_void_p()
            _call(_lib.load().nbo_scaler_create(C.byref(st), C.byref(h)))
            self._h = h
        return self._h

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                _lib.load().nbo_scaler_destroy(h)
            except Exception:
                pass

    def unscale_and_update(self, grads) -> bool:
        g = _free_cache.get("scaler", grads)
        ok = C.c_int(0)
        _call(_lib.load().nbo_scaler_unscale_and_update(self._handle(), g._h, C.byref(ok)))
        return bool(ok.value)

    def scale_factor(self) -> float:
        return self.state().scale

    def scale_loss(self, loss):
        return loss * self.scale_factor()

    def state(self) -> GradScalerState:
        if self._h is None:
            return GradScalerState(**vars(self._init))
        st = _lib.ScalerState()
        _call(_lib.load().nbo_scaler_state_get(self._h, C.byref(st)))
        return GradScalerState(st.scale, st.growth_factor, st.backoff_factor, st.growth_interval,
                               st.consecutive_ok)

    def load_state(self, state: GradScalerState) -> None:
        self._init = GradScalerState(**vars(state))
        if self._h is not None:
            st = _lib.ScalerState(state.scale, state.growth_factor, state.backoff_factor,
                                  state.growth_interval, state.consecutive_ok)
            _call(_lib.load().nbo_scaler_load_state(self._h, C.byref(st)))


def clip_grad_norm(grads, max_norm: float) -> float:
    """nabla-train/src/trainer.rs:500-523."""
    g = _free_cache.get("clip", grads)
    norm = C.c_double(0.0)
    _call(_lib.load().nbo_clip_grad_norm(g._h, float(max_norm), C.byref(norm)))
    return norm.value


def has_non_finite(grads) -> bool:
    """Trainer::has_non_finite (nabla-train/src/trainer.rs:387-400)."""
    g = _free_cache.get("finite", grads)
    found = C.c_int(0)
    _call(_lib.load().nbo_has_non_finite(g._h, C.byref(found)))
    return bool(found.value)


def zero_grad(grads) -> None:
    """nabla-ml/src/autograd/ops.rs:1668-1673."""
    g = _free_cache.get("zero", grads)
    _call(_lib.load().nbo_zero_grad(g._h))


def scale_grad(grads, factor: float) -> None:
    """nabla-ml/src/autograd/ops.rs:1675-1680."""
    g = _free_cache.get("scale", grads)
    _call(_lib.load().nbo_scale_grad(g._h, float(factor)))


def adamw_step(param, grad, m, v, lr, beta1, beta2, eps, weight_decay, step: int) -> None:
    """The free function `adamw_step` (alg.rs:431-469): one AdamW update of one tensor
    with caller-held moments and the step number passed in.  `param`, `grad`, `m`, `v`
    are device tensors of one dtype (f32 or f64); `param`, `m`, `v` are updated in place."""
    import torch

    dtype = {torch.float32: "f32", torch.float64: "f64", torch.bfloat16: "bf16", torch.float16: "f16"}[param.dtype]
    opt = AdamW.new(lr, [_shape2(param)], dtype=dtype).beta1(beta1).beta2(beta2).eps(eps) \
        .weight_decay(weight_decay)
    opt._meta.step_count = int(step) - 1  # step() increments before use (alg.rs:120)
    opt.write_state("m0", m)
    opt.write_state("v0", v)
    opt.step([param], [grad])
    m.copy_(opt.read_state("m0").reshape(m.shape))
    v.copy_(opt.read_state("v0").reshape(v.shape))


def accumulate(accum, grads, zero_grads: bool = False) -> None:
    """buf[i] = &buf[i] + g (nabla-train/src/trainer.rs:262-266), optionally clearing g."""
    a = _free_cache.get("accum_a", accum)
    g = _free_cache.get("accum_g", grads)
    _call(_lib.load().nbo_accumulate(a._h, g._h, int(zero_grads)))


def unscale_accumulate(accum, grads, scaler: Optional["GradScaler"] = None, check_finite: bool = False,
                       write_grads: bool = False, want_sumsq: bool = True) -> Tuple[bool, Optional[float]]:
    """One micro-batch of the accumulating Trainer in a single pass (trainer.rs:230-267):
    finite scan + loss-scale update, buf[i] = &buf[i] + g / scale, and the sum of squares of
    the new buffer.  Returns (ok, sumsq); on ok == False the buffer holds garbage (the
    Trainer discards the accumulation then).  The gradients stay as they were unless
    `write_grads` asks for the reference's in-place result.  Only the last micro-batch of an
    accumulation needs the sum of squares (for the clip): with `want_sumsq=False` the pass has
    nothing to reduce but one bit (one small launch fewer); sumsq is then None."""
    a = _free_cache.get("accum_a", accum)
    g = _free_cache.get("accum_g", grads)
    ok, sumsq = C.c_int(0), C.c_double(0.0)
    flags = (_lib.ACC_CHECK_FINITE if check_finite else 0) | (_lib.ACC_WRITE_GRADS if write_grads else 0)
    _call(_lib.load().nbo_unscale_accumulate(scaler._handle() if scaler else None, a._h, g._h, flags,
                                             C.byref(ok), C.byref(sumsq) if want_sumsq else None))
    return bool(ok.value), (sumsq.value if want_sumsq else None)


def sync() -> None:
    _call(_lib.load().nbo_sync())
