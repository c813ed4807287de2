"""Backend primitives of nabla-core on lists of device tensors.

The reference's optimizers are chains of `Backend` passes
(nabla-core/src/common/backend/mod.rs:82-216, 275-279; CPU semantics
nabla-core/src/cpu/mod.rs:137-139, 181, 211-232, 264-272): `scale`, `axpy_inplace`, `add`,
`emul`, `ediv`, `powf`, `zeros`, `clone_storage`, `cast`, and `Tensor::map(|x| x + s)`
(tensor/ops.rs:563-569).  Here each of them is one multi-tensor launch over a whole
tensor list -- the generalisation of the reference's never-launched `k_multi_axpy3`
(cuda_hip/common/kernels/k_ops.cuh:541-575) from three tensors to any number -- with the
reference's rounding: one IEEE operation per element in the list's element type (for bf16
and f16 the f32 operation followed by `T::from_f32`).

Arguments are sequences of same-dtype device tensors (anything with `data_ptr()`,
`shape`, `dtype`: torch tensors on cuda:0) or `TensorList`s.  Functions that produce a new
tensor list in the reference take the output list as `out=` here; `out` may be one of the
operands.  Everything is asynchronous on the library's stream.
"""
from typing import Sequence, Union

from . import _lib
from .optim import TensorList, _call

OP_SCALE, OP_AXPY, OP_ADD, OP_EMUL, OP_EDIV, OP_POWF, OP_ADD_SCALAR, OP_ZEROS, OP_CLONE = range(9)

Tensors = Union[TensorList, Sequence]


def _list(x: Tensors) -> TensorList:
    return x if isinstance(x, TensorList) else TensorList(x)


def _apply(op: int, out: Tensors, a=None, b=None, s: float = 0.0) -> None:
    lo = _list(out)
    la = _list(a) if a is not None else None
    lb = _list(b) if b is not None else None
    _call(_lib.load().nbo_backend_apply(op, lo._h, la._h if la else None, lb._h if lb else None, float(s)))


def scale(a: Tensors, s: float, out: Tensors) -> None:
    """B::scale (cpu/mod.rs:211-213): out = a * T(s)."""
    _apply(OP_SCALE, out, a, None, s)


def axpy_inplace(y: Tensors, alpha: float, x: Tensors) -> None:
    """B::axpy_inplace (cpu/mod.rs:216-223): y = y + T(alpha) * x, product and sum each
    rounded; shapes must match (tensor/ops.rs:638-646)."""
    _apply(OP_AXPY, y, x, None, alpha)


def add(a: Tensors, b: Tensors, out: Tensors) -> None:
    """B::add (cpu/mod.rs:181)."""
    _apply(OP_ADD, out, a, b)


def emul(a: Tensors, b: Tensors, out: Tensors) -> None:
    """BackendMath::emul (cpu/mod.rs:270)."""
    _apply(OP_EMUL, out, a, b)


def ediv(a: Tensors, b: Tensors, out: Tensors) -> None:
    """BackendMath::ediv (cpu/mod.rs:272)."""
    _apply(OP_EDIV, out, a, b)


def powf(a: Tensors, p: float, out: Tensors) -> None:
    """BackendMath::powf (cpu/mod.rs:264-266).  p = 0.5 is the correctly rounded square
    root (within 1 ulp of any faithful powf); other exponents use the device math library."""
    _apply(OP_POWF, out, a, None, p)


def map_add(a: Tensors, c: float, out: Tensors) -> None:
    """Tensor::map(|x| x + c) as the optimizers use it for `+ eps` (optim/alg.rs:133)."""
    _apply(OP_ADD_SCALAR, out, a, None, c)


def zeros(out: Tensors) -> None:
    """B::zeros (cpu/mod.rs:137-139) into existing storage."""
    _apply(OP_ZEROS, out)


def clone_storage(a: Tensors, out: Tensors) -> None:
    """B::clone_storage (cpu/mod.rs:226-232)."""
    _apply(OP_CLONE, out, a)


def cast(src: Tensors, dst: Tensors) -> None:
    """B::cast default (backend/mod.rs:157-160): dst = U::from_f64(src.to_f64()), between
    any two of f32 / bf16 / f16 / f64."""
    ld, ls = _list(dst), _list(src)  # keep the descriptors alive across the call
    _call(_lib.load().nbo_backend_cast(ld._h, ls._h))
