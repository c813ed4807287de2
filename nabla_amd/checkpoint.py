"""Checkpoint files of nabla-train: `params.nbla`, `optim.nbla`, `meta.txt`
(`nabla-train/src/checkpoint.rs:34-230`; tensor file format
`nabla-ml/src/module/core.rs:21,66-148`).

NBLA: magic "NBLA", u32 tensor count, then per tensor u32 name length, UTF-8 name,
u32 rows, u32 cols, rows*cols f64 values; everything little-endian.  Values are f64
whatever the tensor's element type (module/core.rs:80-84), so f32 / bf16 state
round-trips exactly.  meta.txt is key=value lines; floats are written the way Rust's
Display prints f64.

Tensors cross this module as numpy arrays or torch tensors (device tensors are
copied to the host for writing); loading returns numpy float64 arrays.
"""
from __future__ import annotations

import os
import struct
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .optim import GradScaler, GradScalerState, OptimStateError, rust_f64_str
from .schedule import ScheduleState, parse_schedule_state, schedule_pairs

NBLA_MAGIC = b"NBLA"
META_FILE, PARAMS_FILE, OPTIM_FILE = "meta.txt", "params.nbla", "optim.nbla"


class CheckpointError(Exception):
    """checkpoint.rs:14-20: Io / State / Optim / Parse, told apart by `kind`."""

    def __init__(self, kind: str, message: str):
        super().__init__(f"{kind}: {message}")
        self.kind = kind
        self.message = message


@dataclass
class TrainState:
    """trainer.rs TrainState: epoch, step, grad_accum, rng_state."""

    epoch: int = 0
    step: int = 0
    grad_accum: int = 1
    rng_state: Optional[int] = None


def _to_host_f64(t) -> np.ndarray:
    """Tensor -> 2-D float64 array, through f32 for bf16 / f16 (scalar/mod.rs:342-344)."""
    if isinstance(t, np.ndarray):
        a = t
    else:  # torch tensor
        import torch

        x = t.detach()
        if x.dtype in (torch.bfloat16, torch.float16):
            x = x.float()
        a = x.cpu().numpy()
    if a.ndim == 1:
        a = a.reshape(1, -1)
    elif a.ndim != 2:
        a = a.reshape(-1, a.shape[-1]) if a.ndim else a.reshape(1, 1)
    return np.ascontiguousarray(a, dtype="<f8")


def save_tensors(tensors: Sequence[Tuple[str, object]], path: str) -> None:
    """module/core.rs:66-88."""
    with open(path, "wb") as f:
        f.write(NBLA_MAGIC)
        f.write(struct.pack("<I", len(tensors)))
        for name, t in tensors:
            nb = name.encode("utf-8")
            a = _to_host_f64(t)
            f.write(struct.pack("<I", len(nb)))
            f.write(nb)
            f.write(struct.pack("<II", a.shape[0], a.shape[1]))
            a.tofile(f)


def load_tensors(path: str) -> List[Tuple[str, np.ndarray]]:
    """module/core.rs:90-120."""
    out = []
    with open(path, "rb") as f:
        if f.read(4) != NBLA_MAGIC:
            raise CheckpointError("Io", "not a nabla tensor file")

        def u32():
            b = f.read(4)
            if len(b) != 4:
                raise CheckpointError("Io", "failed to fill whole buffer")
            return struct.unpack("<I", b)[0]

        for _ in range(u32()):
            nlen = u32()
            raw = f.read(nlen)
            if len(raw) != nlen:
                raise CheckpointError("Io", "failed to fill whole buffer")
            try:
                name = raw.decode("utf-8")
            except UnicodeDecodeError as e:
                raise CheckpointError("Io", str(e)) from None
            rows, cols = u32(), u32()
            a = np.fromfile(f, dtype="<f8", count=rows * cols)
            if a.size != rows * cols:
                raise CheckpointError("Io", "failed to fill whole buffer")
            out.append((name, a.reshape(rows, cols)))
    return out


def write_meta(path: str, optimizer, scaler: Optional[GradScaler], schedule: Optional[ScheduleState],
               state: TrainState) -> None:
    """checkpoint.rs:107-150."""
    lines = ["version=1", f"epoch={state.epoch}", f"step={state.step}", f"grad_accum={state.grad_accum}"]
    if state.rng_state is not None:
        lines.append(f"rng.state={state.rng_state}")
    lines += [f"{k}={v}" for k, v in optimizer.meta_pairs()]
    if schedule is not None:
        lines += [f"{k}={v}" for k, v in schedule_pairs(schedule)]
    if scaler is not None:
        st = scaler.state()
        lines += ["scaler.enabled=1", f"scaler.scale={rust_f64_str(st.scale)}",
                  f"scaler.growth_factor={rust_f64_str(st.growth_factor)}",
                  f"scaler.backoff_factor={rust_f64_str(st.backoff_factor)}",
                  f"scaler.growth_interval={st.growth_interval}",
                  f"scaler.consecutive_ok={st.consecutive_ok}"]
    else:
        lines.append("scaler.enabled=0")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def _parse_usize(m, key):
    if key not in m:
        raise CheckpointError("Parse", f"missing {key}")
    v = m[key]
    body = v[1:] if v.startswith("+") else v
    if not body.isascii() or not body.isdigit():
        raise CheckpointError("Parse", f"bad {key}: {v}")
    return int(body)


def _parse_f64(m, key):
    if key not in m:
        raise CheckpointError("Parse", f"missing {key}")
    v = m[key]
    try:
        if v.strip() != v or not v:
            raise ValueError
        return float(v)
    except ValueError:
        raise CheckpointError("Parse", f"bad {key}: {v}") from None


def read_meta(path: str, optimizer):
    """checkpoint.rs:152-212 -> (GradScalerState | None, TrainState, ScheduleState | None)."""
    m: Dict[str, str] = {}
    with open(path) as f:
        for line in f.read().splitlines():
            if not line.strip():
                continue
            if "=" not in line:
                raise CheckpointError("Parse", line)
            k, v = line.split("=", 1)
            m[k] = v
    epoch, step, grad_accum = _parse_usize(m, "epoch"), _parse_usize(m, "step"), _parse_usize(m, "grad_accum")
    try:
        optimizer.load_meta_pairs(m)
    except OptimStateError as e:
        raise CheckpointError("Optim", str(e)) from None
    scaler_state = None
    try:
        enabled = _parse_usize(m, "scaler.enabled") == 1
    except CheckpointError:
        enabled = False
    if enabled:
        scaler_state = GradScalerState(_parse_f64(m, "scaler.scale"), _parse_f64(m, "scaler.growth_factor"),
                                       _parse_f64(m, "scaler.backoff_factor"),
                                       _parse_usize(m, "scaler.growth_interval"),
                                       _parse_usize(m, "scaler.consecutive_ok"))
    try:
        rng = _parse_usize(m, "rng.state")
    except CheckpointError:
        rng = None
    try:
        schedule = parse_schedule_state(m)
    except OptimStateError as e:
        raise CheckpointError("Optim", str(e)) from None
    return scaler_state, TrainState(epoch, step, grad_accum, rng), schedule


def _native(call, *args):
    """Run one of the library's NBLA entry points; its errors become CheckpointError with
    the reference's kinds (checkpoint.rs:14-20)."""
    from . import _lib
    from .optim import NablaPanic, _call

    try:
        _call(call(*args))
    except _lib.NablaOptimError as e:
        raise CheckpointError("Io" if e.status == _lib.ERR_IO else "State", e.message) from None
    except NablaPanic as e:  # shape mismatch of load_state_dict
        raise CheckpointError("State", str(e)) from None
    except OptimStateError as e:
        raise CheckpointError("Optim", str(e)) from None


def _name_array(names):
    import ctypes as C

    return (C.c_char_p * max(len(names), 1))(*[n.encode("utf-8") for n in names])


def save_params_native(path: str, named_tensors: Sequence[Tuple[str, object]]) -> None:
    """params.nbla straight from device tensors (nbo_nbla_save_list): no host copy of the
    whole model, no Python loop over elements."""
    from . import _lib
    from .optim import TensorList

    lst = TensorList([t for _, t in named_tensors])
    _native(_lib.load().nbo_nbla_save_list, path.encode(), lst._h, _name_array([n for n, _ in named_tensors]))


def load_params_native(path: str, named_tensors: Sequence[Tuple[str, object]]) -> None:
    """load_tensors + Module::load_state_dict into the given device tensors
    (nbo_nbla_load_list)."""
    from . import _lib
    from .optim import TensorList

    lst = TensorList([t for _, t in named_tensors])
    _native(_lib.load().nbo_nbla_load_list, path.encode(), lst._h, _name_array([n for n, _ in named_tensors]))


def _group_handles(optimizer):
    import ctypes as C

    subs = optimizer.group_optimizers()
    return len(subs), (C.c_void_p * len(subs))(*[o._handle() for o in subs])


def save_optim_native(path: str, optimizer) -> None:
    """optim.nbla from the optimizer's device state (nbo_optim_save_state; for a
    GroupOptimizer nbo_optim_save_state_groups, keys "g{gi}.m{i}")."""
    from . import _lib

    if hasattr(optimizer, "group_optimizers"):
        n, handles = _group_handles(optimizer)
        _native(_lib.load().nbo_optim_save_state_groups, n, handles, path.encode())
    else:
        _native(_lib.load().nbo_optim_save_state, optimizer._handle(), path.encode())


def load_optim_native(path: str, optimizer) -> None:
    """load_tensors + load_state_tensors into the optimizer's device state
    (nbo_optim_load_state / nbo_optim_load_state_groups)."""
    from . import _lib

    if hasattr(optimizer, "group_optimizers"):
        n, handles = _group_handles(optimizer)
        _native(_lib.load().nbo_optim_load_state_groups, n, handles, path.encode())
    else:
        _native(_lib.load().nbo_optim_load_state, optimizer._handle(), path.encode())


def _group_params_file(call, optimizer, named_tensors: Sequence[Tuple[str, object]], path: str) -> None:
    """params.nbla of a module whose parameters are spread over a GroupOptimizer's groups
    (nbo_optim_save_params_groups / nbo_optim_load_params_groups): a group that keeps master
    weights contributes (or receives) those, the other groups their tensors."""
    import ctypes as C

    tensors = [t for _, t in named_tensors]
    groups = optimizer._groups
    n = len(groups)
    group_of, index_in = [0] * len(tensors), [0] * len(tensors)
    for g, entry in enumerate(groups):
        for k, i in enumerate(entry.indices):
            group_of[i], index_in[i] = g, k
    opts = (C.c_void_p * max(n, 1))(*[e.optimizer._handle() for e in groups])
    lists = [optimizer._lists(e, "p", tensors) for e in groups]
    pl = (C.c_void_p * max(n, 1))(*[lst._h for lst in lists])
    m = len(tensors)
    _native(call, n, opts, pl, m, (C.c_uint32 * max(m, 1))(*group_of), (C.c_uint32 * max(m, 1))(*index_in),
            _name_array([name for name, _ in named_tensors]), path.encode())


def _keeps_master(optimizer) -> bool:
    return bool(getattr(optimizer, "_master", False))


def _groups_keep_master(optimizer) -> bool:
    return hasattr(optimizer, "group_optimizers") and any(_keeps_master(o) for o in optimizer.group_optimizers())


def save_checkpoint(directory: str, params: Sequence[Tuple[str, object]], optimizer,
                    scaler: Optional[GradScaler], schedule: Optional[ScheduleState],
                    state: TrainState, native: bool = False) -> None:
    """checkpoint.rs:38-69.  `params` is the module's state_dict: (name, tensor) pairs.  With
    `native` the two tensor files are written by the library straight from device memory.
    For a mixed-precision optimizer (16-bit parameters over f32 master weights) params.nbla
    holds the master weights, under the parameters' names: the 16-bit tensors are derived from
    them and could not restore them; both files then come straight from device memory."""
    os.makedirs(directory, exist_ok=True)
    if _keeps_master(optimizer):
        from . import _lib

        _native(_lib.load().nbo_optim_save_master, optimizer._handle(), os.path.join(directory, PARAMS_FILE).encode(),
                _name_array([n for n, _ in params]))
        save_optim_native(os.path.join(directory, OPTIM_FILE), optimizer)
        write_meta(os.path.join(directory, META_FILE), optimizer, scaler, schedule, state)
        return
    if _groups_keep_master(optimizer):
        # the groups' master weights, in the module's order under the parameters' names; the
        # tensors of a group without master weights as they are
        from . import _lib

        if len(params) != optimizer._param_count:
            raise CheckpointError("State", "nabla-train: GroupOptimizer param count mismatch")
        _group_params_file(_lib.load().nbo_optim_save_params_groups, optimizer, params,
                           os.path.join(directory, PARAMS_FILE))
        save_optim_native(os.path.join(directory, OPTIM_FILE), optimizer)
        write_meta(os.path.join(directory, META_FILE), optimizer, scaler, schedule, state)
        return
    if native:
        save_params_native(os.path.join(directory, PARAMS_FILE), params)
        save_optim_native(os.path.join(directory, OPTIM_FILE), optimizer)
    else:
        save_tensors(params, os.path.join(directory, PARAMS_FILE))
        save_tensors(optimizer.state_tensors(), os.path.join(directory, OPTIM_FILE))
    write_meta(os.path.join(directory, META_FILE), optimizer, scaler, schedule, state)


def load_checkpoint(directory: str, optimizer, scaler: Optional[GradScaler] = None,
                    into: Optional[Sequence[Tuple[str, object]]] = None):
    """checkpoint.rs:71-105 -> (params, TrainState, ScheduleState | None).  Optimizer
    tensors and meta are loaded into `optimizer`, the scaler state into `scaler`; the
    parameters are returned for the caller's module to take (load_state_dict) -- or, with
    `into` = the module's named device tensors, read into those by the library itself
    (then `params` is None).  For a mixed-precision optimizer params.nbla holds its f32 master
    weights: they go into the optimizer, and `into` (the module's named 16-bit tensors, needed
    for their names) receives the parameters narrowed from them."""
    if _keeps_master(optimizer):
        from . import _lib
        from .optim import TensorList

        if into is None:
            raise ValueError("a mixed-precision optimizer's checkpoint is loaded with into=[(name, 16-bit tensor), ...]: "
                             "params.nbla holds its master weights under the parameters' names")
        _native(_lib.load().nbo_optim_load_master, optimizer._handle(), os.path.join(directory, PARAMS_FILE).encode(),
                _name_array([n for n, _ in into]))
        optimizer.params_from_master(TensorList([t for _, t in into]))
        load_optim_native(os.path.join(directory, OPTIM_FILE), optimizer)
        params = None
    elif _groups_keep_master(optimizer):
        from . import _lib
        from .optim import TensorList

        if into is None:
            raise ValueError("a mixed-precision optimizer's checkpoint is loaded with into=[(name, 16-bit tensor), ...]: "
                             "params.nbla holds its master weights under the parameters' names")
        if len(into) != optimizer._param_count:
            raise CheckpointError("State", "nabla-train: GroupOptimizer param count mismatch")
        # the whole file is checked against all names and shapes before anything is written
        _group_params_file(_lib.load().nbo_optim_load_params_groups, optimizer, into,
                           os.path.join(directory, PARAMS_FILE))
        for idxs, o in zip(optimizer.group_indices(), optimizer.group_optimizers()):
            if _keeps_master(o):
                o.params_from_master(TensorList([into[i][1] for i in idxs]))
        load_optim_native(os.path.join(directory, OPTIM_FILE), optimizer)
        params = None
    elif into is not None:
        load_params_native(os.path.join(directory, PARAMS_FILE), into)
        load_optim_native(os.path.join(directory, OPTIM_FILE), optimizer)
        params = None
    else:
        params = load_tensors(os.path.join(directory, PARAMS_FILE))
        optim_tensors = load_tensors(os.path.join(directory, OPTIM_FILE))
        try:
            import torch

            optimizer.load_state_tensors([(k, torch.from_numpy(v)) for k, v in optim_tensors])
        except OptimStateError as e:
            raise CheckpointError("Optim", str(e)) from None
    scaler_state, train_state, schedule = read_meta(os.path.join(directory, META_FILE), optimizer)
    if scaler is not None and scaler_state is not None:
        scaler.load_state(scaler_state)
    return params, train_state, schedule
