"""Parameter groups of nabla-train (`optim/groups.rs`): name patterns select which
per-group Sgd / Adam / AdamW a parameter belongs to.  Each group is one engine
optimizer; the reference clones parameters in and out of per-group vectors
(groups.rs:281-292), here each group simply gets the list of its own tensors."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field, replace
from typing import Dict, List, Optional, Sequence, Tuple

from . import _lib
from .optim import (Adam, AdamW, GradScaler, NablaPanic, OptimMeta, OptimStateError, Sgd, TensorList, _ListCache,
                    _call, _shape2, rust_f64_str)


# ParamMatch (groups.rs:11-17): ("equals" | "prefix" | "suffix" | "contains", text)
def Equals(v):
    return ("equals", v)


def Prefix(v):
    return ("prefix", v)


def Suffix(v):
    return ("suffix", v)


def Contains(v):
    return ("contains", v)


@dataclass(frozen=True)
class ParamSelector:
    """groups.rs:19-38.  matches=None is ParamSelector::All."""

    matches_any: Optional[Tuple[Tuple[str, str], ...]] = None

    @staticmethod
    def All():
        return ParamSelector(None)

    @staticmethod
    def Any(matches):
        return ParamSelector(tuple(matches))

    def matches(self, name: str) -> bool:
        if self.matches_any is None:
            return True
        for kind, v in self.matches_any:
            if (kind == "equals" and name == v) or (kind == "prefix" and name.startswith(v)) or \
               (kind == "suffix" and name.endswith(v)) or (kind == "contains" and v in name):
                return True
        return False


@dataclass(frozen=True)
class ParamGroupConfig:
    """groups.rs:40-132."""

    name: str
    selector: ParamSelector
    kind: str
    lr: float
    weight_decay: float = 0.0
    momentum: float = 0.0
    beta1: float = 0.9
    beta2: float = 0.999
    eps: float = 1e-8

    @staticmethod
    def adamw(name, selector, lr, weight_decay):
        return ParamGroupConfig(name, selector, "adamw", lr, weight_decay)

    @staticmethod
    def adam(name, selector, lr):
        return ParamGroupConfig(name, selector, "adam", lr)

    @staticmethod
    def sgd(name, selector, lr, momentum, weight_decay):
        return ParamGroupConfig(name, selector, "sgd", lr, weight_decay, momentum, 0.0, 0.0, 0.0)

    def betas(self, beta1, beta2):
        return replace(self, beta1=beta1, beta2=beta2)

    def with_eps(self, eps):
        return replace(self, eps=eps)

    def with_momentum(self, momentum):
        return replace(self, momentum=momentum)

    def with_weight_decay(self, weight_decay):
        return replace(self, weight_decay=weight_decay)


# ParamExclusionPreset::patterns (groups.rs:134-148)
PRESET_PATTERNS = {"bias": ("bias",), "norm": ("norm", "bn", "ln"), "embedding": ("embed", "embedding")}


def _make_optimizer(cfg: ParamGroupConfig, shapes, **kw):
    """GroupOptim::new (groups.rs:449-475)."""
    if cfg.kind == "adamw":
        return AdamW.new(cfg.lr, shapes, **kw).beta1(cfg.beta1).beta2(cfg.beta2).eps(cfg.eps) \
            .weight_decay(cfg.weight_decay)
    if cfg.kind == "adam":
        return Adam.new(cfg.lr, shapes, **kw).beta1(cfg.beta1).beta2(cfg.beta2).eps(cfg.eps)
    if cfg.kind == "sgd":
        return Sgd.new(cfg.lr, shapes, **kw).momentum(cfg.momentum).weight_decay(cfg.weight_decay)
    raise OptimStateError(f"bad optim.kind: {cfg.kind}")


@dataclass
class _GroupEntry:
    indices: List[int]
    name: str
    base_lr: float
    optimizer: object
    lists: _ListCache = field(default_factory=_ListCache)  # this group's param / grad descriptors


class GroupOptimizer:
    """groups.rs:150-427."""

    def __init__(self, groups: List[_GroupEntry], param_count: int, base_lr: float):
        self._groups = groups
        self._param_count = param_count
        self._base_lr = base_lr
        self._all_grads = _ListCache()

    @classmethod
    def from_named_params(cls, named: Sequence[Tuple[str, object]], groups: Sequence[ParamGroupConfig],
                          default_group: Optional[ParamGroupConfig] = None, **kw):
        """groups.rs:168-226: first matching group wins, then the default group."""
        buckets = [(cfg, []) for cfg in groups]
        default_bucket = (default_group, []) if default_group is not None else None
        assigned = [False] * len(named)
        for i, (name, _) in enumerate(named):
            for cfg, idxs in buckets:
                if cfg.selector.matches(name):
                    idxs.append(i)
                    assigned[i] = True
                    break
            else:
                if default_bucket is not None:
                    default_bucket[1].append(i)
                    assigned[i] = True
        if not all(assigned):
            raise OptimStateError("nabla-train: group assignment incomplete")
        entries = []
        for cfg, idxs in buckets + ([default_bucket] if default_bucket else []):
            if not idxs:
                continue
            shapes = [_shape2(named[i][1]) for i in idxs]
            entries.append(_GroupEntry(idxs, cfg.name, cfg.lr, _make_optimizer(cfg, shapes, **kw)))
        base_lr = entries[0].base_lr if entries else 1.0
        return cls(entries, len(named), base_lr)

    from_module = from_named_params

    @classmethod
    def adamw_with_decay_exclusions(cls, named, lr, weight_decay, exclude: Sequence[str], **kw):
        """groups.rs:228-242."""
        matches = []
        for s in exclude:
            matches += [Suffix(s), Contains(s)]
        no_decay = ParamGroupConfig.adamw("no_decay", ParamSelector.Any(matches), lr, 0.0)
        decay = ParamGroupConfig.adamw("decay", ParamSelector.All(), lr, weight_decay)
        return cls.from_named_params(named, [no_decay], decay, **kw)

    @classmethod
    def adamw_with_decay_presets(cls, named, lr, weight_decay, presets: Sequence[str], **kw):
        """groups.rs:244-261; presets are 'bias' | 'norm' | 'embedding'."""
        pats = [p for preset in presets for p in PRESET_PATTERNS[preset]]
        return cls.adamw_with_decay_exclusions(named, lr, weight_decay, pats, **kw)

    def groups(self) -> int:
        return len(self._groups)

    def group_indices(self) -> List[List[int]]:
        return [list(g.indices) for g in self._groups]

    def group_optimizers(self):
        return [g.optimizer for g in self._groups]

    # -- trait Optimizer (groups.rs:268-313) ---------------------------------------------
    def _check(self, params, grads):
        if len(params) != len(grads):
            raise NablaPanic("nabla-train: GroupOptimizer params/grads length mismatch")
        if len(params) != self._param_count:
            raise NablaPanic("nabla-train: GroupOptimizer param count mismatch")

    def _lists(self, group: _GroupEntry, slot: str, tensors) -> TensorList:
        return group.lists.get(slot, [tensors[i] for i in group.indices])

    def step(self, params, grads) -> None:
        self._check(params, grads)
        for g in self._groups:
            g.optimizer.step(self._lists(g, "p", params), self._lists(g, "g", grads))

    def fused_step(self, params, grads, scaler: Optional[GradScaler] = None, max_norm: float = 0.0,
                   zero_grads: bool = False, skip_nonfinite: bool = False, zero_on_skip: bool = False) -> None:
        """The Trainer tail with one unscale / clip decision over all gradients."""
        self._check(params, grads)
        all_grads = self._all_grads.get("g", list(grads))
        n = len(self._groups)
        opts = (C.c_void_p * n)(*[g.optimizer._handle() for g in self._groups])
        pl = (C.c_void_p * n)(*[self._lists(g, "p", params)._h for g in self._groups])
        gl = (C.c_void_p * n)(*[self._lists(g, "g", grads)._h for g in self._groups])
        flags = ((_lib.STEP_ZERO_GRADS if zero_grads else 0) | (_lib.STEP_SKIP_NONFINITE if skip_nonfinite else 0)
                 | (_lib.STEP_ZERO_ON_SKIP if zero_on_skip else 0))
        _call(_lib.load().nbo_fused_step_groups(n, opts, pl, gl, scaler._handle() if scaler else None,
                                                all_grads._h, float(max_norm), flags))

    def fused_step_norm(self, params, grads, sumsq: float, max_norm: float = 0.0,
                        zero_grads: bool = False) -> None:
        """clip + every group's step (+ zeroing) over gradients whose sum of squares is known."""
        self._check(params, grads)
        n = len(self._groups)
        opts = (C.c_void_p * n)(*[g.optimizer._handle() for g in self._groups])
        pl = (C.c_void_p * n)(*[self._lists(g, "p", params)._h for g in self._groups])
        gl = (C.c_void_p * n)(*[self._lists(g, "g", grads)._h for g in self._groups])
        _call(_lib.load().nbo_fused_step_groups_norm(n, opts, pl, gl, float(max_norm), float(sumsq),
                                                     _lib.STEP_ZERO_GRADS if zero_grads else 0))

    def last_step(self):
        """Outcome of the most recent fused step (one decision for all groups)."""
        return self._groups[0].optimizer.last_step()

    def reset(self) -> None:
        for g in self._groups:
            g.optimizer.reset()

    def set_lr(self, lr: float) -> None:
        if self._base_lr <= 0.0:
            for g in self._groups:
                g.optimizer.set_lr(lr)
            return
        scale = lr / self._base_lr
        for g in self._groups:
            g.optimizer.set_lr(g.base_lr * scale)

    # -- trait OptimState (groups.rs:315-427) ----------------------------------------------
    def kind(self) -> str:
        return "adamw"

    def state_tensors(self):
        out = []
        for gi, g in enumerate(self._groups):
            out += [(f"g{gi}.{name}", t) for name, t in g.optimizer.state_tensors()]
        return out

    def load_state_tensors(self, tensors) -> None:
        buckets = [[] for _ in self._groups]
        for name, t in tensors:
            if "." not in name:
                raise OptimStateError(f"bad group tensor key: {name}")
            g, rest = name.split(".", 1)
            if not g.startswith("g"):
                raise OptimStateError(f"bad group tensor key: {name}")
            idx = g[1:]
            digits = idx[1:] if idx.startswith("+") else idx
            if not digits.isascii() or not digits.isdigit():
                raise OptimStateError(f"bad group index: {idx}")
            gi = int(digits)
            if gi >= len(buckets):
                raise OptimStateError(f"group index out of range: {gi}")
            buckets[gi].append((rest, t))
        for g, b in zip(self._groups, buckets):
            g.optimizer.load_state_tensors(b)

    def meta(self) -> OptimMeta:
        return OptimMeta("adamw", self._base_lr, 0.0, 0.0, 0.0, 0.0, 0.0, 0)

    def load_meta(self, meta: OptimMeta) -> None:
        return None

    def meta_pairs(self):
        out = [("optim.group.count", str(len(self._groups)))]
        for gi, g in enumerate(self._groups):
            m = g.optimizer.meta()
            out += [(f"optim.group.{gi}.name", g.name), (f"optim.group.{gi}.kind", m.kind),
                    (f"optim.group.{gi}.lr", rust_f64_str(m.lr)),
                    (f"optim.group.{gi}.beta1", rust_f64_str(m.beta1)),
                    (f"optim.group.{gi}.beta2", rust_f64_str(m.beta2)),
                    (f"optim.group.{gi}.eps", rust_f64_str(m.eps)),
                    (f"optim.group.{gi}.weight_decay", rust_f64_str(m.weight_decay)),
                    (f"optim.group.{gi}.momentum", rust_f64_str(m.momentum)),
                    (f"optim.group.{gi}.step_count", str(m.step_count))]
        return out

    def load_meta_pairs(self, m: Dict[str, str]) -> None:
        def get(key):
            if key not in m:
                raise OptimStateError(f"missing {key}")
            return m[key]

        def usize(key):
            v = get(key)
            body = v[1:] if v.startswith("+") else v
            if not body.isascii() or not body.isdigit():
                raise OptimStateError(f"bad {key}: {v}")
            return int(body)

        def f64(key):
            v = get(key)
            try:
                if v.strip() != v or not v:
                    raise ValueError
                return float(v)
            except ValueError:
                raise OptimStateError(f"bad {key}: {v}") from None

        if usize("optim.group.count") != len(self._groups):
            raise OptimStateError("optim.group.count mismatch")
        for gi, g in enumerate(self._groups):
            if get(f"optim.group.{gi}.name") != g.name:
                raise OptimStateError(f"optim.group.{gi}.name mismatch")
            kind = get(f"optim.group.{gi}.kind")
            if kind not in ("adamw", "adam", "sgd"):
                raise OptimStateError(f"bad optim.kind: {kind}")
            p = f"optim.group.{gi}."
            g.optimizer.load_meta(OptimMeta(kind, f64(p + "lr"), f64(p + "beta1"), f64(p + "beta2"),
                                            f64(p + "eps"), f64(p + "weight_decay"), f64(p + "momentum"),
                                            usize(p + "step_count")))
        if self._groups:
            self._base_lr = self._groups[0].optimizer.meta().lr
