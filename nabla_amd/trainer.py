"""The part of nabla-train's Trainer that runs between `backward()` and the next batch
(`Trainer::train_epoch_with_max_steps`, nabla-train/src/trainer.rs:216-291), for a caller
that produces gradients on the device itself.

Per micro-batch, in the reference's order:
  1. `scaler.unscale_and_update(&mut grads)`; a non-finite gradient drops the micro-batch
     *and* whatever was accumulated so far (trainer.rs:230-237);
  2. `has_non_finite` + `GradNanPolicy` (Skip: the same drop; Stop: an error), :239-251;
  3. accumulation `buf[i] = &buf[i] + g` into a buffer that starts as zeros (:253-267);
  4. once `grad_accum` micro-batches are in: `set_lr(lr_at_step(schedule, base_lr, step))`,
     `clip_grad_norm(buf, max_norm)`, `optimizer.step(params, buf)`, the buffer is zeroed
     and `state.step` advances (:269-291).

With `grad_accum == 1` and at most one of scaler / nan policy, steps 1-4 are one
`fused_step` (three launches, the skip decided on the device); the decision is read back
afterwards only because `state.step` -- which the schedule is a function of -- must not
advance on a skipped step.  With accumulation, steps 1-3 are one pass over the gradients
(`unscale_accumulate`: finite scan, unscale, add into the buffer, and the buffer's sum of
squares for the clip) with the reference's synchronous decision after it, and step 4 is
clip + update + zeroing in one kernel (`fused_step_norm`); with a scaler *and* a nan policy
the two decisions stay separate entry points in the reference's order.
"""
from __future__ import annotations

import enum
from typing import Optional, Sequence

from . import optim as nb
from .checkpoint import TrainState
from .schedule import ScheduleState, lr_at_step


class GradNanPolicy(enum.Enum):
    """trainer.rs:403-406."""

    SKIP = "skip"
    STOP = "stop"


class TrainError(RuntimeError):
    """TrainError::EvalError (the only variant this part of the Trainer returns)."""


class TrainerTail:
    def __init__(self, optimizer, params: Sequence):
        self.optimizer = optimizer
        self.params = list(params)
        self.schedule: Optional[ScheduleState] = None
        self.scaler: Optional[nb.GradScaler] = None
        self.grad_clip: Optional[float] = None
        self.nan_policy: Optional[GradNanPolicy] = None
        self.state = TrainState(epoch=0, step=0, grad_accum=1, rng_state=None)
        self._accum = None
        self._accum_count = 0

    # -- builders (trainer.rs:93-141) ---------------------------------------------------
    def with_schedule(self, schedule, base_lr: float) -> "TrainerTail":
        self.schedule = ScheduleState(base_lr=float(base_lr), schedule=schedule)
        return self

    def with_grad_scaler(self, scaler: nb.GradScaler) -> "TrainerTail":
        self.scaler = scaler
        return self

    def with_grad_accum(self, steps: int) -> "TrainerTail":
        self.state.grad_accum = max(int(steps), 1)
        return self

    def with_nan_policy(self, policy: GradNanPolicy) -> "TrainerTail":
        self.nan_policy = policy
        return self

    def with_grad_clip(self, max_norm: float) -> "TrainerTail":
        self.grad_clip = float(max_norm) if max_norm > 0.0 else None
        return self

    def set_state(self, state: TrainState) -> None:
        self.state = state

    def schedule_state(self) -> Optional[ScheduleState]:
        return self.schedule

    def loss_scale(self) -> float:
        """What the caller multiplies the loss by before backward (trainer.rs:218-221)."""
        return self.scaler.scale_factor() if self.scaler else 1.0

    # -- one micro-batch -------------------------------------------------------------------
    def after_backward(self, grads: Sequence) -> bool:
        """Consume one micro-batch's gradients; returns True if the optimizer stepped.  The
        reference unscales the gradients in place on the way; here they are only read (nothing
        uses them afterwards), except on the path with both a scaler and a nan policy."""
        grads = grads if isinstance(grads, nb.TensorList) else list(grads)
        fusable = self.state.grad_accum == 1 and not (self.scaler and self.nan_policy)
        if fusable:
            return self._fused(grads)
        return self._unfused(grads)

    def _drop(self) -> bool:
        self._accum = None
        self._accum_count = 0
        return False

    def _set_lr(self) -> None:
        if self.schedule is not None:
            self.optimizer.set_lr(lr_at_step(self.schedule.schedule, self.schedule.base_lr, self.state.step))

    def _fused(self, grads) -> bool:
        self._set_lr()  # harmless if the step is then skipped: the next call sets it again
        self.optimizer.fused_step(self.params, grads, scaler=self.scaler, max_norm=self.grad_clip or 0.0,
                                  skip_nonfinite=self.nan_policy is not None)
        if self.scaler is not None or self.nan_policy is not None:
            if self.optimizer.last_step().found_inf:
                if self.scaler is None and self.nan_policy is GradNanPolicy.STOP:
                    raise TrainError("non-finite gradient")
                return False
        self.state.step += 1
        return True

    def _unfused(self, grads) -> bool:
        import torch

        tensors = grads.tensors if isinstance(grads, nb.TensorList) else grads
        if self._accum is None:
            self._accum = [torch.zeros_like(g) for g in tensors]
        if self.scaler is not None and self.nan_policy is not None:
            # both decisions, in the reference's order: a micro-batch whose unscaled gradients
            # overflow is the nan policy's, not the scaler's
            if not self.scaler.unscale_and_update(grads):
                return self._drop()
            if nb.has_non_finite(grads):
                if self.nan_policy is GradNanPolicy.SKIP:
                    return self._drop()
                raise TrainError("non-finite gradient")
            nb.accumulate(self._accum, grads)
            sumsq = None
        else:
            # steps 1-3 in one pass over the gradients; a non-finite micro-batch leaves garbage
            # in the buffer, which is dropped with it
            # (the clip needs the buffer's sum of squares once the last micro-batch is in)
            last = self._accum_count + 1 >= self.state.grad_accum
            ok, sumsq = nb.unscale_accumulate(self._accum, grads, scaler=self.scaler,
                                              check_finite=self.nan_policy is not None, want_sumsq=last)
            if not ok:
                self._drop()
                if self.scaler is None and self.nan_policy is GradNanPolicy.STOP:
                    raise TrainError("non-finite gradient")
                return False
        self._accum_count += 1
        if self._accum_count < self.state.grad_accum:
            return False
        self._set_lr()
        # clip_grad_norm, step and the re-zeroing of the buffer (:274-290)
        if sumsq is None:
            self.optimizer.fused_step(self.params, self._accum, scaler=None, max_norm=self.grad_clip or 0.0,
                                      zero_grads=True)
        else:
            self.optimizer.fused_step_norm(self.params, self._accum, sumsq, max_norm=self.grad_clip or 0.0,
                                           zero_grads=True)
        self._accum_count = 0
        self.state.step += 1
        return True
