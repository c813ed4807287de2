"""TrainerTail (nabla_amd/trainer.py) against the same control flow written out over the
oracle's primitives, line by line after nabla-train/src/trainer.rs:216-291: scaler,
nan policy, accumulation over micro-batches, schedule, clip, step, zeroing."""
import numpy as np
import pytest

import oracle as O
from nabla_amd import optim as nb
from nabla_amd import schedule as S
from nabla_amd.trainer import GradNanPolicy, TrainError, TrainerTail
from tests import helpers as H

SHAPES = [(3, 7), (1, 9000), (64, 33)]


class OracleTrainer:
    """trainer.rs:216-291 over the CPU oracle (f32, AdamW)."""

    def __init__(self, params, meta, grad_accum, scaler, clip, schedule, policy):
        self.p, self.meta = params, meta
        self.m, self.v = H.zeros_like_list(params), H.zeros_like_list(params)
        self.grad_accum, self.scaler, self.clip, self.schedule, self.policy = grad_accum, scaler, clip, schedule, policy
        self.step, self.accum, self.count = 0, None, 0

    def after_backward(self, grads):
        grads = H.copy_list(grads)
        if self.scaler is not None and not O.scaler_unscale_and_update(self.scaler, grads):  # :230-237
            self.accum, self.count = None, 0
            return False
        if self.policy is not None and any(not np.isfinite(g).all() for g in grads):  # :239-251
            if self.policy == "skip":
                self.accum, self.count = None, 0
                return False
            raise TrainError("non-finite gradient")
        if self.accum is None:  # :253-260
            self.accum = H.zeros_like_list(grads)
        self.accum = [O.add(b, g) for b, g in zip(self.accum, grads)]  # :262-266
        self.count += 1
        if self.count < self.grad_accum:
            return False
        if self.schedule is not None:  # :270-273
            self.meta.lr = O.lr_at_step(self.schedule[0], self.schedule[1], self.step)
        if self.clip:  # :274-278
            O.clip_grad_norm(self.accum, self.clip)
        O.set_pow_mode(O.POW_SQRT)
        try:
            O.adam_step(self.meta, self.p, self.accum, self.m, self.v)  # :279-283
        finally:
            O.set_pow_mode(O.POW_LIBM)
        self.count = 0
        self.accum = H.zeros_like_list(self.accum)  # :285-290
        self.step += 1
        return True


def _micro_batches(n, scale, bad_at, seed):
    out = []
    for k in range(n):
        g = [a * np.float32(scale) for a in H.randn_list(SHAPES, seed + 31 * k, 1e-3)]
        if k in bad_at:
            g[1][(17 * k) % g[1].size] = np.inf if k % 2 else np.nan
        out.append(g)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("grad_accum,use_scaler,policy", [
    (3, True, None),        # accumulation with a dynamic loss scale
    (2, False, "skip"),     # accumulation with GradNanPolicy::Skip
    (1, True, None),        # the fused path: scaler
    (1, False, "skip"),     # the fused path: nan policy
    (1, True, "skip"),      # both: unfused even without accumulation
    (1, False, None),       # nothing to decide
])
def test_trainer_tail_matches_the_reference_control_flow(gpu, grad_accum, use_scaler, policy):
    n_micro, bad_at = 14, ({4, 9} if (use_scaler or policy) else set())
    scale0 = 1024.0 if use_scaler else 1.0
    batches = _micro_batches(n_micro, scale0, bad_at, 5000)
    p0 = H.randn_list(SHAPES, 4000, 0.02)
    cosine, base_lr = S.Cosine(warmup_steps=2, total_steps=10, min_lr=1e-5), 1e-3
    o_sched = (O.Schedule(0, 2, 10, 1e-5, 0.0), base_lr)

    p_dev = H.dev_list(p0, SHAPES)
    opt = nb.AdamW.new(base_lr, SHAPES).beta2(0.95).weight_decay(0.1)
    tail = TrainerTail(opt, p_dev).with_grad_accum(grad_accum).with_grad_clip(0.05).with_schedule(cosine, base_lr)
    scaler = None
    if use_scaler:
        scaler = nb.GradScaler.new()
        scaler.load_state(nb.GradScalerState(scale0, 2.0, 0.5, 3, 0))
        tail.with_grad_scaler(scaler)
    if policy:
        tail.with_nan_policy(GradNanPolicy.SKIP)

    ref = OracleTrainer(H.copy_list(p0), O.adamw_meta(base_lr, 0.9, 0.95, 1e-8, 0.1), grad_accum,
                        O.ScalerState(scale0, 2.0, 0.5, 3, 0) if use_scaler else None, 0.05, o_sched, policy)
    for k, g in enumerate(batches):
        if use_scaler:
            assert tail.loss_scale() == ref.scaler.scale, k
        stepped = tail.after_backward(H.dev_list(g, SHAPES))
        assert stepped == ref.after_backward(g), f"micro-batch {k}"
        assert tail.state.step == ref.step, f"micro-batch {k}"
    assert ref.step >= 3
    assert opt.step_count() == ref.meta.step_count == ref.step
    H.assert_bits_equal(H.host_list(p_dev), ref.p, "params")
    H.assert_bits_equal(H.host_list(opt.moments()[0]), ref.m, "m")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), ref.v, "v")
    if use_scaler:
        st = scaler.state()
        assert (st.scale, st.consecutive_ok) == (ref.scaler.scale, ref.scaler.consecutive_ok)


@pytest.mark.gpu
@pytest.mark.parametrize("grad_accum", [1, 2])
def test_nan_policy_stop_is_an_error_and_leaves_the_parameters_alone(gpu, grad_accum):
    p0 = H.randn_list(SHAPES, 4100, 0.02)
    p_dev = H.dev_list(p0, SHAPES)
    tail = TrainerTail(nb.Adam.new(1e-3, SHAPES), p_dev).with_grad_accum(grad_accum).with_nan_policy(GradNanPolicy.STOP)
    bad = _micro_batches(1, 1.0, {0}, 6000)[0]
    with pytest.raises(TrainError, match="non-finite gradient"):
        tail.after_backward(H.dev_list(bad, SHAPES))
    H.assert_bits_equal(H.host_list(p_dev), p0, "params after the error")
    assert tail.state.step == 0


def test_builders_follow_the_reference():
    """trainer.rs:105-141: grad_accum is at least 1, a non-positive clip turns clipping off."""
    tail = TrainerTail(nb.Sgd.new(0.1, [(1, 1)]), []).with_grad_accum(0).with_grad_clip(0.0)
    assert tail.state.grad_accum == 1 and tail.grad_clip is None and tail.loss_scale() == 1.0
    assert tail.with_grad_clip(2.5).grad_clip == 2.5 and tail.with_grad_accum(4).state.grad_accum == 4


# ---- the reference's own Trainer tests (nabla-train/tests/trainer.rs), replayed ------------

@pytest.mark.gpu
def test_reference_train_epoch_updates_weight(gpu):
    """trainer.rs tests :108-132: one f64 weight of 1.0, loss = mse(w, 0) so the gradient is
    2w, Sgd(0.1), two batches -> two steps and a smaller weight (exactly 0.8, then 0.64)."""
    w = H.to_dev(np.ones(1, dtype=np.float64), (1, 1))
    trainer = TrainerTail(nb.Sgd.new(0.1, [(1, 1)], dtype="f64"), [w])
    steps = 0
    for _batch in (0, 1):
        grad = (2.0 * w).contiguous()  # backward of mean((w - 0)^2)
        steps += int(trainer.after_backward([grad]))
    assert steps == 2 and trainer.state.step == 2
    new_w = float(H.to_host(w)[0])
    assert new_w < 1.0 and abs(new_w - 0.64) < 1e-12


@pytest.mark.gpu
def test_reference_checkpoint_roundtrip_with_schedule(gpu, tmp_path):
    """trainer.rs tests :249-304: Sgd(0.1) over two 1x1 parameters, a default GradScaler, a
    Step{1, 0.9} schedule and TrainState{2, 3, 1, Some(42)} survive save -> load."""
    from nabla_amd import checkpoint as ck
    from nabla_amd.schedule import ScheduleState, Step

    shapes = [(1, 1), (1, 1)]
    module = [("w", H.to_dev(np.array([1.5]), (1, 1))), ("b", H.to_dev(np.array([-0.5]), (1, 1)))]
    opt = nb.Sgd.new(0.1, shapes, dtype="f64")
    ck.save_checkpoint(str(tmp_path), module, opt, nb.GradScaler.new(),
                       ScheduleState(base_lr=0.1, schedule=Step(step_size=1, gamma=0.9)),
                       ck.TrainState(epoch=2, step=3, grad_accum=1, rng_state=42))
    opt2, scaler2 = nb.Sgd.new(0.1, shapes, dtype="f64"), nb.GradScaler.new()
    params, state2, schedule2 = ck.load_checkpoint(str(tmp_path), opt2, scaler2)
    assert (state2.epoch, state2.step, state2.rng_state, state2.grad_accum) == (2, 3, 42, 1)
    assert schedule2 is not None and schedule2.base_lr == 0.1 and schedule2.schedule == Step(1, 0.9)
    assert [k for k, _ in params] == ["w", "b"] and float(params[0][1].reshape(-1)[0]) == 1.5
    assert scaler2.state().scale == 65536.0 and opt2.meta().lr == 0.1


@pytest.mark.gpu
@pytest.mark.parametrize("use_scaler", [False, True])
def test_trainer_tail_drives_a_group_optimizer_with_accumulation(gpu, use_scaler):
    """TrainerTail over a GroupOptimizer (no-decay group for biases and norms) with
    grad_accum = 2: the one-pass micro-batch and the known-norm group step against the
    separate entry points -- unscale, accumulate, then the grouped fused step, which is itself
    checked against the oracle in test_next_rows -- on a second copy of everything."""
    import torch

    from nabla_amd import groups as G

    names = ["embed", "l0.w", "l0.bias", "l0.norm", "l1.w", "head"]
    shapes = [(50, 16), (16, 16), (1, 16), (1, 16), (16, 9000), (16, 50)]
    p0 = H.randn_list(shapes, 4200, 0.02)
    scale0 = 2048.0 if use_scaler else 1.0

    def fresh():
        p = H.dev_list(p0, shapes)
        opt = G.GroupOptimizer.adamw_with_decay_exclusions(list(zip(names, p)), 1e-3, 0.1, ["bias", "norm"])
        sc = None
        if use_scaler:
            sc = nb.GradScaler.new()
            sc.load_state(nb.GradScalerState(scale0, 2.0, 0.5, 3, 0))
        return p, opt, sc

    p1, o1, s1 = fresh()
    p2, o2, s2 = fresh()
    tail = TrainerTail(o1, p1).with_grad_accum(2).with_grad_clip(0.05)
    if use_scaler:
        tail.with_grad_scaler(s1)
    buf, count, steps = None, 0, 0
    for k in range(9):
        scale = s2.scale_factor() if use_scaler else 1.0
        g = [a * np.float32(scale) for a in H.randn_list(shapes, 4300 + k, 1e-3)]
        if use_scaler and k == 3:
            g[4][77] = np.inf
        stepped = tail.after_backward(H.dev_list(g, shapes))
        g2 = H.dev_list(g, shapes)
        if use_scaler and not s2.unscale_and_update(g2):
            buf, count = None, 0
            assert not stepped
            continue
        if buf is None:
            buf = [torch.zeros_like(t) for t in g2]
        nb.accumulate(buf, g2)
        count += 1
        if count == 2:
            o2.fused_step(p2, buf, max_norm=0.05, zero_grads=True)
            count, steps = 0, steps + 1
        assert stepped == (count == 0), k
    assert steps == (3 if use_scaler else 4) and tail.state.step == steps
    H.assert_bits_equal(H.host_list(p1), H.host_list(p2), "params")
    for (n1, t1), (n2, t2) in zip(o1.state_tensors(), o2.state_tensors()):
        assert n1 == n2
        H.assert_bits_equal([H.to_host(t1)], [H.to_host(t2)], n1)
    assert o1.last_step().step_count == o2.last_step().step_count == steps
