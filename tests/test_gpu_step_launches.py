"""How many launches a step is, and what a skipped step leaves behind.

The reference's `Adam::step` / `AdamW::step` is one call (alg.rs:109-150, 254-291): here it is
one launch of a kernel that prepares its own per-step scalars and advances step_count exactly
once; a grouped fused step is the norm pass, its second stage and ONE update launch for up to
sixteen groups of one optimizer kind (each with its own hyper-parameters, optim/groups.rs:269-293).
`unscale_and_update` leaves zeros in the gradients when it finds inf / NaN (core.rs:372-375):
the fused step does so with NBO_STEP_ZERO_ON_SKIP."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from nabla_amd import _lib
from nabla_amd import groups as G
from nabla_amd import optim as nb
from tests import helpers as H

pytestmark = pytest.mark.gpu


def _launches(names):
    L = _lib.load()
    out = {}
    for n in names:
        cnt, ms = C.c_uint64(0), C.c_double(0.0)
        _lib.check(L.nbo_profile_read(n.encode(), C.byref(cnt), C.byref(ms)))
        out[n] = cnt.value
    return out


def test_unfused_adam_step_is_one_launch_and_counts_every_step_once(gpu):
    """300 unfused Adam steps over a list of 70 work chunks (most of them ragged): one launch
    per step, step_count == 300, and parameters and moments equal to the oracle's bit for bit --
    a step_count that advanced twice, or not at all, in any of the steps would change every
    later bias correction."""
    shapes = [(3, 5), (1, 9000), (7, 11), (60, 8192), (1, 1), (1, 8191), (2, 8193)]
    p0, g0 = H.randn_list(shapes, 31, 0.02), H.randn_list(shapes, 32, 1e-3)
    p_dev, g_dev = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
    plist, glist = nb.TensorList(p_dev), nb.TensorList(g_dev)
    opt = nb.Adam.new(1e-3, shapes).beta2(0.99)
    L = _lib.load()
    opt.step(plist, glist)
    _lib.check(L.nbo_profile_enable(1))
    for _ in range(299):
        opt.step(plist, glist)
    n = _launches(["nbo_update_f32_adam_self", "nbo_update_f32_adam", "nbo_prep"])
    _lib.check(L.nbo_profile_enable(0))
    assert n == {"nbo_update_f32_adam_self": 299, "nbo_update_f32_adam": 0, "nbo_prep": 0}
    assert opt.step_count() == 300
    pr, m, v, meta = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0), O.adam_meta(1e-3, beta2=0.99)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for _ in range(300):
            O.adam_step(meta, pr, g0, m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    H.assert_bits_equal(H.host_list(p_dev), pr, "params after 300 steps")
    H.assert_bits_equal(H.host_list(opt.moments()[0]), m, "m after 300 steps")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v after 300 steps")


def test_set_lr_load_meta_and_reset_between_one_launch_steps(gpu):
    """The one-launch step takes lr from the call's arguments and step_count from the device:
    set_lr, load_meta (step_count 41 -> the next step is the 42nd) and reset in between."""
    shapes = [(5, 2000), (1, 17)]
    p0, g0 = H.randn_list(shapes, 41, 0.02), H.randn_list(shapes, 42, 1e-3)
    p_dev, g_dev = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
    opt = nb.AdamW.new(1e-3, shapes).weight_decay(0.1)
    pr, m, v = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0)
    meta = O.adamw_meta(1e-3, weight_decay=0.1)
    O.set_pow_mode(O.POW_SQRT)
    try:
        def both(n):
            for _ in range(n):
                opt.step(p_dev, g_dev)
                O.adam_step(meta, pr, g0, m, v)

        both(3)
        opt.set_lr(5e-4)
        meta.lr = 5e-4
        both(2)
        mt = opt.meta()
        assert mt.step_count == 5
        mt.step_count = 41
        opt.load_meta(mt)
        meta.step_count = 41
        both(2)
        assert opt.step_count() == 43 == meta.step_count
        opt.reset()
        m, v = H.zeros_like_list(p0), H.zeros_like_list(p0)
        meta.step_count = 0
        both(2)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert opt.step_count() == 2
    H.assert_bits_equal(H.host_list(p_dev), pr, "params")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")


def test_grouped_fused_step_is_three_launches(gpu):
    """Two groups: norm pass + second stage + one update launch for both, no scalar-preparation launch."""
    names = ["w", "bias", "w2"]
    shapes = [(16, 600), (1, 600), (40, 300)]
    w0 = H.randn_list(shapes, 60, 0.02)
    p_dev = H.dev_list([O.bf16_from_f32(a) for a in w0], shapes)
    opt = G.GroupOptimizer.adamw_with_decay_exclusions(list(zip(names, p_dev)), 2e-4, 0.1, ["bias"], master=True)
    for gi, o in zip(opt.group_indices(), opt.group_optimizers()):
        for k, i in enumerate(gi):
            o.write_state(f"w{k}", H.to_dev(w0[i], shapes[i]))
    g_dev = H.dev_list([O.bf16_from_f32(a) for a in H.randn_list(shapes, 70, 1e-3 * 65536.0)], shapes)
    scaler = nb.GradScaler.new()
    opt.fused_step(p_dev, g_dev, scaler=scaler, max_norm=1.0)
    L = _lib.load()
    _lib.check(L.nbo_profile_enable(1))
    opt.fused_step(p_dev, g_dev, scaler=scaler, max_norm=1.0)
    n = _launches(["nbo_norm_bf16", "nbo_finalize", "nbo_update_bf16_adamw_self", "nbo_update_bf16_adamw", "nbo_prep"])
    _lib.check(L.nbo_profile_enable(0))
    assert n == {"nbo_norm_bf16": 1, "nbo_finalize": 1, "nbo_update_bf16_adamw_self": 1, "nbo_update_bf16_adamw": 0,
                 "nbo_prep": 0}
    assert [o.step_count() for o in opt.group_optimizers()] == [2, 2]


def test_nineteen_groups_of_their_own_hyper_parameters_in_two_launches(gpu):
    """Nineteen f32 AdamW groups, each with its own lr, weight decay and betas, plus tensors of
    ragged sizes: two update launches per step (sixteen groups, then three), every group's
    parameters and moments equal to the oracle's bit for bit after four clipped steps -- a group
    that took another group's scalars, range of workgroups or step_count would differ everywhere."""
    n_groups = 19
    names = [f"t{i}" for i in range(n_groups)] + ["rest0", "rest1"]
    shapes = [(1 + i % 3, 1000 + 977 * i) for i in range(n_groups)] + [(2, 8192), (1, 5)]
    w0 = H.randn_list(shapes, 300, 0.02)
    p_dev = H.dev_list(w0, shapes)
    cfgs = [G.ParamGroupConfig.adamw(f"g{i}", G.ParamSelector.Any([G.Equals(f"t{i}")]), 1e-3 * (1 + i), 0.01 * i)
            .betas(0.9 - 0.01 * i, 0.999 - 0.002 * i) for i in range(n_groups - 1)]
    last = G.ParamGroupConfig.adamw("rest", G.ParamSelector.All(), 5e-4, 0.3)
    opt = G.GroupOptimizer.from_named_params(list(zip(names, p_dev)), cfgs, last)
    idx = opt.group_indices()
    assert len(idx) == n_groups and idx[-1] == [18, 19, 20]
    metas = [O.adamw_meta(c.lr, beta1=c.beta1, beta2=c.beta2, weight_decay=c.weight_decay) for c in cfgs] + \
            [O.adamw_meta(5e-4, weight_decay=0.3)]
    ref = dict(w=H.copy_list(w0), m=H.zeros_like_list(w0), v=H.zeros_like_list(w0))
    L = _lib.load()
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(4):
            g = H.randn_list(shapes, 900 + 7 * step, 1e-2)
            _lib.check(L.nbo_profile_enable(1))
            opt.fused_step(p_dev, H.dev_list(g, shapes), max_norm=0.5)
            n = _launches(["nbo_norm_f32", "nbo_finalize", "nbo_update_f32_adamw_self", "nbo_prep"])
            _lib.check(L.nbo_profile_enable(0))
            assert n == {"nbo_norm_f32": 1, "nbo_finalize": 1, "nbo_update_f32_adamw_self": 2, "nbo_prep": 0}
            gf = H.copy_list(g)
            info = opt.last_step()

            def oracle_step():
                norm = O.clip_grad_norm(gf, 0.5)
                return True, norm

            H.oracle_step_with_device_norm(oracle_step, [gf], [], 0.5, info, f"19 groups, step {step}")
            assert info.clipped == 1
            for gi, meta in zip(idx, metas):
                O.adam_step(meta, [ref["w"][i] for i in gi], [gf[i] for i in gi],
                            [ref["m"][i] for i in gi], [ref["v"][i] for i in gi])
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert [o.step_count() for o in opt.group_optimizers()] == [4] * n_groups
    H.assert_bits_equal(H.host_list(p_dev), ref["w"], "params")
    state = dict(opt.state_tensors())
    for gno, gi in enumerate(idx):
        for k, i in enumerate(gi):
            H.assert_bits_equal([H.to_host(state[f"g{gno}.m{k}"])], [ref["m"][i]], f"g{gno}.m{k}")
            H.assert_bits_equal([H.to_host(state[f"g{gno}.v{k}"])], [ref["v"][i]], f"g{gno}.v{k}")


@pytest.mark.parametrize("grouped", [False, True])
def test_a_skipped_step_leaves_zeros_in_the_gradients_when_asked_to(gpu, grouped):
    """GradScaler::unscale_and_update replaces every gradient by zeros when it finds inf / NaN
    (core.rs:372-375).  With NBO_STEP_ZERO_ON_SKIP the fused step leaves exactly what the oracle's
    unscale_and_update leaves; without it the gradients stay as they were; a step that is not
    skipped never touches them."""
    names = ["w", "bias", "w2"]
    shapes = [(16, 600), (1, 600), (3, 8200)]
    w0 = H.randn_list(shapes, 80, 0.02)
    p_bits = [O.bf16_from_f32(a) for a in w0]
    g_bits = [O.bf16_from_f32(a) for a in H.randn_list(shapes, 81, 1e-3 * 65536.0)]
    g_bad = [b.copy() for b in g_bits]
    g_bad[2][8199] = 0x7FC0  # NaN
    p_dev = H.dev_list(p_bits, shapes)
    if grouped:
        opt = G.GroupOptimizer.adamw_with_decay_exclusions(list(zip(names, p_dev)), 2e-4, 0.1, ["bias"], master=True)
        for gi, o in zip(opt.group_indices(), opt.group_optimizers()):
            for k, i in enumerate(gi):
                o.write_state(f"w{k}", H.to_dev(w0[i], shapes[i]))
        counts = lambda: [o.step_count() for o in opt.group_optimizers()]  # noqa: E731
    else:
        opt = nb.AdamW.new(2e-4, shapes, master=True).weight_decay(0.1)
        for i, a in enumerate(w0):
            opt.write_state(f"w{i}", H.to_dev(a, shapes[i]))
        counts = lambda: [opt.step_count()]  # noqa: E731
    scaler = nb.GradScaler.new()

    # not asked to: the gradients stay, NaN included
    g_dev = H.dev_list(g_bad, shapes)
    opt.fused_step(p_dev, g_dev, scaler=scaler, max_norm=1.0)
    H.assert_bits_equal(H.host_list(g_dev), g_bad, "gradients of a skipped step without the flag")
    # asked to: what the oracle's unscale_and_update leaves
    s = O.default_scaler()
    s.scale = scaler.state().scale
    ref = [b.copy() for b in g_bad]
    assert O.scaler_unscale_and_update(s, ref) is False
    assert all(not r.any() for r in ref)
    opt.fused_step(p_dev, g_dev, scaler=scaler, max_norm=1.0, zero_on_skip=True)
    H.assert_bits_equal(H.host_list(g_dev), ref, "gradients of a skipped step with the flag")
    assert set(counts()) == {0} and scaler.state().scale == s.scale == 16384.0
    H.assert_bits_equal(H.host_list(p_dev), p_bits, "parameters after two skipped steps")
    # a step that runs leaves the gradients alone
    g_dev = H.dev_list(g_bits, shapes)
    opt.fused_step(p_dev, g_dev, scaler=scaler, max_norm=1.0, zero_on_skip=True)
    H.assert_bits_equal(H.host_list(g_dev), g_bits, "gradients of a step that ran")
    assert set(counts()) == {1}
