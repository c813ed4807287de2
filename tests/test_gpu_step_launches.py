"""How many launches a step is, and what a skipped step leaves behind.

The reference's `Adam::step` / `AdamW::step` is one call (alg.rs:109-150, 254-291): here it is
one launch of a kernel that prepares its own per-step scalars and advances step_count exactly
once; a grouped fused step is the norm pass, its second stage and ONE update launch for up to
sixteen groups of one optimizer kind (each with its own hyper-parameters, optim/groups.rs:269-293).
Lists of middle size (512 to 131071 work chunks, nine in ten of them whole) take the update
kernels that run one workgroup per row of a chunk; unfused, those follow the scalar-preparation
launch.
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


def test_a_list_of_middle_size_takes_the_by_row_kernels(gpu):
    """700 work chunks, most of them whole, one tensor ragged and one tiny: the unfused Adam step
    is the scalar preparation plus the by-row kernel, the fused AdamW step the norm pass, its
    second stage and the by-row kernel -- and both give the oracle's bits, step after step."""
    shapes = [(600, 8192), (1, 8192 * 99 + 4099), (3, 5)]
    p0, g0 = H.randn_list(shapes, 131, 0.02), H.randn_list(shapes, 132, 1e-3)
    L = _lib.load()
    O.set_pow_mode(O.POW_SQRT)
    try:
        # unfused Adam
        p_dev, g_dev = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
        opt = nb.Adam.new(1e-3, shapes)
        meta = O.adam_meta(1e-3)
        ref, m, v = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0)
        for step in range(3):
            _lib.check(L.nbo_profile_enable(1))
            opt.step(p_dev, g_dev)
            n = _launches(["nbo_prep", "nbo_update_f32_adam_rows", "nbo_update_f32_adam_self", "nbo_update_f32_adam"])
            _lib.check(L.nbo_profile_enable(0))
            assert n == {"nbo_prep": 1, "nbo_update_f32_adam_rows": 1, "nbo_update_f32_adam_self": 0,
                         "nbo_update_f32_adam": 0}
            O.adam_step(meta, ref, g0, m, v)
        assert opt.step_count() == 3
        H.assert_bits_equal(H.host_list(p_dev), ref, "unfused Adam by row: params")
        H.assert_bits_equal(H.host_list(opt.moments()[0]), m, "m")
        H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")
        del opt

        # fused AdamW with clipping and gradient zeroing
        p_dev = H.dev_list(p0, shapes)
        opt = nb.AdamW.new(2e-4, shapes).beta2(0.95).weight_decay(0.1)
        meta = O.adamw_meta(2e-4, beta2=0.95, weight_decay=0.1)
        ref, m, v = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0)
        for step in range(3):
            g = H.randn_list(shapes, 140 + step, 1e-2)
            g_dev = H.dev_list(g, shapes)
            _lib.check(L.nbo_profile_enable(1))
            opt.fused_step(p_dev, g_dev, max_norm=0.5, zero_grads=True)
            n = _launches(["nbo_norm_f32", "nbo_finalize", "nbo_update_f32_adamw_rows", "nbo_update_f32_adamw", "nbo_prep"])
            _lib.check(L.nbo_profile_enable(0))
            assert n == {"nbo_norm_f32": 1, "nbo_finalize": 1, "nbo_update_f32_adamw_rows": 1, "nbo_update_f32_adamw": 0,
                         "nbo_prep": 0}
            info = opt.last_step()
            gf = H.copy_list(g)
            H.oracle_step_with_device_norm(lambda: (True, O.clip_grad_norm(gf, 0.5)), [gf], [], 0.5, info,
                                           f"by-row fused step {step}")
            O.adam_step(meta, ref, gf, m, v)
            assert info.clipped == 1 and not any(t.any() for t in H.host_list(g_dev))
        H.assert_bits_equal(H.host_list(p_dev), ref, "fused AdamW by row: params")
        H.assert_bits_equal(H.host_list(opt.moments()[0]), m, "m")
        H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")
    finally:
        O.set_pow_mode(O.POW_LIBM)


def test_a_list_of_many_small_tensors_runs_by_row_over_the_rows_that_exist(gpu):
    """700 tensors of 1 to 30000 elements (hardly a whole chunk among them): the optimizer's layout
    carries a map of the rows that exist, the by-row kernels are launched with exactly that many
    workgroups, and mixed-precision AdamW (scaler, clip, one step skipped for an inf) and SGD with
    momentum give the oracle's bits."""
    from nabla_amd.workloads import ragged_sizes

    sizes = ragged_sizes(700, 1, 30000, seed=77)
    shapes = [(1, n) for n in sizes]
    w0 = H.randn_list(shapes, 500, 0.02)
    L = _lib.load()
    O.set_pow_mode(O.POW_SQRT)
    try:
        p_dev = H.dev_list([O.bf16_from_f32(a) for a in w0], shapes)
        opt = nb.AdamW.new(2e-4, shapes, master=True).beta2(0.95).weight_decay(0.1)
        for i, a in enumerate(w0):
            opt.write_state(f"w{i}", H.to_dev(a, shapes[i]))
        scaler, s_ref = nb.GradScaler.new(), O.default_scaler()
        meta = O.adamw_meta(2e-4, beta2=0.95, weight_decay=0.1)
        p_ref = [O.bf16_from_f32(a) for a in w0]
        master, m, v = H.copy_list(w0), H.zeros_like_list(w0), H.zeros_like_list(w0)
        for step in range(4):
            g_bits = [O.bf16_from_f32(a) for a in H.randn_list(shapes, 600 + 13 * step, 1e-3 * 65536.0)]
            if step == 1:
                g_bits[5][0] = 0x7F80
            _lib.check(L.nbo_profile_enable(1))
            opt.fused_step(p_dev, H.dev_list(g_bits, shapes), scaler=scaler, max_norm=1.0)
            n = _launches(["nbo_update_bf16_adamw_rows", "nbo_update_bf16_adamw"])
            _lib.check(L.nbo_profile_enable(0))
            assert n == {"nbo_update_bf16_adamw_rows": 1, "nbo_update_bf16_adamw": 0}
            info = opt.last_step()
            H.oracle_step_with_device_norm(lambda: O.mixed_step(meta, s_ref, 1.0, p_ref, g_bits, master, m, v),
                                           [p_ref, master, m, v], [meta, s_ref], 1.0, info, f"ragged by row, step {step}")
            assert info.found_inf == (1 if step == 1 else 0)
        assert opt.step_count() == 3 == meta.step_count
        H.assert_bits_equal(H.host_list(p_dev), p_ref, "bf16 params")
        for name, ref in (("w", master), ("m", m), ("v", v)):
            H.assert_bits_equal([H.to_host(opt.read_state(f"{name}{i}")) for i in range(len(shapes))], ref, name)
        del opt

        p0, g0 = H.randn_list(shapes, 700, 0.05), H.randn_list(shapes, 800, 1e-2)
        p_dev, g_dev = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
        sgd = nb.Sgd.new(0.05, shapes).momentum(0.9).weight_decay(0.01)
        smeta = O.sgd_meta(0.05, momentum=0.9, weight_decay=0.01)
        ref, vel = H.copy_list(p0), H.zeros_like_list(p0)
        for _ in range(3):
            sgd.step(p_dev, g_dev)
            O.sgd_step(smeta, ref, g0, vel)
        H.assert_bits_equal(H.host_list(p_dev), ref, "Sgd over the ragged list")
    finally:
        O.set_pow_mode(O.POW_LIBM)


def test_grids_folded_into_two_dimensions_cover_every_row_once(gpu):
    """One grid dimension holds fewer than 2^32 threads, so the launches that run one workgroup per
    row of a chunk fold a larger grid into two dimensions.  With NBO_GRID_X_MAX=37 in the
    environment (a test hook of the runtime) every such launch here is folded, its last grid row
    partly unused: the element-wise passes (the accumulating micro-batch with its per-piece sums
    among them), the cast, SGD and the by-row Adam kernels must still do every row exactly once."""
    import os
    import subprocess
    import sys

    code = r"""
import numpy as np, torch
import oracle as O
from nabla_amd import _lib, optim as nb, backend as B
from tests import helpers as H
_lib.init()
shapes = [(520, 8192), (1, 8192 * 3 + 4099), (3, 5)]
p0, g0 = H.randn_list(shapes, 231, 0.02), H.randn_list(shapes, 232, 1e-3)
O.set_pow_mode(O.POW_SQRT)
# element-wise passes
a, g = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
nb.scale_grad(g, 0.3)
sg = H.copy_list(g0); O.scale_grad(sg, 0.3)
H.assert_bits_equal(H.host_list(g), sg, "scale_grad")
nb.accumulate(a, g, True)
H.assert_bits_equal(H.host_list(a), [O.add(x, y) for x, y in zip(p0, sg)], "accumulate")
assert not any(t.any() for t in H.host_list(g))
out = [torch.zeros_like(t) for t in a]
B.add(H.dev_list(p0, shapes), H.dev_list(g0, shapes), out=out)
H.assert_bits_equal(H.host_list(out), [O.add(x, y) for x, y in zip(p0, g0)], "backend add")
# the accumulating micro-batch with its sum of squares: one partial sum per piece, more pieces
# than the second stage adds up itself
a, g = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
ok, sumsq = nb.unscale_accumulate(a, g)
acc = [O.add(x, y) for x, y in zip(p0, g0)]
H.assert_bits_equal(H.host_list(a), acc, "unscale_accumulate")
import math
exact = math.fsum(np.concatenate([np.square(x.astype(np.float64)).ravel() for x in acc]).tolist())
assert ok and abs(sumsq - exact) <= 1e-14 * exact, (sumsq, exact)
half = H.dev_list([np.zeros(x.shape, dtype=np.uint16) for x in p0], shapes)
B.cast(H.dev_list(p0, shapes), half)
H.assert_bits_equal(H.host_list(half), [O.bf16_from_f32(x) for x in p0], "cast")
# SGD with momentum, three steps
p, g = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
opt = nb.Sgd.new(0.05, shapes).momentum(0.9).weight_decay(0.01)
meta = O.sgd_meta(0.05, momentum=0.9, weight_decay=0.01)
ref, vel = H.copy_list(p0), H.zeros_like_list(p0)
for _ in range(3):
    opt.step(p, g); O.sgd_step(meta, ref, g0, vel)
H.assert_bits_equal(H.host_list(p), ref, "Sgd")
# Adam by row (unfused: preparation + by-row kernel), three steps
p = H.dev_list(p0, shapes)
opt = nb.Adam.new(1e-3, shapes)
meta = O.adam_meta(1e-3)
ref, m, v = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0)
for _ in range(3):
    opt.step(p, g); O.adam_step(meta, ref, g0, m, v)
H.assert_bits_equal(H.host_list(p), ref, "Adam")
H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")
print("folded ok")
"""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, NBO_GRID_X_MAX="37", PYTHONPATH=root)
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300, cwd=root, env=env)
    assert r.returncode == 0 and "folded ok" in r.stdout, r.stdout[-2000:] + r.stderr[-3000:]
