"""Optimizer<bf16> and Optimizer<f16> -- tensors, moments and arithmetic all in the 16-bit
type (every operation the f32 operation followed by T::from_f32,
nabla-core/src/common/scalar/mod.rs:253-351) -- against the CPU oracle's bf16 / f16
instantiations of the same pass chains.  Bit-exact against the oracle variant that takes
sqrt for powf(x, 0.5); against the libm variant the parameters stay within 1 ulp of the
16-bit type per step and the moments are identical.

The f16 cases use eps = 1e-3: the default 1e-8 is zero in f16 (below 2^-25), and a
division 0 / 0 gives NaNs whose sign differs between x86 and the GPU."""
import numpy as np
import pytest

import oracle as O
from nabla_amd import optim as nb
from tests import helpers as H

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (1, 3), (3, 5), (1, 4097), (64, 130), (1, 8191), (1, 8192), (1, 8193), (0, 5), (33, 1000)]


HALVES = ["bf16", "f16"]
EPS = {"bf16": 1e-8, "f16": 1e-3}


def _sqrt_mode(fn):
    O.set_pow_mode(O.POW_SQRT)
    try:
        return fn()
    finally:
        O.set_pow_mode(O.POW_LIBM)


@pytest.mark.parametrize("half", HALVES)
@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_half_adam_steps_bit_exact(gpu, kind, half):
    _bf = lambda arrs: H.narrow_list(arrs, half)  # noqa: E731
    eps = EPS[half]
    p0 = _bf(H.randn_list(SHAPES, 7000, 0.5))
    p_dev = H.dev_list(p0, SHAPES)
    if kind == "adam":
        opt, meta = nb.Adam.new(1e-2, SHAPES, dtype=half).eps(eps), O.adam_meta(1e-2, 0.9, 0.999, eps)
    else:
        opt = nb.AdamW.new(1e-2, SHAPES, dtype=half).beta2(0.95).weight_decay(0.1).eps(eps)
        meta = O.adamw_meta(1e-2, 0.9, 0.95, eps, 0.1)
    pr, m, v = H.copy_list(p0), [np.zeros_like(a) for a in p0], [np.zeros_like(a) for a in p0]
    pl, ml, vl = H.copy_list(p0), H.copy_list(m), H.copy_list(v)
    meta_l = O.Meta.from_buffer_copy(meta)
    for step in range(8):
        g = _bf(H.randn_list(SHAPES, 7100 + 13 * step, 1e-2))
        opt.step(p_dev, H.dev_list(g, SHAPES))
        _sqrt_mode(lambda: O.adam_step(meta, pr, g, m, v))
        O.adam_step(meta_l, pl, g, ml, vl)
    assert opt.step_count() == 8
    H.assert_bits_equal(H.host_list(p_dev), pr, "params")
    H.assert_bits_equal(H.host_list(opt.moments()[0]), m, "m")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")
    # the libm lowering of powf: same moments, parameters within 1 ulp per step taken
    H.assert_bits_equal(m, ml, "m, libm variant")
    H.assert_bits_equal(v, vl, "v, libm variant")
    assert H.max_ulp_half(H.host_list(p_dev), pl) <= 8


@pytest.mark.parametrize("half", HALVES)
@pytest.mark.parametrize("momentum,wd", [(0.0, 0.0), (0.9, 0.01)])
def test_half_sgd_bit_exact(gpu, momentum, wd, half):
    _bf = lambda arrs: H.narrow_list(arrs, half)  # noqa: E731
    p0 = _bf(H.randn_list(SHAPES, 7200, 0.5))
    p_dev = H.dev_list(p0, SHAPES)
    opt = nb.Sgd.new(0.05, SHAPES, dtype=half).momentum(momentum).weight_decay(wd)
    meta = O.sgd_meta(0.05, momentum=momentum, weight_decay=wd)
    pr, vel = H.copy_list(p0), [np.zeros_like(a) for a in p0]
    for step in range(6):
        g = _bf(H.randn_list(SHAPES, 7300 + step, 0.1))
        opt.step(p_dev, H.dev_list(g, SHAPES))
        O.sgd_step(meta, pr, g, vel)
    H.assert_bits_equal(H.host_list(p_dev), pr, "params")
    H.assert_bits_equal(H.host_list(opt.velocity()), vel, "velocity")


@pytest.mark.parametrize("half", HALVES)
def test_half_fused_step_with_a_scale_that_is_not_a_power_of_two(gpu, half):
    """scale 3 * 2^k makes T(1/scale) inexact and the unscaled gradients rounded 16-bit
    values, so the 16-bit unscale, norm, clip factor and update all have to round where the
    reference does; every fourth step carries an inf and is skipped."""
    _bf = lambda arrs: H.narrow_list(arrs, half)  # noqa: E731
    eps = EPS[half]
    p0 = _bf(H.randn_list(SHAPES, 7400, 0.5))
    p_dev = H.dev_list(p0, SHAPES)
    opt = nb.AdamW.new(1e-2, SHAPES, dtype=half).beta2(0.95).weight_decay(0.1).eps(eps)
    scaler = nb.GradScaler.new()
    scaler.load_state(nb.GradScalerState(3.0 * 256.0, 2.0, 0.5, 2, 0))
    meta, st = O.adamw_meta(1e-2, 0.9, 0.95, eps, 0.1), O.ScalerState(3.0 * 256.0, 2.0, 0.5, 2, 0)
    pr, m, v = H.copy_list(p0), [np.zeros_like(a) for a in p0], [np.zeros_like(a) for a in p0]
    for step in range(9):
        g32 = [a * np.float32(st.scale) for a in H.randn_list(SHAPES, 7500 + step, 1e-2)]
        if step % 4 == 3:
            g32[4][11] = np.inf
        g = _bf(g32)
        opt.fused_step(p_dev, H.dev_list(g, SHAPES), scaler=scaler, max_norm=0.5)
        info = opt.last_step()
        gr = H.copy_list(g)
        ok = O.scaler_unscale_and_update(st, gr)
        assert info.found_inf == (0 if ok else 1), step
        if ok:
            norm = O.clip_grad_norm(gr, 0.5)
            # the device adds the exact f64 squares block-wise, the reference serially
            assert abs(info.norm - norm) <= 1e-13 * norm and info.clipped == int(norm > 0.5), step
            _sqrt_mode(lambda: O.adam_step(meta, pr, gr, m, v))
        assert info.scale == st.scale and info.step_count == meta.step_count, step
    assert meta.step_count == 7
    H.assert_bits_equal(H.host_list(p_dev), pr, "params")
    H.assert_bits_equal(H.host_list(opt.moments()[0]), m, "m")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")


@pytest.mark.parametrize("half", HALVES)
def test_half_in_place_unscale_clip_and_scale_grad(gpu, half):
    _bf = lambda arrs: H.narrow_list(arrs, half)  # noqa: E731
    g0 = _bf([a * np.float32(700.0) for a in H.randn_list(SHAPES, 7600, 1e-2)])
    g_dev = H.dev_list(g0, SHAPES)
    scaler = nb.GradScaler.new()
    scaler.load_state(nb.GradScalerState(700.0, 2.0, 0.5, 5, 0))
    st = O.ScalerState(700.0, 2.0, 0.5, 5, 0)
    gr = H.copy_list(g0)
    assert scaler.unscale_and_update(g_dev) and O.scaler_unscale_and_update(st, gr)
    H.assert_bits_equal(H.host_list(g_dev), gr, "unscaled")
    norm = O.clip_grad_norm(gr, 0.25)
    assert abs(nb.clip_grad_norm(g_dev, 0.25) - norm) <= 1e-13 * norm
    H.assert_bits_equal(H.host_list(g_dev), gr, "clipped")
    nb.scale_grad(g_dev, 1.0 / 3.0)
    O.scale_grad(gr, 1.0 / 3.0)
    H.assert_bits_equal(H.host_list(g_dev), gr, "scale_grad")
    bad = H.copy_list(g0)
    bad[3][5] = 0x7FC0 if half == "bf16" else np.nan
    bad_dev = H.dev_list(bad, SHAPES)
    assert not scaler.unscale_and_update(bad_dev)
    assert not any(t.any() for t in H.host_list(bad_dev))
    assert scaler.state().scale == 350.0


@pytest.mark.parametrize("half", HALVES)
def test_half_state_export_import_and_dtype_rules(gpu, half):
    import torch

    _bf = lambda arrs: H.narrow_list(arrs, half)  # noqa: E731
    tdt = {"bf16": torch.bfloat16, "f16": torch.float16}[half]
    shapes = [(2, 3), (1, 5000)]
    opt = nb.AdamW.new(1e-2, shapes, dtype=half).eps(EPS[half])
    p = H.dev_list(_bf(H.randn_list(shapes, 7700, 0.5)), shapes)
    opt.step(p, H.dev_list(_bf(H.randn_list(shapes, 7701, 1e-2)), shapes))
    tensors = opt.state_tensors()
    assert [n for n, _ in tensors] == ["m0", "m1", "v0", "v1"]
    assert all(t.dtype == tdt for _, t in tensors)
    other = nb.AdamW.new(1e-2, shapes, dtype=half)
    other.load_state_tensors(tensors)
    H.assert_bits_equal(H.host_list(other.moments()[1]), H.host_list(opt.moments()[1]), "v round trip")
    # neither f32 tensors nor those of the other 16-bit type go into this optimizer, and master
    # weights need f32 state
    with pytest.raises(Exception, match="element type"):
        opt.step(H.dev_list(H.randn_list(shapes, 1, 1.0), shapes), H.dev_list(H.randn_list(shapes, 2, 1.0), shapes))
    wrong = "f16" if half == "bf16" else "bf16"
    with pytest.raises(Exception, match="keep_master|element type"):
        opt.step(H.dev_list(H.narrow_list(H.randn_list(shapes, 1, 1.0), wrong), shapes),
                 H.dev_list(H.narrow_list(H.randn_list(shapes, 2, 1.0), wrong), shapes))
    with pytest.raises(ValueError, match="master"):
        nb.AdamW.new(1e-2, shapes, dtype=half, master=True)
