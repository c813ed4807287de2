"""Parity of the gfx950 engine (through the C ABI) against the CPU oracle on the same
seeded inputs.

Bars (stated by the benchmark contract):
  * integer / decision state -- found_inf, skipped, scale bits, step_count: bit-exact;
  * f32 state (m, v, master, f32 params): within 2 ulp of the oracle that follows the
    reference's libm powf; bit-exact against the oracle variant that takes sqrt for
    powf(x, 0.5) (the only operation where the device deliberately differs);
  * bf16 params: within 1 bf16 ulp (bit-exact against the sqrt variant).
For parameters the 2-ulp bar has one documented escape: when p*(1-wd*lr) and the
update nearly cancel, a 1-ulp change of the update is many ulps of the tiny result;
such an element must instead satisfy |delta| <= steps * 8 * lr * 2^-23.
"""
import numpy as np
import pytest

import oracle as O
from nabla_amd import optim as nb
from tests import helpers as H

pytestmark = pytest.mark.gpu

# sizes around the engine's work-chunk (8192 elements) and vector (4 / 8 elements)
# boundaries, an empty tensor, and a few ordinary ones
RAGGED = [(1, 1), (1, 3), (3, 5), (1, 4095), (1, 4097), (64, 130), (7, 1171), (1, 8191), (1, 8192),
          (1, 8193), (1, 16385), (0, 5), (33, 1000)]


def _param_close(p_dev, p_ref, lr, steps, what):
    """2 ulp, or the documented cancellation bound; how often the bound was needed is counted,
    printed (pytest -s shows it) and capped."""
    return H.tolerance_report(p_dev, p_ref, lr, steps, what)


# ---- config 1: plain SGD on the README MLP parameter set, 100 steps ---------------------

def test_sgd_mlp_100_steps_bit_exact(gpu):
    shapes = H.MLP_SHAPES
    p_ref = H.randn_list(shapes, 100, 0.05)
    p_dev = H.dev_list(p_ref, shapes)
    vel = H.zeros_like_list(p_ref)
    opt = nb.Sgd.new(0.01, shapes)
    meta = O.sgd_meta(0.01)
    for step in range(100):
        g = H.randn_list(shapes, 10_000 + 97 * step, 1e-2)
        g_dev = H.dev_list(g, shapes)
        opt.step(p_dev, g_dev)
        O.sgd_step(meta, p_ref, g, vel)
    H.assert_bits_equal(H.host_list(p_dev), p_ref, "SGD params after 100 steps")


def test_step_with_vars_takes_params_from_the_module_and_grads_from_the_variables(gpu):
    """Optimizer::step_with_vars (optim/core.rs:18-39) on the reference's SGD known
    answer (tests/optim.rs:47-57): p = 1, g = 1, lr = 0.1 gives 0.9."""
    class Module:
        def __init__(self, params):
            self.params = params

        def parameters_mut(self):
            return self.params

    class Var:
        def __init__(self, grad):
            self._grad = grad

        def grad(self):
            return self._grad

    one = np.ones(1, dtype=np.float32)
    module = Module([H.to_dev(one, (1, 1))])
    nb.Sgd.new(0.1, [(1, 1)]).step_with_vars(module, [Var(H.to_dev(one, (1, 1)))])
    assert H.to_host(module.params[0])[0] == np.float32(1.0) + np.float32(-0.1) * np.float32(1.0)
    assert abs(float(H.to_host(module.params[0])[0]) - 0.9) < 1e-6


@pytest.mark.parametrize("momentum,wd", [(0.9, 0.0), (0.0, 0.01), (0.9, 0.01)])
def test_sgd_momentum_weight_decay_bit_exact(gpu, momentum, wd):
    shapes = RAGGED
    p_ref = H.randn_list(shapes, 7, 0.05)
    p_dev = H.dev_list(p_ref, shapes)
    vel = H.zeros_like_list(p_ref)
    opt = nb.Sgd.new(0.05, shapes).momentum(momentum).weight_decay(wd)
    meta = O.sgd_meta(0.05, momentum, wd)
    for step in range(5):
        g = H.randn_list(shapes, 500 + 31 * step, 1e-2)
        opt.step(p_dev, H.dev_list(g, shapes))
        O.sgd_step(meta, p_ref, g, vel)
    H.assert_bits_equal(H.host_list(p_dev), p_ref, "SGD params")
    H.assert_bits_equal(H.host_list(opt.velocity()), vel, "SGD velocity")


# ---- Adam / AdamW, T = f32 ----------------------------------------------------------------

@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_adam_f32_ragged_10_steps(gpu, kind):
    shapes = RAGGED
    lr, steps = 3e-4, 10
    p0 = H.randn_list(shapes, 11, 0.02)
    p_dev = H.dev_list(p0, shapes)
    if kind == "adam":
        opt = nb.Adam.new(lr, shapes)
        metas = [O.adam_meta(lr), O.adam_meta(lr)]
    else:
        opt = nb.AdamW.new(lr, shapes).weight_decay(0.1).beta2(0.95)
        metas = [O.adamw_meta(lr, beta2=0.95, weight_decay=0.1) for _ in range(2)]
    refs = []
    for mode in (O.POW_LIBM, O.POW_SQRT):
        refs.append(dict(p=H.copy_list(p0), m=H.zeros_like_list(p0), v=H.zeros_like_list(p0)))
    for step in range(steps):
        g = H.randn_list(shapes, 900 + 13 * step, 1e-3)
        opt.step(p_dev, H.dev_list(g, shapes))
        for mode, ref, meta in zip((O.POW_LIBM, O.POW_SQRT), refs, metas):
            O.set_pow_mode(mode)
            O.adam_step(meta, ref["p"], g, ref["m"], ref["v"])
        O.set_pow_mode(O.POW_LIBM)
    m_dev, v_dev = (H.host_list(x) for x in opt.moments())
    p_host = H.host_list(p_dev)
    assert opt.step_count() == steps == metas[0].step_count
    # moments never see denom: bit-exact against both variants
    H.assert_bits_equal(m_dev, refs[0]["m"], "m vs libm-powf oracle")
    H.assert_bits_equal(v_dev, refs[0]["v"], "v vs libm-powf oracle")
    # sqrt variant: everything bit-exact
    H.assert_bits_equal(p_host, refs[1]["p"], "params vs sqrt-variant oracle")
    # reference-faithful libm powf: 2 ulp
    _param_close(p_host, refs[0]["p"], lr, steps, "params vs libm-powf oracle")


def test_adam_f64_bit_exact_vs_sqrt_variant(gpu):
    shapes = [(1, 1), (5, 7), (1, 4099)]
    p0 = H.randn_list(shapes, 3, 0.02, np.float64)
    p_dev = H.dev_list(p0, shapes)
    opt = nb.AdamW.new(1e-3, shapes, dtype="f64")
    meta = O.adamw_meta(1e-3)
    ref = dict(p=H.copy_list(p0), m=H.zeros_like_list(p0), v=H.zeros_like_list(p0))
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(4):
            g = H.randn_list(shapes, 40 + step, 1e-3, np.float64)
            opt.step(p_dev, H.dev_list(g, shapes))
            O.adam_step(meta, ref["p"], g, ref["m"], ref["v"])
    finally:
        O.set_pow_mode(O.POW_LIBM)
    m_dev, v_dev = (H.host_list(x) for x in opt.moments())
    H.assert_bits_equal(m_dev, ref["m"], "f64 m")
    H.assert_bits_equal(v_dev, ref["v"], "f64 v")
    H.assert_bits_equal(H.host_list(p_dev), ref["p"], "f64 params")


# ---- the fused Trainer tail: bf16 params/grads, f32 master/m/v -------------------------------

def _mixed_case(shapes, steps, lr, wd, max_norm, scaler_state, grad_sigma, inject=None, seed=1, half="bf16"):
    """Run `steps` fused steps on the device and the same Trainer tail on both oracle
    variants, with parameters and gradients of the 16-bit type `half` over f32 master
    weights and moments.  inject(step, grads_bits) may poison gradients in place.  Returns
    the device results and both references."""
    master0 = H.randn_list(shapes, seed, 0.02)
    p_bits0 = H.narrow_list(master0, half)
    p_dev = H.dev_list(p_bits0, shapes)
    opt = nb.AdamW.new(lr, shapes, master=True).beta2(0.95).weight_decay(wd)
    for i, a in enumerate(master0):
        opt.write_state(f"w{i}", H.to_dev(a, shapes[i]))
    scaler = None
    if scaler_state is not None:
        scaler = nb.GradScaler.new()
        scaler.load_state(nb.GradScalerState(**scaler_state))
    refs = []
    for _ in range(2):
        s = None
        if scaler_state is not None:
            s = O.ScalerState(scaler_state["scale"], scaler_state["growth_factor"],
                              scaler_state["backoff_factor"], scaler_state["growth_interval"],
                              scaler_state["consecutive_ok"])
        refs.append(dict(meta=O.adamw_meta(lr, beta2=0.95, weight_decay=wd), scaler=s,
                         p=H.copy_list(p_bits0), w=H.copy_list(master0),
                         m=H.zeros_like_list(master0), v=H.zeros_like_list(master0), trace=[]))
    scale_now = scaler_state["scale"] if scaler_state else 1.0
    for step in range(steps):
        g32 = H.randn_list(shapes, 5000 + 17 * step + seed, grad_sigma * scale_now)
        g_bits = H.narrow_list(g32, half)
        if inject is not None:
            inject(step, g_bits)
        g_dev = H.dev_list(g_bits, shapes)
        opt.fused_step(p_dev, g_dev, scaler=scaler, max_norm=max_norm)
        info = opt.last_step()
        for mode, ref in zip((O.POW_LIBM, O.POW_SQRT), refs):
            O.set_pow_mode(mode)
            # (if the device's tree-summed norm and the serial one give different clip factors,
            # the oracle repeats the step with the device's norm; counted and reported)
            ran, norm = H.oracle_step_with_device_norm(
                lambda: O.mixed_step(ref["meta"], ref["scaler"], max_norm, ref["p"], g_bits,
                                     ref["w"], ref["m"], ref["v"]),
                [ref["p"], ref["w"], ref["m"], ref["v"]], [ref["meta"], ref["scaler"]], max_norm, info,
                f"mixed case seed {seed} step {step}")
            ref["trace"].append((0 if ran else 1, ref["scaler"].scale if ref["scaler"] else 0.0,
                                 ref["meta"].step_count, norm))
        O.set_pow_mode(O.POW_LIBM)
        if refs[0]["scaler"] is not None:
            scale_now = refs[0]["scaler"].scale
    dev = dict(p=H.host_list(p_dev), w=H.host_list([opt.read_state(f"w{i}") for i in range(len(shapes))]),
               m=H.host_list(opt.moments()[0]), v=H.host_list(opt.moments()[1]),
               trace=[(t.found_inf, t.scale, t.step_count, t.norm, t.clipped) for t in opt.trace()],
               scaler=scaler.state() if scaler else None, step_count=opt.step_count())
    return dev, refs


def _check_mixed(dev, refs, lr, steps):
    libm, sq = refs
    # decisions: bit-exact
    assert [t[0] for t in dev["trace"]] == [t[0] for t in libm["trace"]], "found_inf / skip sequence"
    assert [np.float64(t[1]).tobytes() for t in dev["trace"]] == \
           [np.float64(t[1]).tobytes() for t in libm["trace"]], "loss-scale sequence"
    assert [t[2] for t in dev["trace"]] == [t[2] for t in libm["trace"]], "step_count sequence"
    assert dev["step_count"] == libm["meta"].step_count
    if dev["scaler"] is not None:
        assert dev["scaler"].scale == libm["scaler"].scale
        assert dev["scaler"].consecutive_ok == libm["scaler"].consecutive_ok
    # norm: tree-summed on the device, serial in the reference -> a few f64 ulp
    for d, r in zip(dev["trace"], libm["trace"]):
        assert d[3] == pytest.approx(r[3], rel=1e-12, abs=0.0)
    # the clip factor is f32(max_norm / norm): where the two norms round to different factors
    # the oracle has followed the device's norm (H.oracle_step_with_device_norm), so everything
    # downstream is bit-comparable
    H.assert_bits_equal(dev["m"], sq["m"], "m vs sqrt-variant oracle")
    H.assert_bits_equal(dev["v"], sq["v"], "v vs sqrt-variant oracle")
    H.assert_bits_equal(dev["w"], sq["w"], "master vs sqrt-variant oracle")
    H.assert_bits_equal(dev["p"], sq["p"], "16-bit params vs sqrt-variant oracle")
    H.assert_bits_equal(dev["m"], libm["m"], "m vs libm-powf oracle")
    H.assert_bits_equal(dev["v"], libm["v"], "v vs libm-powf oracle")
    _param_close(dev["w"], libm["w"], lr, steps, "master vs libm-powf oracle")
    assert H.max_ulp_half(dev["p"], libm["p"]) <= 1, "16-bit params vs libm-powf oracle"


def test_mixed_adamw_scaler_clip_llama_like(gpu):
    # a scaled-down Llama block: same tensor roles as the 1.1B / 8B configs
    shapes = H.llama_shapes(2, 256, 64, 704, 1000)
    scaler = dict(scale=65536.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=2000,
                  consecutive_ok=0)
    dev, refs = _mixed_case(shapes, 10, 2e-4, 0.1, 1.0, scaler, 1e-3)
    assert all(t[4] == 1 for t in dev["trace"]), "this case is meant to clip every step"
    _check_mixed(dev, refs, 2e-4, 10)


def test_mixed_adamw_no_clip_no_scaler(gpu):
    dev, refs = _mixed_case(RAGGED, 4, 1e-3, 0.01, 0.0, None, 1e-3)
    _check_mixed(dev, refs, 1e-3, 4)


def test_mixed_f16_adamw_with_dynamic_loss_scale(gpu):
    """f16 parameters and gradients over f32 master weights -- what a GradScaler is for:
    gradients that only survive f16 because they are scaled, an overflow to inf every fifth
    step (the scale backs off, the step is skipped), growth every 3 clean steps."""
    shapes = H.llama_shapes(2, 256, 64, 704, 1000) + RAGGED

    def inject(step, g):
        if step % 5 == 4:
            g[3].view(np.uint16)[7] = [0x7C00, 0xFC00, 0x7E01][(step // 5) % 3]

    scaler = dict(scale=65536.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=3, consecutive_ok=0)
    # sigma 1e-6: most unscaled gradients would be f16 subnormals or zero
    dev, refs = _mixed_case(shapes, 12, 2e-4, 0.1, 1.0, scaler, 1e-6, inject=inject, seed=3, half="f16")
    _check_mixed(dev, refs, 2e-4, 12)
    assert [t[0] for t in dev["trace"]] == [1 if s % 5 == 4 else 0 for s in range(12)]
    assert dev["p"][0].dtype == np.float16 and dev["step_count"] == 10


def test_fused_steps_are_reproducible_run_to_run(gpu):
    """The norm is reduced in a fixed order (fixed grid, butterfly inside a wave, waves
    and blocks in index order), so two runs over the same inputs agree in every bit,
    the reported norms included."""
    shapes = RAGGED + [(257, 1023), (1, 70001)]
    state = dict(scale=1024.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=3, consecutive_ok=0)
    a, _ = _mixed_case(shapes, 6, 2e-4, 0.1, 0.5, state, 1e-3, seed=9)
    b, _ = _mixed_case(shapes, 6, 2e-4, 0.1, 0.5, state, 1e-3, seed=9)
    for key in ("p", "w", "m", "v"):
        H.assert_bits_equal(a[key], b[key], key)
    assert [np.float64(t[3]).tobytes() for t in a["trace"]] == [np.float64(t[3]).tobytes() for t in b["trace"]]
    assert a["trace"] == b["trace"]


def test_dynamic_loss_scale_ragged_trace_bit_exact(gpu):
    """Config 4 at reduced tensor count: ragged sizes, growth every 4 clean steps,
    inf/NaN injected every 4th step (scale only backs off) and, in a second run,
    every 5th step (scale also grows)."""
    sizes = H.ragged_sizes(256, 1, 65536, seed=99)
    shapes = [(1, n) for n in sizes]
    total = sum(sizes)
    rng = np.random.default_rng(5)
    for period, steps in ((4, 16), (5, 15)):
        def inject(step, g_bits, period=period):
            if step % period != period - 1:
                return
            k = max(1, int(total * 1e-6))
            for _ in range(k):
                t = int(rng.integers(len(g_bits)))
                e = int(rng.integers(g_bits[t].size))
                g_bits[t][e] = [0x7F80, 0xFF80, 0x7FC1][int(rng.integers(3))]

        scaler = dict(scale=65536.0, growth_factor=2.0, backoff_factor=0.5, growth_interval=4,
                      consecutive_ok=0)
        dev, refs = _mixed_case(shapes, steps, 2e-4, 0.1, 1.0, scaler, 1e-3, inject=inject, seed=period)
        _check_mixed(dev, refs, 2e-4, steps)
        skipped = [t[0] for t in dev["trace"]]
        assert sum(skipped) == steps // period
        if period == 4:
            # closed form: only 3 clean steps fit between injections, the scale never grows
            assert dev["scaler"].scale == 65536.0 * 0.5 ** (steps // 4)
            assert dev["step_count"] == steps - steps // 4
        else:
            # 4 clean steps, then growth (x2), then the injected step halves it again
            assert dev["scaler"].scale == 65536.0


def test_fused_f32_grads_with_scaler(gpu):
    """T = f32 throughout (no master): the fused path against the in-place reference tail."""
    shapes = RAGGED
    lr = 3e-4
    p0 = H.randn_list(shapes, 21, 0.02)
    p_dev = H.dev_list(p0, shapes)
    opt = nb.Adam.new(lr, shapes)
    scaler = nb.GradScaler.new()
    ref = dict(p=H.copy_list(p0), m=H.zeros_like_list(p0), v=H.zeros_like_list(p0))
    meta, s = O.adam_meta(lr), O.default_scaler()
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(5):
            g = H.randn_list(shapes, 300 + step, 1e-3 * 65536.0)
            if step == 2:
                g[3][17] = np.inf
            g_dev = H.dev_list(g, shapes)
            opt.fused_step(p_dev, g_dev, scaler=scaler, max_norm=0.5, zero_grads=True)
            O.f32_step(meta, s, 0.5, ref["p"], g, ref["m"], ref["v"])
            for t in H.host_list(g_dev):
                assert not t.any(), "NBO_STEP_ZERO_GRADS leaves zeros"
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert opt.step_count() == meta.step_count == 4
    assert scaler.state().scale == s.scale == 32768.0
    H.assert_bits_equal(H.host_list(p_dev), ref["p"], "f32 params")
    H.assert_bits_equal(H.host_list(opt.moments()[0]), ref["m"], "m")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), ref["v"], "v")


# ---- the unfused API: in-place GradScaler / clip_grad_norm / zero_grad ----------------------

def test_unfused_scaler_clip_zero_in_place(gpu):
    shapes = RAGGED
    g = H.randn_list(shapes, 77, 1e-3 * 65536.0)
    g_dev = H.dev_list(g, shapes)
    scaler = nb.GradScaler.new()
    s = O.default_scaler()
    assert scaler.unscale_and_update(g_dev) is True
    assert O.scaler_unscale_and_update(s, g) is True
    H.assert_bits_equal(H.host_list(g_dev), g, "unscaled grads")
    norm_dev = nb.clip_grad_norm(g_dev, 0.01)
    norm_ref = O.clip_grad_norm(g, 0.01)
    assert norm_dev == pytest.approx(norm_ref, rel=1e-13)
    assert norm_ref > 0.01
    H.assert_bits_equal(H.host_list(g_dev), g, "clipped grads")
    before = H.host_list(g_dev)
    assert nb.clip_grad_norm(g_dev, 1e9) == pytest.approx(norm_dev * (0.01 / norm_dev), rel=1e-6)
    H.assert_bits_equal(H.host_list(g_dev), before, "clip leaves grads alone when norm <= max_norm")
    assert nb.clip_grad_norm(g_dev, 0.0) == 0.0 and nb.clip_grad_norm(g_dev, -1.0) == 0.0
    nb.scale_grad(g_dev, 3.0)
    O.scale_grad(g, np.float32(3.0))
    H.assert_bits_equal(H.host_list(g_dev), g, "scale_grad")
    # inf: ok == False, grads zeroed, scale halved, counter reset
    g2 = H.copy_list(g)
    g2[5][100] = -np.inf
    g2_dev = H.dev_list(g2, shapes)
    assert scaler.unscale_and_update(g2_dev) is False
    assert O.scaler_unscale_and_update(s, g2) is False
    for t in H.host_list(g2_dev):
        assert not t.any()
    st = scaler.state()
    assert (st.scale, st.consecutive_ok) == (s.scale, s.consecutive_ok) == (32768.0, 0)
    nb.zero_grad(g_dev)
    for t in H.host_list(g_dev):
        assert not t.any()


# ---- HIP graph capture -----------------------------------------------------------------------

def test_fused_steps_replay_from_a_hip_graph(gpu):
    """A fused step allocates nothing, reads nothing back and keeps step_count and the
    scaler on the device, so a caller may capture it.  Two fused steps are captured once
    and replayed three times, with eager steps in between; after every replay the state
    is compared with the oracle stepping through the same sequence."""
    import torch

    from nabla_amd import _lib

    shapes = [(5, 7), (1, 8200), (3, 1000)]
    w0 = H.randn_list(shapes, 31, 0.02)
    g_bits = [O.bf16_from_f32(a) for a in H.randn_list(shapes, 32, 1e-3 * 65536.0)]
    p_dev = H.dev_list([O.bf16_from_f32(a) for a in w0], shapes)
    g_dev = H.dev_list(g_bits, shapes)
    opt = nb.AdamW.new(2e-4, shapes, master=True).beta2(0.95).weight_decay(0.1)
    for i, a in enumerate(w0):
        opt.write_state(f"w{i}", H.to_dev(a, shapes[i]))
    scaler = nb.GradScaler.new()
    scaler.load_state(nb.GradScalerState(65536.0, 2.0, 0.5, 3, 0))
    plist, glist = nb.TensorList(p_dev), nb.TensorList(g_dev)

    ref = dict(p=[O.bf16_from_f32(a) for a in w0], w=H.copy_list(w0), m=H.zeros_like_list(w0),
               v=H.zeros_like_list(w0))
    meta, s = O.adamw_meta(2e-4, 0.9, 0.95, 1e-8, 0.1), O.ScalerState(65536.0, 2.0, 0.5, 3, 0)

    def oracle_steps(k):
        O.set_pow_mode(O.POW_SQRT)
        try:
            for _ in range(k):
                O.mixed_step(meta, s, 1.0, ref["p"], g_bits, ref["w"], ref["m"], ref["v"])
        finally:
            O.set_pow_mode(O.POW_LIBM)

    def check(what):
        assert opt.step_count() == meta.step_count, what
        assert scaler.state().scale == s.scale and scaler.state().consecutive_ok == s.consecutive_ok, what
        H.assert_bits_equal(H.host_list(p_dev), ref["p"], what + ": params")
        H.assert_bits_equal(H.host_list(opt.moments()[1]), ref["v"], what + ": v")

    stream = torch.cuda.Stream()
    lib = _lib.load()
    _lib.check(lib.nbo_set_stream(stream.cuda_stream))
    try:
        with torch.cuda.stream(stream):
            opt.fused_step(plist, glist, scaler=scaler, max_norm=1.0)  # creates everything eagerly
            stream.synchronize()
            oracle_steps(1)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                opt.fused_step(plist, glist, scaler=scaler, max_norm=1.0)
                opt.fused_step(plist, glist, scaler=scaler, max_norm=1.0)
            stream.synchronize()
            check("capture must not execute")
            for replay in range(3):
                graph.replay()
                stream.synchronize()
                oracle_steps(2)
                check(f"replay {replay}")
                opt.fused_step(plist, glist, scaler=scaler, max_norm=1.0)  # eager, between replays
                stream.synchronize()
                oracle_steps(1)
                check(f"eager step after replay {replay}")
    finally:
        _lib.check(lib.nbo_set_stream(None))
    assert meta.step_count == 10 and s.scale == 65536.0 * 8


def test_reset_and_steps_replay_from_a_hip_graph(gpu):
    """Optimizer::reset clears the moments and step_count with a fill kernel (no memset
    nodes), so it can sit in a captured graph with the steps that follow it.  The graph
    [reset, step, step] is replayed twice with an eager step in between; the oracle does
    the same sequence."""
    import torch

    from nabla_amd import _lib

    shapes = [(3, 5), (1, 9000), (7, 11)]
    p0 = H.randn_list(shapes, 81, 0.02)
    g0 = H.randn_list(shapes, 82, 1e-3)
    p_dev, g_dev = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
    plist, glist = nb.TensorList(p_dev), nb.TensorList(g_dev)
    opt = nb.Adam.new(1e-3, shapes)
    pr, m, v, meta = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0), O.adam_meta(1e-3)

    def oracle(reset, steps):
        nonlocal m, v
        if reset:
            m, v = H.zeros_like_list(p0), H.zeros_like_list(p0)
            meta.step_count = 0
        O.set_pow_mode(O.POW_SQRT)
        try:
            for _ in range(steps):
                O.adam_step(meta, pr, g0, m, v)
        finally:
            O.set_pow_mode(O.POW_LIBM)

    def check(what):
        assert opt.step_count() == meta.step_count, what
        H.assert_bits_equal(H.host_list(p_dev), pr, what + ": params")
        H.assert_bits_equal(H.host_list(opt.moments()[0]), m, what + ": m")
        H.assert_bits_equal(H.host_list(opt.moments()[1]), v, what + ": v")

    stream = torch.cuda.Stream()
    lib = _lib.load()
    _lib.check(lib.nbo_set_stream(stream.cuda_stream))
    try:
        with torch.cuda.stream(stream):
            opt.step(plist, glist)
            opt.step(plist, glist)
            stream.synchronize()
            oracle(False, 2)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                opt.reset()
                opt.step(plist, glist)
                opt.step(plist, glist)
            stream.synchronize()
            check("capture must not execute")
            for replay in range(2):
                graph.replay()
                stream.synchronize()
                oracle(True, 2)
                check(f"replay {replay}")
                opt.step(plist, glist)
                stream.synchronize()
                oracle(False, 1)
                check(f"eager step after replay {replay}")
    finally:
        _lib.check(lib.nbo_set_stream(None))
    assert meta.step_count == 3


def test_adamw_step_free_function(gpu):
    """adamw_step (alg.rs:431-469): caller-held moments, step number passed in."""
    shape = (3, 1001)
    p0, g0 = H.randn_list([shape], 41, 0.02)[0], H.randn_list([shape], 42, 1e-3)[0]
    m0, v0 = np.abs(H.randn_list([shape], 43, 1e-4)[0]), np.abs(H.randn_list([shape], 44, 1e-7)[0])
    p, g, m, v = (H.to_dev(a, shape) for a in (p0, g0, m0, v0))
    nb.adamw_step(p, g, m, v, 1e-3, 0.9, 0.999, 1e-8, 0.01, 5)
    pr, mr, vr = p0.copy(), m0.copy(), v0.copy()
    O.set_pow_mode(O.POW_SQRT)
    try:
        O.adamw_step_single(pr, g0, mr, vr, 1e-3, 0.9, 0.999, 1e-8, 0.01, 5)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    H.assert_bits_equal([H.to_host(p), H.to_host(m), H.to_host(v)], [pr, mr, vr], "adamw_step")


def test_nan_policy_skip_without_scaler(gpu):
    """GradNanPolicy::Skip (trainer.rs:239-245, tests/trainer.rs:148-169): a non-finite
    gradient drops the step -- params, moments and step_count stay as they were -- and
    a finite one afterwards steps normally."""
    shapes = [(2, 3), (1, 5000)]
    p0 = H.randn_list(shapes, 51, 0.05)
    p = H.dev_list(p0, shapes)
    bad = H.randn_list(shapes, 52, 1e-2)
    bad[1][4321] = np.nan
    good = H.randn_list(shapes, 53, 1e-2)
    opt = nb.Adam.new(1e-3, shapes)
    opt.fused_step(p, H.dev_list(bad, shapes), skip_nonfinite=True)
    info = opt.last_step()
    assert (info.found_inf, info.step_count) == (1, 0)
    H.assert_bits_equal(H.host_list(p), p0, "params after a skipped step")
    assert not any(t.any() for t in H.host_list(opt.moments()[0]))
    opt.fused_step(p, H.dev_list(good, shapes), skip_nonfinite=True)
    pr, m, v, meta = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0), O.adam_meta(1e-3)
    O.set_pow_mode(O.POW_SQRT)
    try:
        O.adam_step(meta, pr, good, m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert opt.step_count() == 1
    H.assert_bits_equal(H.host_list(p), pr, "params after the next, finite step")
    # without the policy the reference steps on regardless (trainer.rs:249)
    opt2 = nb.Adam.new(1e-3, shapes)
    p2 = H.dev_list(p0, shapes)
    opt2.fused_step(p2, H.dev_list(bad, shapes))
    assert opt2.step_count() == 1 and np.isnan(H.to_host(p2[1])[4321])


def test_reset_set_lr_and_load_meta(gpu):
    """Optimizer::reset (alg.rs:152-162), set_lr (:164-166), OptimState::load_meta
    (:531-545) and load_state_tensors (:487-516) against the oracle doing the same."""
    shapes = [(1, 3), (2, 4500)]
    p0 = H.randn_list(shapes, 61, 0.02)
    grads = [H.randn_list(shapes, 62 + k, 1e-3) for k in range(6)]
    p = H.dev_list(p0, shapes)
    opt = nb.AdamW.new(1e-3, shapes).weight_decay(0.05)
    pr, m, v = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0)
    meta = O.adamw_meta(1e-3, weight_decay=0.05)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for k in range(2):
            opt.step(p, H.dev_list(grads[k], shapes))
            O.adam_step(meta, pr, grads[k], m, v)
        # set_lr takes effect with the next step (the schedule calls it every step)
        opt.set_lr(5e-4)
        meta.lr = 5e-4
        opt.step(p, H.dev_list(grads[2], shapes))
        O.adam_step(meta, pr, grads[2], m, v)
        assert opt.lr() == 5e-4 and opt.meta().lr == 5e-4 and opt.step_count() == 3
        H.assert_bits_equal(H.host_list(p), pr, "after set_lr")
        # reset: moments to zero, step_count to zero, params and hyper-parameters stay
        opt.reset()
        assert opt.step_count() == 0 and opt.meta().lr == 5e-4
        assert not any(t.any() for t in H.host_list(opt.moments()[0] + opt.moments()[1]))
        m, v = H.zeros_like_list(p0), H.zeros_like_list(p0)
        meta.step_count = 0
        opt.step(p, H.dev_list(grads[3], shapes))
        O.adam_step(meta, pr, grads[3], m, v)
        H.assert_bits_equal(H.host_list(p), pr, "after reset")
        # load_meta: every field of set_state (alg.rs:90-105), including step_count
        opt.load_meta(nb.OptimMeta("adamw", 2e-3, 0.8, 0.9, 1e-6, 0.2, 0.0, 40))
        meta = O.adamw_meta(2e-3, 0.8, 0.9, 1e-6, 0.2, step_count=40)
        # load_state_tensors: replace the moments
        m = [np.abs(a) for a in H.randn_list(shapes, 70, 1e-4)]
        v = [np.abs(a) for a in H.randn_list(shapes, 71, 1e-8)]
        opt.load_state_tensors([(f"m{i}", H.to_dev(a, shapes[i])) for i, a in enumerate(m)] +
                               [(f"v{i}", H.to_dev(a, shapes[i])) for i, a in enumerate(v)] +
                               [("ignored", None)])
        opt.step(p, H.dev_list(grads[4], shapes))
        O.adam_step(meta, pr, grads[4], m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert opt.step_count() == 41 == meta.step_count
    got = opt.meta()
    assert (got.beta1, got.beta2, got.eps, got.weight_decay, got.lr) == (0.8, 0.9, 1e-6, 0.2, 2e-3)
    H.assert_bits_equal(H.host_list(p), pr, "after load_meta + load_state_tensors")
    H.assert_bits_equal(H.host_list(opt.moments()[0]), m, "m")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")
    with pytest.raises(nb.OptimStateError, match="optim kind mismatch"):
        opt.load_meta(nb.OptimMeta("adam", 1e-3, 0.9, 0.999, 1e-8, 0.0, 0.0, 0))
    with pytest.raises(nb.NablaPanic, match="AdamW params/grads length mismatch"):
        opt.step(p, H.dev_list(grads[5], shapes)[:1])
    with pytest.raises(nb.NablaPanic, match="AdamW params count mismatch"):
        opt.step(p[:1], H.dev_list(grads[5], shapes)[:1])
    with pytest.raises(nb.NablaPanic, match="shapes must match"):
        opt.step(p, [H.dev_list(grads[5], shapes)[0], H.to_dev(grads[5][1][:100], (1, 100))])


def test_list_rebind_follows_moved_tensors(gpu):
    """nbo_list_set_ptrs: a list pointed at new tensors of the same shapes steps those, and
    leaves the old ones alone; a list of other shapes is refused."""
    shapes = [(2, 3), (1, 9000)]
    p0 = H.randn_list(shapes, 91, 0.05)
    g0, g1 = H.randn_list(shapes, 92, 1e-2), H.randn_list(shapes, 93, 1e-2)
    p_a, p_b = H.dev_list(p0, shapes), H.dev_list(p0, shapes)
    plist, glist = nb.TensorList(p_a), nb.TensorList(H.dev_list(g0, shapes))
    opt = nb.Sgd.new(0.1, shapes)
    opt.step(plist, glist)
    plist.rebind(p_b)
    g1_dev = H.dev_list(g1, shapes)
    glist.rebind(g1_dev)
    opt.step(plist, glist)
    ra, rb, vel, meta = H.copy_list(p0), H.copy_list(p0), H.zeros_like_list(p0), O.sgd_meta(0.1)
    O.sgd_step(meta, ra, g0, vel)
    O.sgd_step(meta, rb, g1, vel)
    H.assert_bits_equal(H.host_list(p_a), ra, "first tensors: one step with g0")
    H.assert_bits_equal(H.host_list(p_b), rb, "second tensors: one step with g1")
    with pytest.raises(ValueError, match="shapes"):
        plist.rebind(H.dev_list([p0[0]], [shapes[0]]))


def test_a_tensor_object_given_other_storage_is_followed(gpu):
    """Tensors passed as plain sequences are described to the device once and the description
    reused; reuse is decided by the addresses and shapes the description was built from, so
    the same tensor object pointing at other storage (`t.data = ...`) is picked up -- for a
    plain optimizer and for a GroupOptimizer's per-group lists."""
    import torch

    from nabla_amd import groups as G

    shapes = [(2, 3), (1, 9000)]
    p0, g0 = H.randn_list(shapes, 95, 0.05), H.randn_list(shapes, 96, 1e-2)
    for grouped in (False, True):
        params, grads = H.dev_list(p0, shapes), H.dev_list(g0, shapes)
        if grouped:
            cfg = G.ParamGroupConfig.sgd("all", G.ParamSelector.All(), 0.1, 0.0, 0.0)
            opt = G.GroupOptimizer.from_named_params(list(zip(["a", "b"], params)), [], cfg)
        else:
            opt = nb.Sgd.new(0.1, shapes)
        opt.step(params, grads)
        first = [t.clone() for t in params]
        old_storage = [t.data for t in params]
        for t, a in zip(params, p0):  # same objects, other memory, the start values again
            t.data = H.to_dev(a, tuple(t.shape))
        assert all(t.data_ptr() != o.data_ptr() for t, o in zip(params, old_storage))
        opt.step(params, grads)
        want = H.copy_list(p0)
        O.sgd_step(O.sgd_meta(0.1), want, g0, H.zeros_like_list(p0))
        H.assert_bits_equal(H.host_list(params), want, f"new storage stepped once (grouped={grouped})")
        assert all(torch.equal(a, b) for a, b in zip(old_storage, first)), "old storage left alone"


def test_host_tensors_and_short_allocations_are_refused_before_any_launch(gpu):
    """A list is checked against what the HIP runtime knows about each address when it is
    bound: a CPU tensor and a state buffer in host memory passed as a device buffer are
    errors, not GPU faults."""
    import torch

    shapes = [(2, 3)]
    cpu = [torch.zeros(s) for s in shapes]
    with pytest.raises(Exception, match="not memory the HIP runtime knows"):
        nb.TensorList(cpu)
    good = nb.TensorList([torch.zeros(s, device="cuda:0") for s in shapes])
    with pytest.raises(Exception, match="not memory the HIP runtime knows"):
        good.rebind(cpu)
    opt = nb.Adam.new(1e-3, shapes)
    from nabla_amd import _lib

    host = torch.zeros(6)
    rc = _lib.load().nbo_optim_state_write(opt._handle(), b"m0", host.data_ptr(), 6, 1)
    assert rc == _lib.ERR_ARG and b"not memory the HIP runtime knows" in _lib.load().nbo_last_error()
    # pinned host memory is device-accessible and passes
    pinned = torch.zeros(6, pin_memory=True)
    assert _lib.load().nbo_optim_state_write(opt._handle(), b"m0", pinned.data_ptr(), 6, 1) == 0
    nb.sync()


def test_two_host_threads_drive_two_optimizers(gpu):
    """Entry points may be called from several threads (ctypes drops the GIL around each
    call, so the calls do overlap in time); the library runs them one at a time and each
    optimizer's result is what it would be alone."""
    import threading

    shapes = [(3, 5), (1, 9000)]
    cases = []
    for k in range(2):
        p0 = H.randn_list(shapes, 600 + k, 0.05)
        grads = [H.randn_list(shapes, 700 + 10 * k + s, 1e-2) for s in range(25)]
        cases.append(dict(p0=p0, grads=grads, p_dev=H.dev_list(p0, shapes),
                          g_dev=[H.dev_list(g, shapes) for g in grads],
                          opt=nb.AdamW.new(1e-3, shapes).weight_decay(0.01 * (k + 1)), errors=[]))

    def run(c):
        try:
            for g in c["g_dev"]:
                c["opt"].fused_step(c["p_dev"], g, max_norm=0.5)
                c["opt"].last_step()  # a synchronous call in between
        except Exception as e:  # surfaced below, in the main thread
            c["errors"].append(e)

    threads = [threading.Thread(target=run, args=(c,)) for c in cases]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    O.set_pow_mode(O.POW_SQRT)
    try:
        for k, c in enumerate(cases):
            assert not c["errors"], c["errors"]
            pr, m, v = H.copy_list(c["p0"]), H.zeros_like_list(c["p0"]), H.zeros_like_list(c["p0"])
            meta = O.adamw_meta(1e-3, weight_decay=0.01 * (k + 1))
            for g in c["grads"]:
                O.f32_step(meta, None, 0.5, pr, H.copy_list(g), m, v)
            H.assert_bits_equal(H.host_list(c["p_dev"]), pr, f"thread {k}: params")
            assert c["opt"].step_count() == 25
    finally:
        O.set_pow_mode(O.POW_LIBM)


def test_switching_streams_keeps_the_steps_in_order(gpu):
    """nbo_set_stream waits for what is enqueued on the previous stream, so steps issued
    alternately on two non-blocking streams and the null stream run in call order: the result
    is the oracle's for the same sequence."""
    import torch

    from nabla_amd import _lib

    shapes = [(1, 70001), (64, 130), (1, 5)]
    p0 = H.randn_list(shapes, 800, 0.05)
    grads = [H.randn_list(shapes, 810 + s, 1e-2) for s in range(12)]
    p_dev, g_dev = H.dev_list(p0, shapes), [H.dev_list(g, shapes) for g in grads]
    torch.cuda.synchronize()
    opt = nb.AdamW.new(1e-3, shapes)
    lib = _lib.load()
    streams = [torch.cuda.Stream(), torch.cuda.Stream(), None]
    try:
        for s, g in enumerate(g_dev):
            st = streams[s % 3]
            _lib.check(lib.nbo_set_stream(st.cuda_stream if st is not None else None))
            opt.fused_step(p_dev, g, max_norm=0.5)
    finally:
        _lib.check(lib.nbo_set_stream(None))
    nb.sync()
    pr, m, v, meta = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0), O.adamw_meta(1e-3)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for g in grads:
            O.f32_step(meta, None, 0.5, pr, H.copy_list(g), m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    H.assert_bits_equal(H.host_list(p_dev), pr, "params")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")


def test_state_placement_says_what_it_found(gpu):
    """State of 128 MiB per array or more is placed across the HBM's regions when the probe
    can tell regions apart on this GPU; either way the optimizer reports the outcome and the
    reason, and steps give the oracle's bits."""
    shapes = [(4096, 8192 + 8)]  # 33.6 M elements: 134 MB per state array
    p_ref = H.randn_list(shapes, 4242, 0.02)
    p_dev = H.dev_list(p_ref, shapes)
    opt = nb.AdamW.new(1e-3, shapes).weight_decay(0.1)
    m, v = H.zeros_like_list(p_ref), H.zeros_like_list(p_ref)
    meta = O.adamw_meta(1e-3, weight_decay=0.1)
    O.set_pow_mode(O.POW_SQRT)
    O.set_threads(8)
    try:
        for step in range(2):
            g = H.randn_list(shapes, 4300 + step, 1e-3)
            opt.step(p_dev, H.dev_list(g, shapes))
            O.adam_step(meta, p_ref, g, m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
        O.set_threads(1)
    regions, note = opt.state_regions(), opt.state_placement_note()
    print(f"[placement] {regions} regions: {note}")
    assert note, "the placement always leaves a note"
    if regions == 0:
        assert note.startswith("plain allocation")
    else:
        assert regions in (2, 3) and note.startswith(f"{regions} regions") and "threshold" in note
    H.assert_bits_equal(H.host_list(p_dev), p_ref, "params on placed state")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v on placed state")


def test_state_placement_switches(gpu, monkeypatch):
    """NBO_STATE_SPREAD=0 and a chunk limit below what the state needs both end in plain
    allocations, say so, and the optimizer steps as usual."""
    shapes = [(4096, 8192 + 8)]  # 134 MB per state array: placed by default
    for env, reason in ((("NBO_STATE_SPREAD", "0"), "NBO_STATE_SPREAD=0"),
                        (("NBO_PLACEMENT_MAX_GIB", "1"), "chunk limit")):
        monkeypatch.setenv(*env)
        opt = nb.Adam.new(1e-3, shapes)
        regions, note = opt.state_regions(), opt.state_placement_note()  # the first call creates the state
        monkeypatch.delenv(env[0])
        assert regions == 0
        assert note.startswith("plain allocation") and reason in note, note
        p = H.dev_list(H.randn_list(shapes, 1, 0.02), shapes)
        g = H.dev_list(H.randn_list(shapes, 2, 1e-3), shapes)
        opt.step(p, g)
        assert opt.step_count() == 1
