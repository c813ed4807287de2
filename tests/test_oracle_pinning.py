"""Pins the CPU oracle (oracle/nabla_cpu_oracle.c) before anything is checked against it.

Three kinds of evidence, none of which re-uses the oracle's own formulas in floating
point:
  1. the known answers the reference's own tests hold for this path
     (nabla-train/tests/optim.rs, nabla-train/tests/trainer.rs);
  2. exact rational arithmetic (fractions.Fraction) with an explicit
     round-to-nearest-even after every operation of the reference's pass chain --
     a dropped term, a fused multiply-add, a swapped operand or a wrong order of
     operations changes bits here;
  3. closed forms, invariants and library cross-checks (torch.optim, torch's bf16
     cast, the published first output of xorshift64).
"""
import math
from fractions import Fraction

import numpy as np
import pytest

import oracle as O


# ---- exact arithmetic helpers -------------------------------------------------------

def rne(q: Fraction, mant_bits: int, emin: int) -> Fraction:
    """Round an exact rational to the nearest binary float (ties to even) with
    `mant_bits` significand bits and minimum exponent `emin` of the last place."""
    if q == 0:
        return Fraction(0)
    sign = -1 if q < 0 else 1
    q = abs(q)
    e = q.numerator.bit_length() - q.denominator.bit_length() - mant_bits
    while q / Fraction(2) ** e >= 2 ** mant_bits:
        e += 1
    while q / Fraction(2) ** e < 2 ** (mant_bits - 1):
        e -= 1
    e = max(e, emin)
    scaled = q / Fraction(2) ** e
    fl = scaled.numerator // scaled.denominator
    rem = scaled - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return sign * fl * Fraction(2) ** e


def r32(q):  # IEEE binary32
    return rne(Fraction(q), 24, -149)


def r64(q):  # IEEE binary64
    return rne(Fraction(q), 53, -1074)


def sqrt_r32(q: Fraction) -> Fraction:
    """Correctly rounded f32 square root of an exact non-negative rational."""
    if q == 0:
        return Fraction(0)
    # sqrt(q) to 80 extra bits, then round; the truncation cannot flip an f32 rounding
    # for the inputs used here because the 24-bit midpoint squared is never hit exactly
    # unless q is a perfect square of a midpoint, which binary32 inputs cannot be.
    shift = 200
    num = (q.numerator << (2 * shift)) // q.denominator
    root = math.isqrt(num)
    approx = Fraction(root, 1 << shift)
    if root * root != num:
        approx += Fraction(1, 1 << (shift + 2))  # strictly between root and root+1 ulp
    return r32(approx)


def f32_exact(x) -> Fraction:
    return Fraction(float(np.float32(x)))


def as_f32(q: Fraction) -> np.float32:
    return np.float32(float(q))


# ---- 1. the reference's own known answers ---------------------------------------------

def test_kat_sgd_step_updates_param():
    """tests/optim.rs:47-57: 1.0 - 0.1 * 1.0 = 0.9 (f64, 1x1)."""
    p, g, v = [np.array([1.0])], [np.array([1.0])], [np.zeros(1)]
    O.sgd_step(O.sgd_meta(0.1), p, g, v)
    assert abs(p[0][0] - 0.9) < 1e-10


def test_kat_adam_adamw_decrease_param():
    """tests/optim.rs:59-81: after one step from p=1, g=1 the parameter is < 1;
    closed form: step 1 from m=v=0 is p - lr*g/(|g|+eps) (+ decay for AdamW)."""
    for meta, expect in ((O.adam_meta(0.1), 0.9), (O.adamw_meta(0.1), 0.899)):
        p, g = [np.array([1.0])], [np.array([1.0])]
        m, v = [np.zeros(1)], [np.zeros(1)]
        O.adam_step(meta, p, g, m, v)
        assert p[0][0] < 1.0
        assert p[0][0] == pytest.approx(expect, abs=1e-8)
        assert meta.step_count == 1
        assert m[0][0] == pytest.approx(0.1) and v[0][0] == pytest.approx(0.001)


def test_kat_group_weight_decay_exclusion():
    """tests/optim.rs:140-165: SGD lr=1, wd=0.1, g=0: weight 2.0 -> 1.8; wd=0: bias 3.0 -> 3.0."""
    w, b, z = [np.array([2.0])], [np.array([3.0])], [np.zeros(1)]
    O.sgd_step(O.sgd_meta(1.0, 0.0, 0.1), w, z, [np.zeros(1)])
    O.sgd_step(O.sgd_meta(1.0, 0.0, 0.0), b, z, [np.zeros(1)])
    assert abs(w[0][0] - 1.8) < 1e-10 and abs(b[0][0] - 3.0) < 1e-10


def test_kat_grad_scaler_unscale_and_detect_inf():
    """tests/optim.rs:120-138 with the defaults of core.rs:336-344."""
    s = O.default_scaler()
    assert (s.scale, s.growth_factor, s.backoff_factor, s.growth_interval, s.consecutive_ok) == \
        (65536.0, 2.0, 0.5, 2000, 0)
    g = [np.array([2.0])]
    assert O.scaler_unscale_and_update(s, g) is True
    assert g[0][0] == 2.0 / 65536.0 and g[0][0] < 2.0
    assert s.consecutive_ok == 1 and s.scale == 65536.0
    g = [np.array([np.inf])]
    assert O.scaler_unscale_and_update(s, g) is False
    assert abs(g[0][0]) < 1e-12
    assert s.scale == 32768.0 and s.consecutive_ok == 0


def test_kat_clip_grad_norm_scales():
    """tests/trainer.rs:171-203: grads (3), (4): reported norm 5, norm after clip 2.5."""
    g = [np.array([3.0]), np.array([4.0])]
    reported = O.clip_grad_norm(g, 2.5)
    after = math.sqrt(sum(float((x * x).sum()) for x in g))
    assert abs(reported - 5.0) < 1e-10 and abs(after - 2.5) < 1e-10
    # trainer.rs:501-503 and :515
    g = [np.array([3.0]), np.array([4.0])]
    assert O.clip_grad_norm(g, 0.0) == 0.0 and O.clip_grad_norm(g, -1.0) == 0.0
    assert O.clip_grad_norm(g, 5.0) == 5.0 and g[0][0] == 3.0 and g[1][0] == 4.0


def test_kat_lr_schedules():
    """tests/optim.rs:83-118."""
    lin = O.Schedule(1, 0, 10, 0.0, 0.0)
    assert abs(O.lr_at_step(lin, 1.0, 0) - 1.0) < 1e-10 and O.lr_at_step(lin, 1.0, 10) <= 1e-10
    stp = O.Schedule(3, 2, 0, 0.1, 0.0)
    assert abs(O.lr_at_step(stp, 1.0, 0) - 1.0) < 1e-10
    assert abs(O.lr_at_step(stp, 1.0, 2) - 0.1) < 1e-10
    assert abs(O.lr_at_step(stp, 1.0, 4) - 0.01) < 1e-10
    one = O.Schedule(2, 0, 10, 1.0, 0.5)
    assert O.lr_at_step(one, 0.1, 3) > 0.1
    # closed forms: cosine mid-point and end, warm-up ramp
    cos = O.Schedule(0, 10, 110, 0.1, 0.0)
    assert O.lr_at_step(cos, 1.0, 5) == pytest.approx(0.5)
    assert O.lr_at_step(cos, 1.0, 60) == pytest.approx(0.55)
    assert O.lr_at_step(cos, 1.0, 110) == pytest.approx(0.1)


# ---- 2. exact-rational evaluation of every rounding ----------------------------------------

def _rand_f32(rng, n, lo=-8, hi=2):
    return (rng.standard_normal(n) * 10.0 ** rng.uniform(lo, hi, n)).astype(np.float32)


def test_primitives_round_once_per_operation():
    rng = np.random.default_rng(0)
    a, b = _rand_f32(rng, 64), _rand_f32(rng, 64)
    s = np.float32(0.899999976158142)
    out = O.scale(a, s)
    for i in range(a.size):
        assert f32_exact(out[i]) == r32(f32_exact(a[i]) * f32_exact(s))
    out = O.emul(a, b)
    for i in range(a.size):
        assert f32_exact(out[i]) == r32(f32_exact(a[i]) * f32_exact(b[i]))
    out = O.ediv(a, b)
    for i in range(a.size):
        assert f32_exact(out[i]) == r32(f32_exact(a[i]) / f32_exact(b[i]))
    out = O.add(a, b)
    for i in range(a.size):
        assert f32_exact(out[i]) == r32(f32_exact(a[i]) + f32_exact(b[i]))


def test_axpy_is_multiply_then_add_not_fma():
    """cpu/mod.rs:221: *yi = *yi + alpha * xi -- two roundings.  The sample must contain
    elements where a fused multiply-add would give different bits, or the check could
    not tell the two apart."""
    rng = np.random.default_rng(1)
    y, x = _rand_f32(rng, 512, -2, 0), _rand_f32(rng, 512, -2, 0)
    alpha = np.float32(0.1)
    y0 = y.copy()
    O.axpy_inplace(y, alpha, x)
    fused_differs = 0
    for i in range(y.size):
        prod = f32_exact(alpha) * f32_exact(x[i])
        two = r32(f32_exact(y0[i]) + r32(prod))
        one = r32(f32_exact(y0[i]) + prod)
        assert f32_exact(y[i]) == two
        fused_differs += two != one
    assert fused_differs > 10


def _exact_adam(kind, lr, b1, b2, eps, wd, steps, p0, grads, rt=None, exact=None):
    """Adam / AdamW in exact arithmetic with one rounding `rt` (to the element type T,
    default f32) after each operation of alg.rs:120-148, taking the correctly rounded
    f32 sqrt for powf(x, 0.5).  `exact` turns an input element into a Fraction."""
    rt = rt or r32
    exact = exact or f32_exact
    p = [exact(x) for x in p0]
    m = [Fraction(0)] * len(p)
    v = [Fraction(0)] * len(p)
    B1, B2, LR, EPS, WD = (Fraction(x) for x in (b1, b2, lr, eps, wd))
    for t in range(1, steps + 1):
        # f64 scalars: powi by repeated squaring as __powidf2 does, each multiply rounded
        def powi(a, n):
            r, a = Fraction(1), Fraction(a)
            while True:
                if n & 1:
                    r = r64(r * a)
                n >>= 1
                if n == 0:
                    return r
                a = r64(a * a)
        bc1 = r64(1 - powi(B1, t))
        bc2 = r64(1 - powi(B2, t))
        ss = rt(r64(LR / bc1))
        ibc2 = rt(r64(1 / bc2))
        fb1, fomb1 = rt(B1), rt(r64(1 - B1))
        fb2, fomb2 = rt(B2), rt(r64(1 - B2))
        feps = rt(EPS)
        omw = rt(1 - rt(r64(WD * LR)))
        g = [exact(x) for x in grads[t - 1]]
        for i in range(len(p)):
            m[i] = rt(rt(m[i] * fb1) + rt(fomb1 * g[i]))
            v[i] = rt(rt(v[i] * fb2) + rt(fomb2 * rt(g[i] * g[i])))
            denom = rt(rt(sqrt_r32(rt(v[i] * ibc2))) + feps)
            upd = rt(rt(m[i] * ss) / denom)
            if kind == "adamw":
                p[i] = rt(p[i] * omw)
            p[i] = rt(p[i] + (-upd))
    return p, m, v


@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_adam_chain_bit_exact_against_exact_arithmetic(kind):
    rng = np.random.default_rng(2)
    n, steps = 8, 3
    lr, b1, b2, eps, wd = 3e-4, 0.9, 0.95, 1e-8, 0.1
    p0 = (rng.standard_normal(n) * 0.02).astype(np.float32)
    grads = [(rng.standard_normal(n) * 1e-3).astype(np.float32) for _ in range(steps)]
    pe, me, ve = _exact_adam(kind, lr, b1, b2, eps, wd, steps, p0, grads)
    p, m, v = [p0.copy()], [np.zeros(n, np.float32)], [np.zeros(n, np.float32)]
    meta = O.adam_meta(lr, b1, b2, eps) if kind == "adam" else O.adamw_meta(lr, b1, b2, eps, wd)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for t in range(steps):
            O.adam_step(meta, p, [grads[t]], m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    for i in range(n):
        assert f32_exact(m[0][i]) == me[i], f"m[{i}]"
        assert f32_exact(v[0][i]) == ve[i], f"v[{i}]"
        assert f32_exact(p[0][i]) == pe[i], f"p[{i}]"
    # the libm-powf variant: moments identical, params within 2 ulp
    p2, m2, v2 = [p0.copy()], [np.zeros(n, np.float32)], [np.zeros(n, np.float32)]
    meta2 = O.adam_meta(lr, b1, b2, eps) if kind == "adam" else O.adamw_meta(lr, b1, b2, eps, wd)
    for t in range(steps):
        O.adam_step(meta2, p2, [grads[t]], m2, v2)
    assert np.array_equal(m2[0].view(np.uint32), m[0].view(np.uint32))
    assert np.array_equal(v2[0].view(np.uint32), v[0].view(np.uint32))
    assert O.ulp_distance_f32(p2[0], p[0]).max() <= 2


def test_adamw_step_single_equals_adamw_step():
    """adamw_step (alg.rs:431-469) is AdamW::step's body for one tensor."""
    rng = np.random.default_rng(3)
    p0 = (rng.standard_normal(100) * 0.02).astype(np.float32)
    g = (rng.standard_normal(100) * 1e-3).astype(np.float32)
    pa, ma, va = [p0.copy()], [np.zeros_like(p0)], [np.zeros_like(p0)]
    meta = O.adamw_meta(1e-3, 0.9, 0.999, 1e-8, 0.01, step_count=4)
    O.adam_step(meta, pa, [g], ma, va)
    pb, mb, vb = p0.copy(), np.zeros_like(p0), np.zeros_like(p0)
    O.adamw_step_single(pb, g, mb, vb, 1e-3, 0.9, 0.999, 1e-8, 0.01, 5)
    assert np.array_equal(pa[0], pb) and np.array_equal(ma[0], mb) and np.array_equal(va[0], vb)


def test_sgd_momentum_weight_decay_exact():
    """alg.rs:404-413 in exact arithmetic."""
    rng = np.random.default_rng(4)
    n = 16
    p0, g = _rand_f32(rng, n, -2, 0), _rand_f32(rng, n, -3, -1)
    lr, mu, wd = 0.05, 0.9, 0.01
    p, vel = [p0.copy()], [np.zeros(n, np.float32)]
    meta = O.sgd_meta(lr, mu, wd)
    pe = [f32_exact(x) for x in p0]
    ve = [Fraction(0)] * n
    for _ in range(3):
        O.sgd_step(meta, p, [g], vel)
        for i in range(n):
            ge = r32(f32_exact(g[i]) + r32(pe[i] * r32(wd)))
            ve[i] = r32(r32(ve[i] * r32(mu)) + ge)
            pe[i] = r32(pe[i] + r32(-r32(lr) * ve[i]))
    for i in range(n):
        assert f32_exact(p[0][i]) == pe[i] and f32_exact(vel[0][i]) == ve[i]


def test_clip_sum_is_serial_f64_and_scale_is_narrowed_once():
    """trainer.rs:504-521: sum += v*v in f64 in list order; scale_t = T(max_norm / norm)."""
    rng = np.random.default_rng(5)
    g = [_rand_f32(rng, 37, -3, 0), _rand_f32(rng, 5, -3, 0)]
    g0 = [x.copy() for x in g]
    s = Fraction(0)
    for t in g0:
        for x in t:
            s = r64(s + r64(f32_exact(x) * f32_exact(x)))
    norm = O.clip_grad_norm(g, 1e-3)
    assert Fraction(norm) ** 2 == pytest.approx(float(s), rel=1e-15)
    assert norm == math.sqrt(float(s))
    c = r32(r64(Fraction(1e-3) / Fraction(norm)))
    for t, t0 in zip(g, g0):
        for x, x0 in zip(t, t0):
            assert f32_exact(x) == r32(f32_exact(x0) * c)


def test_unscale_multiplies_by_narrowed_reciprocal():
    """core.rs:355,379: inv_scale = T(1/scale); g = g * inv_scale (not g / scale)."""
    s = O.ScalerState(3.0, 2.0, 0.5, 2000, 0)  # 1/3 is inexact: g*T(1/3) != g/3 in general
    rng = np.random.default_rng(6)
    g0 = _rand_f32(rng, 256, -2, 2)
    g = [g0.copy()]
    assert O.scaler_unscale_and_update(s, g)
    inv = r32(r64(Fraction(1) / 3))
    differs_from_division = 0
    for x, x0 in zip(g[0], g0):
        assert f32_exact(x) == r32(f32_exact(x0) * inv)
        differs_from_division += r32(f32_exact(x0) * inv) != r32(f32_exact(x0) / 3)
    assert differs_from_division > 0


# ---- 3. closed forms, invariants, library cross-checks -------------------------------------

def test_powi_matches_exact_powers():
    assert O.powi(0.5, 10) == 2.0 ** -10 and O.powi(2.0, 30) == 2.0 ** 30
    assert O.powi(0.9, 0) == 1.0 and O.powi(0.9, 1) == 0.9 and O.powi(2.0, -2) == 0.25
    for a, n in ((0.9, 7), (0.95, 100), (0.999, 2000), (0.1, 5)):
        exact = Fraction(a) ** n
        got = Fraction(O.powi(a, n))
        # each of the ~2*log2(n) multiplies rounds once; errors scale with the exponent
        assert abs(got - exact) / exact < Fraction(n, 2 ** 52)


def test_zero_gradient_is_pure_decay_and_moments_stay_zero():
    p0 = np.float32([1.0, -2.0, 0.5])
    p, m, v = [p0.copy()], [np.zeros(3, np.float32)], [np.zeros(3, np.float32)]
    meta = O.adamw_meta(0.1, weight_decay=0.1)
    g = [np.zeros(3, np.float32)]
    for _ in range(5):
        O.adam_step(meta, p, g, m, v)
    assert not m[0].any() and not v[0].any()
    omw = np.float32(1.0) - np.float32(0.1 * 0.1)
    expect = p0.copy()
    for _ in range(5):
        expect = expect * omw
    assert np.array_equal(p[0], expect)


def test_constant_gradient_gives_geometric_moments():
    g = [np.full(4, 0.25, np.float32)]
    p, m, v = [np.ones(4, np.float32)], [np.zeros(4, np.float32)], [np.zeros(4, np.float32)]
    meta = O.adam_meta(1e-3)
    for t in range(1, 21):
        O.adam_step(meta, p, g, m, v)
        assert m[0][0] == pytest.approx(0.25 * (1 - 0.9 ** t), rel=1e-5)
        assert v[0][0] == pytest.approx(0.0625 * (1 - 0.999 ** t), rel=1e-5)
    # bias-corrected update is lr * sign(g) for a constant gradient
    assert p[0][0] == pytest.approx(1.0 - 20 * 1e-3, rel=1e-5)


def test_moments_do_not_depend_on_params():
    rng = np.random.default_rng(7)
    g = [(rng.standard_normal(50) * 1e-3).astype(np.float32)]
    res = []
    for scale in (1.0, 100.0):
        p = [(rng.standard_normal(50) * scale).astype(np.float32)]
        m, v = [np.zeros(50, np.float32)], [np.zeros(50, np.float32)]
        meta = O.adamw_meta(1e-3)
        for _ in range(3):
            O.adam_step(meta, p, g, m, v)
        res.append((m[0].copy(), v[0].copy()))
    assert np.array_equal(res[0][0], res[1][0]) and np.array_equal(res[0][1], res[1][1])


def test_matches_torch_optim_within_a_few_ulp():
    """Same mathematics, different rounding order (torch: sqrt(v)/sqrt(bc2) + eps, addcdiv)."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(8)
    p0 = (rng.standard_normal(1000) * 0.02).astype(np.float32)
    grads = [(rng.standard_normal(1000) * 1e-3).astype(np.float32) for _ in range(10)]
    for kind in ("adam", "adamw", "sgd"):
        tp = torch.nn.Parameter(torch.from_numpy(p0.copy()))
        if kind == "adam":
            topt = torch.optim.Adam([tp], lr=3e-4, betas=(0.9, 0.999), eps=1e-8)
            meta = O.adam_meta(3e-4)
        elif kind == "adamw":
            topt = torch.optim.AdamW([tp], lr=3e-4, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
            meta = O.adamw_meta(3e-4, 0.9, 0.95, 1e-8, 0.1)
        else:
            topt = torch.optim.SGD([tp], lr=0.01, momentum=0.9, weight_decay=0.01)
            meta = O.sgd_meta(0.01, 0.9, 0.01)
        p, m, v = [p0.copy()], [np.zeros_like(p0)], [np.zeros_like(p0)]
        for g in grads:
            tp.grad = torch.from_numpy(g.copy())
            topt.step()
            if kind == "sgd":
                O.sgd_step(meta, p, [g], m)
            else:
                O.adam_step(meta, p, [g], m, v)
        np.testing.assert_allclose(p[0], tp.detach().numpy(), rtol=2e-5, atol=2e-9)


def test_bf16_cast_matches_torch_for_all_exponents_and_is_rne():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(9)
    bits = rng.integers(0, 2 ** 32, size=1 << 22, dtype=np.uint64).astype(np.uint32)
    # every exponent with tie / just-above-tie / just-below-tie / max mantissas
    exps = np.arange(256, dtype=np.uint32) << 23
    tails = np.array([0x0000, 0x7FFF, 0x8000, 0x8001, 0x18000, 0x17FFF, 0x7F7FFF, 0x7F8000,
                      0x7FFFFF], dtype=np.uint32)
    edge = (exps[:, None] | tails[None, :]).reshape(-1)
    bits = np.concatenate([bits, edge, edge | np.uint32(0x80000000)])
    f = bits.view(np.float32)
    finite_or_inf = ~np.isnan(f)
    got = O.bf16_from_f32(f)
    ref = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[finite_or_inf], ref[finite_or_inf])
    # NaN: stays NaN, quiet bit set, sign and top payload kept (crate half's rule)
    nan = np.uint32([0x7F800001, 0xFFC12345, 0x7FBFFFFF]).view(np.float32)
    out = O.bf16_from_f32(nan)
    assert list(out) == [0x7FC0, 0xFFC1, 0x7FFF]
    # widening is exact
    h = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    w = O.bf16_to_f32(h)
    assert np.array_equal(w.view(np.uint32), h.astype(np.uint32) << 16)


def test_randn_stream_anchors():
    """xorshift64 with shifts (13, 7, 17): state 1 -> 1082269761 is the published first
    output; the Box-Muller pair built from the first two outputs must reproduce."""
    s = 1
    outs = []
    for _ in range(2):
        s ^= (s << 13) & 0xFFFFFFFFFFFFFFFF
        s ^= s >> 7
        s ^= (s << 17) & 0xFFFFFFFFFFFFFFFF
        outs.append(s)
    assert outs[0] == 1082269761
    u1, u2 = outs[0] / 2.0 ** 64, outs[1] / 2.0 ** 64
    r, th = math.sqrt(-2.0 * math.log(u1)), 2.0 * math.pi * u2
    z = O.randn_f64(3, 1)
    assert z[0] == pytest.approx(r * math.cos(th), rel=1e-15)
    assert z[1] == pytest.approx(r * math.sin(th), rel=1e-15)
    # seed 0 is replaced by 0x123456789ABCDEF0 (constructors.rs:20-24)
    assert np.array_equal(O.randn_f64(8, 0), O.randn_f64(8, 0x123456789ABCDEF0))
    big = O.randn_f64(200_000, 42)
    assert abs(big.mean()) < 0.01 and abs(big.std() - 1.0) < 0.01


def test_scaler_trace_closed_form():
    """growth_interval 4, inf injected every 4th step: only 3 clean steps fit between
    injections, so the scale only halves; every 5th step: it grows once, then halves."""
    for period, steps in ((4, 64), (5, 60)):
        s = O.ScalerState(65536.0, 2.0, 0.5, 4, 0)
        trace = []
        for step in range(steps):
            g = [np.ones(3, np.float32)]
            if step % period == period - 1:
                g[0][1] = np.nan
            ok = O.scaler_unscale_and_update(s, g)
            trace.append((ok, s.scale, s.consecutive_ok))
        skipped = sum(1 for t in trace if not t[0])
        assert skipped == steps // period
        if period == 4:
            assert s.scale == 65536.0 * 0.5 ** 16 == 1.0
            assert max(t[2] for t in trace) == 3
        else:
            assert s.scale == 65536.0
            assert [t[1] for t in trace[:5]] == [65536.0, 65536.0, 65536.0, 131072.0, 65536.0]


def test_found_inf_leaves_everything_but_the_scaler_untouched():
    rng = np.random.default_rng(10)
    shapes = [(3, 5), (1, 9)]
    master = [(rng.standard_normal(r * c) * 0.02).astype(np.float32) for r, c in shapes]
    m = [np.full_like(a, 0.5) for a in master]
    v = [np.full_like(a, 0.25) for a in master]
    p = [O.bf16_from_f32(a) for a in master]
    g = [O.bf16_from_f32(np.ones_like(a)) for a in master]
    g[1][4] = 0x7F80  # +inf
    before = [x.copy() for x in master + m + v + p]
    meta, s = O.adamw_meta(1e-3, step_count=7), O.default_scaler()
    ran, norm = O.mixed_step(meta, s, 1.0, p, g, master, m, v)
    assert not ran and norm == 0.0 and meta.step_count == 7
    assert s.scale == 32768.0 and s.consecutive_ok == 0
    for a, b in zip(before, master + m + v + p):
        assert np.array_equal(a, b)


def test_mixed_step_composition_in_exact_arithmetic():
    """The Trainer tail for bf16 params / grads with f32 master (cast -> unscale -> clip ->
    AdamW -> cast, trainer.rs:230-283) evaluated in exact rationals with a rounding after
    every reference operation: pins the order of the stages (the norm is taken of the
    unscaled gradients, the clip factor multiplies after the unscale factor, params are
    the RNE narrowing of the updated master)."""
    rng = np.random.default_rng(11)
    sizes = [3, 4]
    lr, b1, b2, eps, wd, max_norm, scale = 1e-3, 0.9, 0.95, 1e-8, 0.1, 0.5, 3.0
    master = [(rng.standard_normal(n) * 0.02).astype(np.float32) for n in sizes]
    p_bits = [O.bf16_from_f32(a) for a in master]
    m = [np.zeros(n, np.float32) for n in sizes]
    v = [np.zeros(n, np.float32) for n in sizes]
    meta, s = O.adamw_meta(lr, b1, b2, eps, wd), O.ScalerState(scale, 2.0, 0.5, 2000, 0)
    we = [[f32_exact(x) for x in a] for a in master]
    me = [[Fraction(0)] * n for n in sizes]
    ve = [[Fraction(0)] * n for n in sizes]
    O.set_pow_mode(O.POW_SQRT)
    try:
        for t in (1, 2):
            g_bits = [O.bf16_from_f32((rng.standard_normal(n) * 2.0).astype(np.float32)) for n in sizes]
            ran, norm = O.mixed_step(meta, s, max_norm, p_bits, g_bits, master, m, v)
            assert ran
            # exact: g32 = widen(bf16) ; g = r32(g32 * r32(1/scale)) ; norm over all in list order
            inv = r32(r64(Fraction(1) / Fraction(scale)))
            ge = [[r32(Fraction(float(x)) * inv) for x in O.bf16_to_f32(gb)] for gb in g_bits]
            acc = Fraction(0)
            for t_ in ge:
                for x in t_:
                    acc = r64(acc + r64(x * x))
            assert norm == math.sqrt(float(acc)) and norm > max_norm
            c = r32(r64(Fraction(max_norm) / Fraction(norm)))
            ge = [[r32(x * c) for x in t_] for t_ in ge]
            # AdamW on the master in exact arithmetic (same chain as _exact_adam, step t)
            def powi(a, n):
                r, a = Fraction(1), Fraction(a)
                while True:
                    if n & 1:
                        r = r64(r * a)
                    n >>= 1
                    if n == 0:
                        return r
                    a = r64(a * a)
            bc1, bc2 = r64(1 - powi(b1, t)), r64(1 - powi(b2, t))
            ss, ibc2 = r32(r64(Fraction(lr) / bc1)), r32(r64(1 / bc2))
            fb1, fomb1, fb2, fomb2 = r32(b1), r32(r64(1 - Fraction(b1))), r32(b2), r32(r64(1 - Fraction(b2)))
            omw = r32(1 - r32(r64(Fraction(wd) * Fraction(lr))))
            for k in range(len(sizes)):
                for i in range(sizes[k]):
                    g = ge[k][i]
                    me[k][i] = r32(r32(me[k][i] * fb1) + r32(fomb1 * g))
                    ve[k][i] = r32(r32(ve[k][i] * fb2) + r32(fomb2 * r32(g * g)))
                    denom = r32(sqrt_r32(r32(ve[k][i] * ibc2)) + r32(eps))
                    upd = r32(r32(me[k][i] * ss) / denom)
                    we[k][i] = r32(r32(we[k][i] * omw) + (-upd))
            for k in range(len(sizes)):
                for i in range(sizes[k]):
                    assert f32_exact(master[k][i]) == we[k][i] and f32_exact(m[k][i]) == me[k][i]
                    assert f32_exact(v[k][i]) == ve[k][i]
                    # param = RNE narrowing of the master to 8 significand bits
                    assert Fraction(float(O.bf16_to_f32(p_bits[k][i:i + 1])[0])) == rne(we[k][i], 8, -133)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert meta.step_count == 2 and s.consecutive_ok == 2 and s.scale == scale


# ---- 7. T = bf16 primitives and the generic cast ---------------------------------------

def rbf(q):  # bfloat16: 8 significand bits, f32's exponent range
    return rne(Fraction(q), 8, -133)


def _bf_exact(h) -> Fraction:
    return Fraction(float(O.bf16_to_f32(np.array([h], dtype=np.uint16))[0]))


def test_bf16_primitives_are_the_f32_operation_then_one_rounding_to_bf16():
    """scalar/mod.rs:256-283 and the half crate's operators: convert to f32, operate in
    f32, bf16::from_f32.  Checked in exact arithmetic: RNE to 24 bits, then RNE to 8 bits.
    (For +, * and / of 8-bit significands the two-step rounding provably equals the direct
    one; where a shortcut would show is the inner rounding of axpy, checked below, and the
    f64 -> bf16 cast, checked in the next test.)"""
    rng = np.random.default_rng(7)
    a = O.bf16_from_f32(_rand_f32(rng, 4000, -3, 2))
    b = O.bf16_from_f32(_rand_f32(rng, 4000, -3, 2))
    s = 0.3
    sb = _bf_exact(O.bf16_from_f32(np.array([np.float32(s)]))[0])
    cases = {
        "scale": (O.scale(a, s), lambda x, y: x * sb),
        "emul": (O.emul(a, b), lambda x, y: x * y),
        "ediv": (O.ediv(a, b), lambda x, y: x / y),
        "add": (O.add(a, b), lambda x, y: x + y),
        "map_add": (O.map_add(a, s), lambda x, y: x + sb),
    }
    for name, (out, f) in cases.items():
        for i in range(a.size):
            exact = f(_bf_exact(a[i]), _bf_exact(b[i]))
            assert _bf_exact(out[i]) == rbf(r32(exact)), (name, i)
    # axpy: the product is itself a bf16 value before the sum (two bf16 roundings)
    y = a.copy()
    O.axpy_inplace(y, s, b)
    skipped_inner_rounding_differs = 0
    for i in range(a.size):
        t = rbf(r32(sb * _bf_exact(b[i])))
        want = rbf(r32(_bf_exact(a[i]) + t))
        assert _bf_exact(y[i]) == want, i
        skipped_inner_rounding_differs += want != rbf(r32(_bf_exact(a[i]) + r32(sb * _bf_exact(b[i]))))
    assert skipped_inner_rounding_differs > 10


def test_bf16_powf_follows_the_pow_mode():
    a = O.bf16_from_f32(np.array([0.0, 0.25, 2.0, 3.0, 1e-6, 7e4], dtype=np.float32))
    for mode in (O.POW_LIBM, O.POW_SQRT):
        O.set_pow_mode(mode)
        try:
            out = O.powf(a, 0.5)
        finally:
            O.set_pow_mode(O.POW_LIBM)
        for i in range(a.size):
            # sqrt of a bf16 value, correctly rounded to f32, then to bf16: both candidate
            # lowerings of powf agree after the second rounding on these inputs
            assert _bf_exact(out[i]) == rbf(sqrt_r32(_bf_exact(a[i]))), (mode, i)


def test_cast_goes_through_f64_and_narrows_to_bf16_in_two_steps():
    """backend/mod.rs:157-160 with scalar/mod.rs:219, 338-344: widening is exact,
    f64 -> f32 is one RNE, anything -> bf16 is `from_f32(v as f32)`."""
    rng = np.random.default_rng(8)
    x64 = rng.standard_normal(3000) * 10.0 ** rng.uniform(-6, 6, 3000)
    # exact ties of the second rounding that the first rounding creates
    x64[:4] = [1.0 + 2.0 ** -8 + 2.0 ** -30, 1.0 + 2.0 ** -8 - 2.0 ** -30, -(1.0 + 3 * 2.0 ** -8 - 2.0 ** -40), 0.0]
    to32 = O.cast(x64, np.float32)
    to16 = O.cast(x64, np.uint16)
    two_step_differs = 0
    for i in range(x64.size):
        q = Fraction(float(x64[i]))
        assert f32_exact(to32[i]) == r32(q)
        assert _bf_exact(to16[i]) == rbf(r32(q))
        two_step_differs += rbf(r32(q)) != rbf(q)
    assert two_step_differs >= 2
    assert to16[0] == 0x3F80 and rbf(Fraction(float(x64[0]))) == Fraction(1) + Fraction(1, 128)
    x32 = _rand_f32(rng, 1000)
    assert np.array_equal(O.cast(x32, np.float64), x32.astype(np.float64))
    assert np.array_equal(O.cast(x32, np.uint16), O.bf16_from_f32(x32))
    h = O.bf16_from_f32(x32)
    assert np.array_equal(O.cast(h, np.float32), O.bf16_to_f32(h))
    assert np.array_equal(O.cast(h, np.float64), O.bf16_to_f32(h).astype(np.float64))
    assert np.array_equal(O.cast(h, np.uint16), h) and np.array_equal(O.cast(x32, np.float32), x32)


def test_powf_half_of_negative_zero_and_minus_infinity():
    """C's pow: pow(-0, 0.5) = +0 and pow(-inf, 0.5) = +inf; the sqrt lowering keeps both
    (fabs, select) -- the oracle's two modes must agree on them."""
    x = np.array([-0.0, -np.inf, np.inf, 0.0, 4.0], dtype=np.float32)
    for mode in (O.POW_LIBM, O.POW_SQRT):
        O.set_pow_mode(mode)
        try:
            out = O.powf(x, np.float32(0.5))
        finally:
            O.set_pow_mode(O.POW_LIBM)
        assert np.array_equal(out.view(np.uint32), np.array([0.0, np.inf, np.inf, 0.0, 2.0], dtype=np.float32).view(np.uint32)), mode


@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_bf16_adam_chain_bit_exact_against_exact_arithmetic(kind):
    """Optimizer<bf16>: the same chain with every result -- scalars included -- rounded to
    f32 and then to bf16 (T::from_f64 = from_f32(v as f32); each operation = f32 operation +
    from_f32)."""
    rng = np.random.default_rng(12)
    n, steps = 16, 4
    lr, b1, b2, eps, wd = 1e-2, 0.9, 0.95, 1e-8, 0.1
    rt = lambda q: rbf(r32(q))
    p0 = O.bf16_from_f32((rng.standard_normal(n) * 0.5).astype(np.float32))
    grads = [O.bf16_from_f32((rng.standard_normal(n) * 1e-2).astype(np.float32)) for _ in range(steps)]
    pe, me, ve = _exact_adam(kind, lr, b1, b2, eps, wd, steps, p0, grads, rt=rt, exact=_bf_exact)
    p, m, v = [p0.copy()], [np.zeros(n, np.uint16)], [np.zeros(n, np.uint16)]
    meta = O.adam_meta(lr, b1, b2, eps) if kind == "adam" else O.adamw_meta(lr, b1, b2, eps, wd)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for t in range(steps):
            O.adam_step(meta, p, [grads[t]], m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    for i in range(n):
        assert _bf_exact(m[0][i]) == me[i], f"m[{i}]"
        assert _bf_exact(v[0][i]) == ve[i], f"v[{i}]"
        assert _bf_exact(p[0][i]) == pe[i], f"p[{i}]"
    assert meta.step_count == steps and any(x != 0 for x in m[0]) and any(x != 0 for x in v[0])


def test_bf16_sgd_scaler_and_clip_in_exact_arithmetic():
    rt = lambda q: rbf(r32(q))
    rng = np.random.default_rng(13)
    n = 32
    p0 = O.bf16_from_f32((rng.standard_normal(n) * 0.5).astype(np.float32))
    g0 = O.bf16_from_f32((rng.standard_normal(n) * 3.0).astype(np.float32))
    # Sgd with momentum and weight decay (alg.rs:403-414), two steps
    lr, mom, wd = 0.05, 0.9, 0.01
    p, vel = [p0.copy()], [np.zeros(n, np.uint16)]
    meta = O.sgd_meta(lr, momentum=mom, weight_decay=wd)
    pe, ve = [_bf_exact(x) for x in p0], [Fraction(0)] * n
    flr, fmom, fwd = rt(Fraction(lr)), rt(Fraction(mom)), rt(Fraction(wd))
    for _ in range(2):
        O.sgd_step(meta, p, [g0], vel)
        for i in range(n):
            ge = rt(_bf_exact(g0[i]) + rt(pe[i] * fwd))
            ve[i] = rt(rt(ve[i] * fmom) + ge)
            pe[i] = rt(pe[i] + rt(-flr * ve[i]))
    for i in range(n):
        assert _bf_exact(p[0][i]) == pe[i] and _bf_exact(vel[0][i]) == ve[i], i
    # unscale by a scale that is not a power of two, then clip (core.rs:355,379; trainer.rs:504-521)
    g = [g0.copy()]
    st = O.ScalerState(3.0, 2.0, 0.5, 2, 0)
    assert O.scaler_unscale_and_update(st, g)
    inv = rt(r64(Fraction(1) / 3))
    un = [rt(_bf_exact(x) * inv) for x in g0]
    assert [_bf_exact(x) for x in g[0]] == un
    norm = O.clip_grad_norm(g, 0.5)
    total = Fraction(0)
    for x in un:
        total = r64(total + r64(x * x))
    assert abs(norm - math.sqrt(float(total))) <= 1e-12 * norm
    c = rt(r64(Fraction(0.5) / Fraction(norm)))
    assert [_bf_exact(x) for x in g[0]] == [rt(x * c) for x in un]


def test_bench_lcg_rand_tensor_in_exact_arithmetic():
    """benchmarks/src/lib.rs:7-22: x' = x * 6364136223846793005 + 1442695040888963407 mod
    2^64; value = ((x' >> 33) as f32) / 2^31 - 1, each conversion / operation one rounding."""
    vals, state = O.bench_rand_f32(500, 42)
    x = 42
    for i in range(500):
        x = (x * 6364136223846793005 + 1442695040888963407) % (1 << 64)
        want = r32(r32(r32(Fraction(x >> 33)) / (1 << 31)) - 1)
        assert f32_exact(vals[i]) == want, i
    assert state == x
    # 31 bits over 2^31 lie in [0, 1), so the values lie in [-1, 0): as written in the reference
    assert -1.0 <= vals.min() and vals.max() < 0.0 and abs(float(vals.mean()) + 0.5) < 0.1
    more, _ = O.bench_rand_f32(3, state)  # the stream continues across tensors
    x = (x * 6364136223846793005 + 1442695040888963407) % (1 << 64)
    assert f32_exact(more[0]) == r32(r32(r32(Fraction(x >> 33)) / (1 << 31)) - 1)


# ---- 8. T = f16 -------------------------------------------------------------------------------

def r16(q):  # IEEE binary16: 11 significand bits, subnormals down to 2^-24
    return rne(Fraction(q), 11, -24)


def test_f16_conversions_match_ieee_binary16_everywhere():
    """half::f16::from_f32 / f32::from(f16) restated from the half crate's software path:
    every one of the 65536 patterns widens exactly (against numpy's float16), and every
    f16 value's neighbourhood in f32 -- the value, both ties and one f32 ulp either side of
    them -- narrows as IEEE round-to-nearest-even does, overflow and subnormals included.
    NaN: top ten payload bits kept, quiet bit set."""
    all16 = np.arange(1 << 16, dtype=np.uint16).view(np.float16)
    wide = O.cast(all16, np.float32)
    finite = ~np.isnan(all16)
    assert np.array_equal(wide[finite].view(np.uint32), all16[finite].astype(np.float32).view(np.uint32))
    assert np.isnan(wide[~finite]).all()
    base = all16[finite].astype(np.float32).view(np.uint32).astype(np.int64)
    cand = []
    for off in (0, 0x0FFF, 0x1000, 0x1001, -0x0FFF, -0x1000, -0x1001, 1, -1, 0x1FFF):
        cand.append(base + off)
    bits = np.concatenate(cand)
    bits = bits[(bits >= 0) & (bits < (1 << 32))].astype(np.uint32)
    x = bits.view(np.float32)
    x = x[~np.isnan(x)]
    got = O.cast(x, np.float16)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    for i in range(0, x.size, 9973):  # and a sample against exact rational rounding
        q = r16(Fraction(float(x[i])))
        if abs(q) < 65520:
            assert Fraction(float(got[i])) == q, hex(int(x[i:i + 1].view(np.uint32)[0]))
    nan_in = np.array([0x7FC00000, 0xFFC00000, 0x7F800001, 0x7FA5A000, 0xFF80E000], dtype=np.uint32).view(np.float32)
    nan_out = O.cast(nan_in, np.float16).view(np.uint16)
    assert list(nan_out) == [0x7E00, 0xFE00, 0x7E00, 0x7F2D, 0xFE07]


@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_f16_adam_chain_bit_exact_against_exact_arithmetic(kind):
    """Optimizer<f16>: every result rounded to f32 and then to f16."""
    rng = np.random.default_rng(21)
    n, steps = 16, 4
    lr, b1, b2, eps, wd = 1e-2, 0.9, 0.95, 1e-4, 0.1  # eps representable in f16 (1e-8 narrows to 0)
    rt = lambda q: r16(r32(q))
    fx = lambda x: Fraction(float(x))
    p0 = (rng.standard_normal(n) * 0.5).astype(np.float16)
    grads = [(rng.standard_normal(n) * 1e-1).astype(np.float16) for _ in range(steps)]
    pe, me, ve = _exact_adam(kind, lr, b1, b2, eps, wd, steps, p0, grads, rt=rt, exact=fx)
    p, m, v = [p0.copy()], [np.zeros(n, np.float16)], [np.zeros(n, np.float16)]
    meta = O.adam_meta(lr, b1, b2, eps) if kind == "adam" else O.adamw_meta(lr, b1, b2, eps, wd)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for t in range(steps):
            O.adam_step(meta, p, [grads[t]], m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    for i in range(n):
        assert fx(m[0][i]) == me[i] and fx(v[0][i]) == ve[i] and fx(p[0][i]) == pe[i], i
    assert any(x != 0 for x in v[0])


def test_f16_mixed_step_is_the_f32_step_between_two_casts():
    rng = np.random.default_rng(22)
    n = 64
    w0 = (rng.standard_normal(n) * 0.1).astype(np.float32)
    g16 = (rng.standard_normal(n) * 4.0).astype(np.float16)
    meta, s = O.adamw_meta(1e-3, weight_decay=0.1), O.ScalerState(1024.0, 2.0, 0.5, 2, 0)
    p, w, m, v = [w0.astype(np.float16)], [w0.copy()], [np.zeros(n, np.float32)], [np.zeros(n, np.float32)]
    ran, norm = O.mixed_step(meta, s, 0.01, p, [g16], w, m, v)
    meta2, s2 = O.adamw_meta(1e-3, weight_decay=0.1), O.ScalerState(1024.0, 2.0, 0.5, 2, 0)
    w2, m2, v2 = [w0.copy()], [np.zeros(n, np.float32)], [np.zeros(n, np.float32)]
    ran2, norm2 = O.f32_step(meta2, s2, 0.01, w2, [g16.astype(np.float32)], m2, v2)
    assert ran and ran2 and norm == norm2
    assert np.array_equal(w[0].view(np.uint32), w2[0].view(np.uint32))
    with np.errstate(over="ignore"):
        assert np.array_equal(p[0].view(np.uint16), w2[0].astype(np.float16).view(np.uint16))
