"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU half: the oracle on this host reproduces the committed bits -- moments, SGD
params, decisions and the sqrt-variant params exactly; the libm-powf params within
2 ulp, because glibc selects its powf build by CPU model.
GPU half: the HIP engine, through the C ABI, against the same committed data.
"""
import os

import numpy as np
import pytest

import oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
SHAPES = [(1, 1), (3, 5), (1, 1000), (2, 4100)]
N = len(SHAPES)


def _load(name):
    return dict(np.load(os.path.join(GOLD, name)))


def _bits_equal(a, b):
    return a.dtype == b.dtype and np.array_equal(a.view(np.uint8), b.view(np.uint8))


# ---- CPU: oracle vs fixture -------------------------------------------------------------------

def test_oracle_reproduces_sgd_fixture():
    d = _load("sgd_f32.npz")
    p = [d[f"p0_{i}"].copy() for i in range(N)]
    vel = [np.zeros_like(a) for a in p]
    meta = O.sgd_meta(0.01)
    for step in range(3):
        O.sgd_step(meta, p, [d[f"g{step}_{i}"] for i in range(N)], vel)
    for i in range(N):
        assert _bits_equal(p[i], d[f"p_{i}"])


@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_oracle_reproduces_adam_fixture(kind):
    d = _load(f"{kind}_f32.npz")
    for mode, key in ((O.POW_SQRT, "p_sqrt"), (O.POW_LIBM, "p_libm")):
        p = [d[f"p0_{i}"].copy() for i in range(N)]
        m, v = [np.zeros_like(a) for a in p], [np.zeros_like(a) for a in p]
        meta = O.adam_meta(3e-4) if kind == "adam" else O.adamw_meta(2e-4, 0.9, 0.95, 1e-8, 0.1)
        O.set_pow_mode(mode)
        try:
            for step in range(3):
                O.adam_step(meta, p, [d[f"g{step}_{i}"] for i in range(N)], m, v)
        finally:
            O.set_pow_mode(O.POW_LIBM)
        for i in range(N):
            assert _bits_equal(m[i], d[f"m_{i}"]) and _bits_equal(v[i], d[f"v_{i}"])
            if mode == O.POW_SQRT:
                assert _bits_equal(p[i], d[f"{key}_{i}"])
            else:
                assert O.ulp_distance_f32(p[i], d[f"{key}_{i}"]).max() <= 2


def _narrow(a, half):
    return O.bf16_from_f32(a) if half == "bf16" else O.cast(a, np.float16)


@pytest.mark.parametrize("half", ["bf16", "f16"])
def test_oracle_reproduces_mixed_fixture(half):
    d = _load(f"mixed_adamw_{half}.npz")
    w = [d[f"w0_{i}"].copy() for i in range(N)]
    p = [_narrow(a, half) for a in w]
    m, v = [np.zeros_like(a) for a in w], [np.zeros_like(a) for a in w]
    meta, s = O.adamw_meta(2e-4, 0.9, 0.95, 1e-8, 0.1), O.ScalerState(65536.0, 2.0, 0.5, 2, 0)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(6):
            ran, norm = O.mixed_step(meta, s, 1.0, p, [d[f"g{step}_{i}"] for i in range(N)], w, m, v)
            f, scale, sc, nrm = d["trace"][step]
            assert (0.0 if ran else 1.0, s.scale, float(meta.step_count), norm) == (f, scale, sc, nrm)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert list(d["trace"][:, 0]) == [0, 0, 0, 1, 0, 0]
    assert list(d["trace"][:, 1]) == [65536.0, 131072.0, 131072.0, 65536.0, 65536.0, 131072.0]
    for i in range(N):
        assert _bits_equal(p[i], d[f"p_sqrt_{i}"]) and _bits_equal(w[i], d[f"w_sqrt_{i}"])
        assert _bits_equal(m[i], d[f"m_{i}"]) and _bits_equal(v[i], d[f"v_{i}"])
        assert O.ulp_distance_bf16(d[f"p_libm_{i}"].view(np.uint16), d[f"p_sqrt_{i}"].view(np.uint16)).max() <= 1
        # the two lowerings of powf differ by an ulp of the update; where decay and update nearly
        # cancel that is more than 2 ulp of the small result, and bounded by steps * 8 * lr * 2^-23
        far = O.ulp_distance_f32(d[f"w_libm_{i}"], d[f"w_sqrt_{i}"]) > 2
        assert np.abs(d[f"w_libm_{i}"][far].astype(np.float64) - d[f"w_sqrt_{i}"][far]).max(initial=0.0) \
            <= 6 * 8 * 2e-4 * 2.0 ** -23


# ---- GPU: HIP engine vs fixture ------------------------------------------------------------------

@pytest.mark.gpu
def test_device_matches_sgd_fixture(gpu):
    from nabla_amd import optim as nb
    from tests import helpers as H

    d = _load("sgd_f32.npz")
    p = H.dev_list([d[f"p0_{i}"] for i in range(N)], SHAPES)
    opt = nb.Sgd.new(0.01, SHAPES)
    for step in range(3):
        opt.step(p, H.dev_list([d[f"g{step}_{i}"] for i in range(N)], SHAPES))
    H.assert_bits_equal(H.host_list(p), [d[f"p_{i}"] for i in range(N)], "SGD fixture")


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_device_matches_adam_fixture(gpu, kind):
    from nabla_amd import optim as nb
    from tests import helpers as H

    d = _load(f"{kind}_f32.npz")
    p = H.dev_list([d[f"p0_{i}"] for i in range(N)], SHAPES)
    opt = nb.Adam.new(3e-4, SHAPES) if kind == "adam" else \
        nb.AdamW.new(2e-4, SHAPES).beta2(0.95).weight_decay(0.1)
    for step in range(3):
        opt.step(p, H.dev_list([d[f"g{step}_{i}"] for i in range(N)], SHAPES))
    m, v = opt.moments()
    H.assert_bits_equal(H.host_list(m), [d[f"m_{i}"] for i in range(N)], "m fixture")
    H.assert_bits_equal(H.host_list(v), [d[f"v_{i}"] for i in range(N)], "v fixture")
    got = H.host_list(p)
    H.assert_bits_equal(got, [d[f"p_sqrt_{i}"] for i in range(N)], "params, sqrt variant")
    assert H.max_ulp_f32(got, [d[f"p_libm_{i}"] for i in range(N)]) <= 2


@pytest.mark.gpu
@pytest.mark.parametrize("half", ["bf16", "f16"])
def test_device_matches_mixed_fixture(gpu, half):
    from nabla_amd import optim as nb
    from tests import helpers as H

    d = _load(f"mixed_adamw_{half}.npz")
    w0 = [d[f"w0_{i}"] for i in range(N)]
    p = H.dev_list([_narrow(a, half) for a in w0], SHAPES)
    opt = nb.AdamW.new(2e-4, SHAPES, master=True).beta2(0.95).weight_decay(0.1)
    for i in range(N):
        opt.write_state(f"w{i}", H.to_dev(w0[i], SHAPES[i]))
    scaler = nb.GradScaler.new()
    scaler.load_state(nb.GradScalerState(65536.0, 2.0, 0.5, 2, 0))
    for step in range(6):
        opt.fused_step(p, H.dev_list([d[f"g{step}_{i}"] for i in range(N)], SHAPES), scaler=scaler,
                       max_norm=1.0)
    tr = opt.trace()
    assert [t.found_inf for t in tr] == [int(x) for x in d["trace"][:, 0]]
    assert [t.scale for t in tr] == list(d["trace"][:, 1])
    assert [t.step_count for t in tr] == [int(x) for x in d["trace"][:, 2]]
    for t, ref in zip(tr, d["trace"][:, 3]):
        assert t.norm == pytest.approx(ref, rel=1e-12)
    H.assert_bits_equal(H.host_list(p), [d[f"p_sqrt_{i}"] for i in range(N)], "16-bit params")
    H.assert_bits_equal(H.host_list([opt.read_state(f"w{i}") for i in range(N)]),
                        [d[f"w_sqrt_{i}"] for i in range(N)], "master")
    m, v = opt.moments()
    H.assert_bits_equal(H.host_list(m), [d[f"m_{i}"] for i in range(N)], "m")
    H.assert_bits_equal(H.host_list(v), [d[f"v_{i}"] for i in range(N)], "v")
    assert H.max_ulp_half(H.host_list(p), [d[f"p_libm_{i}"] for i in range(N)]) <= 1
