"""The parity tests' own machinery, checked on the CPU: the oracle's clip-norm hook and the
helper that lets an oracle step follow the device's norm."""
from types import SimpleNamespace

import numpy as np

import oracle as O
from tests import helpers as H


def _grads():
    return [O.randn_f32(1000, 7, 1.0), O.randn_f32(333, 8, 1.0)]


def test_clip_norm_hook_replaces_the_norm_but_not_the_return_value():
    g = _grads()
    own = O.clip_grad_norm(H.copy_list(g), 1e30)  # no clipping: just the serial norm
    assert abs(own - np.sqrt(sum(float(np.sum(a.astype(np.float64) ** 2)) for a in g))) < 1e-12 * own
    fake = own * 2.0
    a, b = H.copy_list(g), H.copy_list(g)
    O.set_clip_norm_override(fake)
    try:
        ret = O.clip_grad_norm(a, 1.0)
    finally:
        O.set_clip_norm_override(-1.0)
    assert ret == own, "the hook must not change what clip_grad_norm returns"
    c = np.float32(1.0 / fake)
    H.assert_bits_equal(a, [x * c for x in g], "gradients scaled with the overriding norm")
    assert O.clip_grad_norm(b, 1.0) == own  # hook off again
    H.assert_bits_equal(b, [x * np.float32(1.0 / own) for x in g], "gradients scaled with the serial norm")


def test_an_oracle_step_follows_the_device_norm_only_when_the_factor_differs():
    shapes = [(1, 1000), (1, 333)]
    g = _grads()
    p0 = H.randn_list(shapes, 3, 0.02)
    serial = O.clip_grad_norm(H.copy_list(g), 1e30)
    # a max_norm for which max_norm / serial sits on a rounding boundary of f32: the middle
    # between two neighbouring f32 values, so that a norm a few f64 ulps away narrows differently
    f = np.float32(0.37)
    middle = (float(f) + float(np.nextafter(f, np.float32(1)))) / 2.0
    max_norm = middle * serial

    def factor(n):
        return np.float32(max_norm / n)

    def run(dev_norm):
        meta = O.adam_meta(1e-3)
        p, m, v = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0)
        before = H.NORM_FOLLOWED["events"]
        ran, norm = H.oracle_step_with_device_norm(
            lambda: O.f32_step(meta, None, max_norm, p, H.copy_list(g), m, v), [p, m, v], [meta], max_norm,
            SimpleNamespace(found_inf=0, norm=dev_norm) if dev_norm else None, "cpu check")
        assert ran and norm == serial
        return p, m, meta.step_count, H.NORM_FOLLOWED["events"] - before

    p_plain, m_plain, sc, ev = run(None)
    assert sc == 1 and ev == 0
    # the same norm: nothing is repeated
    p_same, _, sc, ev = run(serial)
    assert ev == 0 and sc == 1
    H.assert_bits_equal(p_same, p_plain, "params")
    # norms a few f64 ulps away, to either side: one that narrows to the same factor changes
    # nothing, one that narrows to the other factor makes the oracle repeat its step with it
    same = flipped = None
    for j in range(1, 200):
        for cand in (serial * (1.0 + j * 2.0 ** -52), serial * (1.0 - j * 2.0 ** -52)):
            if factor(cand) == factor(serial):
                same = same or cand
            else:
                flipped = flipped or cand
    assert same is not None and flipped is not None, "the boundary was placed a few f64 ulps from the serial norm"
    assert run(same)[3] == 0
    p_f, m_f, sc, ev = run(flipped)
    assert ev == 1 and sc == 1, "the step was repeated once, and step_count advanced once"
    c = factor(flipped)
    assert c != factor(serial)
    meta = O.adam_meta(1e-3)
    p, m, v = H.copy_list(p0), H.zeros_like_list(p0), H.zeros_like_list(p0)
    O.adam_step(meta, p, [a * c for a in g], m, v)
    H.assert_bits_equal(p_f, p, "params follow the device's norm")
    H.assert_bits_equal(m_f, m, "m follows the device's norm")
    assert any(not np.array_equal(a, b) for a, b in zip(m_f, m_plain)), "the two factors give different moments"
    # norms further apart than the bar are refused, not followed
    try:
        run(serial * (1.0 + 1e-9))
    except AssertionError as e:
        assert "device norm" in str(e)
    else:
        raise AssertionError("norms 1e-9 apart must be refused")
