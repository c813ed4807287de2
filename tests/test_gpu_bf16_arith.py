"""The all-16-bit optimizers' division and square root against the exact operations, exhaustively:
every pair of 16-bit patterns, every 16-bit pattern."""
import ctypes as C

import pytest

from nabla_amd import _lib


@pytest.mark.gpu
@pytest.mark.parametrize("half", ["bf16", "f16"])
def test_16_bit_division_and_square_root_equal_the_exact_operations_for_every_operand(gpu, half):
    """Optimizer<bf16> / Optimizer<f16> divide and take square roots of 16-bit numbers (the f32
    operation, rounded to the type: common/scalar/mod.rs:253-351).  The bf16 kernels use the
    hardware's approximate reciprocal and square root where the operands' 8 significant bits
    guarantee the same bf16, and the exact operation elsewhere; for f16 the compiler lowers the
    division whose result is narrowed to f16 more cheaply than a correctly rounded f32 division.
    The library compares what the kernels compute with the exact operation (through f64; bf16 also
    bit for bit with the correctly rounded f32 operation) on the device for all 2^32 quotients and
    all 2^16 square roots, signed zeros, subnormals and infinities included."""
    _lib.init()
    lib = _lib.load()
    div, sq, pair, arg = C.c_uint64(1), C.c_uint64(1), C.c_uint64(0), C.c_uint64(0)
    _lib.check(lib.nbo_selftest_half_arith({"bf16": _lib.DT_BF16, "f16": _lib.DT_F16}[half], C.byref(div), C.byref(sq), C.byref(pair), C.byref(arg)))
    assert (div.value, sq.value) == (0, 0), (
        f"{div.value} quotients differ (e.g. {pair.value >> 16:#06x} / {pair.value & 0xFFFF:#06x}), "
        f"{sq.value} square roots (e.g. of {arg.value:#06x})")


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["adam", "adamw"])
def test_bf16_adam_over_gradients_of_every_magnitude_is_bit_exact(gpu, kind):
    """Optimizer<bf16> steps whose gradients span 1e-30 .. 1e25 (and exact zeros) in every vector:
    second moments that are subnormal (the square root's exact path), that overflow to infinity
    (a denominator whose reciprocal is zero: the quotient's exact path) and ordinary ones side by
    side in one wave, against the oracle's bf16 chain bit for bit -- the all-bf16 update kernels
    take the exact operation only in the lanes that need it."""
    import numpy as np

    import oracle as O
    from nabla_amd import optim as nb
    from tests import helpers as H

    shapes = [(1, 8192 * 2 + 37), (5, 1001), (1, 7)]
    rng = np.random.default_rng(77)

    def grads(step):
        out = []
        for a in H.randn_list(shapes, 8100 + step, 1.0):
            mag = 10.0 ** rng.integers(-30, 26, size=a.shape).astype(np.float64)
            g = (a.astype(np.float64) * mag).astype(np.float32)
            g[rng.random(a.shape) < 0.05] = 0.0
            out.append(g)
        return H.narrow_list(out, "bf16")

    p0 = H.narrow_list(H.randn_list(shapes, 8000, 0.5), "bf16")
    p_dev = H.dev_list(p0, shapes)
    if kind == "adam":
        opt, meta = nb.Adam.new(1e-2, shapes, dtype="bf16"), O.adam_meta(1e-2, 0.9, 0.999, 1e-8)
    else:
        opt = nb.AdamW.new(1e-2, shapes, dtype="bf16").beta2(0.95).weight_decay(0.1)
        meta = O.adamw_meta(1e-2, 0.9, 0.95, 1e-8, 0.1)
    pr, m, v = H.copy_list(p0), [np.zeros_like(a) for a in p0], [np.zeros_like(a) for a in p0]
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(6):
            g = grads(step)
            opt.step(p_dev, H.dev_list(g, shapes))
            O.adam_step(meta, pr, g, m, v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    vs = np.concatenate([O.bf16_to_f32(x).ravel() for x in v])
    assert np.isinf(vs).any() and ((vs > 0) & (vs < 1.2e-38)).any(), "the inputs must reach both exact paths"
    H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")
    H.assert_bits_equal(H.host_list(opt.moments()[0]), m, "m")
    H.assert_bits_equal(H.host_list(p_dev), pr, "params")
