"""The Backend primitives as multi-tensor launches (nabla_amd.backend over
nbo_backend_apply / nbo_backend_cast) against the CPU oracle's restatement of
nabla-core/src/cpu/mod.rs: bit-exact for every operation and element type, except powf
with an exponent other than 0.5 (device math library, within 2 ulp of libm)."""
import numpy as np
import pytest

import oracle as O
from nabla_amd import backend as B
from nabla_amd import optim as nb
from tests import helpers as H

pytestmark = pytest.mark.gpu

# around the work-chunk (8192) and vector (4 / 2 elements) boundaries, an empty tensor
SHAPES = [(1, 1), (1, 3), (3, 5), (1, 4097), (64, 130), (1, 8191), (1, 8192), (1, 8193), (0, 7), (5, 3300)]
NP_DTYPE = {"f32": np.float32, "f64": np.float64}


def _inputs(dtype, seed, sigma=1.0, positive=False):
    base = H.randn_list(SHAPES, seed, sigma, np.float64)
    if positive:
        base = [np.abs(a) + 1e-3 for a in base]
    if dtype in ("bf16", "f16"):
        return [O.cast(a, np.uint16 if dtype == "bf16" else np.float16) for a in base]
    return [a.astype(NP_DTYPE[dtype]) for a in base]


def _empty_like(arrs):
    return H.dev_list([np.zeros_like(a) for a in arrs], SHAPES)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f64", "f16"])
def test_every_primitive_bit_exact(gpu, dtype):
    a, b = _inputs(dtype, 900), _inputs(dtype, 950, positive=True)
    da, db = H.dev_list(a, SHAPES), H.dev_list(b, SHAPES)
    s = 0.3

    out = _empty_like(a)
    B.scale(da, s, out=out)
    H.assert_bits_equal(H.host_list(out), [O.scale(x, s) for x in a], "scale")

    B.add(da, db, out=out)
    H.assert_bits_equal(H.host_list(out), [O.add(x, y) for x, y in zip(a, b)], "add")

    B.emul(da, db, out=out)
    H.assert_bits_equal(H.host_list(out), [O.emul(x, y) for x, y in zip(a, b)], "emul")

    B.ediv(da, db, out=out)
    H.assert_bits_equal(H.host_list(out), [O.ediv(x, y) for x, y in zip(a, b)], "ediv")

    B.map_add(da, 1e-3, out=out)
    H.assert_bits_equal(H.host_list(out), [O.map_add(x, 1e-3) for x in a], "map(|x| x + c)")

    y = H.dev_list(b, SHAPES)
    B.axpy_inplace(y, -s, da)
    want = H.copy_list(b)
    for w, x in zip(want, a):
        O.axpy_inplace(w, -s, x)
    H.assert_bits_equal(H.host_list(y), want, "axpy_inplace")

    O.set_pow_mode(O.POW_SQRT)
    try:
        want = [O.powf(x, 0.5) for x in b]
    finally:
        O.set_pow_mode(O.POW_LIBM)
    B.powf(db, 0.5, out=out)
    H.assert_bits_equal(H.host_list(out), want, "powf(x, 0.5)")

    B.clone_storage(da, out=out)
    H.assert_bits_equal(H.host_list(out), a, "clone_storage")
    B.zeros(out)
    assert not any(t.any() for t in H.host_list(out))
    # in place: the output list may be an operand
    B.emul(da, db, out=da)
    H.assert_bits_equal(H.host_list(da), [O.emul(x, y) for x, y in zip(a, b)], "emul in place")


@pytest.mark.parametrize("dtype,tol", [("f32", 2), ("f64", 2)])
def test_powf_general_exponent_within_2_ulp_of_libm(gpu, dtype, tol):
    b = _inputs(dtype, 960, positive=True)
    out = _empty_like(b)
    for p in (2.0, 1.5, -0.5, 0.3333):
        B.powf(H.dev_list(b, SHAPES), p, out=out)
        for got, x in zip(H.host_list(out), b):
            if not x.size:
                continue
            want = O.powf(x, p)
            if dtype == "f32":
                assert int(O.ulp_distance_f32(got, want).max()) <= tol, p
            else:
                ulp = np.abs(got.view(np.int64) - want.view(np.int64))
                assert int(ulp.max()) <= tol, p


def test_powf_half_special_cases_follow_c_pow(gpu):
    x = np.array([-0.0, -np.inf, np.inf, 0.0, 4.0, -1.0], dtype=np.float32)
    d = H.to_dev(x, (1, 6))
    B.powf([d], 0.5, out=[d])
    got = H.to_host(d)
    assert np.array_equal(got[:5].view(np.uint32),
                          np.array([0.0, np.inf, np.inf, 0.0, 2.0], dtype=np.float32).view(np.uint32))
    assert np.isnan(got[5])


@pytest.mark.parametrize("src,dst", [("f64", "bf16"), ("f64", "f32"), ("f32", "bf16"), ("bf16", "f32"),
                                     ("bf16", "f64"), ("f32", "f64"), ("f32", "f32"), ("f64", "f16"),
                                     ("f32", "f16"), ("f16", "f32"), ("f16", "f64"), ("f16", "bf16"),
                                     ("bf16", "f16")])
def test_cast_bit_exact(gpu, src, dst):
    np_of = {"f32": np.float32, "f64": np.float64, "bf16": np.uint16, "f16": np.float16}
    a = H.randn_list(SHAPES, 970, 3.0, np.float64)
    a[3][:3] = [1.0 + 2.0 ** -8 + 2.0 ** -30, -(1.0 + 3 * 2.0 ** -8 - 2.0 ** -40), 1e-42]  # double-rounding ties, f32 subnormal
    a = [O.cast(x, np_of[src]) for x in a]
    out = H.dev_list([np.zeros(x.shape, dtype=np_of[dst]) for x in a], SHAPES)
    B.cast(H.dev_list(a, SHAPES), out)
    H.assert_bits_equal(H.host_list(out), [O.cast(x, np_of[dst]) for x in a], f"cast {src} -> {dst}")


def test_unaligned_tensors_take_the_element_path(gpu):
    """Views into one buffer at odd element offsets: addresses that are not 16-byte
    aligned must give the same bits."""
    import torch

    n = [5, 4099, 8200]
    a = [O.randn_f32(k, 980 + i) for i, k in enumerate(n)]
    b = [O.randn_f32(k, 990 + i) for i, k in enumerate(n)]
    buf_a = torch.zeros(sum(n) + 8, dtype=torch.float32, device="cuda:0")
    buf_o = torch.zeros(sum(n) + 8, dtype=torch.float32, device="cuda:0")
    va, vo, off = [], [], 1
    for k, x in zip(n, a):
        va.append(buf_a[off:off + k].reshape(1, k))
        vo.append(buf_o[off:off + k].reshape(1, k))
        va[-1].copy_(torch.from_numpy(x).reshape(1, k))
        off += k + 1
    assert any(v.data_ptr() % 16 for v in va)
    db = H.dev_list(b, [(1, k) for k in n])
    B.add(va, db, out=vo)
    H.assert_bits_equal(H.host_list(vo), [O.add(x, y) for x, y in zip(a, b)], "add on unaligned views")


def test_shape_and_dtype_mismatches_are_the_reference_panics(gpu):
    a = H.dev_list([np.zeros(6, np.float32)], [(2, 3)])
    with pytest.raises(nb.NablaPanic, match=r"axpy_inplace \(2x3\) vs \(3x2\) -- shapes must match"):
        B.axpy_inplace(a, 1.0, H.dev_list([np.zeros(6, np.float32)], [(3, 2)]))
    with pytest.raises(nb.NablaPanic, match="tensor lists differ in length"):
        B.add(a, a + a, out=a)
    with pytest.raises(Exception, match="element type"):
        B.add(a, H.dev_list([np.zeros(6, np.float64)], [(2, 3)]), out=a)


def test_adamw_as_a_chain_of_primitives_equals_the_fused_kernel(gpu):
    """AdamW::step written out pass by pass as the reference does (optim/alg.rs:109-150),
    every pass a multi-tensor primitive launch on the device, against the fused update
    kernel: same bits after every step.  The scalars are narrowed on the host exactly as
    alg.rs:121-135 does."""
    shapes = [(3, 5), (1, 9001), (129, 257), (1, 8192)]
    p0 = H.randn_list(shapes, 1000, 0.02)
    lr, b1, b2, eps, wd = 1e-3, 0.9, 0.95, 1e-8, 0.1
    fused_p = H.dev_list(p0, shapes)
    opt = nb.AdamW.new(lr, shapes).beta1(b1).beta2(b2).eps(eps).weight_decay(wd)
    p = H.dev_list(p0, shapes)
    m, v = H.dev_list(H.zeros_like_list(p0), shapes), H.dev_list(H.zeros_like_list(p0), shapes)
    t1, t2 = H.dev_list(H.zeros_like_list(p0), shapes), H.dev_list(H.zeros_like_list(p0), shapes)
    f32 = np.float32
    for step in range(1, 6):
        g = H.dev_list(H.randn_list(shapes, 2000 + 10 * step, 1e-3), shapes)
        opt.step(fused_p, g)
        bc1, bc2 = 1.0 - O.powi(b1, step), 1.0 - O.powi(b2, step)
        ss, ibc2, wd_lr = float(f32(lr / bc1)), float(f32(1.0 / bc2)), f32(wd * lr)
        B.scale(m, b1, out=m)                      # m = &m * beta1
        B.axpy_inplace(m, 1.0 - b1, g)             # m.axpy_inplace(1 - beta1, g)
        B.scale(v, b2, out=v)                      # v = &v * beta2
        B.emul(g, g, out=t1)                       # g_sq = g.emul(g)
        B.axpy_inplace(v, 1.0 - b2, t1)            # v.axpy_inplace(1 - beta2, &g_sq)
        B.scale(v, ibc2, out=t1)                   # v_scaled = &v * inv_bc2
        B.powf(t1, 0.5, out=t1)                    # .powf(0.5)
        B.map_add(t1, eps, out=t1)                 # .map(|x| x + eps)
        B.scale(m, ss, out=t2)                     # m_scaled = &m * step_size
        B.ediv(t2, t1, out=t2)                     # update = m_scaled.ediv(&denom)
        B.scale(p, float(f32(1.0) - wd_lr), out=p)  # p = &p * (1 - wd_lr), computed in T
        B.axpy_inplace(p, -1.0, t2)                # p.axpy_inplace(-1, &update)
        H.assert_bits_equal(H.host_list(p), H.host_list(fused_p), f"params after step {step}")
        H.assert_bits_equal(H.host_list(m), H.host_list(opt.moments()[0]), f"m after step {step}")
        H.assert_bits_equal(H.host_list(v), H.host_list(opt.moments()[1]), f"v after step {step}")


def test_f32_to_bf16_rounding_for_every_high_half_and_boundary_low_half(gpu):
    """The device narrows f32 to bf16 with gfx950's conversion instruction.  Every 16-bit
    high half (all signs, exponents, top mantissa bits, infinities and NaNs) is combined
    with the low halves that decide a rounding -- 0, 1, just below the tie, the tie, just
    above it, all ones -- and must give half::bf16::from_f32's bits, NaN payloads included."""
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    x = bits.view(np.float32)
    n = x.size
    src = H.to_dev(x, (1, n))
    dst = H.to_dev(np.zeros(n, dtype=np.uint16), (1, n))
    B.cast([src], [dst])
    got, want = H.to_host(dst), O.bf16_from_f32(x)
    assert np.array_equal(got, want), f"first difference at input bits {bits[np.nonzero(got != want)[0][0]]:#010x}"


def test_f32_to_f16_and_back_for_every_high_half_and_boundary_low_bits(gpu):
    """The device converts between f32 and f16 with gfx950's conversion instructions.  An f16
    keeps 10 mantissa bits, so bit 12 of an f32 decides the rounding of a normal result;
    every 16-bit high half (all signs, exponents, infinities, NaNs; the exponents that land
    among f16's subnormals and beyond its largest value included) is combined with low halves
    around that tie and must give half::f16::from_f32's bits, NaN payloads included.  Every
    one of the 65536 f16 patterns must widen to f32::from(f16)'s bits."""
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x0FFF, 0x1000, 0x1001, 0x2000, 0x2FFF, 0x3000, 0x3001, 0x7FFF, 0x8000,
                     0xE000, 0xEFFF, 0xF000, 0xF001, 0xFFFF], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    x = bits.view(np.float32)
    n = x.size
    dst = H.to_dev(np.zeros(n, dtype=np.float16), (1, n))
    B.cast([H.to_dev(x, (1, n))], [dst])
    got, want = H.to_host(dst).view(np.uint16), O.cast(x, np.float16).view(np.uint16)
    assert np.array_equal(got, want), f"first difference at input bits {bits[np.nonzero(got != want)[0][0]]:#010x}"

    h = np.arange(1 << 16, dtype=np.uint16).view(np.float16)
    wide = H.to_dev(np.zeros(h.size, dtype=np.float32), (1, h.size))
    B.cast([H.to_dev(h, (1, h.size))], [wide])
    got, want = H.to_host(wide).view(np.uint32), O.cast(h, np.float32).view(np.uint32)
    assert np.array_equal(got, want), f"first difference at f16 bits {np.nonzero(got != want)[0][0]:#06x}"
