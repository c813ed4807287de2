"""The element-wise passes and the SGD step run one workgroup per 4 KiB piece (one row) of a
work chunk, and leave a chunk that is ragged or not vector-aligned to the workgroup of its first
piece.  Every combination of whole / ragged chunks and aligned / unaligned addresses must give
the oracle's bits: a piece done twice, skipped, or done by both paths would show here.

Lists of several tensors as views into one buffer, at an aligned offset and at an odd element
offset; sizes below one piece, between piece and chunk, exactly one chunk, chunks plus a ragged
rest, and a few whole chunks."""
import numpy as np
import pytest

import oracle as O
from nabla_amd import optim as nb
from tests import helpers as H

pytestmark = pytest.mark.gpu

# Two lists: in the first nine chunks in ten are whole, so the passes run one workgroup per piece
# (and its ragged and unaligned chunks are the exceptions inside such a launch); the second is a
# list of small tensors, which the library runs one workgroup per chunk (and the optimizers by row
# over a map of the rows that exist).
SIZES_OF = {"mostly whole": [5, 1024, 4099, 8192, 8200, 3 * 8192, 20011, 40 * 8192],
            "small tensors": [5, 1024, 4099, 8192, 8200, 3 * 8192, 20011]}
NP = {"f32": np.float32, "f64": np.float64}


def _views(arrs, odd, torch_dtype):
    """The arrays as (1, n) views into one device buffer; with `odd`, each starts one element
    past a 16-byte boundary."""
    import torch

    pad = 16
    total = sum((a.size + pad + 15) // 16 * 16 for a in arrs) + pad
    buf = torch.zeros(total, dtype=torch_dtype, device="cuda:0")
    views, off = [], 0
    for a in arrs:
        start = off + (1 if odd else 0)
        v = buf[start:start + a.size].reshape(1, a.size)
        src = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16) if a.dtype == np.uint16 else torch.from_numpy(a.copy())
        v.copy_(src.reshape(1, a.size))
        views.append(v)
        off += (a.size + pad + 15) // 16 * 16
    assert all((v.data_ptr() % 16 != 0) == odd for v in views)
    return buf, views


def _make(dtype, seed, sigma, odd, sizes):
    import torch

    if dtype == "bf16":
        arrs = [O.bf16_from_f32(O.randn_f32(n, seed + i, sigma)) for i, n in enumerate(sizes)]
        return arrs, _views(arrs, odd, torch.bfloat16)
    arrs = [(O.randn_f64(n, seed + i) * sigma).astype(NP[dtype]) for i, n in enumerate(sizes)]
    return arrs, _views(arrs, odd, torch.float32 if dtype == "f32" else torch.float64)


def _as_f32(arrs):
    return [O.bf16_to_f32(a) if a.dtype == np.uint16 else a for a in arrs]


def _like(ref_f32, like):
    return [O.bf16_from_f32(a) if b.dtype == np.uint16 else a for a, b in zip(ref_f32, like)]


@pytest.mark.parametrize("kind", list(SIZES_OF))
@pytest.mark.parametrize("odd", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "bf16", "f64"])
def test_scale_zero_and_accumulate_over_views(gpu, dtype, odd, kind):
    sizes = SIZES_OF[kind]
    g0, (gbuf, g) = _make(dtype, 11, 1.0, odd, sizes)
    a0, (abuf, a) = _make(dtype, 31, 1.0, odd, sizes)
    before_g, before_a = gbuf.clone(), abuf.clone()

    # scale_grad: g * T(factor), rounded to the element type
    nb.scale_grad(g, 0.3)
    ref = [x.copy() for x in g0]
    O.scale_grad(ref, 0.3)
    H.assert_bits_equal(H.host_list(g), ref, f"scale_grad {dtype} odd={odd} {kind}")

    # accumulate: a + g in the element type (bf16: the f32 sum rounded)
    nb.accumulate(a, g)
    acc = [O.add(x, y) for x, y in zip(a0, ref)]
    H.assert_bits_equal(H.host_list(a), acc, f"accumulate {dtype} odd={odd} {kind}")
    H.assert_bits_equal(H.host_list(g), ref, "accumulate leaves the gradients")

    # accumulate and clear
    nb.accumulate(a, g, True)
    acc = [O.add(x, y) for x, y in zip(acc, ref)]
    H.assert_bits_equal(H.host_list(a), acc, f"accumulate + zero {dtype} odd={odd}")
    assert not any(t.any() for t in H.host_list(g))

    # zero_grad
    nb.zero_grad(a)
    assert not any(t.any() for t in H.host_list(a))

    # nothing outside the views was touched: the gaps between them still hold zeros
    import torch

    for buf, before, views in ((gbuf, before_g, g), (abuf, before_a, a)):
        mask = torch.ones_like(buf, dtype=torch.bool)
        base = buf.data_ptr()
        for v in views:
            s = (v.data_ptr() - base) // buf.element_size()
            mask[s:s + v.numel()] = False
        assert bool((buf[mask] == before[mask]).all()) and not bool(buf[mask].any())


@pytest.mark.parametrize("kind", list(SIZES_OF))
@pytest.mark.parametrize("odd", [False, True])
@pytest.mark.parametrize("dtype", ["f32", "f64"])
@pytest.mark.parametrize("momentum,wd", [(0.0, 0.0), (0.9, 0.01)])
def test_sgd_steps_over_views(gpu, dtype, odd, momentum, wd, kind):
    sizes = SIZES_OF[kind]
    p0, (pbuf, p) = _make(dtype, 51, 0.05, odd, sizes)
    g0, (_, g) = _make(dtype, 71, 1e-2, odd, sizes)
    shapes = [(1, n) for n in sizes]
    opt = nb.Sgd.new(0.05, shapes, dtype=dtype).momentum(momentum).weight_decay(wd)
    meta = O.sgd_meta(0.05, momentum=momentum, weight_decay=wd)
    ref, vel = [x.copy() for x in p0], [np.zeros_like(x) for x in p0]
    for _ in range(3):
        opt.step(p, g)
        O.sgd_step(meta, ref, g0, vel)
    H.assert_bits_equal(H.host_list(p), ref, f"Sgd {dtype} odd={odd} momentum={momentum}")
    H.assert_bits_equal(H.host_list(g), g0, "Sgd leaves the gradients")


@pytest.mark.parametrize("kind", list(SIZES_OF))
@pytest.mark.parametrize("odd", [False, True])
def test_backend_add_cast_and_adam_over_views(gpu, odd, kind):
    """The backend primitives (two rows per workgroup), the cast (one workgroup per 2048 elements)
    and the unfused and fused Adam kinds over the same two lists."""
    import torch

    from nabla_amd import backend as B

    sizes = SIZES_OF[kind]
    shapes = [(1, n) for n in sizes]
    a0, (_, a) = _make("f32", 91, 1.0, odd, sizes)
    b0, (_, b) = _make("f32", 92, 1.0, odd, sizes)
    _, (obuf, o) = _make("f32", 93, 1.0, odd, sizes)
    B.add(a, b, out=o)
    H.assert_bits_equal(H.host_list(o), [O.add(x, y) for x, y in zip(a0, b0)], f"backend add odd={odd} {kind}")
    B.axpy_inplace(o, 0.25, a)
    ref = [O.add(x, y) for x, y in zip(a0, b0)]
    for r, x in zip(ref, a0):
        O.axpy_inplace(r, 0.25, x)
    H.assert_bits_equal(H.host_list(o), ref, f"backend axpy odd={odd} {kind}")
    h0, (_, h) = _make("bf16", 94, 1.0, odd, sizes)
    B.cast(a, h)
    H.assert_bits_equal(H.host_list(h), [O.bf16_from_f32(x) for x in a0], f"cast f32 -> bf16 odd={odd} {kind}")
    B.cast(h, o)
    H.assert_bits_equal(H.host_list(o), [O.bf16_to_f32(O.bf16_from_f32(x)) for x in a0], f"cast bf16 -> f32 odd={odd} {kind}")

    O.set_pow_mode(O.POW_SQRT)
    try:
        p0, (_, p) = _make("f32", 95, 0.02, odd, sizes)
        g0, (_, g) = _make("f32", 96, 1e-3, odd, sizes)
        opt = nb.Adam.new(1e-3, shapes)
        meta = O.adam_meta(1e-3)
        ref, m, v = [x.copy() for x in p0], [np.zeros_like(x) for x in p0], [np.zeros_like(x) for x in p0]
        for _ in range(3):
            opt.step(p, g)
            O.adam_step(meta, ref, g0, m, v)
        H.assert_bits_equal(H.host_list(p), ref, f"Adam odd={odd} {kind}")
        H.assert_bits_equal(H.host_list(opt.moments()[1]), v, "v")
        fused = nb.AdamW.new(2e-4, shapes).weight_decay(0.1)
        fmeta = O.adamw_meta(2e-4, weight_decay=0.1)
        m, v = [np.zeros_like(x) for x in p0], [np.zeros_like(x) for x in p0]
        for _ in range(2):
            fused.fused_step(p, g)
            O.adam_step(fmeta, ref, g0, m, v)
        H.assert_bits_equal(H.host_list(p), ref, f"fused AdamW odd={odd} {kind}")
    finally:
        O.set_pow_mode(O.POW_LIBM)


@pytest.mark.parametrize("kind", list(SIZES_OF))
@pytest.mark.parametrize("p_off,g_off", [(0, 0), (1, 1), (1, 3), (0, 5), (2, 0)])
def test_mixed_adamw_over_views_misaligned_each_in_its_own_way(gpu, kind, p_off, g_off):
    """bf16 parameters and gradients over f32 master weights, the parameter views starting p_off
    elements and the gradient views g_off elements past a 16-byte boundary: the update reads the
    state in whole aligned vectors and the tensors at element alignment, whatever the two offsets
    are, with and without zeroing of the gradients; neighbours of every view stay untouched."""
    import torch

    sizes = SIZES_OF[kind]
    shapes = [(1, n) for n in sizes]

    def views(arrs, off_elems):
        pad = 16
        total = sum((a.size + pad + 15) // 16 * 16 for a in arrs) + pad
        buf = torch.full((total,), 7.0, dtype=torch.bfloat16, device="cuda:0")
        out, off = [], 0
        for a in arrs:
            v = buf[off + off_elems:off + off_elems + a.size].reshape(1, a.size)
            v.copy_(torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).reshape(1, a.size))
            out.append(v)
            off += (a.size + pad + 15) // 16 * 16
        return buf, out

    master0 = [O.randn_f32(n, 300 + i, 0.02) for i, n in enumerate(sizes)]
    p_bits = [O.bf16_from_f32(x) for x in master0]
    pbuf, p = views(p_bits, p_off)
    opt = nb.AdamW.new(1e-3, shapes, master=True).beta2(0.95).weight_decay(0.1)
    for i, a in enumerate(master0):
        opt.write_state(f"w{i}", H.to_dev(a.reshape(1, -1), shapes[i]))
    meta = O.adamw_meta(1e-3, beta2=0.95, weight_decay=0.1)
    ref = dict(p=[x.copy() for x in p_bits], w=[x.copy() for x in master0],
               m=[np.zeros_like(x) for x in master0], v=[np.zeros_like(x) for x in master0])
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(3):
            g_bits = [O.bf16_from_f32(O.randn_f32(n, 400 + 31 * step + i, 1e-2)) for i, n in enumerate(sizes)]
            gbuf, g = views(g_bits, g_off)
            opt.fused_step(p, g, zero_grads=step == 1)
            O.mixed_step(meta, None, 0.0, ref["p"], g_bits, ref["w"], ref["m"], ref["v"])
            got_g = H.host_list(g)
            if step == 1:
                assert not any(x.any() for x in got_g), "gradients zeroed"
            else:
                H.assert_bits_equal(got_g, g_bits, "gradients untouched")
            # what lies between the views keeps its fill
            mask = torch.ones_like(gbuf, dtype=torch.bool)
            for v in g:
                start = (v.data_ptr() - gbuf.data_ptr()) // 2
                mask[start:start + v.numel()] = False
            assert bool((gbuf[mask] == 7.0).all()), "gaps between the gradient views"
    finally:
        O.set_pow_mode(O.POW_LIBM)
    H.assert_bits_equal(H.host_list(p), ref["p"], f"params p_off={p_off} g_off={g_off} {kind}")
    H.assert_bits_equal(H.host_list([opt.read_state(f"w{i}") for i in range(len(shapes))]),
                        ref["w"], "master")
    H.assert_bits_equal(H.host_list(opt.moments()[1]), ref["v"], "v")
    mask = torch.ones_like(pbuf, dtype=torch.bool)
    for v in p:
        start = (v.data_ptr() - pbuf.data_ptr()) // 2
        mask[start:start + v.numel()] = False
    assert bool((pbuf[mask] == 7.0).all()), "gaps between the parameter views"
