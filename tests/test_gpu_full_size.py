"""The benchmark configurations at their full sizes.

The oracle cannot chew through 8 G parameters, so at full size the device results are
checked (a) through what does not depend on size -- the decision trace, the global
norm against an independent f64 reduction, step counts -- and (b) element for element
on slices of every tensor (head, tail, seeded work-chunk boundaries): every
operation of the step is element-wise once the two global scalars (found_inf, norm)
are known, so the oracle run on a slice must reproduce that slice bit for bit --
(c) over every element, for what torch can restate exactly on the device (the
moments' multiply / add passes, the bf16 narrowing of the master weights), and (d) one
whole tensor, the largest, against the oracle for one step.
Synthetic inputs come from torch's generator on the device; oracle and device consume
the same bytes.
"""
import numpy as np
import pytest

import oracle as O
from nabla_amd import optim as nb
from nabla_amd import workloads as W
from tests import helpers as H

pytestmark = pytest.mark.gpu

SL = 4096  # elements of the head and tail slices
CHUNK = 8192  # the engine's work unit: one workgroup per CHUNK consecutive elements of a tensor


def _slices(n, key=0):
    """Index ranges checked inside tensor number `key` of n elements: head, tail, and 512
    elements around each of six seeded work-chunk boundaries (a chunk-map or offset mistake
    shows where one workgroup's elements end and the next one's begin), the last boundary
    before the ragged tail among them."""
    if n <= 3 * SL:
        return [(0, n)]
    rng = np.random.default_rng(7919 * key + n)
    nb = (n - 1) // CHUNK  # boundaries at CHUNK, 2 * CHUNK, ..., nb * CHUNK
    picks = {nb, max(1, nb // 2)} | {int(b) for b in rng.integers(1, nb + 1, size=4)}
    cuts = [(0, SL), (n - SL, n)] + [(b * CHUNK - 256, min(b * CHUNK + 256, n)) for b in picks]
    cuts.sort()
    merged = [cuts[0]]
    for a, b in cuts[1:]:
        if a <= merged[-1][1]:
            merged[-1] = (merged[-1][0], max(merged[-1][1], b))
        else:
            merged.append((a, b))
    return merged


def _take(t, n, key=0):
    """Host copy of the checked slices of device tensor t, concatenated."""
    flat = t.reshape(-1)
    import torch

    return H.to_host(torch.cat([flat[a:b] for a, b in _slices(n, key)]))


def _take_list(tensors, shapes):
    return [_take(t, r * c, i) for i, (t, (r, c)) in enumerate(zip(tensors, shapes))]


def test_gpt2_small_adam_f32_10_steps(gpu):
    """Config 2: Adam f32, 148 tensors, 124,439,808 params, fresh grads each step."""
    import torch

    shapes = W.gpt2_small_shapes()
    assert len(shapes) == 148 and W.n_params(shapes) == 124_439_808
    torch.manual_seed(2)
    p = [torch.randn(s, device=gpu) * 0.02 for s in shapes]
    ref_p = _take_list(p, shapes)
    ref_m, ref_v = H.zeros_like_list(ref_p), H.zeros_like_list(ref_p)
    opt = nb.Adam.new(3e-4, shapes)
    meta = O.adam_meta(3e-4)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(10):
            g = [torch.randn(s, device=gpu) * 1e-3 for s in shapes]
            opt.step(p, g)
            O.adam_step(meta, ref_p, _take_list(g, shapes), ref_m, ref_v)
    finally:
        O.set_pow_mode(O.POW_LIBM)
    assert opt.step_count() == 10
    m, v = opt.moments()
    H.assert_bits_equal(_take_list(m, shapes), ref_m, "m slices")
    H.assert_bits_equal(_take_list(v, shapes), ref_v, "v slices")
    H.assert_bits_equal(_take_list(p, shapes), ref_p, "param slices")


def _f32_scalar(x, dev):
    import torch

    return torch.tensor(float(np.float32(x)), dtype=torch.float32, device=dev)


def _mixed_full(gpu, shapes, steps, seed, whole_tensor=None):
    """Configs 3 / 5: AdamW, bf16 params/grads, f32 master/m/v, scale 65536, clip 1.0.

    Checked at full size:
      * decisions and the global norm (against an f64 reduction by torch) every step;
      * slices of every tensor (head, tail, seeded work-chunk boundaries) against the oracle's
        pass chain, bit for bit, and against its libm-powf variant within the stated bars;
      * every element of m and v against the reference's moment passes (alg.rs:138-142) done
        with torch on the device, one IEEE multiply or add per kernel, bit for bit: a chunk
        that was skipped, done twice or written to the wrong place shows here;
      * params == bf16(master) for every element of every tensor;
      * with `whole_tensor` = i: all of tensor i against the oracle for the last step, from the
        device's own state before that step.
    """
    import torch

    lr, wd, b1, b2 = 2e-4, 0.1, 0.9, 0.95
    torch.manual_seed(seed)
    n_t = len(shapes)
    opt = nb.AdamW.new(lr, shapes, master=True).beta2(b2).weight_decay(wd)
    params = [torch.empty(s, dtype=torch.bfloat16, device=gpu) for s in shapes]
    ref_w = []
    for i, s in enumerate(shapes):
        w = torch.randn(s, device=gpu) * 0.02
        opt.write_state(f"w{i}", w)
        ref_w.append(_take(w, s[0] * s[1], i))
        del w
    opt.params_from_master(params)
    ref_m, ref_v = H.zeros_like_list(ref_w), H.zeros_like_list(ref_w)
    # second reference: the reference-faithful libm powf variant (2 ulp / 1 bf16 ulp bar)
    lib_w, lib_m, lib_v = H.copy_list(ref_w), H.zeros_like_list(ref_w), H.zeros_like_list(ref_w)
    # the moments of every element, evolved by torch
    full_m = [torch.zeros(s, dtype=torch.float32, device=gpu) for s in shapes]
    full_v = [torch.zeros(s, dtype=torch.float32, device=gpu) for s in shapes]
    t_b1, t_omb1 = _f32_scalar(b1, gpu), _f32_scalar(1.0 - b1, gpu)
    t_b2, t_omb2 = _f32_scalar(b2, gpu), _f32_scalar(1.0 - b2, gpu)
    scaler = nb.GradScaler.new()
    meta = O.adamw_meta(lr, b1, b2, 1e-8, wd)
    lib_meta = O.adamw_meta(lr, b1, b2, 1e-8, wd)
    inv = np.float32(1.0 / 65536.0)
    whole = None
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(steps):
            grads, sumsq = [], torch.zeros((), dtype=torch.float64, device=gpu)
            for s in shapes:
                g = (torch.randn(s, device=gpu) * (1e-3 * 65536.0)).to(torch.bfloat16)
                u = g.float() * float(inv)
                sumsq += (u.double() ** 2).sum()
                grads.append(g)
                del u
            if whole_tensor is not None and step == steps - 1:
                i = whole_tensor  # the device's state of one whole tensor before the last step
                whole = dict(w=H.to_host(opt.read_state(f"w{i}")), m=H.to_host(opt.read_state(f"m{i}")),
                             v=H.to_host(opt.read_state(f"v{i}")), g=H.to_host(grads[i]))
            opt.fused_step(params, grads, scaler=scaler, max_norm=1.0)
            info = opt.last_step()
            # size-independent: decisions and the global norm
            assert (info.found_inf, info.scale, info.step_count) == (0, 65536.0, step + 1)
            norm_ref = float(torch.sqrt(sumsq))
            assert info.norm == pytest.approx(norm_ref, rel=1e-9)
            assert info.clipped == 1 and norm_ref > 1.0
            # slices: the reference's chain with the device's (verified) norm
            c = np.float32(1.0 / info.norm)
            g32 = [(O.bf16_to_f32(_take(g, s[0] * s[1], i)) * inv) * c
                   for i, (g, s) in enumerate(zip(grads, shapes))]
            O.adam_step(meta, ref_w, g32, ref_m, ref_v)
            O.set_pow_mode(O.POW_LIBM)
            O.adam_step(lib_meta, lib_w, g32, lib_m, lib_v)
            O.set_pow_mode(O.POW_SQRT)
            # every element: m = m * b1; m = m + (1 - b1) * g; v = v * b2; v = v + (1 - b2) * (g * g),
            # each product and sum a kernel of its own, hence one rounding each
            t_inv, t_c = _f32_scalar(inv, gpu), _f32_scalar(c, gpu)
            for g, fm, fv in zip(grads, full_m, full_v):
                u = (g.float() * t_inv) * t_c
                fm.mul_(t_b1)
                fm.add_(u * t_omb1)
                fv.mul_(t_b2)
                q = u * u
                fv.add_(q * t_omb2)
                del u, q
            del grads
    finally:
        O.set_pow_mode(O.POW_LIBM)
    H.assert_bits_equal([_take(opt.read_state(f"m{i}"), s[0] * s[1], i) for i, s in enumerate(shapes)], ref_m,
                        "m slices")
    H.assert_bits_equal([_take(opt.read_state(f"v{i}"), s[0] * s[1], i) for i, s in enumerate(shapes)], ref_v,
                        "v slices")
    H.assert_bits_equal([_take(opt.read_state(f"w{i}"), s[0] * s[1], i) for i, s in enumerate(shapes)], ref_w,
                        "master slices")
    H.assert_bits_equal(_take_list(params, shapes), [O.bf16_from_f32(a) for a in ref_w],
                        "bf16 param slices")
    # against libm powf: moments identical, master within 2 ulp (or the cancellation
    # bound |d| <= steps * 8 * lr * 2^-23), bf16 params within 1 ulp
    H.assert_bits_equal(lib_m, ref_m, "m, libm variant")
    H.assert_bits_equal(lib_v, ref_v, "v, libm variant")
    H.tolerance_report(ref_w, lib_w, lr, steps, f"{n_t}-tensor set, master slices (= device bits) vs libm-powf oracle")
    assert H.max_ulp_bf16([O.bf16_from_f32(a) for a in ref_w], [O.bf16_from_f32(a) for a in lib_w]) <= 1
    # full coverage on the device: the moments of every element, and params == bf16(master)
    for i in range(n_t):
        mi, vi, wi = opt.read_state(f"m{i}"), opt.read_state(f"v{i}"), opt.read_state(f"w{i}")
        assert torch.equal(mi.view(torch.int32), full_m[i].view(torch.int32)), f"m of tensor {i}, all elements"
        assert torch.equal(vi.view(torch.int32), full_v[i].view(torch.int32)), f"v of tensor {i}, all elements"
        assert torch.equal(wi.to(torch.bfloat16).view(torch.int16), params[i].view(torch.int16)), \
            f"params of tensor {i} are bf16(master), all elements"
        del mi, vi, wi
    if whole is not None:
        i = whole_tensor
        wm = O.adamw_meta(lr, b1, b2, 1e-8, wd)
        wm.step_count = steps - 1
        g32 = [(O.bf16_to_f32(whole["g"]) * inv) * np.float32(1.0 / info.norm)]
        w_, m_, v_ = [whole["w"]], [whole["m"]], [whole["v"]]
        O.set_threads(16)
        O.set_pow_mode(O.POW_SQRT)
        try:
            O.adam_step(wm, w_, g32, m_, v_)
        finally:
            O.set_pow_mode(O.POW_LIBM)
            O.set_threads(1)
        H.assert_bits_equal([H.to_host(opt.read_state(f"m{i}"))], m_, f"all of m{i} after the last step")
        H.assert_bits_equal([H.to_host(opt.read_state(f"v{i}"))], v_, f"all of v{i} after the last step")
        H.assert_bits_equal([H.to_host(opt.read_state(f"w{i}"))], w_, f"all of w{i} after the last step")
        H.assert_bits_equal([H.to_host(params[i])], [O.bf16_from_f32(w_[0])], f"all of bf16 tensor {i}")


def test_llama_1b_mixed_adamw_10_steps(gpu):
    shapes = W.llama_1b_shapes()
    assert len(shapes) == 200 and W.n_params(shapes) == 1_100_046_336
    _mixed_full(gpu, shapes, 10, seed=3, whole_tensor=len(shapes) - 1)


def test_llama3_8b_mixed_adamw_7_steps(gpu):
    """Config 5: 2 warm-up + 5 timed steps in the benchmark; the same 7 steps here."""
    shapes = W.llama_8b_shapes()
    assert len(shapes) == 290 and W.n_params(shapes) == 8_030_257_152
    assert shapes[-1] == (128256, 4096)  # lm_head, the largest tensor: checked whole on the last step
    _mixed_full(gpu, shapes, 7, seed=5, whole_tensor=len(shapes) - 1)


def test_adamw_chain_of_primitives_on_one_full_size_llama3_layer(gpu):
    """The reference's own formulation of AdamW::step (optim/alg.rs:109-150) -- twelve Backend
    passes with their temporaries, each a multi-tensor primitive launch here -- against the fused
    update kernel on one Llama-3-8B layer at its real shapes (218,112,000 parameters, f32): every
    element of parameters and moments, compared on the device, after each of three steps."""
    import torch

    from nabla_amd import backend as B

    shapes = W.llama_8b_shapes()[:9]  # q, k, v, o, gate, up, down and the two norm vectors of layer 0
    assert W.n_params(shapes) == 218_112_000
    lr, b1, b2, eps, wd = 2e-4, 0.9, 0.95, 1e-8, 0.1
    torch.manual_seed(11)
    p = [torch.randn(s, device=gpu) * 0.02 for s in shapes]
    fused_p = [t.clone() for t in p]
    opt = nb.AdamW.new(lr, shapes).beta1(b1).beta2(b2).eps(eps).weight_decay(wd)
    m, v = [torch.zeros_like(t) for t in p], [torch.zeros_like(t) for t in p]
    t1, t2 = [torch.empty_like(t) for t in p], [torch.empty_like(t) for t in p]
    lp, lm, lv, l1, l2 = (nb.TensorList(x) for x in (p, m, v, t1, t2))
    f32 = np.float32
    for step in range(1, 4):
        g = [torch.randn(s, device=gpu) * 1e-3 for s in shapes]
        lg = nb.TensorList(g)
        opt.step(fused_p, g)
        bc1, bc2 = 1.0 - O.powi(b1, step), 1.0 - O.powi(b2, step)
        ss, ibc2, wd_lr = float(f32(lr / bc1)), float(f32(1.0 / bc2)), f32(wd * lr)
        B.scale(lm, b1, out=lm)                      # m = &m * beta1
        B.axpy_inplace(lm, 1.0 - b1, lg)             # m.axpy_inplace(1 - beta1, g)
        B.scale(lv, b2, out=lv)                      # v = &v * beta2
        B.emul(lg, lg, out=l1)                       # g_sq = g.emul(g)
        B.axpy_inplace(lv, 1.0 - b2, l1)             # v.axpy_inplace(1 - beta2, &g_sq)
        B.scale(lv, ibc2, out=l1)                    # v_scaled = &v * inv_bc2
        B.powf(l1, 0.5, out=l1)                      # .powf(0.5)
        B.map_add(l1, eps, out=l1)                   # .map(|x| x + eps)
        B.scale(lm, ss, out=l2)                      # m_scaled = &m * step_size
        B.ediv(l2, l1, out=l2)                       # update = m_scaled.ediv(&denom)
        B.scale(lp, float(f32(1.0) - wd_lr), out=lp)  # p = &p * (1 - wd_lr), computed in T
        B.axpy_inplace(lp, -1.0, l2)                 # p.axpy_inplace(-1, &update)
        fm, fv = opt.moments()
        for i in range(len(shapes)):
            assert torch.equal(p[i].view(torch.int32), fused_p[i].view(torch.int32)), f"params {i}, step {step}"
            assert torch.equal(m[i].view(torch.int32), fm[i].view(torch.int32)), f"m {i}, step {step}"
            assert torch.equal(v[i].view(torch.int32), fv[i].view(torch.int32)), f"v {i}, step {step}"
        del fm, fv, g, lg


def test_ragged_4096_dynamic_scale_64_steps(gpu):
    """Config 4 in full: 4096 tensors, sizes log-uniform in [1, 65536], packed back to
    back (so most tensor addresses are only 2-byte aligned), growth interval 4, inf/NaN
    injected every 4th step at a seeded 1e-6 of the positions; 64 steps.  Everything is
    compared with the oracle run on the whole set."""
    import torch

    sizes = W.ragged_sizes()
    shapes = [(1, n) for n in sizes]
    total = sum(sizes)
    offs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int64)
    lr, wd = 2e-4, 0.1
    rng = np.random.default_rng(4)
    w0 = (rng.standard_normal(total) * 0.02).astype(np.float32)
    flat_p = H.to_dev(O.bf16_from_f32(w0))
    flat_g = torch.empty(total, dtype=torch.bfloat16, device=gpu)
    views_p = [flat_p[offs[i]:offs[i + 1]] for i in range(len(sizes))]
    views_g = [flat_g[offs[i]:offs[i + 1]] for i in range(len(sizes))]
    assert any(v.data_ptr() % 16 for v in views_p), "the packed layout is meant to be unaligned"
    opt = nb.AdamW.new(lr, shapes, master=True).beta2(0.95).weight_decay(wd)
    opt.master_from_params(views_p)  # master = f32(bf16 params)
    plist, glist = nb.TensorList(views_p), nb.TensorList(views_g)
    scaler = nb.GradScaler.new()
    scaler.load_state(nb.GradScalerState(65536.0, 2.0, 0.5, 4, 0))

    ref_w_flat = O.bf16_to_f32(O.bf16_from_f32(w0))
    ref_p_flat = O.bf16_from_f32(w0)
    ref_m_flat, ref_v_flat = np.zeros(total, np.float32), np.zeros(total, np.float32)
    split = lambda a: [a[offs[i]:offs[i + 1]] for i in range(len(sizes))]  # noqa: E731
    ref_w, ref_p, ref_m, ref_v = split(ref_w_flat), split(ref_p_flat), split(ref_m_flat), split(ref_v_flat)
    meta, s = O.adamw_meta(lr, 0.9, 0.95, 1e-8, wd), O.ScalerState(65536.0, 2.0, 0.5, 4, 0)
    O.set_threads(8)
    O.set_pow_mode(O.POW_SQRT)
    ref_trace = []
    try:
        for step in range(64):
            g_bits = O.bf16_from_f32((rng.standard_normal(total) * (1e-3 * s.scale)).astype(np.float32))
            if step % 4 == 3:
                for pos in rng.integers(0, total, size=max(1, int(total * 1e-6))):
                    g_bits[pos] = (0x7F80, 0xFF80, 0x7FC0)[int(rng.integers(3))]
            flat_g.copy_(H.to_dev(g_bits))
            opt.fused_step(plist, glist, scaler=scaler, max_norm=1.0)
            ran, norm = O.mixed_step(meta, s, 1.0, ref_p, split(g_bits), ref_w, ref_m, ref_v)
            ref_trace.append((0 if ran else 1, s.scale, meta.step_count, norm))
    finally:
        O.set_pow_mode(O.POW_LIBM)
        O.set_threads(1)
    tr = opt.trace()
    assert [(t.found_inf, t.scale, t.step_count) for t in tr] == [t[:3] for t in ref_trace]
    for t, r in zip(tr, ref_trace):
        assert t.norm == pytest.approx(r[3], rel=1e-12)
    # closed form of the schedule: 16 skips, scale halves 16 times, 48 optimizer steps
    assert sum(t.found_inf for t in tr) == 16 and tr[-1].scale == 1.0 and tr[-1].step_count == 48
    st = scaler.state()
    assert (st.scale, st.consecutive_ok) == (s.scale, s.consecutive_ok)
    m, v = opt.moments()
    H.assert_bits_equal(H.host_list(m), ref_m, "m")
    H.assert_bits_equal(H.host_list(v), ref_v, "v")
    H.assert_bits_equal(H.host_list([opt.read_state(f"w{i}") for i in range(len(sizes))]), ref_w, "master")
    H.assert_bits_equal([H.to_host(flat_p)], [ref_p_flat], "bf16 params")


def test_one_tensor_longer_than_2_pow_32_elements(gpu):
    """Element offsets are 64-bit throughout (the reference's own kernels take
    `unsigned n`).  One bf16 tensor of 2^32 + 3 * 8192 + 5 elements -- its chunk indices
    and byte offsets pass 2^32 and 2^33 -- plus a small tensor after it, through two fused
    AdamW steps (bf16 arithmetic, so the state stays at 26 GB): slices at the head,
    around element 2^32, in the last full chunk and in the ragged tail must match the
    oracle bit for bit, and the global norm an independent f64 reduction."""
    import torch

    n_big = (1 << 32) + 3 * 8192 + 5
    shapes = [(1, n_big), (3, 1000)]
    cuts = [[(0, SL), ((1 << 32) - SL // 2, (1 << 32) + SL // 2), (n_big - 5 - 8192, n_big - 5 - 8192 + SL),
             (n_big - SL, n_big)], [(0, 3000)]]

    def take(t, k):
        flat = t.reshape(-1)
        return H.to_host(torch.cat([flat[a:b] for a, b in cuts[k]]))

    torch.manual_seed(77)
    params = [(torch.randn(s, device=gpu, dtype=torch.bfloat16) * 0.5) for s in shapes]
    ref_p = [take(t, k) for k, t in enumerate(params)]
    ref_m, ref_v = [np.zeros_like(a) for a in ref_p], [np.zeros_like(a) for a in ref_p]
    opt = nb.AdamW.new(1e-2, shapes, dtype="bf16").beta2(0.95).weight_decay(0.1)
    meta = O.adamw_meta(1e-2, 0.9, 0.95, 1e-8, 0.1)
    O.set_pow_mode(O.POW_SQRT)
    try:
        for step in range(2):
            grads = [(torch.randn(s, device=gpu, dtype=torch.bfloat16) * 1e-2) for s in shapes]
            sumsq = sum((g.double() ** 2).sum() for g in grads)
            opt.fused_step(params, grads, max_norm=1.0)
            info = opt.last_step()
            norm_ref = float(torch.sqrt(sumsq))
            assert info.norm == pytest.approx(norm_ref, rel=1e-9) and info.clipped == 1
            assert info.step_count == step + 1
            # the clip factor is a bf16 value; the slices then follow the reference's chain
            g_sl = [take(g, k) for k, g in enumerate(grads)]
            c = 1.0 / info.norm
            g_sl = [O.scale(a, c) for a in g_sl]  # g.map(|x| x * scale_t), trainer.rs:519
            O.adam_step(meta, ref_p, g_sl, ref_m, ref_v)
            del grads
    finally:
        O.set_pow_mode(O.POW_LIBM)
    m = [opt.read_state("m0"), opt.read_state("m1")]
    v = [opt.read_state("v0"), opt.read_state("v1")]
    H.assert_bits_equal([take(t, k) for k, t in enumerate(params)], ref_p, "param slices")
    H.assert_bits_equal([take(t, k) for k, t in enumerate(m)], ref_m, "m slices")
    H.assert_bits_equal([take(t, k) for k, t in enumerate(v)], ref_v, "v slices")
    # a chunk nobody should have touched twice or skipped: every element moved
    assert bool((params[0].reshape(-1)[(1 << 32) - 8:(1 << 32) + 8] != 0).all())
