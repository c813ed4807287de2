"""nbo_fused_step_noalloc -- the fused step whose norm pass keeps its partial results in the
library's statically allocated device array instead of the buffer nbo_init allocated -- against
nbo_fused_step on the same inputs, bit for bit, through the C ABI.

The array is shared by all calls on the GPU and keeps the previous call's contents, so the
sequence is chosen to leave stale data where a wrong grid or a missing write would pick it up:
a large list (all 2048 slots written, an inf in the last chunks so that a high slot's flag is
set and the step is skipped), then a small list (a few slots; it must not see that flag), then
the large list again without the inf.
"""
import numpy as np
import pytest

import oracle as O
from nabla_amd import optim as nb
from tests import helpers as H

pytestmark = pytest.mark.gpu

BIG = [(2100, 8192), (1, 8191), (3, 5), (64, 130)]  # 2100 + 3 chunks: the norm grid is at its cap
SMALL = [(1, 1), (1, 4097), (7, 1171), (0, 5), (33, 1000)]  # 9 chunks


class _Pair:
    """The same optimizer twice: one stepped through nbo_fused_step, one through the
    allocation-free entry point."""

    def __init__(self, shapes, seed, max_norm):
        self.shapes = shapes
        self.max_norm = max_norm  # below the gradients' norm, so that every step that runs clips
        master0 = H.randn_list(shapes, seed, 0.02)
        p_bits0 = H.narrow_list(master0, "bf16")
        self.sides = []
        for no_alloc in (False, True):
            opt = nb.AdamW.new(2e-4, shapes, master=True).beta2(0.95).weight_decay(0.1)
            for i, a in enumerate(master0):
                opt.write_state(f"w{i}", H.to_dev(a, shapes[i]))
            scaler = nb.GradScaler.new()
            scaler.load_state(nb.GradScalerState(scale=1024.0, growth_factor=2.0, backoff_factor=0.5,
                                                 growth_interval=2, consecutive_ok=0))
            self.sides.append(dict(no_alloc=no_alloc, opt=opt, scaler=scaler,
                                   p=H.dev_list(p_bits0, shapes)))
        # the oracle's copy of the same state
        self.ref = dict(meta=O.adamw_meta(2e-4, beta2=0.95, weight_decay=0.1),
                        scaler=O.ScalerState(1024.0, 2.0, 0.5, 2, 0), p=H.copy_list(p_bits0),
                        w=H.copy_list(master0), m=H.zeros_like_list(master0), v=H.zeros_like_list(master0))

    def step(self, seed, poison=None):
        g32 = H.randn_list(self.shapes, seed, 1e-3 * self.ref["scaler"].scale)
        g_bits = H.narrow_list(g32, "bf16")
        if poison is not None:
            t, e, bits = poison
            g_bits[t][e] = bits
        for s in self.sides:
            g_dev = H.dev_list(g_bits, self.shapes)
            s["opt"].fused_step(s["p"], g_dev, scaler=s["scaler"], max_norm=self.max_norm,
                                no_alloc=s["no_alloc"])
        O.set_pow_mode(O.POW_SQRT)
        try:
            ran, _ = O.mixed_step(self.ref["meta"], self.ref["scaler"], self.max_norm, self.ref["p"], g_bits,
                                  self.ref["w"], self.ref["m"], self.ref["v"])
        finally:
            O.set_pow_mode(O.POW_LIBM)
        return ran

    def check(self, what):
        out = []
        for s in self.sides:
            opt, n = s["opt"], len(self.shapes)
            out.append(dict(p=H.host_list(s["p"]), w=H.host_list([opt.read_state(f"w{i}") for i in range(n)]),
                            m=H.host_list(opt.moments()[0]), v=H.host_list(opt.moments()[1]),
                            trace=[(t.found_inf, np.float64(t.scale).tobytes(), t.step_count,
                                    np.float64(t.norm).tobytes(), t.clipped) for t in opt.trace()],
                            scaler=(s["scaler"].state().scale, s["scaler"].state().consecutive_ok)))
        a, b = out
        for key in ("p", "w", "m", "v"):
            H.assert_bits_equal(b[key], a[key], f"{what}: {key}, allocation-free vs ordinary entry point")
            H.assert_bits_equal(b[key], self.ref[key], f"{what}: {key}, allocation-free entry point vs oracle")
        assert b["trace"] == a["trace"], f"{what}: step records (found_inf, scale, step_count, norm bits, clipped)"
        assert b["scaler"] == a["scaler"] == (self.ref["scaler"].scale, self.ref["scaler"].consecutive_ok)
        return b


def test_allocation_free_fused_step_equals_the_ordinary_one_on_two_calls_in_a_row(gpu):
    big, small = _Pair(BIG, 1, 1.0), _Pair(SMALL, 2, 0.05)
    # 1. large list with +inf in chunk 2047 of its first tensor: the workgroup that owns slot 2047
    #    raises its flag, a slot the 9-chunk list below never writes
    assert not big.step(100, poison=(0, 2047 * 8192 + 5, 0x7F80))
    r = big.check("large list with an inf")
    assert r["trace"][-1][0] == 1 and r["trace"][-1][2] == 0, "the step with the inf is skipped"
    # 2. straight after it, a smaller list: the flags and sums the first call left in slots 9.. are stale
    assert small.step(200)
    r = small.check("small list after the large one")
    assert r["trace"][-1][0] == 0 and r["trace"][-1][2] == 1 and r["trace"][-1][4] == 1
    # 3. the large list again, now clean, then the small one with a NaN
    assert big.step(300)
    r = big.check("large list, clean")
    assert r["trace"][-1][0] == 0 and r["trace"][-1][2] == 1 and r["trace"][-1][4] == 1
    assert not small.step(400, poison=(2, 8000, 0x7FC1))
    r = small.check("small list with a NaN")
    assert r["trace"][-1][0] == 1 and r["trace"][-1][2] == 1


def test_allocation_free_fused_step_allocates_nothing_and_times_nothing(gpu):
    """What the entry point is for: the call makes no device allocation and, even while the
    library's per-kernel timing is switched on, creates no events -- its three launches are not
    timed, where the ordinary entry point's are.  Free device memory is the same before and
    after, and the step still does its work."""
    import ctypes as C

    import torch

    from nabla_amd import _lib

    L = _lib.load()
    shapes = SMALL
    master0 = H.randn_list(shapes, 5, 0.02)
    opt = nb.AdamW.new(2e-4, shapes, master=True).beta2(0.95).weight_decay(0.1)
    for i, a in enumerate(master0):
        opt.write_state(f"w{i}", H.to_dev(a, shapes[i]))
    p = nb.TensorList(H.dev_list(H.narrow_list(master0, "bf16"), shapes))
    g = nb.TensorList(H.dev_list(H.narrow_list(H.randn_list(shapes, 6, 1e-3 * 65536.0), "bf16"), shapes))
    scaler = nb.GradScaler.new()
    opt.fused_step(p, g, scaler=scaler, max_norm=0.05, no_alloc=True)  # descriptors, handles: all made by now
    nb.sync()
    torch.cuda.synchronize()

    def launches():
        out = {}
        for k in ("nbo_norm_bf16", "nbo_finalize", "nbo_update_bf16_adamw", "nbo_update_bf16_adamw_rows"):
            cnt, ms = C.c_uint64(0), C.c_double(0.0)
            _lib.check(L.nbo_profile_read(k.encode(), C.byref(cnt), C.byref(ms)))
            out[k] = cnt.value
        # the update kernel comes by chunk and by row; the library picks one by the list's shape
        out["nbo_update_bf16_adamw"] += out.pop("nbo_update_bf16_adamw_rows")
        return out

    _lib.check(L.nbo_profile_enable(1))
    try:
        free_before = torch.cuda.mem_get_info()[0]
        for _ in range(3):
            opt.fused_step(p, g, scaler=scaler, max_norm=0.05, no_alloc=True)
        nb.sync()
        assert torch.cuda.mem_get_info()[0] == free_before, "free device memory changed across the calls"
        assert launches() == {"nbo_norm_bf16": 0, "nbo_finalize": 0, "nbo_update_bf16_adamw": 0}, \
            "the allocation-free entry point's launches must not be bracketed by (newly created) events"
        opt.fused_step(p, g, scaler=scaler, max_norm=0.05)  # the ordinary one is timed
        assert launches() == {"nbo_norm_bf16": 1, "nbo_finalize": 1, "nbo_update_bf16_adamw": 1}
    finally:
        _lib.check(L.nbo_profile_enable(0))
    assert opt.step_count() == 5 and opt.last_step().clipped == 1
