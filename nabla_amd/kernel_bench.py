"""Throughput of every kernel other than the dominant one, on one large tensor list, and the
memory system's own ceilings.

    python -m nabla_amd.kernel_bench [--elements 805e6] [--reps 5]
    python -m nabla_amd.kernel_bench --ceilings [--gib 2] [--reps 10]

Each entry point is timed with the library's own per-kernel HIP events on its launch stream
(`nbo_profile_enable` / `nbo_profile_read`) and priced at its algorithmic bytes per element;
prints one markdown table row per measurement.  `bench.py` covers the optimizer step itself.

`--ceilings` measures what the HBM gives the update kernels' access shape (one workgroup per
32 KiB window of every stream, 128-bit accesses, all loads issued before the first use) for a
pure read, a pure fill, a copy and in-place read-modify-write over 1, 2, 3 and 6 streams, with
all streams in one plain allocation and with the streams placed across the HBM's regions the
way optimizer state is (`nbo_hbm_ceiling`).  The best 1:1 read/write rate among them is what
an optimizer update can reach at most.
"""
from __future__ import annotations

import argparse
import ctypes as C

PATTERNS = [  # nbo_probe_pattern: name, streams read, rewritten in place, written
    ("read, 1 stream", 1, 0, 0), ("read, 3 streams", 3, 0, 0), ("fill, 1 stream", 0, 0, 1),
    ("fill, 3 streams", 0, 0, 3), ("copy", 1, 0, 1), ("read-modify-write, 1 stream", 0, 1, 0),
    ("read-modify-write, 2 streams", 0, 2, 0), ("read-modify-write, 3 streams", 0, 3, 0),
    ("read-modify-write, 6 streams", 0, 6, 0), ("1 read + 3 read-modify-write + 1 written (update's shape)", 1, 3, 1)]


def measure_ceilings(gib: float = 2.0, reps: int = 10, patterns=None, settle_ms: int = 1500, spreads=(0, 1),
                     quiet_s: float = 2.0):
    """[(pattern name, spread, best GB/s, mean GB/s, regions, read:write)] over `patterns`
    (indices into PATTERNS; default all), each with plain and with region-spread buffers.
    Every measurement waits `quiet_s` before it allocates and then launches untimed for
    `settle_ms`: the driver clears freed device memory in the background, each measurement frees
    the previous one's buffers, and the placement search frees its spare chunks."""
    import time

    from . import _lib

    _lib.init()
    L = _lib.load()
    nbytes = int(gib * (1 << 30)) // 32768 * 32768
    out = []
    for pat in (range(len(PATTERNS)) if patterns is None else patterns):
        name, ro, rmw, wo = PATTERNS[pat]
        for spread in spreads:
            if spread and ro + rmw + wo < 2:
                continue  # a single stream has nothing to be spread against
            best, mean, regions = C.c_double(), C.c_double(), C.c_int()
            # the previous measurement's buffers have just been freed: the driver is still clearing
            # them, which would disturb the placement search's own short probes
            time.sleep(quiet_s)
            _lib.check(L.nbo_hbm_ceiling(pat, spread, nbytes, reps, settle_ms, C.byref(best), C.byref(mean),
                                         C.byref(regions)))
            out.append((name, spread, best.value, mean.value, regions.value, f"{ro + rmw}:{rmw + wo}"))
    return out


def ceilings_main(args) -> None:
    print(f"{args.gib} GiB per stream, {args.reps} launches each after 1.5 s of untimed launches; GB/s = bytes read + "
          "written per launch / duration\n")
    print("| pattern | read : written streams | buffers | regions | best GB/s | mean GB/s |")
    print("|---|---|---|---|---|---|")
    rows = measure_ceilings(args.gib, args.reps)
    for name, spread, best, mean, regions, rw in rows:
        where = "across regions" if spread else "one plain allocation"
        print(f"| {name} | {rw} | {where} | {regions if spread else '-'} | {best:.0f} | {mean:.0f} |", flush=True)
    one_to_one = [r for r in rows if r[5] in ("1:1", "2:2", "3:3", "6:6", "4:4")]
    top = max(one_to_one, key=lambda r: r[3])
    print(f"\nBest 1:1 read/write rate: {top[3]:.0f} GB/s mean ({top[2]:.0f} best launch), {top[0]}, "
          f"{'across regions' if top[1] else 'one plain allocation'}.")


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--elements", type=float, default=805e6)
    ap.add_argument("--reps", type=int, default=None)
    ap.add_argument("--ceilings", action="store_true", help="measure the memory system's ceilings instead")
    ap.add_argument("--gib", type=float, default=2.0, help="--ceilings: GiB per stream")
    ap.add_argument("--summarize", metavar="DIR", help="turn the rocprofv3 output under DIR into profiles/ summaries "
                                                        "(see nabla_amd/profile_summary.py) instead of measuring")
    args = ap.parse_args()
    if args.summarize:
        from . import profile_summary

        profile_summary.main(args.summarize)
        return
    if args.ceilings:
        args.reps = args.reps or 10
        ceilings_main(args)
        return
    args.reps = args.reps or 5

    import torch

    from . import _lib
    from . import backend as B
    from . import optim as nb

    _lib.init()
    L = _lib.load()
    dev = torch.device("cuda:0")
    big = max(int(args.elements) // (8192 * 8192), 1)
    shapes = [(8192, 8192)] * big + [(1, 4096)] * 8
    n = sum(r * c for r, c in shapes)

    def mk(dt, sigma=1.0):
        return [(torch.randn(s, device=dev, dtype=torch.float32) * sigma).to(dt) for s in shapes]

    print(f"{n} elements in {len(shapes)} tensors, {args.reps} launches each\n")
    print("| entry point | kernel | ms | bytes / element | GB/s |")
    print("|---|---|---|---|---|")

    def timeit(name, fn, bytes_per_elem, kname):
        fn()
        _lib.check(L.nbo_sync())
        _lib.check(L.nbo_profile_enable(1))
        for _ in range(args.reps):
            fn()
        _lib.check(L.nbo_sync())
        cnt, ms = C.c_uint64(0), C.c_double(0)
        _lib.check(L.nbo_profile_read(kname.encode(), C.byref(cnt), C.byref(ms)))
        _lib.check(L.nbo_profile_enable(0))
        t = ms.value / max(cnt.value, 1)
        print(f"| {name} | `{kname}` | {t:.3f} | {bytes_per_elem} | {n * bytes_per_elem / t / 1e6:.0f} |", flush=True)

    types = ((torch.float32, "f32", 4), (torch.bfloat16, "bf16", 2), (torch.float16, "f16", 2),
             (torch.float64, "f64", 8))
    for dt, tag, sz in types:
        a, b, o = nb.TensorList(mk(dt)), nb.TensorList(mk(dt)), nb.TensorList(mk(dt))
        scaler = nb.GradScaler.new()

        def fresh_scale():
            scaler.load_state(nb.GradScalerState(65536.0, 2.0, 0.5, 1 << 40, 0))

        timeit(f"accumulate {tag}", lambda: nb.accumulate(a, b), 3 * sz, f"nbo_accum_{tag}")
        timeit(f"accumulate + zero {tag}", lambda: nb.accumulate(a, b, True), 4 * sz, f"nbo_accum_{tag}")
        nb.zero_grad(a)

        def micro():
            fresh_scale()
            nb.unscale_accumulate(a, b, scaler=scaler)

        timeit(f"unscale_accumulate {tag}", micro, 3 * sz, f"nbo_accnorm_{tag}")
        timeit(f"zero_grad {tag}", lambda: nb.zero_grad(a), sz, f"nbo_scale_{tag}")
        timeit(f"scale_grad {tag}", lambda: nb.scale_grad(b, 0.5), 2 * sz, f"nbo_scale_{tag}")
        timeit(f"clip_grad_norm {tag}, norm pass", lambda: nb.clip_grad_norm(b, 1e30), sz, f"nbo_norm_{tag}")
        if tag in ("bf16", "f16"):  # in place on 16-bit lists the arithmetic is the lists' own

            def unscale():
                fresh_scale()
                scaler.unscale_and_update(b)

            timeit(f"unscale_and_update {tag}, scan", unscale, sz, f"nbo_norm_p{tag}")
        timeit(f"backend add {tag}", lambda: B.add(a, b, out=o), 3 * sz, f"nbo_ew_{tag}")
        timeit(f"backend axpy_inplace {tag}", lambda: B.axpy_inplace(o, 0.5, a), 3 * sz, f"nbo_ew_{tag}")
        timeit(f"backend scale {tag}", lambda: B.scale(a, 0.5, out=o), 2 * sz, f"nbo_ew_{tag}")
        timeit(f"backend powf(0.5) {tag}", lambda: B.powf(a, 0.5, out=o), 2 * sz, f"nbo_ew_{tag}")
        del a, b, o
        torch.cuda.empty_cache()
    src, dst = nb.TensorList(mk(torch.float32)), nb.TensorList(mk(torch.bfloat16))
    timeit("cast f32 -> bf16", lambda: B.cast(src, dst), 6, "nbo_cast_list")
    timeit("cast bf16 -> f32", lambda: B.cast(dst, src), 6, "nbo_cast_list")
    del src, dst
    torch.cuda.empty_cache()
    p, g = mk(torch.float32, 0.02), mk(torch.float32, 1e-3)
    pl, gl = nb.TensorList(p), nb.TensorList(g)
    sgd = nb.Sgd.new(0.01, shapes)
    timeit("Sgd::step f32", lambda: sgd.step(pl, gl), 12, "nbo_update_f32_sgd")
    del sgd
    sgdm = nb.Sgd.new(0.01, shapes).momentum(0.9)
    timeit("Sgd::step f32, momentum", lambda: sgdm.step(pl, gl), 20, "nbo_update_f32_sgd")
    del sgdm
    adam = nb.Adam.new(1e-3, shapes)
    timeit("Adam::step f32", lambda: adam.step(pl, gl), 28, "nbo_update_f32_adam")
    del adam, pl, gl, p, g


if __name__ == "__main__":
    main()
