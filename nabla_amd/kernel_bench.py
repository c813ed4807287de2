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


SHAPES = [  # nbo_probe_shape
    "the update kernels' own: 256 threads per 32 KiB window, 8 rows through registers",
    "512-thread workgroups, 8 rows through registers (64 KiB windows)",
    "1024-thread workgroups, 4 rows through registers (64 KiB windows)",
    "loads straight into LDS (global_load_lds_dwordx4), 64 KiB of LDS per workgroup",
    "loads straight into LDS, 128-144 KiB of LDS per workgroup",
    "8 rows through registers + the 64 KiB of LDS rows, together in flight",
    "512 threads: 4 waves only load (into LDS), 4 waves only store; double-buffered, 8 windows per workgroup",
    "next window's loads issued before the current window's stores (2 x 4 rows in registers, 8 windows per workgroup)",
    "shape 0's window, 8 of them per workgroup one after the other (nothing overlapped)",
    "next window's loads global -> LDS while the current one (LDS -> registers) is stored; 256 threads, <= 64 KiB LDS",
    "the same with 512 threads and twice the LDS",
    "the same with 256 threads and twice the rows",
    "shape 0's eight rows taken from 2 places of every stream at once (windows of 4 rows, a grid apart)",
    "shape 0's eight rows taken from 4 places of every stream at once (windows of 2 rows)",
    "shape 0's eight rows taken from 8 places of every stream at once (windows of 1 row)",
    "shape 0 with four rows per workgroup (16 KiB windows, twice the workgroups)",
    "shape 0 with two rows per workgroup (8 KiB windows)",
    "shape 0 with one row per workgroup: one vector of every stream per thread (4 KiB windows, eight times the workgroups)",
]
NEIGHBOURS = 0x80000000  # flag on a compare run's window count: the windows of a workgroup are neighbours
FULL_PATTERNS = (4, 5, 7, 9)  # the 1:1 read/write patterns every shape exists for


def measure_ceilings(gib: float = 2.0, reps: int = 10, patterns=None, settle_ms: int = 1500, spreads=(0, 1),
                     quiet_s: float = 2.0, shape: int = 0):
    """[(pattern name, spread, best GB/s, mean GB/s, regions, read:write)] over `patterns`
    (indices into PATTERNS; default all), each with plain and with region-spread buffers,
    moved in access shape `shape` (index into SHAPES).
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
            _lib.check(L.nbo_hbm_ceiling_shape(pat, shape, spread, nbytes, reps, settle_ms, C.byref(best),
                                               C.byref(mean), C.byref(regions), None))
            out.append((name, spread, best.value, mean.value, regions.value, f"{ro + rmw}:{rmw + wo}"))
    return out


def compare_shapes(pattern: int, shapes, iters=None, gib: float = 2.0, rounds: int = 5, reps: int = 5,
                   settle_ms: int = 1500, spread: int = 1):
    """Mean and best GB/s of several access shapes over the SAME buffers, measured in turn
    `rounds` times (`nbo_hbm_ceiling_compare`): [(shape, iters, mean, best)], regions."""
    from . import _lib

    _lib.init()
    L = _lib.load()
    n = len(shapes)
    iters = list(iters) if iters is not None else [0] * n
    nbytes = int(gib * (1 << 30)) // 32768 * 32768
    best, mean, regions = (C.c_double * n)(), (C.c_double * n)(), C.c_int()
    _lib.check(L.nbo_hbm_ceiling_compare(pattern, n, (C.c_int * n)(*shapes), (C.c_uint32 * n)(*iters), spread, nbytes,
                                         rounds, reps, settle_ms, best, mean, C.byref(regions)))
    return [(shapes[k], iters[k], mean[k], best[k]) for k in range(n)], regions.value


def compare_main(args) -> None:
    """Every access shape over the same buffers, for the four 1:1 read/write patterns."""
    import time

    runs = [(sh, 0) for sh in range(len(SHAPES))] + [(7, 2), (7, 4), (7, 32), (8, 2), (9, 32),
                                                       (7, 2 | NEIGHBOURS), (7, 8 | NEIGHBOURS), (8, 2 | NEIGHBOURS)]
    print(f"{args.gib} GiB per stream; per pattern all shapes share one set of buffers (placed across regions; a "
          f"single stream: one plain allocation) and are measured in turn, {args.rounds} rounds of {args.reps} "
          "launches each; mean (best) GB/s\n")
    print("| shape (windows per workgroup) | " + " | ".join(PATTERNS[p][0] for p in FULL_PATTERNS) + " |")
    print("|---|" + "---|" * len(FULL_PATTERNS))
    cols = []
    for pat in FULL_PATTERNS:
        time.sleep(2.0)
        single = sum(PATTERNS[pat][1:]) < 2
        rows, _ = compare_shapes(pat, [r[0] for r in runs], [r[1] for r in runs], args.gib, args.rounds, args.reps,
                                 spread=0 if single else 1)
        cols.append(rows)
    for k, (sh, it) in enumerate(runs):
        label = f"{sh}: {SHAPES[sh]}" + (f" [{it & ~NEIGHBOURS} windows per workgroup"
                                         f"{', neighbours' if it & NEIGHBOURS else ''}]" if it else "")
        print(f"| {label} | " + " | ".join(f"{c[k][2]:.0f} ({c[k][3]:.0f})" for c in cols) + " |", flush=True)


def ceilings_main(args) -> None:
    print(f"{args.gib} GiB per stream, {args.reps} launches each after 1.5 s of untimed launches; GB/s = bytes read + "
          "written per launch / duration\n")
    print("| pattern | read : written streams | buffers | regions | best GB/s | mean GB/s |")
    print("|---|---|---|---|---|---|")
    rows = [] if args.shapes_only else measure_ceilings(args.gib, args.reps)
    for name, spread, best, mean, regions, rw in rows:
        where = "across regions" if spread else "one plain allocation"
        print(f"| {name} | {rw} | {where} | {regions if spread else '-'} | {best:.0f} | {mean:.0f} |", flush=True)
    one_to_one = [r for r in rows if r[5] in ("1:1", "2:2", "3:3", "6:6", "4:4")]
    if one_to_one:
        top = max(one_to_one, key=lambda r: r[3])
        print(f"\nBest 1:1 read/write rate: {top[3]:.0f} GB/s mean ({top[2]:.0f} best launch), {top[0]}, "
              f"{'across regions' if top[1] else 'one plain allocation'}.")
    print("\nOther access shapes over the 1:1 read/write patterns, streams placed across regions (a single "
          "stream: one plain allocation):\n")
    print("| shape | " + " | ".join(PATTERNS[p][0] for p in FULL_PATTERNS) + " |")
    print("|---|" + "---|" * len(FULL_PATTERNS))
    for shape in range(len(SHAPES)):
        cells = []
        for pat in FULL_PATTERNS:
            single = sum(PATTERNS[pat][1:]) < 2  # one stream: nothing to spread it against
            r = measure_ceilings(args.gib, args.reps, patterns=(pat,), spreads=(0,) if single else (1,), shape=shape)[0]
            cells.append(f"{r[3]:.0f} ({r[2]:.0f})")
        print(f"| {shape}: {SHAPES[shape]} | " + " | ".join(cells) + " |", flush=True)
    print("\nmean (best) GB/s")


ADAM_F32 = ("nbo_update_f32_adam_self", "nbo_update_f32_adam_rows", "nbo_update_f32_adam")


def _ran(L, knames):
    """(name, ms per launch) of the kernel among `knames` (a name or several: the library picks
    one of an update kernel's forms by the list's size) that the timed calls launched."""
    from . import _lib

    best = None
    for k in ((knames,) if isinstance(knames, str) else knames):
        cnt, ms = C.c_uint64(0), C.c_double(0)
        _lib.check(L.nbo_profile_read(k.encode(), C.byref(cnt), C.byref(ms)))
        if cnt.value and (best is None or cnt.value > best[2]):
            best = (k, ms.value / cnt.value, cnt.value)
    if best is None:
        raise RuntimeError(f"none of {knames} was launched")
    return best[0], best[1]


def placed_main(args) -> None:
    """What placing the caller's own tensors buys: parameters and gradients (and a third list)
    as flat buffers from `nbo_alloc_placed`, all in one region against spread over regions, for
    the kernels whose streams are the caller's tensors."""
    import time

    import torch

    from . import _lib
    from . import backend as B
    from . import optim as nb
    from .placed import PlacedBuffers, carved_bytes

    _lib.init()
    L = _lib.load()
    big = max(int(args.elements) // (8192 * 8192), 1)
    shapes = [(8192, 8192)] * big + [(1, 4096)] * 8
    n = sum(r * c for r, c in shapes)
    print(f"{n} f32 elements in {len(shapes)} tensors per list, {args.reps} launches each; the lists are flat buffers from "
          "`nbo_alloc_placed`, region numbers per list as given (equal numbers: the same HBM region)\n")
    print("| entry point | kernel | regions of the lists | ms | bytes / element | GB/s |")
    print("|---|---|---|---|---|---|")

    def timeit(name, fn, bytes_per_elem, kname, where):
        fn()
        _lib.check(L.nbo_sync())
        _lib.check(L.nbo_profile_enable(1))
        for _ in range(args.reps):
            fn()
        _lib.check(L.nbo_sync())
        kname, t = _ran(L, kname)
        _lib.check(L.nbo_profile_enable(0))
        print(f"| {name} | `{kname}` | {where} | {t:.3f} | {bytes_per_elem} | {n * bytes_per_elem / t / 1e6:.0f} |", flush=True)

    nbytes = carved_bytes(shapes, 4)
    for regions in ((0, 0, 0), (0, 1, 0), (0, 1, 1), (-1, -1, -1)):
        time.sleep(3.0)  # the driver is still clearing what the previous search released
        try:
            bufs = PlacedBuffers(nbytes, regions)
        except Exception as e:  # e.g. no third region on this box
            print(f"| (regions {regions}: {e}) | | | | | |", flush=True)
            continue
        time.sleep(4.0)
        tensors = [bufs.carve(k, shapes, torch.float32) for k in range(3)]
        for t3, sigma in zip(tensors, (0.02, 1e-3, 1.0)):
            for t in t3:
                t.normal_(0.0, sigma)
        p, g, o = (nb.TensorList(t) for t in tensors)
        where = f"params {regions[0]}, grads {regions[1]}, third {regions[2]}"
        sgd = nb.Sgd.new(0.01, shapes)
        timeit("Sgd::step f32", lambda: sgd.step(p, g), 12, "nbo_update_f32_sgd", where)
        del sgd
        adam = nb.Adam.new(1e-3, shapes)
        timeit("Adam::step f32", lambda: adam.step(p, g), 28, ADAM_F32,
               where + f"; m, v: {adam.state_placement_note().split(';')[0]}")
        del adam
        timeit("accumulate f32", lambda: nb.accumulate(p, g), 12, "nbo_accum_f32", where)
        timeit("backend add f32", lambda: B.add(p, g, out=o), 12, "nbo_ew_f32", where)
        timeit("backend scale f32", lambda: B.scale(p, 0.5, out=o), 8, "nbo_ew_f32", where)
        timeit("scale_grad f32", lambda: nb.scale_grad(g, 0.5), 8, "nbo_scale_f32", where)
        del p, g, o, tensors
        bufs.close()


def flow_main(args) -> None:
    """One training step's tail as the reference's four calls (unscale_and_update, clip_grad_norm,
    step, zero_grad: trainer.rs:230-290, each reading its decision back to the host) against the
    one fused call, f32 AdamW over the same list with a GradScaler and a clip that bites."""
    import time

    import torch

    from . import _lib
    from . import optim as nb

    _lib.init()
    L = _lib.load()
    dev = torch.device("cuda:0")
    big = max(int(args.elements) // (8192 * 8192), 1)
    shapes = [(8192, 8192)] * big + [(1, 4096)] * 8
    n = sum(r * c for r, c in shapes)
    p = nb.TensorList([torch.randn(s, device=dev) * 0.02 for s in shapes])
    g0 = [torch.randn(s, device=dev) * (1e-3 * 65536.0) for s in shapes]
    g = nb.TensorList([t.clone() for t in g0])
    rows = []
    for fused in (False, True):
        opt = nb.AdamW.new(2e-4, shapes).beta2(0.95).weight_decay(0.1)
        scaler = nb.GradScaler.new()
        scaler.load_state(nb.GradScalerState(65536.0, 2.0, 0.5, 1 << 40, 0))

        def step():
            for t, t0 in zip(g.tensors, g0):  # the backward pass's part: fresh scaled gradients (not timed apart)
                t.copy_(t0)
            if fused:
                opt.fused_step(p, g, scaler=scaler, max_norm=1.0, zero_grads=True)
            else:
                if scaler.unscale_and_update(g):
                    nb.clip_grad_norm(g, 1.0)
                    opt.step(p, g)
                nb.zero_grad(g)

        def refill():
            for t, t0 in zip(g.tensors, g0):
                t.copy_(t0)

        for _ in range(2):
            step()
        _lib.check(L.nbo_sync())
        torch.cuda.synchronize()
        # the refill alone, to take it out of the figure
        t0 = time.perf_counter()
        for _ in range(args.reps):
            refill()
        torch.cuda.synchronize()
        t_refill = (time.perf_counter() - t0) / args.reps
        t0 = time.perf_counter()
        for _ in range(args.reps):
            step()
        _lib.check(L.nbo_sync())
        torch.cuda.synchronize()
        rows.append(((time.perf_counter() - t0) / args.reps - t_refill) * 1e3)
        del opt
    # bytes per parameter: unscale 4 (scan) + 8 (scale in place), clip 4 (norm) + 8 (scale), step 28, zero 4;
    # fused: norm pass 4, update 28 + 4 (the zeros)
    print(f"{n} f32 elements in {len(shapes)} tensors, {args.reps} steps each; the gradients are refilled before every "
          "step (a device copy, timed alone and subtracted)\n")
    print("| the step's tail | calls | HBM bytes / param | ms | GB/s |")
    print("|---|---|---|---|---|")
    print(f"| as the reference's four calls | unscale_and_update, clip_grad_norm, AdamW::step, zero_grad | 56 | "
          f"{rows[0]:.3f} | {n * 56 / rows[0] / 1e6:.0f} |")
    print(f"| fused | nbo_fused_step with NBO_STEP_ZERO_GRADS | 36 | {rows[1]:.3f} | {n * 36 / rows[1] / 1e6:.0f} |")
    print(f"\nThe fused call takes {rows[1] / rows[0] * 100:.0f} % of the four calls' time.")


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--elements", type=float, default=805e6)
    ap.add_argument("--reps", type=int, default=None)
    ap.add_argument("--ceilings", action="store_true", help="measure the memory system's ceilings instead")
    ap.add_argument("--gib", type=float, default=2.0, help="--ceilings: GiB per stream")
    ap.add_argument("--shapes-only", action="store_true", help="--ceilings: only the table of access shapes")
    ap.add_argument("--compare", action="store_true",
                    help="all access shapes over the same buffers, measured in turn (differences of a per cent "
                         "show here; --ceilings allocates anew for every row)")
    ap.add_argument("--rounds", type=int, default=5, help="--compare: rounds over all shapes")
    ap.add_argument("--placed", action="store_true",
                    help="the kernels over the caller's tensors with those tensors placed in named HBM regions "
                         "(nbo_alloc_placed): one region against several")
    ap.add_argument("--flow", action="store_true",
                    help="a training step's tail as the reference's four calls against the one fused call")
    ap.add_argument("--summarize", metavar="DIR", help="turn the rocprofv3 output under DIR into profiles/ summaries "
                                                        "(see nabla_amd/profile_summary.py) instead of measuring")
    args = ap.parse_args()
    if args.summarize:
        from . import profile_summary

        profile_summary.main(args.summarize)
        return
    if args.flow:
        args.reps = args.reps or 10
        flow_main(args)
        return
    if args.compare:
        args.reps = args.reps or 5
        compare_main(args)
        return
    if args.placed:
        args.reps = args.reps or 5
        placed_main(args)
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
        kname, t = _ran(L, kname)
        _lib.check(L.nbo_profile_enable(0))
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

        def micro_no_sum():
            fresh_scale()
            nb.unscale_accumulate(a, b, scaler=scaler, want_sumsq=False)

        timeit(f"unscale_accumulate {tag}, no sum of squares", micro_no_sum, 3 * sz, f"nbo_accscale_{tag}")
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
    timeit("Adam::step f32", lambda: adam.step(pl, gl), 28, ADAM_F32)
    del adam, pl, gl, p, g


if __name__ == "__main__":
    main()
