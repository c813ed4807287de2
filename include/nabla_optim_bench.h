/*
 * nabla_optim_bench.h -- measurement entry points of libnabla_optim.so.
 *
 * None of these has a counterpart in the reference's optimizer interface, and no optimizer
 * step needs them: they time the library's own launches, measure what the MI355X memory
 * system gives an access pattern, for benchmarks and profiles, and check the library's own
 * arithmetic exhaustively.  The drop-in boundary is nabla_optim.h alone.  The probe kernels
 * live in a code object of their own that is loaded when one of these functions first needs it.
 */
#ifndef NABLA_OPTIM_BENCH_H
#define NABLA_OPTIM_BENCH_H

#include "nabla_optim.h"

#ifdef __cplusplus
extern "C" {
#endif

#pragma GCC visibility push(default)

/* Device-to-device streaming copy of `bytes` (multiple of 16) with a plain copy kernel;
 * used to calibrate HBM byte counters against a known transfer. */
int nbo_copy_bytes(const void *src_dev, void *dst_dev, uint64_t bytes);

/* Which streams a probe kernel touches. */
typedef enum nbo_probe_pattern {
    NBO_PATTERN_READ1 = 0,       /* 1 stream read */
    NBO_PATTERN_READ3 = 1,       /* 3 streams read */
    NBO_PATTERN_FILL1 = 2,       /* 1 stream written */
    NBO_PATTERN_FILL3 = 3,       /* 3 streams written */
    NBO_PATTERN_COPY = 4,        /* 1 stream read, 1 written */
    NBO_PATTERN_RMW1 = 5,        /* N streams read and rewritten in place */
    NBO_PATTERN_RMW2 = 6,
    NBO_PATTERN_RMW3 = 7,
    NBO_PATTERN_RMW6 = 8,
    NBO_PATTERN_R1_RMW3_W1 = 9   /* 1 read, 3 in place, 1 written: the mixed-precision update's streams */
} nbo_probe_pattern;

/* How a probe kernel moves the bytes.  Shape 0 exists for every pattern, the others for the
 * four 1:1 read/write patterns (COPY, RMW1, RMW3, R1_RMW3_W1). */
typedef enum nbo_probe_shape {
    NBO_SHAPE_UPDATE = 0,     /* the update kernels' own: 256 threads per 32 KiB window of every stream, all
                                 loads issued stream by stream before the first use, through registers */
    NBO_SHAPE_WG512 = 1,      /* the same with 512-thread workgroups, 64 KiB windows */
    NBO_SHAPE_WG1024 = 2,     /* 1024-thread workgroups, 4 rows each, 64 KiB windows */
    NBO_SHAPE_LDS = 3,        /* loads straight into LDS (global_load_lds_dwordx4), 64 KiB of LDS per workgroup */
    NBO_SHAPE_LDS_DEEP = 4,   /* the same with 128-144 KiB of LDS per workgroup */
    NBO_SHAPE_REGS_LDS = 5,   /* shape 0's eight rows through registers and shape 3's rows through LDS together */
    NBO_SHAPE_SPLIT = 6,      /* 512 threads: four waves only load (into LDS), four only store, double-buffered */
    NBO_SHAPE_PIPELINED = 7,  /* next window's loads issued before the current window's stores (registers) */
    NBO_SHAPE_LOOP = 8,       /* shape 0's window, several per workgroup one after the other, nothing overlapped */
    NBO_SHAPE_LDS_PIPELINED = 9,        /* next window's loads travel global -> LDS while the current window,
                                           moved from LDS into registers, is stored; 256 threads */
    NBO_SHAPE_LDS_PIPELINED_WG512 = 10, /* the same with 512 threads and twice the LDS */
    NBO_SHAPE_LDS_PIPELINED_DEEP = 11,  /* shape 9 with twice the rows */
    NBO_SHAPE_FRONTS2 = 12,   /* shape 0's eight rows taken from 2 places of every stream at once (a grid apart) */
    NBO_SHAPE_FRONTS4 = 13,   /* ... from 4 places */
    NBO_SHAPE_FRONTS8 = 14,   /* ... from 8 places */
    NBO_SHAPE_ROWS4 = 15,     /* shape 0 with four rows per workgroup (16 KiB windows) */
    NBO_SHAPE_ROWS2 = 16,     /* ... two rows (8 KiB windows) */
    NBO_SHAPE_ROWS1 = 17,     /* ... one row: every thread loads one vector of every stream, stores, and is done (4 KiB
                                 windows, eight times as many workgroups as shape 0) */
    NBO_SHAPE_COUNT = 18
} nbo_probe_shape;

/* What the memory system gives an access pattern, measured with the library's probe kernels:
 * the yardstick the update kernels' throughput is judged against.  spread = 0: all streams lie
 * back to back in one plain allocation; spread = 1: they are slices of up to three arrays
 * placed across the HBM's regions exactly as optimizer state is (*regions then receives what
 * nbo_optim_state_regions would report).  Allocates and frees its buffers (bytes_per_stream: a
 * multiple of 32 KiB), launches untimed for settle_ms milliseconds (at least once: the driver
 * clears freed device memory in the background, which competes for bandwidth for about a second
 * after a large free) and then `reps` times, timed; *best_gbps / *mean_gbps are bytes moved per
 * launch (reads + writes) over the shortest / the mean duration.  Synchronous.
 * nbo_hbm_ceiling is nbo_hbm_ceiling_shape with NBO_SHAPE_UPDATE and no check.
 * With `mismatches` non-null the streams that are rewritten in place are read back afterwards
 * and every element is compared with the number of launches made (each launch adds 1.0 to every
 * element of such a stream, which starts at zero); *mismatches receives the number of elements
 * that differ -- anything but 0 means the kernel skipped, repeated or misplaced an access. */
int nbo_hbm_ceiling(int pattern, int spread, uint64_t bytes_per_stream, int reps, uint32_t settle_ms,
                    double *best_gbps, double *mean_gbps, int *regions);
int nbo_hbm_ceiling_shape(int pattern, int shape, int spread, uint64_t bytes_per_stream, int reps,
                          uint32_t settle_ms, double *best_gbps, double *mean_gbps, int *regions,
                          uint64_t *mismatches);

/* Several shapes over the same buffers, so that their figures differ by the shape alone and not
 * by the placement or the moment: `rounds` times over shapes[0 .. n_shapes) in turn, `reps`
 * timed launches each; best_gbps / mean_gbps are arrays of n_shapes.  iters (may be null)
 * overrides the windows per workgroup of the looping shapes (0: their default of 8); with bit 31
 * set those windows are neighbours instead of a whole grid apart. */
int nbo_hbm_ceiling_compare(int pattern, int n_shapes, const int *shapes, const uint32_t *iters, int spread,
                            uint64_t bytes_per_stream, int rounds, int reps, uint32_t settle_ms,
                            double *best_gbps, double *mean_gbps, int *regions);

/* What placing the caller's own tensors would buy.  MI355X's HBM behaves as regions of 96 GiB of
 * physical memory; the optimizer's state is spread over them by probing (nbo_optim_create), and
 * this gives memory for parameters and gradients the same treatment, for measurement: n_buffers
 * (2 or 3) device buffers of `bytes` bytes each; buffer k lies wholly in the region numbered
 * region[k] (0, 1 or 2: equal numbers share a region, different numbers lie in different ones;
 * rounded up to whole GiB), or, with -1 for every buffer, the buffers rotate over the regions GiB
 * by GiB as the optimizer's state arrays do.  NBO_ERR_TOO_LARGE with the reason in
 * nbo_last_error() when the search finds no second region or memory runs short.  Measured
 * (python -m nabla_amd.kernel_bench --placed): the kernels over the caller's tensors gain nothing
 * (-3 to +0 %), which is why the drop-in header offers no such allocator. */
typedef struct nbo_placed nbo_placed;
int nbo_alloc_placed(uint32_t n_buffers, uint64_t bytes, const int *region, void **out_ptrs, nbo_placed **out);
int nbo_free_placed(nbo_placed *p);
/* One sentence on what the search found (as nbo_optim_state_placement_note). */
int nbo_placed_note(nbo_placed *p, char *buf, uint64_t buf_bytes);

/* Self-test of the all-16-bit optimizers' arithmetic (half_type NBO_DT_BF16 or NBO_DT_F16).  Their
 * division and square root -- 16-bit operands, the f32 result rounded to the type -- do not run the
 * correctly rounded f32 operation where something cheaper provably rounds to the same 16 bits (bf16:
 * the hardware's approximate reciprocal and square root, by this library; f16: the compiler's
 * lowering of a division whose result is narrowed to f16).  This runs all 2^32 pairs of patterns
 * through the division and all 2^16 patterns through the square root and counts the results that
 * differ from the exact operation's: the f64 operation narrowed to f32 and then to the type (any NaN
 * equals any NaN) and, for bf16, also bit for bit the correctly rounded f32 operation followed by
 * bf16::from_f32.  Anything but 0 and 0 is a bug; *example_pair (numerator << 16 | denominator) and
 * *example_arg (may be null) then name one case each.  A few milliseconds.  Synchronous. */
int nbo_selftest_half_arith(int half_type, uint64_t *div_mismatches, uint64_t *sqrt_mismatches,
                            uint64_t *example_pair, uint64_t *example_arg);

/* Per-kernel timing: while enabled, every kernel launch is bracketed by HIP events on
 * the launch stream.  nbo_profile_read synchronises and returns the number of
 * launches of `kernel_name` (e.g. "nbo_update_bf16_adamw") since profiling was
 * enabled and the sum of their durations.  (The reference times its steps with host
 * timers around a stream sync, nabla-train/src/profiler.rs:176-197.) */
int nbo_profile_enable(int on);
int nbo_profile_read(const char *kernel_name, uint64_t *launches, double *total_ms);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif
#endif
