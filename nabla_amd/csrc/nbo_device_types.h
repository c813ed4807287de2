// Plain-old-data layouts shared by the gfx950 kernels and the host runtime.
// Everything here is passed either by value as the single kernel argument or
// lives in device memory; no pointers to host memory appear in any of them.
#ifndef NBO_DEVICE_TYPES_H
#define NBO_DEVICE_TYPES_H

#include <stdint.h>

// One work unit ("chunk") is this many consecutive elements of one tensor.  A
// 256-thread workgroup handles a chunk in CHUNK / (256 * vec) rows of 128-bit
// accesses; 8192 with all 8 f32 rows in flight measured best on MI355X (6.3-6.4 TB/s
// against 6.2-6.3 for 4096 and 16384).
#ifndef NBO_CHUNK
#define NBO_CHUNK 8192u
#endif
// The element-wise passes over the caller's lists (scale, zero, accumulate; the backend
// primitives) run one workgroup per "piece" of every list: 4 KiB is one 128-bit vector per
// thread -- load, compute, store, done.  Many short-lived workgroups measured 16-21 % faster
// than eight rows per workgroup for the one- and two-list passes (5.5 -> 6.5-6.7 TB/s on 738 M
// elements); the backend primitives carry more arithmetic and pointers per workgroup and do
// best at two rows (6.0-6.5 TB/s against 5.3-5.9).
#ifndef NBO_EW_PIECE_BYTES
#define NBO_EW_PIECE_BYTES 4096u
#endif
#ifndef NBO_BACKEND_PIECE_BYTES
#define NBO_BACKEND_PIECE_BYTES 8192u
#endif
// groups of four elements per thread of the cast pass (738 M elements, f32 -> bf16 / bf16 -> f32: one group
// 5.55 / 5.82 TB/s, two 6.45 / 6.05, four 6.2 / 5.7)
#ifndef NBO_CAST_QUADS
#define NBO_CAST_QUADS 2u
#endif
#define NBO_CAST_ROW (4u * NBO_CAST_QUADS * NBO_BLOCK) // elements per workgroup of the cast pass
#ifndef NBO_BLOCK
#define NBO_BLOCK 256u
#endif

// The norm pass runs a fixed grid so that its per-block partial sums, and hence
// the reduced norm, do not depend on anything but the tensor list itself.
#ifndef NBO_NORM_GRID_MAX
#define NBO_NORM_GRID_MAX 2048u
#endif
// Per-step trace ring kept on the device (found_inf / skipped / scale / step_count).
#define NBO_TRACE_LEN 1024u

// Element storage types of caller tensors.  NBO_PBF16 is bf16 storage with bf16
// arithmetic (the reference's Optimizer<bf16>: every operation rounds to bf16), as
// opposed to NBO_BF16 = bf16 tensors over f32 state; it only selects kernels.  NBO_F16 /
// NBO_PF16 are the same pair for IEEE binary16.
enum { NBO_F32 = 0, NBO_BF16 = 1, NBO_F64 = 2, NBO_F16 = 3, NBO_PBF16 = 4, NBO_PF16 = 5 };
// OptimKind order of the reference (nabla-train/src/optim/core.rs:46-51).
enum { NBO_ADAMW = 0, NBO_ADAM = 1, NBO_SGD = 2 };

// Packed tensor-list descriptor, resident in device memory.
//   n[t]             element count of tensor t
//   chunk_begin[t]   index of tensor t's first chunk (chunk_begin[nt] = nchunks)
//   chunk_tensor[c]  tensor that chunk c belongs to
// Element offsets into the optimizer's state arena are in soff[t].
struct NboLayoutDev {
    const uint64_t *n;
    const uint64_t *soff;
    const uint32_t *chunk_begin;
    const uint32_t *chunk_tensor;
    uint32_t nt;
    uint32_t nchunks;
    // Lists of many small tensors, for the kernels that run one workgroup per row of a chunk: the
    // rows that exist, in order, as chunk * 16 + row (null: every chunk counts as whole and
    // workgroup w is row w % rows-per-chunk of chunk w / rows-per-chunk).
    const uint32_t *row_map;
    uint32_t nrows;
    uint32_t pad;
};

// GradScalerState (optim/core.rs:326-332), device resident.
struct NboScalerDev {
    double scale, growth_factor, backoff_factor;
    uint64_t growth_interval, consecutive_ok;
};

// Result of the norm / found_inf pass after its deterministic second stage.
// inv_scale and clip are the two factors the reference multiplies every gradient
// element by (core.rs:379, trainer.rs:519); 1.0 when the respective stage is off.
struct NboGradFactors {
    double sumsq;       // sum of squares of the unscaled gradients
    double norm;        // sqrt(sumsq); what clip_grad_norm returns
    double inv_scale64; // T::from_f64(1/scale) for T = f64
    double clip64;      // T::from_f64(max_norm/norm) for T = f64
    float inv_scale32;  // same, narrowed for T = f32
    float clip32;
    uint32_t found_inf; // 1: a gradient was inf/NaN, step is skipped
    uint32_t clipped;   // 1: norm > max_norm, gradients are rescaled
};

// OptimMeta (optim/core.rs:53-62) plus the per-step scalars derived from it
// (alg.rs:120-135, 266-277, 393-395), device resident.
struct NboOptimDev {
    double lr, beta1, beta2, eps, weight_decay, momentum;
    uint64_t step_count;
    uint32_t kind;
    uint32_t skip; // this step is skipped (found_inf)
    // scalars narrowed to T exactly as the reference narrows them
    float b1, omb1, b2, omb2, eps_t, ss, ibc2, omw;
    float neg_lr, momentum_t, wd_t;
    float wd_lr_t; // T::from_f64(weight_decay * lr) for T = f32 (bf16 narrows it once more)
    double d_b1, d_omb1, d_b2, d_omb2, d_eps, d_ss, d_ibc2, d_omw;
    double d_neg_lr, d_momentum, d_wd;
    // Counts the workgroups of a "_self" update launch that have read step_count; the one that
    // brings it to the grid size knows that all have, advances step_count in place and puts the
    // counter back to zero.  Zero between launches.
    uint32_t ticket;
    uint32_t pad;
};

// Hyper-parameters as the host holds them; handed to the device with every step so
// that set_lr and friends need no copy of their own.
struct NboHyper {
    double lr, beta1, beta2, eps, weight_decay, momentum;
    uint32_t kind;
    uint32_t pad;
};

// One entry of the device-side step trace.
struct NboTraceEntry {
    double scale;        // scaler scale after the step's update
    double norm;         // pre-clip norm (0 if skipped)
    uint64_t step_count; // optimizer step_count after the step
    uint32_t found_inf;
    uint32_t clipped;
};

struct NboTraceDev {
    uint64_t count; // total entries ever written; entry i lives at i % NBO_TRACE_LEN
    NboTraceEntry e[NBO_TRACE_LEN];
};

// ---- kernel argument blocks (each kernel takes exactly one, by value) ----------

// The optimizer's state: one planar device array per state "part".  Part 0 is the
// first moment (SGD: velocity), part 1 the second moment (Adam / AdamW), the last
// part the f32 master weights when kept.  Within a part, tensor t starts at element
// soff[t] (a multiple of NBO_CHUNK: every tensor is padded to whole chunks).  The
// parts are separate allocations so that the host can place them in different
// regions of HBM.  (A tiled variant that puts the parts of each chunk back to back
// measured 1-2 % slower on MI355X.)
struct NboArenaDev {
    void *part[3];
    uint32_t nparts;
    uint32_t part_v; // index of the second-moment part (unused for SGD)
    uint32_t part_w; // index of the master part (unused without master)
    uint32_t pad;
};

struct NboUpdateArgs {
    NboLayoutDev L;
    const uint64_t *p_ptrs; // caller parameter tensors (device addresses)
    const uint64_t *g_ptrs; // caller gradient tensors
    NboArenaDev arena;
    const NboOptimDev *opt;
    const NboGradFactors *gf; // null: gradients are used as they are
    uint32_t zero_grads;      // bit 0: write zeros over the gradients after reading them (and on a skipped
                              // step); bit 1: on a skipped step only (core.rs:372-375)
    // SGD outside the fused tail needs no device-side state at all (it has no
    // step_count and cannot be skipped): with `direct` set its three scalars come from
    // here and `opt` is not read, which saves the scalar-preparation launch
    uint32_t direct;
    double sgd_lr, sgd_momentum, sgd_weight_decay;
    // The "_self" kernels prepare the step's scalars themselves (every workgroup, from
    // opt->step_count, `hyper` and *gf); the workgroup that is the last to have read
    // step_count (opt->ticket counts them) writes the advanced step_count back through opt_rw
    // (= opt) and, if set, a trace entry (with the scaler's scale after its update).  Unused
    // by the other kernels.
    NboHyper hyper;
    NboOptimDev *opt_rw;
    NboTraceDev *trace;
    const NboScalerDev *scaler;
};

// Argument block of the "_self" update kernels: one launch over several groups' lists.
// Workgroups [first_wg[k], first_wg[k + 1]) work on group k; first_wg[n_groups] is the grid.
#define NBO_GROUPS_PER_LAUNCH 16u
struct NboGroupedUpdateArgs {
    NboUpdateArgs g[NBO_GROUPS_PER_LAUNCH];
    uint32_t first_wg[NBO_GROUPS_PER_LAUNCH + 1];
    uint32_t n_groups;
};

struct NboFinalizeArgs {
    const double *partial_sumsq;
    const uint32_t *partial_flag;
    uint32_t grid;
    uint32_t check_finite; // GradScaler semantics (found_inf => skip); 0 for plain clip
    NboScalerDev *scaler;  // may be null
    NboGradFactors *gf;    // out
    NboOptimDev *opt;      // may be null: if set, also advance step_count + scalars
    NboTraceDev *trace;    // may be null
    double max_norm;       // <= 0 disables clipping (trainer.rs:501-503)
    NboHyper hyper;        // copied into *opt before the scalars are derived
    double sumsq_in;       // with use_sumsq_in: the sum of squares, already known (grid = 0)
    uint32_t use_sumsq_in;
    uint32_t pad;
    uint32_t *any_bad;     // may be null: a word some pass ORed its non-finite findings into; read, then cleared
};

struct NboNormArgs {
    NboLayoutDev L;
    const uint64_t *g_ptrs;
    const NboScalerDev *scaler; // null: no unscale, inv_scale = 1
    double *partial_sumsq;      // [grid]
    uint32_t *partial_flag;     // [grid]
    uint32_t grid;
    uint32_t pad;
};


struct NboPrepArgs {
    NboOptimDev *opt;
    const NboGradFactors *gf;   // may be null
    const NboScalerDev *scaler; // may be null; only read, for the trace entry
    NboTraceDev *trace;         // may be null
    NboHyper hyper;
};

// One micro-batch of the accumulating Trainer in a single pass (trainer.rs:230-267): finite
// scan of g, acc[i] = acc[i] + T(g[i] * inv_scale), and -- nbo_accnorm_* -- the sum of squares of
// the new acc.  Both forms run like the element-wise passes, one short-lived workgroup per piece
// (per chunk of a list of small tensors), and OR whether they met a non-finite gradient into
// *any_bad, which the second stage reads and clears.
struct NboAccNormArgs {
    NboLayoutDev L;
    const uint64_t *acc_ptrs;
    const uint64_t *g_ptrs;
    const NboScalerDev *scaler; // null: no unscale, inv_scale = 1
    double *partial_sumsq;      // [grid]: one sum of squares per workgroup (nbo_accnorm_* only)
    uint32_t *partial_flag;     // [grid] or null: zeroed, for a second stage that reads flags beside the sums
    uint32_t grid;              // workgroups that have a piece (a folded launch may have more)
    uint32_t write_grads;       // also store the unscaled gradients in place, as the reference does
    uint32_t *any_bad;
    uint32_t by_chunk; // see NboAccumArgs
    uint32_t pad;
};

// Between a pass that leaves one partial sum per piece and the second stage, which reads at most
// NBO_NORM_GRID_MAX of them: workgroup j adds in[j * per .. min(n, (j + 1) * per)) in a fixed
// order into out[j] and clears out_flag[j].
struct NboSumPartialsArgs {
    const double *in;
    double *out;
    uint32_t *out_flag;
    uint32_t n;
    uint32_t per;
};

// a[i] = a[i] + b[i] over two lists of the same shapes (gradient accumulation).
struct NboAccumArgs {
    NboLayoutDev L;
    const uint64_t *a_ptrs;
    const uint64_t *b_ptrs;
    uint32_t zero_b; // also clear b after it has been added
    uint32_t by_chunk; // one workgroup per chunk, not per piece (a list of many small tensors)
};

struct NboScaleArgs {
    NboLayoutDev L;
    const uint64_t *g_ptrs;
    const NboGradFactors *gf; // if set: multiply by inv_scale (mode 0) or clip (mode 1);
                              // on found_inf (mode 0) write zeros instead
    double factor;            // used when gf is null
    uint32_t mode;            // 0 unscale, 1 clip, 2 plain factor, 3 zero fill
    uint32_t by_chunk;        // one workgroup per chunk, not per piece (a list of many small tensors)
};

struct NboCastArgs {
    NboLayoutDev L;
    const uint64_t *src_ptrs;
    const uint64_t *dst_ptrs;
    NboArenaDev arena; // the master part is one side of the cast
    uint32_t mode;      // 0: master(f32) <- src widen; 1: dst <- master(f32) narrow
    uint32_t half_type; // NBO_BF16 or NBO_F16: the tensors' element type
};

struct NboFillArgs {
    void *p;
    uint64_t bytes;
};

// nbo_selftest_{bf16,f16}_arith: out[0] = pairs (a, b) of 16-bit patterns whose quotient differs between
// the kernels' division and the exact one, out[1] = the same for the square root's arguments,
// out[2], out[3] = one such pair (a << 16 | b) and one such argument.  The caller zeroes out[].
struct NboSelftestArgs {
    unsigned long long *out;
};

// Backend primitives on tensor lists (nabla-core/src/common/backend/mod.rs:82-216,
// 275-279): one IEEE operation per element, every result rounded to the element type.
enum {
    NBO_EW_SCALE = 0,      // out = a * s
    NBO_EW_AXPY = 1,       // out = out + s * a      (two roundings, in place on out)
    NBO_EW_ADD = 2,        // out = a + b
    NBO_EW_EMUL = 3,       // out = a * b
    NBO_EW_EDIV = 4,       // out = a / b
    NBO_EW_POWF = 5,       // out = powf(a, s)
    NBO_EW_ADD_SCALAR = 6, // out = a + s
    NBO_EW_ZEROS = 7,      // out = 0
    NBO_EW_COPY = 8,       // out = a
    NBO_EW_COUNT = 9
};

struct NboEwArgs {
    NboLayoutDev L;
    const uint64_t *out_ptrs;
    const uint64_t *a_ptrs; // null for NBO_EW_ZEROS
    const uint64_t *b_ptrs; // null unless the operation has two tensor operands
    double s;               // narrowed to the element type on the device
    uint32_t op;
    uint32_t by_chunk; // one workgroup per chunk, not per piece (a list of many small tensors)
};

// Element-type conversion of a tensor list through f64, as BackendCore::cast's default
// (backend/mod.rs:157-160).
struct NboCastListArgs {
    NboLayoutDev L;
    const uint64_t *dst_ptrs;
    const uint64_t *src_ptrs;
    uint32_t dst_type, src_type; // NBO_F32 / NBO_BF16 / NBO_F64
    uint32_t by_chunk;           // one workgroup per chunk, not per row (a list of many small tensors)
    uint32_t pad;
};

// Memory-system ceiling probe: which streams are read, rewritten in place or only written.
enum {
    NBO_PROBE_READ1 = 0,      // 1 stream read
    NBO_PROBE_READ3 = 1,      // 3 streams read
    NBO_PROBE_FILL1 = 2,      // 1 stream written
    NBO_PROBE_FILL3 = 3,      // 3 streams written
    NBO_PROBE_COPY = 4,       // stream 0 read, stream 1 written
    NBO_PROBE_RMW1 = 5,       // N streams read and rewritten in place
    NBO_PROBE_RMW2 = 6,
    NBO_PROBE_RMW3 = 7,
    NBO_PROBE_RMW6 = 8,
    NBO_PROBE_R1_RMW3_W1 = 9, // the mixed-precision update's shape: 1 read, 3 in place, 1 written
    NBO_PROBE_COUNT = 10
};

struct NboStreamProbeArgs {
    void *buf[8];   // streams in the order read-only, in place, write-only
    uint32_t iters;      // windows per workgroup, for the shapes whose workgroups loop
    uint32_t contiguous; // those windows are neighbours (1) or a whole grid apart (0)
};

#endif
