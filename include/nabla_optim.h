/*
 * nabla_optim.h -- C ABI of the MI355X (gfx950) fused optimizer-step engine.
 *
 * This is the drop-in boundary for ONE path of fumishiki/nabla: the optimizer
 * step of nabla-train (Sgd / Adam / AdamW step, GradScaler unscale + found-inf +
 * dynamic scale, clip_grad_norm, zero_grad, exportable moments and master
 * weights).  A Rust `impl Optimizer<T, B>` / `impl OptimState<T, B>` in
 * nabla-train binds these symbols through `extern "C"`; nothing here needs a
 * C++ or torch type.  Each declaration cites the reference item it replaces
 * (paths relative to the reference checkout).
 *
 * Conventions
 *   - Every function returns an nbo_status.  Nothing aborts or throws; the
 *     language-level shim turns NBO_ERR_LEN_MISMATCH / NBO_ERR_COUNT_MISMATCH /
 *     NBO_ERR_SHAPE into the reference's panics and the NBO_ERR_STATE_* /
 *     NBO_ERR_KIND codes into its Err(String) values.  nbo_last_error() returns
 *     the message of the calling thread's last failure.
 *   - Tensors are dense row-major (rows, cols) matrices in device memory owned by
 *     the caller (nabla-core/src/cpu/mod.rs:7-11,28-30 layout); only rows*cols
 *     matters to the arithmetic.  The engine owns moments and master weights.
 *   - All work is enqueued on one HIP stream (the null stream unless
 *     nbo_set_stream is called), in call order; calls that return a value to the
 *     host (ok flags, norms, state reads) synchronise that stream, the others do
 *     not.  One caller at a time: the reference's Optimizer takes &mut self and
 *     has no Send bound (optim/core.rs:9-44).
 *   - Device 0, like the reference's HIP context (cuda_hip/hip/core.rs:331-355).
 */
#ifndef NABLA_OPTIM_H
#define NABLA_OPTIM_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#pragma GCC visibility push(default)

typedef enum nbo_status {
    NBO_OK = 0,
    NBO_ERR_LEN_MISMATCH = 1,   /* params.len() != grads.len()         alg.rs:110-114 */
    NBO_ERR_COUNT_MISMATCH = 2, /* params.len() != optimizer's count   alg.rs:115-119 */
    NBO_ERR_SHAPE = 3,          /* "shapes must match"                 tensor/ops.rs:638-646 */
    NBO_ERR_STATE_KEY = 4,      /* "bad tensor key: {name}"            alg.rs:491-494 */
    NBO_ERR_STATE_INDEX = 5,    /* "m index out of range: {i}"         alg.rs:495-497 */
    NBO_ERR_KIND = 6,           /* "optim kind mismatch"               alg.rs:531-545 */
    NBO_ERR_DTYPE = 7,          /* element types of the lists / optimizer do not fit */
    NBO_ERR_ARG = 8,            /* null pointer, zero-sized list, bad enum value */
    NBO_ERR_NO_MASTER = 9,      /* bf16 / f16 step before master weights were set */
    NBO_ERR_TOO_LARGE = 10,     /* more than 2^24-1 chunks of 8192 elements (1.4e11 elements) */
    NBO_ERR_NO_DEVICE = 11,     /* no gfx950 device / code object not loadable */
    NBO_ERR_IO = 12,            /* checkpoint file: io::Error of save_tensors / load_tensors */
    NBO_ERR_HIP = 1000          /* NBO_ERR_HIP + hipError_t */
} nbo_status;

/* Element type of caller tensors. */
typedef enum nbo_dtype { NBO_DT_F32 = 0, NBO_DT_BF16 = 1, NBO_DT_F64 = 2, NBO_DT_F16 = 3 } nbo_dtype;

/* OptimKind, in the reference's order (optim/core.rs:46-51). */
typedef enum nbo_kind { NBO_KIND_ADAMW = 0, NBO_KIND_ADAM = 1, NBO_KIND_SGD = 2 } nbo_kind;

/* OptimMeta (optim/core.rs:53-62).  Hyper-parameters cross the boundary as f64 and
 * are narrowed to the arithmetic type inside, exactly as alg.rs:122-135 does. */
typedef struct nbo_meta {
    int32_t kind;
    int32_t reserved;
    double lr, beta1, beta2, eps, weight_decay, momentum;
    uint64_t step_count;
} nbo_meta;

/* GradScalerState (optim/core.rs:326-332). */
typedef struct nbo_scaler_state {
    double scale, growth_factor, backoff_factor;
    uint64_t growth_interval, consecutive_ok;
} nbo_scaler_state;

/* What one fused step decided; also one entry of the step trace. */
typedef struct nbo_step_info {
    double scale;        /* scaler scale after this step's update (0 without scaler) */
    double norm;         /* pre-clip global norm; 0 if skipped or clipping disabled */
    uint64_t step_count; /* optimizer step_count after the step */
    uint32_t found_inf;  /* 1: a gradient was inf/NaN, the step was skipped */
    uint32_t clipped;    /* 1: norm > max_norm, gradients were rescaled */
} nbo_step_info;

typedef struct nbo_list nbo_list;     /* a list of same-dtype device tensors */
typedef struct nbo_optim nbo_optim;   /* Sgd / Adam / AdamW + its state */
typedef struct nbo_scaler nbo_scaler; /* GradScaler */

/* ---- runtime -------------------------------------------------------------------- */

/* Load the precompiled gfx950 code object on device 0 and create the runtime
 * (the reference does this lazily in cuda_hip/hip/core.rs:331-355; every other
 * entry point calls it implicitly). */
int nbo_init(void);
/* Use `hip_stream` (a hipStream_t) for all subsequent work; NULL = the null stream,
 * which is what the reference's HIP backend launches on (hip/backend.rs:337).  Waits for
 * what is already enqueued on the previous stream (the two share the library's scratch and
 * the optimizers' state), so call it outside stream capture. */
int nbo_set_stream(void *hip_stream);
/* B::sync (common/backend/mod.rs:82-216): wait for all enqueued work. */
int nbo_sync(void);
const char *nbo_last_error(void);
const char *nbo_status_string(int status);
/* "major.minor.patch" of this library. */
const char *nbo_version(void);

/* ---- tensor lists: the &[&Tensor<T,B>] / &mut [&mut Tensor<T,B>] arguments ----- */

/* `dev_ptrs[i]` is the device address of tensor i (RtcStorage buffer of the HIP
 * backend, common/rtc.rs:34-37), rows[i] x cols[i] elements of `dtype`.  The
 * packed descriptor is built and uploaded once; nbo_list_set_ptrs re-uploads the
 * addresses when the caller's tensors have moved.  Both check every address against
 * what the HIP runtime knows about it -- device-accessible memory, the tensor ending
 * inside its allocation -- and return NBO_ERR_ARG otherwise (a host pointer or an
 * oversized shape would fault the GPU); NBO_CHECK_POINTERS=0 in the environment skips
 * that.  The same holds for the device buffers of nbo_optim_state_read / _write.  A tensor
 * may start at any address that is a multiple of its element size (views into flat buffers,
 * tensors packed back to back): whole 16-byte vectors are used wherever the addresses allow,
 * and 16-bit tensors over f32 state are accessed in whole vectors at any even address. */
int nbo_list_create(uint64_t n_tensors, const uint64_t *rows, const uint64_t *cols, int dtype,
                    const void *const *dev_ptrs, nbo_list **out);
int nbo_list_set_ptrs(nbo_list *list, const void *const *dev_ptrs);
int nbo_list_destroy(nbo_list *list);

/* ---- optimizer: Sgd / Adam / AdamW (optim/alg.rs) -------------------------------- */

/* Sgd::new / Adam::new / AdamW::new (alg.rs:319-330, 181-199, 20-39) + the builder
 * setters, all at once through `meta` (meta->kind selects the algorithm;
 * meta->step_count seeds step_count).  Moments are created zero-filled.
 * state_dtype: NBO_DT_F32, NBO_DT_F64, NBO_DT_BF16 or NBO_DT_F16 -- the arithmetic type T,
 * which is also the type of the moments and of the caller's tensors (T = bf16 / f16: every
 * operation is the f32 operation followed by T::from_f32, common/scalar/mod.rs:253-351).
 * keep_master != 0 (f32 state only): additionally hold f32 master weights so that the
 * caller's parameters and gradients may be bf16 or f16 while the arithmetic stays T = f32.
 * State of 128 MiB per array or more is assembled from physical chunks chosen so that
 * the arrays lie in different regions of the HBM (nbo_optim_state_regions tells the
 * outcome); that takes up to a few seconds here and nothing per step. */
int nbo_optim_create(const nbo_meta *meta, uint64_t n_tensors, const uint64_t *rows,
                     const uint64_t *cols, int state_dtype, int keep_master, nbo_optim **out);
int nbo_optim_destroy(nbo_optim *opt);

/* Optimizer::step (optim/core.rs:10; alg.rs:109-150, 254-291, 382-416).  Gradients
 * are used as they are.  Asynchronous. */
int nbo_optim_step(nbo_optim *opt, nbo_list *params, nbo_list *grads);
/* Optimizer::reset (alg.rs:152-162, 293-303, 418-423). */
int nbo_optim_reset(nbo_optim *opt);
/* Optimizer::set_lr (alg.rs:164-166, 305-307, 425-427). */
int nbo_optim_set_lr(nbo_optim *opt, double lr);
/* OptimState::meta / load_meta (alg.rs:518-545, 595-615, 650-670).  load_meta
 * returns NBO_ERR_KIND when meta->kind differs from the optimizer's. */
int nbo_optim_get_meta(nbo_optim *opt, nbo_meta *out);
int nbo_optim_load_meta(nbo_optim *opt, const nbo_meta *meta);

/* OptimState::state_tensors / load_state_tensors (alg.rs:476-516, 553-593, 623-648),
 * one tensor at a time.  `name` is "m{i}" / "v{i}" (Adam, AdamW), "v{i}" (Sgd
 * velocity), or "w{i}" for the f32 master weights (no counterpart in the reference,
 * which has no mixed-precision optimizer).  `n_elems` must equal rows*cols of
 * tensor i; elements have the optimizer's state dtype.  `on_device` says whether
 * `buf` is a device or a host address. */
int nbo_optim_state_read(nbo_optim *opt, const char *name, void *buf, uint64_t n_elems,
                         int on_device);
int nbo_optim_state_write(nbo_optim *opt, const char *name, const void *buf, uint64_t n_elems,
                          int on_device);
/* master = f32(params) for bf16 or f16 parameter lists (Tensor::cast, tensor/shape.rs:489-493),
 * and the converse params = bf16(master) / f16(master). */
int nbo_optim_master_from_params(nbo_optim *opt, nbo_list *params_half);
int nbo_optim_params_from_master(nbo_optim *opt, nbo_list *params_half);

/* How the optimizer's state arrays were placed in HBM: *regions = 0 for plain
 * allocations, otherwise the number of HBM regions their chunks were spread over (no
 * counterpart in the reference; see nbo_placement.hpp). */
int nbo_optim_state_regions(nbo_optim *opt, int *regions);
/* One line on the same, for logs: what the placement found ("3 regions, chunks of 2048 MiB;
 * 44 chunks created, 130 probes; same region 5385 GB/s, threshold 6020 GB/s, ...") or why plain
 * allocations were taken instead ("plain allocations: <reason>").  At most buf_bytes - 1
 * characters and a terminating NUL are written. */
int nbo_optim_state_placement_note(nbo_optim *opt, char *buf, uint64_t buf_bytes);

/* ---- GradScaler (optim/core.rs:254-260, 334-413) ---------------------------------- */

/* GradScaler::new + load_state; state == NULL gives the defaults of core.rs:336-344. */
int nbo_scaler_create(const nbo_scaler_state *state, nbo_scaler **out);
int nbo_scaler_destroy(nbo_scaler *s);
int nbo_scaler_state_get(nbo_scaler *s, nbo_scaler_state *out); /* GradScaler::state */
int nbo_scaler_load_state(nbo_scaler *s, const nbo_scaler_state *state);
/* GradScaler::unscale_and_update (core.rs:351-388), in place, in the gradients' own type.
 * *ok = 1 if all gradients were finite (they are now unscaled), 0 otherwise (they
 * are now zeros, scale was backed off).  Synchronous. */
int nbo_scaler_unscale_and_update(nbo_scaler *s, nbo_list *grads, int *ok);

/* ---- gradient utilities ------------------------------------------------------------ */

/* clip_grad_norm (nabla-train/src/trainer.rs:500-523), in place, in the gradients'
 * own type; *norm receives the pre-clip norm (0 when max_norm <= 0).  Synchronous. */
int nbo_clip_grad_norm(nbo_list *grads, double max_norm, double *norm);
/* Trainer::has_non_finite (nabla-train/src/trainer.rs:387-400): *found = 1 if any gradient
 * element is inf or NaN.  One read-only pass; synchronous (the Trainer branches on it). */
int nbo_has_non_finite(nbo_list *grads, int *found);
/* zero_grad (nabla-ml/src/autograd/ops.rs:1668-1673; trainer.rs:285-290). */
int nbo_zero_grad(nbo_list *grads);
/* scale_grad (autograd/ops.rs:1675-1680), in the gradients' own type. */
int nbo_scale_grad(nbo_list *grads, double factor);

/* ---- the fused Trainer tail ---------------------------------------------------------- */

#define NBO_STEP_ZERO_GRADS 1u     /* trainer.rs:285-290 folded into the update */
#define NBO_STEP_SKIP_NONFINITE 2u /* GradNanPolicy::Skip (trainer.rs:239-245) without a scaler */
#define NBO_STEP_ZERO_ON_SKIP 4u   /* a skipped step leaves zeros in the gradients, as unscale_and_update
                                      does when it finds inf / NaN (optim/core.rs:372-375) */

/* One Trainer iteration after backward (trainer.rs:230-291) in three launches:
 *   scaler.unscale_and_update(grads)  -> found_inf, skip, scale update
 *   clip_grad_norm(grads, max_norm)   -> only when max_norm > 0
 *   optimizer.step(params, grads)     -> unscale and clip factors applied on the fly
 *   params = bf16(master)             -> for bf16 lists (f16(master) for f16 lists)
 *   zero grads                        -> with NBO_STEP_ZERO_GRADS
 * `scaler` may be NULL.  Gradients are not modified (except for the optional
 * zeroing): the two factors are applied inside the update, element by element,
 * with the same roundings as the reference's in-place passes.  The skip decision
 * is taken on the device; nothing is read back.  On a skipped step the reference's
 * unscale_and_update replaces the gradients by zeros (core.rs:372-375); this call does that
 * with NBO_STEP_ZERO_ON_SKIP (or NBO_STEP_ZERO_GRADS, which zeroes after every step) and
 * otherwise leaves them as they are, inf / NaN included.  Asynchronous. */
int nbo_fused_step(nbo_optim *opt, nbo_scaler *scaler, nbo_list *params, nbo_list *grads,
                   double max_norm, uint32_t flags);
/* nbo_fused_step for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in
 * the reference.  Same arguments, same three launches and bit-identical results; the only
 * difference is where the norm pass keeps its per-workgroup partial results: not in the
 * buffer nbo_init allocated but in a 32 KiB array that is part of the library's device image
 * (one copy per GPU, held until the process ends).  The call itself makes no hipMalloc /
 * hipFree and creates no events (nbo_profile_enable does not time its launches); the handles
 * it takes were created, with their allocations, beforehand.
 * Limit: the norm pass may use at most NBO_NOALLOC_MAX_PARTIALS (2048) workgroups, which is
 * also the grid cap of the ordinary entry point, so every list the library accepts fits;
 * a library rebuilt with a larger cap returns NBO_ERR_TOO_LARGE here instead of overrunning
 * the array.  All calls on one GPU share the array: it keeps the previous call's contents
 * (every slot a call reads is first written by that call, so nothing needs clearing), and two
 * calls that overlap on one GPU -- different streams or threads -- race on it.  Asynchronous. */
int nbo_fused_step_noalloc(nbo_optim *opt, nbo_scaler *scaler, nbo_list *params, nbo_list *grads,
                           double max_norm, uint32_t flags);
/* The same tail for GroupOptimizer (optim/groups.rs:269-293): one unscale / found-inf /
 * clip decision over `all_grads` (every gradient, in the module's order), then each
 * group's update with its own hyper-parameters.  params[g] / grads[g] are the lists of
 * group g's tensors; together the groups must cover all_grads.  Three launches: the norm
 * pass, its second stage and one update launch for up to sixteen groups of one optimizer kind
 * and element type (further groups, or groups of another kind, add a launch).  Asynchronous. */
int nbo_fused_step_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                          nbo_list *const *grads, nbo_scaler *scaler, nbo_list *all_grads,
                          double max_norm, uint32_t flags);
/* Gradient accumulation of the Trainer, buf[i] = &buf[i] + g (trainer.rs:262-266),
 * optionally zeroing the gradients in the same pass.  Asynchronous. */
int nbo_accumulate(nbo_list *accum, nbo_list *grads, int zero_grads);
/* One micro-batch of the accumulating Trainer in a single pass over the gradients
 * (trainer.rs:230-267): the finite scan and loss-scale update of
 * GradScaler::unscale_and_update (core.rs:351-388; `scaler` may be null: no unscale),
 * buf[i] = &buf[i] + T(g * T(1 / scale)), and the sum of squares of the new buffer, which
 * the clip of the last micro-batch needs (trainer.rs:504-513; hand it to
 * nbo_fused_step_norm).  *ok = 0 on a non-finite gradient (with a scaler, or with
 * NBO_ACC_CHECK_FINITE for GradNanPolicy): the buffer then holds garbage, as the Trainer
 * discards the accumulation (trainer.rs:232-236, 241-245).  The gradients themselves stay
 * as they were unless NBO_ACC_WRITE_GRADS asks for the reference's in-place result
 * (unscaled, or zeros when non-finite).  Results are those of
 * nbo_scaler_unscale_and_update followed by nbo_accumulate, bit for bit.  accum_sumsq may be
 * null -- only the last micro-batch of an accumulation needs the sum of squares -- and the
 * pass then has nothing to reduce but one bit (one small launch fewer).  The sum is added up in
 * f64 in a fixed order, the same bits on every run; the order is not the norm pass's, so the
 * norm nbo_fused_step_norm derives from it can differ from nbo_fused_step's in the last bits of
 * the f64.  Synchronous. */
#define NBO_ACC_CHECK_FINITE 1u
#define NBO_ACC_WRITE_GRADS 2u
int nbo_unscale_accumulate(nbo_scaler *scaler, nbo_list *accum, nbo_list *grads, uint32_t flags, int *ok,
                           double *accum_sumsq);
/* clip_grad_norm + Optimizer::step (+ zeroing with NBO_STEP_ZERO_GRADS) over gradients whose
 * sum of squares is already known -- from nbo_unscale_accumulate, if nothing has written the
 * buffer since -- so the norm pass is not run again (trainer.rs:274-290).  No scaler and no
 * finite check: both belong to the micro-batches.  Asynchronous. */
int nbo_fused_step_norm(nbo_optim *opt, nbo_list *params, nbo_list *grads, double max_norm, double sumsq,
                        uint32_t flags);
/* The same for GroupOptimizer (optim/groups.rs:269-293): `sumsq` is that of all the groups'
 * gradients together.  Asynchronous. */
int nbo_fused_step_groups_norm(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                               nbo_list *const *grads, double max_norm, double sumsq, uint32_t flags);
/* ---- Backend primitives on tensor lists ------------------------------------------------
 * The single passes the reference's optimizers are chains of, as multi-tensor launches:
 * BackendCore::{scale, axpy_inplace, add, zeros, clone_storage}
 * (nabla-core/src/common/backend/mod.rs:82-216; CPU semantics nabla-core/src/cpu/mod.rs:137-139,
 * 181, 211-232), BackendMath::{powf, emul, ediv} (backend/mod.rs:275-279; cpu/mod.rs:264-272) and
 * Tensor::map(|x| x + s) (nabla-train/src/optim/alg.rs:133).  One IEEE operation per element
 * in the lists' element type (bf16 / f16: the f32 operation, then T::from_f32,
 * common/scalar/mod.rs:253-351); `s` is narrowed with T::from_f64.  All lists share shapes and
 * element type; `out` may alias an operand.  powf with s = 0.5 is the correctly rounded
 * square root, other exponents use the device math library (within 2 ulp of libm).  The
 * generalisation of the reference's unused k_multi_axpy3 kernel
 * (cuda_hip/common/kernels/k_ops.cuh:541-575) is NBO_BACKEND_AXPY.  Asynchronous. */
typedef enum nbo_backend_op {
    NBO_BACKEND_SCALE = 0,      /* out = a * s */
    NBO_BACKEND_AXPY = 1,       /* out = out + s * a   (product and sum each rounded) */
    NBO_BACKEND_ADD = 2,        /* out = a + b */
    NBO_BACKEND_EMUL = 3,       /* out = a * b */
    NBO_BACKEND_EDIV = 4,       /* out = a / b */
    NBO_BACKEND_POWF = 5,       /* out = powf(a, s) */
    NBO_BACKEND_ADD_SCALAR = 6, /* out = a + s */
    NBO_BACKEND_ZEROS = 7,      /* out = 0             (a, b unused) */
    NBO_BACKEND_CLONE = 8       /* out = a */
} nbo_backend_op;
int nbo_backend_apply(int op, nbo_list *out, nbo_list *a, nbo_list *b, double s);
/* BackendCore::cast, default implementation (backend/mod.rs:157-160): dst = U::from_f64(
 * src.to_f64()) per element, between any two of f32 / bf16 / f16 / f64 (f64 -> bf16 or f16
 * rounds to f32 first, as their from_f64 does).  Asynchronous. */
int nbo_backend_cast(nbo_list *dst, nbo_list *src);

/* Outcome of the optimizer's most recent fused step.  Synchronous. */
int nbo_optim_last_step(nbo_optim *opt, nbo_step_info *out);
/* The last `max_entries` (at most 1024) fused-step outcomes, oldest first; *n_out
 * receives how many were written, *total how many fused steps ran in all. */
int nbo_optim_trace_read(nbo_optim *opt, nbo_step_info *out, uint64_t max_entries,
                         uint64_t *n_out, uint64_t *total);

/* ---- checkpoint tensor files (NBLA) ------------------------------------------------------
 * nabla-train's checkpoints keep parameters and optimizer state in two tensor files,
 * params.nbla and optim.nbla (nabla-train/src/checkpoint.rs:34-105), in the format of
 * save_tensors / load_tensors (nabla-ml/src/module/core.rs:21,66-120): "NBLA", u32 count,
 * per tensor u32 name length, UTF-8 name, u32 rows, u32 cols, rows*cols f64 values, all
 * little-endian; values pass through T::to_f64 / T::from_f64.  Device memory is streamed
 * through a bounded host buffer.  Synchronous. */

/* save_tensors over the tensors of `list` under `names[i]` (params.nbla from a module's
 * state_dict; for a mixed-precision optimizer pass a list of its f32 master weights). */
int nbo_nbla_save_list(const char *path, nbo_list *list, const char *const *names);
/* load_tensors + Module::load_state_dict (module/core.rs:281-304): every tensor of the
 * file must carry one of `names` ("unknown parameter key: k") and that tensor's shape
 * ("shape mismatch for 'k': expected (r, c), got (r, c)"); tensors of the list that the
 * file does not mention keep their values.  Nothing is written unless the file checks out. */
int nbo_nbla_load_list(const char *path, nbo_list *list, const char *const *names);
/* optim.nbla: OptimState::state_tensors (alg.rs:476-485, 553-562, 623-629) -- m0.., v0..
 * (Sgd: v0.. = velocity) -- written by save_tensors. */
int nbo_optim_save_state(nbo_optim *opt, const char *path);
/* load_tensors + OptimState::load_state_tensors (alg.rs:487-516, 564-593, 631-648):
 * "bad tensor key: k", "m index out of range: i", "missing m{i}" / "missing v{i}"; other
 * prefixes are ignored.  Nothing is written unless the whole file checks out. */
int nbo_optim_load_state(nbo_optim *opt, const char *path);
/* params.nbla of a mixed-precision optimizer (one created with keep_master): its f32 master
 * weights under names[i], in the place of the module's state_dict (checkpoint.rs:54-58) -- the
 * 16-bit parameters are derived from them and would not restore them.  nbo_optim_load_master is
 * load_tensors + Module::load_state_dict (module/core.rs:281-304) into the master weights, with
 * load_state_dict's errors plus "missing parameter key: k" (every master tensor must be in the
 * file); afterwards the master weights count as set, and nbo_optim_params_from_master gives the
 * 16-bit parameters.  Nothing is written unless the file checks out. */
int nbo_optim_save_master(nbo_optim *opt, const char *path, const char *const *names);
int nbo_optim_load_master(nbo_optim *opt, const char *path, const char *const *names);
/* The same for GroupOptimizer's OptimState (optim/groups.rs:320-350): group gi's tensors
 * carry the keys "g{gi}.m{i}" / "g{gi}.v{i}"; loading refuses any other key ("bad group tensor
 * key: k", "bad group index: x", "group index out of range: gi") and then applies each
 * group's own checks.  Nothing is written unless the whole file checks out. */
int nbo_optim_save_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path);
int nbo_optim_load_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path);
/* params.nbla of a module whose parameters are spread over a GroupOptimizer's groups
 * (checkpoint.rs:54-58, 88-90; optim/groups.rs:168-226): parameter i of the module, named
 * names[i], is tensor index_in_group[i] of group group_of[i]; params[g] lists group g's tensors
 * in the group's order.  What is written for a parameter is its group's f32 master weight if
 * the group keeps master weights, else the tensor itself.  Loading is load_tensors +
 * Module::load_state_dict (module/core.rs:281-304) with its errors ("unknown parameter key: k",
 * "shape mismatch for 'k': ...") plus "missing parameter key: k" for a parameter whose group
 * keeps master weights; nothing is written unless the whole file checks out, the master
 * weights then count as set, and nbo_optim_params_from_master per group gives the 16-bit
 * parameters. */
int nbo_optim_save_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                                 uint64_t n_params, const uint32_t *group_of, const uint32_t *index_in_group,
                                 const char *const *names, const char *path);
int nbo_optim_load_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                                 uint64_t n_params, const uint32_t *group_of, const uint32_t *index_in_group,
                                 const char *const *names, const char *path);

#pragma GCC visibility pop

#ifdef __cplusplus
}
#endif
#endif
