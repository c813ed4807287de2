/*
 * nabla_cpu_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the arithmetic that fumishiki/nabla's CPU backend performs on
 * the optimizer-step path (Sgd / Adam / AdamW step, GradScaler::unscale_and_update,
 * clip_grad_norm, zero_grad, bf16<->f32 casts, the xorshift64 + Box-Muller randn
 * input generator, lr_at_step).  It exists to CHECK the HIP engine; the shipped
 * library never links, loads or calls it.  Only tests, the smoke check and the
 * benchmark's cpu_baseline leg may use it.
 *
 * Every function cites the reference file:line it follows (paths relative to the
 * reference checkout).  The restatement keeps the reference's structure: each
 * Backend primitive is one whole-tensor pass producing one IEEE rounding per
 * element, and the optimizers are chains of those passes.
 *
 * Pinning status (what independent evidence fixes each function):
 *   - sgd / scaler / clip / zero_grad / lr_at_step: the reference's own known
 *     answers in nabla-train/tests/optim.rs and tests/trainer.rs (f64, 1x1), plus
 *     exact-rational brute force of every single rounding on tiny inputs.
 *   - adam / adamw: the reference tests only assert "param decreased"; pinned
 *     here by closed forms (step 1 from m=v=0 is sign-SGD; g==0 is pure decay;
 *     constant g gives geometric series for m and v), by exact-rational
 *     evaluation of each rounding, and by torch.optim at a few-ulp tolerance.
 *   - powf(x, 0.5): PARITY UNPINNED in the last ulp.  Rust's f32::powf lowers to
 *     llvm.pow.f32; whether the built reference calls libm powf or LLVM rewrites
 *     the constant-0.5 call into sqrt cannot be decided without compiling it.
 *     Both candidates are provided (ORC_POW_LIBM, ORC_POW_SQRT); they differ by
 *     at most 1 ulp of denom and never touch m or v.
 *   - f64::powi: restated as the compiler-rt/compiler-builtins __powidf2 loop;
 *     no reference test pins it (PARITY UNPINNED beyond the algorithm's text).
 *   - bf16 narrowing: arithmetic lives in the third-party crate `half` 2.7.1
 *     (Cargo.lock:418-421), not vendored in the reference; its published
 *     round-to-nearest-even algorithm is restated and cross-checked against
 *     torch's bf16 cast for all non-NaN inputs.  No reference test exercises
 *     bf16 (PARITY UNPINNED for NaN payloads).
 *   - T = bf16 instantiations (primitives, Sgd / Adam / AdamW, scaler, clip): the
 *     reference's tests never instantiate an optimizer at half::bf16.  Each operation
 *     is restated from scalar/mod.rs:253-351 (f32 operation, then bf16::from_f32) and
 *     the `half` crate's documented operators, and checked in exact arithmetic (round
 *     to 24 bits, then to 8) including the inner rounding of axpy and the two-step
 *     f64 -> bf16 cast.  PARITY UNPINNED against any output of the reference.
 *   - f16 conversions and the T = f16 instantiations: half::f16::from_f32 /
 *     f32::from(f16) are restated from the same crate's published algorithm and
 *     checked against IEEE binary16 as numpy's float16 implements it (every one of the
 *     65536 patterns widened; narrowing on random values, every tie and the subnormal
 *     and overflow boundaries); the pass chains are the same source as for bf16,
 *     checked in exact arithmetic (round to 24 bits, then to 11).  No reference test
 *     runs f16 on this path: PARITY UNPINNED for NaN payloads and against any output
 *     of the reference.
 *   - the benchmarks' LCG rand_tensor (benchmarks/src/lib.rs:7-22): exact arithmetic.
 */
#ifndef NABLA_CPU_ORACLE_H
#define NABLA_CPU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* denom = powf(v*ibc2, 0.5): which candidate lowering of f32::powf to follow. */
enum { ORC_POW_LIBM = 0, ORC_POW_SQRT = 1 };
void orc_set_pow_mode(int mode);
int orc_get_pow_mode(void);
/* Test hook, not part of the reference: norm >= 0 makes every clip_grad_norm decide and scale
 * with `norm` in the place of sqrt(its own serial sum); the return value stays its own norm.
 * A negative value switches the hook off. */
void orc_set_clip_norm_override(double norm);

/* Worker threads for the passes the reference runs under rayon par_iter
 * (nabla-core/src/cpu/mod.rs:44-64,211-223,264-272).  Passes the reference runs
 * serially (Tensor::map/from_fn, the scaler scan, the clip sum) stay serial. */
void orc_set_threads(int n);
int orc_get_threads(void);

/* f64::powi(a, n) -- alg.rs:122-123 via __powidf2 repeated squaring. */
double orc_powi(double a, int n);

/* half::bf16::from_f32 / f32::from(bf16) -- scalar/mod.rs:338-344. */
uint16_t orc_bf16_from_f32(float v);
float orc_bf16_to_f32(uint16_t h);
void orc_cast_bf16_to_f32(const uint16_t *src, float *dst, size_t n);
void orc_cast_f32_to_bf16(const float *src, uint16_t *dst, size_t n);

/* Tensor::randn(r, c, seed) as f64 values before T::from_f64 --
 * tensor/constructors.rs:14-41,206-223. */
void orc_randn_f64(double *out, size_t n, uint64_t seed);
void orc_randn_scaled_f32(float *out, size_t n, uint64_t seed, double sigma);
/* rand_tensor of the reference's benchmarks -- benchmarks/src/lib.rs:7-22.  *state is
 * the LCG state (42 at program start), advanced by n draws. */
void orc_bench_rand_f32(float *out, size_t n, uint64_t *state);

/* OptimMeta -- optim/core.rs:53-62.  kind: 0 AdamW, 1 Adam, 2 Sgd (enum order
 * of OptimKind, core.rs:46-51). */
typedef struct {
    int32_t kind;
    double lr, beta1, beta2, eps, weight_decay, momentum;
    uint64_t step_count;
} orc_meta;

/* GradScalerState -- optim/core.rs:326-332; defaults core.rs:336-344. */
typedef struct {
    double scale, growth_factor, backoff_factor;
    uint64_t growth_interval, consecutive_ok;
} orc_scaler_state;
void orc_scaler_default(orc_scaler_state *s);

/* LrSchedule / lr_at_step -- optim/core.rs:81-173.
 * kind: 0 Cosine{warmup,total,min_lr=a}, 1 Linear{warmup,total},
 *       2 OneCycle{max_lr=a,total,pct_start=b}, 3 Step{step_size=warmup,gamma=a}. */
typedef struct {
    int32_t kind;
    uint64_t warmup_steps, total_steps;
    double a, b;
} orc_schedule;
double orc_lr_at_step(const orc_schedule *s, double base_lr, uint64_t step);

/* ---- per-dtype API: T = f32 and T = f64 ------------------------------------ */
#define ORC_DECLARE(SUF, T)                                                                 \
    /* Backend primitives, one pass each (cpu/mod.rs:211-223,264-272,181) */                \
    void orc_scale_##SUF(const T *a, T s, T *out, size_t n);                                \
    void orc_axpy_inplace_##SUF(T *y, T alpha, const T *x, size_t n);                       \
    void orc_emul_##SUF(const T *a, const T *b, T *out, size_t n);                          \
    void orc_ediv_##SUF(const T *a, const T *b, T *out, size_t n);                          \
    void orc_add_##SUF(const T *a, const T *b, T *out, size_t n);                           \
    void orc_powf_##SUF(const T *a, T p, T *out, size_t n);                                 \
    /* Tensor::map(|x| x + c) and map(|x| x * c): serial from_fn (cpu/mod.rs:142-154) */    \
    void orc_map_add_##SUF(const T *a, T c, T *out, size_t n);                              \
    void orc_map_mul_##SUF(const T *a, T c, T *out, size_t n);                              \
    /* Sgd::step alg.rs:382-416 */                                                          \
    void orc_sgd_step_##SUF(const orc_meta *meta, size_t nt, const uint64_t *sizes,         \
                            T **params, T *const *grads, T **velocity);                     \
    /* Adam::step alg.rs:254-291 and AdamW::step alg.rs:109-150 (meta->kind selects);       \
     * increments meta->step_count exactly as the reference does. */                        \
    void orc_adam_step_##SUF(orc_meta *meta, size_t nt, const uint64_t *sizes, T **params,  \
                             T *const *grads, T **m, T **v);                                \
    /* adamw_step free function alg.rs:431-469 (one tensor, step passed in). */             \
    void orc_adamw_step_single_##SUF(T *param, const T *grad, T *m, T *v, size_t n,         \
                                     double lr, double beta1, double beta2, double eps,     \
                                     double weight_decay, uint64_t step);                   \
    /* GradScaler::unscale_and_update core.rs:351-388; returns 1 for ok, 0 for inf/nan. */  \
    int orc_scaler_unscale_and_update_##SUF(orc_scaler_state *s, size_t nt,                 \
                                            const uint64_t *sizes, T **grads);              \
    /* clip_grad_norm trainer.rs:500-523; returns the pre-clip norm. */                     \
    double orc_clip_grad_norm_##SUF(size_t nt, const uint64_t *sizes, T **grads,            \
                                    double max_norm);                                       \
    /* zero_grad autograd/ops.rs:1668-1673, trainer.rs:285-290 */                           \
    void orc_zero_grad_##SUF(size_t nt, const uint64_t *sizes, T **grads);                  \
    /* scale_grad autograd/ops.rs:1675-1680: g = &g * factor (B::scale) */                  \
    void orc_scale_grad_##SUF(size_t nt, const uint64_t *sizes, T **grads, T factor);

ORC_DECLARE(f32, float)
ORC_DECLARE(f64, double)

/* T = half::bf16, values passed as their 16-bit patterns: every operation is the f32
 * operation followed by bf16::from_f32 (scalar/mod.rs:253-351); scalars are narrowed with
 * bf16::from_f64 = from_f32(v as f32).  The same functions as for f32 / f64. */
ORC_DECLARE(bf16, uint16_t)
uint16_t orc_bf16_from_f64(double v);
/* T = half::f16 likewise (IEEE binary16 patterns). */
ORC_DECLARE(f16, uint16_t)
uint16_t orc_f16_from_f32(float v);
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f16_from_f64(double v);
/* B::cast default, backend/mod.rs:157-160.  Types: 0 = f32, 1 = bf16, 2 = f64, 3 = f16. */
void orc_cast(const void *src, int src_type, void *dst, int dst_type, size_t n);

/*
 * One Trainer iteration tail for the mixed-precision configs, composed from the
 * primitives above in the Trainer's order (trainer.rs:216-291):
 *   g32 = cast(g_bf16); ok = scaler.unscale_and_update(g32); if !ok skip;
 *   clip_grad_norm(g32, max_norm); optimizer.step(master, g32);
 *   p_bf16 = cast(master); (grads re-zeroed by the caller if it wishes).
 * scaler may be NULL (no unscale), max_norm <= 0 disables clipping exactly as
 * trainer.rs:501-503.  Returns 1 if the step ran, 0 if it was skipped;
 * *norm_out receives clip_grad_norm's return value (0 if skipped / disabled).
 */
int orc_mixed_step(orc_meta *meta, orc_scaler_state *scaler, double max_norm, size_t nt,
                   const uint64_t *sizes, uint16_t **params_bf16, uint16_t *const *grads_bf16,
                   float **master, float **m, float **v, double *norm_out);

/* The same composition for f16 tensors over f32 state: half_type 1 = bf16, 3 = f16. */
int orc_mixed_step_half(orc_meta *meta, orc_scaler_state *scaler, double max_norm, size_t nt,
                        const uint64_t *sizes, uint16_t **params_h, uint16_t *const *grads_h, int half_type,
                        float **master, float **m, float **v, double *norm_out);

/* Same tail for T = f32 throughout (params are the f32 tensors themselves);
 * grads are modified in place like the reference does. */
int orc_f32_step(orc_meta *meta, orc_scaler_state *scaler, double max_norm, size_t nt,
                 const uint64_t *sizes, float **params, float **grads, float **m, float **v,
                 double *norm_out);

#ifdef __cplusplus
}
#endif
#endif
