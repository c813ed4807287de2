/*
 * nabla_cpu_oracle.c -- TEST INFRASTRUCTURE ONLY (see nabla_cpu_oracle.h).
 *
 * CPU restatement of nabla's CPU-backend arithmetic on the optimizer-step path.
 * Build with: gcc -O2 -ffp-contract=off -fno-fast-math -fopenmp (oracle/Makefile).
 */
#define _GNU_SOURCE
#include "nabla_cpu_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static int g_pow_mode = ORC_POW_LIBM;
static int g_threads = 1;
/* Test hook: with a value >= 0, clip_grad_norm takes this as the norm instead of the square root
 * of its own serial sum (which it still computes, and still returns).  The device adds the
 * squares in a tree, so its norm can differ from the serial one in the last bits of the f64, and
 * once in some thousand steps that changes the f32 clip factor; a parity test then repeats the
 * oracle's step with the device's norm and still demands equal bits. */
static double g_norm_override = -1.0;
/* Below this many elements a pass is not worth forking threads for; the result
 * does not depend on it (every pass is element-wise). */
#define PAR_MIN 32768L

void orc_set_pow_mode(int mode) { g_pow_mode = mode == ORC_POW_SQRT ? ORC_POW_SQRT : ORC_POW_LIBM; }
int orc_get_pow_mode(void) { return g_pow_mode; }
void orc_set_clip_norm_override(double norm) { g_norm_override = norm; }
void orc_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int orc_get_threads(void) { return g_threads; }

/* f64::powi(n) (alg.rs:122-123, core.rs:170) lowers to llvm.powi.f64.i32, i.e. the
 * __powidf2 routine of compiler-rt / Rust's compiler-builtins: square-and-multiply
 * from the low bit, reciprocal at the end for negative exponents. */
double orc_powi(double a, int n)
{
    int recip = n < 0;
    unsigned int b = recip ? 0u - (unsigned int)n : (unsigned int)n;
    double r = 1.0;
    for (;;) {
        if (b & 1u) r *= a;
        b >>= 1;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0 / r : r;
}

/* half::bf16::from_f32 (crate half 2.7.1, called from scalar/mod.rs:338-340):
 * NaN keeps its top payload bits and gets the quiet bit; otherwise round to
 * nearest even on the 16 dropped bits. */
uint16_t orc_bf16_from_f32(float v)
{
    uint32_t x;
    memcpy(&x, &v, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    uint32_t round_bit = 0x00008000u;
    if ((x & round_bit) != 0 && (x & (3u * round_bit - 1u)) != 0) return (uint16_t)((x >> 16) + 1u);
    return (uint16_t)(x >> 16);
}

/* f32::from(bf16) (scalar/mod.rs:342-344): the 16 bits become the high half. */
float orc_bf16_to_f32(uint16_t h)
{
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* half::f16::from_f32 (crate half 2.7.1, software path `f32_to_f16_fallback`; the F16C
 * instruction it uses where the CPU has it gives the same bits): IEEE binary16, round to
 * nearest even, subnormals kept, overflow to infinity; NaN keeps its top ten payload
 * bits and gets the quiet bit. */
uint16_t orc_f16_from_f32(float v)
{
    uint32_t x;
    memcpy(&x, &v, 4);
    uint32_t sign = x & 0x80000000u, exp = x & 0x7F800000u, man = x & 0x007FFFFFu;
    if (exp == 0x7F800000u) {
        uint32_t nan_bit = man == 0 ? 0u : 0x0200u;
        return (uint16_t)((sign >> 16) | 0x7C00u | nan_bit | (man >> 13));
    }
    uint32_t half_sign = sign >> 16;
    int32_t half_exp = (int32_t)(exp >> 23) - 127 + 15;
    if (half_exp >= 0x1F) return (uint16_t)(half_sign | 0x7C00u);
    if (half_exp <= 0) {
        if (14 - half_exp > 24) return (uint16_t)half_sign; /* too small: signed zero */
        man |= 0x00800000u;
        uint32_t half_man = man >> (14 - half_exp);
        uint32_t round_bit = 1u << (13 - half_exp);
        if ((man & round_bit) != 0 && (man & (3u * round_bit - 1u)) != 0) half_man += 1;
        return (uint16_t)(half_sign | half_man);
    }
    uint32_t bits = half_sign | ((uint32_t)half_exp << 10) | (man >> 13);
    uint32_t round_bit = 0x00001000u;
    if ((man & round_bit) != 0 && (man & (3u * round_bit - 1u)) != 0) bits += 1; /* may carry into the exponent */
    return (uint16_t)bits;
}

/* f32::from(f16) (software path `f16_to_f32_fallback`): exact. */
float orc_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x03FFu, x;
    float f;
    if (exp == 0x1Fu) {
        x = sign | 0x7F800000u | (man ? (0x00400000u | (man << 13)) : 0u);
    } else if (exp == 0) {
        f = ldexpf((float)man, -24); /* subnormal or zero: man * 2^-24, exact */
        memcpy(&x, &f, 4);
        x |= sign;
    } else {
        x = sign | ((exp + 112u) << 23) | (man << 13);
    }
    memcpy(&f, &x, 4);
    return f;
}

/* Tensor::cast (tensor/shape.rs:489-493) -> default B::cast
 * (backend/mod.rs:157-160): U::from_f64(get().to_f64()), serial from_fn. */
void orc_cast_bf16_to_f32(const uint16_t *src, float *dst, size_t n)
{
    size_t i;
    for (i = 0; i < n; i++) dst[i] = (float)(double)orc_bf16_to_f32(src[i]);
}

void orc_cast_f32_to_bf16(const float *src, uint16_t *dst, size_t n)
{
    size_t i;
    for (i = 0; i < n; i++) dst[i] = orc_bf16_from_f32((float)(double)src[i]);
}

/* XorShift64 + Box-Muller -- tensor/constructors.rs:14-41,206-223. */
void orc_randn_f64(double *out, size_t n, uint64_t seed)
{
    uint64_t s = seed == 0 ? 0x123456789ABCDEF0ull : seed;
    size_t i = 0;
    while (i < n) {
        double u1, u2, r, theta;
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        u1 = (double)s / (double)UINT64_MAX;
        if (!(u1 > 1e-300)) u1 = 1e-300; /* f64::max(1e-300) */
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        u2 = (double)s / (double)UINT64_MAX;
        r = sqrt(-2.0 * log(u1));
        theta = 2.0 * 3.14159265358979323846264338327950288 * u2;
        out[i] = r * cos(theta);
        if (i + 1 < n) out[i + 1] = r * sin(theta);
        i += 2;
    }
}

/* rand_tensor of the reference's benchmarks (benchmarks/src/lib.rs:7-22): a 64-bit LCG
 * (Knuth's MMIX constants) whose top 31 bits, over 2^31, minus one become the value
 * (so it lies in [-1, 0)).  *state is the
 * thread-local SEED, 42 at program start. */
void orc_bench_rand_f32(float *out, size_t n, uint64_t *state)
{
    uint64_t x = *state;
    size_t i;
    for (i = 0; i < n; i++) {
        x = x * 6364136223846793005ull + 1442695040888963407ull;
        out[i] = (float)(x >> 33) / (float)(1ull << 31) - 1.0f;
    }
    *state = x;
}

void orc_randn_scaled_f32(float *out, size_t n, uint64_t seed, double sigma)
{
    double *tmp = (double *)malloc((n ? n : 1) * sizeof(double));
    size_t i;
    if (!tmp) abort();
    orc_randn_f64(tmp, n, seed);
    for (i = 0; i < n; i++) out[i] = (float)(tmp[i] * sigma);
    free(tmp);
}

void orc_scaler_default(orc_scaler_state *s) /* core.rs:336-344 */
{
    s->scale = 65536.0;
    s->growth_factor = 2.0;
    s->backoff_factor = 0.5;
    s->growth_interval = 2000;
    s->consecutive_ok = 0;
}

/* lr_at_step and helpers -- optim/core.rs:81-173 */
static double warmup_lr(double base_lr, uint64_t step, uint64_t warmup_steps)
{
    uint64_t w = warmup_steps > 1 ? warmup_steps : 1;
    return base_lr * (double)step / (double)w;
}

static double decay_progress(uint64_t step, uint64_t start, uint64_t total)
{
    uint64_t d = total - start; /* usize subtraction, as written */
    if (d < 1) d = 1;
    return (double)(step - start) / (double)d;
}

/* Rust's `x as usize` (core.rs:161): truncation toward zero, saturating, NaN -> 0 */
static uint64_t f64_as_usize(double x)
{
    if (!(x > 0.0)) return 0;
    if (x >= 18446744073709551616.0) return UINT64_MAX;
    return (uint64_t)x;
}

static double cosine_decay(double high, double low, double progress)
{
    return low + 0.5 * (high - low) * (1.0 + cos(3.14159265358979323846264338327950288 * progress));
}

double orc_lr_at_step(const orc_schedule *s, double base_lr, uint64_t step)
{
    switch (s->kind) {
    case 0: /* Cosine :132-143 */
        if (step < s->warmup_steps) return warmup_lr(base_lr, step, s->warmup_steps);
        return cosine_decay(base_lr, s->a, decay_progress(step, s->warmup_steps, s->total_steps));
    case 1: { /* Linear :144-154 */
        if (step < s->warmup_steps) return warmup_lr(base_lr, step, s->warmup_steps);
        double p = 1.0 - decay_progress(step, s->warmup_steps, s->total_steps);
        return base_lr * (p > 0.0 ? p : 0.0);
    }
    case 2: { /* OneCycle :155-167 */
        uint64_t up = f64_as_usize((double)s->total_steps * s->b);
        if (step < up) {
            uint64_t t = up > 1 ? up : 1;
            return base_lr + (s->a - base_lr) * (double)step / (double)t;
        }
        return cosine_decay(s->a, base_lr, decay_progress(step, up, s->total_steps));
    }
    default: { /* Step :168-171 */
        uint64_t sz = s->warmup_steps > 1 ? s->warmup_steps : 1;
        return base_lr * orc_powi(s->a, (int32_t)(uint32_t)(step / sz)); /* `k as i32`: low 32 bits */
    }
    }
}

#define T float
#define FN(x) x##_f32
#define POW_T powf
#define SQRT_T sqrtf
#define FABS_T fabsf
#define FROM_F64(x) ((float)(x))
#define TO_F64(x) ((double)(x))
#define NEG_T(x) (-(x))
#define SUB_T(a, b) ((a) - (b))
#include "oracle_impl.inc"
#undef T
#undef FN
#undef POW_T
#undef SQRT_T
#undef FABS_T
#undef FROM_F64
#undef TO_F64
#undef NEG_T
#undef SUB_T

#define T double
#define FN(x) x##_f64
#define POW_T pow
#define SQRT_T sqrt
#define FABS_T fabs
#define FROM_F64(x) ((double)(x))
#define TO_F64(x) ((double)(x))
#define NEG_T(x) (-(x))
#define SUB_T(a, b) ((a) - (b))
#include "oracle_impl.inc"
#undef T
#undef FN
#undef POW_T
#undef SQRT_T
#undef FABS_T
#undef FROM_F64
#undef TO_F64
#undef NEG_T
#undef SUB_T

/* ---- T = half::bf16 and T = half::f16 (oracle_half.inc) ---------------------------------- */
uint16_t orc_bf16_from_f64(double v) { return orc_bf16_from_f32((float)v); } /* scalar/mod.rs:338-340 */
uint16_t orc_f16_from_f64(double v) { return orc_f16_from_f32((float)v); }

static float pow_f32_mode(float x, float p)
{
    if (g_pow_mode == ORC_POW_SQRT && p == 0.5f) {
        float r = fabsf(sqrtf(x));
        return x == -INFINITY ? INFINITY : r;
    }
    return powf(x, p);
}

#define HFN(x) x##_bf16
#define H_TO_F32(h) orc_bf16_to_f32(h)
#define H_FROM_F32(f) orc_bf16_from_f32(f)
#include "oracle_half.inc"
#undef HFN
#undef H_TO_F32
#undef H_FROM_F32

#define HFN(x) x##_f16
#define H_TO_F32(h) orc_f16_to_f32(h)
#define H_FROM_F32(f) orc_f16_from_f32(f)
#include "oracle_half.inc"
#undef HFN
#undef H_TO_F32
#undef H_FROM_F32

/* B::cast default (backend/mod.rs:157-160): U::from_f64(x.to_f64()) per element.
 * Types: 0 = f32, 1 = bf16, 2 = f64, 3 = f16. */
void orc_cast(const void *src, int src_type, void *dst, int dst_type, size_t n)
{
    size_t i;
    for (i = 0; i < n; i++) {
        double v = src_type == 0   ? (double)((const float *)src)[i]
                   : src_type == 1 ? (double)orc_bf16_to_f32(((const uint16_t *)src)[i])
                   : src_type == 3 ? (double)orc_f16_to_f32(((const uint16_t *)src)[i])
                                   : ((const double *)src)[i];
        if (dst_type == 0) ((float *)dst)[i] = (float)v;
        else if (dst_type == 1) ((uint16_t *)dst)[i] = orc_bf16_from_f64(v);
        else if (dst_type == 3) ((uint16_t *)dst)[i] = orc_f16_from_f64(v);
        else ((double *)dst)[i] = v;
    }
}

int orc_f32_step(orc_meta *meta, orc_scaler_state *scaler, double max_norm, size_t nt,
                 const uint64_t *sizes, float **params, float **grads, float **m, float **v,
                 double *norm_out)
{
    if (norm_out) *norm_out = 0.0;
    if (scaler) { /* trainer.rs:230-237 */
        int ok = orc_scaler_unscale_and_update_f32(scaler, nt, sizes, grads);
        if (!ok) return 0;
    }
    double norm = orc_clip_grad_norm_f32(nt, sizes, grads, max_norm); /* :274-278 */
    if (norm_out) *norm_out = norm;
    if (meta->kind == 2) /* :279-283 */
        orc_sgd_step_f32(meta, nt, sizes, params, grads, m);
    else
        orc_adam_step_f32(meta, nt, sizes, params, grads, m, v);
    return 1;
}

/* half_type: 1 = bf16, 3 = f16 (the type codes of orc_cast) */
int orc_mixed_step_half(orc_meta *meta, orc_scaler_state *scaler, double max_norm, size_t nt,
                        const uint64_t *sizes, uint16_t **params_h, uint16_t *const *grads_h, int half_type,
                        float **master, float **m, float **v, double *norm_out)
{
    size_t i;
    float **g32 = (float **)malloc((nt ? nt : 1) * sizeof(float *));
    if (!g32) abort();
    for (i = 0; i < nt; i++) { /* g32 = g_half.cast::<f32>() */
        g32[i] = alloc_f32((size_t)sizes[i]);
        orc_cast(grads_h[i], half_type, g32[i], 0, (size_t)sizes[i]);
    }
    int ran = orc_f32_step(meta, scaler, max_norm, nt, sizes, master, g32, m, v, norm_out);
    if (ran)
        for (i = 0; i < nt; i++) /* p_half = master.cast::<half>() */
            orc_cast(master[i], 0, params_h[i], half_type, (size_t)sizes[i]);
    for (i = 0; i < nt; i++) free(g32[i]);
    free(g32);
    return ran;
}

int orc_mixed_step(orc_meta *meta, orc_scaler_state *scaler, double max_norm, size_t nt,
                   const uint64_t *sizes, uint16_t **params_bf16, uint16_t *const *grads_bf16,
                   float **master, float **m, float **v, double *norm_out)
{
    return orc_mixed_step_half(meta, scaler, max_norm, nt, sizes, params_bf16, grads_bf16, 1, master, m, v,
                               norm_out);
}
