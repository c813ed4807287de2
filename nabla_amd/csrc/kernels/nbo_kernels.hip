// gfx950 (CDNA4) device code for the fused optimizer-step engine.
//
// Built device-only into a code object that the host runtime loads with
// hipModuleLoadData and launches with hipModuleLaunchKernel; every kernel takes
// one by-value argument block from nbo_device_types.h.
//
// What is computed (reference = fumishiki/nabla, CPU backend):
//   nbo_update_*    Sgd::step / Adam::step / AdamW::step   nabla-train/src/optim/alg.rs:382-416, 254-291, 109-150
//   nbo_norm_*      finite scan of GradScaler::unscale_and_update (optim/core.rs:357-368)
//                   + sum of squares of clip_grad_norm (trainer.rs:504-513), first stage
//   nbo_finalize    second stage, scaler update (core.rs:369-385), clip decision
//                   (trainer.rs:514-517) and the per-step scalars (alg.rs:120-135)
//   nbo_scale_*     the in-place gradient rescale / zero of core.rs:372-380,
//                   trainer.rs:518-520, autograd/ops.rs:1668-1680
//   nbo_cast_*      bf16 / f16 <-> f32 casts (common/scalar/mod.rs:338-344), casts between lists
//   nbo_ew_*        the Backend primitives as single passes (nabla-core/src/cpu/mod.rs:211-272)
//   nbo_accum_*     gradient accumulation buf += g (trainer.rs:253-267)
//   nbo_accnorm_*   a whole micro-batch of the accumulating Trainer in one pass: finite scan,
//                   unscale, accumulate, first stage of the buffer's sum of squares (trainer.rs:230-267);
//                   nbo_accscale_* the same without the sum, nbo_sum_partials between the first
//                   stage's per-piece sums and the second stage
//
// Numerics contract: every arithmetic operation of the reference is one IEEE
// round-to-nearest operation here, in the same order, never contracted into an
// FMA (the file is compiled with -ffp-contract=off and carries the pragma
// below); division and square root are the correctly rounded ones.  The one
// deliberate difference is denom: the reference calls powf(x, 0.5), this code
// takes sqrt(x), which is within 1 ulp of any faithful powf.
//
// Memory access: the path is HBM-bound (about 0.5 flop per byte), so the
// kernels are organised around 128-bit per-lane accesses that are contiguous
// across the 64 lanes of a wavefront (1 KiB per wave per instruction), all
// loads of a chunk issued before the first use, and streaming (non-temporal)
// hints on data that is not touched again until the next step.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../nbo_device_types.h"

#pragma clang fp contract(off)

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
// the same 128 bits at an address that is only element-aligned (global memory takes such
// accesses in one instruction; the type keeps the compiler from assuming more)
typedef float f32x4_e __attribute__((ext_vector_type(4), aligned(4)));
typedef double f64x2_e __attribute__((ext_vector_type(2), aligned(8)));
typedef uint32_t u32x2_e __attribute__((ext_vector_type(2), aligned(2)));

#define DEV static __device__ __forceinline__
#define MEMBER __device__ __forceinline__

// Tuning knobs (the defaults are the measured best on MI355X).
#ifndef NBO_UNROLL
#define NBO_UNROLL 8 // 128-bit rows per thread whose loads are issued back to back (f32;
                     // half as many for f64, whose vectors hold half the elements)
#endif
#ifndef NBO_NT_LOADS
#define NBO_NT_LOADS 1
#endif
#ifndef NBO_NT_STORES
#define NBO_NT_STORES 1
#endif
#if NBO_NT_LOADS
#define NBO_LOAD(p) __builtin_nontemporal_load(p)
#else
#define NBO_LOAD(p) (*(p))
#endif
#if NBO_NT_STORES
#define NBO_STORE(v, p) __builtin_nontemporal_store(v, p)
#else
#define NBO_STORE(v, p) (*(p) = (v))
#endif
// Caller tensor addresses arrive as integers; telling the compiler that they are
// global memory turns flat_* accesses into global_* ones.
#define GLOBAL_PTR(type, p) ((__attribute__((address_space(1))) type *)(uintptr_t)(p))

// Number of the workgroup in a launch whose grid the host may have folded into two dimensions
// (one dimension holds fewer than 2^32 threads, i.e. 2^24 workgroups; the passes that run one
// workgroup per row of a chunk can need more).  The last row of the grid may be partly unused:
// such kernels compare the number with the count of workgroups they have work for.
DEV uint32_t folded_workgroup() { return blockIdx.y * gridDim.x + blockIdx.x; }

// ---------------------------------------------------------------------------------
// bf16 <-> f32, bit for bit what half::bf16 does (from_f32: NaN keeps its payload and
// gets the quiet bit, everything else rounds to nearest even).
DEV float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// gfx950 converts f32 to bf16 in hardware (v_cvt_pk_bf16_f32); the instruction gives
// half::bf16::from_f32's result for every one of the 2^32 inputs, NaN payloads included
// (the rule: `(x >> 16) | 0x40` for NaN, else `(x + 0x7FFF + ((x >> 16) & 1)) >> 16`).
DEV uint32_t f32_to_bf16_bits(float f) { return (uint32_t)__builtin_bit_cast(unsigned short, (__bf16)f); }

DEV bool nonfinite_f32(float f) { return (__float_as_uint(f) & 0x7F800000u) == 0x7F800000u; }
DEV bool nonfinite_f64(double d)
{
    return ((uint32_t)(__double_as_longlong(d) >> 32) & 0x7FF00000u) == 0x7FF00000u;
}

// f16: the device's conversion instructions (v_cvt_f16_f32 / v_cvt_f32_f16) give
// half::f16::from_f32's and f32::from(f16)'s bits for every input -- round to nearest even,
// subnormals kept, overflow to infinity, NaN payloads truncated with the quiet bit set.
DEV uint32_t f32_to_f16_bits(float f) { return (uint32_t)__builtin_bit_cast(unsigned short, (_Float16)f); }
DEV float f16_bits_to_f32(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (unsigned short)h); }

// T = half::bf16 / half::f16 as an arithmetic type: a 16-bit pattern whose every operation
// is the f32 operation followed by T::from_f32 (common/scalar/mod.rs:253-351 and the half
// crate's operators).  Conversion from float / double is T::from_f64 = from_f32(v as f32).
enum { FMT_BF16 = 0, FMT_F16 = 1 };
template <int FMT> struct Half16 {
    uint16_t bits;
    static __device__ __forceinline__ uint16_t narrow(float x)
    {
        return (uint16_t)(FMT == FMT_BF16 ? f32_to_bf16_bits(x) : f32_to_f16_bits(x));
    }
    __device__ __forceinline__ Half16() : bits(0) {}
    __device__ __forceinline__ Half16(float x) : bits(narrow(x)) {}
    __device__ __forceinline__ Half16(double x) : bits(narrow((float)x)) {}
    __device__ __forceinline__ Half16(int x) : bits(narrow((float)x)) {}
    __device__ __forceinline__ float f() const { return FMT == FMT_BF16 ? bf16_bits_to_f32(bits) : f16_bits_to_f32(bits); }
    __device__ __forceinline__ explicit operator double() const { return (double)f(); }
    // inf or NaN: all exponent bits set
    __device__ __forceinline__ bool nonfinite() const
    {
        return FMT == FMT_BF16 ? (bits & 0x7F80u) == 0x7F80u : (bits & 0x7C00u) == 0x7C00u;
    }
};
typedef Half16<FMT_BF16> BF;
typedef Half16<FMT_F16> HF;
template <int FMT> DEV Half16<FMT> operator*(Half16<FMT> a, Half16<FMT> b) { return Half16<FMT>(a.f() * b.f()); }
template <int FMT> DEV Half16<FMT> operator+(Half16<FMT> a, Half16<FMT> b) { return Half16<FMT>(a.f() + b.f()); }
template <int FMT> DEV Half16<FMT> operator-(Half16<FMT> a, Half16<FMT> b) { return Half16<FMT>(a.f() - b.f()); }
template <int FMT> DEV Half16<FMT> operator/(Half16<FMT> a, Half16<FMT> b) { return Half16<FMT>(a.f() / b.f()); }
template <int FMT> DEV Half16<FMT> half_from_bits(uint32_t b)
{
    Half16<FMT> r;
    r.bits = (uint16_t)b;
    return r;
}

// bf16 / bf16 and sqrt(bf16), rounded to f32 and then to bf16 as above, without the correctly
// rounded f32 operation (eleven and fourteen instructions; with them the all-bf16 Adam kernels
// were compute-bound: some 76 vector instructions per element for 12 bytes, 6.27 TB/s at most).
// Both operands have 8 significant bits, so a quotient is either exactly a bf16 rounding boundary
// (a 9-bit number) or at least 2^-17 of its size away from every one, and a square root is never
// on one and at least 2^-18 away: an approximation good to a few units of the f32's last place
// rounds to the same bf16, once a quotient that close to a boundary is taken to be on it.  The
// hardware's reciprocal and square root are such approximations unless the reciprocal is not a
// normal number, the quotient not finite or the square root's argument subnormal (the
// instructions flush those); then the exact operation is done.  That the results are the exact
// operations' bits has been checked for all 2^32 pairs and all 2^16 arguments
// (the kernel nbo_selftest_bf16_arith below).
enum { CLS_NAN = 0x003, CLS_INF = 0x204, CLS_DENORMAL = 0x090, CLS_ZERO = 0x060 };
DEV BF div_exact(BF a, BF b) { return BF(a.f() / b.f()); }
DEV BF sqrt_exact(BF x) { return BF(__builtin_sqrtf(x.f())); }
DEV BF operator/(BF a, BF b)
{
    const float x = a.f(), y = b.f();
    const float rc = __builtin_amdgcn_rcpf(y);
    const float q = x * rc;
    if (__builtin_expect(__builtin_amdgcn_classf(rc, CLS_NAN | CLS_INF | CLS_DENORMAL | CLS_ZERO) ||
                             __builtin_amdgcn_classf(q, CLS_NAN | CLS_INF),
                         0))
        return div_exact(a, b);
    // within 4 units of a multiple of 8 units (every rounding boundary is one): onto it
    return BF(__uint_as_float((__float_as_uint(q) + 4u) & ~7u));
}
DEV BF sqrt_fast(BF v)
{
    const float x = v.f();
    if (__builtin_expect(__builtin_amdgcn_classf(x, CLS_DENORMAL), 0)) return sqrt_exact(v);
    return BF(__builtin_amdgcn_sqrtf(x));
}

// f64::powi as compiler-rt's __powidf2 (alg.rs:122-123).
DEV double powi_f64(double a, int n)
{
    bool recip = n < 0;
    uint32_t b = recip ? 0u - (uint32_t)n : (uint32_t)n;
    double r = 1.0;
    for (;;) {
        if (b & 1u) r *= a;
        b >>= 1;
        if (b == 0) break;
        a *= a;
    }
    return recip ? 1.0 / r : r;
}

// ---------------------------------------------------------------------------------
// Storage access.  ST names the caller-tensor element type together with the arithmetic
// type T: NBO_F32 (float), NBO_F64 (double), NBO_BF16 / NBO_F16 (16-bit tensors, T = float:
// the f32-master composition), NBO_PBF16 / NBO_PF16 (16-bit tensors with T the same 16-bit
// type, every operation rounded to it).  One "vector" is VEC consecutive elements = 16 bytes
// of T.
template <int ST> struct Traits;
template <> struct Traits<NBO_F32> {
    typedef float T;
    enum { VEC = 4, SBYTES = 4 };
};
template <> struct Traits<NBO_BF16> {
    typedef float T;
    enum { VEC = 4, SBYTES = 2 };
};
template <> struct Traits<NBO_F64> {
    typedef double T;
    enum { VEC = 2, SBYTES = 8 };
};

template <> struct Traits<NBO_PBF16> {
    typedef BF T;
    enum { VEC = 8, SBYTES = 2 };
};
template <> struct Traits<NBO_F16> { // f16 tensors over f32 state
    typedef float T;
    enum { VEC = 4, SBYTES = 2 };
};
template <> struct Traits<NBO_PF16> { // f16 tensors, state and arithmetic
    typedef HF T;
    enum { VEC = 8, SBYTES = 2 };
};

// arena (engine-owned, always 16-byte aligned) vectors of T
DEV void ld_state(const float *p, float (&x)[4])
{
    f32x4 v = NBO_LOAD(GLOBAL_PTR(const f32x4, p));
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
}
DEV void ld_state(const double *p, double (&x)[2])
{
    f64x2 v = NBO_LOAD(GLOBAL_PTR(const f64x2, p));
    x[0] = v.x; x[1] = v.y;
}
DEV void st_state(float *p, const float (&x)[4])
{
    f32x4 v = {x[0], x[1], x[2], x[3]};
    NBO_STORE(v, GLOBAL_PTR(f32x4, p));
}
DEV void st_state(double *p, const double (&x)[2])
{
    f64x2 v = {x[0], x[1]};
    NBO_STORE(v, GLOBAL_PTR(f64x2, p));
}

// ... at an address that is a whole number of elements, but not of vectors, into the array
DEV void ld_state_e(const float *p, float (&x)[4])
{
    f32x4_e v = NBO_LOAD(GLOBAL_PTR(const f32x4_e, p));
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
}
DEV void ld_state_e(const double *p, double (&x)[2])
{
    f64x2_e v = NBO_LOAD(GLOBAL_PTR(const f64x2_e, p));
    x[0] = v.x; x[1] = v.y;
}
DEV void st_state_e(float *p, const float (&x)[4])
{
    f32x4_e v = {x[0], x[1], x[2], x[3]};
    NBO_STORE(v, GLOBAL_PTR(f32x4_e, p));
}
DEV void st_state_e(double *p, const double (&x)[2])
{
    f64x2_e v = {x[0], x[1]};
    NBO_STORE(v, GLOBAL_PTR(f64x2_e, p));
}

template <int FMT> DEV void ld_state(const Half16<FMT> *p, Half16<FMT> (&x)[8])
{
    const u32x4 v = NBO_LOAD(GLOBAL_PTR(const u32x4, p));
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        x[2 * k] = half_from_bits<FMT>(w[k] & 0xFFFFu);
        x[2 * k + 1] = half_from_bits<FMT>(w[k] >> 16);
    }
}
template <int FMT> DEV void st_state(Half16<FMT> *p, const Half16<FMT> (&x)[8])
{
    u32x4 v;
    v.x = (uint32_t)x[0].bits | ((uint32_t)x[1].bits << 16);
    v.y = (uint32_t)x[2].bits | ((uint32_t)x[3].bits << 16);
    v.z = (uint32_t)x[4].bits | ((uint32_t)x[5].bits << 16);
    v.w = (uint32_t)x[6].bits | ((uint32_t)x[7].bits << 16);
    NBO_STORE(v, GLOBAL_PTR(u32x4, p));
}

// 16-bit state is only ever accessed at vector alignment (see Peel)
template <int FMT> DEV void ld_state_e(const Half16<FMT> *p, Half16<FMT> (&x)[8]) { ld_state(p, x); }
template <int FMT> DEV void st_state_e(Half16<FMT> *p, const Half16<FMT> (&x)[8]) { st_state(p, x); }

// caller tensors: vector of VEC storage elements at byte address p
template <int ST> struct IO;
template <> struct IO<NBO_F32> {
    DEV void ldv(const char *p, float (&x)[4]) { ld_state((const float *)p, x); }
    DEV void stv(char *p, const float (&x)[4]) { st_state((float *)p, x); }
    DEV void ldv_e(const char *p, float (&x)[4]) { ld_state_e((const float *)p, x); }
    DEV void stv_e(char *p, const float (&x)[4]) { st_state_e((float *)p, x); }
    DEV float ld1(const char *p) { return *GLOBAL_PTR(const float, p); }
    DEV void st1(char *p, float x) { *GLOBAL_PTR(float, p) = x; }
};
template <> struct IO<NBO_F64> {
    DEV void ldv(const char *p, double (&x)[2]) { ld_state((const double *)p, x); }
    DEV void stv(char *p, const double (&x)[2]) { st_state((double *)p, x); }
    DEV void ldv_e(const char *p, double (&x)[2]) { ld_state_e((const double *)p, x); }
    DEV void stv_e(char *p, const double (&x)[2]) { st_state_e((double *)p, x); }
    DEV double ld1(const char *p) { return *GLOBAL_PTR(const double, p); }
    DEV void st1(char *p, double x) { *GLOBAL_PTR(double, p) = x; }
};
template <> struct IO<NBO_BF16> {
    DEV void widen(uint32_t lo, uint32_t hi, float (&x)[4])
    {
        x[0] = __uint_as_float(lo << 16);
        x[1] = __uint_as_float(lo & 0xFFFF0000u);
        x[2] = __uint_as_float(hi << 16);
        x[3] = __uint_as_float(hi & 0xFFFF0000u);
    }
    DEV void ldv(const char *p, float (&x)[4])
    {
        u32x2 v = NBO_LOAD(GLOBAL_PTR(const u32x2, p));
        widen(v.x, v.y, x);
    }
    DEV void stv(char *p, const float (&x)[4])
    {
        u32x2 v;
        v.x = f32_to_bf16_bits(x[0]) | (f32_to_bf16_bits(x[1]) << 16);
        v.y = f32_to_bf16_bits(x[2]) | (f32_to_bf16_bits(x[3]) << 16);
        NBO_STORE(v, GLOBAL_PTR(u32x2, p));
    }
    // ... at an address that is a whole number of elements, but not of vectors
    DEV void ldv_e(const char *p, float (&x)[4])
    {
        u32x2_e v = NBO_LOAD(GLOBAL_PTR(const u32x2_e, p));
        widen(v.x, v.y, x);
    }
    DEV void stv_e(char *p, const float (&x)[4])
    {
        u32x2_e v;
        v.x = f32_to_bf16_bits(x[0]) | (f32_to_bf16_bits(x[1]) << 16);
        v.y = f32_to_bf16_bits(x[2]) | (f32_to_bf16_bits(x[3]) << 16);
        NBO_STORE(v, GLOBAL_PTR(u32x2_e, p));
    }
    DEV float ld1(const char *p) { return bf16_bits_to_f32(*GLOBAL_PTR(const uint16_t, p)); }
    DEV void st1(char *p, float x) { *GLOBAL_PTR(uint16_t, p) = (uint16_t)f32_to_bf16_bits(x); }
};

template <int FMT> struct IOHalf16 {
    typedef Half16<FMT> H;
    DEV void ldv(const char *p, H (&x)[8]) { ld_state((const H *)p, x); }
    DEV void stv(char *p, const H (&x)[8]) { st_state((H *)p, x); }
    DEV void ldv_e(const char *p, H (&x)[8]) { ld_state((const H *)p, x); } // (only ever at vector alignment)
    DEV void stv_e(char *p, const H (&x)[8]) { st_state((H *)p, x); }
    DEV H ld1(const char *p) { return half_from_bits<FMT>(*GLOBAL_PTR(const uint16_t, p)); }
    DEV void st1(char *p, H x) { *GLOBAL_PTR(uint16_t, p) = x.bits; }
};
template <> struct IO<NBO_PBF16> : IOHalf16<FMT_BF16> {};
template <> struct IO<NBO_PF16> : IOHalf16<FMT_F16> {};
template <> struct IO<NBO_F16> {
    DEV void widen(uint32_t lo, uint32_t hi, float (&x)[4])
    {
        x[0] = f16_bits_to_f32(lo & 0xFFFFu);
        x[1] = f16_bits_to_f32(lo >> 16);
        x[2] = f16_bits_to_f32(hi & 0xFFFFu);
        x[3] = f16_bits_to_f32(hi >> 16);
    }
    DEV void ldv(const char *p, float (&x)[4])
    {
        u32x2 v = NBO_LOAD(GLOBAL_PTR(const u32x2, p));
        widen(v.x, v.y, x);
    }
    DEV void stv(char *p, const float (&x)[4])
    {
        u32x2 v;
        v.x = f32_to_f16_bits(x[0]) | (f32_to_f16_bits(x[1]) << 16);
        v.y = f32_to_f16_bits(x[2]) | (f32_to_f16_bits(x[3]) << 16);
        NBO_STORE(v, GLOBAL_PTR(u32x2, p));
    }
    DEV void ldv_e(const char *p, float (&x)[4])
    {
        u32x2_e v = NBO_LOAD(GLOBAL_PTR(const u32x2_e, p));
        widen(v.x, v.y, x);
    }
    DEV void stv_e(char *p, const float (&x)[4])
    {
        u32x2_e v;
        v.x = f32_to_f16_bits(x[0]) | (f32_to_f16_bits(x[1]) << 16);
        v.y = f32_to_f16_bits(x[2]) | (f32_to_f16_bits(x[3]) << 16);
        NBO_STORE(v, GLOBAL_PTR(u32x2_e, p));
    }
    DEV float ld1(const char *p) { return f16_bits_to_f32(*GLOBAL_PTR(const uint16_t, p)); }
    DEV void st1(char *p, float x) { *GLOBAL_PTR(uint16_t, p) = (uint16_t)f32_to_f16_bits(x); }
};

// ---------------------------------------------------------------------------------
// Per-step scalars in the arithmetic type T.
template <typename T> struct Scal;
template <> struct Scal<float> {
    float b1, omb1, b2, omb2, eps, ss, ibc2, omw, neg_lr, mom, wd, inv, clip;
    bool use_mom, use_wd;
    __device__ Scal(const NboOptimDev *o, const NboGradFactors *f)
        : b1(o->b1), omb1(o->omb1), b2(o->b2), omb2(o->omb2), eps(o->eps_t), ss(o->ss),
          ibc2(o->ibc2), omw(o->omw), neg_lr(o->neg_lr), mom(o->momentum_t), wd(o->wd_t),
          inv(f ? f->inv_scale32 : 1.0f), clip(f ? f->clip32 : 1.0f),
          use_mom(o->momentum != 0.0), use_wd(o->weight_decay != 0.0)
    {
    }
    // Sgd::step's own narrowing (alg.rs:393-397)
    __device__ Scal(double lr, double momentum, double weight_decay)
        : b1(0), omb1(0), b2(0), omb2(0), eps(0), ss(0), ibc2(0), omw(0), neg_lr(-(float)lr),
          mom((float)momentum), wd((float)weight_decay), inv(1.0f), clip(1.0f), use_mom(momentum != 0.0),
          use_wd(weight_decay != 0.0)
    {
    }
};
template <> struct Scal<double> {
    double b1, omb1, b2, omb2, eps, ss, ibc2, omw, neg_lr, mom, wd, inv, clip;
    bool use_mom, use_wd;
    __device__ Scal(const NboOptimDev *o, const NboGradFactors *f)
        : b1(o->d_b1), omb1(o->d_omb1), b2(o->d_b2), omb2(o->d_omb2), eps(o->d_eps),
          ss(o->d_ss), ibc2(o->d_ibc2), omw(o->d_omw), neg_lr(o->d_neg_lr), mom(o->d_momentum),
          wd(o->d_wd), inv(f ? f->inv_scale64 : 1.0), clip(f ? f->clip64 : 1.0),
          use_mom(o->momentum != 0.0), use_wd(o->weight_decay != 0.0)
    {
    }
    __device__ Scal(double lr, double momentum, double weight_decay)
        : b1(0), omb1(0), b2(0), omb2(0), eps(0), ss(0), ibc2(0), omw(0), neg_lr(-lr), mom(momentum),
          wd(weight_decay), inv(1.0), clip(1.0), use_mom(momentum != 0.0), use_wd(weight_decay != 0.0)
    {
    }
};

// T = bf16 / f16: T::from_f64(x) is from_f32(x as f32), so every scalar is the f32-narrowed
// one rounded once more; `T::one() - wd_lr` is a subtraction in T (alg.rs:135).
template <int FMT> struct Scal<Half16<FMT>> {
    typedef Half16<FMT> H;
    H b1, omb1, b2, omb2, eps, ss, ibc2, omw, neg_lr, mom, wd, inv, clip;
    bool use_mom, use_wd;
    __device__ Scal(const NboOptimDev *o, const NboGradFactors *f)
        : b1(o->b1), omb1(o->omb1), b2(o->b2), omb2(o->omb2), eps(o->eps_t), ss(o->ss), ibc2(o->ibc2),
          omw(H(1.0f) - H(o->wd_lr_t)), neg_lr(o->neg_lr), mom(o->momentum_t), wd(o->wd_t),
          inv(f ? f->inv_scale32 : 1.0f), clip(f ? f->clip32 : 1.0f), use_mom(o->momentum != 0.0),
          use_wd(o->weight_decay != 0.0)
    {
    }
    __device__ Scal(double lr, double momentum, double weight_decay)
        : b1(), omb1(), b2(), omb2(), eps(), ss(), ibc2(), omw(), neg_lr(-(float)lr), mom(momentum),
          wd(weight_decay), inv(1.0f), clip(1.0f), use_mom(momentum != 0.0), use_wd(weight_decay != 0.0)
    {
    }
};

template <int FMT> DEV Half16<FMT> sqrt_rn(Half16<FMT> x) { return Half16<FMT>(__builtin_sqrtf(x.f())); }
DEV BF sqrt_rn(BF x) { return sqrt_fast(x); }
DEV float sqrt_rn(float x) { return __builtin_sqrtf(x); }
DEV double sqrt_rn(double x) { return __builtin_sqrt(x); }

// One element of the update.  KIND: NBO_ADAMW, NBO_ADAM, NBO_SGD.
// Each statement is one rounding, in the order of the reference's pass chain.
template <typename T, int KIND> DEV void step_elem(T &p, T g, T &m, T &v, const Scal<T> &s)
{
    g = g * s.inv;  // core.rs:379   g.map(|x| x * inv_scale); exact identity when inv == 1
    g = g * s.clip; // trainer.rs:519 g.map(|x| x * scale_t);   exact identity when clip == 1
    if (KIND == NBO_SGD) {
        // alg.rs:399-414
        T ge = g;
        if (s.use_wd) {
            T pw = p * s.wd;
            ge = g + pw;
        }
        if (s.use_mom) {
            T vm = m * s.mom;
            m = vm + ge;
            ge = m;
        }
        T t = s.neg_lr * ge;
        p = p + t;
    } else {
        // alg.rs:138-148 / 281-289
        T m1 = m * s.b1;
        T t1 = s.omb1 * g;
        m = m1 + t1;
        T v1 = v * s.b2;
        T q = g * g;
        T t2 = s.omb2 * q;
        v = v1 + t2;
        T sc = v * s.ibc2;
        T r = sqrt_rn(sc); // reference: powf(sc, 0.5)
        T d = r + s.eps;
        T nn = m * s.ss;
        T u = nn / d;
        if (KIND == NBO_ADAMW) p = p * s.omw;
        T nu = (T)(-1) * u;
        p = p + nu;
    }
}

// ---------------------------------------------------------------------------------
// Chunk addressing shared by all multi-tensor kernels.
struct ChunkRef {
    uint32_t t;    // tensor index
    uint32_t cnt;  // elements of the chunk that exist (1..NBO_CHUNK)
    uint64_t base; // first element of the chunk within its tensor
    uint64_t soff; // tensor's element offset in the state arena
};

DEV ChunkRef chunk_ref(const NboLayoutDev &L, uint32_t c)
{
    ChunkRef r;
    r.t = L.chunk_tensor[c];
    r.base = (uint64_t)(c - L.chunk_begin[r.t]) * NBO_CHUNK;
    uint64_t rem = L.n[r.t] - r.base;
    r.cnt = rem < (uint64_t)NBO_CHUNK ? (uint32_t)rem : NBO_CHUNK;
    r.soff = L.soff ? L.soff[r.t] : 0;
    return r;
}

// Address of chunk c within state part `part` of the arena.
template <typename T> DEV T *state_part(const NboArenaDev &A, const ChunkRef &c, uint32_t part)
{
    return (T *)A.part[part] + c.soff + c.base;
}

// How a chunk of cnt elements is walked when the caller's tensors need not be vector-aligned:
// `head` single elements up to the first address at which every tensor involved is aligned to
// a whole vector of vbytes, then `nvec` whole vectors, then single elements for the rest.
// That works when all tensors are misaligned by the same whole number of elements (tensors
// packed back to back into flat parameter and gradient buffers are); otherwise, or when
// `whole_vectors_only` forbids a shifted start, every element goes singly (head = cnt).
struct Peel {
    uint32_t head, nvec;
};
DEV Peel peel(uint32_t cnt, uint32_t vec, uint32_t sb, bool whole_vectors_only, uintptr_t a0, uintptr_t a1,
              uintptr_t a2)
{
    const uint32_t vbytes = vec * sb;
    const uint32_t mis = (uint32_t)a0 & (vbytes - 1);
    Peel r = {cnt, 0};
    if ((((uint32_t)a1 & (vbytes - 1)) != mis) || (((uint32_t)a2 & (vbytes - 1)) != mis) || (mis % sb) != 0) return r;
    if (mis != 0 && whole_vectors_only) return r;
    const uint32_t head = mis ? (vbytes - mis) / sb : 0;
    if (head >= cnt) return r;
    r.head = head;
    r.nvec = (cnt - head) / vec;
    return r;
}
DEV Peel peel(uint32_t cnt, uint32_t vec, uint32_t sb, bool wvo, uintptr_t a0) { return peel(cnt, vec, sb, wvo, a0, a0, a0); }
DEV Peel peel(uint32_t cnt, uint32_t vec, uint32_t sb, bool wvo, uintptr_t a0, uintptr_t a1)
{
    return peel(cnt, vec, sb, wvo, a0, a1, a0);
}

DEV uint64_t prep_step(NboOptimDev *o, const NboHyper &h, const NboGradFactors *f, uint64_t step_count);
DEV void trace_step(NboTraceDev *t, uint64_t entries, const NboGradFactors *f, uint64_t step_count, double scale);

// A per-step scalar that every lane has computed alike, moved to a scalar register (the
// vector units do all f64 arithmetic; without this the scalars would occupy a vector register each).
DEV float uniform(float x) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(x))); }
DEV double uniform(double x)
{
    const uint64_t b = (uint64_t)__double_as_longlong(x);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b), hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    return __longlong_as_double((long long)(((uint64_t)hi << 32) | lo));
}
// ... for the scalars of a whole step (the fields Scal reads)
DEV void make_uniform(NboOptimDev &o)
{
    o.b1 = uniform(o.b1); o.omb1 = uniform(o.omb1); o.b2 = uniform(o.b2); o.omb2 = uniform(o.omb2);
    o.eps_t = uniform(o.eps_t); o.ss = uniform(o.ss); o.ibc2 = uniform(o.ibc2); o.omw = uniform(o.omw);
    o.neg_lr = uniform(o.neg_lr); o.momentum_t = uniform(o.momentum_t); o.wd_t = uniform(o.wd_t);
    o.wd_lr_t = uniform(o.wd_lr_t);
    o.d_b1 = uniform(o.d_b1); o.d_omb1 = uniform(o.d_omb1); o.d_b2 = uniform(o.d_b2); o.d_omb2 = uniform(o.d_omb2);
    o.d_eps = uniform(o.d_eps); o.d_ss = uniform(o.d_ss); o.d_ibc2 = uniform(o.d_ibc2); o.d_omw = uniform(o.d_omw);
    o.d_neg_lr = uniform(o.d_neg_lr); o.d_momentum = uniform(o.d_momentum); o.d_wd = uniform(o.d_wd);
}

// ---------------------------------------------------------------------------------
// Optimizer update: one workgroup per chunk.
//
// SELF: the launch prepares its own per-step scalars instead of reading what a launch before
// it left in a.opt.  Every workgroup derives them from a.opt->step_count, the hyper-parameters
// in the argument block and the decision in a.gf (the f64 prologue of alg.rs:120-135, some
// hundred operations).  step_count has to advance exactly once, and only after every
// workgroup has read it: each workgroup, once its read has returned, adds one to a counter in
// device memory, and the workgroup whose addition completes the grid -- nobody waits for
// anybody -- writes the advanced step_count and the trace entry and clears the counter.
//
// BY_ROW (the SGD kernels outside a grouped step, and the "_rows" kernels of the Adam kinds):
// one workgroup per row of a chunk -- every thread loads one vector of every stream, computes,
// stores and is done; the chunk's single elements (a ragged end, an unaligned start) go with
// its first row, and a row the chunk does not have ends at once.  With SGD's two or three
// streams that is 15-20 % faster than eight rows per workgroup (as it is for the element-wise
// passes, see stream_pieces).  The Adam kinds' five streams move the same bytes per second
// either way on the largest lists (0.3 % fewer by row on the 8B set) and 0.5-2 % more by row
// below some 4 G parameters (GPT-2-small f32 0.555 -> 0.543 ms, the 1.1 G mixed set 5.18 -> 5.14
// ms, f64 lists 2 %; measured in alternating launches inside one process): the host takes the
// "_rows" kernels for lists below NBO_ROWS_MAX_CHUNKS chunks.  16-bit state and arithmetic
// (four rows to a chunk as it is) is level or slower by row and has no such kernels.
template <int ST, int KIND, bool BY_ROW = false>
DEV void update_chunk(const NboUpdateArgs &a, const NboOptimDev *o, uint32_t wg)
{
    typedef typename Traits<ST>::T T;
    enum {
        VEC = Traits<ST>::VEC,
        SB = Traits<ST>::SBYTES,
        ROW = NBO_BLOCK * VEC,
        ROWS = NBO_CHUNK / ROW,
        UMAX = sizeof(T) == 8 ? NBO_UNROLL / 2 : NBO_UNROLL,
        U = ROWS < UMAX ? ROWS : UMAX,
        ITERS = ROWS / U
    };
    static_assert(ROWS % U == 0 && ROWS * ROW == NBO_CHUNK, "chunk must be a whole number of unrolled rows");
    const bool mixed = ST == NBO_BF16 || ST == NBO_F16; // f32 master lives in the arena
    const bool has_v = KIND != NBO_SGD;
    const uint32_t tid = threadIdx.x;
    uint32_t ci = wg, row0 = 0;
    if (BY_ROW) {
        if (a.L.row_map) { // a list of many small tensors: only the rows that exist were launched
            if (wg >= a.L.nrows) return; // (the unused end of a folded grid)
            const uint32_t e = a.L.row_map[wg];
            ci = e >> 4;
            row0 = e & 15u;
        } else {
            ci = wg / ROWS;
            row0 = wg % ROWS;
            if (ci >= a.L.nchunks) return;
        }
    }
    const ChunkRef c = chunk_ref(a.L, ci);

    char *pp = (char *)a.p_ptrs[c.t] + c.base * SB;
    char *pg = (char *)a.g_ptrs[c.t] + c.base * SB;
    T *am = state_part<T>(a.arena, c, 0);
    T *av = has_v ? state_part<T>(a.arena, c, a.arena.part_v) : nullptr;
    T *aw = mixed ? state_part<T>(a.arena, c, a.arena.part_w) : nullptr;
    const bool zero_g = (a.zero_grads & 1u) != 0;
    const uint32_t vbytes = VEC * SB;
    const bool vec_ok = ((((uintptr_t)pp) | ((uintptr_t)pg)) & (vbytes - 1)) == 0;

    const bool direct = KIND == NBO_SGD && a.direct != 0;
    // (by row: how the chunk is walked decides first whether this row exists at all)
    // 16-bit tensors over f32 state: the state moves six times the tensors' bytes, and the arena is
    // vector-aligned at every chunk's start -- so the state is accessed in whole aligned vectors
    // from the chunk's first element on, and it is the tensors that are read and written at element
    // alignment where they are not vector-aligned (packed back to back, or each misaligned
    // differently).  The 4096-tensor packed set: 0.123 -> 0.115 ms.
    const Peel whole = {0, c.cnt / VEC};
    const Peel pl = mixed ? whole : peel(c.cnt, VEC, SB, sizeof(T) < 4, (uintptr_t)pp, (uintptr_t)pg);
    if (BY_ROW && row0 != 0 && row0 * NBO_BLOCK >= pl.nvec) return;
    if (!direct && o->skip) {
        // found_inf: parameters, moments and step_count stay untouched
        // (trainer.rs:230-236); the gradients become zeros (core.rs:372-375) if the caller
        // asked for zeroing, after every step or after a skipped one only.
        if (a.zero_grads != 0 && row0 == 0)
            for (uint32_t i = tid; i < c.cnt; i += NBO_BLOCK) IO<ST>::st1(pg + (uint64_t)i * SB, (T)0);
        return;
    }
    const Scal<T> s = direct ? Scal<T>(a.sgd_lr, a.sgd_momentum, a.sgd_weight_decay) : Scal<T>(o, a.gf);
    const bool use_m = KIND != NBO_SGD || s.use_mom;

    if (!BY_ROW && c.cnt == NBO_CHUNK && vec_ok) {
        for (int it = 0; it < ITERS; it++) {
            // U rows of the workgroup at once.  The memory instructions are issued stream by
            // stream -- every row's gradient load, then every row's master load, ... and after
            // all rows are computed every row's master store, ... -- not row by row: the memory
            // then sees longer runs per stream, which measured 1.3 % faster on the 8B set (35.0
            // against 35.5 ms in alternating launches inside one process; loads or stores alone
            // in this order: next to nothing).
            const uint32_t e0 = it * (U * ROW) + tid * VEC;
            T g[U][VEC], p[U][VEC], m[U][VEC] = {}, v[U][VEC] = {};
#pragma unroll
            for (int u = 0; u < U; u++) IO<ST>::ldv(pg + (uint64_t)(e0 + u * ROW) * SB, g[u]);
#pragma unroll
            for (int u = 0; u < U; u++) {
                if (mixed) ld_state(aw + e0 + u * ROW, p[u]);
                else IO<ST>::ldv(pp + (uint64_t)(e0 + u * ROW) * SB, p[u]);
            }
            if (use_m) {
#pragma unroll
                for (int u = 0; u < U; u++) ld_state(am + e0 + u * ROW, m[u]);
            }
            if (has_v) {
#pragma unroll
                for (int u = 0; u < U; u++) ld_state(av + e0 + u * ROW, v[u]);
            }
#pragma unroll
            for (int u = 0; u < U; u++)
#pragma unroll
                for (int k = 0; k < VEC; k++) step_elem<T, KIND>(p[u][k], g[u][k], m[u][k], v[u][k], s);
            // the scheduling barriers keep the compiler from interleaving the stores with the
            // arithmetic again
            __builtin_amdgcn_sched_barrier(0);
            if (mixed) {
#pragma unroll
                for (int u = 0; u < U; u++) st_state(aw + e0 + u * ROW, p[u]);
            }
            if (use_m) {
#pragma unroll
                for (int u = 0; u < U; u++) st_state(am + e0 + u * ROW, m[u]);
            }
            if (has_v) {
#pragma unroll
                for (int u = 0; u < U; u++) st_state(av + e0 + u * ROW, v[u]);
            }
#pragma unroll
            for (int u = 0; u < U; u++) IO<ST>::stv(pp + (uint64_t)(e0 + u * ROW) * SB, p[u]);
            if (zero_g) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    T z[VEC] = {};
                    IO<ST>::stv(pg + (uint64_t)(e0 + u * ROW) * SB, z);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }

    // ragged chunk, or caller tensors that are not vector-aligned: single elements up to the
    // first vector-aligned address of the caller's tensors, whole vectors from there (the state
    // arrays are then read at element alignment, which needs 32- or 64-bit state), single
    // elements for the rest -- or, 16-bit tensors over f32 state, whole vectors from the start
    // (by row: the one vector of this row, if the chunk reaches that far)
    for (uint32_t q = BY_ROW ? row0 * NBO_BLOCK + tid : tid; q < pl.nvec; q += BY_ROW ? NBO_CHUNK : NBO_BLOCK) {
        const uint32_t e = pl.head + q * VEC;
        T g[VEC], p[VEC], m[VEC] = {}, v[VEC] = {};
        if (mixed) {
            IO<ST>::ldv_e(pg + (uint64_t)e * SB, g);
            ld_state(aw + e, p);
            if (use_m) ld_state(am + e, m);
            if (has_v) ld_state(av + e, v);
        } else {
            IO<ST>::ldv(pg + (uint64_t)e * SB, g);
            IO<ST>::ldv(pp + (uint64_t)e * SB, p);
            if (use_m) ld_state_e(am + e, m);
            if (has_v) ld_state_e(av + e, v);
        }
#pragma unroll
        for (int k = 0; k < VEC; k++) step_elem<T, KIND>(p[k], g[k], m[k], v[k], s);
        if (mixed) {
            st_state(aw + e, p);
            IO<ST>::stv_e(pp + (uint64_t)e * SB, p);
            if (use_m) st_state(am + e, m);
            if (has_v) st_state(av + e, v);
        } else {
            IO<ST>::stv(pp + (uint64_t)e * SB, p);
            if (use_m) st_state_e(am + e, m);
            if (has_v) st_state_e(av + e, v);
        }
        if (zero_g) {
            T z[VEC] = {};
            if (mixed) IO<ST>::stv_e(pg + (uint64_t)e * SB, z);
            else IO<ST>::stv(pg + (uint64_t)e * SB, z);
        }
    }
    // elements [0, head) and [head + nvec * VEC, cnt)
    if (BY_ROW && row0 != 0) return;
    const uint32_t n_single = c.cnt - pl.nvec * VEC;
    for (uint32_t i = tid; i < n_single; i += NBO_BLOCK) {
        const uint32_t e = i < pl.head ? i : i + pl.nvec * VEC;
        T g = IO<ST>::ld1(pg + (uint64_t)e * SB);
        T p = mixed ? aw[e] : IO<ST>::ld1(pp + (uint64_t)e * SB);
        T m = use_m ? am[e] : (T)0;
        T v = has_v ? av[e] : (T)0;
        step_elem<T, KIND>(p, g, m, v, s);
        if (mixed) aw[e] = p;
        IO<ST>::st1(pp + (uint64_t)e * SB, p);
        if (use_m) am[e] = m;
        if (has_v) av[e] = v;
        if (zero_g) IO<ST>::st1(pg + (uint64_t)e * SB, (T)0);
    }
}

// wg of nwg: the workgroup's number among those that work on a's lists (the whole grid, or
// one group's share of a grouped launch)
template <int ST, int KIND, bool SELF = false> DEV void update_body(const NboUpdateArgs &a, uint32_t wg, uint32_t nwg)
{
    if (!SELF) {
        update_chunk<ST, KIND, KIND == NBO_SGD>(a, a.opt, wg);
        return;
    }
    uint32_t sc_lo = (uint32_t)a.opt->step_count, sc_hi = (uint32_t)(a.opt->step_count >> 32);
    // the value is in registers -- the read has returned -- before anything below is issued
    asm volatile("" : "+v"(sc_lo), "+v"(sc_hi)::"memory");
    uint32_t readers_before = 0;
    if (threadIdx.x == 0)
        readers_before = __hip_atomic_fetch_add(&a.opt_rw->ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    NboOptimDev own = {};
    own.step_count = ((uint64_t)sc_hi << 32) | sc_lo;
    prep_step(&own, a.hyper, a.gf, own.step_count);
    make_uniform(own);
    update_chunk<ST, KIND>(a, &own, wg);
    // the counter's answer is not looked at before the chunk is done: it has long arrived then
    __builtin_amdgcn_sched_barrier(0);
    if (threadIdx.x == 0 && readers_before == nwg - 1) {
        a.opt_rw->step_count = own.step_count;
        if (a.trace) trace_step(a.trace, a.trace->count, a.gf, own.step_count, a.scaler ? a.scaler->scale : 0.0);
        __hip_atomic_store(&a.opt_rw->ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

#define NBO_UPDATE_KERNEL(name, ST, KIND)                                                   \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboUpdateArgs a) \
    {                                                                                       \
        update_body<ST, KIND>(a, KIND == NBO_SGD ? folded_workgroup() : blockIdx.x, gridDim.x); \
    }

NBO_UPDATE_KERNEL(nbo_update_f32_adamw, NBO_F32, NBO_ADAMW)
NBO_UPDATE_KERNEL(nbo_update_f32_adam, NBO_F32, NBO_ADAM)
NBO_UPDATE_KERNEL(nbo_update_f32_sgd, NBO_F32, NBO_SGD)
NBO_UPDATE_KERNEL(nbo_update_bf16_adamw, NBO_BF16, NBO_ADAMW)
NBO_UPDATE_KERNEL(nbo_update_bf16_adam, NBO_BF16, NBO_ADAM)
NBO_UPDATE_KERNEL(nbo_update_bf16_sgd, NBO_BF16, NBO_SGD)
NBO_UPDATE_KERNEL(nbo_update_f64_adamw, NBO_F64, NBO_ADAMW)
NBO_UPDATE_KERNEL(nbo_update_f64_adam, NBO_F64, NBO_ADAM)
NBO_UPDATE_KERNEL(nbo_update_f64_sgd, NBO_F64, NBO_SGD)
NBO_UPDATE_KERNEL(nbo_update_pbf16_adamw, NBO_PBF16, NBO_ADAMW)
NBO_UPDATE_KERNEL(nbo_update_pbf16_adam, NBO_PBF16, NBO_ADAM)
NBO_UPDATE_KERNEL(nbo_update_pbf16_sgd, NBO_PBF16, NBO_SGD)
NBO_UPDATE_KERNEL(nbo_update_f16_adamw, NBO_F16, NBO_ADAMW)
NBO_UPDATE_KERNEL(nbo_update_f16_adam, NBO_F16, NBO_ADAM)
NBO_UPDATE_KERNEL(nbo_update_f16_sgd, NBO_F16, NBO_SGD)
NBO_UPDATE_KERNEL(nbo_update_pf16_adamw, NBO_PF16, NBO_ADAMW)
NBO_UPDATE_KERNEL(nbo_update_pf16_adam, NBO_PF16, NBO_ADAM)
NBO_UPDATE_KERNEL(nbo_update_pf16_sgd, NBO_PF16, NBO_SGD)

// The Adam kinds one workgroup per row (see update_chunk), for 32- and 64-bit state; SGD's kernels
// above are by row already.
#define NBO_UPDATE_ROWS_KERNEL(name, ST, KIND)                                              \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboUpdateArgs a)     \
    {                                                                                       \
        update_chunk<ST, KIND, true>(a, a.opt, folded_workgroup());                         \
    }
NBO_UPDATE_ROWS_KERNEL(nbo_update_f32_adamw_rows, NBO_F32, NBO_ADAMW)
NBO_UPDATE_ROWS_KERNEL(nbo_update_f32_adam_rows, NBO_F32, NBO_ADAM)
NBO_UPDATE_ROWS_KERNEL(nbo_update_bf16_adamw_rows, NBO_BF16, NBO_ADAMW)
NBO_UPDATE_ROWS_KERNEL(nbo_update_bf16_adam_rows, NBO_BF16, NBO_ADAM)
NBO_UPDATE_ROWS_KERNEL(nbo_update_f64_adamw_rows, NBO_F64, NBO_ADAMW)
NBO_UPDATE_ROWS_KERNEL(nbo_update_f64_adam_rows, NBO_F64, NBO_ADAM)
NBO_UPDATE_ROWS_KERNEL(nbo_update_f16_adamw_rows, NBO_F16, NBO_ADAMW)
NBO_UPDATE_ROWS_KERNEL(nbo_update_f16_adam_rows, NBO_F16, NBO_ADAM)

// Launches that prepare their own scalars: the unfused Optimizer::step (one launch per call, as
// the reference's one call) and a grouped fused step, whose groups -- each with its own lists,
// state, hyper-parameters and step_count (optim/groups.rs:269-293) -- share ONE launch: the
// argument block carries up to NBO_GROUPS_PER_LAUNCH groups' arguments, and a workgroup first
// finds the group whose range of the grid it lies in.
#define NBO_UPDATE_SELF_KERNEL(name, ST, KIND)                                                    \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboGroupedUpdateArgs ga)   \
    {                                                                                             \
        uint32_t gi = 0;                                                                          \
        for (uint32_t k = 1; k < ga.n_groups; k++) gi = blockIdx.x >= ga.first_wg[k] ? k : gi;    \
        update_body<ST, KIND, true>(ga.g[gi], blockIdx.x - ga.first_wg[gi],                       \
                                    ga.first_wg[gi + 1] - ga.first_wg[gi]);                       \
    }
NBO_UPDATE_SELF_KERNEL(nbo_update_f32_adamw_self, NBO_F32, NBO_ADAMW)
NBO_UPDATE_SELF_KERNEL(nbo_update_f32_adam_self, NBO_F32, NBO_ADAM)
NBO_UPDATE_SELF_KERNEL(nbo_update_bf16_adamw_self, NBO_BF16, NBO_ADAMW)
NBO_UPDATE_SELF_KERNEL(nbo_update_bf16_adam_self, NBO_BF16, NBO_ADAM)
NBO_UPDATE_SELF_KERNEL(nbo_update_f64_adamw_self, NBO_F64, NBO_ADAMW)
NBO_UPDATE_SELF_KERNEL(nbo_update_f64_adam_self, NBO_F64, NBO_ADAM)
NBO_UPDATE_SELF_KERNEL(nbo_update_f16_adamw_self, NBO_F16, NBO_ADAMW)
NBO_UPDATE_SELF_KERNEL(nbo_update_f16_adam_self, NBO_F16, NBO_ADAM)
NBO_UPDATE_SELF_KERNEL(nbo_update_pbf16_adamw_self, NBO_PBF16, NBO_ADAMW)
NBO_UPDATE_SELF_KERNEL(nbo_update_pbf16_adam_self, NBO_PBF16, NBO_ADAM)
NBO_UPDATE_SELF_KERNEL(nbo_update_pf16_adamw_self, NBO_PF16, NBO_ADAMW)
NBO_UPDATE_SELF_KERNEL(nbo_update_pf16_adam_self, NBO_PF16, NBO_ADAM)
// SGD has no step_count; inside a grouped fused step its group still needs the skip decision and
// a trace entry
NBO_UPDATE_SELF_KERNEL(nbo_update_f32_sgd_self, NBO_F32, NBO_SGD)
NBO_UPDATE_SELF_KERNEL(nbo_update_bf16_sgd_self, NBO_BF16, NBO_SGD)
NBO_UPDATE_SELF_KERNEL(nbo_update_f64_sgd_self, NBO_F64, NBO_SGD)
NBO_UPDATE_SELF_KERNEL(nbo_update_f16_sgd_self, NBO_F16, NBO_SGD)
NBO_UPDATE_SELF_KERNEL(nbo_update_pbf16_sgd_self, NBO_PBF16, NBO_SGD)
NBO_UPDATE_SELF_KERNEL(nbo_update_pf16_sgd_self, NBO_PF16, NBO_SGD)

// ---------------------------------------------------------------------------------
// Deterministic block reduction: xor-butterfly inside each 64-lane wavefront, then
// the four wave results are added in wave order by thread 0.
DEV double block_sum(double x, double *lds)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x = x + __shfl_xor(x, off, 64);
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0) lds[wave] = x;
    __syncthreads();
    double r = 0.0;
    if (threadIdx.x == 0) {
        r = lds[0];
        for (uint32_t w = 1; w < NBO_BLOCK / 64; w++) r = r + lds[w];
    }
    __syncthreads();
    return r; // valid in thread 0
}

DEV uint32_t block_or(uint32_t x, uint32_t *lds)
{
    x = __any(x != 0) ? 1u : 0u; // wave-wide
    const uint32_t wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63u) == 0) lds[wave] = x;
    __syncthreads();
    uint32_t r = 0;
    if (threadIdx.x == 0)
        for (uint32_t w = 0; w < NBO_BLOCK / 64; w++) r |= lds[w];
    __syncthreads();
    return r;
}

// Per-step scalars (alg.rs:120-135 AdamW, 265-277 Adam, 393-395 Sgd).  A skipped
// step leaves step_count alone, because the reference never calls step() then.  step_count is
// o->step_count, which the caller has read (early, where it waits for other loads anyway);
// returns its value after the step.
DEV uint64_t prep_step(NboOptimDev *o, const NboHyper &h, const NboGradFactors *f, uint64_t step_count)
{
    o->lr = h.lr;
    o->beta1 = h.beta1;
    o->beta2 = h.beta2;
    o->eps = h.eps;
    o->weight_decay = h.weight_decay;
    o->momentum = h.momentum;
    o->kind = h.kind;
    if (f && f->found_inf) {
        o->skip = 1;
        return step_count;
    }
    o->skip = 0;
    if (o->kind == NBO_SGD) {
        const float lr_t = (float)o->lr;
        o->neg_lr = -lr_t;
        o->momentum_t = (float)o->momentum;
        o->wd_t = (float)o->weight_decay;
        o->d_neg_lr = -o->lr;
        o->d_momentum = o->momentum;
        o->d_wd = o->weight_decay;
        return step_count;
    }
    step_count += 1;
    o->step_count = step_count;
    const int step = (int)step_count;
    const double bc1 = 1.0 - powi_f64(o->beta1, step);
    const double bc2 = 1.0 - powi_f64(o->beta2, step);
    const double step_size = o->lr / bc1;
    const double omb1 = 1.0 - o->beta1;
    const double omb2 = 1.0 - o->beta2;
    const double wd_lr = o->weight_decay * o->lr;
    const double ibc2 = 1.0 / bc2;
    o->b1 = (float)o->beta1;
    o->omb1 = (float)omb1;
    o->b2 = (float)o->beta2;
    o->omb2 = (float)omb2;
    o->eps_t = (float)o->eps;
    o->ss = (float)step_size;
    o->ibc2 = (float)ibc2;
    const float wd_lr_t = (float)wd_lr;
    o->wd_lr_t = wd_lr_t;
    o->omw = 1.0f - wd_lr_t; // T::one() - wd_lr, in T (alg.rs:135)
    o->d_b1 = o->beta1;
    o->d_omb1 = omb1;
    o->d_b2 = o->beta2;
    o->d_omb2 = omb2;
    o->d_eps = o->eps;
    o->d_ss = step_size;
    o->d_ibc2 = ibc2;
    o->d_omw = 1.0 - wd_lr;
    return step_count;
}

// entries = t->count, read by the caller
DEV void trace_step(NboTraceDev *t, uint64_t entries, const NboGradFactors *f, uint64_t step_count, double scale)
{
    const uint64_t i = entries;
    NboTraceEntry e;
    e.scale = scale;
    e.norm = f ? f->norm : 0.0;
    e.step_count = step_count;
    e.found_inf = f ? f->found_inf : 0u;
    e.clipped = f ? f->clipped : 0u;
    t->e[i % NBO_TRACE_LEN] = e;
    t->count = i + 1;
}

extern "C" __global__ __launch_bounds__(64) void nbo_prep(const NboPrepArgs a)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const uint64_t entries = a.trace ? a.trace->count : 0;
    const uint64_t step_count = prep_step(a.opt, a.hyper, a.gf, a.opt->step_count);
    if (a.trace) trace_step(a.trace, entries, a.gf, step_count, a.scaler ? a.scaler->scale : 0.0);
}

// Second stage: reduce the per-block partials in a fixed order, then the scalar
// logic of GradScaler::unscale_and_update (core.rs:369-385) and clip_grad_norm
// (trainer.rs:501-517).  Run by one whole workgroup.  (Letting the norm pass's last workgroup
// do this instead of a launch of its own was tried and is slower: the device-wide ticket
// counter that finds the last workgroup costs the pass more than the launch it saves.)
DEV void finalize_body(const NboFinalizeArgs &a, double *lds_d, uint32_t *lds_u)
{
    const uint32_t tid = threadIdx.x;
    // Everything this kernel reads is asked for here, at once: a read takes about a microsecond
    // to come back, and one after the other -- partial sums, the word of a pass without them, the
    // scaler, the step count, the trace's length -- they were most of the kernel's five.
    enum { PER = NBO_NORM_GRID_MAX / NBO_BLOCK };
    static_assert(PER * NBO_BLOCK == NBO_NORM_GRID_MAX, "whole rounds of the workgroup");
    double part[PER];
    uint32_t flag[PER];
#pragma unroll
    for (int j = 0; j < PER; j++) {
        const uint32_t i = tid + j * NBO_BLOCK;
        part[j] = i < a.grid ? a.partial_sumsq[i] : 0.0;
        flag[j] = i < a.grid ? a.partial_flag[i] : 0u;
    }
    uint32_t word = 0;
    uint64_t step_count = 0, entries = 0;
    NboScalerDev s = {};
    if (tid == 0) {
        if (a.any_bad) word = *a.any_bad;
        if (a.scaler) s = *a.scaler;
        if (a.opt) step_count = a.opt->step_count;
        if (a.trace) entries = a.trace->count;
    }
    // (the sums are squares, never -0.0: adding the 0.0 of a slot that does not exist changes nothing)
    double acc = 0.0;
    uint32_t bad = 0;
#pragma unroll
    for (int j = 0; j < PER; j++) {
        acc = acc + part[j];
        bad |= flag[j];
    }
    const double reduced = block_sum(acc, lds_d);
    uint32_t any_bad = block_or(bad, lds_u);
    if (tid != 0) return;
    if (a.any_bad) { // what a pass without partial results found, and the word clean again for the next one
        any_bad |= word;
        *a.any_bad = 0;
    }

    NboGradFactors f;
    const double sumsq = a.use_sumsq_in ? a.sumsq_in : reduced;
    f.sumsq = sumsq;
    const bool found = a.check_finite && any_bad;
    double inv = 1.0;
    double scale_after = 0.0;
    if (a.scaler) {
        inv = 1.0 / s.scale; // core.rs:355, from the scale before its update
        if (found) {
            s.scale = s.scale * s.backoff_factor;
            s.consecutive_ok = 0;
        } else {
            s.consecutive_ok += 1;
            if (s.consecutive_ok >= s.growth_interval) {
                s.scale = s.scale * s.growth_factor;
                s.consecutive_ok = 0;
            }
        }
        *a.scaler = s;
        scale_after = s.scale;
    }
    f.inv_scale64 = inv;
    f.inv_scale32 = (float)inv;
    f.found_inf = found ? 1u : 0u;
    f.norm = 0.0;
    f.clip64 = 1.0;
    f.clip32 = 1.0f;
    f.clipped = 0;
    if (!found && a.max_norm > 0.0) {
        const double norm = __builtin_sqrt(sumsq);
        f.norm = norm;
        if (norm > a.max_norm && norm > 0.0) {
            const double c = a.max_norm / norm;
            f.clip64 = c;
            f.clip32 = (float)c;
            f.clipped = 1;
        }
    }
    *a.gf = f;
    if (a.opt) step_count = prep_step(a.opt, a.hyper, &f, step_count);
    if (a.trace) trace_step(a.trace, entries, &f, step_count, scale_after);
}

extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_finalize(const NboFinalizeArgs a)
{
    __shared__ double lds_d[NBO_BLOCK / 64];
    __shared__ uint32_t lds_u[NBO_BLOCK / 64];
    finalize_body(a, lds_d, lds_u);
}

// First stage of the norm / found_inf pass.  A fixed grid walks the chunks with
// stride grid, so each block's partial sum depends only on the tensor list.
//   u = g * inv_scale rounded to T (the unscaled gradient the reference stores),
//   sumsq += (f64)u * (f64)u   (trainer.rs:509-510)
// For f32/bf16 inputs the f64 product is exact, so fma(d, d, acc) rounds exactly
// like the reference's separate multiply and add; for f64 inputs it would not, so
// that case keeps the two roundings.
template <int ST> DEV double sq_acc(double acc, typename Traits<ST>::T u)
{
    const double d = (double)u;
    if (ST == NBO_F64) {
        const double q = d * d;
        return acc + q;
    }
    return __builtin_fma(d, d, acc);
}

template <int ST> DEV bool nonfinite(typename Traits<ST>::T x);
template <> __device__ __forceinline__ bool nonfinite<NBO_F32>(float x) { return nonfinite_f32(x); }
template <> __device__ __forceinline__ bool nonfinite<NBO_BF16>(float x) { return nonfinite_f32(x); }
template <> __device__ __forceinline__ bool nonfinite<NBO_F64>(double x) { return nonfinite_f64(x); }
template <> __device__ __forceinline__ bool nonfinite<NBO_PBF16>(BF x) { return x.nonfinite(); }
template <> __device__ __forceinline__ bool nonfinite<NBO_F16>(float x) { return nonfinite_f32(x); }
template <> __device__ __forceinline__ bool nonfinite<NBO_PF16>(HF x) { return x.nonfinite(); }

// A 16-bit pattern as the arithmetic type of storage ST (exact).
template <int ST> DEV typename Traits<ST>::T from_half_bits(uint32_t b);
template <> __device__ __forceinline__ float from_half_bits<NBO_BF16>(uint32_t b) { return bf16_bits_to_f32(b); }
template <> __device__ __forceinline__ float from_half_bits<NBO_F16>(uint32_t b) { return f16_bits_to_f32(b); }
template <> __device__ __forceinline__ BF from_half_bits<NBO_PBF16>(uint32_t b) { return half_from_bits<FMT_BF16>(b); }
template <> __device__ __forceinline__ HF from_half_bits<NBO_PF16>(uint32_t b) { return half_from_bits<FMT_F16>(b); }

template <int ST> DEV void norm_body(const NboNormArgs &a)
{
    typedef typename Traits<ST>::T T;
    enum { SB = Traits<ST>::SBYTES, VEC = Traits<ST>::VEC };
    __shared__ double lds_d[NBO_BLOCK / 64];
    __shared__ uint32_t lds_u[NBO_BLOCK / 64];
    const uint32_t tid = threadIdx.x;
    const T inv = a.scaler ? (T)(1.0 / a.scaler->scale) : (T)1; // core.rs:355
    double acc = 0.0;
    uint32_t bad = 0;

    for (uint32_t ci = blockIdx.x; ci < a.L.nchunks; ci += a.grid) {
        const ChunkRef c = chunk_ref(a.L, ci);
        const char *pg = (const char *)a.g_ptrs[c.t] + c.base * SB;
        // single elements up to the first 16-byte boundary, whole 128-bit vectors, single
        // elements for the rest; every thread adds its elements in this order
        constexpr uint32_t EPV = 16 / SB; // elements per 128-bit vector
        const Peel pl = peel(c.cnt, EPV, SB, false, (uintptr_t)pg);
        for (uint32_t e = tid; e < pl.head; e += NBO_BLOCK) {
            const T x = IO<ST>::ld1(pg + (uint64_t)e * SB);
            bad |= (uint32_t)nonfinite<ST>(x);
            acc = sq_acc<ST>(acc, x * inv);
        }
        const char *pv = pg + (uint64_t)pl.head * SB;
        if constexpr (SB == 2) {
            // 8 half-width elements per 128-bit load.  Inf / NaN test on both halves of a word
            // at once: adding the exponent field's lowest bit to the masked exponent carries
            // into the sign position exactly when the exponent is all ones.
            constexpr bool is_bf = ST == NBO_BF16 || ST == NBO_PBF16;
            constexpr uint32_t EXP_MASK = is_bf ? 0x7F807F80u : 0x7C007C00u;
            constexpr uint32_t EXP_LSB = is_bf ? 0x00800080u : 0x04000400u;
            uint32_t carries = 0;
            for (uint32_t q = tid; q < pl.nvec; q += NBO_BLOCK) {
                const u32x4 w = __builtin_nontemporal_load(GLOBAL_PTR(const u32x4, pv) + q);
                const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    carries |= (ww[k] & EXP_MASK) + EXP_LSB;
                    const T lo = from_half_bits<ST>(ww[k] & 0xFFFFu), hi = from_half_bits<ST>(ww[k] >> 16);
                    acc = sq_acc<ST>(acc, (T)(lo * inv));
                    acc = sq_acc<ST>(acc, (T)(hi * inv));
                }
            }
            bad |= (uint32_t)((carries & 0x80008000u) != 0);
        } else {
            for (uint32_t q = tid; q < pl.nvec; q += NBO_BLOCK) {
                T x[VEC];
                IO<ST>::ldv(pv + (uint64_t)q * VEC * SB, x);
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    bad |= (uint32_t)nonfinite<ST>(x[k]);
                    acc = sq_acc<ST>(acc, x[k] * inv);
                }
            }
        }
        for (uint32_t e = pl.head + pl.nvec * EPV + tid; e < c.cnt; e += NBO_BLOCK) {
            const T x = IO<ST>::ld1(pg + (uint64_t)e * SB);
            bad |= (uint32_t)nonfinite<ST>(x);
            acc = sq_acc<ST>(acc, x * inv);
        }
    }
    const double bs = block_sum(acc, lds_d);
    const uint32_t bo = block_or(bad, lds_u);
    if (tid == 0) {
        a.partial_sumsq[blockIdx.x] = bs;
        a.partial_flag[blockIdx.x] = bo;
    }
}

#define NBO_NORM_KERNEL(name, ST)                                                           \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboNormArgs a)       \
    {                                                                                       \
        norm_body<ST>(a);                                                                   \
    }
NBO_NORM_KERNEL(nbo_norm_f32, NBO_F32)
NBO_NORM_KERNEL(nbo_norm_bf16, NBO_BF16)
NBO_NORM_KERNEL(nbo_norm_f64, NBO_F64)
// bf16 gradients of a bf16 optimizer: the unscaled gradient is itself a bf16 value
// (g * bf16(1/scale), rounded to bf16) before it is squared.
NBO_NORM_KERNEL(nbo_norm_pbf16, NBO_PBF16)
NBO_NORM_KERNEL(nbo_norm_f16, NBO_F16)
NBO_NORM_KERNEL(nbo_norm_pf16, NBO_PF16)

// Vector accesses of the element-wise passes: 128 bits wide for every element type, i.e. 8
// elements of a 16-bit tensor computed in f32 (the update kernels take those 4 at a time, in
// step with their 128-bit f32 state vectors).  A vector can be held as the raw bits it was
// loaded as (a 16-bit tensor's eight values would take twice the registers once widened) and
// unpacked into EV values of the arithmetic type only where they are used.
template <typename T> struct Bits128;
template <> struct Bits128<float> {
    enum { EV = 4 };
    DEV void unpack(int, u32x4 v, float (&x)[4])
    {
        x[0] = __uint_as_float(v.x); x[1] = __uint_as_float(v.y); x[2] = __uint_as_float(v.z); x[3] = __uint_as_float(v.w);
    }
    DEV u32x4 pack(int, const float (&x)[4])
    {
        const u32x4 v = {__float_as_uint(x[0]), __float_as_uint(x[1]), __float_as_uint(x[2]), __float_as_uint(x[3])};
        return v;
    }
};
template <> struct Bits128<double> {
    enum { EV = 2 };
    // (one cast of the whole vector: assembled from its 32-bit halves, the compiler fetched the
    // first element a second time with a load of its own, and the f64 passes ran 10 % slower)
    DEV void unpack(int, u32x4 v, double (&x)[2])
    {
        const f64x2 d = __builtin_bit_cast(f64x2, v);
        x[0] = d.x;
        x[1] = d.y;
    }
    DEV u32x4 pack(int, const double (&x)[2])
    {
        const f64x2 d = {x[0], x[1]};
        return __builtin_bit_cast(u32x4, d);
    }
};
template <int FMT> struct Bits128<Half16<FMT>> {
    enum { EV = 8 };
    DEV void unpack(int, u32x4 v, Half16<FMT> (&x)[8])
    {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            x[2 * k] = half_from_bits<FMT>(w[k] & 0xFFFFu);
            x[2 * k + 1] = half_from_bits<FMT>(w[k] >> 16);
        }
    }
    DEV u32x4 pack(int, const Half16<FMT> (&x)[8])
    {
        const u32x4 v = {(uint32_t)x[0].bits | ((uint32_t)x[1].bits << 16), (uint32_t)x[2].bits | ((uint32_t)x[3].bits << 16),
                         (uint32_t)x[4].bits | ((uint32_t)x[5].bits << 16), (uint32_t)x[6].bits | ((uint32_t)x[7].bits << 16)};
        return v;
    }
};
// 16-bit tensors computed in f32
struct Bits128HalfWide {
    enum { EV = 8 };
    DEV void unpack(int st, u32x4 v, float (&x)[8])
    {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int k = 0; k < 4; k++) {
            x[2 * k] = st == NBO_BF16 ? bf16_bits_to_f32(w[k] & 0xFFFFu) : f16_bits_to_f32(w[k] & 0xFFFFu);
            x[2 * k + 1] = st == NBO_BF16 ? bf16_bits_to_f32(w[k] >> 16) : f16_bits_to_f32(w[k] >> 16);
        }
    }
    DEV u32x4 pack(int st, const float (&x)[8])
    {
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; k++)
            w[k] = st == NBO_BF16 ? f32_to_bf16_bits(x[2 * k]) | (f32_to_bf16_bits(x[2 * k + 1]) << 16)
                                  : f32_to_f16_bits(x[2 * k]) | (f32_to_f16_bits(x[2 * k + 1]) << 16);
        const u32x4 v = {w[0], w[1], w[2], w[3]};
        return v;
    }
};
template <int ST> struct EwBits : Bits128<typename Traits<ST>::T> {};
template <> struct EwBits<NBO_BF16> : Bits128HalfWide {};
template <> struct EwBits<NBO_F16> : Bits128HalfWide {};

template <int ST> struct EwIO {
    typedef typename Traits<ST>::T T;
    enum { EV = EwBits<ST>::EV };
    DEV u32x4 ld(const char *p) { return NBO_LOAD(GLOBAL_PTR(const u32x4, p)); }
    DEV void st(char *p, u32x4 v) { NBO_STORE(v, GLOBAL_PTR(u32x4, p)); }
    DEV void unpack(u32x4 v, T (&x)[EV]) { EwBits<ST>::unpack(ST, v, x); }
    DEV u32x4 pack(const T (&x)[EV]) { return EwBits<ST>::pack(ST, x); }
    DEV void ld(const char *p, T (&x)[EV]) { unpack(ld(p), x); }
    DEV void st(char *p, const T (&x)[EV]) { st(p, pack(x)); }
};

// ---------------------------------------------------------------------------------
// Element-wise passes over NS tensor lists of one layout: one workgroup per piece of
// PIECE_BYTES of every list (a whole number of rows of one 128-bit vector per thread), every
// row of every list loaded before the first is used.  `op` supplies: loads(s) / stores(s) --
// whether list s is read / written; apply(x) -- the arithmetic on one vector of every list;
// ragged(c, p) -- a chunk that is not whole or not vector-aligned, element by element (done by
// the workgroup of the chunk's first piece).
template <int ST, int NS, uint32_t PIECE_BYTES, typename Op>
DEV void stream_pieces(const NboLayoutDev &L, const uint64_t *const (&lists)[NS], Op &op, bool by_chunk)
{
    typedef typename Traits<ST>::T T;
    enum {
        SB = Traits<ST>::SBYTES,
        VEC = EwIO<ST>::EV,
        ROWB = NBO_BLOCK * VEC * SB,
        PIECE = PIECE_BYTES < NBO_CHUNK * SB ? PIECE_BYTES : NBO_CHUNK * SB,
        R = PIECE / ROWB,
        PPC = NBO_CHUNK * SB / PIECE
    };
    static_assert(R >= 1 && PPC >= 1 && R * PPC * ROWB == NBO_CHUNK * SB, "pieces divide the chunk");
    // by_chunk: a list of many small tensors, most of whose chunks are ragged ends of a row or two.
    // A workgroup per piece would find most pieces missing (after looking the chunk up); such a list
    // is launched one workgroup per chunk instead, each walking its chunk like a ragged one.
    const uint32_t piece = by_chunk ? folded_workgroup() * PPC : folded_workgroup();
    if (piece / PPC >= L.nchunks) return; // the unused end of a folded grid
    const ChunkRef c = chunk_ref(L, piece / PPC);
    char *p[NS];
    uintptr_t all = 0;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        p[s] = (char *)lists[s][c.t] + c.base * SB;
        all |= (uintptr_t)p[s];
    }
    if (by_chunk || c.cnt != NBO_CHUNK || (all & (VEC * SB - 1)) != 0) {
        if (piece % PPC == 0) op.ragged(c, p);
        return;
    }
    const uint64_t off = (uint64_t)(piece % PPC) * (R * ROWB) + threadIdx.x * (VEC * SB);
    u32x4 x[NS][R] = {};
#pragma unroll
    for (int s = 0; s < NS; s++)
        if (op.loads(s)) {
#pragma unroll
            for (int u = 0; u < R; u++) x[s][u] = EwIO<ST>::ld(p[s] + off + u * ROWB);
        }
#pragma unroll
    for (int u = 0; u < R; u++) {
        T v[NS][VEC];
#pragma unroll
        for (int s = 0; s < NS; s++) EwIO<ST>::unpack(x[s][u], v[s]);
        op.apply(v);
#pragma unroll
        for (int s = 0; s < NS; s++) x[s][u] = EwIO<ST>::pack(v[s]);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NS; s++)
        if (op.stores(s)) {
#pragma unroll
            for (int u = 0; u < R; u++) EwIO<ST>::st(p[s] + off + u * ROWB, x[s][u]);
        }
}

// ---------------------------------------------------------------------------------
// In-place gradient passes of the unfused API: multiply by a factor, or zero.
template <int ST> struct ScaleOp {
    typedef typename Traits<ST>::T T;
    enum { SB = Traits<ST>::SBYTES, VEC = Traits<ST>::VEC };
    bool zero;
    T f;
    MEMBER bool loads(int) const { return !zero; }
    MEMBER bool stores(int) const { return true; }
    MEMBER void apply(T (&x)[1][EwIO<ST>::EV]) const
    {
#pragma unroll
        for (int k = 0; k < EwIO<ST>::EV; k++) x[0][k] = zero ? (T)0 : x[0][k] * f;
    }
    MEMBER void ragged(const ChunkRef &c, char *const (&ptr)[1]) const
    {
        const uint32_t tid = threadIdx.x;
        char *pg = ptr[0];
        const Peel pl = peel(c.cnt, VEC, SB, false, (uintptr_t)pg);
        for (uint32_t q = tid; q < pl.nvec; q += NBO_BLOCK) {
            T x[VEC] = {};
            char *p = pg + ((uint64_t)pl.head + (uint64_t)q * VEC) * SB;
            if (!zero) {
                IO<ST>::ldv(p, x);
#pragma unroll
                for (int k = 0; k < VEC; k++) x[k] = x[k] * f;
            }
            IO<ST>::stv(p, x);
        }
        const uint32_t n_single = c.cnt - pl.nvec * VEC; // elements [0, head) and [head + nvec * VEC, cnt)
        for (uint32_t i = tid; i < n_single; i += NBO_BLOCK) {
            const uint32_t e = i < pl.head ? i : i + pl.nvec * VEC;
            char *p = pg + (uint64_t)e * SB;
            const T x = zero ? (T)0 : IO<ST>::ld1(p) * f;
            IO<ST>::st1(p, x);
        }
    }
};

template <int ST> DEV void scale_body(const NboScaleArgs &a)
{
    typedef typename Traits<ST>::T T;
    ScaleOp<ST> op;
    op.zero = a.mode == 3;
    op.f = (T)a.factor;
    if (a.gf) {
        if (a.mode == 0) {
            if (a.gf->found_inf) op.zero = true;
            op.f = sizeof(T) == 4 ? (T)a.gf->inv_scale32 : (T)a.gf->inv_scale64;
        } else if (a.mode == 1) {
            if (!a.gf->clipped) return; // trainer.rs:515: untouched when norm <= max_norm
            op.f = sizeof(T) == 4 ? (T)a.gf->clip32 : (T)a.gf->clip64;
        } else if (a.mode == 4) {
            if (!a.gf->found_inf) return; // core.rs:372-375 alone: zeros on a non-finite gradient
            op.zero = true;
        }
    }
    const uint64_t *const lists[1] = {a.g_ptrs};
    stream_pieces<ST, 1, NBO_EW_PIECE_BYTES>(a.L, lists, op, a.by_chunk != 0);
}

#define NBO_SCALE_KERNEL(name, ST)                                                          \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboScaleArgs a)      \
    {                                                                                       \
        scale_body<ST>(a);                                                                  \
    }
NBO_SCALE_KERNEL(nbo_scale_f32, NBO_F32)
// in place on bf16 tensors the arithmetic is bf16's: factor narrowed to bf16, product
// rounded to bf16
NBO_SCALE_KERNEL(nbo_scale_bf16, NBO_PBF16)
NBO_SCALE_KERNEL(nbo_scale_f16, NBO_PF16)
NBO_SCALE_KERNEL(nbo_scale_f64, NBO_F64)

// Gradient accumulation of the Trainer: buf[i] = &buf[i] + g (trainer.rs:262-266 ->
// B::add, cpu/mod.rs:181: one rounding in T; for bf16 the f32 sum is rounded to bf16,
// scalar/mod.rs:253-351), optionally clearing g afterwards.
template <int ST> struct AccumOp {
    typedef typename Traits<ST>::T T;
    enum { SB = Traits<ST>::SBYTES, VEC = Traits<ST>::VEC };
    bool zero_b;
    MEMBER bool loads(int) const { return true; }
    MEMBER bool stores(int s) const { return s == 0 || zero_b; }
    MEMBER void apply(T (&x)[2][EwIO<ST>::EV]) const
    {
#pragma unroll
        for (int k = 0; k < EwIO<ST>::EV; k++) {
            x[0][k] = x[0][k] + x[1][k];
            x[1][k] = (T)0;
        }
    }
    MEMBER void ragged(const ChunkRef &c, char *const (&ptr)[2]) const
    {
        const uint32_t tid = threadIdx.x;
        char *pa = ptr[0], *pb = ptr[1];
        const Peel pl = peel(c.cnt, VEC, SB, false, (uintptr_t)pa, (uintptr_t)pb);
        for (uint32_t q = tid; q < pl.nvec; q += NBO_BLOCK) {
            const uint64_t off = ((uint64_t)pl.head + (uint64_t)q * VEC) * SB;
            T x[VEC], y[VEC];
            IO<ST>::ldv(pa + off, x);
            IO<ST>::ldv(pb + off, y);
#pragma unroll
            for (int k = 0; k < VEC; k++) x[k] = x[k] + y[k];
            IO<ST>::stv(pa + off, x);
            if (zero_b) {
                T z[VEC] = {};
                IO<ST>::stv(pb + off, z);
            }
        }
        const uint32_t n_single = c.cnt - pl.nvec * VEC; // elements [0, head) and [head + nvec * VEC, cnt)
        for (uint32_t i = tid; i < n_single; i += NBO_BLOCK) {
            const uint64_t off = (uint64_t)(i < pl.head ? i : i + pl.nvec * VEC) * SB;
            const T x = IO<ST>::ld1(pa + off) + IO<ST>::ld1(pb + off);
            IO<ST>::st1(pa + off, x);
            if (zero_b) IO<ST>::st1(pb + off, (T)0);
        }
    }
};

template <int ST> DEV void accum_body(const NboAccumArgs &a)
{
    AccumOp<ST> op;
    op.zero_b = a.zero_b != 0;
    const uint64_t *const lists[2] = {a.a_ptrs, a.b_ptrs};
    stream_pieces<ST, 2, NBO_EW_PIECE_BYTES>(a.L, lists, op, a.by_chunk != 0);
}

#define NBO_ACCUM_KERNEL(name, ST)                                                          \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboAccumArgs a)      \
    {                                                                                       \
        accum_body<ST>(a);                                                                  \
    }
NBO_ACCUM_KERNEL(nbo_accum_f32, NBO_F32)
NBO_ACCUM_KERNEL(nbo_accum_bf16, NBO_BF16)
NBO_ACCUM_KERNEL(nbo_accum_f64, NBO_F64)
NBO_ACCUM_KERNEL(nbo_accum_f16, NBO_F16)

// One micro-batch of the accumulating Trainer in one pass (trainer.rs:230-267): the finite
// scan of GradScaler::unscale_and_update over g (core.rs:357-368), u = g * T(1 / scale)
// (core.rs:376-380), buf = buf + u (trainer.rs:262-266), and -- SUMSQ -- the first stage of the
// sum of squares of the new buf, which clip_grad_norm needs once the last micro-batch is in
// (trainer.rs:504-513).  On a non-finite gradient buf receives garbage: the Trainer discards the
// accumulation then.  It runs like the element-wise passes, one short-lived workgroup per piece,
// 6.3-6.5 TB/s (a fixed grid of workgroups that stride over the chunks, as the norm pass has it,
// reached 5.0-5.6 with these three streams).  Whether a gradient was non-finite is one bit, and
// an OR needs no order: a workgroup that met one ORs it into *a.any_bad, which the second stage
// reads and clears.  The sum of squares does need an order: every workgroup leaves the sum over
// its piece, and nbo_sum_partials and the second stage add those up in a fixed order.
template <int ST, bool SUMSQ> struct AccScaleOp {
    typedef typename Traits<ST>::T T;
    enum { SB = Traits<ST>::SBYTES, VEC = Traits<ST>::VEC, EV = EwIO<ST>::EV };
    T inv;
    bool write_g;
    uint32_t bad;
    double acc;
    MEMBER bool loads(int) const { return true; }
    MEMBER bool stores(int s) const { return s == 0 || write_g; }
    MEMBER void apply(T (&x)[2][EV])
    {
#pragma unroll
        for (int k = 0; k < EV; k++) {
            bad |= (uint32_t)nonfinite<ST>(x[1][k]);
            x[1][k] = x[1][k] * inv;
            x[0][k] = x[0][k] + x[1][k];
            if (SUMSQ) acc = sq_acc<ST>(acc, x[0][k]);
        }
    }
    // the norm pass's walk: single elements up to the first 16-byte boundary, whole vectors,
    // single elements for the rest (buffer and gradients misaligned alike, else all single)
    MEMBER void ragged(const ChunkRef &c, char *const (&ptr)[2])
    {
        const uint32_t tid = threadIdx.x;
        char *pa = ptr[0], *pg = ptr[1];
        const Peel pl = peel(c.cnt, VEC, SB, false, (uintptr_t)pa, (uintptr_t)pg);
        auto single = [&](uint32_t e) {
            const uint64_t off = (uint64_t)e * SB;
            const T g = IO<ST>::ld1(pg + off);
            bad |= (uint32_t)nonfinite<ST>(g);
            const T u = g * inv;
            const T b = IO<ST>::ld1(pa + off) + u;
            if (SUMSQ) acc = sq_acc<ST>(acc, b);
            IO<ST>::st1(pa + off, b);
            if (write_g) IO<ST>::st1(pg + off, u);
        };
        for (uint32_t e = tid; e < pl.head; e += NBO_BLOCK) single(e);
        for (uint32_t q = tid; q < pl.nvec; q += NBO_BLOCK) {
            const uint64_t off = ((uint64_t)pl.head + (uint64_t)q * VEC) * SB;
            T g[VEC], b[VEC];
            IO<ST>::ldv(pg + off, g);
            IO<ST>::ldv(pa + off, b);
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                bad |= (uint32_t)nonfinite<ST>(g[k]);
                g[k] = g[k] * inv;
                b[k] = b[k] + g[k];
                if (SUMSQ) acc = sq_acc<ST>(acc, b[k]);
            }
            IO<ST>::stv(pa + off, b);
            if (write_g) IO<ST>::stv(pg + off, g);
        }
        for (uint32_t e = pl.head + pl.nvec * VEC + tid; e < c.cnt; e += NBO_BLOCK) single(e);
    }
};

template <int ST, bool SUMSQ> DEV void accscale_body(const NboAccNormArgs &a)
{
    typedef typename Traits<ST>::T T;
    __shared__ double lds_d[NBO_BLOCK / 64];
    AccScaleOp<ST, SUMSQ> op;
    op.inv = a.scaler ? (T)(1.0 / a.scaler->scale) : (T)1; // core.rs:355
    op.write_g = a.write_grads != 0;
    op.bad = 0;
    op.acc = 0.0;
    const uint64_t *const lists[2] = {a.acc_ptrs, a.g_ptrs};
    stream_pieces<ST, 2, NBO_EW_PIECE_BYTES>(a.L, lists, op, a.by_chunk != 0);
    // one addition per wave that found something: in a healthy step, none at all
    if (__builtin_amdgcn_ballot_w64(op.bad != 0) != 0 && (threadIdx.x & 63u) == 0)
        __hip_atomic_fetch_or(a.any_bad, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (!SUMSQ) return;
    // (a workgroup whose piece a ragged chunk does not have, or past the end of a folded grid,
    // has added nothing: its sum is the zero it must leave)
    const double bs = block_sum(op.acc, lds_d);
    const uint32_t wg = folded_workgroup();
    if (threadIdx.x == 0 && wg < a.grid) {
        a.partial_sumsq[wg] = bs;
        if (a.partial_flag) a.partial_flag[wg] = 0;
    }
}

extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_sum_partials(const NboSumPartialsArgs a)
{
    __shared__ double lds_d[NBO_BLOCK / 64];
    const uint64_t lo = (uint64_t)blockIdx.x * a.per;
    const uint64_t hi = lo + a.per < a.n ? lo + a.per : a.n;
    double acc = 0.0;
    for (uint64_t i = lo + threadIdx.x; i < hi; i += NBO_BLOCK) acc = acc + a.in[i];
    const double bs = block_sum(acc, lds_d);
    if (threadIdx.x == 0) {
        a.out[blockIdx.x] = bs;
        a.out_flag[blockIdx.x] = 0;
    }
}

#define NBO_ACCSCALE_KERNEL(name, ST)                                                       \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboAccNormArgs a)    \
    {                                                                                       \
        accscale_body<ST, false>(a);                                                        \
    }
NBO_ACCSCALE_KERNEL(nbo_accscale_f32, NBO_F32)
NBO_ACCSCALE_KERNEL(nbo_accscale_bf16, NBO_PBF16)
NBO_ACCSCALE_KERNEL(nbo_accscale_f64, NBO_F64)
NBO_ACCSCALE_KERNEL(nbo_accscale_f16, NBO_PF16)

#define NBO_ACCNORM_KERNEL(name, ST)                                                        \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboAccNormArgs a)    \
    {                                                                                       \
        accscale_body<ST, true>(a);                                                         \
    }
// 16-bit lists: unscale and add in the lists' own type, as the in-place passes do
NBO_ACCNORM_KERNEL(nbo_accnorm_f32, NBO_F32)
NBO_ACCNORM_KERNEL(nbo_accnorm_bf16, NBO_PBF16)
NBO_ACCNORM_KERNEL(nbo_accnorm_f64, NBO_F64)
NBO_ACCNORM_KERNEL(nbo_accnorm_f16, NBO_PF16)

// ---------------------------------------------------------------------------------
// Master-weight casts: arena f32 <- bf16 / f16 tensors (exact widening) and
// bf16 / f16 tensors <- arena f32 (round to nearest even).
template <int ST> DEV void cast_master_body(const NboCastArgs &a)
{
    const ChunkRef c = chunk_ref(a.L, blockIdx.x);
    float *aw = state_part<float>(a.arena, c, a.arena.part_w);
    char *pt = (char *)(a.mode == 0 ? a.src_ptrs[c.t] : a.dst_ptrs[c.t]) + c.base * 2;
    // whole 4-element vectors while the caller's address allows, then single elements
    const uint32_t nvec = (((uintptr_t)pt) & 7u) == 0 ? c.cnt / 4 : 0;
    for (uint32_t q = threadIdx.x; q < nvec; q += NBO_BLOCK) {
        float x[4];
        if (a.mode == 0) {
            IO<ST>::ldv(pt + (uint64_t)q * 8, x);
            st_state(aw + q * 4, x);
        } else {
            ld_state(aw + q * 4, x);
            IO<ST>::stv(pt + (uint64_t)q * 8, x);
        }
    }
    for (uint32_t e = nvec * 4 + threadIdx.x; e < c.cnt; e += NBO_BLOCK) {
        if (a.mode == 0) aw[e] = IO<ST>::ld1(pt + (uint64_t)e * 2);
        else IO<ST>::st1(pt + (uint64_t)e * 2, aw[e]);
    }
}
extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_cast_master(const NboCastArgs a)
{
    if (a.half_type == NBO_F16) cast_master_body<NBO_F16>(a);
    else cast_master_body<NBO_BF16>(a);
}

// ---------------------------------------------------------------------------------
// Backend primitives on tensor lists: the single passes the reference's optimizers are
// chains of (BackendCore::{scale, axpy_inplace, add, zeros, clone_storage},
// BackendMath::{powf, emul, ediv}, nabla-core/src/cpu/mod.rs:137-139, 181, 211-232,
// 264-272; Tensor::map(|x| x + s) as used at nabla-train/src/optim/alg.rs:133).  Every
// operation is one IEEE operation in the arithmetic type, rounded to the element type:
// for bf16 that is the f32 operation followed by bf16::from_f32
// (common/scalar/mod.rs:253-351), including the product inside axpy.
template <int ST> DEV typename Traits<ST>::T to_storage_precision(typename Traits<ST>::T x) { return x; }
template <> __device__ __forceinline__ float to_storage_precision<NBO_BF16>(float x)
{
    return bf16_bits_to_f32(f32_to_bf16_bits(x));
}
template <> __device__ __forceinline__ float to_storage_precision<NBO_F16>(float x)
{
    return f16_bits_to_f32(f32_to_f16_bits(x));
}

// powf(x, 0.5) is taken as the correctly rounded square root with C's pow special
// cases (pow(-0, 0.5) = +0, pow(-inf, 0.5) = +inf); other exponents use the device
// math library's pow.
DEV float pow_elem(float x, float p)
{
    if (p == 0.5f) return x == -__builtin_inff() ? __builtin_inff() : __builtin_fabsf(__builtin_sqrtf(x));
    return powf(x, p);
}
DEV double pow_elem(double x, double p)
{
    if (p == 0.5) return x == -__builtin_inf() ? __builtin_inf() : __builtin_fabs(__builtin_sqrt(x));
    return pow(x, p);
}

// ... of a bf16 list's element, whose result is rounded to bf16: the hardware's square root where
// that rounds to the same bf16 (see sqrt_fast above; with the exact one this pass was compute-bound,
// 5.7 TB/s against the f32 list's 6.3)
DEV float pow_elem_bf16(float x, float p)
{
    if (p == 0.5f && !__builtin_amdgcn_classf(x, CLS_DENORMAL))
        return x == -__builtin_inff() ? __builtin_inff() : __builtin_fabsf(__builtin_amdgcn_sqrtf(x));
    return pow_elem(x, p);
}

template <int ST, typename T> DEV T ew_elem(uint32_t op, T o, T a, T b, T s)
{
    if constexpr (ST == NBO_BF16) {
        if (op == NBO_EW_POWF) return pow_elem_bf16(a, s);
    }
    switch (op) {
    case NBO_EW_SCALE: return a * s;
    case NBO_EW_AXPY: return o + to_storage_precision<ST>(s * a);
    case NBO_EW_ADD: return a + b;
    case NBO_EW_EMUL: return a * b;
    case NBO_EW_EDIV: return a / b;
    case NBO_EW_POWF: return pow_elem(a, s);
    case NBO_EW_ADD_SCALAR: return a + s;
    case NBO_EW_COPY: return a;
    default: return (T)0; // NBO_EW_ZEROS
    }
}

template <int ST> struct EwOp {
    typedef typename Traits<ST>::T T;
    enum { SB = Traits<ST>::SBYTES, VEC = EwIO<ST>::EV };
    uint32_t op;
    bool use_a, use_b, use_o;
    T s;
    MEMBER bool loads(int i) const { return i == 0 ? use_o : i == 1 ? use_a : use_b; }
    MEMBER bool stores(int i) const { return i == 0; }
    MEMBER void apply(T (&x)[3][VEC]) const
    {
#pragma unroll
        for (int k = 0; k < VEC; k++) x[0][k] = ew_elem<ST, T>(op, x[0][k], x[1][k], x[2][k], s);
    }
    MEMBER void ragged(const ChunkRef &c, char *const (&ptr)[3]) const
    {
        const uint32_t tid = threadIdx.x;
        char *po = ptr[0];
        const char *pa = ptr[1], *pb = ptr[2];
        const Peel pl = peel(c.cnt, VEC, SB, false, (uintptr_t)po, (uintptr_t)pa, (uintptr_t)pb);
        for (uint32_t q = tid; q < pl.nvec; q += NBO_BLOCK) {
            const uint64_t off = ((uint64_t)pl.head + (uint64_t)q * VEC) * SB;
            T o[VEC] = {}, x[VEC] = {}, y[VEC] = {};
            if (use_a) EwIO<ST>::ld(pa + off, x);
            if (use_b) EwIO<ST>::ld(pb + off, y);
            if (use_o) EwIO<ST>::ld(po + off, o);
#pragma unroll
            for (int k = 0; k < VEC; k++) o[k] = ew_elem<ST, T>(op, o[k], x[k], y[k], s);
            EwIO<ST>::st(po + off, o);
        }
        const uint32_t n_single = c.cnt - pl.nvec * VEC; // elements [0, head) and [head + nvec * VEC, cnt)
        for (uint32_t i = tid; i < n_single; i += NBO_BLOCK) {
            const uint64_t off = (uint64_t)(i < pl.head ? i : i + pl.nvec * VEC) * SB;
            const T x = use_a ? IO<ST>::ld1(pa + off) : (T)0;
            const T y = use_b ? IO<ST>::ld1(pb + off) : (T)0;
            const T o = use_o ? IO<ST>::ld1(po + off) : (T)0;
            IO<ST>::st1(po + off, ew_elem<ST, T>(op, o, x, y, s));
        }
    }
};

template <int ST> DEV void ew_body(const NboEwArgs &a)
{
    typedef typename Traits<ST>::T T;
    EwOp<ST> op;
    op.op = a.op;
    op.use_a = a.op != NBO_EW_ZEROS;
    op.use_b = a.op == NBO_EW_ADD || a.op == NBO_EW_EMUL || a.op == NBO_EW_EDIV;
    op.use_o = a.op == NBO_EW_AXPY;
    op.s = to_storage_precision<ST>((T)a.s);
    // an operand the operation does not have stands for the output: never read, same alignment
    const uint64_t *const lists[3] = {a.out_ptrs, op.use_a ? a.a_ptrs : a.out_ptrs, op.use_b ? a.b_ptrs : a.out_ptrs};
    stream_pieces<ST, 3, NBO_BACKEND_PIECE_BYTES>(a.L, lists, op, a.by_chunk != 0);
}

#define NBO_EW_KERNEL(name, ST)                                                             \
    extern "C" __global__ __launch_bounds__(NBO_BLOCK) void name(const NboEwArgs a)         \
    {                                                                                       \
        ew_body<ST>(a);                                                                     \
    }
NBO_EW_KERNEL(nbo_ew_f32, NBO_F32)
NBO_EW_KERNEL(nbo_ew_bf16, NBO_BF16)
NBO_EW_KERNEL(nbo_ew_f64, NBO_F64)
NBO_EW_KERNEL(nbo_ew_f16, NBO_F16)

// BackendCore::cast, default implementation (common/backend/mod.rs:157-160):
// U::from_f64(x.to_f64()) per element.  Widening is exact; f64 -> f32 rounds to nearest
// even; anything -> bf16 goes through f32 first (bf16::from_f64 = from_f32(v as f32),
// scalar/mod.rs:338-340), so f64 -> bf16 rounds twice, as the reference does.
template <int ST> DEV double cast_load1(const char *p, uint64_t e)
{
    return (double)IO<ST>::ld1(p + e * Traits<ST>::SBYTES);
}
template <int ST> DEV void cast_store1(char *p, uint64_t e, double v)
{
    typedef typename Traits<ST>::T T;
    IO<ST>::st1(p + e * Traits<ST>::SBYTES, (T)v); // (float)v rounds to nearest even; bf16 narrows once more
}
// four consecutive elements at element index e (a multiple of 4) of a suitably aligned tensor
template <int ST> DEV void cast_load4(const char *p, uint64_t e, double (&v)[4])
{
    typedef typename Traits<ST>::T T;
    enum { VEC = Traits<ST>::VEC };
#pragma unroll
    for (int h = 0; h < 4 / VEC; h++) {
        T x[VEC];
        IO<ST>::ldv(p + (e + h * VEC) * Traits<ST>::SBYTES, x);
#pragma unroll
        for (int k = 0; k < VEC; k++) v[h * VEC + k] = (double)x[k];
    }
}
template <int ST> DEV void cast_store4(char *p, uint64_t e, const double (&v)[4])
{
    typedef typename Traits<ST>::T T;
    enum { VEC = Traits<ST>::VEC };
#pragma unroll
    for (int h = 0; h < 4 / VEC; h++) {
        T x[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) x[k] = (T)v[h * VEC + k];
        IO<ST>::stv(p + (e + h * VEC) * Traits<ST>::SBYTES, x);
    }
}

template <int SRC, int DST> DEV void cast_body(const NboCastListArgs &a, uint32_t wg)
{
    enum { SS = Traits<SRC>::SBYTES, DS = Traits<DST>::SBYTES };
    // one workgroup per NBO_CAST_ROW elements of a chunk (NBO_CAST_QUADS groups of four per thread,
    // all loaded before the first is stored), as the other element-wise passes run; a ragged or
    // misaligned chunk is done by its first workgroup
    const uint32_t row = wg % (NBO_CHUNK / NBO_CAST_ROW);
    const ChunkRef c = chunk_ref(a.L, wg / (NBO_CHUNK / NBO_CAST_ROW));
    const char *ps = (const char *)a.src_ptrs[c.t] + c.base * SS;
    char *pd = (char *)a.dst_ptrs[c.t] + c.base * DS;
    // groups of four while both addresses allow whole vectors (16 bytes at most per access)
    const uint32_t sa = SS * 4 > 16 ? 16 : SS * 4, da = DS * 4 > 16 ? 16 : DS * 4;
    const bool vec_ok = (((uintptr_t)ps & (sa - 1)) | ((uintptr_t)pd & (da - 1))) == 0;
    if (!a.by_chunk && vec_ok && c.cnt == NBO_CHUNK) {
        double v[NBO_CAST_QUADS][4];
        const uint64_t e = (uint64_t)row * NBO_CAST_ROW + threadIdx.x * 4;
#pragma unroll
        for (uint32_t j = 0; j < NBO_CAST_QUADS; j++) cast_load4<SRC>(ps, e + j * (4 * NBO_BLOCK), v[j]);
#pragma unroll
        for (uint32_t j = 0; j < NBO_CAST_QUADS; j++) cast_store4<DST>(pd, e + j * (4 * NBO_BLOCK), v[j]);
        return;
    }
    if (row != 0) return;
    const uint32_t nquad = vec_ok ? c.cnt / 4 : 0;
    for (uint32_t q = threadIdx.x; q < nquad; q += NBO_BLOCK) {
        double v[4];
        cast_load4<SRC>(ps, (uint64_t)q * 4, v);
        cast_store4<DST>(pd, (uint64_t)q * 4, v);
    }
    for (uint32_t e = nquad * 4 + threadIdx.x; e < c.cnt; e += NBO_BLOCK)
        cast_store1<DST>(pd, e, cast_load1<SRC>(ps, e));
}

template <int SRC> DEV void cast_from(const NboCastListArgs &a, uint32_t wg)
{
    if (a.dst_type == NBO_F32) cast_body<SRC, NBO_F32>(a, wg);
    else if (a.dst_type == NBO_BF16) cast_body<SRC, NBO_BF16>(a, wg);
    else if (a.dst_type == NBO_F16) cast_body<SRC, NBO_F16>(a, wg);
    else cast_body<SRC, NBO_F64>(a, wg);
}

extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_cast_list(const NboCastListArgs a)
{
    // (by_chunk: a list of many small tensors, one workgroup per chunk -- see stream_pieces)
    const uint32_t wg = a.by_chunk ? folded_workgroup() * (NBO_CHUNK / NBO_CAST_ROW) : folded_workgroup();
    if (wg / (NBO_CHUNK / NBO_CAST_ROW) >= a.L.nchunks) return; // the unused end of a folded grid
    if (a.src_type == NBO_F32) cast_from<NBO_F32>(a, wg);
    else if (a.src_type == NBO_BF16) cast_from<NBO_BF16>(a, wg);
    else if (a.src_type == NBO_F16) cast_from<NBO_F16>(a, wg);
    else cast_from<NBO_F64>(a, wg);
}

// Zero-fill of an arbitrary byte range: single bytes up to the first 16-byte boundary,
// 128-bit stores for the body, single bytes for the rest.  Takes the place of
// hipMemsetAsync so that everything the library enqueues is a kernel launch (a caller
// may capture a reset or a step into a HIP graph).
extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_fill_zero(const NboFillArgs a)
{
    char *p = (char *)a.p;
    const uint64_t to_boundary = (16u - (uint32_t)((uintptr_t)p & 15u)) & 15u;
    const uint64_t head = to_boundary < a.bytes ? to_boundary : a.bytes;
    const uint64_t nvec = (a.bytes - head) / 16;
    const uint64_t tail0 = head + nvec * 16;
    const uint64_t gid = (uint64_t)blockIdx.x * NBO_BLOCK + threadIdx.x;
    const uint64_t stride = (uint64_t)gridDim.x * NBO_BLOCK;
    const u32x4 z = {0u, 0u, 0u, 0u};
    for (uint64_t i = gid; i < nvec; i += stride)
        __builtin_nontemporal_store(z, GLOBAL_PTR(u32x4, p + head) + i);
    if (gid < head) p[gid] = 0;
    if (gid < a.bytes - tail0) p[tail0 + gid] = 0;
}

// Every one of the 2^32 pairs of 16-bit patterns through the kernels' 16-bit division, every one of
// the 2^16 patterns through their 16-bit square root, compared with the exact operations.  bf16:
// bit for bit with the correctly rounded f32 operation followed by bf16::from_f32 (what the
// kernels computed before they took the hardware's approximations).  Both types: with the f64
// operation narrowed to f32 and then to the type -- for operands of 8 or 11 significant bits that
// is the correctly rounded f32 result (a quotient or root that is not exact in 25 bits lies far
// from every 25-bit number), and it owes nothing to how the compiler lowers an f32 division;
// any NaN equals any NaN there.  Workgroup a, thread t: numerator pattern a, denominators t,
// t + 256, ...
template <int FMT> DEV bool same_or_both_nan(Half16<FMT> x, Half16<FMT> y)
{
    const uint32_t exp = FMT == FMT_BF16 ? 0x7F80u : 0x7C00u, man = FMT == FMT_BF16 ? 0x007Fu : 0x03FFu;
    const bool xn = (x.bits & exp) == exp && (x.bits & man) != 0, yn = (y.bits & exp) == exp && (y.bits & man) != 0;
    return x.bits == y.bits || (xn && yn);
}
template <int FMT> DEV void selftest_half_arith(const NboSelftestArgs &a)
{
    typedef Half16<FMT> H;
    const H x = half_from_bits<FMT>(blockIdx.x);
    unsigned long long bad = 0, example = 0;
    for (uint32_t b = threadIdx.x; b < 65536u; b += NBO_BLOCK) {
        const H y = half_from_bits<FMT>(b);
        const H got = x / y;
        bool ok = same_or_both_nan(got, H((float)((double)x.f() / (double)y.f())));
        if (FMT == FMT_BF16) ok = ok && got.bits == div_exact(half_from_bits<FMT_BF16>(blockIdx.x), half_from_bits<FMT_BF16>(b)).bits;
        if (!ok) {
            bad++;
            example = ((unsigned long long)blockIdx.x << 16) | b;
        }
    }
    if (bad) {
        atomicAdd(&a.out[0], bad);
        a.out[2] = example;
    }
    if (threadIdx.x == 0) {
        const H got = sqrt_rn(x);
        bool ok = same_or_both_nan(got, H((float)__builtin_sqrt((double)x.f())));
        if (FMT == FMT_BF16) {
            ok = ok && got.bits == sqrt_exact(half_from_bits<FMT_BF16>(blockIdx.x)).bits;
            // ... and the bf16 lists' powf(x, 0.5), which takes the same shortcut
            const float xf = x.f();
            ok = ok && f32_to_bf16_bits(pow_elem_bf16(xf, 0.5f)) == f32_to_bf16_bits(pow_elem(xf, 0.5f));
        }
        if (!ok) {
            atomicAdd(&a.out[1], 1ull);
            a.out[3] = blockIdx.x;
        }
    }
}
extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_selftest_bf16_arith(const NboSelftestArgs a)
{
    selftest_half_arith<FMT_BF16>(a);
}
extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_selftest_f16_arith(const NboSelftestArgs a)
{
    selftest_half_arith<FMT_F16>(a);
}

// Placement probe: every workgroup reads and rewrites the same 8 rows of NBO_BLOCK
// 128-bit vectors of two buffers together.  Two buffers in the same region of HBM run
// measurably slower than two in different regions; the host times this to classify
// freshly created chunks (their contents do not matter yet).  The host launches
// bytes / (16 * 8 * NBO_BLOCK) workgroups of NBO_BLOCK threads, so every access stays
// inside the two windows.
extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_probe_rmw2(f32x4 *a, f32x4 *b)
{
    const uint64_t c0 = (uint64_t)blockIdx.x * (8 * NBO_BLOCK);
    f32x4 va[8], vb[8];
#pragma unroll
    for (int u = 0; u < 8; u++) {
        const uint64_t i = c0 + u * NBO_BLOCK + threadIdx.x;
        va[u] = __builtin_nontemporal_load(a + i);
        vb[u] = __builtin_nontemporal_load(b + i);
    }
#pragma unroll
    for (int u = 0; u < 8; u++) {
        const uint64_t i = c0 + u * NBO_BLOCK + threadIdx.x;
        __builtin_nontemporal_store(va[u] + 1.0f, a + i);
        __builtin_nontemporal_store(vb[u] + 1.0f, b + i);
    }
}
