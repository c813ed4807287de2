// gfx950 measurement kernels: what the MI355X memory system gives a set of streams, with the
// optimizer arithmetic taken out.  A code object of its own, loaded only when one of the
// measurement entry points (include/nabla_optim_bench.h) is first called; nothing an optimizer
// step launches lives here.
//
// A "stream" is a dense array of 128-bit vectors.  Every kernel works on RO streams that are
// only read, RMW streams that are read and rewritten in place (every element + 1.0f, so that a
// test can tell from the contents that each vector was read and written exactly once) and WO
// streams that are only written.  What differs between the kernels is the access shape:
//
//   shape 0  the update kernels' own: a 256-thread workgroup per 32 KiB window of every stream
//            (8 rows of 256 vectors), every load issued -- stream by stream -- before the first
//            use, then every store, through vector registers
//   shape 1  the same with 512-thread workgroups (64 KiB windows)
//   shape 2  1024-thread workgroups, 4 rows (64 KiB windows; one workgroup fills a compute unit)
//   shape 3  loads that bypass the vector registers: global -> LDS directly
//            (global_load_lds_dwordx4), read back with ds_read_b128, as many rows deep as 64 KiB
//            of LDS per workgroup hold (two workgroups per compute unit)
//   shape 4  the same as deep as 128-144 KiB of LDS hold (one workgroup per compute unit)
//   shape 5  shape 0's eight rows through registers plus shape 3's rows through LDS at the same
//            time: more bytes in flight per compute unit than the register file alone allows
//   shape 6  a 512-thread workgroup whose waves 0-3 only load (global -> LDS) and whose waves 4-7
//            only store (LDS -> global), double-buffered over `iters` windows
//   shape 7  a grid-striding workgroup that issues the next window's loads before it stores the
//            current one (two windows of 4 rows in registers), over `iters` windows
//   shape 8  shape 0's window, `iters` of them per workgroup one after the other (nothing overlapped)
//   shape 9  the next window's loads go global -> LDS while the current window, moved from LDS
//            into registers, is stored; 256 threads, 64 KiB of LDS (copy, rmw1: 32 KiB)
//   shape 10 the same with 512 threads and twice the LDS
//   shape 11 shape 9 with twice the rows (one workgroup per compute unit)
//   shapes 12-14  shape 0's eight rows taken from 2, 4 or 8 places of every stream at once
//   (contiguous = 1 in the arguments makes the looping shapes 7 and 8 take neighbouring
//   windows instead of windows a whole grid apart)
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../nbo_device_types.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));

#define DEV static __device__ __forceinline__
#define GLOBAL_PTR(type, p) ((__attribute__((address_space(1))) type *)(uintptr_t)(p))
#define LDS_PTR(type, p) ((__attribute__((address_space(3))) type *)(p))

// Plain streaming copy used only to calibrate the HBM byte counters of a profile
// against a transfer of known size.
extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_copy_f32x4(const f32x4 *src, f32x4 *dst,
                                                                      uint64_t nvec)
{
    const uint64_t stride = (uint64_t)gridDim.x * NBO_BLOCK;
    for (uint64_t i = (uint64_t)blockIdx.x * NBO_BLOCK + threadIdx.x; i < nvec; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// Start contents for a checked run: float i of the stream holds i mod 1024, so that a probe
// which hands a lane another lane's vector is caught as well as one that skips a window.
extern "C" __global__ __launch_bounds__(NBO_BLOCK) void nbo_probe_fill_index(f32x4 *dst, uint64_t nvec)
{
    const uint64_t stride = (uint64_t)gridDim.x * NBO_BLOCK;
    for (uint64_t i = (uint64_t)blockIdx.x * NBO_BLOCK + threadIdx.x; i < nvec; i += stride) {
        const float b = (float)((i * 4) & 1023u);
        const f32x4 v = {b, b + 1.0f, b + 2.0f, b + 3.0f};
        dst[i] = v;
    }
}

DEV f32x4 ldg(const void *base, uint64_t i) { return __builtin_nontemporal_load(GLOBAL_PTR(const f32x4, base) + i); }
DEV void stg(void *base, uint64_t i, f32x4 v) { __builtin_nontemporal_store(v, GLOBAL_PTR(f32x4, base) + i); }

// 16 bytes per lane from global memory straight into LDS: lane l of the issuing wave writes
// lds_wave_base + 16 * l (the LDS address is wave-uniform and travels in M0).  Completion is
// counted by vmcnt like any other vector memory load.
DEV void ldg_to_lds(const void *base, uint64_t i, char *lds_wave_base)
{
    __builtin_amdgcn_global_load_lds(GLOBAL_PTR(const f32x4, base) + i, LDS_PTR(void, lds_wave_base), 16, 0, 0);
}
DEV void wait_vmem() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// ... until at most N vector memory operations are outstanding: they complete in issue order,
// so everything but the N issued last is done
template <int N> DEV void wait_vmem_but()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Keeps read-only loads alive without ever storing: a sum of finite inputs is not NaN.
DEV void keep(const NboStreamProbeArgs &a, f32x4 acc)
{
    if (acc.x != acc.x) *GLOBAL_PTR(float, a.buf[0]) = acc.y + acc.z + acc.w;
}

// ---------------------------------------------------------------------------------
// Shapes 0-2: everything through vector registers, one window per workgroup.
template <int RO, int RMW, int WO, int BLOCK, int ROWS> DEV void probe_regs(const NboStreamProbeArgs &a)
{
    enum { NLOAD = RO + RMW };
    const uint64_t c0 = (uint64_t)blockIdx.x * (ROWS * BLOCK) + threadIdx.x;
    f32x4 x[NLOAD > 0 ? NLOAD : 1][ROWS];
#pragma unroll
    for (int s = 0; s < NLOAD; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) x[s][u] = ldg(a.buf[s], c0 + u * BLOCK);
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < RO; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) acc = acc + x[s][u];
#pragma unroll
    for (int s = RO; s < NLOAD; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) x[s][u] = x[s][u] + 1.0f;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = RO; s < NLOAD; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, x[s][u]);
#pragma unroll
    for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, acc);
    if (RO > 0 && WO == 0) keep(a, acc);
}

// ---------------------------------------------------------------------------------
// Shapes 3-5: RV rows through registers and RL rows through LDS, one window of RV + RL rows per
// 256-thread workgroup.  Every wave reads back only the LDS bytes it loaded itself, so waiting
// for its own loads is all the synchronisation there is.
template <int RO, int RMW, int WO, int RV, int RL> DEV void probe_lds(const NboStreamProbeArgs &a)
{
    enum { NLOAD = RO + RMW, BLOCK = 256, ROWS = RV + RL };
    static_assert(NLOAD > 0 && RL > 0, "the LDS shapes need something to load");
    __shared__ __attribute__((aligned(16))) char lds[NLOAD * RL * BLOCK * 16];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint64_t c0 = (uint64_t)blockIdx.x * (ROWS * BLOCK) + threadIdx.x;
    f32x4 x[NLOAD][RV > 0 ? RV : 1];
    // stream after stream: the register rows, then the LDS rows
#pragma unroll
    for (int s = 0; s < NLOAD; s++) {
#pragma unroll
        for (int u = 0; u < RV; u++) x[s][u] = ldg(a.buf[s], c0 + u * BLOCK);
#pragma unroll
        for (int u = 0; u < RL; u++)
            ldg_to_lds(a.buf[s], c0 + (RV + u) * BLOCK, lds + ((s * RL + u) * BLOCK + wave * 64) * 16);
    }
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (RV > 0) {
#pragma unroll
        for (int s = 0; s < RO; s++)
#pragma unroll
            for (int u = 0; u < RV; u++) acc = acc + x[s][u];
#pragma unroll
        for (int s = RO; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < RV; u++) x[s][u] = x[s][u] + 1.0f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = RO; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < RV; u++) stg(a.buf[s], c0 + u * BLOCK, x[s][u]);
#pragma unroll
        for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
            for (int u = 0; u < RV; u++) stg(a.buf[s], c0 + u * BLOCK, acc);
    }
    // the loads into LDS were issued before the register rows' stores
    wait_vmem_but<RV * (RMW + WO)>();
    // the LDS rows, four at a time through registers
    enum { G = RL < 4 ? RL : 4 };
#pragma unroll
    for (int u0 = 0; u0 < RL; u0 += G) {
        f32x4 y[NLOAD][G];
#pragma unroll
        for (int s = 0; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < G; u++)
                if (u0 + u < RL) y[s][u] = *(const f32x4 *)(lds + ((s * RL + u0 + u) * BLOCK + wave * 64 + lane) * 16);
        f32x4 acc2 = acc;
#pragma unroll
        for (int s = 0; s < RO; s++)
#pragma unroll
            for (int u = 0; u < G; u++)
                if (u0 + u < RL) acc2 = acc2 + y[s][u];
#pragma unroll
        for (int s = RO; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < G; u++)
                if (u0 + u < RL) stg(a.buf[s], c0 + (RV + u0 + u) * BLOCK, y[s][u] + 1.0f);
#pragma unroll
        for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
            for (int u = 0; u < G; u++)
                if (u0 + u < RL) stg(a.buf[s], c0 + (RV + u0 + u) * BLOCK, acc2);
        acc = acc2;
    }
    if (RO > 0 && WO == 0) keep(a, acc);
}

// ---------------------------------------------------------------------------------
// Shape 6: waves 0-3 of a 512-thread workgroup load window i + 1 into one half of the LDS while
// waves 4-7 store window i from the other half.  Workgroup b takes windows b, b + grid, ...
// (`iters` of them; the host launches grid = windows / iters workgroups).
template <int RO, int RMW, int WO, int ROWS> DEV void probe_split(const NboStreamProbeArgs &a)
{
    enum { NLOAD = RO + RMW, HALF = 256 };
    static_assert(NLOAD > 0, "the split shape needs something to load");
    __shared__ __attribute__((aligned(16))) char lds[2][NLOAD * ROWS * HALF * 16];
    const bool loader = threadIdx.x < HALF;
    const uint32_t t = threadIdx.x & (HALF - 1), lane = t & 63u, wave = t >> 6;
    const uint32_t iters = a.iters;
    auto window = [&](uint32_t i) { return ((uint64_t)blockIdx.x + (uint64_t)i * gridDim.x) * (ROWS * HALF) + t; };
    auto issue = [&](uint32_t i) {
        const uint64_t c0 = window(i);
#pragma unroll
        for (int s = 0; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++)
                ldg_to_lds(a.buf[s], c0 + u * HALF, lds[i & 1] + ((s * ROWS + u) * HALF + wave * 64) * 16);
    };
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (loader) issue(0);
    for (uint32_t i = 0; i < iters; i++) {
        if (loader) wait_vmem();
        // half i & 1 is full, and the storing waves are done reading the other half
        __syncthreads();
        if (loader) {
            if (i + 1 < iters) issue(i + 1);
        } else {
            const uint64_t c0 = window(i);
            const char *h = lds[i & 1];
            f32x4 y[NLOAD][ROWS];
#pragma unroll
            for (int s = 0; s < NLOAD; s++)
#pragma unroll
                for (int u = 0; u < ROWS; u++) y[s][u] = *(const f32x4 *)(h + ((s * ROWS + u) * HALF + wave * 64 + lane) * 16);
#pragma unroll
            for (int s = 0; s < RO; s++)
#pragma unroll
                for (int u = 0; u < ROWS; u++) acc = acc + y[s][u];
#pragma unroll
            for (int s = RO; s < NLOAD; s++)
#pragma unroll
                for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * HALF, y[s][u] + 1.0f);
#pragma unroll
            for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
                for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * HALF, acc);
        }
    }
    if (RO > 0 && WO == 0 && !loader) keep(a, acc);
}

// ---------------------------------------------------------------------------------
// Shape 7: the next window's loads are issued before the current window's stores, so a
// workgroup never stops loading while it stores.  Windows of 4 rows, two of them in registers.
template <int RO, int RMW, int WO> DEV void probe_pipe(const NboStreamProbeArgs &a)
{
    enum { NLOAD = RO + RMW, BLOCK = 256, ROWS = 4 };
    const uint32_t iters = a.iters;
    auto window = [&](uint32_t i) {
        const uint64_t w = a.contiguous ? (uint64_t)blockIdx.x * iters + i : (uint64_t)blockIdx.x + (uint64_t)i * gridDim.x;
        return w * (ROWS * BLOCK) + threadIdx.x;
    };
    f32x4 cur[NLOAD > 0 ? NLOAD : 1][ROWS], nxt[NLOAD > 0 ? NLOAD : 1][ROWS];
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (iters > 0) {
        const uint64_t c0 = window(0);
#pragma unroll
        for (int s = 0; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) cur[s][u] = ldg(a.buf[s], c0 + u * BLOCK);
    }
    for (uint32_t i = 0; i < iters; i++) {
        if (i + 1 < iters) {
            const uint64_t c1 = window(i + 1);
#pragma unroll
            for (int s = 0; s < NLOAD; s++)
#pragma unroll
                for (int u = 0; u < ROWS; u++) nxt[s][u] = ldg(a.buf[s], c1 + u * BLOCK);
        }
        __builtin_amdgcn_sched_barrier(0);
        const uint64_t c0 = window(i);
#pragma unroll
        for (int s = 0; s < RO; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) acc = acc + cur[s][u];
#pragma unroll
        for (int s = RO; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, cur[s][u] + 1.0f);
#pragma unroll
        for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, acc);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) cur[s][u] = nxt[s][u];
    }
    if (RO > 0 && WO == 0) keep(a, acc);
}

// ---------------------------------------------------------------------------------
// Shape 8: shape 0's window (8 rows through registers, loads then stores) but a workgroup takes
// `iters` windows one after the other -- fewer, longer-lived workgroups, nothing overlapped.
template <int RO, int RMW, int WO> DEV void probe_loop(const NboStreamProbeArgs &a)
{
    enum { NLOAD = RO + RMW, BLOCK = 256, ROWS = 8 };
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint32_t i = 0; i < a.iters; i++) {
        const uint64_t w = a.contiguous ? (uint64_t)blockIdx.x * a.iters + i : (uint64_t)blockIdx.x + (uint64_t)i * gridDim.x;
        const uint64_t c0 = w * (ROWS * BLOCK) + threadIdx.x;
        f32x4 x[NLOAD > 0 ? NLOAD : 1][ROWS];
#pragma unroll
        for (int s = 0; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) x[s][u] = ldg(a.buf[s], c0 + u * BLOCK);
#pragma unroll
        for (int s = 0; s < RO; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) acc = acc + x[s][u];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = RO; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, x[s][u] + 1.0f);
#pragma unroll
        for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, acc);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (RO > 0 && WO == 0) keep(a, acc);
}

// ---------------------------------------------------------------------------------
// Shapes 9 and 10: the next window travels global -> LDS (no registers) while the current one,
// already moved from LDS into registers, is stored.  One LDS buffer of ROWS rows per workgroup:
// a wave reads its part of it into registers, at once re-issues the loads of the window after
// into the same bytes, and only then stores.  BLOCK = 256 or 512 threads.
template <int RO, int RMW, int WO, int BLOCK, int ROWS> DEV void probe_lds_pipe(const NboStreamProbeArgs &a)
{
    enum { NLOAD = RO + RMW, NST = ROWS * (RMW + WO) };
    static_assert(NLOAD > 0, "the LDS shapes need something to load");
    __shared__ __attribute__((aligned(16))) char lds[NLOAD * ROWS * BLOCK * 16];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t iters = a.iters;
    auto window = [&](uint32_t i) { return ((uint64_t)blockIdx.x + (uint64_t)i * gridDim.x) * (ROWS * BLOCK) + threadIdx.x; };
    auto issue = [&](uint32_t i) {
        const uint64_t c0 = window(i);
#pragma unroll
        for (int s = 0; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++)
                ldg_to_lds(a.buf[s], c0 + u * BLOCK, lds + ((s * ROWS + u) * BLOCK + wave * 64) * 16);
    };
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (iters > 0) issue(0);
    for (uint32_t i = 0; i < iters; i++) {
        // window i's loads were issued before window i - 1's stores
        if (i == 0) wait_vmem();
        else wait_vmem_but<NST>();
        f32x4 y[NLOAD][ROWS];
#pragma unroll
        for (int s = 0; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) y[s][u] = *(const f32x4 *)(lds + ((s * ROWS + u) * BLOCK + wave * 64 + lane) * 16);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        if (i + 1 < iters) issue(i + 1);
        __builtin_amdgcn_sched_barrier(0);
        const uint64_t c0 = window(i);
#pragma unroll
        for (int s = 0; s < RO; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) acc = acc + y[s][u];
#pragma unroll
        for (int s = RO; s < NLOAD; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, y[s][u] + 1.0f);
#pragma unroll
        for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
            for (int u = 0; u < ROWS; u++) stg(a.buf[s], c0 + u * BLOCK, acc);
        __builtin_amdgcn_sched_barrier(0);
    }
    if (RO > 0 && WO == 0) keep(a, acc);
}

// ---------------------------------------------------------------------------------
// Shapes 12-14: shape 0's eight rows per workgroup, all loaded before the first store, but taken
// from F places of every stream at once: workgroup b covers rows [0, 8 / F) of the windows
// b, b + grid, ..., b + (F - 1) * grid (windows of 8 / F rows).  The chip then walks every
// stream along F fronts instead of one.
template <int RO, int RMW, int WO, int F> DEV void probe_fronts(const NboStreamProbeArgs &a)
{
    enum { NLOAD = RO + RMW, BLOCK = 256, ROWS = 8, R = ROWS / F };
    static_assert(R * F == ROWS, "fronts divide the eight rows");
    uint64_t c[ROWS];
#pragma unroll
    for (int u = 0; u < ROWS; u++)
        c[u] = ((uint64_t)blockIdx.x + (uint64_t)(u / R) * gridDim.x) * (R * BLOCK) + (u % R) * BLOCK + threadIdx.x;
    f32x4 x[NLOAD > 0 ? NLOAD : 1][ROWS];
#pragma unroll
    for (int s = 0; s < NLOAD; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) x[s][u] = ldg(a.buf[s], c[u]);
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int s = 0; s < RO; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) acc = acc + x[s][u];
#pragma unroll
    for (int s = RO; s < NLOAD; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) x[s][u] = x[s][u] + 1.0f;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = RO; s < NLOAD; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) stg(a.buf[s], c[u], x[s][u]);
#pragma unroll
    for (int s = NLOAD; s < NLOAD + WO; s++)
#pragma unroll
        for (int u = 0; u < ROWS; u++) stg(a.buf[s], c[u], acc);
    if (RO > 0 && WO == 0) keep(a, acc);
}

// one kernel per pattern and shape, so that each has the register budget (and occupancy) of its own
#define PROBE_KERNEL(name, block, body)                                                          \
    extern "C" __global__ __launch_bounds__(block) void name(const NboStreamProbeArgs a) { body(a); }

// shape 0, all ten patterns
PROBE_KERNEL(nbo_probe_read1, 256, (probe_regs<1, 0, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_read3, 256, (probe_regs<3, 0, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_fill1, 256, (probe_regs<0, 0, 1, 256, 8>))
PROBE_KERNEL(nbo_probe_fill3, 256, (probe_regs<0, 0, 3, 256, 8>))
PROBE_KERNEL(nbo_probe_copy, 256, (probe_regs<1, 0, 1, 256, 8>))
PROBE_KERNEL(nbo_probe_rmw1, 256, (probe_regs<0, 1, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_rmw2s, 256, (probe_regs<0, 2, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_rmw3, 256, (probe_regs<0, 3, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_rmw6, 256, (probe_regs<0, 6, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1, 256, (probe_regs<1, 3, 1, 256, 8>))

// shapes 1-7 for the four 1:1 read/write patterns: copy, rmw1, rmw3, r1_rmw3_w1.  The LDS rows
// per pattern are what the stated LDS budget holds (NBO_PROBE_LDS_ROWS in nbo_device_types.h
// repeats them for the host).
PROBE_KERNEL(nbo_probe_copy_s1, 512, (probe_regs<1, 0, 1, 512, 8>))
PROBE_KERNEL(nbo_probe_rmw1_s1, 512, (probe_regs<0, 1, 0, 512, 8>))
PROBE_KERNEL(nbo_probe_rmw3_s1, 512, (probe_regs<0, 3, 0, 512, 8>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s1, 512, (probe_regs<1, 3, 1, 512, 8>))

PROBE_KERNEL(nbo_probe_copy_s2, 1024, (probe_regs<1, 0, 1, 1024, 4>))
PROBE_KERNEL(nbo_probe_rmw1_s2, 1024, (probe_regs<0, 1, 0, 1024, 4>))
PROBE_KERNEL(nbo_probe_rmw3_s2, 1024, (probe_regs<0, 3, 0, 1024, 4>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s2, 1024, (probe_regs<1, 3, 1, 1024, 4>))

PROBE_KERNEL(nbo_probe_copy_s3, 256, (probe_lds<1, 0, 1, 0, 16>))
PROBE_KERNEL(nbo_probe_rmw1_s3, 256, (probe_lds<0, 1, 0, 0, 16>))
PROBE_KERNEL(nbo_probe_rmw3_s3, 256, (probe_lds<0, 3, 0, 0, 5>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s3, 256, (probe_lds<1, 3, 1, 0, 4>))

PROBE_KERNEL(nbo_probe_copy_s4, 256, (probe_lds<1, 0, 1, 0, 32>))
PROBE_KERNEL(nbo_probe_rmw1_s4, 256, (probe_lds<0, 1, 0, 0, 32>))
PROBE_KERNEL(nbo_probe_rmw3_s4, 256, (probe_lds<0, 3, 0, 0, 12>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s4, 256, (probe_lds<1, 3, 1, 0, 8>))

PROBE_KERNEL(nbo_probe_copy_s5, 256, (probe_lds<1, 0, 1, 8, 16>))
PROBE_KERNEL(nbo_probe_rmw1_s5, 256, (probe_lds<0, 1, 0, 8, 16>))
PROBE_KERNEL(nbo_probe_rmw3_s5, 256, (probe_lds<0, 3, 0, 8, 5>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s5, 256, (probe_lds<1, 3, 1, 8, 4>))

PROBE_KERNEL(nbo_probe_copy_s6, 512, (probe_split<1, 0, 1, 8>))
PROBE_KERNEL(nbo_probe_rmw1_s6, 512, (probe_split<0, 1, 0, 8>))
PROBE_KERNEL(nbo_probe_rmw3_s6, 512, (probe_split<0, 3, 0, 4>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s6, 512, (probe_split<1, 3, 1, 4>))

PROBE_KERNEL(nbo_probe_copy_s7, 256, (probe_pipe<1, 0, 1>))
PROBE_KERNEL(nbo_probe_rmw1_s7, 256, (probe_pipe<0, 1, 0>))
PROBE_KERNEL(nbo_probe_rmw3_s7, 256, (probe_pipe<0, 3, 0>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s7, 256, (probe_pipe<1, 3, 1>))

PROBE_KERNEL(nbo_probe_copy_s8, 256, (probe_loop<1, 0, 1>))
PROBE_KERNEL(nbo_probe_rmw1_s8, 256, (probe_loop<0, 1, 0>))
PROBE_KERNEL(nbo_probe_rmw3_s8, 256, (probe_loop<0, 3, 0>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s8, 256, (probe_loop<1, 3, 1>))

PROBE_KERNEL(nbo_probe_copy_s9, 256, (probe_lds_pipe<1, 0, 1, 256, 8>))
PROBE_KERNEL(nbo_probe_rmw1_s9, 256, (probe_lds_pipe<0, 1, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_rmw3_s9, 256, (probe_lds_pipe<0, 3, 0, 256, 4>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s9, 256, (probe_lds_pipe<1, 3, 1, 256, 4>))

PROBE_KERNEL(nbo_probe_copy_s10, 512, (probe_lds_pipe<1, 0, 1, 512, 8>))
PROBE_KERNEL(nbo_probe_rmw1_s10, 512, (probe_lds_pipe<0, 1, 0, 512, 8>))
PROBE_KERNEL(nbo_probe_rmw3_s10, 512, (probe_lds_pipe<0, 3, 0, 512, 4>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s10, 512, (probe_lds_pipe<1, 3, 1, 512, 4>))

PROBE_KERNEL(nbo_probe_copy_s11, 256, (probe_lds_pipe<1, 0, 1, 256, 16>))
PROBE_KERNEL(nbo_probe_rmw1_s11, 256, (probe_lds_pipe<0, 1, 0, 256, 16>))
PROBE_KERNEL(nbo_probe_rmw3_s11, 256, (probe_lds_pipe<0, 3, 0, 256, 8>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s11, 256, (probe_lds_pipe<1, 3, 1, 256, 8>))

PROBE_KERNEL(nbo_probe_copy_s12, 256, (probe_fronts<1, 0, 1, 2>))
PROBE_KERNEL(nbo_probe_rmw1_s12, 256, (probe_fronts<0, 1, 0, 2>))
PROBE_KERNEL(nbo_probe_rmw3_s12, 256, (probe_fronts<0, 3, 0, 2>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s12, 256, (probe_fronts<1, 3, 1, 2>))

PROBE_KERNEL(nbo_probe_copy_s13, 256, (probe_fronts<1, 0, 1, 4>))
PROBE_KERNEL(nbo_probe_rmw1_s13, 256, (probe_fronts<0, 1, 0, 4>))
PROBE_KERNEL(nbo_probe_rmw3_s13, 256, (probe_fronts<0, 3, 0, 4>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s13, 256, (probe_fronts<1, 3, 1, 4>))

PROBE_KERNEL(nbo_probe_copy_s14, 256, (probe_fronts<1, 0, 1, 8>))
PROBE_KERNEL(nbo_probe_rmw1_s14, 256, (probe_fronts<0, 1, 0, 8>))
PROBE_KERNEL(nbo_probe_rmw3_s14, 256, (probe_fronts<0, 3, 0, 8>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s14, 256, (probe_fronts<1, 3, 1, 8>))

// shapes 15-17: shape 0 with 4, 2 and 1 rows per workgroup -- more, shorter-lived workgroups
PROBE_KERNEL(nbo_probe_copy_s15, 256, (probe_regs<1, 0, 1, 256, 4>))
PROBE_KERNEL(nbo_probe_rmw1_s15, 256, (probe_regs<0, 1, 0, 256, 4>))
PROBE_KERNEL(nbo_probe_rmw3_s15, 256, (probe_regs<0, 3, 0, 256, 4>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s15, 256, (probe_regs<1, 3, 1, 256, 4>))

PROBE_KERNEL(nbo_probe_copy_s16, 256, (probe_regs<1, 0, 1, 256, 2>))
PROBE_KERNEL(nbo_probe_rmw1_s16, 256, (probe_regs<0, 1, 0, 256, 2>))
PROBE_KERNEL(nbo_probe_rmw3_s16, 256, (probe_regs<0, 3, 0, 256, 2>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s16, 256, (probe_regs<1, 3, 1, 256, 2>))

PROBE_KERNEL(nbo_probe_copy_s17, 256, (probe_regs<1, 0, 1, 256, 1>))
PROBE_KERNEL(nbo_probe_rmw1_s17, 256, (probe_regs<0, 1, 0, 256, 1>))
PROBE_KERNEL(nbo_probe_rmw3_s17, 256, (probe_regs<0, 3, 0, 256, 1>))
PROBE_KERNEL(nbo_probe_r1_rmw3_w1_s17, 256, (probe_regs<1, 3, 1, 256, 1>))
