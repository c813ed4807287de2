// Runtime, module loading, launches and descriptor building for the fused
// optimizer-step engine.
#include "nbo_host.hpp"
#include "nbo_noalloc.hpp"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <mutex>

// The gfx950 code object, embedded by nbo_code_object.S.
extern "C" const unsigned char nbo_code_object[];
// The measurement kernels' code object, likewise.
extern "C" const unsigned char nbo_bench_code_object[];

namespace nbo {

static thread_local std::string g_last_error;

void set_last_error(const std::string &msg) { g_last_error = msg; }
const char *get_last_error() { return g_last_error.c_str(); }

void fail(int status, const std::string &msg) { throw Error{status, msg}; }

void hip_check(hipError_t e, const char *what)
{
    if (e == hipSuccess) return;
    std::string msg = std::string("HIP ") + what + " failed: " + hipGetErrorString(e);
    // Leave no sticky error behind for the caller's own HIP calls to trip over.
    (void)hipGetLastError();
    fail(NBO_ERR_HIP + (int)e, msg);
}

static const char *const kKernelNames[K_COUNT] = {
    "nbo_update_f32_adamw",  "nbo_update_f32_adam",  "nbo_update_f32_sgd",
    "nbo_update_bf16_adamw", "nbo_update_bf16_adam", "nbo_update_bf16_sgd",
    "nbo_update_f64_adamw",  "nbo_update_f64_adam",  "nbo_update_f64_sgd",
    "nbo_norm_f32",          "nbo_norm_bf16",        "nbo_norm_f64",
    "nbo_scale_f32",         "nbo_scale_bf16",       "nbo_scale_f64",
    "nbo_prep",              "nbo_finalize",         "nbo_cast_master",
    "nbo_sum_partials",      "nbo_probe_rmw2",       "nbo_accum_f32",
    "nbo_accum_bf16",        "nbo_accum_f64",        "nbo_fill_zero",
    "nbo_ew_f32",            "nbo_ew_bf16",          "nbo_ew_f64",
    "nbo_cast_list",         "nbo_update_pbf16_adamw", "nbo_update_pbf16_adam",
    "nbo_update_pbf16_sgd",  "nbo_norm_pbf16",
    "nbo_update_f16_adamw",  "nbo_update_f16_adam",  "nbo_update_f16_sgd",
    "nbo_update_pf16_adamw", "nbo_update_pf16_adam", "nbo_update_pf16_sgd",
    "nbo_norm_f16",          "nbo_norm_pf16",        "nbo_scale_f16",
    "nbo_accum_f16",         "nbo_ew_f16",           "nbo_accnorm_f32",
    "nbo_accnorm_bf16",      "nbo_accnorm_f64",      "nbo_accnorm_f16",
    "nbo_update_f32_adamw_self",   "nbo_update_f32_adam_self",   "nbo_update_f32_sgd_self",
    "nbo_update_bf16_adamw_self",  "nbo_update_bf16_adam_self",  "nbo_update_bf16_sgd_self",
    "nbo_update_f64_adamw_self",   "nbo_update_f64_adam_self",   "nbo_update_f64_sgd_self",
    "nbo_update_f16_adamw_self",   "nbo_update_f16_adam_self",   "nbo_update_f16_sgd_self",
    "nbo_update_pbf16_adamw_self", "nbo_update_pbf16_adam_self", "nbo_update_pbf16_sgd_self",
    "nbo_update_pf16_adamw_self",  "nbo_update_pf16_adam_self",  "nbo_update_pf16_sgd_self",
    "nbo_update_f32_adamw_rows",   "nbo_update_f32_adam_rows",   "nbo_update_bf16_adamw_rows",
    "nbo_update_bf16_adam_rows",   "nbo_update_f64_adamw_rows",  "nbo_update_f64_adam_rows",
    "nbo_update_f16_adamw_rows",   "nbo_update_f16_adam_rows",
    "nbo_accscale_f32",            "nbo_accscale_bf16",          "nbo_accscale_f64",
    "nbo_accscale_f16",            "nbo_selftest_bf16_arith",    "nbo_selftest_f16_arith",
};
static_assert(K_UPDATE_SELF_BASE + 18 == K_UPDATE_ROWS_BASE, "six families of three self-preparing update kernels");
static_assert(K_UPDATE_ROWS_BASE + 8 == K_ACCSCALE_BASE && K_ACCSCALE_F16 + 3 == K_COUNT,
              "four families of two by-row update kernels, four micro-batch kernels without the sum");

static std::mutex g_runtime_mu;
static Runtime *g_runtime = nullptr;

Runtime &Runtime::get()
{
    std::lock_guard<std::mutex> lock(g_runtime_mu);
    if (!g_runtime) g_runtime = new Runtime(); // throws Error; retried on the next call
    return *g_runtime;
}

Runtime *Runtime::existing()
{
    std::lock_guard<std::mutex> lock(g_runtime_mu);
    return g_runtime;
}

Runtime::Runtime()
{
    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev < 1) {
        (void)hipGetLastError();
        fail(NBO_ERR_NO_DEVICE, "no HIP device is visible; this library runs on gfx950 only");
    }
    hip_check(hipSetDevice(0), "hipSetDevice(0)");
    if (const char *gx = std::getenv("NBO_GRID_X_MAX")) { // test hook: fold the grids of small lists as well
        const long v = std::atol(gx);
        if (v >= 1 && v <= 0xFFFFFF) grid_x_max_ = (uint32_t)v;
    }
    hipDeviceProp_t prop;
    hip_check(hipGetDeviceProperties(&prop, 0), "hipGetDeviceProperties");
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        fail(NBO_ERR_NO_DEVICE, std::string("device 0 is ") + prop.gcnArchName +
                                    "; the embedded code object is built for gfx950 only");
    e = hipModuleLoadData(&module_, nbo_code_object);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        fail(NBO_ERR_NO_DEVICE,
             std::string("hipModuleLoadData of the embedded gfx950 code object failed: ") +
                 hipGetErrorString(e));
    }
    for (int k = 0; k < K_COUNT; k++)
        if (kKernelNames[k]) hip_check(hipModuleGetFunction(&fn_[k], module_, kKernelNames[k]), kKernelNames[k]);
    pinned_bytes_ = 8 << 20; // two halves of 4 MiB
    hip_check(hipHostMalloc(&pinned_, pinned_bytes_, hipHostMallocDefault), "hipHostMalloc");
    for (hipEvent_t &e : staged_) hip_check(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
    for (hipEvent_t &e : probe_ev_) hip_check(hipEventCreate(&e), "hipEventCreate");
    partial_sumsq_ = (double *)dmalloc(NBO_NORM_GRID_MAX * sizeof(double));
    partial_flag_ = (uint32_t *)dmalloc(NBO_NORM_GRID_MAX * sizeof(uint32_t));
    gf_scratch_ = (NboGradFactors *)dmalloc(sizeof(NboGradFactors));
    any_bad_ = (uint32_t *)dmalloc(256);
    dzero(any_bad_, 256);
    // The statically allocated scratch of the allocation-free entry point: its device address
    // is looked up here, once, with the device current.  A failure is kept for that entry point
    // to report; nothing else depends on it.
    static_scratch_status_ = noalloc_setup(&device_);
    if (static_scratch_status_ != hipSuccess) (void)hipGetLastError();
}

void Runtime::sync() { hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }

double *Runtime::piece_partials(size_t count)
{
    if (count > piece_partials_cap_) {
        sync(); // a pass still in flight may be writing the old array
        dfree(piece_partials_);
        piece_partials_ = nullptr;
        piece_partials_cap_ = 0;
        piece_partials_ = (double *)dmalloc(count * sizeof(double));
        piece_partials_cap_ = count;
    }
    return piece_partials_;
}

void Runtime::set_stream(hipStream_t s)
{
    if (s == stream_) return;
    // What is already enqueued on the previous stream shares the reduction scratch, the
    // staging buffer and the optimizers' state with what follows on the new one, and nothing
    // orders two streams: finish it first.
    hip_check(hipStreamSynchronize(stream_), "hipStreamSynchronize (previous stream)");
    stream_ = s;
}

hipFunction_t Runtime::function(int kernel) const
{
    if (kernel >= 0 && kernel < K_COUNT && fn_[kernel]) return fn_[kernel];
    if (kernel >= K_COUNT && (size_t)(kernel - K_COUNT) < bench_fn_.size()) return bench_fn_[kernel - K_COUNT];
    fail(NBO_ERR_ARG, "internal: unknown kernel id " + std::to_string(kernel));
}

const char *Runtime::kernel_name(int kernel) const
{
    if (kernel >= 0 && kernel < K_COUNT && kKernelNames[kernel]) return kKernelNames[kernel];
    if (kernel >= K_COUNT && (size_t)(kernel - K_COUNT) < bench_names_.size())
        return bench_names_[kernel - K_COUNT].c_str();
    return "?";
}

int Runtime::bench_kernel(const char *name)
{
    for (size_t k = 0; k < bench_names_.size(); k++)
        if (bench_names_[k] == name) return K_COUNT + (int)k;
    if (!bench_module_) {
        const hipError_t e = hipModuleLoadData(&bench_module_, nbo_bench_code_object);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            bench_module_ = nullptr;
            fail(NBO_ERR_HIP + (int)e, std::string("hipModuleLoadData of the measurement code object failed: ") +
                                           hipGetErrorString(e));
        }
    }
    hipFunction_t f = nullptr;
    hip_check(hipModuleGetFunction(&f, bench_module_, name), name);
    bench_names_.push_back(name);
    bench_fn_.push_back(f);
    return K_COUNT + (int)bench_names_.size() - 1;
}

void Runtime::launch_raw(int kernel, uint32_t grid, uint32_t block, void *arg_struct, bool may_time, uint32_t idle_lds,
                         bool folded)
{
    if (grid == 0) return;
    uint32_t gx = grid, gy = 1;
    if (folded && grid > grid_x_max_) {
        gx = grid_x_max_;
        gy = (uint32_t)(((uint64_t)grid + gx - 1) / gx);
    }
    const hipFunction_t fn = function(kernel);
    void *args[1] = {arg_struct};
    ProfRec rec = {kernel, nullptr, nullptr};
    const bool timed = profiling_ && may_time; // timing creates two events per launch
    if (timed) {
        hip_check(hipEventCreate(&rec.begin), "hipEventCreate");
        hip_check(hipEventCreate(&rec.end), "hipEventCreate");
        hip_check(hipEventRecord(rec.begin, stream_), "hipEventRecord");
    }
    hip_check(hipModuleLaunchKernel(fn, gx, gy, 1, block, 1, 1, idle_lds, stream_, args, nullptr), kernel_name(kernel));
    if (timed) {
        hip_check(hipEventRecord(rec.end, stream_), "hipEventRecord");
        prof_.push_back(rec);
    }
}

void Runtime::profile_enable(bool on)
{
    for (ProfRec &r : prof_) {
        (void)hipEventDestroy(r.begin);
        (void)hipEventDestroy(r.end);
    }
    prof_.clear();
    profiling_ = on;
}

void Runtime::profile_read(const char *kernel_name, uint64_t *launches, double *total_ms)
{
    int id = -1;
    for (int k = 0; k < K_COUNT; k++)
        if (kKernelNames[k] && std::strcmp(kernel_name, kKernelNames[k]) == 0) id = k;
    for (size_t k = 0; k < bench_names_.size(); k++)
        if (bench_names_[k] == kernel_name) id = K_COUNT + (int)k;
    if (id < 0) {
        // perhaps a measurement kernel that has not been launched yet
        try {
            id = bench_kernel(kernel_name);
        } catch (const Error &) {
            fail(NBO_ERR_ARG, std::string("unknown kernel name: ") + kernel_name);
        }
    }
    sync();
    uint64_t n = 0;
    double ms = 0.0;
    for (const ProfRec &r : prof_) {
        if (r.kernel != id) continue;
        float t = 0.0f;
        hip_check(hipEventElapsedTime(&t, r.begin, r.end), "hipEventElapsedTime");
        ms += t;
        n++;
    }
    *launches = n;
    *total_ms = ms;
}

void Runtime::launch_copy(const void *src, void *dst, uint64_t nvec)
{
    if (nvec == 0) return;
    const int k = bench_kernel("nbo_copy_f32x4");
    uint64_t blocks = (nvec + NBO_BLOCK - 1) / NBO_BLOCK;
    // four 128-bit vectors per thread in flight keeps the loop short without
    // starving the memory system
    uint64_t grid = (blocks + 3) / 4;
    if (grid > 0x7FFFFFFFull) grid = 0x7FFFFFFFull;
    void *args[3] = {(void *)&src, (void *)&dst, (void *)&nvec};
    ProfRec rec = {k, nullptr, nullptr};
    if (profiling_) {
        hip_check(hipEventCreate(&rec.begin), "hipEventCreate");
        hip_check(hipEventCreate(&rec.end), "hipEventCreate");
        hip_check(hipEventRecord(rec.begin, stream_), "hipEventRecord");
    }
    hip_check(hipModuleLaunchKernel(function(k), (uint32_t)grid, 1, 1, NBO_BLOCK, 1, 1, 0, stream_, args, nullptr),
              "nbo_copy_f32x4");
    if (profiling_) {
        hip_check(hipEventRecord(rec.end, stream_), "hipEventRecord");
        prof_.push_back(rec);
    }
}

void Runtime::launch_fill_index(void *dst, uint64_t nvec)
{
    if (nvec == 0) return;
    const int k = bench_kernel("nbo_probe_fill_index");
    uint64_t grid = (nvec + NBO_BLOCK - 1) / NBO_BLOCK;
    if (grid > 65536) grid = 65536;
    void *args[2] = {(void *)&dst, (void *)&nvec};
    hip_check(hipModuleLaunchKernel(function(k), (uint32_t)grid, 1, 1, NBO_BLOCK, 1, 1, 0, stream_, args, nullptr),
              "nbo_probe_fill_index");
}

double Runtime::probe_pair_gbps(void *a, void *b, size_t bytes)
{
    // each workgroup covers 8 rows of NBO_BLOCK 128-bit vectors of both buffers; a tail
    // that does not fill a workgroup is left out, so nothing is touched past `bytes`
    const uint64_t per_wg = 8ull * NBO_BLOCK;
    const uint32_t grid = (uint32_t)(bytes / 16 / per_wg);
    if (grid == 0) return 0.0;
    void *args[2] = {(void *)&a, (void *)&b};
    const hipEvent_t e0 = probe_ev_[0], e1 = probe_ev_[1];
    float best = 0.0f;
    for (int rep = 0; rep < 4; rep++) {
        hip_check(hipEventRecord(e0, stream_), "hipEventRecord");
        hip_check(hipModuleLaunchKernel(fn_[K_PROBE], grid, 1, 1, NBO_BLOCK, 1, 1, 0, stream_, args, nullptr),
                  kKernelNames[K_PROBE]);
        hip_check(hipEventRecord(e1, stream_), "hipEventRecord");
        hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
        float ms = 0.0f;
        hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
        if (rep > 0 && (best == 0.0f || ms < best)) best = ms; // first run warms up
    }
    return best > 0.0f ? 4.0 * (double)grid * (double)per_wg * 16 / best / 1e6 : 0.0;
}

uint64_t Runtime::time_launches(int kernel, uint32_t grid, uint32_t block, void *arg_struct, int reps,
                                uint32_t settle_ms, double *best_ms, double *mean_ms)
{
    void *args[1] = {arg_struct};
    const hipFunction_t fn = function(kernel);
    const hipEvent_t e0 = probe_ev_[0], e1 = probe_ev_[1];
    auto one = [&]() {
        hip_check(hipEventRecord(e0, stream_), "hipEventRecord");
        hip_check(hipModuleLaunchKernel(fn, grid, 1, 1, block, 1, 1, 0, stream_, args, nullptr), kernel_name(kernel));
        hip_check(hipEventRecord(e1, stream_), "hipEventRecord");
        hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
        float ms = 0.0f;
        hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
        return (double)ms;
    };
    // warm-up, and time for the driver's background clearing of memory freed just before (the
    // placement search's spare chunks, an earlier measurement's buffers) to finish
    uint64_t launches = 0;
    const auto t0 = std::chrono::steady_clock::now();
    do {
        (void)one();
        launches++;
    } while (std::chrono::duration_cast<std::chrono::milliseconds>(std::chrono::steady_clock::now() - t0).count() <
             (long long)settle_ms);
    double best = 0.0, sum = 0.0;
    for (int rep = 0; rep < reps; rep++) {
        const double ms = one();
        sum += ms;
        if (best == 0.0 || ms < best) best = ms;
    }
    *best_ms = best;
    *mean_ms = reps > 0 ? sum / reps : 0.0;
    return launches + (uint64_t)(reps > 0 ? reps : 0);
}

// Both directions run the two halves of the pinned buffer as a pipeline: while the DMA
// engine fills (or drains) one half, the host copies the other.
void Runtime::read_back(void *host_dst, const void *dev_src, size_t bytes)
{
    char *out = (char *)host_dst;
    const char *src = (const char *)dev_src;
    const size_t half = pinned_bytes_ / 2;
    const size_t nchunks = (bytes + half - 1) / half;
    auto issue = [&](size_t k) {
        const size_t n = std::min(half, bytes - k * half);
        hip_check(hipMemcpyAsync((char *)pinned_ + (k & 1) * half, src + k * half, n, hipMemcpyDeviceToHost, stream_),
                  "hipMemcpyAsync D2H");
        hip_check(hipEventRecord(staged_[k & 1], stream_), "hipEventRecord");
    };
    if (nchunks) issue(0);
    for (size_t k = 0; k < nchunks; k++) {
        if (k + 1 < nchunks) issue(k + 1);
        hip_check(hipEventSynchronize(staged_[k & 1]), "hipEventSynchronize");
        std::memcpy(out + k * half, (const char *)pinned_ + (k & 1) * half, std::min(half, bytes - k * half));
    }
}

void Runtime::upload(void *dev_dst, const void *host_src, size_t bytes)
{
    char *dst = (char *)dev_dst;
    const char *src = (const char *)host_src;
    const size_t half = pinned_bytes_ / 2;
    const size_t nchunks = (bytes + half - 1) / half;
    for (size_t k = 0; k < nchunks; k++) {
        const size_t n = std::min(half, bytes - k * half);
        // the half is free again once the transfer issued from it two chunks ago is done
        if (k >= 2) hip_check(hipEventSynchronize(staged_[k & 1]), "hipEventSynchronize");
        std::memcpy((char *)pinned_ + (k & 1) * half, src + k * half, n);
        hip_check(hipMemcpyAsync(dst + k * half, (const char *)pinned_ + (k & 1) * half, n, hipMemcpyHostToDevice,
                                 stream_),
                  "hipMemcpyAsync H2D");
        hip_check(hipEventRecord(staged_[k & 1], stream_), "hipEventRecord");
    }
    if (nchunks) sync(); // the staging buffer is reused by the next call
}

void *Runtime::dmalloc(size_t bytes)
{
    void *p = nullptr;
    hip_check(hipMalloc(&p, bytes ? bytes : 16), "hipMalloc");
    return p;
}

void Runtime::dfree(void *p)
{
    if (p) (void)hipFree(p);
}

void Runtime::dzero(void *p, size_t bytes)
{
    if (bytes == 0) return;
    NboFillArgs a = {p, bytes};
    // eight 128-bit stores per thread for large ranges; the kernel strides over the rest
    uint64_t grid = (bytes / 16 + 8ull * NBO_BLOCK - 1) / (8ull * NBO_BLOCK);
    if (grid < 1) grid = 1;
    if (grid > (1u << 20)) grid = 1u << 20;
    launch(K_FILL_ZERO, (uint32_t)grid, NBO_BLOCK, a);
}

// ---------------------------------------------------------------------------------

static uint64_t align_up(uint64_t x, uint64_t a) { return (x + a - 1) / a * a; }

void Layout::build(uint64_t nt, const uint64_t *r, const uint64_t *c, bool with_arena, uint32_t row_elems)
{
    rows.assign(r, r + nt);
    cols.assign(c, c + nt);
    n.resize(nt);
    soff.assign(nt, 0);
    std::vector<uint32_t> chunk_begin(nt + 1, 0);
    uint64_t chunks = 0, off = 0, whole = 0;
    for (uint64_t t = 0; t < nt; t++) {
        if (cols[t] != 0 && rows[t] > UINT64_MAX / cols[t])
            fail(NBO_ERR_TOO_LARGE, "tensor element count overflows 64 bits");
        n[t] = rows[t] * cols[t];
        chunk_begin[t] = (uint32_t)chunks;
        chunks += (n[t] + NBO_CHUNK - 1) / NBO_CHUNK;
        whole += n[t] / NBO_CHUNK;
        // one workgroup per chunk: the launch's total thread count has to stay below 2^32
        if (chunks * NBO_BLOCK > 0xFFFFFFFFull)
            fail(NBO_ERR_TOO_LARGE, "tensor list too large for one launch (more than 2^32 threads)");
        // every tensor is padded to whole chunks, so a chunk never straddles two
        // state tiles
        soff[t] = off;
        off += align_up(n[t], NBO_CHUNK);
    }
    chunk_begin[nt] = (uint32_t)chunks;
    nchunks = (uint32_t)chunks;
    whole_chunks = (uint32_t)whole;
    arena_elems = off;
    std::vector<uint32_t> chunk_tensor(nchunks);
    for (uint64_t t = 0; t < nt; t++)
        for (uint32_t ch = chunk_begin[t]; ch < chunk_begin[t + 1]; ch++) chunk_tensor[ch] = (uint32_t)t;

    // the rows that exist, for by-row launches over a list of many small tensors
    std::vector<uint32_t> row_map;
    if (row_elems && !mostly_whole() && nchunks < NBO_ROWS_MAX_CHUNKS) {
        for (uint64_t t = 0; t < nt; t++)
            for (uint32_t ch = chunk_begin[t]; ch < chunk_begin[t + 1]; ch++) {
                const uint64_t left = n[t] - (uint64_t)(ch - chunk_begin[t]) * NBO_CHUNK;
                const uint64_t cnt = left < NBO_CHUNK ? left : NBO_CHUNK;
                const uint32_t nrow = (uint32_t)((cnt + row_elems - 1) / row_elems); // >= 1: a chunk is never empty
                for (uint32_t rw = 0; rw < nrow; rw++) row_map.push_back(ch << 4 | rw);
            }
    }

    // one blob: n | soff | chunk_begin | chunk_tensor | row_map, each 16-byte aligned
    const size_t o_n = 0;
    const size_t o_soff = align_up(o_n + nt * 8, 16);
    const size_t o_cb = align_up(o_soff + nt * 8, 16);
    const size_t o_ct = align_up(o_cb + (nt + 1) * 4, 16);
    const size_t o_rm = align_up(o_ct + (size_t)nchunks * 4, 16);
    const size_t total = align_up(o_rm + row_map.size() * 4, 16);
    std::vector<unsigned char> host(total, 0);
    if (!row_map.empty()) std::memcpy(host.data() + o_rm, row_map.data(), row_map.size() * 4);
    std::memcpy(host.data() + o_n, n.data(), nt * 8);
    std::memcpy(host.data() + o_soff, soff.data(), nt * 8);
    std::memcpy(host.data() + o_cb, chunk_begin.data(), (nt + 1) * 4);
    std::memcpy(host.data() + o_ct, chunk_tensor.data(), (size_t)nchunks * 4);
    Runtime &rt = Runtime::get();
    blob = rt.dmalloc(total);
    rt.upload(blob, host.data(), total);
    char *b = (char *)blob;
    dev.n = (const uint64_t *)(b + o_n);
    dev.soff = with_arena ? (const uint64_t *)(b + o_soff) : nullptr;
    dev.chunk_begin = (const uint32_t *)(b + o_cb);
    dev.chunk_tensor = (const uint32_t *)(b + o_ct);
    dev.nt = (uint32_t)nt;
    dev.nchunks = nchunks;
    dev.row_map = row_map.empty() ? nullptr : (const uint32_t *)(b + o_rm);
    dev.nrows = (uint32_t)row_map.size();
}

void Layout::release()
{
    if (blob) Runtime::get().dfree(blob);
    blob = nullptr;
}

} // namespace nbo
