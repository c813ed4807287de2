// extern "C" entry points of include/nabla_optim.h.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>

#include "nbo_api_guard.hpp"
#include "nbo_host.hpp"
#include "nbo_noalloc.hpp"

using namespace nbo;

namespace nbo {
std::recursive_mutex &api_mutex()
{
    static std::recursive_mutex m;
    return m;
}
} // namespace nbo

namespace {

const char *kind_name(int kind)
{
    return kind == NBO_KIND_ADAMW ? "AdamW" : kind == NBO_KIND_ADAM ? "Adam" : "SGD";
}

NboHyper hyper_of(const nbo_optim *o)
{
    NboHyper h;
    h.lr = o->meta.lr;
    h.beta1 = o->meta.beta1;
    h.beta2 = o->meta.beta2;
    h.eps = o->meta.eps;
    h.weight_decay = o->meta.weight_decay;
    h.momentum = o->meta.momentum;
    h.kind = (uint32_t)o->meta.kind;
    h.pad = 0;
    return h;
}

// The reference's two length asserts (alg.rs:110-119 and siblings), then the shape
// assert of axpy_inplace (tensor/ops.rs:638-646), then what only this engine can get
// wrong: element types.
void check_step_args(const nbo_optim *opt, const nbo_list *params, const nbo_list *grads)
{
    require(opt && params && grads, NBO_ERR_ARG, "null optimizer or tensor list");
    const char *k = kind_name(opt->meta.kind);
    if (params->layout.nt() != grads->layout.nt())
        fail(NBO_ERR_LEN_MISMATCH, std::string("nabla-train: ") + k + " params/grads length mismatch");
    if (params->layout.nt() != opt->layout.nt())
        fail(NBO_ERR_COUNT_MISMATCH, std::string("nabla-train: ") + k + " params count mismatch");
    for (uint64_t t = 0; t < opt->layout.nt(); t++) {
        const bool same = params->layout.rows[t] == grads->layout.rows[t] &&
                          params->layout.cols[t] == grads->layout.cols[t] &&
                          params->layout.rows[t] == opt->layout.rows[t] &&
                          params->layout.cols[t] == opt->layout.cols[t];
        if (!same)
            fail(NBO_ERR_SHAPE,
                 "nabla: axpy_inplace (" + std::to_string(opt->layout.rows[t]) + "x" +
                     std::to_string(opt->layout.cols[t]) + ") vs (" +
                     std::to_string(grads->layout.rows[t]) + "x" +
                     std::to_string(grads->layout.cols[t]) + ") -- shapes must match (tensor " +
                     std::to_string(t) + ")");
    }
    require(params->dtype == grads->dtype, NBO_ERR_DTYPE, "params and grads differ in element type");
    if (is_half(params->dtype) && opt->state_dtype == params->dtype) {
        // Optimizer<bf16> / Optimizer<f16>: state and arithmetic in the tensors' type, no master copy
    } else if (is_half(params->dtype)) {
        require(opt->state_dtype == NBO_DT_F32 && opt->keep_master, NBO_ERR_DTYPE,
                "bf16 / f16 tensors need an optimizer created with state of their own type, or with f32 "
                "state and keep_master");
        require(opt->master_valid, NBO_ERR_NO_MASTER,
                "bf16 / f16 step before the master weights were set (nbo_optim_master_from_params or "
                "nbo_optim_state_write \"w{i}\")");
    } else {
        require(params->dtype == opt->state_dtype, NBO_ERR_DTYPE,
                "tensor element type differs from the optimizer's state type");
    }
}

// which of a fused step's flags ask the update kernel to write zeros over the gradients
uint32_t zero_mode(uint32_t flags)
{
    return ((flags & NBO_STEP_ZERO_GRADS) ? 1u : 0u) | ((flags & NBO_STEP_ZERO_ON_SKIP) ? 2u : 0u);
}

NboUpdateArgs update_args(nbo_optim *opt, nbo_list *params, nbo_list *grads, bool with_gf,
                          uint32_t zero_grads, const NboGradFactors *shared_gf = nullptr)
{
    NboUpdateArgs a = {};
    a.L = opt->layout.dev;
    a.p_ptrs = params->ptrs_dev;
    a.g_ptrs = grads->ptrs_dev;
    a.arena = opt->arena;
    a.opt = opt->dev;
    a.gf = shared_gf ? shared_gf : with_gf ? opt->gf : nullptr;
    a.zero_grads = zero_grads;
    return a;
}

// the optimizer's own arithmetic type is a 16-bit one (Optimizer<bf16> / Optimizer<f16>)
bool pure_half(const nbo_optim *opt) { return is_half(opt->state_dtype); }

// kernel id for element type `dtype`: f32 / bf16 / f64 are `base + dtype`, f16 has its own
int kernel_for(int base, int f16_id, int dtype) { return dtype == NBO_DT_F16 ? f16_id : base + dtype; }

// LDS per workgroup that leaves a compute unit room for four workgroups (160 KiB / 40 KiB)
constexpr uint32_t NBO_WRITE_HEAVY_IDLE_LDS = 40960;

// Element-type family of an optimizer's update kernels: f32 0, bf16 over f32 master weights 1,
// f64 2, f16 over f32 master weights 3, bf16 throughout 4, f16 throughout 5.
int update_family(const nbo_optim *opt, const nbo_list *params)
{
    return opt->state_dtype == NBO_DT_BF16 ? 4 : opt->state_dtype == NBO_DT_F16 ? 5 :
           params->dtype == NBO_DT_F16 ? 3 : params->dtype; // f32 0, bf16 1, f64 2
}

// Lists of fewer chunks than this take the Adam kinds' by-row kernels.  Measured in alternating
// launches inside one process, whole fused step, by chunk against by row: GPT-2-small f32 0.637 /
// 0.625 ms, 1.1 G mixed 5.177 / 5.135, 1.9 G 9.00 / 8.96, 2.8 G 13.10 / 13.10, 4.1 G 19.22 / 19.13,
// 8 G 37.42 / 37.51; f64 lists of 0.3 and 0.8 G parameters 2 % faster by row.  Short-lived
// workgroups fill and drain the chip in an eighth of the time, and below some 4 G parameters the
// steady state is no slower.
// ... and an unfused Adam / AdamW step over fewer chunks than this stays one launch: below some
// 20 us of work a second launch costs more than the shape gains.
constexpr uint32_t NBO_ROWS_MIN_CHUNKS_UNFUSED = 512;

// By row, a chunk is eight (f64: sixteen) workgroups whether it is whole or the ragged end of a
// tensor, and a workgroup of a row the chunk does not have still looks its chunk up before it
// ends: launched that way, a list of many small tensors is slower by row (the 4096-tensor ragged
// set: 0.150 against 0.137 ms per step).  Such a list -- fewer than nine chunks in ten whole --
// carries a map of the rows that exist (Layout::build), and the launch has a workgroup for each
// of those and no other.  16-bit state and arithmetic has four rows to a chunk as it is and is
// level or slower by row (1.1 G parameters: 2.86 against 2.80 ms): never.
bool update_by_row(const nbo_optim *opt)
{
    if (opt->meta.kind == NBO_KIND_SGD) return true; // the SGD kernels are by row throughout
    return !pure_half(opt) && opt->layout.nchunks < NBO_ROWS_MAX_CHUNKS &&
           (opt->layout.mostly_whole() || opt->layout.dev.row_map != nullptr);
}

int update_kernel(const nbo_optim *opt, const nbo_list *params)
{
    const int kind = opt->meta.kind;
    if (kind != NBO_KIND_SGD && update_by_row(opt)) return K_UPDATE_ROWS_BASE + update_family(opt, params) * 2 + kind;
    if (opt->state_dtype == NBO_DT_BF16) return K_UPDATE_PBF16_BASE + kind;
    if (opt->state_dtype == NBO_DT_F16) return K_UPDATE_PF16_BASE + kind;
    if (params->dtype == NBO_DT_F16) return K_UPDATE_F16_BASE + kind;
    return K_UPDATE_BASE + params->dtype * 3 + kind;
}

// Grid of update_kernel(): one workgroup per chunk, or, by row, one per row of a chunk (a row:
// one vector of 2, 4 or 8 elements per thread; update_chunk's BY_ROW in the kernels).
uint32_t update_grid(const nbo_optim *opt, const nbo_list *params)
{
    if (!update_by_row(opt)) return opt->layout.nchunks;
    if (opt->layout.dev.row_map) return opt->layout.dev.nrows;
    const uint32_t vec = is_half(opt->state_dtype) ? 8u : params->dtype == NBO_DT_F64 ? 2u : 4u;
    const uint64_t rows = (uint64_t)opt->layout.nchunks * (NBO_CHUNK / (NBO_BLOCK * vec));
    require(rows <= 0xFFFFFFFFull, NBO_ERR_TOO_LARGE, "list too large for one launch");
    return (uint32_t)rows;
}

// SGD with momentum writes two streams for its three reads: like the other passes that write about
// as much as they read it runs faster with four workgroups to a compute unit than with eight
// (6.28 against 6.02 TB/s on 738 M f32 elements; plain SGD, one write for two reads, loses by
// the same cap, 5.8 against 6.4).
uint32_t update_idle_lds(const nbo_optim *opt)
{
    return opt->meta.kind == NBO_KIND_SGD && opt->meta.momentum != 0.0 ? NBO_WRITE_HEAVY_IDLE_LDS : 0u;
}

// ... of the kernels that prepare the step's scalars themselves
int self_update_kernel(const nbo_optim *opt, const nbo_list *params)
{
    return K_UPDATE_SELF_BASE + update_family(opt, params) * 3 + opt->meta.kind;
}

// One launch that prepares its own scalars, advances step_count (unless *gf says the step is
// skipped) and writes the trace entry.  Not for an empty list: no workgroup would run.
bool self_update_possible(const nbo_optim *opt) { return opt->layout.nchunks > 0; }

NboUpdateArgs self_update_args(nbo_optim *opt, nbo_list *params, nbo_list *grads, const NboGradFactors *gf,
                               uint32_t zero_grads, NboTraceDev *trace, const NboScalerDev *scaler)
{
    NboUpdateArgs a = update_args(opt, params, grads, false, zero_grads, gf);
    a.hyper = hyper_of(opt);
    a.opt_rw = opt->dev;
    a.trace = trace;
    a.scaler = scaler;
    return a;
}

void launch_self_update(nbo_optim *opt, nbo_list *params, nbo_list *grads, const NboGradFactors *gf, uint32_t zero_grads,
                        NboTraceDev *trace, const NboScalerDev *scaler)
{
    static_assert(sizeof(NboGroupedUpdateArgs) <= 4096, "the argument block of a launch");
    NboGroupedUpdateArgs ga = {};
    ga.g[0] = self_update_args(opt, params, grads, gf, zero_grads, trace, scaler);
    ga.first_wg[1] = opt->layout.nchunks;
    ga.n_groups = 1;
    Runtime::get().launch(self_update_kernel(opt, params), opt->layout.nchunks, NBO_BLOCK, ga);
}

uint32_t norm_grid(const Layout &L)
{
    return L.nchunks < NBO_NORM_GRID_MAX ? L.nchunks : NBO_NORM_GRID_MAX;
}

// Where a norm pass leaves its per-workgroup partial results for its second stage.
struct NormScratch {
    double *partial_sumsq;  // [NBO_NORM_GRID_MAX]
    uint32_t *partial_flag; // [NBO_NORM_GRID_MAX]
    bool may_time;          // launches may be bracketed by timing events
};

NormScratch runtime_scratch(Runtime &rt)
{
    return NormScratch{rt.partial_sumsq(), rt.partial_flag(), true};
}

// The norm / found_inf pass over `grads` and its second stage `f` (everything but the partial
// results and the grid filled in by the caller): two launches; for an empty list, the second
// stage alone.
void launch_norm(nbo_list *grads, const NboScalerDev *scaler, bool half_arithmetic, const NormScratch &ws,
                 NboFinalizeArgs f)
{
    Runtime &rt = Runtime::get();
    f.partial_sumsq = ws.partial_sumsq;
    f.partial_flag = ws.partial_flag;
    f.grid = norm_grid(grads->layout);
    NboNormArgs a = {};
    a.L = grads->layout.dev;
    a.g_ptrs = grads->ptrs_dev;
    a.scaler = scaler;
    a.partial_sumsq = ws.partial_sumsq;
    a.partial_flag = ws.partial_flag;
    a.grid = f.grid;
    // bf16 / f16 gradients are unscaled in f32 when they feed f32 state (the mixed-precision
    // composition) and in their own type when the optimizer itself is of that type or they are
    // scaled in place
    int k = kernel_for(K_NORM_BASE, K_NORM_F16, grads->dtype);
    if (half_arithmetic && grads->dtype == NBO_DT_BF16) k = K_NORM_PBF16;
    if (half_arithmetic && grads->dtype == NBO_DT_F16) k = K_NORM_PF16;
    rt.launch_raw(k, a.grid, NBO_BLOCK, &a, ws.may_time); // nothing for an empty list
    rt.launch_raw(K_FINALIZE, 1, NBO_BLOCK, &f, ws.may_time);
}

void launch_norm(nbo_list *grads, const NboScalerDev *scaler, bool half_arithmetic, const NboFinalizeArgs &f)
{
    launch_norm(grads, scaler, half_arithmetic, runtime_scratch(Runtime::get()), f);
}

// The three launches of one fused Trainer tail; `ws` is where the norm pass's partial results
// travel from the first launch to the second.
void fused_step_launches(nbo_optim *opt, nbo_scaler *scaler, nbo_list *params, nbo_list *grads, double max_norm,
                         uint32_t flags, const NormScratch &ws)
{
    Runtime &rt = Runtime::get();
    NboFinalizeArgs f = {};
    // without scaler, clipping and nan policy the pass has nothing to decide, but
    // it still runs so that the trace records every step
    f.check_finite = (scaler || (flags & NBO_STEP_SKIP_NONFINITE)) ? 1u : 0u;
    f.scaler = scaler ? scaler->dev : nullptr;
    f.gf = opt->gf;
    f.opt = opt->dev;
    f.trace = opt->trace;
    f.max_norm = max_norm;
    f.hyper = hyper_of(opt);
    launch_norm(grads, scaler ? scaler->dev : nullptr, pure_half(opt), ws, f);
    NboUpdateArgs a = update_args(opt, params, grads, true, zero_mode(flags));
    rt.launch_raw(update_kernel(opt, params), update_grid(opt, params), NBO_BLOCK, &a, ws.may_time, update_idle_lds(opt),
                  update_by_row(opt));
}

// Grid of the element-wise passes (stream_pieces in the kernels): one workgroup per piece of
// `piece_bytes` (a whole chunk if that is smaller) of a list -- or, for a list of many small
// tensors (fewer than nine chunks in ten whole), one per chunk: most pieces of such a list do not
// exist, and a workgroup has to look its chunk up to find that out (the 4096-tensor ragged set:
// scale_grad 65 us by piece, 38 us by chunk).  *by_chunk tells the kernel which it is.
uint32_t ew_grid(const Layout &layout, int dtype, uint32_t piece_bytes, uint32_t *by_chunk)
{
    *by_chunk = layout.mostly_whole() ? 0u : 1u;
    if (*by_chunk) return layout.nchunks;
    const uint32_t chunk_bytes = NBO_CHUNK * (dtype == NBO_DT_F64 ? 8u : is_half(dtype) ? 2u : 4u);
    const uint64_t pieces = (uint64_t)layout.nchunks * (chunk_bytes / (piece_bytes < chunk_bytes ? piece_bytes : chunk_bytes));
    require(pieces <= 0xFFFFFFFFull, NBO_ERR_TOO_LARGE, "list too large for one launch");
    return (uint32_t)pieces;
}

void launch_scale(nbo_list *grads, const NboGradFactors *gf, double factor, uint32_t mode)
{
    NboScaleArgs a = {};
    a.L = grads->layout.dev;
    a.g_ptrs = grads->ptrs_dev;
    a.gf = gf;
    a.factor = factor;
    a.mode = mode;
    // a pure fill (nothing is read) measured 5-9 % faster with four workgroups per compute unit
    // than with eight: 7.3 against 6.7 TB/s on 738 M f32 elements
    const uint32_t grid = ew_grid(grads->layout, grads->dtype, NBO_EW_PIECE_BYTES, &a.by_chunk);
    Runtime::get().launch_folded(kernel_for(K_SCALE_BASE, K_SCALE_F16, grads->dtype), grid, NBO_BLOCK, a,
                                 mode == 3 ? NBO_WRITE_HEAVY_IDLE_LDS : 0u);
}

// "m12" -> ('m', 12) with the reference's parsing rules (alg.rs:491-507): the prefix
// letter, then what Rust's str::parse::<usize> accepts.
void parse_state_name(const nbo_optim *opt, const char *name, char *which, uint64_t *index)
{
    require(name != nullptr, NBO_ERR_ARG, "null state name");
    const char c = name[0];
    const bool adam_like = opt->meta.kind != NBO_KIND_SGD;
    const bool known = c == 'v' || (c == 'm' && adam_like) || (c == 'w' && opt->keep_master);
    if (!known) fail(NBO_ERR_STATE_KEY, std::string("bad tensor key: ") + name);
    const char *p = name + 1;
    if (*p == '+') p++;
    if (*p == '\0') fail(NBO_ERR_STATE_KEY, std::string("bad tensor key: ") + name);
    uint64_t v = 0;
    for (; *p; p++) {
        if (*p < '0' || *p > '9') fail(NBO_ERR_STATE_KEY, std::string("bad tensor key: ") + name);
        if (v > (UINT64_MAX - (uint64_t)(*p - '0')) / 10)
            fail(NBO_ERR_STATE_KEY, std::string("bad tensor key: ") + name);
        v = v * 10 + (uint64_t)(*p - '0');
    }
    if (v >= opt->layout.nt())
        fail(NBO_ERR_STATE_INDEX, std::string(1, c) + " index out of range: " + std::to_string(v));
    *which = c;
    *index = v;
}

// Index of the arena part a state-name prefix refers to.
uint32_t state_part_index(const nbo_optim *opt, char which)
{
    if (which == 'w') return opt->arena.part_w;
    if (opt->meta.kind == NBO_KIND_SGD) return 0; // velocity
    return which == 'm' ? 0 : opt->arena.part_v;
}

// A kernel that is handed a host address, or a shape larger than the allocation behind the
// address, faults the GPU -- which can take the whole machine's GPUs down with it -- so every
// tensor is checked against what the HIP runtime knows about its address before a list is
// (re)bound: the address must be device-accessible memory the runtime has allocated or
// registered, and the tensor must end inside that allocation.  (An allocator that hands out
// pieces of a larger block is only checked against the block.)  NBO_CHECK_POINTERS=0 in the
// environment skips the check.
bool pointer_checks_enabled()
{
    static const bool on = [] {
        const char *v = std::getenv("NBO_CHECK_POINTERS");
        return !(v && v[0] == '0' && v[1] == '\0');
    }();
    return on;
}

void check_tensor_address(const void *ptr, uint64_t bytes, uint64_t t)
{
    char where[64];
    std::snprintf(where, sizeof(where), "tensor %llu at %p", (unsigned long long)t, ptr);
    hipPointerAttribute_t attr;
    const hipError_t e = hipPointerGetAttributes(&attr, ptr);
    if (e != hipSuccess) (void)hipGetLastError();
    if (e != hipSuccess || attr.type == hipMemoryTypeUnregistered)
        fail(NBO_ERR_ARG, std::string(where) + ": not memory the HIP runtime knows (a host pointer?)");
    hipDeviceptr_t base = nullptr;
    size_t size = 0;
    if (hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)ptr) != hipSuccess) {
        (void)hipGetLastError(); // not every kind of memory has a range to ask for: nothing to compare with
        return;
    }
    const uintptr_t end = (uintptr_t)base + size, p = (uintptr_t)ptr;
    if (p < (uintptr_t)base || bytes > end - p)
        fail(NBO_ERR_ARG, std::string(where) + ": " + std::to_string(bytes) + " bytes do not fit the allocation (" +
                              std::to_string(end - p) + " bytes from there to its end)");
}

// Copies the n elements of tensor i's part `part` between the arena and a dense
// buffer.
void part_copy(nbo_optim *opt, uint64_t i, uint32_t part, void *buf, bool on_device, bool to_engine)
{
    Runtime &rt = Runtime::get();
    const size_t eb = opt->elem_bytes();
    const size_t bytes = (size_t)opt->layout.n[i] * eb;
    if (bytes == 0) return;
    char *dev = (char *)opt->arena.part[part] + (size_t)opt->layout.soff[i] * eb;
    if (on_device && pointer_checks_enabled()) check_tensor_address(buf, bytes, i);
    if (on_device)
        hip_check(hipMemcpyAsync(to_engine ? (void *)dev : buf, to_engine ? buf : (void *)dev, bytes,
                                 hipMemcpyDeviceToDevice, rt.stream()),
                  "hipMemcpyAsync D2D");
    else if (to_engine)
        rt.upload(dev, buf, bytes);
    else
        rt.read_back(buf, dev, bytes);
}

void state_copy(nbo_optim *opt, const char *name, void *buf, uint64_t n_elems, int on_device,
                bool to_engine)
{
    require(opt != nullptr, NBO_ERR_ARG, "null optimizer");
    require(buf != nullptr || n_elems == 0, NBO_ERR_ARG, "null buffer");
    char which;
    uint64_t i;
    parse_state_name(opt, name, &which, &i);
    if (n_elems != opt->layout.n[i])
        fail(NBO_ERR_SHAPE, std::string("state tensor ") + name + " has " +
                                std::to_string(opt->layout.n[i]) + " elements, buffer has " +
                                std::to_string(n_elems));
    part_copy(opt, i, state_part_index(opt, which), buf, on_device != 0, to_engine);
    if (to_engine && which == 'w') {
        // the master weights count as set once a tensor has been written; the caller
        // writes them all before stepping, as a checkpoint load does
        opt->master_valid = true;
    }
}

// Zero-fills one part of the whole arena (asynchronous).
void part_zero(nbo_optim *opt, uint32_t part)
{
    const size_t eb = opt->elem_bytes();
    Runtime::get().dzero(opt->arena.part[part], (size_t)opt->layout.arena_elems * eb);
}

// Allocates the state parts (region-aware, see nbo_placement.hpp), zero-filled.
void alloc_state_parts(nbo_optim *o)
{
    const size_t bytes = (size_t)o->layout.arena_elems * o->elem_bytes();
    o->placement.allocate(o->arena.nparts, bytes, o->arena.part);
    for (uint32_t k = 0; k < o->arena.nparts; k++) Runtime::get().dzero(o->arena.part[k], bytes);
}

void fill_info(const NboTraceEntry &e, nbo_step_info *out)
{
    out->scale = e.scale;
    out->norm = e.norm;
    out->step_count = e.step_count;
    out->found_inf = e.found_inf;
    out->clipped = e.clipped;
}

} // namespace

extern "C" {

int nbo_init(void)
{
    return guarded([] { Runtime::get(); });
}

int nbo_set_stream(void *hip_stream)
{
    return guarded([&] { Runtime::get().set_stream((hipStream_t)hip_stream); });
}

int nbo_sync(void)
{
    return guarded([] { Runtime::get().sync(); });
}

const char *nbo_last_error(void) { return get_last_error(); }

const char *nbo_status_string(int status)
{
    switch (status) {
    case NBO_OK: return "ok";
    case NBO_ERR_LEN_MISMATCH: return "params/grads length mismatch";
    case NBO_ERR_COUNT_MISMATCH: return "params count mismatch";
    case NBO_ERR_SHAPE: return "shapes must match";
    case NBO_ERR_STATE_KEY: return "bad tensor key";
    case NBO_ERR_STATE_INDEX: return "index out of range";
    case NBO_ERR_KIND: return "optim kind mismatch";
    case NBO_ERR_DTYPE: return "element type mismatch";
    case NBO_ERR_ARG: return "invalid argument";
    case NBO_ERR_NO_MASTER: return "master weights not set";
    case NBO_ERR_TOO_LARGE: return "tensor list too large";
    case NBO_ERR_NO_DEVICE: return "no usable gfx950 device";
    case NBO_ERR_IO: return "checkpoint file i/o error";
    default: return status >= NBO_ERR_HIP ? "HIP runtime error" : "unknown status";
    }
}

const char *nbo_version(void) { return "0.1.0"; }

// ---- tensor lists -----------------------------------------------------------------

static void list_upload_ptrs(nbo_list *list, const void *const *dev_ptrs)
{
    const uint64_t nt = list->layout.nt();
    require(nt == 0 || dev_ptrs != nullptr, NBO_ERR_ARG, "null pointer array");
    const uint64_t eb = list->dtype == NBO_DT_F64 ? 8 : is_half(list->dtype) ? 2 : 4;
    std::vector<uint64_t> ptrs(nt);
    for (uint64_t t = 0; t < nt; t++) {
        require(dev_ptrs[t] != nullptr || list->layout.n[t] == 0, NBO_ERR_ARG,
                "null device address for a non-empty tensor");
        if (list->layout.n[t] && pointer_checks_enabled())
            check_tensor_address(dev_ptrs[t], list->layout.n[t] * eb, t);
        ptrs[t] = (uint64_t)(uintptr_t)dev_ptrs[t];
    }
    if (nt) Runtime::get().upload(list->ptrs_dev, ptrs.data(), nt * 8);
    list->ptrs.swap(ptrs);
}

int nbo_list_create(uint64_t n_tensors, const uint64_t *rows, const uint64_t *cols, int dtype,
                    const void *const *dev_ptrs, nbo_list **out)
{
    return guarded([&] {
        require(out != nullptr, NBO_ERR_ARG, "null output pointer");
        *out = nullptr;
        require(n_tensors == 0 || (rows && cols && dev_ptrs), NBO_ERR_ARG, "null shape or pointer array");
        require(dtype == NBO_DT_F32 || dtype == NBO_DT_BF16 || dtype == NBO_DT_F64 || dtype == NBO_DT_F16,
                NBO_ERR_ARG, "unknown dtype");
        require(n_tensors < (1ull << 31), NBO_ERR_TOO_LARGE, "too many tensors");
        Runtime &rt = Runtime::get();
        nbo_list *l = new nbo_list();
        try {
            l->dtype = dtype;
            l->layout.build(n_tensors, rows, cols, false);
            l->ptrs_dev = (uint64_t *)rt.dmalloc(n_tensors * 8);
            list_upload_ptrs(l, dev_ptrs);
            *out = l;
        } catch (...) {
            l->layout.release();
            rt.dfree(l->ptrs_dev);
            delete l;
            throw;
        }
    });
}

int nbo_list_set_ptrs(nbo_list *list, const void *const *dev_ptrs)
{
    return guarded([&] {
        require(list != nullptr, NBO_ERR_ARG, "null list");
        list_upload_ptrs(list, dev_ptrs);
    });
}

int nbo_list_destroy(nbo_list *list)
{
    return guarded([&] {
        if (!list) return;
        Runtime &rt = Runtime::get();
        rt.sync();
        list->layout.release();
        rt.dfree(list->ptrs_dev);
        delete list;
    });
}

// ---- optimizer ----------------------------------------------------------------------

int nbo_optim_create(const nbo_meta *meta, uint64_t n_tensors, const uint64_t *rows,
                     const uint64_t *cols, int state_dtype, int keep_master, nbo_optim **out)
{
    return guarded([&] {
        require(out != nullptr, NBO_ERR_ARG, "null output pointer");
        *out = nullptr;
        require(meta != nullptr, NBO_ERR_ARG, "null meta");
        require(n_tensors == 0 || (rows && cols), NBO_ERR_ARG, "null shape array");
        require(meta->kind >= NBO_KIND_ADAMW && meta->kind <= NBO_KIND_SGD, NBO_ERR_ARG,
                "unknown optimizer kind");
        require(state_dtype == NBO_DT_F32 || state_dtype == NBO_DT_F64 || is_half(state_dtype),
                NBO_ERR_DTYPE, "optimizer state is f32, f64, bf16 or f16");
        require(!keep_master || state_dtype == NBO_DT_F32, NBO_ERR_DTYPE,
                "master weights are f32: keep_master needs f32 state");
        require(n_tensors < (1ull << 31), NBO_ERR_TOO_LARGE, "too many tensors");
        Runtime &rt = Runtime::get();
        nbo_optim *o = new nbo_optim();
        try {
            o->meta = *meta;
            o->state_dtype = state_dtype;
            o->keep_master = keep_master != 0;
            // (a by-row update workgroup takes one 128-bit vector of state per thread)
            o->layout.build(n_tensors, rows, cols, true,
                            is_half(state_dtype) ? 0u : NBO_BLOCK * (state_dtype == NBO_DT_F64 ? 2u : 4u));
            const bool adam_like = meta->kind != NBO_KIND_SGD;
            o->arena.nparts = 1u + (adam_like ? 1u : 0u) + (o->keep_master ? 1u : 0u);
            o->arena.part_v = 1;
            o->arena.part_w = adam_like ? 2 : 1;
            alloc_state_parts(o);
            o->dev = (NboOptimDev *)rt.dmalloc(sizeof(NboOptimDev));
            o->gf = (NboGradFactors *)rt.dmalloc(sizeof(NboGradFactors));
            o->trace = (NboTraceDev *)rt.dmalloc(sizeof(NboTraceDev));
            rt.dzero(o->gf, sizeof(NboGradFactors));
            rt.dzero(o->trace, sizeof(NboTraceDev));
            NboOptimDev d = {};
            d.lr = meta->lr;
            d.beta1 = meta->beta1;
            d.beta2 = meta->beta2;
            d.eps = meta->eps;
            d.weight_decay = meta->weight_decay;
            d.momentum = meta->momentum;
            d.step_count = meta->kind == NBO_KIND_SGD ? 0 : meta->step_count;
            d.kind = (uint32_t)meta->kind;
            rt.upload(o->dev, &d, sizeof(d));
            *out = o;
        } catch (...) {
            o->layout.release();
            o->placement.release();
            rt.dfree(o->dev);
            rt.dfree(o->gf);
            rt.dfree(o->trace);
            delete o;
            throw;
        }
    });
}

int nbo_optim_destroy(nbo_optim *opt)
{
    return guarded([&] {
        if (!opt) return;
        Runtime &rt = Runtime::get();
        rt.sync();
        opt->layout.release();
        opt->placement.release();
        rt.dfree(opt->dev);
        rt.dfree(opt->gf);
        rt.dfree(opt->trace);
        delete opt;
    });
}

int nbo_optim_step(nbo_optim *opt, nbo_list *params, nbo_list *grads)
{
    return guarded([&] {
        check_step_args(opt, params, grads);
        Runtime &rt = Runtime::get();
        NboUpdateArgs a = update_args(opt, params, grads, false, 0u);
        if (opt->meta.kind == NBO_KIND_SGD) {
            // no step_count, no skip: one launch, scalars in the argument block
            a.direct = 1;
            a.sgd_lr = opt->meta.lr;
            a.sgd_momentum = opt->meta.momentum;
            a.sgd_weight_decay = opt->meta.weight_decay;
        } else if (self_update_possible(opt) &&
                   !(update_by_row(opt) && opt->layout.nchunks >= NBO_ROWS_MIN_CHUNKS_UNFUSED)) {
            // Adam::step / AdamW::step is one call (alg.rs:109-150, 254-291): one launch
            launch_self_update(opt, params, grads, nullptr, 0u, nullptr, nullptr);
            return;
        } else {
            // a list of middle size: the by-row kernel behind the scalar preparation (1.5 us in
            // front of it) is faster than the one launch, 0.543 against 0.555 ms for GPT-2-small
            // (the self-preparing kernels cannot run by row: their once-per-workgroup counter
            // would take eight times the additions to one address)
            NboPrepArgs p = {};
            p.opt = opt->dev;
            p.hyper = hyper_of(opt);
            rt.launch(K_PREP, 1, 64, p);
        }
        rt.launch_raw(update_kernel(opt, params), update_grid(opt, params), NBO_BLOCK, &a, true, update_idle_lds(opt),
                      update_by_row(opt));
    });
}

int nbo_optim_reset(nbo_optim *opt)
{
    return guarded([&] {
        require(opt != nullptr, NBO_ERR_ARG, "null optimizer");
        Runtime &rt = Runtime::get();
        part_zero(opt, 0);
        if (opt->meta.kind != NBO_KIND_SGD) part_zero(opt, opt->arena.part_v);
        // step_count = 0 (Adam / AdamW); Sgd has none
        rt.dzero(&opt->dev->step_count, sizeof(uint64_t));
    });
}

int nbo_optim_set_lr(nbo_optim *opt, double lr)
{
    return guarded([&] {
        require(opt != nullptr, NBO_ERR_ARG, "null optimizer");
        opt->meta.lr = lr; // reaches the device with the next step's argument block
    });
}

int nbo_optim_get_meta(nbo_optim *opt, nbo_meta *out)
{
    return guarded([&] {
        require(opt && out, NBO_ERR_ARG, "null optimizer or output");
        *out = opt->meta;
        out->reserved = 0;
        if (opt->meta.kind == NBO_KIND_SGD) {
            // Sgd::meta reports zeros for what it does not have (alg.rs:650-661)
            out->beta1 = out->beta2 = out->eps = 0.0;
            out->step_count = 0;
        } else {
            uint64_t sc = 0;
            Runtime::get().read_back(&sc, &opt->dev->step_count, sizeof(sc));
            out->step_count = sc;
            out->momentum = 0.0;
            if (opt->meta.kind == NBO_KIND_ADAM) out->weight_decay = 0.0;
        }
    });
}

int nbo_optim_load_meta(nbo_optim *opt, const nbo_meta *meta)
{
    return guarded([&] {
        require(opt && meta, NBO_ERR_ARG, "null optimizer or meta");
        if (meta->kind != opt->meta.kind) fail(NBO_ERR_KIND, "optim kind mismatch");
        // set_state of each kind copies exactly these fields (alg.rs:90-105, 244-250, 374-378)
        opt->meta.lr = meta->lr;
        if (opt->meta.kind == NBO_KIND_SGD) {
            opt->meta.momentum = meta->momentum;
            opt->meta.weight_decay = meta->weight_decay;
            return;
        }
        opt->meta.beta1 = meta->beta1;
        opt->meta.beta2 = meta->beta2;
        opt->meta.eps = meta->eps;
        if (opt->meta.kind == NBO_KIND_ADAMW) opt->meta.weight_decay = meta->weight_decay;
        const uint64_t sc = meta->step_count;
        Runtime::get().upload(&opt->dev->step_count, &sc, sizeof(sc));
    });
}

int nbo_optim_state_read(nbo_optim *opt, const char *name, void *buf, uint64_t n_elems,
                         int on_device)
{
    return guarded([&] { state_copy(opt, name, buf, n_elems, on_device, false); });
}

int nbo_optim_state_write(nbo_optim *opt, const char *name, const void *buf, uint64_t n_elems,
                          int on_device)
{
    return guarded([&] { state_copy(opt, name, const_cast<void *>(buf), n_elems, on_device, true); });
}

static void cast_master(nbo_optim *opt, nbo_list *params, uint32_t mode)
{
    require(opt && params, NBO_ERR_ARG, "null optimizer or list");
    require(opt->keep_master, NBO_ERR_DTYPE, "optimizer was created without master weights");
    require(is_half(params->dtype), NBO_ERR_DTYPE, "master casts take a bf16 or f16 list");
    if (params->layout.nt() != opt->layout.nt())
        fail(NBO_ERR_COUNT_MISMATCH, "params count mismatch");
    for (uint64_t t = 0; t < opt->layout.nt(); t++)
        if (params->layout.rows[t] != opt->layout.rows[t] || params->layout.cols[t] != opt->layout.cols[t])
            fail(NBO_ERR_SHAPE, "shapes must match (tensor " + std::to_string(t) + ")");
    NboCastArgs a = {};
    a.L = opt->layout.dev;
    a.src_ptrs = params->ptrs_dev;
    a.dst_ptrs = params->ptrs_dev;
    a.arena = opt->arena;
    a.mode = mode;
    a.half_type = (uint32_t)params->dtype; // NBO_DT_BF16 / NBO_DT_F16 are the device's codes too
    Runtime::get().launch(K_CAST_MASTER, opt->layout.nchunks, NBO_BLOCK, a);
}

int nbo_optim_master_from_params(nbo_optim *opt, nbo_list *params_half)
{
    return guarded([&] {
        cast_master(opt, params_half, 0);
        opt->master_valid = true;
    });
}

int nbo_optim_params_from_master(nbo_optim *opt, nbo_list *params_half)
{
    return guarded([&] {
        require(opt != nullptr, NBO_ERR_ARG, "null optimizer");
        require(opt->master_valid, NBO_ERR_NO_MASTER, "master weights not set");
        cast_master(opt, params_half, 1);
    });
}

int nbo_optim_state_regions(nbo_optim *opt, int *regions)
{
    return guarded([&] {
        require(opt && regions, NBO_ERR_ARG, "null optimizer or output");
        *regions = opt->placement.regions_used();
    });
}

int nbo_optim_state_placement_note(nbo_optim *opt, char *buf, uint64_t buf_bytes)
{
    return guarded([&] {
        require(opt && buf && buf_bytes > 0, NBO_ERR_ARG, "null optimizer or buffer");
        const std::string &n = opt->placement.note();
        const size_t k = n.size() < buf_bytes - 1 ? n.size() : (size_t)(buf_bytes - 1);
        std::memcpy(buf, n.data(), k);
        buf[k] = '\0';
    });
}

// ---- GradScaler ------------------------------------------------------------------------

int nbo_scaler_create(const nbo_scaler_state *state, nbo_scaler **out)
{
    return guarded([&] {
        require(out != nullptr, NBO_ERR_ARG, "null output pointer");
        *out = nullptr;
        Runtime &rt = Runtime::get();
        NboScalerDev d;
        if (state) {
            d.scale = state->scale;
            d.growth_factor = state->growth_factor;
            d.backoff_factor = state->backoff_factor;
            d.growth_interval = state->growth_interval;
            d.consecutive_ok = state->consecutive_ok;
        } else { // GradScaler::new (core.rs:336-344)
            d.scale = 65536.0;
            d.growth_factor = 2.0;
            d.backoff_factor = 0.5;
            d.growth_interval = 2000;
            d.consecutive_ok = 0;
        }
        nbo_scaler *s = new nbo_scaler();
        try {
            s->dev = (NboScalerDev *)rt.dmalloc(sizeof(NboScalerDev));
            rt.upload(s->dev, &d, sizeof(d));
            *out = s;
        } catch (...) {
            rt.dfree(s->dev);
            delete s;
            throw;
        }
    });
}

int nbo_scaler_destroy(nbo_scaler *s)
{
    return guarded([&] {
        if (!s) return;
        Runtime &rt = Runtime::get();
        rt.sync();
        rt.dfree(s->dev);
        delete s;
    });
}

int nbo_scaler_state_get(nbo_scaler *s, nbo_scaler_state *out)
{
    return guarded([&] {
        require(s && out, NBO_ERR_ARG, "null scaler or output");
        NboScalerDev d;
        Runtime::get().read_back(&d, s->dev, sizeof(d));
        out->scale = d.scale;
        out->growth_factor = d.growth_factor;
        out->backoff_factor = d.backoff_factor;
        out->growth_interval = d.growth_interval;
        out->consecutive_ok = d.consecutive_ok;
    });
}

int nbo_scaler_load_state(nbo_scaler *s, const nbo_scaler_state *state)
{
    return guarded([&] {
        require(s && state, NBO_ERR_ARG, "null scaler or state");
        NboScalerDev d;
        d.scale = state->scale;
        d.growth_factor = state->growth_factor;
        d.backoff_factor = state->backoff_factor;
        d.growth_interval = state->growth_interval;
        d.consecutive_ok = state->consecutive_ok;
        Runtime::get().upload(s->dev, &d, sizeof(d));
    });
}

int nbo_scaler_unscale_and_update(nbo_scaler *s, nbo_list *grads, int *ok)
{
    return guarded([&] {
        require(s && grads && ok, NBO_ERR_ARG, "null scaler, list or output");
        Runtime &rt = Runtime::get();
        NboFinalizeArgs f = {};
        f.check_finite = 1;
        f.scaler = s->dev;
        f.gf = rt.gf_scratch();
        launch_norm(grads, s->dev, true, f);
        launch_scale(grads, rt.gf_scratch(), 1.0, 0);
        NboGradFactors g;
        rt.read_back(&g, rt.gf_scratch(), sizeof(g));
        *ok = g.found_inf ? 0 : 1;
    });
}

// ---- gradient utilities -------------------------------------------------------------------

int nbo_clip_grad_norm(nbo_list *grads, double max_norm, double *norm)
{
    return guarded([&] {
        require(grads && norm, NBO_ERR_ARG, "null list or output");
        *norm = 0.0;
        if (max_norm <= 0.0) return; // trainer.rs:501-503
        Runtime &rt = Runtime::get();
        NboFinalizeArgs f = {};
        f.gf = rt.gf_scratch();
        f.max_norm = max_norm;
        launch_norm(grads, nullptr, false, f);
        launch_scale(grads, rt.gf_scratch(), 1.0, 1);
        NboGradFactors g;
        rt.read_back(&g, rt.gf_scratch(), sizeof(g));
        *norm = g.norm;
    });
}

int nbo_has_non_finite(nbo_list *grads, int *found)
{
    return guarded([&] {
        require(grads && found, NBO_ERR_ARG, "null list or output");
        Runtime &rt = Runtime::get();
        NboFinalizeArgs f = {};
        f.check_finite = 1;
        f.gf = rt.gf_scratch();
        launch_norm(grads, nullptr, false, f);
        NboGradFactors g;
        rt.read_back(&g, rt.gf_scratch(), sizeof(g));
        *found = g.found_inf ? 1 : 0;
    });
}

int nbo_zero_grad(nbo_list *grads)
{
    return guarded([&] {
        require(grads != nullptr, NBO_ERR_ARG, "null list");
        launch_scale(grads, nullptr, 0.0, 3);
    });
}

int nbo_scale_grad(nbo_list *grads, double factor)
{
    return guarded([&] {
        require(grads != nullptr, NBO_ERR_ARG, "null list");
        launch_scale(grads, nullptr, factor, 2);
    });
}

// ---- fused Trainer tail ---------------------------------------------------------------------

int nbo_fused_step(nbo_optim *opt, nbo_scaler *scaler, nbo_list *params, nbo_list *grads,
                   double max_norm, uint32_t flags)
{
    return guarded([&] {
        check_step_args(opt, params, grads);
        fused_step_launches(opt, scaler, params, grads, max_norm, flags, runtime_scratch(Runtime::get()));
    });
}

int nbo_fused_step_noalloc(nbo_optim *opt, nbo_scaler *scaler, nbo_list *params, nbo_list *grads,
                           double max_norm, uint32_t flags)
{
    return guarded([&] {
        check_step_args(opt, params, grads);
        // the handles were created through the runtime, so it exists; nothing is created here
        Runtime *rt = Runtime::existing();
        require(rt != nullptr, NBO_ERR_ARG, "nbo_fused_step_noalloc: the runtime does not exist (call nbo_init first)");
        if (rt->static_scratch_status() != hipSuccess)
            fail(NBO_ERR_HIP + (int)rt->static_scratch_status(),
                 std::string("nbo_fused_step_noalloc: the address of the library's static device scratch could "
                             "not be looked up at nbo_init: ") +
                     hipGetErrorString(rt->static_scratch_status()));
        char *ws = (char *)noalloc_scratch(rt->device());
        require(ws != nullptr, NBO_ERR_ARG, "nbo_fused_step_noalloc: no static device scratch on this device");
        // one partial sum and one flag per workgroup of the norm grid have to fit the array
        const uint32_t need = norm_grid(grads->layout);
        if (need > NBO_NOALLOC_MAX_PARTIALS)
            fail(NBO_ERR_TOO_LARGE, "nbo_fused_step_noalloc: the norm pass over this gradient list needs " +
                                        std::to_string(need) + " partial results, the static scratch holds " +
                                        std::to_string(NBO_NOALLOC_MAX_PARTIALS));
        // Every slot the finalize launch reads ([0, grid)) is written by this call's norm launch
        // first, so nothing left behind by an earlier call needs clearing.
        const NormScratch w = {(double *)ws, (uint32_t *)(ws + NBO_NOALLOC_FLAGS_OFFSET), false};
        fused_step_launches(opt, scaler, params, grads, max_norm, flags, w);
    });
}

// Argument checks shared by the two group entry points; returns how many tensors the groups cover.
static uint64_t check_group_args(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                                 nbo_list *const *grads, int grads_dtype)
{
    require(n_groups == 0 || (opts && params && grads), NBO_ERR_ARG, "null group arrays");
    uint64_t covered = 0;
    for (uint64_t g = 0; g < n_groups; g++) {
        check_step_args(opts[g], params[g], grads[g]);
        require(grads[g]->dtype == grads_dtype, NBO_ERR_DTYPE,
                "group gradients differ in element type from the whole list");
        require(pure_half(opts[g]) == pure_half(opts[0]), NBO_ERR_DTYPE,
                "groups mix bf16 and f32 optimizer state");
        covered += grads[g]->layout.nt();
    }
    return covered;
}

// Every group's scalars and update from the one decision in the runtime's scratch, in ONE
// launch for up to NBO_GROUPS_PER_LAUNCH groups of one optimizer kind and element types (what a
// GroupOptimizer<O> holds, optim/groups.rs:269-293); groups of another kind or type start a launch
// of their own, and an empty group, in which no workgroup would run, gets the scalar part alone.
static void launch_group_updates(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                                 nbo_list *const *grads, nbo_scaler *scaler, uint32_t flags)
{
    Runtime &rt = Runtime::get();
    NboGroupedUpdateArgs ga = {};
    int kernel = -1;
    uint64_t wgs = 0;
    auto flush = [&] {
        if (ga.n_groups) rt.launch(kernel, (uint32_t)wgs, NBO_BLOCK, ga);
        ga.n_groups = 0;
        wgs = 0;
    };
    for (uint64_t g = 0; g < n_groups; g++) {
        if (!self_update_possible(opts[g])) {
            NboPrepArgs p = {};
            p.opt = opts[g]->dev;
            p.gf = rt.gf_scratch();
            p.scaler = scaler ? scaler->dev : nullptr;
            p.trace = opts[g]->trace;
            p.hyper = hyper_of(opts[g]);
            rt.launch(K_PREP, 1, 64, p);
            continue;
        }
        const int k = self_update_kernel(opts[g], params[g]);
        if (ga.n_groups == NBO_GROUPS_PER_LAUNCH || (ga.n_groups && k != kernel) ||
            wgs + opts[g]->layout.nchunks > 0x7FFFFFFFull)
            flush();
        kernel = k;
        ga.g[ga.n_groups] = self_update_args(opts[g], params[g], grads[g], rt.gf_scratch(), zero_mode(flags),
                                             opts[g]->trace, scaler ? scaler->dev : nullptr);
        ga.first_wg[ga.n_groups] = (uint32_t)wgs;
        wgs += opts[g]->layout.nchunks;
        ga.first_wg[++ga.n_groups] = (uint32_t)wgs;
    }
    flush();
}

int nbo_fused_step_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                          nbo_list *const *grads, nbo_scaler *scaler, nbo_list *all_grads,
                          double max_norm, uint32_t flags)
{
    return guarded([&] {
        require(all_grads != nullptr, NBO_ERR_ARG, "null gradient list");
        if (check_group_args(n_groups, opts, params, grads, all_grads->dtype) != all_grads->layout.nt())
            fail(NBO_ERR_COUNT_MISMATCH, "nabla-train: GroupOptimizer param count mismatch");
        Runtime &rt = Runtime::get();
        // one decision for all groups: the reference unscales and clips the whole
        // gradient list before any group's step (trainer.rs:230-283)
        NboFinalizeArgs f = {};
        f.check_finite = (scaler || (flags & NBO_STEP_SKIP_NONFINITE)) ? 1u : 0u;
        f.scaler = scaler ? scaler->dev : nullptr;
        f.gf = rt.gf_scratch();
        f.max_norm = max_norm;
        launch_norm(all_grads, scaler ? scaler->dev : nullptr, n_groups > 0 && pure_half(opts[0]), f);
        launch_group_updates(n_groups, opts, params, grads, scaler, flags);
    });
}

int nbo_fused_step_groups_norm(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                               nbo_list *const *grads, double max_norm, double sumsq, uint32_t flags)
{
    return guarded([&] {
        require(sumsq >= 0.0, NBO_ERR_ARG, "the sum of squares is negative or NaN");
        check_group_args(n_groups, opts, params, grads, n_groups ? grads[0]->dtype : (int)NBO_DT_F32);
        Runtime &rt = Runtime::get();
        NboFinalizeArgs f = {};
        f.partial_sumsq = rt.partial_sumsq();
        f.partial_flag = rt.partial_flag();
        f.grid = 0; // nothing to reduce: the sum of squares comes with the call
        f.use_sumsq_in = 1;
        f.sumsq_in = sumsq;
        f.gf = rt.gf_scratch();
        f.max_norm = max_norm;
        rt.launch(K_FINALIZE, 1, NBO_BLOCK, f);
        launch_group_updates(n_groups, opts, params, grads, nullptr, flags);
    });
}

// The asserts of the accumulation `&buf[i] + g` (trainer.rs:262-266 -> tensor/ops.rs add).
static void check_accum_args(const nbo_list *accum, const nbo_list *grads)
{
    require(accum && grads, NBO_ERR_ARG, "null list");
    if (accum->layout.nt() != grads->layout.nt())
        fail(NBO_ERR_LEN_MISMATCH, "nabla-train: accumulation buffers / grads length mismatch");
    for (uint64_t t = 0; t < accum->layout.nt(); t++)
        if (accum->layout.rows[t] != grads->layout.rows[t] || accum->layout.cols[t] != grads->layout.cols[t])
            fail(NBO_ERR_SHAPE, "nabla: add -- shapes are not broadcast-compatible (tensor " +
                                    std::to_string(t) + ")");
    require(accum->dtype == grads->dtype, NBO_ERR_DTYPE, "lists differ in element type");
}

int nbo_accumulate(nbo_list *accum, nbo_list *grads, int zero_grads)
{
    return guarded([&] {
        check_accum_args(accum, grads);
        NboAccumArgs a = {};
        a.L = accum->layout.dev;
        a.a_ptrs = accum->ptrs_dev;
        a.b_ptrs = grads->ptrs_dev;
        a.zero_b = zero_grads ? 1u : 0u;
        // with the gradients cleared the pass writes as much as it reads: fewer workgroups in flight (+6 %)
        const uint32_t grid = ew_grid(accum->layout, accum->dtype, NBO_EW_PIECE_BYTES, &a.by_chunk);
        Runtime::get().launch_folded(kernel_for(K_ACCUM_BASE, K_ACCUM_F16, accum->dtype), grid, NBO_BLOCK, a,
                                     zero_grads ? NBO_WRITE_HEAVY_IDLE_LDS : 0u);
    });
}

int nbo_unscale_accumulate(nbo_scaler *scaler, nbo_list *accum, nbo_list *grads, uint32_t flags, int *ok,
                           double *accum_sumsq)
{
    return guarded([&] {
        check_accum_args(accum, grads);
        require(ok != nullptr, NBO_ERR_ARG, "null output");
        Runtime &rt = Runtime::get();
        NboAccNormArgs a = {};
        a.L = accum->layout.dev;
        a.acc_ptrs = accum->ptrs_dev;
        a.g_ptrs = grads->ptrs_dev;
        a.scaler = scaler ? scaler->dev : nullptr;
        a.write_grads = (flags & NBO_ACC_WRITE_GRADS) ? 1u : 0u;
        a.any_bad = rt.any_bad();
        // both forms run like the element-wise passes; whether a gradient was non-finite reaches
        // the second stage as one bit
        a.grid = ew_grid(accum->layout, accum->dtype, NBO_EW_PIECE_BYTES, &a.by_chunk);
        NboFinalizeArgs f = {};
        f.partial_sumsq = rt.partial_sumsq();
        f.partial_flag = rt.partial_flag();
        f.any_bad = rt.any_bad();
        if (!accum_sumsq) {
            // nobody asked for the sum of squares (every micro-batch but the last): nothing to reduce
            rt.launch_folded(kernel_for(K_ACCSCALE_BASE, K_ACCSCALE_F16, accum->dtype), a.grid, NBO_BLOCK, a);
            f.grid = 0;
        } else if (a.grid <= NBO_NORM_GRID_MAX) {
            // one sum per workgroup, few enough for the second stage to add up itself
            a.partial_sumsq = rt.partial_sumsq();
            a.partial_flag = rt.partial_flag();
            rt.launch_folded(kernel_for(K_ACCNORM_BASE, K_ACCNORM_F16, accum->dtype), a.grid, NBO_BLOCK, a);
            f.grid = a.grid;
        } else {
            // ... or too many: a launch in between adds runs of `per` of them
            a.partial_sumsq = rt.piece_partials(a.grid);
            rt.launch_folded(kernel_for(K_ACCNORM_BASE, K_ACCNORM_F16, accum->dtype), a.grid, NBO_BLOCK, a);
            NboSumPartialsArgs r = {};
            r.in = a.partial_sumsq;
            r.out = rt.partial_sumsq();
            r.out_flag = rt.partial_flag();
            r.n = a.grid;
            r.per = (a.grid + NBO_NORM_GRID_MAX - 1) / NBO_NORM_GRID_MAX;
            f.grid = (a.grid + r.per - 1) / r.per;
            rt.launch(K_SUM_PARTIALS, f.grid, NBO_BLOCK, r);
        }
        f.check_finite = (scaler || (flags & NBO_ACC_CHECK_FINITE)) ? 1u : 0u;
        f.scaler = scaler ? scaler->dev : nullptr;
        f.gf = rt.gf_scratch();
        rt.launch(K_FINALIZE, 1, NBO_BLOCK, f);
        if (a.write_grads && f.check_finite) launch_scale(grads, rt.gf_scratch(), 1.0, 4);
        NboGradFactors g;
        rt.read_back(&g, rt.gf_scratch(), sizeof(g));
        *ok = g.found_inf ? 0 : 1;
        if (accum_sumsq) *accum_sumsq = g.sumsq;
    });
}

int nbo_fused_step_norm(nbo_optim *opt, nbo_list *params, nbo_list *grads, double max_norm, double sumsq,
                        uint32_t flags)
{
    return guarded([&] {
        check_step_args(opt, params, grads);
        require(sumsq >= 0.0, NBO_ERR_ARG, "the sum of squares is negative or NaN");
        Runtime &rt = Runtime::get();
        NboFinalizeArgs f = {};
        f.partial_sumsq = rt.partial_sumsq();
        f.partial_flag = rt.partial_flag();
        f.grid = 0; // nothing to reduce: the sum of squares comes with the call
        f.use_sumsq_in = 1;
        f.sumsq_in = sumsq;
        f.gf = opt->gf;
        f.opt = opt->dev;
        f.trace = opt->trace;
        f.max_norm = max_norm;
        f.hyper = hyper_of(opt);
        rt.launch(K_FINALIZE, 1, NBO_BLOCK, f);
        const NboUpdateArgs a =
            update_args(opt, params, grads, true, zero_mode(flags));
        rt.launch_raw(update_kernel(opt, params), update_grid(opt, params), NBO_BLOCK, const_cast<NboUpdateArgs *>(&a), true,
                      update_idle_lds(opt), update_by_row(opt));
    });
}

// ---- Backend primitives on tensor lists ----------------------------------------------------

// The shape assert every binary Backend operation of the reference starts with
// (tensor/ops.rs:638-646 for axpy_inplace; add / emul / ediv likewise).
static void require_same_shapes(const nbo_list *x, const nbo_list *y, const char *op)
{
    if (x->layout.nt() != y->layout.nt())
        fail(NBO_ERR_LEN_MISMATCH, std::string("nabla: ") + op + " -- tensor lists differ in length");
    for (uint64_t t = 0; t < x->layout.nt(); t++)
        if (x->layout.rows[t] != y->layout.rows[t] || x->layout.cols[t] != y->layout.cols[t])
            fail(NBO_ERR_SHAPE, std::string("nabla: ") + op + " (" + std::to_string(x->layout.rows[t]) + "x" +
                                    std::to_string(x->layout.cols[t]) + ") vs (" +
                                    std::to_string(y->layout.rows[t]) + "x" +
                                    std::to_string(y->layout.cols[t]) + ") -- shapes must match (tensor " +
                                    std::to_string(t) + ")");
}

static_assert((int)NBO_BACKEND_SCALE == (int)NBO_EW_SCALE && (int)NBO_BACKEND_AXPY == (int)NBO_EW_AXPY &&
                  (int)NBO_BACKEND_ADD == (int)NBO_EW_ADD && (int)NBO_BACKEND_EMUL == (int)NBO_EW_EMUL &&
                  (int)NBO_BACKEND_EDIV == (int)NBO_EW_EDIV && (int)NBO_BACKEND_POWF == (int)NBO_EW_POWF &&
                  (int)NBO_BACKEND_ADD_SCALAR == (int)NBO_EW_ADD_SCALAR &&
                  (int)NBO_BACKEND_ZEROS == (int)NBO_EW_ZEROS && (int)NBO_BACKEND_CLONE == (int)NBO_EW_COPY,
              "public operation codes and the kernels' must agree");

int nbo_backend_apply(int op, nbo_list *out, nbo_list *a, nbo_list *b, double s)
{
    return guarded([&] {
        static const char *const names[NBO_EW_COUNT] = {"scale", "axpy_inplace", "add",   "emul", "ediv",
                                                        "powf",  "map",          "zeros", "clone_storage"};
        require(op >= 0 && op < (int)NBO_EW_COUNT, NBO_ERR_ARG, "unknown backend operation");
        require(out != nullptr, NBO_ERR_ARG, "null output list");
        const bool needs_a = op != NBO_EW_ZEROS;
        const bool needs_b = op == NBO_EW_ADD || op == NBO_EW_EMUL || op == NBO_EW_EDIV;
        require(!needs_a || a != nullptr, NBO_ERR_ARG, "null operand list");
        require(!needs_b || b != nullptr, NBO_ERR_ARG, "null second operand list");
        if (needs_a) {
            require_same_shapes(out, a, names[op]);
            require(a->dtype == out->dtype, NBO_ERR_DTYPE, "operand and output differ in element type");
        }
        if (needs_b) {
            require_same_shapes(out, b, names[op]);
            require(b->dtype == out->dtype, NBO_ERR_DTYPE, "operands differ in element type");
        }
        NboEwArgs e = {};
        e.L = out->layout.dev;
        e.out_ptrs = out->ptrs_dev;
        e.a_ptrs = needs_a ? a->ptrs_dev : nullptr;
        e.b_ptrs = needs_b ? b->ptrs_dev : nullptr;
        e.s = s;
        e.op = (uint32_t)op;
        const uint32_t grid = ew_grid(out->layout, out->dtype, NBO_BACKEND_PIECE_BYTES, &e.by_chunk);
        Runtime::get().launch_folded(kernel_for(K_EW_BASE, K_EW_F16, out->dtype), grid, NBO_BLOCK, e);
    });
}

int nbo_backend_cast(nbo_list *dst, nbo_list *src)
{
    return guarded([&] {
        require(dst && src, NBO_ERR_ARG, "null list");
        require_same_shapes(dst, src, "cast");
        NboCastListArgs c = {};
        c.L = dst->layout.dev;
        c.dst_ptrs = dst->ptrs_dev;
        c.src_ptrs = src->ptrs_dev;
        c.dst_type = (uint32_t)dst->dtype;
        c.src_type = (uint32_t)src->dtype;
        c.by_chunk = dst->layout.mostly_whole() ? 0u : 1u;
        const uint64_t rows = (uint64_t)dst->layout.nchunks * (c.by_chunk ? 1u : NBO_CHUNK / NBO_CAST_ROW);
        require(rows <= 0xFFFFFFFFull, NBO_ERR_TOO_LARGE, "list too large for one launch");
        Runtime::get().launch_folded(K_CAST_LIST, (uint32_t)rows, NBO_BLOCK, c);
    });
}

int nbo_optim_last_step(nbo_optim *opt, nbo_step_info *out)
{
    return guarded([&] {
        require(opt && out, NBO_ERR_ARG, "null optimizer or output");
        std::memset(out, 0, sizeof(*out));
        Runtime &rt = Runtime::get();
        uint64_t count = 0;
        rt.read_back(&count, &opt->trace->count, sizeof(count));
        if (count == 0) return;
        NboTraceEntry e;
        rt.read_back(&e, &opt->trace->e[(count - 1) % NBO_TRACE_LEN], sizeof(e));
        fill_info(e, out);
    });
}

int nbo_optim_trace_read(nbo_optim *opt, nbo_step_info *out, uint64_t max_entries, uint64_t *n_out,
                         uint64_t *total)
{
    return guarded([&] {
        require(opt && n_out, NBO_ERR_ARG, "null optimizer or output");
        require(out || max_entries == 0, NBO_ERR_ARG, "null entry buffer");
        NboTraceDev *t = (NboTraceDev *)std::malloc(sizeof(NboTraceDev));
        require(t != nullptr, NBO_ERR_ARG, "host allocation failed");
        try {
            Runtime::get().read_back(t, opt->trace, sizeof(NboTraceDev));
        } catch (...) {
            std::free(t);
            throw;
        }
        uint64_t have = t->count < NBO_TRACE_LEN ? t->count : NBO_TRACE_LEN;
        if (have > max_entries) have = max_entries;
        for (uint64_t k = 0; k < have; k++)
            fill_info(t->e[(t->count - have + k) % NBO_TRACE_LEN], &out[k]);
        *n_out = have;
        if (total) *total = t->count;
        std::free(t);
    });
}

// ---- checkpoint tensor files -------------------------------------------------------------------

int nbo_nbla_save_list(const char *path, nbo_list *list, const char *const *names)
{
    return guarded([&] {
        require(list != nullptr, NBO_ERR_ARG, "null list");
        nbla_save_list(path, list, names);
    });
}

int nbo_nbla_load_list(const char *path, nbo_list *list, const char *const *names)
{
    return guarded([&] {
        require(list != nullptr, NBO_ERR_ARG, "null list");
        nbla_load_list(path, list, names);
    });
}

int nbo_optim_save_state(nbo_optim *opt, const char *path)
{
    return guarded([&] {
        require(opt != nullptr, NBO_ERR_ARG, "null optimizer");
        optim_save_state(opt, path);
    });
}

int nbo_optim_load_state(nbo_optim *opt, const char *path)
{
    return guarded([&] {
        require(opt != nullptr, NBO_ERR_ARG, "null optimizer");
        optim_load_state(opt, path);
    });
}

int nbo_optim_save_master(nbo_optim *opt, const char *path, const char *const *names)
{
    return guarded([&] {
        require(opt != nullptr && path != nullptr, NBO_ERR_ARG, "null optimizer or path");
        optim_save_master(opt, path, names);
    });
}

int nbo_optim_load_master(nbo_optim *opt, const char *path, const char *const *names)
{
    return guarded([&] {
        require(opt != nullptr && path != nullptr, NBO_ERR_ARG, "null optimizer or path");
        optim_load_master(opt, path, names);
    });
}

static void require_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path)
{
    require(path != nullptr, NBO_ERR_ARG, "null path");
    require(n_groups == 0 || opts != nullptr, NBO_ERR_ARG, "null group array");
    for (uint64_t g = 0; g < n_groups; g++) require(opts[g] != nullptr, NBO_ERR_ARG, "null optimizer");
}

int nbo_optim_save_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path)
{
    return guarded([&] {
        require_groups(n_groups, opts, path);
        optim_save_state_groups(n_groups, opts, path);
    });
}

int nbo_optim_load_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path)
{
    return guarded([&] {
        require_groups(n_groups, opts, path);
        optim_load_state_groups(n_groups, opts, path);
    });
}

int nbo_optim_save_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                                 uint64_t n_params, const uint32_t *group_of, const uint32_t *index_in_group,
                                 const char *const *names, const char *path)
{
    return guarded([&] {
        require_groups(n_groups, opts, path);
        require(n_groups == 0 || params != nullptr, NBO_ERR_ARG, "null list array");
        optim_save_params_groups(n_groups, opts, params, n_params, group_of, index_in_group, names, path);
    });
}

int nbo_optim_load_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params,
                                 uint64_t n_params, const uint32_t *group_of, const uint32_t *index_in_group,
                                 const char *const *names, const char *path)
{
    return guarded([&] {
        require_groups(n_groups, opts, path);
        require(n_groups == 0 || params != nullptr, NBO_ERR_ARG, "null list array");
        optim_load_params_groups(n_groups, opts, params, n_params, group_of, index_in_group, names, path);
    });
}

} // extern "C"
