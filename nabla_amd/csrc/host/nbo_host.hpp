// Host runtime of the fused optimizer-step engine: internal classes behind the C ABI
// of include/nabla_optim.h.  Device work goes through hipModuleLaunchKernel on
// kernels of the embedded gfx950 code object and hipMemcpyAsync;
// nothing here computes optimizer arithmetic on the host.
#ifndef NBO_HOST_HPP
#define NBO_HOST_HPP

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <string>
#include <vector>

#include "../../../include/nabla_optim.h"
#include "../nbo_device_types.h"
#include "nbo_placement.hpp"

namespace nbo {

// 16-bit element types: bf16 and IEEE binary16
inline bool is_half(int dtype) { return dtype == NBO_DT_BF16 || dtype == NBO_DT_F16; }
static_assert((int)NBO_DT_F32 == (int)NBO_F32 && (int)NBO_DT_BF16 == (int)NBO_BF16 && (int)NBO_DT_F64 == (int)NBO_F64 &&
                  (int)NBO_DT_F16 == (int)NBO_F16,
              "the public element type codes are the device's storage codes");

// Thrown internally, converted to a status code at the C boundary.
struct Error {
    int status;
    std::string msg;
};

[[noreturn]] void fail(int status, const std::string &msg);
void hip_check(hipError_t e, const char *what);
void set_last_error(const std::string &msg);
const char *get_last_error();

enum KernelId {
    K_UPDATE_BASE = 0, // + st * 3 + kind, st = f32 / bf16 / f64 (f16 has ids of its own below)
    K_NORM_BASE = 9,   // + st
    K_SCALE_BASE = 12, // + st
    K_PREP = 15,
    K_FINALIZE = 16,
    K_CAST_MASTER = 17,
    K_SUM_PARTIALS = 18, // per-piece sums of squares -> at most NBO_NORM_GRID_MAX of them
    K_PROBE = 19,
    K_ACCUM_BASE = 20, // + st
    K_FILL_ZERO = 23,
    K_EW_BASE = 24, // + st
    K_CAST_LIST = 27,
    K_UPDATE_PBF16_BASE = 28, // + kind: bf16 tensors with bf16 state and arithmetic
    K_NORM_PBF16 = 31,
    K_UPDATE_F16_BASE = 32,  // + kind: f16 tensors over f32 state and master weights
    K_UPDATE_PF16_BASE = 35, // + kind: f16 tensors with f16 state and arithmetic
    K_NORM_F16 = 38,
    K_NORM_PF16 = 39,
    K_SCALE_F16 = 40,
    K_ACCUM_F16 = 41,
    K_EW_F16 = 42,
    K_ACCNORM_BASE = 43, // + st (f32 / bf16 / f64)
    K_ACCNORM_F16 = 46,
    // update kernels that prepare their own per-step scalars: + family * 3 + kind, family =
    // f32, bf16, f64, f16, pbf16, pf16
    K_UPDATE_SELF_BASE = 47,
    // Adam / AdamW one workgroup per row of a chunk: + family * 2 + kind (adamw 0, adam 1), family =
    // f32, bf16, f64, f16 (state of 32 or 64 bits)
    K_UPDATE_ROWS_BASE = 65,
    K_ACCSCALE_BASE = 73, // + st (f32 / bf16 / f64): a micro-batch without the sum of squares
    K_ACCSCALE_F16 = 76,
    K_SELFTEST_BF16 = 77,
    K_SELFTEST_F16 = 78,
    K_COUNT = 79 // ids from here on are measurement kernels, handed out by Runtime::bench_kernel
};

// Lists of fewer chunks than this take the Adam kinds' by-row kernels (nbo_capi.cpp has the measurements).
constexpr uint32_t NBO_ROWS_MAX_CHUNKS = 524288;

// Process-wide runtime: device 0, the loaded module, the stream, scratch buffers.
class Runtime {
public:
    static Runtime &get(); // creates on first use; throws Error on failure
    static Runtime *existing(); // the runtime if it has been created, else null; creates nothing
    hipStream_t stream() const { return stream_; }
    void set_stream(hipStream_t s);
    void sync();

    // idle_lds: bytes of LDS every workgroup is given and never touches.  It caps the workgroups
    // a compute unit holds (160 KiB / idle_lds of them): passes that write at least as much as
    // they read run faster with fewer in flight.
    template <typename Args>
    void launch(int kernel, uint32_t grid, uint32_t block, const Args &args, uint32_t idle_lds = 0)
    {
        launch_raw(kernel, grid, block, const_cast<Args *>(&args), true, idle_lds);
    }
    // For the kernels that take their workgroup number from folded_workgroup(): a grid of more
    // than grid_x_max() workgroups is folded into two dimensions (one dimension of a launch holds
    // fewer than 2^32 threads).
    template <typename Args>
    void launch_folded(int kernel, uint32_t grid, uint32_t block, const Args &args, uint32_t idle_lds = 0)
    {
        launch_raw(kernel, grid, block, const_cast<Args *>(&args), true, idle_lds, true);
    }
    // may_time = false: never bracket the launch with timing events, whatever profile_enable
    // says (creating events allocates host memory)
    void launch_raw(int kernel, uint32_t grid, uint32_t block, void *arg_struct, bool may_time = true,
                    uint32_t idle_lds = 0, bool folded = false);
    // 2^24 - 1 workgroups of NBO_BLOCK threads; NBO_GRID_X_MAX in the environment lowers it, so that
    // a test can fold the grids of small lists
    uint32_t grid_x_max() const { return grid_x_max_; }
    // Id of kernel `name` of the measurement code object (nbo_bench_kernels.hip), which is
    // loaded when the first such id is asked for; the id works with launch, time_launches and
    // the per-kernel timing like the ids above.
    int bench_kernel(const char *name);
    void launch_copy(const void *src, void *dst, uint64_t nvec);
    // float i of the nvec 128-bit vectors at dst = i mod 1024 (start contents of a checked probe run)
    void launch_fill_index(void *dst, uint64_t nvec);
    // Bandwidth (GB/s, best of three) of reading and rewriting `bytes` bytes at a and at
    // b together: the probe StatePlacement classifies HBM regions with.  Synchronous.
    double probe_pair_gbps(void *a, void *b, size_t bytes);
    // Untimed launches for `settle_ms` milliseconds (at least one), then `reps` launches each
    // bracketed by events on the stream: shortest and mean duration in ms.  Returns how many
    // launches were made in all.  Synchronous.
    uint64_t time_launches(int kernel, uint32_t grid, uint32_t block, void *arg_struct, int reps, uint32_t settle_ms,
                       double *best_ms, double *mean_ms);

    // synchronous transfers through a double-buffered pinned staging buffer
    void read_back(void *host_dst, const void *dev_src, size_t bytes);
    void upload(void *dev_dst, const void *host_src, size_t bytes);

    void *dmalloc(size_t bytes);
    void dfree(void *p);
    void dzero(void *p, size_t bytes); // a fill kernel, asynchronous on the stream

    // Per-kernel timing with HIP events recorded on the launch stream, for the
    // benchmark's roofline figure.  Off by default.
    void profile_enable(bool on);
    void profile_read(const char *kernel_name, uint64_t *launches, double *total_ms);

    double *partial_sumsq() const { return partial_sumsq_; }
    uint32_t *partial_flag() const { return partial_flag_; }
    NboGradFactors *gf_scratch() const { return gf_scratch_; }
    // one word, zero between uses: passes without partial results OR their non-finite findings into it
    uint32_t *any_bad() const { return any_bad_; }
    // room for `count` per-piece sums of squares; grows (after a synchronisation) when a larger
    // list comes along, never shrinks
    double *piece_partials(size_t count);
    // the device this runtime lives on, and how the look-up of the statically allocated
    // scratch's address went there
    int device() const { return device_; }
    hipError_t static_scratch_status() const { return static_scratch_status_; }

private:
    Runtime();
    hipFunction_t function(int kernel) const;
    const char *kernel_name(int kernel) const;
    hipModule_t module_ = nullptr;
    hipFunction_t fn_[K_COUNT] = {};
    uint32_t grid_x_max_ = 0xFFFFFFu;
    hipModule_t bench_module_ = nullptr; // loaded on first use
    std::vector<std::string> bench_names_;
    std::vector<hipFunction_t> bench_fn_;
    hipStream_t stream_ = nullptr;
    void *pinned_ = nullptr;
    size_t pinned_bytes_ = 0;
    hipEvent_t staged_[2] = {}; // one per half of the staging buffer
    hipEvent_t probe_ev_[2] = {}; // timing of the placement probe
    double *partial_sumsq_ = nullptr;
    uint32_t *partial_flag_ = nullptr;
    NboGradFactors *gf_scratch_ = nullptr;
    uint32_t *any_bad_ = nullptr;
    double *piece_partials_ = nullptr;
    size_t piece_partials_cap_ = 0;
    int device_ = 0;
    hipError_t static_scratch_status_ = hipSuccess;
    struct ProfRec {
        int kernel;
        hipEvent_t begin, end;
    };
    bool profiling_ = false;
    std::vector<ProfRec> prof_;
};

// Host + device copy of the packed tensor-list descriptor.
struct Layout {
    std::vector<uint64_t> rows, cols, n, soff;
    uint64_t arena_elems = 0; // elements an arena needs (with per-tensor alignment)
    uint32_t nchunks = 0;
    uint32_t whole_chunks = 0; // chunks of NBO_CHUNK elements (the others are the ragged ends of tensors)
    void *blob = nullptr; // one device allocation holding all tables
    NboLayoutDev dev = {};

    // row_elems != 0: the elements a by-row update workgroup takes (one vector per thread); a list in
    // which fewer than nine chunks in ten are whole then gets a map of the rows that exist
    // (dev.row_map), so that a by-row launch has a workgroup for every row and none besides
    void build(uint64_t nt, const uint64_t *rows, const uint64_t *cols, bool with_arena, uint32_t row_elems = 0);
    bool mostly_whole() const { return (uint64_t)whole_chunks * 10 >= (uint64_t)nchunks * 9; }
    void release();
    uint64_t nt() const { return n.size(); }
};

} // namespace nbo

struct nbo_list {
    nbo::Layout layout;
    int dtype = NBO_DT_F32;
    std::vector<uint64_t> ptrs;
    uint64_t *ptrs_dev = nullptr;
};

struct nbo_scaler {
    NboScalerDev *dev = nullptr;
};

struct nbo_optim {
    nbo::Layout layout;
    nbo_meta meta = {};    // hyper-parameters: host copy is authoritative
    int state_dtype = NBO_DT_F32;
    bool keep_master = false;
    bool master_valid = false;
    nbo::StatePlacement placement; // owns the memory behind arena.part[]
    NboArenaDev arena = {};        // m, v and master
    NboOptimDev *dev = nullptr; // step_count lives here: the device decides skips
    NboGradFactors *gf = nullptr;
    NboTraceDev *trace = nullptr;
    size_t elem_bytes() const { return state_dtype == NBO_DT_F64 ? 8 : nbo::is_half(state_dtype) ? 2 : 4; }
};

// Buffers handed out by nbo_alloc_placed: whole arrays in named HBM regions.
struct nbo_placed {
    nbo::StatePlacement placement;
};

namespace nbo {
// NBLA tensor files (nbo_nbla.cpp)
void nbla_save_list(const char *path, const nbo_list *list, const char *const *names);
void nbla_load_list(const char *path, nbo_list *list, const char *const *names);
void optim_save_state(const nbo_optim *opt, const char *path);
void optim_load_state(nbo_optim *opt, const char *path);
void optim_save_master(const nbo_optim *opt, const char *path, const char *const *names);
void optim_load_master(nbo_optim *opt, const char *path, const char *const *names);
void optim_save_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path);
void optim_load_state_groups(uint64_t n_groups, nbo_optim *const *opts, const char *path);
void optim_save_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params, uint64_t n_params,
                              const uint32_t *group_of, const uint32_t *index_in_group, const char *const *names,
                              const char *path);
void optim_load_params_groups(uint64_t n_groups, nbo_optim *const *opts, nbo_list *const *params, uint64_t n_params,
                              const uint32_t *group_of, const uint32_t *index_in_group, const char *const *names,
                              const char *path);
} // namespace nbo

#endif
