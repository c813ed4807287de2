// extern "C" entry points of include/nabla_optim_bench.h: timing of the library's launches and
// the memory-system probes.  Nothing an optimizer step calls is in this file.
#include <cstring>
#include <string>
#include <vector>

#include "../../../include/nabla_optim_bench.h"
#include "nbo_api_guard.hpp"
#include "nbo_host.hpp"

using namespace nbo;

namespace {

// streams read, rewritten in place, written -- per nbo_probe_pattern
const int kStreams[NBO_PROBE_COUNT][3] = {{1, 0, 0}, {3, 0, 0}, {0, 0, 1}, {0, 0, 3}, {1, 0, 1},
                                          {0, 1, 0}, {0, 2, 0}, {0, 3, 0}, {0, 6, 0}, {1, 3, 1}};
const char *const kPatternKernel[NBO_PROBE_COUNT] = {
    "nbo_probe_read1", "nbo_probe_read3", "nbo_probe_fill1", "nbo_probe_fill3", "nbo_probe_copy",
    "nbo_probe_rmw1",  "nbo_probe_rmw2s", "nbo_probe_rmw3",  "nbo_probe_rmw6",  "nbo_probe_r1_rmw3_w1"};
static_assert((int)NBO_PATTERN_READ1 == (int)NBO_PROBE_READ1 && (int)NBO_PATTERN_COPY == (int)NBO_PROBE_COPY &&
                  (int)NBO_PATTERN_RMW3 == (int)NBO_PROBE_RMW3 &&
                  (int)NBO_PATTERN_R1_RMW3_W1 == (int)NBO_PROBE_R1_RMW3_W1 &&
                  (int)NBO_PATTERN_R1_RMW3_W1 + 1 == (int)NBO_PROBE_COUNT,
              "public pattern codes and the kernels' must agree");

// Launch geometry of one (pattern, shape) kernel of nbo_bench_kernels.hip.
struct ShapeGeometry {
    uint32_t block;       // threads per workgroup
    uint32_t window_vecs; // 128-bit vectors of every stream one window covers
    uint32_t iters;       // windows per workgroup
};

// Index of the pattern among the four that have every shape, or -1.
int full_pattern_index(int pattern)
{
    switch (pattern) {
    case NBO_PATTERN_COPY: return 0;
    case NBO_PATTERN_RMW1: return 1;
    case NBO_PATTERN_RMW3: return 2;
    case NBO_PATTERN_R1_RMW3_W1: return 3;
    default: return -1;
    }
}

ShapeGeometry geometry(int pattern, int shape)
{
    // LDS rows of shapes 3 and 4 and rows per half of shape 6, for copy, rmw1, rmw3, r1_rmw3_w1:
    // what 64 KiB / 128-144 KiB of LDS hold at 4 KiB per row and loaded stream
    static const uint32_t lds_rows[4] = {16, 16, 5, 4}, lds_deep_rows[4] = {32, 32, 12, 8},
                          split_rows[4] = {8, 8, 4, 4}, pipe_rows[4] = {8, 8, 4, 4};
    const int fp = full_pattern_index(pattern);
    switch (shape) {
    case NBO_SHAPE_UPDATE: return {256, 256 * 8, 1};
    case NBO_SHAPE_WG512: return {512, 512 * 8, 1};
    case NBO_SHAPE_WG1024: return {1024, 1024 * 4, 1};
    case NBO_SHAPE_LDS: return {256, 256 * lds_rows[fp], 1};
    case NBO_SHAPE_LDS_DEEP: return {256, 256 * lds_deep_rows[fp], 1};
    case NBO_SHAPE_REGS_LDS: return {256, 256 * (8 + lds_rows[fp]), 1};
    case NBO_SHAPE_SPLIT: return {512, 256 * split_rows[fp], 8};
    case NBO_SHAPE_PIPELINED: return {256, 256 * 4, 8};
    case NBO_SHAPE_LOOP: return {256, 256 * 8, 8};
    case NBO_SHAPE_LDS_PIPELINED: return {256, 256 * pipe_rows[fp], 8};
    case NBO_SHAPE_LDS_PIPELINED_WG512: return {512, 512 * pipe_rows[fp], 8};
    case NBO_SHAPE_LDS_PIPELINED_DEEP: return {256, 256 * 2 * pipe_rows[fp], 8};
    // the front shapes' workgroups cover F windows of 8 / F rows; "iters" = F makes the grid come out right
    case NBO_SHAPE_FRONTS2: return {256, 256 * 4, 2};
    case NBO_SHAPE_FRONTS4: return {256, 256 * 2, 4};
    case NBO_SHAPE_FRONTS8: return {256, 256 * 1, 8};
    case NBO_SHAPE_ROWS4: return {256, 256 * 4, 1};
    case NBO_SHAPE_ROWS2: return {256, 256 * 2, 1};
    default: return {256, 256 * 1, 1}; // NBO_SHAPE_ROWS1
    }
}

// One shape of a comparison: its kernel and launch geometry over streams of nvec vectors.
struct ShapeRun {
    int kernel;
    ShapeGeometry geo;
    uint32_t grid;
    uint32_t contiguous;
    uint64_t covered_vecs;
};

ShapeRun shape_run(Runtime &rt, int pattern, int shape, uint32_t iters_override, uint64_t nvec)
{
    require(shape >= 0 && shape < (int)NBO_SHAPE_COUNT, NBO_ERR_ARG, "unknown probe shape");
    require(shape == NBO_SHAPE_UPDATE || full_pattern_index(pattern) >= 0, NBO_ERR_ARG,
            "this shape exists for the copy, rmw1, rmw3 and r1_rmw3_w1 patterns only");
    ShapeRun r;
    r.geo = geometry(pattern, shape);
    const bool fronts = shape >= NBO_SHAPE_FRONTS2 && shape <= NBO_SHAPE_FRONTS8; // their count is compiled in
    r.contiguous = (iters_override & 0x80000000u) ? 1u : 0u;
    iters_override &= 0x7FFFFFFFu;
    if (iters_override && r.geo.iters > 1 && !fronts) r.geo.iters = iters_override; // only the looping shapes have a choice
    // whole windows only, and a whole number of them per workgroup: what is left over at the end
    // of the streams is not touched, so no access leaves [0, bytes_per_stream) of any stream
    const uint64_t grid64 = nvec / r.geo.window_vecs / r.geo.iters;
    require(grid64 >= 1 && grid64 <= 0x7FFFFFFFull, NBO_ERR_ARG,
            "bytes per stream too small (or too large) for this shape");
    r.grid = (uint32_t)grid64;
    r.covered_vecs = (uint64_t)r.grid * r.geo.iters * r.geo.window_vecs;
    std::string kname = kPatternKernel[pattern];
    if (shape != NBO_SHAPE_UPDATE) kname += "_s" + std::to_string(shape);
    r.kernel = rt.bench_kernel(kname.c_str());
    return r;
}

// `rounds` times over all shapes in turn, each `reps` timed launches on the same buffers: what
// differs between two shapes' figures is then the shape, not the placement or the moment.
void hbm_ceiling(int pattern, int n_shapes, const int *shapes, const uint32_t *iters, int spread,
                 uint64_t bytes_per_stream, int rounds, int reps, uint32_t settle_ms, double *best_gbps,
                 double *mean_gbps, int *regions, uint64_t *mismatches)
{
    require(pattern >= 0 && pattern < (int)NBO_PROBE_COUNT, NBO_ERR_ARG, "unknown probe pattern");
    require(n_shapes >= 1 && n_shapes <= 64 && shapes, NBO_ERR_ARG, "1 to 64 shapes");
    require(best_gbps && mean_gbps, NBO_ERR_ARG, "null output");
    require(reps >= 1 && reps <= 1000 && rounds >= 1 && rounds <= 1000, NBO_ERR_ARG, "1 to 1000 repetitions");
    require(settle_ms <= 60000, NBO_ERR_ARG, "at most 60 s of untimed launches");
    require(bytes_per_stream >= 32768 && bytes_per_stream % 32768 == 0 && bytes_per_stream / 32768 <= 0x7FFFFFFFull,
            NBO_ERR_ARG, "bytes per stream: a multiple of 32 KiB, at most 2^31 - 1 of them");
    require(!mismatches || n_shapes == 1, NBO_ERR_ARG, "the contents check takes one shape at a time");
    const uint64_t nvec = bytes_per_stream / 16;
    Runtime &rt = Runtime::get();
    std::vector<ShapeRun> runs;
    for (int k = 0; k < n_shapes; k++) runs.push_back(shape_run(rt, pattern, shapes[k], iters ? iters[k] : 0, nvec));
    const int ro = kStreams[pattern][0], rmw = kStreams[pattern][1], wo = kStreams[pattern][2];
    const uint32_t ns = (uint32_t)(ro + rmw + wo);
    // Streams are equal slices of up to three arrays.  spread: the arrays come from the
    // region-aware placement the optimizer state uses, stream s lies in array s mod 3, so
    // neighbouring streams sit in different HBM regions at every offset.  Otherwise one plain
    // allocation holds all streams back to back.
    StatePlacement place;
    void *part[3] = {nullptr, nullptr, nullptr};
    const uint32_t nparts = spread ? (ns < 3 ? ns : 3) : 1;
    const uint32_t per_part = (ns + nparts - 1) / nparts;
    const size_t part_bytes = (size_t)per_part * bytes_per_stream;
    if (spread) {
        place.allocate(nparts, part_bytes, part);
    } else {
        part[0] = rt.dmalloc(part_bytes);
    }
    try {
        for (uint32_t k = 0; k < nparts; k++) rt.dzero(part[k], part_bytes);
        NboStreamProbeArgs a = {};
        for (uint32_t s = 0; s < ns; s++) a.buf[s] = (char *)part[s % nparts] + (size_t)(s / nparts) * bytes_per_stream;
        if (mismatches)
            for (int s = ro; s < ro + rmw; s++) rt.launch_fill_index(a.buf[s], nvec);
        std::vector<double> best(n_shapes, 0.0), sum(n_shapes, 0.0);
        uint64_t launches = 0;
        for (int round = 0; round < rounds; round++)
            for (int k = 0; k < n_shapes; k++) {
                a.iters = runs[k].geo.iters;
                a.contiguous = runs[k].contiguous;
                double b = 0.0, m = 0.0;
                // the first measurement waits out the driver's clearing of what was freed before;
                // later ones only need one untimed launch of the new kernel
                launches += rt.time_launches(runs[k].kernel, runs[k].grid, runs[k].geo.block, &a, reps,
                                             round == 0 && k == 0 ? settle_ms : 0, &b, &m);
                sum[k] += m;
                if (best[k] == 0.0 || b < best[k]) best[k] = b;
            }
        for (int k = 0; k < n_shapes; k++) {
            const double moved = (double)(ro + 2 * rmw + wo) * (double)runs[k].covered_vecs * 16.0;
            const double mean_ms = sum[k] / rounds;
            best_gbps[k] = best[k] > 0.0 ? moved / best[k] / 1e6 : 0.0;
            mean_gbps[k] = mean_ms > 0.0 ? moved / mean_ms / 1e6 : 0.0;
        }
        if (regions) *regions = spread ? place.regions_used() : 0;
        if (mismatches) {
            // float i of an in-place stream started as i mod 1024 and has gained 1.0 per launch
            // inside the covered part
            uint64_t bad = 0;
            std::vector<float> host(1u << 20);
            const uint64_t nfloat = bytes_per_stream / 4, covered = runs[0].covered_vecs * 4;
            for (int s = ro; s < ro + rmw; s++)
                for (uint64_t off = 0; off < nfloat; off += host.size()) {
                    const uint64_t n = nfloat - off < host.size() ? nfloat - off : host.size();
                    rt.read_back(host.data(), (const char *)a.buf[s] + off * 4, n * 4);
                    for (uint64_t i = 0; i < n; i++)
                        bad += host[i] != (float)((off + i) & 1023u) + (off + i < covered ? (float)launches : 0.0f);
                }
            *mismatches = bad;
        }
    } catch (...) {
        if (!spread) rt.dfree(part[0]);
        throw;
    }
    rt.sync();
    if (!spread) rt.dfree(part[0]);
}

} // namespace

extern "C" {

int nbo_copy_bytes(const void *src_dev, void *dst_dev, uint64_t bytes)
{
    return guarded([&] {
        require(src_dev && dst_dev, NBO_ERR_ARG, "null address");
        require(bytes % 16 == 0 && ((uintptr_t)src_dev % 16) == 0 && ((uintptr_t)dst_dev % 16) == 0, NBO_ERR_ARG,
                "copy needs 16-byte aligned addresses and size");
        Runtime::get().launch_copy(src_dev, dst_dev, bytes / 16);
    });
}

int nbo_selftest_half_arith(int half_type, uint64_t *div_mismatches, uint64_t *sqrt_mismatches, uint64_t *example_pair,
                            uint64_t *example_arg)
{
    return guarded([&] {
        require(div_mismatches && sqrt_mismatches, NBO_ERR_ARG, "null output");
        require(half_type == NBO_DT_BF16 || half_type == NBO_DT_F16, NBO_ERR_DTYPE, "bf16 or f16");
        Runtime &rt = Runtime::get();
        unsigned long long *out = (unsigned long long *)rt.dmalloc(4 * sizeof(unsigned long long));
        try {
            rt.dzero(out, 4 * sizeof(unsigned long long));
            NboSelftestArgs a = {out};
            rt.launch(half_type == NBO_DT_BF16 ? K_SELFTEST_BF16 : K_SELFTEST_F16, 65536, NBO_BLOCK, a);
            unsigned long long r[4];
            rt.read_back(r, out, sizeof(r));
            *div_mismatches = r[0];
            *sqrt_mismatches = r[1];
            if (example_pair) *example_pair = r[2];
            if (example_arg) *example_arg = r[3];
        } catch (...) {
            rt.dfree(out);
            throw;
        }
        rt.dfree(out);
    });
}

int nbo_hbm_ceiling(int pattern, int spread, uint64_t bytes_per_stream, int reps, uint32_t settle_ms,
                    double *best_gbps, double *mean_gbps, int *regions)
{
    return guarded([&] {
        const int shape = NBO_SHAPE_UPDATE;
        hbm_ceiling(pattern, 1, &shape, nullptr, spread, bytes_per_stream, 1, reps, settle_ms, best_gbps, mean_gbps,
                    regions, nullptr);
    });
}

int nbo_hbm_ceiling_shape(int pattern, int shape, int spread, uint64_t bytes_per_stream, int reps,
                          uint32_t settle_ms, double *best_gbps, double *mean_gbps, int *regions,
                          uint64_t *mismatches)
{
    return guarded([&] {
        hbm_ceiling(pattern, 1, &shape, nullptr, spread, bytes_per_stream, 1, reps, settle_ms, best_gbps, mean_gbps,
                    regions, mismatches);
    });
}

int nbo_hbm_ceiling_compare(int pattern, int n_shapes, const int *shapes, const uint32_t *iters, int spread,
                            uint64_t bytes_per_stream, int rounds, int reps, uint32_t settle_ms,
                            double *best_gbps, double *mean_gbps, int *regions)
{
    return guarded([&] {
        hbm_ceiling(pattern, n_shapes, shapes, iters, spread, bytes_per_stream, rounds, reps, settle_ms, best_gbps,
                    mean_gbps, regions, nullptr);
    });
}

// ---- the caller's own tensors in named HBM regions (a measurement, see the header) ------------

int nbo_alloc_placed(uint32_t n_buffers, uint64_t bytes, const int *region, void **out_ptrs, nbo_placed **out)
{
    return guarded([&] {
        require(out != nullptr, NBO_ERR_ARG, "null output pointer");
        *out = nullptr;
        require(n_buffers >= 2 && n_buffers <= 3 && region && out_ptrs, NBO_ERR_ARG,
                "two or three buffers, with a region number each");
        bool rotate = true; // every region number -1: the rotation the optimizer's own state gets
        for (uint32_t k = 0; k < n_buffers; k++) rotate = rotate && region[k] == -1;
        for (uint32_t k = 0; k < n_buffers && !rotate; k++)
            require(region[k] >= 0 && region[k] < 3, NBO_ERR_ARG, "region numbers are 0, 1 or 2 (or -1 for all buffers)");
        require(bytes > 0, NBO_ERR_ARG, "zero-sized buffers");
        Runtime::get(); // the probe kernel lives in the runtime's code object
        nbo_placed *p = new nbo_placed();
        void *ptrs[3] = {nullptr, nullptr, nullptr};
        bool placed = false;
        try {
            if (rotate) {
                p->placement.allocate(n_buffers, (size_t)bytes, ptrs);
                placed = p->placement.regions_used() >= 2;
            } else {
                placed = p->placement.allocate_whole(n_buffers, (size_t)bytes, region, ptrs);
            }
        } catch (...) {
            delete p;
            throw;
        }
        if (!placed) {
            const std::string why = p->placement.note();
            delete p;
            fail(NBO_ERR_TOO_LARGE, "nbo_alloc_placed: " + why);
        }
        for (uint32_t k = 0; k < n_buffers; k++) out_ptrs[k] = ptrs[k];
        *out = p;
    });
}

int nbo_free_placed(nbo_placed *p)
{
    return guarded([&] {
        if (!p) return;
        Runtime::get().sync();
        delete p; // ~StatePlacement unmaps and releases
    });
}

int nbo_placed_note(nbo_placed *p, char *buf, uint64_t buf_bytes)
{
    return guarded([&] {
        require(p && buf && buf_bytes > 0, NBO_ERR_ARG, "null handle or buffer");
        const std::string &n = p->placement.note();
        const size_t k = n.size() < buf_bytes - 1 ? n.size() : (size_t)(buf_bytes - 1);
        std::memcpy(buf, n.data(), k);
        buf[k] = '\0';
    });
}

int nbo_profile_enable(int on)
{
    return guarded([&] { Runtime::get().profile_enable(on != 0); });
}

int nbo_profile_read(const char *kernel_name, uint64_t *launches, double *total_ms)
{
    return guarded([&] {
        require(kernel_name && launches && total_ms, NBO_ERR_ARG, "null argument");
        Runtime::get().profile_read(kernel_name, launches, total_ms);
    });
}

} // extern "C"
