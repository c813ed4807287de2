// Region-aware placement of the optimizer's state arrays (see nbo_placement.hpp).
#include "nbo_placement.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "nbo_host.hpp"

namespace nbo {

namespace {

constexpr size_t kGiB = (size_t)1 << 30;
constexpr size_t kMapGranule = (size_t)2 << 20;
// Two buffers of 1-2 GiB read-modify-written together run at 5.0-5.9 TB/s when both
// lie in the same 96 GiB region of MI355X's HBM and at 6.3-6.5 TB/s when they do not.
constexpr double kSameRegionBelowGBps = 6100.0;
// Below this size per part the step is too short for placement to matter.
constexpr size_t kMinPlacedBytes = (size_t)128 << 20;

size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

bool ok(hipError_t e)
{
    if (e == hipSuccess) return true;
    (void)hipGetLastError();
    return false;
}

hipMemAllocationProp device_prop()
{
    hipMemAllocationProp prop = {};
    prop.type = hipMemAllocationTypePinned;
    prop.location.type = hipMemLocationTypeDevice;
    prop.location.id = 0;
    return prop;
}

bool set_rw(void *va, size_t size)
{
    hipMemAccessDesc acc = {};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = 0;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    return ok(hipMemSetAccess(va, size, &acc, 1));
}

} // namespace

void StatePlacement::release()
{
    for (const Range &r : ranges_) {
        (void)hipMemUnmap(r.va, r.size);
        (void)hipMemAddressFree(r.va, r.size);
    }
    ranges_.clear();
    for (hipMemGenericAllocationHandle_t h : handles_) (void)hipMemRelease(h);
    handles_.clear();
    for (void *p : plain_) (void)hipFree(p);
    plain_.clear();
    (void)hipGetLastError();
    regions_used_ = 0;
}

void StatePlacement::allocate(uint32_t nparts, size_t bytes, void **out)
{
    release();
    for (uint32_t k = 0; k < 3; k++) out[k] = nullptr;
    const char *env = std::getenv("NBO_STATE_SPREAD");
    const bool spread = !(env && env[0] == '0');
    if (spread && nparts > 1 && bytes >= kMinPlacedBytes && try_placed(nparts, bytes, out)) return;
    Runtime &rt = Runtime::get();
    try {
        for (uint32_t k = 0; k < nparts; k++) {
            plain_.push_back(rt.dmalloc(bytes));
            out[k] = plain_.back();
        }
    } catch (...) {
        release();
        throw;
    }
}

bool StatePlacement::try_placed(uint32_t nparts, size_t bytes, void **out)
{
    Runtime &rt = Runtime::get();
    const size_t chunk = bytes >= 16 * kGiB ? 2 * kGiB : kGiB;
    const size_t window = chunk; // probe size: whole chunks against each other
    // a part smaller than one chunk still gets a whole chunk of its own (regions can
    // only be told apart at this granularity); larger parts are whole chunks plus a tail
    const size_t full = bytes < chunk ? 1 : bytes / chunk;
    const size_t tail = bytes < chunk ? 0 : round_up(bytes - full * chunk, kMapGranule);
    const size_t part_va = full * chunk + tail;
    const size_t total_full = full * nparts;
    size_t free_b = 0, total_b = 0;
    if (!ok(hipMemGetInfo(&free_b, &total_b))) return false;
    const size_t reserve = 2 * kGiB;
    if (free_b < reserve + nparts * part_va) return false; // let hipMalloc report the shortage
    const size_t budget = (free_b - reserve - nparts * tail) / chunk;
    if (budget < total_full) return false;

    const char *dbg = std::getenv("NBO_PLACEMENT_DEBUG");
    const int debug = dbg ? std::atoi(dbg) : 0;
    const hipMemAllocationProp prop = device_prop();
    // everything created below is tracked here and torn down unless `keep` says otherwise
    struct Chunk {
        hipMemGenericAllocationHandle_t h;
        bool mapped_in_staging;
        bool keep;
    };
    std::vector<Chunk> chunks;
    void *staging = nullptr;
    const size_t staging_size = budget * chunk;
    struct PartRange {
        void *va;
        size_t mapped; // bytes mapped so far, from the start of the range
    };
    std::vector<PartRange> part_ranges;
    std::vector<hipMemGenericAllocationHandle_t> tails;
    bool success = false;

    auto cleanup = [&]() {
        for (size_t i = 0; i < chunks.size(); i++) {
            if (chunks[i].mapped_in_staging) (void)hipMemUnmap((char *)staging + i * chunk, chunk);
            if (!(success && chunks[i].keep)) (void)hipMemRelease(chunks[i].h);
        }
        if (staging) (void)hipMemAddressFree(staging, staging_size);
        if (!success) {
            for (const PartRange &r : part_ranges) {
                if (r.mapped) (void)hipMemUnmap(r.va, r.mapped);
                (void)hipMemAddressFree(r.va, part_va);
            }
            for (hipMemGenericAllocationHandle_t h : tails) (void)hipMemRelease(h);
        }
        (void)hipGetLastError();
    };

    try {
        if (!ok(hipMemAddressReserve(&staging, staging_size, 0, nullptr, 0))) {
            staging = nullptr;
            cleanup();
            return false;
        }
        std::vector<std::vector<size_t>> region_chunks; // chunk indices per region
        std::vector<char *> region_rep;                 // one mapped chunk per region
        // Which regions the parts will use.  Three parts rotate over all three regions.
        // Two parts use the two regions found last: the first region found is where this
        // process's most recent allocations went, and the caller's parameters and
        // gradients -- read and written in the same kernel -- are most likely there.
        const size_t first_used = nparts == 2 ? 1 : 0;
        const size_t need_each = (total_full + (3 - first_used) - 1) / (3 - first_used);
        auto enough = [&]() {
            if (region_chunks.size() < 3) return false;
            for (size_t r = first_used; r < 3; r++)
                if (region_chunks[r].size() < need_each) return false;
            return true;
        };
        while (chunks.size() < budget && !enough()) {
            Chunk c = {};
            if (!ok(hipMemCreate(&c.h, chunk, &prop, 0))) break;
            const size_t idx = chunks.size();
            char *p = (char *)staging + idx * chunk;
            chunks.push_back(c);
            if (!ok(hipMemMap(p, chunk, 0, c.h, 0))) break;
            chunks[idx].mapped_in_staging = true;
            if (!set_rw(p, chunk)) break;
            if (idx == 0) {
                // the two halves of one chunk certainly share a region: the probe must
                // call that pair "same", or it cannot tell anything on this system
                if (rt.probe_pair_gbps(p, p + chunk / 2, chunk / 2) >= kSameRegionBelowGBps) {
                    cleanup();
                    return false;
                }
            }
            int region = -1;
            for (size_t r = 0; r < region_rep.size() && region < 0; r++) {
                const double g = rt.probe_pair_gbps(region_rep[r], p, window);
                if (debug > 1) std::fprintf(stderr, "[nbo placement] chunk %zu vs region %zu: %.0f GB/s\n", idx, r, g);
                if (g < kSameRegionBelowGBps) region = (int)r;
            }
            if (region < 0) {
                if (region_rep.size() == 3) {
                    // a fourth "region" is measurement noise on this part: count the chunk
                    // to the smallest region rather than trusting it
                    region = 0;
                    for (size_t r = 1; r < 3; r++)
                        if (region_chunks[r].size() < region_chunks[region].size()) region = (int)r;
                } else {
                    region_rep.push_back(p);
                    region_chunks.emplace_back();
                    region = (int)region_rep.size() - 1;
                }
            }
            region_chunks[region].push_back(idx);
        }
        size_t have = 0;
        for (const auto &r : region_chunks) have += r.size();
        if (have < total_full) { // ran out of memory before collecting enough chunks
            cleanup();
            return false;
        }
        if (debug) {
            std::fprintf(stderr, "[nbo placement] %zu chunks of %zu MiB created; per region:", chunks.size(), chunk >> 20);
            for (const auto &r : region_chunks) std::fprintf(stderr, " %zu", r.size());
            std::fprintf(stderr, "; %zu needed\n", total_full);
        }
        // chunk i of part j prefers the ((i + j) mod U)-th of the U regions in use; when
        // that one has run dry, whichever region still has most chunks
        const size_t R = region_chunks.size();
        std::vector<size_t> use;
        for (size_t r = (R == 3 ? first_used : 0); r < R; r++) use.push_back(r);
        size_t in_use = 0;
        for (size_t r : use) in_use += region_chunks[r].size();
        if (in_use < total_full) { // not enough there: every region is fair game
            use.clear();
            for (size_t r = 0; r < R; r++) use.push_back(r);
        }
        std::vector<std::vector<size_t>> pick(nparts);
        for (size_t i = 0; i < full; i++)
            for (uint32_t j = 0; j < nparts; j++) {
                size_t r = use[(i + j) % use.size()];
                if (region_chunks[r].empty())
                    for (size_t q : use)
                        if (region_chunks[q].size() > region_chunks[r].size()) r = q;
                pick[j].push_back(region_chunks[r].back());
                region_chunks[r].pop_back();
            }
        // move the chosen chunks from the staging range into the parts' own ranges
        for (uint32_t j = 0; j < nparts; j++) {
            void *va = nullptr;
            if (!ok(hipMemAddressReserve(&va, part_va, 0, nullptr, 0))) {
                cleanup();
                return false;
            }
            part_ranges.push_back({va, 0});
            for (size_t i = 0; i < full; i++) {
                const size_t idx = pick[j][i];
                if (!ok(hipMemUnmap((char *)staging + idx * chunk, chunk))) {
                    cleanup();
                    return false;
                }
                chunks[idx].mapped_in_staging = false;
                if (!ok(hipMemMap((char *)va + i * chunk, chunk, 0, chunks[idx].h, 0))) {
                    cleanup();
                    return false;
                }
                part_ranges.back().mapped = (i + 1) * chunk;
                chunks[idx].keep = true;
            }
            if (tail) {
                hipMemGenericAllocationHandle_t th;
                if (!ok(hipMemCreate(&th, tail, &prop, 0))) {
                    cleanup();
                    return false;
                }
                tails.push_back(th);
                if (!ok(hipMemMap((char *)va + full * chunk, tail, 0, th, 0))) {
                    cleanup();
                    return false;
                }
                part_ranges.back().mapped = part_va;
            }
            if (!set_rw(va, part_va)) {
                cleanup();
                return false;
            }
        }
        success = true;
        regions_used_ = (int)use.size();
        for (uint32_t j = 0; j < nparts; j++) {
            out[j] = part_ranges[j].va;
            ranges_.push_back({part_ranges[j].va, part_va});
        }
        for (const Chunk &c : chunks)
            if (c.keep) handles_.push_back(c.h);
        for (hipMemGenericAllocationHandle_t h : tails) handles_.push_back(h);
        cleanup(); // releases the chunks that were not chosen and the staging range
        return true;
    } catch (...) {
        cleanup();
        return false;
    }
}

} // namespace nbo
