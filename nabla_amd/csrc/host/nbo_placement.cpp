// Region-aware placement of the optimizer's state arrays (see nbo_placement.hpp).
#include "nbo_placement.hpp"

#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "nbo_host.hpp"
#include "nbo_placement_plan.hpp"

namespace nbo {

namespace {

constexpr size_t kGiB = (size_t)1 << 30;
constexpr size_t kMapGranule = (size_t)2 << 20;
// Memory left alone while chunks are being created.
constexpr size_t kReserveBytes = (size_t)2 << 30;
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

namespace {
std::string fmt(const char *f, double a = 0, double b = 0, double c = 0, double d = 0)
{
    char buf[256];
    std::snprintf(buf, sizeof(buf), f, a, b, c, d);
    return buf;
}
} // namespace

void StatePlacement::allocate(uint32_t nparts, size_t bytes, void **out)
{
    release();
    note_.clear();
    for (uint32_t k = 0; k < 3; k++) out[k] = nullptr;
    const char *env = std::getenv("NBO_STATE_SPREAD");
    const bool spread = !(env && env[0] == '0');
    if (!spread) note_ = "plain allocations: NBO_STATE_SPREAD=0";
    else if (nparts < 2) note_ = "plain allocation: a single state array has nothing to be spread against";
    else if (bytes < kMinPlacedBytes) note_ = "plain allocations: less than 128 MiB per state array";
    else if (try_placed(nparts, bytes, out)) return;
    if (std::getenv("NBO_PLACEMENT_DEBUG")) std::fprintf(stderr, "[nbo placement] %s\n", note_.c_str());
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

bool StatePlacement::allocate_whole(uint32_t nparts, size_t bytes, const int *slot_of, void **out)
{
    release();
    note_.clear();
    for (uint32_t k = 0; k < 3; k++) out[k] = nullptr;
    if (nparts < 2 || nparts > 3) note_ = "two or three arrays can be placed against each other";
    else if (bytes < kMinPlacedBytes) note_ = "less than 128 MiB per array: regions are told apart in chunks of 1 GiB";
    else if (try_placed(nparts, bytes, out, slot_of)) return true;
    if (std::getenv("NBO_PLACEMENT_DEBUG")) std::fprintf(stderr, "[nbo placement] %s\n", note_.c_str());
    return false;
}

bool StatePlacement::try_placed(uint32_t nparts, size_t bytes, void **out, const int *slot_of)
{
    Runtime &rt = Runtime::get();
    // 1 GiB: large enough for a steady probe, small enough that a chunk the driver pieced
    // together from scattered physical memory rarely straddles two regions
    const size_t chunk = kGiB;
    // a part smaller than one chunk still gets a whole chunk of its own (regions can
    // only be told apart at this granularity); larger parts are whole chunks plus a tail
    // (whole arrays in named regions are rounded up to whole chunks: a tail would lie anywhere)
    const size_t full = slot_of ? (bytes + chunk - 1) / chunk : bytes < chunk ? 1 : bytes / chunk;
    const size_t tail = slot_of || bytes < chunk ? 0 : round_up(bytes - full * chunk, kMapGranule);
    const size_t part_va = full * chunk + tail;
    const size_t total_full = full * nparts;
    auto give_up = [&](const std::string &why) {
        note_ = "plain allocations: " + why;
        return false;
    };
    size_t free_b = 0, total_b = 0;
    if (!ok(hipMemGetInfo(&free_b, &total_b))) return give_up("hipMemGetInfo failed");
    if (free_b < kReserveBytes + nparts * part_va) return give_up("not enough free memory to choose chunks from");
    // The search creates at most `cap` chunks (plan::chunk_cap): enough to walk past one region
    // boundary, within half of what is free; NBO_PLACEMENT_MAX_GIB if set.
    size_t user_cap = 0;
    if (const char *e = std::getenv("NBO_PLACEMENT_MAX_GIB")) {
        const double gib = std::atof(e);
        if (gib > 0.0) user_cap = (size_t)(gib * (double)kGiB / (double)chunk);
    }
    const size_t reach = (size_t)104 * kGiB / chunk; // one 96 GiB region and a bit
    const size_t cap = plan::chunk_cap(total_full, (free_b - kReserveBytes - nparts * tail) / chunk, user_cap, reach);
    if (cap < total_full) return give_up("the chunk limit is below what the state arrays need");

    const char *dbg = std::getenv("NBO_PLACEMENT_DEBUG");
    const int debug = dbg ? std::atoi(dbg) : 0;
    const hipMemAllocationProp prop = device_prop();
    // everything created below is tracked here and torn down unless `keep` says otherwise
    struct Chunk {
        hipMemGenericAllocationHandle_t h;
        bool mapped_in_staging;
        bool ready; // mapped and accessible: may be handed to the probe
        bool keep;
    };
    std::vector<Chunk> chunks;
    void *staging = nullptr;
    const size_t staging_size = cap * chunk;
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
    auto fail_with = [&](const std::string &why) {
        cleanup();
        return give_up(why);
    };

    try {
        if (!ok(hipMemAddressReserve(&staging, staging_size, 0, nullptr, 0))) {
            staging = nullptr;
            return fail_with("no virtual address range for the search");
        }
        auto chunk_va = [&](size_t i) { return (char *)staging + i * chunk; };
        // creates and maps chunks until `target` exist; false when the driver refuses one
        auto create_until = [&](size_t target) {
            while (chunks.size() < target) {
                Chunk c = {};
                if (!ok(hipMemCreate(&c.h, chunk, &prop, 0))) return false;
                const size_t idx = chunks.size();
                chunks.push_back(c);
                if (!ok(hipMemMap(chunk_va(idx), chunk, 0, c.h, 0))) return false;
                chunks[idx].mapped_in_staging = true;
                if (!set_rw(chunk_va(idx), chunk)) return false;
                chunks[idx].ready = true;
            }
            return true;
        };
        plan::RegionFinder finder;
        auto probe = [&](size_t a, size_t b) {
            const double g = rt.probe_pair_gbps(chunk_va(a), chunk_va(b), chunk);
            if (debug > 1) std::fprintf(stderr, "[nbo placement] chunk %zu with chunk %zu: %.0f GB/s\n", a, b, g);
            return g;
        };
        // the two halves of one chunk certainly share a region: what "same" measures on this GPU now
        auto halves = [&](size_t a) {
            const double g = rt.probe_pair_gbps(chunk_va(a), chunk_va(a) + chunk / 2, chunk / 2);
            if (debug > 1) std::fprintf(stderr, "[nbo placement] chunk %zu, its two halves: %.0f GB/s\n", a, g);
            return g;
        };
        auto counts = [&]() {
            std::vector<size_t> n;
            for (const auto &r : finder.chunks_per_region()) n.push_back(r.size());
            return n;
        };
        size_t target = std::min(cap, total_full + 2);
        for (;;) {
            const bool created = create_until(target);
            size_t usable = chunks.size();
            if (usable && !chunks.back().ready) usable--; // the driver refused to map it or to open it for access
            finder.add_chunks(usable, probe, halves);
            if (slot_of ? !plan::assign_whole(counts(), std::vector<int>(slot_of, slot_of + nparts), full).empty()
                        : plan::enough(counts(), nparts, full))
                break;
            if (!created || chunks.size() >= cap) break;
            target = std::min(cap, chunks.size() + std::max<size_t>({2, total_full / 4, chunks.size() / 4}));
        }
        std::vector<std::vector<size_t>> region_chunks = finder.chunks_per_region();
        if (debug) {
            std::fprintf(stderr, "[nbo placement] %zu chunks of %zu MiB created (limit %zu), %zu probes, threshold %.0f GB/s; per region:",
                         chunks.size(), chunk >> 20, cap, finder.probes(), finder.threshold());
            for (const auto &r : region_chunks) std::fprintf(stderr, " %zu", r.size());
            std::fprintf(stderr, "; %zu needed\n", total_full);
        }
        const bool one_region_will_do = slot_of && std::all_of(slot_of, slot_of + nparts, [&](int x) { return x == slot_of[0]; });
        if (region_chunks.size() < 2 && !one_region_will_do)
            return fail_with(fmt("%.0f chunks created and probed, all read as one region (two halves of a chunk: %.0f GB/s)",
                                 (double)chunks.size(), finder.same_pair()));
        std::vector<std::vector<int>> pick_region;
        if (slot_of) { // every array wholly in its slot's region
            const std::vector<int> region_of_slot =
                plan::assign_whole(counts(), std::vector<int>(slot_of, slot_of + nparts), full);
            if (!region_of_slot.empty())
                for (uint32_t j = 0; j < nparts; j++)
                    pick_region.push_back(std::vector<int>(full, region_of_slot[(size_t)slot_of[j]]));
        } else {
            pick_region = plan::assign(counts(), nparts, full);
        }
        if (pick_region.empty()) return fail_with("ran out of memory before enough chunks were collected");
        std::vector<std::vector<size_t>> pick(nparts);
        for (uint32_t j = 0; j < nparts; j++)
            for (size_t i = 0; i < full; i++) {
                std::vector<size_t> &pool = region_chunks[(size_t)pick_region[j][i]];
                pick[j].push_back(pool.back());
                pool.pop_back();
            }
        // move the chosen chunks from the staging range into the parts' own ranges
        for (uint32_t j = 0; j < nparts; j++) {
            void *va = nullptr;
            if (!ok(hipMemAddressReserve(&va, part_va, 0, nullptr, 0))) return fail_with("no virtual address range for a state array");
            part_ranges.push_back({va, 0});
            for (size_t i = 0; i < full; i++) {
                const size_t idx = pick[j][i];
                if (!ok(hipMemUnmap(chunk_va(idx), chunk))) return fail_with("hipMemUnmap failed");
                chunks[idx].mapped_in_staging = false;
                if (!ok(hipMemMap((char *)va + i * chunk, chunk, 0, chunks[idx].h, 0))) return fail_with("hipMemMap failed");
                part_ranges.back().mapped = (i + 1) * chunk;
                chunks[idx].keep = true;
            }
            if (tail) {
                hipMemGenericAllocationHandle_t th;
                if (!ok(hipMemCreate(&th, tail, &prop, 0))) return fail_with("the tail of a state array could not be created");
                tails.push_back(th);
                if (!ok(hipMemMap((char *)va + full * chunk, tail, 0, th, 0))) return fail_with("hipMemMap failed");
                part_ranges.back().mapped = part_va;
            }
            if (!set_rw(va, part_va)) return fail_with("hipMemSetAccess failed");
        }
        // Check the finished layout: wherever the plan put two arrays into different regions at
        // the first position, the probe over those two mapped chunks must read "different" again.
        size_t checked = 0;
        for (uint32_t j = 0; j < nparts; j++)
            for (uint32_t k = j + 1; k < nparts; k++) {
                if (pick_region[j][0] == pick_region[k][0]) continue;
                const double g = rt.probe_pair_gbps(part_ranges[j].va, part_ranges[k].va, chunk);
                if (debug > 1) std::fprintf(stderr, "[nbo placement] check, arrays %u and %u: %.0f GB/s\n", j, k, g);
                if (!(g >= finder.threshold()))
                    return fail_with(fmt("the finished layout did not check out: arrays %.0f and %.0f read %.0f GB/s together, "
                                         "below the threshold of %.0f",
                                         (double)j, (double)k, g, finder.threshold()));
                checked++;
            }
        success = true;
        std::vector<int> distinct;
        for (const auto &p : pick_region)
            for (int r : p)
                if (std::find(distinct.begin(), distinct.end(), r) == distinct.end()) distinct.push_back(r);
        regions_used_ = (int)distinct.size();
        note_ = fmt("%.0f regions, chunks of %.0f MiB", (double)regions_used_, (double)(chunk >> 20)) +
                fmt("; %.0f chunks created, %.0f probes", (double)chunks.size(), (double)finder.probes()) +
                fmt("; same region %.0f GB/s, threshold %.0f GB/s, %.0f array pairs checked", finder.same_pair(), finder.threshold(),
                    (double)checked);
        for (uint32_t j = 0; j < nparts; j++) {
            out[j] = part_ranges[j].va;
            ranges_.push_back({part_ranges[j].va, part_va});
        }
        for (const Chunk &c : chunks)
            if (c.keep) handles_.push_back(c.h);
        for (hipMemGenericAllocationHandle_t h : tails) handles_.push_back(h);
        cleanup(); // releases the chunks that were not chosen and the staging range
        if (debug) std::fprintf(stderr, "[nbo placement] %s\n", note_.c_str());
        return true;
    } catch (...) {
        cleanup();
        return give_up("an error while choosing chunks");
    }
}

} // namespace nbo
