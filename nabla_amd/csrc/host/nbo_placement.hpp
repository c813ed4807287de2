// Region-aware placement of the optimizer's state arrays in MI355X HBM.
#ifndef NBO_PLACEMENT_HPP
#define NBO_PLACEMENT_HPP

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

namespace nbo {

// Owns the device memory of up to three equally sized state arrays ("parts").
//
// Why this is not three hipMalloc calls.  MI355X's HBM3E behaves as three regions with a
// throughput ceiling each (its 12-high stacks have three ranks behind every channel): in-place
// read-modify-write streams that all fall into one region reach 5.3-5.4 TB/s, the same streams
// spread over two or three regions 6.2-6.3 TB/s.  Which region a piece of physical memory
// belongs to cannot be asked for, and consecutive allocations often share one: a process that
// allocates m, v and master back to back pays 5-15 % on every optimizer step.
//
// What it does instead.  The parts are assembled from 1-2 GiB physical chunks (hipMemCreate)
// stitched into contiguous virtual ranges (hipMemMap).  Chunks are created in rounds and sorted
// into regions by a pairwise bandwidth probe (two chunks of one region are measurably slower
// together than two of different regions): every chunk is probed against the first one, the
// threshold between "same" and "different" is the middle of the widest gap among those
// measurements (no absolute bandwidth enters), and chunks that differ from the first are probed
// against the first chunk of each further region.  Creation stops once two or three regions
// hold their share of the chunks needed, or at a limit: twice the chunks needed plus eight, or
// 104 GiB if that is more (regions are runs of up to 96 GiB of consecutively created chunks, and
// a search that is to find a second one must be allowed to walk that far) but then never more
// than half of the free memory; NBO_PLACEMENT_MAX_GIB overrides the limit.  Until the search is
// done it holds what it has created.  Chunk i of part j then comes from the
// ((i + j) mod U)-th of the U regions in use, so that at every position of the update's walk
// the parts sit in different regions and each region serves an equal share of the traffic.
// Three parts use all regions found; two parts (Adam / AdamW without master weights) use the
// two regions found last and leave the first to the caller's own tensors.  A part smaller than
// a chunk gets one whole chunk.  The finished layout is probed once more, and chunks that were
// created but not chosen are released.  The decisions themselves live in
// nbo_placement_plan.hpp, free of GPU calls.
//
// Small state (< 128 MiB per part), a single part, NBO_STATE_SPREAD=0, a GPU on which the probe
// shows no second region, or any failure along the way fall back to plain hipMalloc; note()
// says which.
class StatePlacement {
public:
    StatePlacement() = default;
    StatePlacement(const StatePlacement &) = delete;
    StatePlacement &operator=(const StatePlacement &) = delete;
    ~StatePlacement() { release(); }

    // Allocates nparts (<= 3) arrays of `bytes` bytes each; out[k] receives their device
    // addresses.  Contents are unspecified.  Throws nbo::Error on out-of-memory.
    void allocate(uint32_t nparts, size_t bytes, void **out);
    // The same search, another layout: array j lies wholly in one region, the one numbered
    // slot_of[j] (0, 1 or 2; equal numbers share a region, different numbers get different ones).
    // For memory the caller itself reads and writes -- parameters in one region, gradients in
    // another -- rather than the engine's state.  Returns false, having allocated nothing, where
    // allocate() would have fallen back to plain hipMalloc (note() says why).
    bool allocate_whole(uint32_t nparts, size_t bytes, const int *slot_of, void **out);
    void release();

    // How the last allocate() went, for logs and tests: 0 = plain hipMalloc,
    // otherwise the number of HBM regions the chunks were drawn from.
    int regions_used() const { return regions_used_; }
    // One line on the same: what was found, or why plain allocations were taken.
    const std::string &note() const { return note_; }

private:
    bool try_placed(uint32_t nparts, size_t bytes, void **out, const int *slot_of = nullptr);

    std::vector<void *> plain_;                               // hipMalloc'ed parts
    std::vector<hipMemGenericAllocationHandle_t> handles_;    // chunks in use
    struct Range {
        void *va;
        size_t size;
    };
    std::vector<Range> ranges_; // reserved virtual ranges (mapped)
    int regions_used_ = 0;
    std::string note_;
};

} // namespace nbo

#endif
