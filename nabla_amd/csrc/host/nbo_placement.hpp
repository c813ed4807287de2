// Region-aware placement of the optimizer's state arrays in MI355X HBM.
#ifndef NBO_PLACEMENT_HPP
#define NBO_PLACEMENT_HPP

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <vector>

namespace nbo {

// Owns the device memory of up to three equally sized state arrays ("parts").
//
// Why this is not three hipMalloc calls.  On MI355X the 288 GB of HBM3E behave as
// three regions of 96 GiB of physical address space with a throughput ceiling each:
// in-place read-modify-write streams that all fall into one region reach 5.4 TB/s,
// the same streams spread over two or three regions 6.3 TB/s (measured with a
// three-stream microbenchmark; the boundary sits exactly at multiples of 96 GiB of a
// single large allocation).  A process that allocates m, v and master back to back
// gets them from one region and pays 5-15 % on every optimizer step.
//
// What it does instead.  The parts are assembled from 1-2 GiB physical chunks
// (hipMemCreate) stitched into contiguous virtual ranges (hipMemMap).  Chunks are
// created one at a time and each is classified by a pairwise bandwidth probe against
// one representative chunk per region found so far -- two chunks of the same region
// are measurably slower together than two of different regions.  Creation stops once
// every region to be used holds its share of the chunks needed; chunk i of part j
// then comes from the ((i + j) mod U)-th of the U regions in use, so that at every
// position of the update's walk the parts sit in different regions and each region
// serves an equal share of the traffic.  Three parts use all three regions; two parts
// (Adam / AdamW without master weights) use the two regions found last and leave the
// first to the caller's own tensors.  A part smaller than a chunk gets one whole chunk.
// Chunks that were created but not chosen are released again.
//
// Small state (< 128 MiB per part), a single part, NBO_STATE_SPREAD=0, or any failure
// along the way fall back to plain hipMalloc.
class StatePlacement {
public:
    StatePlacement() = default;
    StatePlacement(const StatePlacement &) = delete;
    StatePlacement &operator=(const StatePlacement &) = delete;
    ~StatePlacement() { release(); }

    // Allocates nparts (<= 3) arrays of `bytes` bytes each; out[k] receives their device
    // addresses.  Contents are unspecified.  Throws nbo::Error on out-of-memory.
    void allocate(uint32_t nparts, size_t bytes, void **out);
    void release();

    // How the last allocate() went, for logs and tests: 0 = plain hipMalloc,
    // otherwise the number of HBM regions the chunks were drawn from.
    int regions_used() const { return regions_used_; }

private:
    bool try_placed(uint32_t nparts, size_t bytes, void **out);

    std::vector<void *> plain_;                               // hipMalloc'ed parts
    std::vector<hipMemGenericAllocationHandle_t> handles_;    // chunks in use
    struct Range {
        void *va;
        size_t size;
    };
    std::vector<Range> ranges_; // reserved virtual ranges (mapped)
    int regions_used_ = 0;
};

} // namespace nbo

#endif
