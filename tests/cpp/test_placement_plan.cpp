// The decisions of the state placement (nabla_amd/csrc/host/nbo_placement_plan.hpp) on the CPU,
// with made-up bandwidth measurements in place of the GPU probe: three regions, two regions,
// one region, a noisy fourth kind, regions that run dry, a faster and a slower GPU.
#include <cassert>
#include <cmath>
#include <cstdio>
#include <functional>
#include <vector>

#include "../../nabla_amd/csrc/host/nbo_placement_plan.hpp"

using namespace nbo::plan;

#define CHECK(cond)                                                                        \
    do {                                                                                   \
        if (!(cond)) {                                                                     \
            std::fprintf(stderr, "%s:%d: CHECK failed: %s\n", __FILE__, __LINE__, #cond);  \
            return 1;                                                                      \
        }                                                                                  \
    } while (0)

// A GPU whose chunk i lies in region truth[i]; pairs of one region measure `same`, others `diff`,
// each with a deterministic scatter of +-spread.
// truth -1 marks a chunk pieced together from two regions: it measures half-way against everything.
struct FakeGpu {
    std::vector<int> truth;
    double same, diff, spread;
    size_t calls = 0;
    double operator()(size_t a, size_t b)
    {
        calls++;
        const double wobble = spread * (double)((int)((a * 7 + b * 13) % 11) - 5) / 5.0;
        if (truth[a] < 0 || truth[b] < 0) return 0.5 * (same + diff) * (1.0 + wobble);
        return (truth[a] == truth[b] ? same : diff) * (1.0 + wobble);
    }
};
// the two halves of chunk a
struct FakeHalves {
    FakeGpu *gpu;
    double operator()(size_t a)
    {
        gpu->calls++;
        return gpu->same * (1.0 + 0.01 * (double)(a % 3));
    }
};

static std::vector<size_t> counts(const RegionFinder &f)
{
    std::vector<size_t> n;
    for (const auto &r : f.chunks_per_region()) n.push_back(r.size());
    return n;
}

static bool matches_truth(const RegionFinder &f, const std::vector<int> &truth)
{
    // same label in the finder <=> same region in truth, over all classified chunks
    const auto &r = f.region_of();
    for (size_t a = 0; a < r.size(); a++)
        for (size_t b = a + 1; b < r.size(); b++) {
            if (r[a] < 0 || r[b] < 0) continue;
            if ((r[a] == r[b]) != (truth[a] == truth[b])) return false;
        }
    return true;
}

int main()
{
    // gap_threshold: the middle of the widest gap above the anchor's own measure, nothing when
    // the values are of one kind
    CHECK(std::isinf(gap_threshold({5400, 5450, 5300, 5500}, 5400)));
    {
        const double t = gap_threshold({5481, 5466, 5215, 5359, 6402, 6398, 6397}, 5395);
        CHECK(t > 5481 && t < 6397);
    }
    CHECK(std::isinf(gap_threshold({}, 5400)));
    CHECK(std::isinf(gap_threshold({0.0, -1.0}, 5400)));
    CHECK(std::isinf(gap_threshold({6400, 6390}, 0.0))); // no measure of "same": nothing can be told
    // measured on one GPU: every chunk in the anchor's region, two disturbed (slow) probes; the
    // gap below the cluster is scatter, not a second region
    CHECK(std::isinf(gap_threshold({5590, 5566, 5656, 5613, 5622, 5616, 5618, 5614, 5654, 5050, 5075, 5517, 5567, 5424}, 5453)));
    // a single early sample a little above the anchor's own measure is no gap either
    CHECK(std::isinf(gap_threshold({5726}, 5385)));
    CHECK(std::isfinite(gap_threshold({5726, 6337}, 5385)));

    // three regions in runs, as measured on one MI355X (5.2-5.7 vs 6.3-6.5 TB/s)
    {
        FakeGpu gpu{{0, 0, 0, 0, 0, 1, 1, 1, 1, 2, 2, 2, 2}, 5450, 6400, 0.04};
        RegionFinder f;
        f.add_chunks(6, std::ref(gpu), FakeHalves{&gpu});
        CHECK(f.regions() == 2 && matches_truth(f, gpu.truth));
        const size_t probes_before = f.probes();
        f.add_chunks(13, std::ref(gpu), FakeHalves{&gpu});
        CHECK(f.regions() == 3 && matches_truth(f, gpu.truth));
        CHECK((counts(f) == std::vector<size_t>{5, 4, 4}));
        CHECK(f.probes() > probes_before && gpu.calls == f.probes()); // nothing measured twice
        CHECK(enough(counts(f), 3, 4) && !enough(counts(f), 3, 5));
    }
    // the same layout on a GPU twice as slow and on one 20 % faster: only ratios matter
    for (double k : {0.5, 1.2}) {
        FakeGpu gpu{{0, 1, 2, 0, 1, 2, 0, 1, 2}, 5450 * k, 6400 * k, 0.03};
        RegionFinder f;
        f.add_chunks(9, std::ref(gpu), FakeHalves{&gpu});
        CHECK(f.regions() == 3 && matches_truth(f, gpu.truth));
    }
    // one region only: no gap, everything reads "same", nothing to spread over
    {
        FakeGpu gpu{std::vector<int>(10, 0), 5450, 6400, 0.04};
        RegionFinder f;
        f.add_chunks(10, std::ref(gpu), FakeHalves{&gpu});
        CHECK(f.regions() == 1 && std::isinf(f.threshold()));
        CHECK(!enough(counts(f), 3, 2));
        CHECK(gpu.calls == 3 * 10 - 3); // every chunk against each of the three anchors tried, and their halves
    }
    // two regions: enough for two arrays, and for three (two of them then share at each position)
    {
        FakeGpu gpu{{0, 0, 0, 1, 1, 1, 1, 0}, 5450, 6400, 0.02};
        RegionFinder f;
        f.add_chunks(8, std::ref(gpu), FakeHalves{&gpu});
        CHECK(f.regions() == 2 && matches_truth(f, gpu.truth));
        CHECK(enough(counts(f), 2, 4) && enough(counts(f), 3, 2) && !enough(counts(f), 3, 3));
        CHECK((choose_regions(counts(f), 3, 2) == std::vector<size_t>{0, 1}));
    }
    // a fourth kind can only be noise: such chunks stay unused
    {
        FakeGpu gpu{{0, 1, 2, 3, 0, 1, 2, 3}, 5450, 6400, 0.02};
        RegionFinder f;
        f.add_chunks(8, std::ref(gpu), FakeHalves{&gpu});
        CHECK(f.regions() == 3);
        CHECK(f.region_of()[3] == -1 && f.region_of()[7] == -1);
        CHECK((counts(f) == std::vector<size_t>{2, 2, 2}));
    }
    // a failed probe (0 GB/s) reads "same": the chunk joins the first region rather than opening one
    {
        size_t n = 0;
        auto probe = [&](size_t, size_t b) { n++; return b == 2 ? 0.0 : 6400.0; };
        auto halves = [&](size_t) { return 5400.0; };
        RegionFinder f;
        f.add_chunks(4, probe, halves);
        CHECK(f.region_of()[2] == 0);
    }

    // chunk 0 alone in its region (as after a caller's own allocations): the rest still sorts out
    {
        FakeGpu gpu{{0, 1, 0, 1, 1, 2, 2, 1, 2, 2}, 5450, 6400, 0.03};
        RegionFinder f;
        f.add_chunks(10, std::ref(gpu), FakeHalves{&gpu});
        CHECK(f.anchor() == 0 && f.regions() == 3 && matches_truth(f, gpu.truth));
        CHECK((counts(f) == std::vector<size_t>{2, 4, 4}));
    }
    // chunk 0 straddles two regions and measures half-way against everything: no gap, so chunk 1
    // becomes the anchor; the straddling chunk lands somewhere, the others sort out
    {
        FakeGpu gpu{{-1, 0, 0, 1, 1, 0, 1, 1, 0, 1}, 5450, 6400, 0.01};
        RegionFinder f;
        f.add_chunks(10, std::ref(gpu), FakeHalves{&gpu});
        CHECK(std::isfinite(f.threshold()));
        // the straddling chunk forms a "region" of its own, the others sort out around it
        std::vector<int> truth = gpu.truth;
        truth[0] = 7;
        CHECK(f.regions() == 3 && matches_truth(f, truth));
        CHECK((counts(f) == std::vector<size_t>{1, 4, 5}));
        // ... and the one-chunk region does not keep the search going: the other two suffice
        CHECK(enough(counts(f), 3, 2) && (choose_regions(counts(f), 3, 2) == std::vector<size_t>{1, 2}));
        const auto pick = assign(counts(f), 3, 2);
        for (const auto &p : pick)
            for (int r : p) CHECK(r != 0);
    }
    // no gap around chunk 0 and none around chunk 1: the third anchor settles it
    {
        size_t n = 0;
        const std::vector<int> truth{-1, -1, 0, 1, 0, 1, 0, 1};
        auto probe = [&](size_t a, size_t b) {
            n++;
            if (truth[a] < 0 || truth[b] < 0) return 5900.0 + 10.0 * (double)((a + b) % 5);
            return truth[a] == truth[b] ? 5450.0 : 6400.0;
        };
        auto halves = [&](size_t a) { return truth[a] < 0 ? 5880.0 : 5440.0; };
        RegionFinder f;
        f.add_chunks(8, probe, halves);
        CHECK(f.anchor() == 2 && std::isfinite(f.threshold()) && f.regions() >= 2);
        CHECK(f.region_of()[2] == f.region_of()[4] && f.region_of()[3] == f.region_of()[5] &&
              f.region_of()[2] != f.region_of()[3]);
    }

    // assign: rotation over three regions, every position has its arrays in different regions
    {
        const auto pick = assign({4, 4, 4}, 3, 4);
        CHECK(pick.size() == 3 && pick[0].size() == 4);
        std::vector<size_t> used(3, 0);
        for (size_t i = 0; i < 4; i++) {
            CHECK(pick[0][i] != pick[1][i] && pick[1][i] != pick[2][i] && pick[0][i] != pick[2][i]);
            for (int j = 0; j < 3; j++) {
                CHECK(pick[j][i] == (int)((i + j) % 3));
                used[pick[j][i]]++;
            }
        }
        CHECK((used == std::vector<size_t>{4, 4, 4}));
    }
    // three arrays, three regions that each hold plenty: two of them are used, not three (two regions
    // measured 35.0-35.2 ms per update of the 8B set, three 35.4)
    {
        CHECK(choose_regions({10, 10, 10}, 3, 4).size() == 2);
        const auto pick = assign({10, 10, 10}, 3, 4);
        std::vector<size_t> used(3, 0);
        for (size_t i = 0; i < 4; i++)
            for (int j = 0; j < 3; j++) used[pick[j][i]]++;
        CHECK(std::count(used.begin(), used.end(), (size_t)0) == 1 && std::count(used.begin(), used.end(), (size_t)6) == 2);
    }
    // within a region the chunks that measured lowest with its leader (surest to be all of that region)
    // are handed out first
    {
        const std::vector<int> truth{0, 0, 0, 1, 1, 1, 0, 1};
        const std::vector<double> wobble{0, 120, 10, 0, 90, 20, 60, 5}; // how far from its own kind a chunk measures
        auto probe = [&](size_t a, size_t b) { return (truth[a] == truth[b] ? 5450.0 : 6400.0) + wobble[a] + wobble[b]; };
        auto halves = [&](size_t) { return 5440.0; };
        RegionFinder f;
        f.add_chunks(8, probe, halves);
        const auto pools = f.chunks_per_region();
        CHECK(pools.size() == 2);
        CHECK((pools[0] == std::vector<size_t>{1, 6, 2, 0}) && (pools[1] == std::vector<size_t>{4, 5, 7, 3}));
    }
    // two arrays and three regions: the first region is left to the caller's tensors
    {
        const auto pick = assign({6, 3, 3}, 2, 3);
        for (size_t i = 0; i < 3; i++) CHECK(pick[0][i] != 0 && pick[1][i] != 0 && pick[0][i] != pick[1][i]);
        // ... unless the other two do not hold enough
        const auto pick2 = assign({6, 2, 2}, 2, 3);
        CHECK(pick2.size() == 2);
        size_t from0 = 0;
        for (size_t i = 0; i < 3; i++) {
            CHECK(pick2[0][i] != pick2[1][i]);
            from0 += (pick2[0][i] == 0) + (pick2[1][i] == 0);
        }
        CHECK(from0 == 2);
    }
    // a region runs dry half-way: the rest comes from what is left, still apart where possible
    {
        const auto pick = assign({6, 2, 4}, 3, 4);
        CHECK(pick.size() == 3);
        std::vector<size_t> used(3, 0);
        for (size_t i = 0; i < 4; i++)
            for (int j = 0; j < 3; j++) used[pick[j][i]]++;
        CHECK((used == std::vector<size_t>{6, 2, 4}));
        for (size_t i = 0; i < 2; i++) // while all three last, the arrays are apart
            CHECK(pick[0][i] != pick[1][i] && pick[1][i] != pick[2][i] && pick[0][i] != pick[2][i]);
    }
    // exhaustion: fewer chunks than needed gives no plan
    CHECK(assign({3, 3, 3}, 3, 4).empty());
    CHECK(assign({}, 3, 1).empty());
    // two regions, three arrays: never all three in one region
    {
        const auto pick = assign({5, 4}, 3, 3);
        CHECK(pick.size() == 3);
        for (size_t i = 0; i < 3; i++) CHECK(!(pick[0][i] == pick[1][i] && pick[1][i] == pick[2][i]));
    }

    // whole arrays in named regions: equal numbers share a region, different numbers do not; the
    // slot that needs most gets the region that has most; not enough of anything gives no plan
    {
        const auto r = assign_whole({5, 9}, {0, 1}, 4); // two arrays of 4 chunks, apart
        CHECK(r.size() == kMaxRegions && r[0] != r[1] && r[0] >= 0 && r[1] >= 0 && r[2] == -1);
        const auto same = assign_whole({5, 9}, {1, 1}, 4); // both in one region: the one with 9
        CHECK(same.size() == kMaxRegions && same[1] == 1 && same[0] == -1);
        const auto two_one = assign_whole({4, 9}, {0, 0, 2}, 4); // slot 0 needs 8: region 1; slot 2 the other
        CHECK(two_one.size() == kMaxRegions && two_one[0] == 1 && two_one[2] == 0);
        CHECK(assign_whole({3, 9}, {0, 1}, 4).empty());       // the second region is too small
        CHECK(assign_whole({9}, {0, 1}, 4).empty());          // one region found, two asked for
        CHECK(assign_whole({9, 9, 9}, {0, 1, 2}, 9).size() == kMaxRegions);
        CHECK(assign_whole({9, 9}, {0, 3}, 1).empty());       // no such slot
    }

    // the creation limit: twice the need plus eight or far enough to cross a region boundary
    // (within half of what is free), a user's limit instead, never more than is free
    CHECK(chunk_cap(12, 250, 0, 104) == 104);
    CHECK(chunk_cap(12, 100, 0, 104) == 50);
    CHECK(chunk_cap(12, 40, 0, 104) == 32);
    CHECK(chunk_cap(87, 250, 0, 104) == 182);
    CHECK(chunk_cap(42, 60, 0, 104) == 60);
    CHECK(chunk_cap(12, 250, 20, 104) == 20);
    std::puts("placement plan: all checks passed");
    return 0;
}
