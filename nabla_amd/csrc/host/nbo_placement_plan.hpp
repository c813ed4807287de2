// The decisions of the region-aware state placement, free of any GPU call so that they can be
// tested on the CPU with made-up measurements: which chunks share a region of the HBM, whether
// enough chunks of each region are at hand, and which region each chunk of each state array
// comes from.  nbo_placement.cpp supplies the measurements (a two-buffer bandwidth probe) and
// does the mapping.
#ifndef NBO_PLACEMENT_PLAN_HPP
#define NBO_PLACEMENT_PLAN_HPP

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <limits>
#include <map>
#include <utility>
#include <vector>

namespace nbo {
namespace plan {

constexpr size_t kMaxRegions = 3;
// Two chunks of one region read and rewritten together run 10-20 % slower than two chunks of
// different regions.  Values of one kind scatter by a few per cent -- mostly downwards: a probe
// that is disturbed is slower, never faster -- and a chunk the driver pieced together from two
// regions measures half-way.  The measurements are therefore split into a low and a high class
// where that separates them best (largest between-class variance), and the split is taken for
// "same" against "different" only if the class means are at least kMinClassRatio apart and the
// threshold lies between 3 and 30 % above what the anchor chunk measures against itself
// (`same_pair`, its two halves, certainly of the low kind).  Anything else is scatter.
constexpr double kMinClassRatio = 1.08;
constexpr double kMinAboveSame = 1.03, kMaxAboveSame = 1.30;

// Threshold between "same region" and "different region" from measurements that all involve
// one fixed chunk: the geometric mean of the two class means, or +infinity when the values do
// not fall into two such classes (every value then reads "same").  No absolute bandwidth
// enters, so a faster, slower or busier GPU moves both kinds together.
inline double gap_threshold(std::vector<double> samples, double same_pair)
{
    const double inf = std::numeric_limits<double>::infinity();
    if (!(same_pair > 0.0)) return inf;
    samples.push_back(same_pair);
    samples.erase(std::remove_if(samples.begin(), samples.end(), [](double v) { return !(v > 0.0); }), samples.end());
    std::sort(samples.begin(), samples.end());
    const size_t n = samples.size();
    if (n < 2) return inf;
    double total = 0.0;
    for (double v : samples) total += v;
    double best = -1.0, lo_mean = 0.0, hi_mean = 0.0, lo_sum = 0.0;
    for (size_t k = 0; k + 1 < n; k++) { // low class: samples[0..k]
        lo_sum += samples[k];
        const double m0 = lo_sum / (double)(k + 1), m1 = (total - lo_sum) / (double)(n - k - 1);
        const double between = (double)(k + 1) * (double)(n - k - 1) * (m1 - m0) * (m1 - m0);
        if (between > best) {
            best = between;
            lo_mean = m0;
            hi_mean = m1;
        }
    }
    if (!(hi_mean >= lo_mean * kMinClassRatio)) return inf;
    const double thr = std::sqrt(lo_mean * hi_mean);
    if (thr < same_pair * kMinAboveSame || thr > same_pair * kMaxAboveSame) return inf;
    return thr;
}

// Sorts chunks into at most three regions.  Chunks arrive in rounds (add_chunks).  One chunk is
// the anchor: every other chunk is measured against it, and the threshold between "same region"
// and "different region" is read off those measurements together with the anchor's own two
// halves (which certainly share a region).  Chunk 0 is the anchor unless its measurements show
// no gap -- a chunk whose physical memory straddles two regions measures half-way against
// everything -- in which case chunks 1 and 2 are tried.  Chunks that do not share the anchor's
// region are measured against the first chunk of each further region ("leader") in turn.  A
// chunk that differs from three leaders is left unused (region -1): a fourth kind can only be
// noise.
class RegionFinder {
public:
    static constexpr size_t kMaxAnchors = 3;

    // Chunks [0, total) now exist.  probe(a, b) measures chunks a and b together, halves(a) the
    // two halves of chunk a (GB/s; <= 0 on failure, which reads "same").  Re-sorts everything,
    // measuring only what has not been measured before.
    template <typename Probe, typename Halves> void add_chunks(size_t total, Probe &&probe, Halves &&halves)
    {
        total_ = total;
        region_of_.assign(total_, -1);
        leaders_.clear();
        threshold_ = std::numeric_limits<double>::infinity();
        anchor_ = 0;
        if (total_ == 0) return;
        for (size_t a = 0; a < kMaxAnchors && a < total_; a++) {
            std::vector<double> v;
            for (size_t i = 0; i < total_; i++)
                if (i != a) v.push_back(measure(a, i, probe));
            const double t = gap_threshold(v, base_of(a, halves));
            if (std::isfinite(t)) {
                threshold_ = t;
                anchor_ = a;
                break;
            }
            if (total_ < 4) break; // too few measurements to blame the anchor
        }
        leaders_.push_back(anchor_);
        for (size_t i = 0; i < total_; i++) {
            int region = -1;
            for (size_t k = 0; k < leaders_.size() && region < 0; k++)
                if (measure(leaders_[k], i, probe) < threshold_) region = (int)k;
            if (region < 0 && leaders_.size() < kMaxRegions) {
                leaders_.push_back(i);
                region = (int)leaders_.size() - 1;
            }
            region_of_[i] = region;
        }
    }

    double threshold() const { return threshold_; } // +infinity: no second region seen yet
    double same_pair() const { return bases_.count(anchor_) ? bases_.at(anchor_) : 0.0; } // the anchor's halves
    size_t anchor() const { return anchor_; }
    size_t regions() const { return leaders_.size(); }
    const std::vector<int> &region_of() const { return region_of_; }
    const std::vector<size_t> &leaders() const { return leaders_; }
    size_t probes() const { return cache_.size() + bases_.size(); }
    // The chunks of every region, the ones that measured slowest together with their region's
    // leader -- the ones most surely all of that region; a chunk the driver pieced together
    // from several regions measures higher -- at the back, where they are taken from first.
    std::vector<std::vector<size_t>> chunks_per_region() const
    {
        std::vector<std::vector<size_t>> out(leaders_.size());
        for (size_t i = 0; i < region_of_.size(); i++)
            if (region_of_[i] >= 0) out[(size_t)region_of_[i]].push_back(i);
        for (size_t k = 0; k < out.size(); k++)
            std::stable_sort(out[k].begin(), out[k].end(), [&](size_t x, size_t y) {
                return with_leader(k, x) > with_leader(k, y);
            });
        return out;
    }

private:
    double with_leader(size_t k, size_t i) const // what chunk i measured together with region k's leader
    {
        if (leaders_[k] == i) return 0.0;
        auto it = cache_.find(std::pair<size_t, size_t>(std::min(leaders_[k], i), std::max(leaders_[k], i)));
        return it == cache_.end() ? 0.0 : it->second;
    }
    template <typename Halves> double base_of(size_t a, Halves &&halves)
    {
        auto it = bases_.find(a);
        if (it != bases_.end()) return it->second;
        const double g = halves(a);
        bases_[a] = g;
        return g;
    }
    template <typename Probe> double measure(size_t a, size_t b, Probe &&probe)
    {
        if (a == b) return 0.0; // a chunk shares its own region
        const std::pair<size_t, size_t> key(std::min(a, b), std::max(a, b));
        auto it = cache_.find(key);
        if (it != cache_.end()) return it->second;
        const double g = probe(key.first, key.second);
        cache_[key] = g;
        return g;
    }

    double threshold_ = std::numeric_limits<double>::infinity();
    size_t total_ = 0, anchor_ = 0;
    std::vector<int> region_of_;
    std::vector<size_t> leaders_;
    std::map<std::pair<size_t, size_t>, double> cache_;
    std::map<size_t, double> bases_;
};

// Which regions the state arrays rotate over, given how many chunks of each region are at hand:
// the first of these sets whose every region holds an equal share of the full * nparts chunks
// needed.  Three arrays: all three regions, else the pair holding most.  Two arrays: the two
// regions found last -- the first region found is where this process's most recent allocations
// went, the caller's parameters and gradients most likely among them -- else any other pair.
// Empty: no set will do yet.  A region with a handful of chunks (the remainder of a region the
// caller's own tensors fill) is simply not used.
inline std::vector<size_t> choose_regions(const std::vector<size_t> &avail, uint32_t nparts, size_t full)
{
    const size_t R = avail.size(), total = full * nparts;
    auto holds = [&](const std::vector<size_t> &set) {
        const size_t each = (total + set.size() - 1) / set.size();
        for (size_t r : set)
            if (avail[r] < each) return false;
        return true;
    };
    std::vector<std::vector<size_t>> candidates;
    std::vector<std::vector<size_t>> pairs;
    if (R >= 3) pairs = {{1, 2}, {0, 2}, {0, 1}};
    else if (R == 2) pairs = {{0, 1}};
    if (nparts >= 3) // the pair holding most first
        std::stable_sort(pairs.begin(), pairs.end(), [&](const std::vector<size_t> &x, const std::vector<size_t> &y) {
            return avail[x[0]] + avail[x[1]] > avail[y[0]] + avail[y[1]];
        });
    candidates.insert(candidates.end(), pairs.begin(), pairs.end());
    if (R >= 3 && nparts >= 3) candidates.push_back({0, 1, 2});
    for (const auto &set : candidates)
        if (holds(set)) return set;
    return {};
}

// True once the chunks at hand let every array rotate evenly over two or three regions.  (Two
// regions give nearly all of the gain of three: the search does not go on for a third.)
inline bool enough(const std::vector<size_t> &avail, uint32_t nparts, size_t full)
{
    return !choose_regions(avail, nparts, full).empty();
}

// pick[j][i] = region that chunk i of array j comes from: the ((i + j) mod U)-th of the U
// regions in use, so that at every position of the update's walk the arrays sit in different
// regions and every region serves an equal share of the traffic; when that region has run dry,
// the one with most chunks left that the array's neighbours at this position do not use, else
// the one with most chunks left.  Empty result: not enough chunks.
inline std::vector<std::vector<int>> assign(std::vector<size_t> avail, uint32_t nparts, size_t full)
{
    std::vector<std::vector<int>> pick;
    size_t total = 0;
    for (size_t a : avail) total += a;
    if (avail.empty() || total < full * nparts) return pick;
    std::vector<size_t> use = choose_regions(avail, nparts, full);
    if (use.empty()) // no even rotation possible: every region is fair game, fullest first when one runs dry
        for (size_t r = 0; r < avail.size(); r++) use.push_back(r);
    pick.assign(nparts, std::vector<int>());
    for (size_t i = 0; i < full; i++) {
        std::vector<int> taken_here;
        for (uint32_t j = 0; j < nparts; j++) {
            size_t r = use[(i + j) % use.size()];
            if (avail[r] == 0) {
                // prefer a region no other array uses at this position
                size_t best = avail.size();
                for (size_t q = 0; q < avail.size(); q++) {
                    if (avail[q] == 0) continue;
                    const bool clash = std::find(taken_here.begin(), taken_here.end(), (int)q) != taken_here.end();
                    const bool best_clash =
                        best < avail.size() && std::find(taken_here.begin(), taken_here.end(), (int)best) != taken_here.end();
                    if (best == avail.size() || (best_clash && !clash) || (best_clash == clash && avail[q] > avail[best]))
                        best = q;
                }
                r = best;
            }
            avail[r]--;
            pick[j].push_back((int)r);
            taken_here.push_back((int)r);
        }
    }
    return pick;
}

// Whole arrays in one region each (the caller's own tensors: parameters here, gradients there).
// slot_of[j] names the region array j is to lie in -- a number below kMaxRegions; equal numbers
// share a region, different numbers get different regions.  Returns the region (index into
// `avail`) of every slot in use, -1 for unused slots; the slot that needs most chunks gets the
// region that has most.  Empty result: the chunks at hand do not allow it.
inline std::vector<int> assign_whole(const std::vector<size_t> &avail, const std::vector<int> &slot_of, size_t full)
{
    std::vector<size_t> need(kMaxRegions, 0);
    for (int s : slot_of) {
        if (s < 0 || (size_t)s >= kMaxRegions) return {};
        need[(size_t)s] += full;
    }
    std::vector<size_t> slots, regions;
    for (size_t s = 0; s < kMaxRegions; s++)
        if (need[s]) slots.push_back(s);
    for (size_t r = 0; r < avail.size(); r++) regions.push_back(r);
    if (slots.size() > regions.size()) return {};
    std::stable_sort(slots.begin(), slots.end(), [&](size_t a, size_t b) { return need[a] > need[b]; });
    std::stable_sort(regions.begin(), regions.end(), [&](size_t a, size_t b) { return avail[a] > avail[b]; });
    std::vector<int> out(kMaxRegions, -1);
    for (size_t k = 0; k < slots.size(); k++) {
        if (avail[regions[k]] < need[slots[k]]) return {};
        out[slots[k]] = (int)regions[k];
    }
    return out;
}

// How many chunks the search may create (and hold until it is done) before it settles for what
// it has.  Regions are runs of consecutively created chunks, up to 96 GiB long, so a search that
// is to find a second region must be allowed to walk that far: twice what the arrays need plus
// eight chunks, or `reach_chunks` (what covers one region and a bit) if that is more -- but
// for the sake of whoever else allocates meanwhile never beyond half of what is free, unless the
// arrays themselves need more.  A user's limit replaces all of that.
inline size_t chunk_cap(size_t needed, size_t free_chunks, size_t user_cap_chunks, size_t reach_chunks)
{
    size_t cap = 2 * needed + 8;
    const size_t reach = std::min(reach_chunks, free_chunks / 2);
    if (reach > cap) cap = reach;
    if (user_cap_chunks) cap = user_cap_chunks;
    return std::min(cap, free_chunks);
}

} // namespace plan
} // namespace nbo

#endif
