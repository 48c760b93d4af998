// counter_ranges.hpp — host-side bookkeeping for the counters that launches recorded under stream
// capture take from the library's device array (finish_counters, reduce.hip).  A recorded launch
// may replay at any later time next to eager work, so its counters belong to the graph it was
// recorded into and come back only when that graph is destroyed (or its capture fails).  Plain
// C++ (no HIP): a first-fit free list over [begin, end) whose neighbours are merged on release.
#pragma once
#include <cstdint>
#include <map>
#include <utility>
#include <vector>

namespace dxh {

class CounterRanges {
public:
    CounterRanges(int64_t begin, int64_t end) { if (end > begin) free_[begin] = end - begin; capacity_ = end > begin ? end - begin : 0; }
    // offset of `n` consecutive counters, or -1 when no free run is long enough
    int64_t take(int64_t n) {
        if (n <= 0) return -1;
        for (auto it = free_.begin(); it != free_.end(); ++it) {
            if (it->second < n) continue;
            const int64_t off = it->first, left = it->second - n;
            free_.erase(it);
            if (left > 0) free_[off + n] = left;
            in_use_ += n;
            return off;
        }
        return -1;
    }
    void give(int64_t off, int64_t n) {
        if (n <= 0) return;
        in_use_ -= n;
        auto next = free_.lower_bound(off);
        if (next != free_.begin()) {  // merge with the run that ends where this one starts
            auto prev = std::prev(next);
            if (prev->first + prev->second == off) { off = prev->first; n += prev->second; free_.erase(prev); }
        }
        if (next != free_.end() && off + n == next->first) { n += next->second; free_.erase(next); }
        free_[off] = n;
    }
    // bookkeeping per owner: ranges taken while a capture is open on `stream` are handed to the
    // graph the capture ends in, and go back to the pool with that graph
    int64_t take_for_capture(const void *stream, int64_t n) {
        const int64_t off = take(n);
        if (off >= 0) open_[stream].push_back({off, n});
        return off;
    }
    void capture_ended(const void *stream, const void *graph) {  // graph == nullptr: the capture failed
        auto it = open_.find(stream);
        if (it == open_.end()) return;
        if (graph) {
            auto &dst = owned_[graph];
            dst.insert(dst.end(), it->second.begin(), it->second.end());
        } else {
            release(it->second);
        }
        open_.erase(it);
    }
    void graph_destroyed(const void *graph) {
        auto it = owned_.find(graph);
        if (it == owned_.end()) return;
        release(it->second);
        owned_.erase(it);
    }
    int64_t in_use() const { return in_use_; }
    int64_t capacity() const { return capacity_; }
    size_t free_runs() const { return free_.size(); }

private:
    void release(const std::vector<std::pair<int64_t, int64_t>> &ranges) {
        for (const auto &r : ranges) give(r.first, r.second);
    }
    std::map<int64_t, int64_t> free_;  // offset -> length
    std::map<const void *, std::vector<std::pair<int64_t, int64_t>>> open_, owned_;
    int64_t in_use_ = 0, capacity_ = 0;
};

}  // namespace dxh
