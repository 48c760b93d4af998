// stream_picker.hpp — where each launch of a batch goes when independent launches may overlap.
//
// Kernels of one stream run strictly in order; launches on different streams overlap.  A launch reads and
// writes named tensors.  Two launches must stay in order when one writes what the other reads or writes
// (read after write, write after read, write after write).  This class keeps, per side stream, the names
// its launches have read and written since the last join, and decides for every new launch:
//   * kernel-only and no clash with any stream  -> the next side stream in turn;
//   * a clash with one stream                    -> that stream (it runs behind what it depends on);
//   * a clash with several streams               -> the first of them, which must first be made to wait for
//                                                   an event recorded on each of the others (`wait_for`);
//   * not kernel-only, or too much remembered    -> the default stream (`stream` = -1), which the caller
//                                                   orders behind everything and everything behind it
//                                                   (`busy()` before the call names the streams that have
//                                                   something to wait for); the memory is cleared.
// Plain host code without a device call in it: the executor turns a Choice into streams and events
// (executor.hpp), a host-only check replays random programs against a happens-before model
// (tests/stream_picker_check.cpp).
#pragma once
#include <cstddef>
#include <string>
#include <unordered_set>
#include <vector>

namespace deepx {

class StreamPicker {
public:
    struct Choice {
        int stream = -1;             // side stream index, or -1 = the default stream (a join of everything)
        std::vector<int> wait_for;   // side streams whose work so far the chosen stream must wait for first
    };

    explicit StreamPicker(int streams = 0, size_t max_remembered = 4096) : sides_(streams > 0 ? (size_t)streams : 0), max_remembered_(max_remembered) {}
    int streams() const { return (int)sides_.size(); }
    void resize(int streams) { sides_.assign(streams > 0 ? (size_t)streams : 0, Side{}); next_ = 0; }

    // everything launched so far is known to be ordered before whatever comes next (a launch on the default
    // stream, a device-wide wait)
    void joined() {
        for (Side &s : sides_) { s.reads.clear(); s.writes.clear(); }
    }
    // side streams that have launched something since the last join
    std::vector<int> busy() const {
        std::vector<int> b;
        for (size_t k = 0; k < sides_.size(); ++k) if (!sides_[k].reads.empty() || !sides_[k].writes.empty()) b.push_back((int)k);
        return b;
    }
    size_t remembered() const {
        size_t n = 0;
        for (const Side &s : sides_) n += s.reads.size() + s.writes.size();
        return n;
    }

    // force_join: something the picker cannot see is in flight (a replayed graph on a stream of its own)
    Choice place(const std::vector<std::string> &reads, const std::vector<std::string> &writes, bool kernel_only, bool force_join = false) {
        Choice c;
        if (sides_.empty() || !kernel_only || force_join || remembered() > max_remembered_) {
            joined();
            return c;
        }
        std::vector<int> hit;
        for (size_t k = 0; k < sides_.size(); ++k) {
            const Side &s = sides_[k];
            bool clash = false;
            for (const std::string &w : writes) clash = clash || s.writes.count(w) || s.reads.count(w);
            for (const std::string &r : reads) clash = clash || s.writes.count(r);
            if (clash) hit.push_back((int)k);
        }
        c.stream = hit.empty() ? (int)(next_++ % sides_.size()) : hit[0];
        c.wait_for.assign(hit.begin() + (hit.empty() ? 0 : 1), hit.end());
        sides_[(size_t)c.stream].reads.insert(reads.begin(), reads.end());
        sides_[(size_t)c.stream].writes.insert(writes.begin(), writes.end());
        return c;
    }
    // the caller could not act on a Choice (a stream or event call failed): it falls back to the default stream
    void abandon() { joined(); }

private:
    struct Side { std::unordered_set<std::string> reads, writes; };
    std::vector<Side> sides_;
    size_t next_ = 0, max_remembered_;
};

}  // namespace deepx
