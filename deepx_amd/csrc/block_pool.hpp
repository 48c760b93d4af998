// Device blocks that have been freed, kept by size class for the next allocation of that class.
//
// The reference allocates and frees every tensor with the driver (cudaMalloc / cudaFree,
// executor/op-cuda/src/deepx/tensorfunc/tensorlife_miaobyte.hpp:20,31), and its front allocates the result of every
// op right before the op (front/py/deepx/nn/functional/leaffunc.py:30-38).  On this runtime hipMalloc of a tensor costs
// about 30 us and hipFree waits for the device (200-280 us behind running kernels), more than the kernels of a
// transformer block take, so blocks are handed out again instead.
//
// Plain host C++ over two function pointers, so the bookkeeping runs on the CPU without a device.
// What the pool does NOT know is which launches still use a block when it is freed: a block is handed out again
// at once, and whoever gets it must make its first use wait for the launches made before the free.  A first use on
// the NULL stream does (that stream waits for every blocking stream of the device); so does one on the stream that
// ran those launches.  The executor launches on the NULL stream unless it was told to spread lines over side streams,
// and then a `deltensor` line first makes every stream wait for what the others were given before it.
#pragma once
#include <cstddef>
#include <cstdint>
#include <iterator>
#include <map>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace dxh {

class BlockPool {
public:
    using AllocFn = int (*)(void **, size_t);  // 0 = success, like hipMalloc
    using FreeFn = int (*)(void *);

    struct Stats {
        uint64_t hits = 0;      // allocations served from a kept block
        uint64_t misses = 0;    // allocations that went to the driver
        uint64_t kept = 0;      // frees that kept the block
        uint64_t released = 0;  // blocks given back to the driver (cap, trim, or to make room after a failed allocation)
        uint64_t kept_bytes = 0, kept_blocks = 0;  // in the pool now
        uint64_t live_bytes = 0, live_blocks = 0;  // handed out now (by class size)
    };

    BlockPool(AllocFn a, FreeFn f, size_t max_kept_bytes) : alloc_(a), free_(f), max_kept_(max_kept_bytes) {}
    BlockPool(const BlockPool &) = delete;
    BlockPool &operator=(const BlockPool &) = delete;
    ~BlockPool() { trim(0); }

    // The size a request is rounded up to: eight classes per doubling (at most 12.5 % over the request), no step wider
    // than 2 MiB, nothing under 512 bytes.  0 = the request does not fit size_t after rounding.
    static size_t size_class(size_t bytes) {
        if (bytes <= 512) return 512;
        if (bytes > (SIZE_MAX >> 1)) return 0;
        int lg = 0;
        for (size_t b = bytes; b > 1; b >>= 1) ++lg;  // 2^lg <= bytes
        size_t step = (size_t)1 << (lg - 3);
        if (step > ((size_t)2 << 20)) step = (size_t)2 << 20;
        return (bytes + step - 1) & ~(step - 1);
    }

    // A block of at least `bytes`; the driver's error code when it has none to give even after every kept block went back.
    int alloc(void **ptr, size_t bytes) {
        if (!ptr) return -1;
        *ptr = nullptr;
        const size_t cls = size_class(bytes);
        if (cls == 0) return -1;
        std::lock_guard<std::mutex> lock(mu_);
        auto it = kept_.find(cls);
        if (it != kept_.end() && !it->second.empty()) {
            *ptr = it->second.back();
            it->second.pop_back();
            stats_.kept_bytes -= cls;
            --stats_.kept_blocks;
            ++stats_.hits;
        } else {
            int rc = alloc_(ptr, cls);
            if (rc != 0 && stats_.kept_blocks > 0) {  // the kept blocks may be what is in the way
                trim_locked(0);
                rc = alloc_(ptr, cls);
            }
            if (rc != 0) { *ptr = nullptr; return rc; }
            ++stats_.misses;
        }
        live_[*ptr] = cls;
        stats_.live_bytes += cls;
        ++stats_.live_blocks;
        return 0;
    }

    // Takes back a block that alloc() handed out; -1 for any other pointer (twice the same one included), which is left alone.
    int free(void *ptr) {
        if (!ptr) return 0;
        std::lock_guard<std::mutex> lock(mu_);
        auto it = live_.find(ptr);
        if (it == live_.end()) return -1;
        const size_t cls = it->second;
        live_.erase(it);
        stats_.live_bytes -= cls;
        --stats_.live_blocks;
        if (cls > max_kept_) {  // would never fit under the cap
            ++stats_.released;
            return free_(ptr);
        }
        if (stats_.kept_bytes + cls > max_kept_) trim_locked(max_kept_ - cls);
        kept_[cls].push_back(ptr);
        stats_.kept_bytes += cls;
        ++stats_.kept_blocks;
        ++stats_.kept;
        return 0;
    }

    // Gives kept blocks back to the driver, largest classes first, until at most `keep_bytes` stay; returns the bytes released.
    size_t trim(size_t keep_bytes) {
        std::lock_guard<std::mutex> lock(mu_);
        return trim_locked(keep_bytes);
    }

    bool owns(const void *ptr) {
        std::lock_guard<std::mutex> lock(mu_);
        return live_.count(const_cast<void *>(ptr)) != 0;
    }
    void set_max_kept(size_t bytes) {
        std::lock_guard<std::mutex> lock(mu_);
        max_kept_ = bytes;
        trim_locked(bytes);
    }
    Stats stats() {
        std::lock_guard<std::mutex> lock(mu_);
        return stats_;
    }

private:
    size_t trim_locked(size_t keep_bytes) {
        size_t gone = 0;
        while (stats_.kept_bytes > keep_bytes && !kept_.empty()) {
            auto last = std::prev(kept_.end());
            if (last->second.empty()) { kept_.erase(last); continue; }
            free_(last->second.back());
            last->second.pop_back();
            stats_.kept_bytes -= last->first;
            --stats_.kept_blocks;
            ++stats_.released;
            gone += last->first;
        }
        return gone;
    }

    AllocFn alloc_;
    FreeFn free_;
    size_t max_kept_;
    std::mutex mu_;
    std::map<size_t, std::vector<void *>> kept_;   // class size -> blocks, last freed on top (its lines are the likeliest to be in a cache still)
    std::unordered_map<void *, size_t> live_;      // handed out -> class size
    Stats stats_;
};

}  // namespace dxh
