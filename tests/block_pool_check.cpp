// Host-only check of deepx_amd/csrc/block_pool.hpp, compiled and run by tests/test_block_pool.py.
// The "driver" here is a table of fake addresses with a byte budget, so that running out of memory can be staged.
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <set>
#include <vector>
#include "block_pool.hpp"

#define CHECK(c) do { if (!(c)) { std::printf("FAILED line %d: %s\n", __LINE__, #c); return 1; } } while (0)

namespace {
std::map<void *, size_t> g_driver;  // what the fake driver has handed out
size_t g_budget = 0, g_used = 0;
uintptr_t g_next = 0x10000;
int g_allocs = 0, g_frees = 0;
int fake_alloc(void **p, size_t bytes) {
    if (g_used + bytes > g_budget) { *p = nullptr; return 2; }  // "out of memory"
    *p = (void *)g_next;
    g_next += (bytes + 0xfff) & ~(uintptr_t)0xfff;
    g_driver[*p] = bytes;
    g_used += bytes;
    ++g_allocs;
    return 0;
}
int fake_free(void *p) {
    auto it = g_driver.find(p);
    if (it == g_driver.end()) return 1;  // the pool must never free what the driver did not give, or twice
    g_used -= it->second;
    g_driver.erase(it);
    ++g_frees;
    return 0;
}
void reset(size_t budget) { g_driver.clear(); g_budget = budget; g_used = 0; g_allocs = g_frees = 0; }
}  // namespace

int main() {
    using dxh::BlockPool;
    {   // classes: never under the request, at most an eighth over it (512 bytes at the low end, 2 MiB steps at the high end),
        // monotone, and a class is its own class
        size_t before = 0;
        std::mt19937_64 rng(7);
        std::vector<size_t> sizes;
        for (size_t b = 0; b < 70000; ++b) sizes.push_back(b);
        for (int i = 0; i < 200000; ++i) sizes.push_back((size_t)(rng() >> (rng() % 40 + 10)));
        for (size_t s : {(size_t)1 << 20, ((size_t)1 << 20) + 1, (size_t)19922944, (size_t)268435456, ((size_t)288 << 30), ((size_t)1 << 40) + 12345}) sizes.push_back(s);
        for (size_t b : sizes) {
            const size_t c = BlockPool::size_class(b);
            CHECK(c >= b && c >= 512);
            CHECK(c == 512 || c - b <= b / 8);
            CHECK(c == 512 || c - b < ((size_t)2 << 20));
            CHECK(BlockPool::size_class(c) == c);
        }
        for (size_t b = 0; b < 70000; ++b) { const size_t c = BlockPool::size_class(b); CHECK(c >= before); before = c; }
        CHECK(BlockPool::size_class(SIZE_MAX) == 0 && BlockPool::size_class(SIZE_MAX / 2 + 2) == 0);
        // the shapes the benchmark configurations allocate are classes of their own: no padding on them
        for (size_t b : {(size_t)4096 * 4096 * 4, (size_t)8192 * 8192 * 4, (size_t)2048 * 4864 * 2, (size_t)2048 * 896 * 2}) CHECK(BlockPool::size_class(b) - b <= b / 8);
    }
    {   // the front's pattern: allocate a result, use it, free it, for ever: the driver is asked once per size
        reset((size_t)1 << 40);
        BlockPool pool(fake_alloc, fake_free, (size_t)1 << 36);
        void *first = nullptr;
        for (int i = 0; i < 100000; ++i) {
            void *a = nullptr, *b = nullptr;
            CHECK(pool.alloc(&a, 2048 * 4864 * 2) == 0 && pool.alloc(&b, 2048 * 896 * 2) == 0 && a && b && a != b);
            if (!first) first = a;
            CHECK(a == first);  // last freed, first handed out
            CHECK(pool.owns(a) && pool.owns(b));
            CHECK(pool.free(b) == 0 && pool.free(a) == 0);
            CHECK(!pool.owns(a));
        }
        CHECK(g_allocs == 2 && g_frees == 0);
        const BlockPool::Stats s = pool.stats();
        CHECK(s.misses == 2 && s.hits == 2 * 100000 - 2 && s.kept == 2 * 100000 && s.released == 0);
        CHECK(s.live_blocks == 0 && s.live_bytes == 0 && s.kept_blocks == 2);
        CHECK(s.kept_bytes == BlockPool::size_class(2048 * 4864 * 2) + BlockPool::size_class(2048 * 896 * 2));
        CHECK(pool.trim((size_t)1 << 40) == 0);
        CHECK(pool.trim(0) == s.kept_bytes && g_frees == 2 && g_used == 0);
    }
    {   // pointers the pool did not hand out, or got back already, are refused and nothing is freed for them
        reset((size_t)1 << 30);
        BlockPool pool(fake_alloc, fake_free, (size_t)1 << 30);
        void *a = nullptr;
        int local = 0;
        CHECK(pool.alloc(&a, 1000) == 0);
        CHECK(pool.free(&local) == -1 && pool.free(nullptr) == 0);
        CHECK(pool.free(a) == 0 && pool.free(a) == -1);
        CHECK(g_frees == 0 && pool.stats().kept_blocks == 1);
        CHECK(pool.alloc(nullptr, 8) == -1);
        void *z = nullptr;
        CHECK(pool.alloc(&z, 0) == 0 && z != nullptr);  // a zero-element tensor owns a pointer of its own
        void *z2 = nullptr;
        CHECK(pool.alloc(&z2, 0) == 0 && z2 != z);
        CHECK(pool.alloc(&z, SIZE_MAX) == -1 && z == nullptr);
    }
    {   // the cap: a free that would go over it releases larger kept blocks first; a block that alone is over it is not kept
        reset((size_t)1 << 30);
        BlockPool pool(fake_alloc, fake_free, 10 << 20);
        void *big = nullptr, *mid = nullptr, *small = nullptr, *huge = nullptr;
        CHECK(pool.alloc(&big, 6 << 20) == 0 && pool.alloc(&mid, 3 << 20) == 0 && pool.alloc(&small, 2 << 20) == 0 && pool.alloc(&huge, 11 << 20) == 0);
        CHECK(pool.free(huge) == 0 && g_frees == 1 && pool.stats().kept_blocks == 0);
        CHECK(pool.free(big) == 0 && pool.free(mid) == 0 && g_frees == 1 && pool.stats().kept_bytes == (9u << 20));
        CHECK(pool.free(small) == 0);  // 11 MiB would be kept: the 6 MiB block goes
        CHECK(g_frees == 2 && pool.stats().kept_bytes == (5u << 20) && pool.stats().kept_blocks == 2 && !g_driver.count(big));
        pool.set_max_kept(2 << 20);
        CHECK(pool.stats().kept_bytes == (2u << 20) && g_frees == 3);
        pool.set_max_kept(0);  // nothing is kept any more: every free goes to the driver
        CHECK(pool.stats().kept_blocks == 0);
        void *p = nullptr;
        CHECK(pool.alloc(&p, 4096) == 0 && pool.free(p) == 0 && pool.stats().kept_blocks == 0 && g_used == 0);
    }
    {   // the driver runs out while the pool keeps blocks of other sizes: they go back and the allocation succeeds;
        // with nothing kept the driver's own error code comes through
        reset(100 << 20);
        BlockPool pool(fake_alloc, fake_free, (size_t)1 << 30);
        std::vector<void *> blocks(9);
        for (void *&b : blocks) CHECK(pool.alloc(&b, 10 << 20) == 0);
        for (void *b : blocks) CHECK(pool.free(b) == 0);
        CHECK(g_used == (90u << 20));
        void *wide = nullptr;
        CHECK(pool.alloc(&wide, 64 << 20) == 0 && wide);
        CHECK(pool.stats().kept_blocks == 0 && g_used == (64u << 20));
        void *more = nullptr;
        CHECK(pool.alloc(&more, 64 << 20) == 2 && more == nullptr);
        CHECK(pool.stats().live_blocks == 1);
        CHECK(pool.free(wide) == 0);
    }
    {   // random traffic: no block is handed out twice at a time, live and kept bytes add up, and when the pool goes
        // away the driver has everything back that was freed
        reset((size_t)1 << 40);
        std::mt19937 rng(11);
        size_t live_expected = 0;
        std::vector<std::pair<void *, size_t>> mine;
        {
            BlockPool pool(fake_alloc, fake_free, 64 << 20);
            std::set<void *> out;
            for (int step = 0; step < 200000; ++step) {
                if (mine.empty() || rng() % 100 < 52) {
                    const size_t bytes = (size_t)1 << (rng() % 22);
                    void *p = nullptr;
                    CHECK(pool.alloc(&p, bytes + rng() % 64) == 0 && p);
                    CHECK(out.insert(p).second);
                    const size_t cls = BlockPool::size_class(bytes + 63);
                    CHECK(g_driver.count(p) && g_driver[p] >= bytes && g_driver[p] <= cls);
                    mine.push_back({p, g_driver[p]});
                    live_expected += g_driver[p];
                } else {
                    const size_t k = rng() % mine.size();
                    CHECK(pool.free(mine[k].first) == 0);
                    out.erase(mine[k].first);
                    live_expected -= mine[k].second;
                    mine[k] = mine.back();
                    mine.pop_back();
                }
                const BlockPool::Stats s = pool.stats();
                CHECK(s.live_bytes == live_expected && s.live_blocks == mine.size());
                CHECK(s.kept_bytes <= (64u << 20) && s.kept_bytes + s.live_bytes == g_used);
            }
            CHECK(pool.stats().hits > 50000);
        }
        CHECK(g_used == live_expected);  // what the caller never freed is all that is left
    }
    std::printf("ok\n");
    return 0;
}
