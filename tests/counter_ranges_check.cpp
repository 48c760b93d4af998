// Host-only check of deepx_amd/csrc/counter_ranges.hpp, compiled and run by tests/test_counter_ranges.py.
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>
#include "counter_ranges.hpp"

#define CHECK(c) do { if (!(c)) { std::printf("FAILED line %d: %s\n", __LINE__, #c); return 1; } } while (0)

int main() {
    using dxh::CounterRanges;
    {   // what a long-lived server does: record a batch, drop the graph, record again, for ever
        CounterRanges pool(32768, 65536);
        int stream_tag = 0;
        for (int round = 0; round < 100000; ++round) {
            const void *graph = (const void *)(uintptr_t)(round + 1);
            for (int launch = 0; launch < 5; ++launch) CHECK(pool.take_for_capture(&stream_tag, 40 + 17 * launch) >= 32768);
            pool.capture_ended(&stream_tag, graph);
            CHECK(pool.in_use() == 40 * 5 + 17 * 10);
            pool.graph_destroyed(graph);
            CHECK(pool.in_use() == 0 && pool.free_runs() == 1);
        }
    }
    {   // a capture that fails gives its counters back at once; an unknown graph or stream is ignored
        CounterRanges pool(0, 1000);
        int s1 = 0, s2 = 0;
        CHECK(pool.take_for_capture(&s1, 600) == 0);
        CHECK(pool.take_for_capture(&s2, 600) == -1);  // does not fit beside it
        CHECK(pool.take_for_capture(&s2, 400) == 600);
        CHECK(pool.take(1) == -1 && pool.take(0) == -1 && pool.take(-3) == -1);
        pool.capture_ended(&s1, nullptr);
        CHECK(pool.in_use() == 400);
        pool.capture_ended(&s1, nullptr);
        pool.graph_destroyed(&pool);
        CHECK(pool.in_use() == 400);
        pool.capture_ended(&s2, &s2);
        pool.graph_destroyed(&s2);
        CHECK(pool.in_use() == 0 && pool.free_runs() == 1 && pool.take(1000) == 0);
    }
    {   // many graphs alive at once, destroyed in random order: no counter is handed out twice, runs merge back
        CounterRanges pool(100, 100 + 4096);
        std::mt19937 rng(7);
        std::vector<int> owner(100 + 4096, 0);
        std::vector<std::pair<int, std::vector<std::pair<int64_t, int64_t>>>> alive;
        int stream_tag = 0, next = 1;
        for (int step = 0; step < 20000; ++step) {
            if (alive.empty() || rng() % 3) {
                std::vector<std::pair<int64_t, int64_t>> got;
                const int launches = 1 + rng() % 4;
                for (int l = 0; l < launches; ++l) {
                    const int64_t n = 1 + rng() % 128, off = pool.take_for_capture(&stream_tag, n);
                    if (off < 0) continue;  // full: the caller falls back to two launches
                    CHECK(off >= 100 && off + n <= 100 + 4096);
                    for (int64_t i = off; i < off + n; ++i) { CHECK(owner[i] == 0); owner[i] = next; }
                    got.push_back({off, n});
                }
                pool.capture_ended(&stream_tag, (const void *)(uintptr_t)next);
                alive.push_back({next++, got});
            } else {
                const size_t k = rng() % alive.size();
                for (auto &r : alive[k].second)
                    for (int64_t i = r.first; i < r.first + r.second; ++i) owner[i] = 0;
                pool.graph_destroyed((const void *)(uintptr_t)alive[k].first);
                alive.erase(alive.begin() + k);
            }
            int64_t held = 0;
            for (int v : owner) held += v != 0;
            CHECK(held == pool.in_use());
        }
        for (auto &g : alive) pool.graph_destroyed((const void *)(uintptr_t)g.first);
        CHECK(pool.in_use() == 0 && pool.free_runs() == 1 && pool.capacity() == 4096);
    }
    std::printf("ok\n");
    return 0;
}
