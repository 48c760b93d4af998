// Host-only check of deepx_amd/executor/stream_picker.hpp, compiled and run by tests/test_stream_picker.py:
// random programs over a handful of tensor names, every placement replayed in a happens-before model.
#include <bitset>
#include <cstdio>
#include <random>
#include <string>
#include <vector>
#include "stream_picker.hpp"

#define CHECK(c) do { if (!(c)) { std::printf("FAILED line %d: %s\n", __LINE__, #c); return 1; } } while (0)

namespace {
constexpr int kMaxOps = 400;
struct Op { std::vector<std::string> reads, writes; bool kernel_only; };

bool clash(const Op &a, const Op &b) {  // must a stay before b
    for (const std::string &w : a.writes) {
        for (const std::string &x : b.reads) if (w == x) return true;
        for (const std::string &x : b.writes) if (w == x) return true;
    }
    for (const std::string &r : a.reads)
        for (const std::string &x : b.writes) if (r == x) return true;
    return false;
}
}  // namespace

int main() {
    using deepx::StreamPicker;
    std::mt19937 rng(20261);
    long placed_aside = 0, joins = 0, waits = 0;
    for (int trial = 0; trial < 600; ++trial) {
        const int streams = 1 + trial % 4;                       // 1 stream: everything in one line, still a valid answer
        const size_t cap = trial % 7 == 0 ? 12 : 4096;            // a tiny memory forces joins
        const int names = 3 + (int)(rng() % 10), count = 20 + (int)(rng() % (kMaxOps - 20));
        StreamPicker picker(streams, cap);
        std::vector<Op> ops;
        std::vector<std::bitset<kMaxOps>> before;                 // before[i][j]: op j is ordered before op i
        std::vector<int> last_on(streams, -1);                    // last op placed on each side stream
        int last_default = -1;                                    // last op on the default stream: before everything after it
        for (int i = 0; i < count; ++i) {
            Op op;
            const int nr = (int)(rng() % 3), nw = 1 + (int)(rng() % 2);
            for (int k = 0; k < nr; ++k) op.reads.push_back("t" + std::to_string(rng() % names));
            for (int k = 0; k < nw; ++k) op.writes.push_back("t" + std::to_string(rng() % names));
            op.kernel_only = rng() % 12 != 0;
            const bool force = rng() % 40 == 0;
            const StreamPicker::Choice c = picker.place(op.reads, op.writes, op.kernel_only, force);
            CHECK(c.stream >= -1 && c.stream < streams);
            CHECK(op.kernel_only && !force ? true : c.stream == -1);
            std::bitset<kMaxOps> b;
            auto after = [&](int j) { if (j >= 0) { b |= before[(size_t)j]; b.set((size_t)j); } };
            after(last_default);
            if (c.stream < 0) {
                CHECK(c.wait_for.empty());
                for (int s = 0; s < streams; ++s) after(last_on[(size_t)s]);
                last_default = i;
                ++joins;
            } else {
                after(last_on[(size_t)c.stream]);
                for (int s : c.wait_for) {
                    CHECK(s >= 0 && s < streams && s != c.stream);
                    after(last_on[(size_t)s]);
                    ++waits;
                }
                last_on[(size_t)c.stream] = i;
                ++placed_aside;
            }
            for (int j = 0; j < i; ++j)
                if (clash(ops[(size_t)j], op)) CHECK(b.test((size_t)j));  // every hazard is ordered
            ops.push_back(op);
            before.push_back(b);
        }
    }
    CHECK(placed_aside > 50000 && joins > 1000 && waits > 1000);
    {   // launches that share nothing are dealt out in turn, and a writer of what two streams read waits for both
        StreamPicker p(3);
        CHECK(p.place({"x"}, {"a"}, true).stream == 0);
        CHECK(p.place({"x"}, {"b"}, true).stream == 1);
        CHECK(p.place({"x"}, {"c"}, true).stream == 2);
        CHECK(p.place({"x"}, {"d"}, true).stream == 0);
        const StreamPicker::Choice c = p.place({"y"}, {"x"}, true);  // x is read on all three
        CHECK(c.stream == 0 && c.wait_for.size() == 2 && c.wait_for[0] == 1 && c.wait_for[1] == 2);
        CHECK(p.place({"b"}, {"e"}, true).stream == 1);               // reads what stream 1 wrote: behind it, no wait
        CHECK(p.place({}, {"z"}, false).stream == -1 && p.remembered() == 0);
        CHECK(p.place({"a"}, {"f"}, true).stream == 1);               // after a join nothing clashes: next in turn
    }
    {   // no side streams at all: everything on the default stream
        StreamPicker p(0);
        CHECK(p.place({"x"}, {"y"}, true).stream == -1);
    }
    std::printf("ok\n");
    return 0;
}
