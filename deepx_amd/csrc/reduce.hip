// reduce.hip — sum / prod / reducemax / reducemin over arbitrary axes (gfx950).
//
// Semantics: executor/op-ompsimd/src/deepx/tensorfunc/reduce_miaobyte.hpp:19-345 with the
// axis handling of executor/deepxcore/src/deepx/shape_reduce.cpp:11-85.  The reference
// visits every input element and accumulates into the output under an atomic; here the
// shape is first canonicalised (size-1 axes dropped, neighbouring axes of equal
// kept/reduced status merged), then reduced axis-group by axis-group, last group first:
//
//   row stage   [pre, R]        R contiguous: a group of G lanes (G = 1..64, or the whole
//                               256-thread workgroup) owns one row chunk; 16-byte loads,
//                               V independent accumulators per lane, wave shuffle
//                               reduction, LDS across the four waves.
//   col stage   [pre, R, post]  R strided: lanes run along `post` (coalesced 16-byte
//                               loads), TY row-lanes per workgroup walk R, LDS tree
//                               across the row-lanes.
//
// When a stage has too few workgroups to fill 256 CUs, R is split into S chunks whose
// partials ([pre, S, post], accumulate type) go to the caller's workspace and are reduced
// by one more stage; results are deterministic (no atomic accumulation).  A split col
// stage over the caller's input normally finishes inside the same launch: every workgroup
// stores its partial tile and counts itself in on the tile's counter, and the one that
// arrives last adds the S partials in a fixed order (reduce_col_fused_kernel; the counters
// live in a file-scope device array and return to zero, see finish_counters).  Both stage
// kinds are HBM-bound: algorithmic bytes = input once + output once.
#include "reduce_order.hpp"
#include "counter_ranges.hpp"
#include <map>
#include <mutex>
#include <vector>

namespace dxh {

// ---- row stage ---------------------------------------------------------------------------
// in [pre, R] (R contiguous) -> out [pre, S]; chunk s covers r in [s*chunk, min(R,(s+1)*chunk)).
// G lanes cooperate on one (row, chunk); G in {1,2,..,64} packs 256/G rows per workgroup,
// G == 256 gives the whole workgroup to one row.
template <int K, typename Tin, typename Tout, typename TS, int V, bool NTL>
__device__ __forceinline__ void reduce_row_body(racc_t<TS> *lds, const Tin *__restrict__ in, Tout *__restrict__ out,
                                                             int64_t pre, int64_t R, int S, int64_t chunk, int G) {
    using A = racc_t<TS>;
    using VT = vec_t<Tin, V>;
    const int rows_per_block = kBlock / G;
    const int lane = threadIdx.x % G;
    const int64_t row = (int64_t)blockIdx.x * rows_per_block + threadIdx.x / G;
    const int s = blockIdx.y;
    const bool active = row < pre;
    A acc[V];
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = rinit<K, A, TS>();
    if (active) {
        const int64_t r0 = (int64_t)s * chunk;
        const int64_t r1 = (r0 + chunk < R) ? r0 + chunk : R;
        const int64_t len = r1 - r0;
        const Tin *p = in + row * R + r0;
        const VT *pv = reinterpret_cast<const VT *>(p);
        const int64_t lv = len / V;
        // 8 independent 16-byte loads in flight per lane, then 4, then singles
        row_lane_fold<K, A, V>(acc, lane, G, lv, [&](int64_t i) __attribute__((always_inline)) { return ld_sel<NTL>(&pv[i]); });
        for (int64_t j = lv * V + lane; j < len; j += G) acc[0] = rop<K, A>(acc[0], rload<A>(p[j]));
    }
    // lanes of one group are adjacent, so xor-shuffles below G stay inside the group
    const A v = row_group_fold<K, A, V>(acc, G);
    if (G == kBlock) {
        if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = v;
        __syncthreads();
        if (threadIdx.x == 0) {
            A r = lds[0];
#pragma unroll
            for (int w = 1; w < kBlock / kWave; ++w) r = rop<K, A>(r, lds[w]);
            if (active) out[row * S + s] = rstore<Tout, A>(r);
        }
    } else if (lane == 0 && active) {
        out[row * S + s] = rstore<Tout, A>(v);
    }
}
// ntl: loads carry the nt hint (chosen per launch, see nt_load_reduce in common.hpp)
template <int K, typename Tin, typename Tout, typename TS, int V>
__global__ __launch_bounds__(kBlock) void reduce_row_kernel(const Tin *__restrict__ in, Tout *__restrict__ out, int64_t pre, int64_t R, int S, int64_t chunk, int G, int ntl) {
    using A = racc_t<TS>;
    __shared__ A lds[kBlock / kWave];
    if (ntl) reduce_row_body<K, Tin, Tout, TS, V, true>(lds, in, out, pre, R, S, chunk, G);
    else reduce_row_body<K, Tin, Tout, TS, V, false>(lds, in, out, pre, R, S, chunk, G);
}

// ---- col stage ---------------------------------------------------------------------------
// in [pre, R, post] -> out [pre, S, post].  Workgroup = TX column-lanes x TY row-lanes
// (TX*TY == 256); a column-lane owns V adjacent columns.  Linear block id -> (p, s, ctile).
// DEST 1: the partial tile is written through to memory (device-scope stores), for a reader in another
// workgroup of the same launch.  DEST 2: nothing is stored; row-lane 0's part of `lds` holds the tile
// (value k of column-lane tx at lds[k * TY * TX + tx]) and the caller goes on with it.
template <int K, typename Tin, typename Tout, typename TS, int V, bool NTL, int DEST = 0>
__device__ __forceinline__ void reduce_col_body(racc_t<TS> *lds, const Tin *__restrict__ in, Tout *__restrict__ out,
                                                             int64_t pre, int64_t R, int64_t post, int S, int64_t chunk,
                                                             int TX, int ctiles) {
    using A = racc_t<TS>;
    using VT = vec_t<Tin, V>;
    const int TY = kBlock / TX;
    const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    int64_t b = blockIdx.x;
    const int ct = (int)(b % ctiles); b /= ctiles;
    const int s = (int)(b % S);
    const int64_t p = b / S;
    const int64_t postv = post / V;  // launcher guarantees post % V == 0
    const int64_t cv = (int64_t)ct * TX + tx;
    const bool active = cv < postv;
    A acc[V];
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = rinit<K, A, TS>();
    if (active) {
        const int64_t r0 = (int64_t)s * chunk;
        const int64_t r1 = (r0 + chunk < R) ? r0 + chunk : R;
        const VT *base = reinterpret_cast<const VT *>(in + p * R * post) + cv;
        int64_t r = r0 + ty;
        // batches of 8 rows per lane, software-pipelined: the loads of the next batch are issued
        // before the current one is folded, so 8..16 loads per lane stay in flight
        if (r + 7 * (int64_t)TY < r1) {
            VT x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) x[u] = ld_sel<NTL>(&base[(r + u * (int64_t)TY) * postv]);
            r += 8 * (int64_t)TY;
            auto fold = [&](const VT(&b)[8]) __attribute__((always_inline)) {
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    A t0 = rop<K, A>(rop<K, A>(rload<A>(b[0].v[k]), rload<A>(b[1].v[k])), rop<K, A>(rload<A>(b[2].v[k]), rload<A>(b[3].v[k])));
                    A t1 = rop<K, A>(rop<K, A>(rload<A>(b[4].v[k]), rload<A>(b[5].v[k])), rop<K, A>(rload<A>(b[6].v[k]), rload<A>(b[7].v[k])));
                    acc[k] = rop<K, A>(acc[k], rop<K, A>(t0, t1));
                }
            };
            for (; r + 7 * (int64_t)TY < r1; r += 8 * (int64_t)TY) {
                VT y[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) y[u] = ld_sel<NTL>(&base[(r + u * (int64_t)TY) * postv]);
                fold(x);
#pragma unroll
                for (int u = 0; u < 8; ++u) x[u] = y[u];
            }
            fold(x);
        }
        for (; r < r1; r += TY) {
            VT x = ld_sel<NTL>(&base[r * postv]);
#pragma unroll
            for (int k = 0; k < V; ++k) acc[k] = rop<K, A>(acc[k], rload<A>(x.v[k]));
        }
    }
#pragma unroll
    for (int k = 0; k < V; ++k) lds[(k * TY + ty) * TX + tx] = acc[k];
    __syncthreads();
    for (int h = TY >> 1; h > 0; h >>= 1) {
        if (ty < h) {
#pragma unroll
            for (int k = 0; k < V; ++k)
                lds[(k * TY + ty) * TX + tx] = rop<K, A>(lds[(k * TY + ty) * TX + tx], lds[(k * TY + ty + h) * TX + tx]);
        }
        __syncthreads();
    }
    if constexpr (DEST == 2) return;
    if (ty == 0 && active) {
        Tout *o = out + (p * S + s) * post + cv * V;
#pragma unroll
        for (int k = 0; k < V; ++k) {
            if constexpr (DEST == 1) __hip_atomic_store(o + k, rstore<Tout, A>(lds[(k * TY) * TX + tx]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else o[k] = rstore<Tout, A>(lds[(k * TY) * TX + tx]);
        }
    }
}
// ntl: loads carry the nt hint (chosen per launch, see nt_load_reduce in common.hpp)
template <int K, typename Tin, typename Tout, typename TS, int V>
__global__ __launch_bounds__(kBlock) void reduce_col_kernel(const Tin *__restrict__ in, Tout *__restrict__ out, int64_t pre, int64_t R, int64_t post, int S, int64_t chunk, int TX, int ctiles, int ntl) {
    using A = racc_t<TS>;
    __shared__ A lds[kBlock * V];
    if (ntl) reduce_col_body<K, Tin, Tout, TS, V, true>(lds, in, out, pre, R, post, S, chunk, TX, ctiles);
    else reduce_col_body<K, Tin, Tout, TS, V, false>(lds, in, out, pre, R, post, S, chunk, TX, ctiles);
}

// Split col stage and its second pass in one launch.  `part` [pre, S, post] takes the partial
// tiles as before; `cnt[p * ctiles + ct]` counts the workgroups of output tile (p, ct) that have
// stored theirs.  The partials are stored and loaded with device-scope accesses (written through
// to memory, read past the reader's own L2: the workgroups of a tile run on different XCDs), and
// every lane waits for the acknowledgement of its stores (s_waitcnt vmcnt(0)) before the barrier
// that precedes the count.  A release /
// acquire pair on the counter would do the same by writing back and invalidating whole L2s once
// per workgroup, which cost 30 us of 45 on [8192,8192].  The workgroup that arrives last adds the
// partials in an order fixed by the launch shape, so the result does not depend on which one it
// was, and puts the counter back to zero for the next launch.
template <int K, typename Tin, typename Tfin, typename TS, int V>
__global__ __launch_bounds__(kBlock) void reduce_col_fused_kernel(const Tin *__restrict__ in, racc_t<TS> *part, Tfin *__restrict__ fout, unsigned *cnt,
                                                                    int64_t pre, int64_t R, int64_t post, int S, int64_t chunk, int TX, int ctiles, int ntl) {
    using A = racc_t<TS>;
    __shared__ A lds[kBlock * V];
    __shared__ int is_last;
    if (ntl) reduce_col_body<K, Tin, A, TS, V, true, 1>(lds, in, part, pre, R, post, S, chunk, TX, ctiles);
    else reduce_col_body<K, Tin, A, TS, V, false, 1>(lds, in, part, pre, R, post, S, chunk, TX, ctiles);
    // Every lane waits until its own partial-tile stores have been acknowledged before it enters the
    // barrier.  They are write-through stores (sc1), whose acknowledgement comes from memory, past
    // this XCD's L2: once all lanes are through the barrier the whole tile is in memory, so the count
    // below cannot become visible before the data it announces.  This is the wait an agent-scope
    // release fence would insert, without that fence's write-back of the whole L2.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int ct = (int)(blockIdx.x % ctiles);
    const int64_t p = blockIdx.x / ctiles / S;
    if (threadIdx.x == 0) {
        unsigned *c = cnt + p * ctiles + ct;
        const unsigned old = __hip_atomic_fetch_add(c, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const int last = old == (unsigned)(S - 1);
        if (last) __hip_atomic_store(c, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        is_last = last;
    }
    __syncthreads();
    if (!is_last) return;
    // The partial tiles are read with device-scope loads (sc1: served from memory, never from a stale
    // line of this XCD's L2) that are issued after the count was seen; the compiler may not move
    // them above this point either.
    __atomic_signal_fence(__ATOMIC_SEQ_CST);
    // The S partial tiles are folded like S rows of a col stage: row-lane ty takes slices ty, ty + TY,
    // ... (independent loads, a few in flight), then the same LDS tree across the row-lanes.
    const int TY = kBlock / TX, tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    const int64_t cv = (int64_t)ct * TX + tx;
    const bool active = cv < post / V;
    A acc[V];
#pragma unroll
    for (int k = 0; k < V; ++k) acc[k] = rinit<K, A, TS>();
    if (active) {
        const A *q = part + p * S * post + cv * V;
        auto ld = [&](int s, int k) __attribute__((always_inline)) { return __hip_atomic_load(q + (int64_t)s * post + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); };
        // every load of a batch is issued before the first is used: the partials come from memory
        // (past the L2), and a lane that waited for them one by one would add a memory round trip
        // per slice to the end of the launch
        int s = ty;
        for (; s + 7 * TY < S; s += 8 * TY) {
            A x[8][V];
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int k = 0; k < V; ++k) x[u][k] = ld(s + u * TY, k);
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int k = 0; k < V; ++k) acc[k] = rop<K, A>(acc[k], x[u][k]);
        }
        for (; s + 3 * TY < S; s += 4 * TY) {
            A x[4][V];
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int k = 0; k < V; ++k) x[u][k] = ld(s + u * TY, k);
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int k = 0; k < V; ++k) acc[k] = rop<K, A>(acc[k], x[u][k]);
        }
        for (; s < S; s += TY) {
#pragma unroll
            for (int k = 0; k < V; ++k) acc[k] = rop<K, A>(acc[k], ld(s, k));
        }
    }
#pragma unroll
    for (int k = 0; k < V; ++k) lds[(k * TY + ty) * TX + tx] = acc[k];
    __syncthreads();
    for (int h = TY >> 1; h > 0; h >>= 1) {
        if (ty < h) {
#pragma unroll
            for (int k = 0; k < V; ++k)
                lds[(k * TY + ty) * TX + tx] = rop<K, A>(lds[(k * TY + ty) * TX + tx], lds[(k * TY + ty + h) * TX + tx]);
        }
        __syncthreads();
    }
    if (ty == 0 && active) {
        Tfin *o = fout + p * post + cv * V;
#pragma unroll
        for (int k = 0; k < V; ++k) o[k] = rstore<Tfin, A>(lds[(k * TY) * TX + tx]);
    }
}

// A col stage cut into exactly TWO slices whose accumulate type has 4 bytes and whose op does not care
// which operand comes first (sums and products; integer max / min): the halves meet in one round trip.
// Every output element has a 64-bit slot, zero between launches.  A workgroup swaps (1 << 32 | its value's
// bits) into the slot of each of its elements with one device-scope atomic exchange; what comes back is
// either zero — the other half has not been here, and will find this value — or the other half's value,
// which this workgroup then combines with its own, stores to the output and replaces by zero again.  The
// two halves of a tile may each turn out second for some elements and first for others: every element
// is combined and stored exactly once, by whichever half came second for it, and a op b == b op a makes
// the result the same either way.  Against the counter scheme above (partial stores and their
// acknowledgement, the count, the loads of the partials: three dependent round trips to memory at the end
// of the launch) this is one.
template <int K, typename Tin, typename Tfin, typename TS, int V>
__global__ __launch_bounds__(kBlock) void reduce_col_xchg_kernel(const Tin *__restrict__ in, Tfin *__restrict__ fout, unsigned long long *slots,
                                                                   int64_t pre, int64_t R, int64_t post, int64_t chunk, int TX, int ctiles, int ntl) {
    using A = racc_t<TS>;
    static_assert(sizeof(A) == 4, "value and flag share one 64-bit slot");
    __shared__ A lds[kBlock * V];
    if (ntl) reduce_col_body<K, Tin, A, TS, V, true, 2>(lds, in, nullptr, pre, R, post, 2, chunk, TX, ctiles);
    else reduce_col_body<K, Tin, A, TS, V, false, 2>(lds, in, nullptr, pre, R, post, 2, chunk, TX, ctiles);
    const int TY = kBlock / TX, tx = threadIdx.x % TX, ty = threadIdx.x / TX;
    if (ty != 0) return;  // row-lane 0 holds the tile (the LDS tree ended with a barrier)
    const int ct = (int)(blockIdx.x % ctiles);
    const int64_t p = blockIdx.x / ctiles / 2;
    const int64_t cv = (int64_t)ct * TX + tx;
    if (cv >= post / V) return;
    const int64_t e0 = p * post + cv * V;
    A mine[V];
    unsigned long long got[V];
#pragma unroll
    for (int k = 0; k < V; ++k) {  // all exchanges of the lane are in flight together
        mine[k] = lds[(k * TY) * TX + tx];
        got[k] = __hip_atomic_exchange(slots + e0 + k, (1ull << 32) | (unsigned long long)__builtin_bit_cast(uint32_t, mine[k]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int k = 0; k < V; ++k) {
        if ((got[k] >> 32) == 0) continue;  // first at this element: the other half finishes it
        const A other = __builtin_bit_cast(A, (uint32_t)got[k]);
        fout[e0 + k] = rstore<Tfin, A>(rop<K, A>(mine[k], other));
        __hip_atomic_store(slots + e0 + k, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Counters of reduce_col_fused_kernel: zero at module load, and every launch leaves them zero.
// Kernels of one stream run in order, so an eager stream owns one slice for as long as it is
// known here (dxh_stream_destroy gives it back).  A launch recorded under stream capture may
// later replay on any stream next to eager work, so it takes counters of its own from the
// second half of the array: they belong to the graph that the capture ends in and return to the
// pool when that graph is destroyed (counter_ranges.hpp; dxh_graph_end_capture and
// dxh_graph_destroy report both events here).  When either half is used up the caller falls back
// to two launches.
constexpr int kFinishSlice = 32768, kFinishSlices = 32, kFinishCounters = 2 * kFinishSlice * kFinishSlices;  // 8 MiB: a launch that finishes by exchange takes two words per output element
static __device__ __align__(256) unsigned g_finish_counters[kFinishCounters];
namespace {
struct FinishState {
    unsigned *base = nullptr;
    bool resolved = false;
    std::map<hipStream_t, int> slice;
    std::vector<int> free_slices;
    int slices_used = 0;
    CounterRanges captured{(int64_t)kFinishSlice * kFinishSlices, kFinishCounters};
};
std::mutex g_finish_mutex;
std::map<int, FinishState> g_finish;  // by device
}  // namespace

unsigned *finish_counters(hipStream_t st, int64_t need) {
    if (need > kFinishSlice || !tuning().reduce_fused_finish) return nullptr;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    const bool capturing = stream_is_capturing(st);
    std::lock_guard<std::mutex> lock(g_finish_mutex);
    FinishState &f = g_finish[dev];
    if (!f.resolved) {
        if (capturing) return nullptr;  // nothing but launches while a capture is open
        f.resolved = true;
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_finish_counters)) != hipSuccess) { (void)hipGetLastError(); ptr = nullptr; }
        f.base = (unsigned *)ptr;
    }
    if (!f.base) return nullptr;
    need = (need + 1) & ~(int64_t)1;  // ranges start on even words: a launch may use its words in pairs, as 64-bit slots
    if (capturing) {
        const int64_t off = f.captured.take_for_capture((const void *)st, need);
        return off < 0 ? nullptr : f.base + off;
    }
    auto it = f.slice.find(st);
    if (it == f.slice.end()) {
        int idx;
        if (!f.free_slices.empty()) { idx = f.free_slices.back(); f.free_slices.pop_back(); }
        else if (f.slices_used < kFinishSlices) idx = f.slices_used++;
        else return nullptr;
        it = f.slice.emplace(st, idx).first;
    }
    return f.base + (int64_t)it->second * kFinishSlice;
}

// graph == nullptr: the capture on `st` failed and no graph will ever replay its launches
void finish_capture_ended(hipStream_t st, const void *graph) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return; }
    std::lock_guard<std::mutex> lock(g_finish_mutex);
    auto d = g_finish.find(dev);
    if (d != g_finish.end()) d->second.captured.capture_ended((const void *)st, graph);
}
void finish_graph_destroyed(const void *graph) {
    std::lock_guard<std::mutex> lock(g_finish_mutex);
    for (auto &d : g_finish) d.second.captured.graph_destroyed(graph);
}
void finish_capture_stats(int64_t *in_use, int64_t *capacity) {
    int dev = 0;
    *in_use = 0;
    *capacity = (int64_t)kFinishCounters - (int64_t)kFinishSlice * kFinishSlices;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return; }
    std::lock_guard<std::mutex> lock(g_finish_mutex);
    auto d = g_finish.find(dev);
    if (d != g_finish.end()) *in_use = d->second.captured.in_use();
}

void reduce_stream_release(hipStream_t st) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return; }
    std::lock_guard<std::mutex> lock(g_finish_mutex);
    auto d = g_finish.find(dev);
    if (d == g_finish.end()) return;
    auto it = d->second.slice.find(st);
    if (it == d->second.slice.end()) return;
    d->second.free_slices.push_back(it->second);
    d->second.slice.erase(it);
}

// fill `n` outputs with the identity (a reduced axis of size 0), or copy (nothing to reduce)
template <int K, typename TS>
__global__ __launch_bounds__(kBlock) void reduce_fill_kernel(TS *__restrict__ out, int64_t n) {
    using A = racc_t<TS>;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) out[i] = rstore<TS, A>(rinit<K, A, TS>());
}

// ---- host-side plan ----------------------------------------------------------------------
struct Stage {
    bool row;            // row stage (post == 1) or col stage
    int64_t pre, R, post;
    int S;               // chunks of R
    int64_t chunk;
    int G;               // row: lanes per row
    int TX, ctiles;      // col: column lanes, column tiles
    int tx_pref;         // col: column lanes fixed by the planner (0: col_lanes decides)
    int V;               // vector length in elements of the stage's input type (1 or 16/size)
    bool may_split;      // col stage: parallelism may come from splitting R
    bool in_is_acc, out_is_acc;
    size_t out_off;      // offset of the output inside the workspace when out_is_acc
};
struct Plan {
    int64_t nout = 0, nred = 1;
    bool copy_only = false;
    std::vector<Stage> stages;
    size_t ws_bytes = 0;
};

inline int pow2_ceil(int64_t x) { int p = 1; while (p < x && p < (1 << 30)) p <<= 1; return p; }

// Column-lane count of a col stage: as wide as the tuning allows (long contiguous row segments),
// narrowed while that leaves fewer workgroups than CUs.  A stage that may still split R stops at
// 32 lanes (512-byte segments) and gets the rest of its parallelism from the split; the second
// pass over partials cannot split and narrows down to 16.
inline int col_lanes(int64_t pre, int64_t postv, bool may_split) {
    int tx = (int)std::min<int64_t>(tuning().reduce_col_max_lanes, pow2_ceil(postv));
    const int floor_tx = may_split ? 32 : 16;
    while (tx > floor_tx && pre * ((postv + tx - 1) / tx) < kCUs) tx >>= 1;
    return tx;
}

// normalise dims like checkedDims (shape_reduce.cpp:11-45); returns false if out of range
inline bool reduced_mask(int ndim, const int32_t *dims, int ndims, bool *mask) {
    for (int i = 0; i < ndim; ++i) mask[i] = (ndims == 0);
    for (int i = 0; i < ndims; ++i) {
        int d = dims[i];
        if (d < 0) d += ndim;
        if (d < 0 || d >= ndim) return false;
        mask[d] = true;
    }
    return true;
}

inline int build_plan(int esize, int asize, const int32_t *shape, int ndim, const int32_t *dims, int ndims, Plan &pl) {
    if (!shape || ndim < 1 || ndim > DXH_MAX_DIMS || ndims < 0 || (ndims > 0 && !dims)) return DXH_ERR_ARG;
    bool mask[DXH_MAX_DIMS];
    if (!reduced_mask(ndim, dims, ndims, mask)) return DXH_ERR_ARG;
    struct D { int64_t n; bool red; };
    std::vector<D> d;
    pl.nout = 1; pl.nred = 1;
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] < 0) return DXH_ERR_ARG;
        if (mask[i]) pl.nred *= shape[i]; else pl.nout *= shape[i];
        if (shape[i] == 1) continue;
        if (!d.empty() && d.back().red == mask[i]) d.back().n *= shape[i];
        else d.push_back({shape[i], mask[i]});
    }
    if (pl.nout == 0 || pl.nred == 0) return DXH_OK;  // nothing to read
    bool any = false;
    for (auto &x : d) any |= x.red;
    if (!any) { pl.copy_only = true; return DXH_OK; }

    const int64_t kTarget = tuning().reduce_target_blocks;
    bool first = true;
    size_t off = 0;
    auto push = [&](Stage st, bool last) {
        st.in_is_acc = !first;
        st.out_is_acc = !last;
        const int in_size = st.in_is_acc ? asize : esize;
        const int vfull = kVecBytes / in_size;
        if (st.row) {
            // vector loads need every row chunk to start on a 16-byte boundary
            st.V = (st.R % vfull == 0 && st.chunk % vfull == 0) ? vfull : 1;
        } else {
            st.V = (st.post % vfull == 0) ? vfull : 1;
            int64_t postv = st.post / st.V;
            st.TX = st.tx_pref ? st.tx_pref : col_lanes(st.pre, postv, st.may_split);
            st.ctiles = (int)((postv + st.TX - 1) / st.TX);
        }
        if (st.out_is_acc) {
            st.out_off = off;
            size_t bytes = (size_t)(st.pre * st.S * st.post) * asize;
            off += (bytes + 255) & ~(size_t)255;
        }
        pl.stages.push_back(st);
        first = false;
    };

    while (true) {
        int p = -1, groups = 0;
        for (int i = 0; i < (int)d.size(); ++i) if (d[i].red) { p = i; ++groups; }
        if (p < 0) break;
        int64_t pre = 1, post = 1;
        for (int i = 0; i < p; ++i) pre *= d[i].n;
        for (int i = p + 1; i < (int)d.size(); ++i) post *= d[i].n;
        const int64_t R = d[p].n;
        const bool last_group = groups == 1;
        Stage st{};
        st.pre = pre; st.R = R; st.post = post; st.row = (post == 1);
        const int in_size = pl.stages.empty() ? esize : asize;
        const int vfull = kVecBytes / in_size;
        int S = 1;
        if (st.row) {
            // lanes per row: one 16-byte vector per lane per trip, up to the whole workgroup
            int64_t vecs = (R + vfull - 1) / vfull;
            // each lane should have several independent 16-byte loads of its own: the whole
            // workgroup on one row only when that still leaves `loads` vectors per lane, else a
            // sub-wave group of lanes per row and 256/G rows per workgroup
            const int64_t loads = tuning().reduce_row_loads;
            int G = vecs >= (int64_t)kBlock * loads ? kBlock : (int)std::min<int64_t>(kWave, pow2_ceil((vecs + loads - 1) / loads));
            // very short rows: at least 4 lanes (64 contiguous bytes) per row keep a wave's loads coalesced
            G = std::max<int>(G, (int)std::min<int64_t>(4, pow2_ceil(vecs)));
            // a small input: rather fewer vectors per lane than fewer workgroups than two per CU
            // (fp32 [8192,64]: 4 lanes per row make 128 workgroups, 16 lanes per row 512)
            while (G < kWave && G < pow2_ceil(vecs) && (pre + (kBlock / G) - 1) / (kBlock / G) < 2 * kCUs) G <<= 1;
            int64_t blocks0 = (pre + (kBlock / G) - 1) / (kBlock / G);
            if (G == kBlock && blocks0 < kTarget) {
                int64_t min_chunk = 8192;  // elements: 8+ vector trips per lane
                int64_t smax = std::max<int64_t>(1, R / min_chunk);
                S = (int)std::min<int64_t>((kTarget + blocks0 - 1) / blocks0, smax);
            }
            st.G = G;
        } else {
            int V = (post % vfull == 0) ? vfull : 1;
            int64_t postv = post / V;
            st.may_split = true;
            int TX = col_lanes(pre, postv, true);
            int TY = kBlock / TX;
            int64_t blocks0 = pre * ((postv + TX - 1) / TX);
            // One workgroup per CU is the fastest split when it comes out as a single full round
            // (fp32 [8192,8192]: 64 column tiles x 4 slices = 256 workgroups, 44 us; 45 us with 1024).
            // When the tiles do not divide the CUs like that, a few workgroups too many would run
            // as a second, nearly empty round: then four times as many, smaller ones keep every CU
            // busy to the end (fp32 [8192,8256]: 260 workgroups 60 us, 1040 workgroups 49 us).
            int64_t col_target = tuning().reduce_col_target_blocks;
            const int64_t min_rows = (int64_t)TY * tuning().reduce_col_min_rows;
            const int64_t smax = std::max<int64_t>(1, R / min_rows);
            if (blocks0 < col_target) {
                S = (int)std::min<int64_t>((col_target + blocks0 - 1) / blocks0, smax);
                if (blocks0 * S > col_target && col_target == kCUs) {
                    col_target *= 4;
                    S = (int)std::min<int64_t>((col_target + blocks0 - 1) / blocks0, smax);
                }
            }
            // Four slices of 512-byte strips or two slices of 256-byte strips are the same number of workgroups
            // and stream alike (fp32 [8192,8192]: 44.2 and 43.4 us with the counted finish); two slices can
            // finish by one exchange per element instead of three round trips (reduce_col_xchg_kernel).
            if (S == 4 && TX == 32 && V == vfull && tuning().reduce_fused_finish == 1) { st.tx_pref = 16; S = 2; }
            if (S == 1) st.may_split = false;  // nothing to split: narrow TX for parallelism instead
        }
        st.S = S;
        int64_t chunk = (R + S - 1) / S;
        chunk = (chunk + vfull - 1) / vfull * vfull;  // keep chunk starts vector aligned
        st.chunk = chunk;
        st.S = (int)((R + chunk - 1) / chunk);
        push(st, last_group && st.S == 1);
        if (st.S > 1) {
            // second pass over the S partials: [pre, S, post]
            Stage s2{};
            s2.pre = pre; s2.R = st.S; s2.post = post; s2.row = (post == 1); s2.S = 1; s2.chunk = st.S;
            if (s2.row) {
                int64_t vecs = (s2.R + (kVecBytes / asize) - 1) / (kVecBytes / asize);
                s2.G = vecs >= 2 * kWave ? kBlock : (int)std::min<int64_t>(kWave, pow2_ceil(vecs));
            }
            push(s2, last_group);
        }
        // drop the reduced group and re-merge the kept neighbours
        d.erase(d.begin() + p);
        if (p > 0 && p < (int)d.size() && !d[p - 1].red && !d[p].red) { d[p - 1].n *= d[p].n; d.erase(d.begin() + p); }
    }
    pl.ws_bytes = off;
    return DXH_OK;
}

int reduce_rows_group(int esize, int64_t rows, int64_t cols) {
    if (rows < 1 || cols < 1 || rows > INT32_MAX || cols > INT32_MAX || (esize != 4 && esize != 2)) return 0;
    const int32_t shape[2] = {(int32_t)rows, (int32_t)cols}, dims[1] = {1};
    Plan pl;
    if (build_plan(esize, sizeof(float), shape, 2, dims, 1, pl) != DXH_OK || pl.copy_only || pl.stages.size() != 1) return 0;
    const Stage &st = pl.stages[0];
    if (!st.row || st.S != 1 || st.V != kVecBytes / esize || st.G > kWave || st.pre != rows || st.R != cols) return 0;
    return st.G;
}
int sum_rows_group_f32(int64_t rows, int64_t cols) { return reduce_rows_group((int)sizeof(float), rows, cols); }

template <int K, typename Tin, typename Tout, typename TS>
int launch_stage(const Stage &st, const void *in, void *out, hipStream_t stream) {
    constexpr int VF = kVecBytes / (int)sizeof(Tin);
    const size_t in_bytes = (size_t)(st.pre * st.R * st.post) * sizeof(Tin);
    const int ntl = st.row ? nt_load_reduce(in_bytes) : nt_load_reduce_col(in_bytes);
    if (st.row) {
        const int rows_per_block = kBlock / st.G;
        int64_t gx = (st.pre + rows_per_block - 1) / rows_per_block;
        if (gx > 0x7fffffff || st.S > 65535) return DXH_ERR_SHAPE;
        dim3 grid((unsigned)gx, (unsigned)st.S);
        if (st.V == VF && aligned(in, kVecBytes))
            reduce_row_kernel<K, Tin, Tout, TS, VF><<<grid, kBlock, 0, stream>>>((const Tin *)in, (Tout *)out, st.pre, st.R, st.S, st.chunk, st.G, ntl);
        else
            reduce_row_kernel<K, Tin, Tout, TS, 1><<<grid, kBlock, 0, stream>>>((const Tin *)in, (Tout *)out, st.pre, st.R, st.S, st.chunk, st.G, ntl);
    } else {
        bool vec = st.V == VF && aligned(in, kVecBytes);
        int TX = st.TX, ctiles = st.ctiles;
        if (!vec && st.V != 1) {  // planned for vectors but the pointer is misaligned
            TX = col_lanes(st.pre, st.post, st.may_split);
            ctiles = (int)((st.post + TX - 1) / TX);
        }
        int64_t gx = st.pre * st.S * ctiles;
        if (gx > 0x7fffffff) return DXH_ERR_SHAPE;
        if (vec)
            reduce_col_kernel<K, Tin, Tout, TS, VF><<<(unsigned)gx, kBlock, 0, stream>>>((const Tin *)in, (Tout *)out, st.pre, st.R, st.post, st.S, st.chunk, TX, ctiles, ntl);
        else
            reduce_col_kernel<K, Tin, Tout, TS, 1><<<(unsigned)gx, kBlock, 0, stream>>>((const Tin *)in, (Tout *)out, st.pre, st.R, st.post, st.S, st.chunk, TX, ctiles, ntl);
    }
    return launch_status();
}

// Split col stage `st` over the caller's input together with its second pass `s2`: one launch
// when counters are to be had.  Returns kNotFused when the pair has to run as two launches.
constexpr int kNotFused = -1003;
template <int K, typename Tfin, typename TS>
int launch_fused_col(const Stage &st, const void *in, void *part, void *fout, hipStream_t stream) {
    using A = racc_t<TS>;
    constexpr int VF = kVecBytes / (int)sizeof(TS);
    if (st.V != VF || !aligned(in, kVecBytes)) return kNotFused;
    const int64_t gx = st.pre * st.S * st.ctiles;
    if (gx > 0x7fffffff) return kNotFused;
    const int ntl = nt_load_reduce_col((size_t)(st.pre * st.R * st.post) * sizeof(TS));
    // two slices of a 4-byte accumulator under an op that commutes bit for bit: one exchange per element
    if constexpr (sizeof(A) == 4 && (K == R_SUM || K == R_PROD || std::is_integral_v<A>)) {
        if (st.S == 2 && 2 * st.pre * st.post <= kFinishSlice && tuning().reduce_fused_finish == 1) {
            if (unsigned *words = finish_counters(stream, 2 * st.pre * st.post)) {
                reduce_col_xchg_kernel<K, TS, Tfin, TS, VF><<<(unsigned)gx, kBlock, 0, stream>>>((const TS *)in, (Tfin *)fout, reinterpret_cast<unsigned long long *>(words), st.pre, st.R, st.post, st.chunk, st.TX, st.ctiles, ntl);
                return launch_status();
            }
        }
    }
    unsigned *cnt = finish_counters(stream, st.pre * st.ctiles);
    if (!cnt) return kNotFused;
    reduce_col_fused_kernel<K, TS, Tfin, TS, VF><<<(unsigned)gx, kBlock, 0, stream>>>((const TS *)in, (A *)part, (Tfin *)fout, cnt, st.pre, st.R, st.post, st.S, st.chunk, st.TX, st.ctiles, ntl);
    return launch_status();
}

template <int K, typename TS>
int reduce_typed(const void *in, const int32_t *shape, int ndim, const int32_t *dims, int ndims, void *out,
                 void *workspace, size_t workspace_bytes, hipStream_t stream) {
    using A = racc_t<TS>;
    Plan pl;
    int rc = build_plan(sizeof(TS), sizeof(A), shape, ndim, dims, ndims, pl);
    if (rc != DXH_OK) return rc;
    if (pl.nout == 0) return DXH_OK;
    if (!out) return DXH_ERR_ARG;
    if (!aligned(out, sizeof(TS))) return DXH_ERR_ALIGN;
    if (pl.nred == 0) {
        reduce_fill_kernel<K, TS><<<stream_grid(pl.nout, kBlock, 8), kBlock, 0, stream>>>((TS *)out, pl.nout);
        return launch_status();
    }
    if (!in) return DXH_ERR_ARG;
    if (!aligned(in, sizeof(TS))) return DXH_ERR_ALIGN;
    if (pl.copy_only) {
        if (in == out) return DXH_OK;
        return (int)hipMemcpyAsync(out, in, (size_t)pl.nout * sizeof(TS), hipMemcpyDeviceToDevice, stream);
    }
    if (pl.ws_bytes > 0 && (!workspace || workspace_bytes < pl.ws_bytes || !aligned(workspace, 256))) return DXH_ERR_WORKSPACE;
    const void *cur = in;
    for (size_t i = 0; i < pl.stages.size(); ++i) {
        const Stage &st = pl.stages[i];
        void *dst = st.out_is_acc ? (void *)((char *)workspace + st.out_off) : out;
        if (!st.row && st.S > 1 && !st.in_is_acc && i + 1 < pl.stages.size()) {
            const Stage &s2 = pl.stages[i + 1];  // the pass over this stage's S partials
            void *fin = s2.out_is_acc ? (void *)((char *)workspace + s2.out_off) : out;
            rc = s2.out_is_acc ? launch_fused_col<K, A, TS>(st, cur, dst, fin, stream) : launch_fused_col<K, TS, TS>(st, cur, dst, fin, stream);
            if (rc != kNotFused) {
                if (rc != DXH_OK) return rc;
                cur = fin;
                ++i;
                continue;
            }
        }
        if (!st.in_is_acc && !st.out_is_acc) rc = launch_stage<K, TS, TS, TS>(st, cur, dst, stream);
        else if (!st.in_is_acc && st.out_is_acc) rc = launch_stage<K, TS, A, TS>(st, cur, dst, stream);
        else if (st.in_is_acc && st.out_is_acc) rc = launch_stage<K, A, A, TS>(st, cur, dst, stream);
        else rc = launch_stage<K, A, TS, TS>(st, cur, dst, stream);
        if (rc != DXH_OK) return rc;
        cur = dst;
    }
    return DXH_OK;
}

template <int K>
int reduce_all(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims, int ndims, void *out,
               void *ws, size_t wsb, void *stream) {
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return reduce_typed<K, double>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    case DXH_F32: return reduce_typed<K, float>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    case DXH_F16: return reduce_typed<K, f16_t>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    case DXH_BF16: return reduce_typed<K, bf16_t>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    case DXH_I64: return reduce_typed<K, int64_t>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    case DXH_I32: return reduce_typed<K, int32_t>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    case DXH_I16: return reduce_typed<K, int16_t>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    case DXH_I8: return reduce_typed<K, int8_t>(in, shape, ndim, dims, ndims, out, ws, wsb, st);
    default: return DXH_ERR_DTYPE;
    }
}

}  // namespace dxh

using namespace dxh;

extern "C" {

int dxh_reduce_workspace_bytes(int dtype, const int32_t *shape, int ndim, const int32_t *dims, int ndims, size_t *bytes) {
    if (!bytes) return DXH_ERR_ARG;
    *bytes = 0;
    int es = dtype_size(dtype);
    if (!es || dtype == DXH_BOOL) return DXH_ERR_DTYPE;
    int as = (dtype == DXH_F64 || dtype == DXH_I64) ? 8 : 4;
    Plan pl;
    int rc = build_plan(es, as, shape, ndim, dims, ndims, pl);
    if (rc != DXH_OK) return rc;
    *bytes = pl.ws_bytes;
    return DXH_OK;
}

int dxh_sum(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims, int ndims, void *out,
            void *workspace, size_t workspace_bytes, void *stream) {
    return reduce_all<R_SUM>(dtype, in, shape, ndim, dims, ndims, out, workspace, workspace_bytes, stream);
}
int dxh_prod(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims, int ndims, void *out,
             void *workspace, size_t workspace_bytes, void *stream) {
    return reduce_all<R_PROD>(dtype, in, shape, ndim, dims, ndims, out, workspace, workspace_bytes, stream);
}
int dxh_reducemax(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims, int ndims, void *out,
                  void *workspace, size_t workspace_bytes, void *stream) {
    return reduce_all<R_MAX>(dtype, in, shape, ndim, dims, ndims, out, workspace, workspace_bytes, stream);
}
int dxh_reducemin(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims, int ndims, void *out,
                  void *workspace, size_t workspace_bytes, void *stream) {
    return reduce_all<R_MIN>(dtype, in, shape, ndim, dims, ndims, out, workspace, workspace_bytes, stream);
}

}  // extern "C"

// ---- dxh_sum for callers that cannot allocate ---------------------------------------------
// The partial results that dxh_sum keeps in the caller's workspace live here in a file-scope
// device array instead: one copy per GPU, held until the process ends.  In host code the array's
// name is only a stand-in for the symbol; its device address is looked up once per device with
// hipGetSymbolAddress (that device current) and only that pointer is ever handed to a kernel.
// Nothing in it has to start at zero: a stage writes every partial it later reads.  Calls that
// overlap on one GPU (two streams, two threads) share the array and race.
constexpr size_t kScratchBytes = (size_t)4 << 20;
static_assert(kScratchBytes == DXH_SUM_NOALLOC_SCRATCH_BYTES, "the limit is part of the ABI");
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];
bool g_scratch_resolved[kMaxDevices];
}  // namespace

namespace dxh {
// Device address of `scratch` on the current device; looked up on the first call per device.
// The lookup is not a stream operation and is refused while `st` is being captured.
int scratch_pointer(hipStream_t st, bool may_be_capturing, void **ptr) {
    *ptr = nullptr;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { (void)hipGetLastError(); return (int)e; }
    if (dev < 0 || dev >= kMaxDevices) return DXH_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_resolved[dev]) {
        if (may_be_capturing && stream_is_capturing(st)) return DXH_ERR_NOT_READY;
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) { (void)hipGetLastError(); return (int)e; }
        g_scratch_ptr[dev] = p;
        g_scratch_resolved[dev] = true;
    }
    *ptr = g_scratch_ptr[dev];
    return DXH_OK;
}
// dxh_set_device is the library's set-up call for a device: both file-scope arrays are resolved
// there, so that a first reduction under stream capture finds them ready.
void reduce_device_init() {
    void *p = nullptr;
    (void)scratch_pointer(nullptr, false, &p);
    (void)finish_counters(nullptr, 1);
}
}  // namespace dxh

extern "C" int dxh_sum_noalloc(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *dims, int ndims, void *out,
                    void *stream) {
    size_t need = 0;
    int rc = dxh_reduce_workspace_bytes(dtype, shape, ndim, dims, ndims, &need);
    if (rc != DXH_OK) return rc;
    if (need > kScratchBytes) return DXH_ERR_TOO_LARGE;
    void *ws = nullptr;
    rc = scratch_pointer(as_stream(stream), true, &ws);
    if (rc != DXH_OK) return rc;
    return reduce_all<R_SUM>(dtype, in, shape, ndim, dims, ndims, out, ws, kScratchBytes, stream);
}
