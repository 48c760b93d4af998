// matmul_common.hpp — pieces shared by the matrix-pipe GEMM kernels: vector typedefs, compile-time
// loops, the XCD-aware workgroup -> tile map and the launch-side helpers.
#pragma once
#include <utility>
#include "common.hpp"

namespace dxh {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // native vector: arrays of it stay in registers
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F> __device__ __forceinline__ void static_for(F f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }
template <int V> using ic = std::integral_constant<int, V>;

// Issue order inside a scheduling region of a matrix-pipe kernel: after each of `mfmas` MFMAs an
// even share of the region's LDS reads, LDS writes and global loads (counts are upper bounds: a
// paired ds_read2 counts once), so that the matrix pipe always has the next MFMA queued while the
// memory instructions are issued underneath it.  Left alone, the compiler reads each operand
// right before the MFMA that uses it and the pipe idles for an LDS latency every few MFMAs.
template <typename M, typename R, typename W, typename L>
__device__ __forceinline__ void interleave(M, R, W, L) {
    constexpr int nm = M::value, nr = R::value, nw = W::value, nl = L::value;
    static_for<nm>([&](auto x) __attribute__((always_inline)) {
        constexpr int m = decltype(x)::value;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
        constexpr int r = nr * (m + 1) / nm - nr * m / nm, wr = nw * (m + 1) / nm - nw * m / nm, l = nl * (m + 1) / nm - nl * m / nm;
        if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);   // LDS reads
        if constexpr (wr > 0) __builtin_amdgcn_sched_group_barrier(0x200, wr, 0);  // LDS writes
        if constexpr (l > 0) __builtin_amdgcn_sched_group_barrier(0x020, l, 0);   // global loads
    });
}


// ---- XCD-aware workgroup -> tile map (shared by the MFMA kernels) ---------------------------
// Workgroups are dealt round-robin to the 8 XCDs, each with a private L2.  XCD x takes the
// contiguous range [x*chunk, (x+1)*chunk) of a grouped tile order (group_m tile rows at a time,
// column-major inside a group), i.e. a compact, roughly square patch of C whose A and B panels
// fit its L2.  The grid is 8*chunk workgroups; those past the last tile exit at once.
struct TileMap { int tiles_m, tiles_n, total, chunk, group_m; };
struct TileCoord { int batch, tm, tn; bool valid; };
inline bool make_tile_map(int64_t batch, int64_t m, int64_t n, int tm, int tn, TileMap &map) {
    const int64_t tiles_m = (m + tm - 1) / tm, tiles_n = (n + tn - 1) / tn, total = batch * tiles_m * tiles_n;
    if (total > 0x0fffffff) return false;
    map.tiles_m = (int)tiles_m; map.tiles_n = (int)tiles_n; map.total = (int)total;
    map.chunk = (int)((total + 7) / 8);
    int group_m = 1;  // tile rows per group: the chunk of one XCD should cover a roughly square patch of C
    while ((int64_t)(group_m + 1) * (group_m + 1) * tm <= (int64_t)map.chunk * tn && group_m + 1 <= tiles_m) ++group_m;
    map.group_m = group_m;
    return true;
}
__device__ __forceinline__ TileCoord tile_of_block(const TileMap &map) {
    TileCoord c;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    int logical = xcd * map.chunk + slot;
    c.valid = logical < map.total;
    const int per_batch = map.tiles_m * map.tiles_n;
    c.batch = logical / per_batch;
    logical -= c.batch * per_batch;
    const int in_group = map.group_m * map.tiles_n;
    const int first_m = (logical / in_group) * map.group_m;
    const int size_m = (map.tiles_m - first_m < map.group_m) ? map.tiles_m - first_m : map.group_m;
    const int within = logical % in_group;
    c.tm = first_m + within % size_m;
    c.tn = within / size_m;
    return c;
}

inline int compute_units() {
    static const int cus = [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) {
            (void)hipGetLastError();
            v = 256;
        }
        return v;
    }();
    return cus;
}


// ---- device scratch of one matmul call ---------------------------------------------------------
// Partial tiles of a product cut along K and zero-padded operand copies live in the caller's
// workspace (dxh_matmul's `workspace` argument); nothing here allocates.  The launchers carve what
// they need from it with take().  dxh_matmul_workspace_bytes runs the same launchers in planning
// mode: every decision is taken as for a real call, take() only adds up, and no kernel is launched.
struct Scratch {
    char *base = nullptr;
    size_t bytes = 0, used = 0;
    bool planning = false;
    void *take(size_t n) {
        n = (n + 255) & ~(size_t)255;
        const size_t off = used;
        used += n;
        if (planning) return reinterpret_cast<void *>((uintptr_t)256);  // aligned, never dereferenced
        return (base && used <= bytes) ? base + off : nullptr;
    }
};

// ---- split-K -------------------------------------------------------------------------------
// A product with few output tiles and a long K leaves most CUs idle.  Such a product is cut along
// K into `splits` slices of `ksub` (a multiple of the kernel's K step): the slice of workgroup
// batch index x is x % splits of batch x / splits, its partial tile goes to the call's scratch in
// the accumulator type, laid out [batch][split][M][N], and splitk_reduce_kernel adds the slices in
// slice order (same result on every run, eager or replayed from a graph) and rounds once to the
// output type.  Cutting pays for a second launch only when the uncut K loop is long: K >= min_k,
// slices of at least min_k / 4.
struct KSplit { int splits, ksub; };
// No plan asks for more scratch than this: 1 GiB of 288 (padded copies of a [2048,768]x[768,50257]
// bf16 product need 283 MB); beyond it a product stays uncut / takes the element-wise kernel.
constexpr int64_t kWorkspaceMaxBytes = (int64_t)1 << 30;
inline KSplit choose_ksplit(int64_t tiles, int64_t k, int kstep, int64_t min_k, int64_t partial_bytes) {
    KSplit r{1, (int)k};
    const int64_t cus = compute_units(), ksteps = (k + kstep - 1) / kstep, knob = tuning().matmul_splitk;
    int64_t want;
    if (knob == 1) return r;
    if (knob >= 2) {
        want = knob;
    } else {
        if (tiles * 2 > cus || k < min_k) return r;
        want = (2 * cus + tiles - 1) / tiles;  // two workgroups per CU
        if (want > 4 * k / min_k) want = 4 * k / min_k;
    }
    if (want > ksteps) want = ksteps;
    if (want > 1024) want = 1024;
    if (want < 2 || want * partial_bytes > kWorkspaceMaxBytes) return r;
    const int64_t per = (ksteps + want - 1) / want;
    r.ksub = (int)(per * kstep);
    r.splits = (int)((k + r.ksub - 1) / r.ksub);
    if (r.splits < 2) return KSplit{1, (int)k};
    return r;
}

template <typename TA, typename TO> __device__ __forceinline__ TO splitk_round(TA v) {
    if constexpr (std::is_same_v<TA, TO>) return v;
    else return store_acc<TO>(v);
}
// out[b][e] = sum over s (ascending) of ws[b][s][e]; one element per lane and trip (coalesced)
template <typename TA, typename TO>
__global__ __launch_bounds__(kBlock) void splitk_reduce_kernel(const TA *__restrict__ ws, TO *__restrict__ out, int splits, int64_t mn, int64_t total) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
        const int64_t b = i / mn, e = i - b * mn;
        const TA *p = ws + b * splits * mn + e;
        TA acc = p[0];
        for (int s = 1; s < splits; ++s) acc += p[(int64_t)s * mn];
        out[i] = splitk_round<TA, TO>(acc);
    }
}
template <typename TA, typename TO>
int launch_splitk_reduce(const TA *ws, TO *out, int64_t batch, int64_t mn, int splits, hipStream_t st) {
    const int64_t total = batch * mn;
    int64_t blocks = (total + kBlock - 1) / kBlock;
    if (blocks > 8192) blocks = 8192;
    splitk_reduce_kernel<TA, TO><<<(unsigned)blocks, kBlock, 0, st>>>(ws, out, splits, mn, total);
    return launch_status();
}

// ---- rows that are not 16-byte aligned (odd K or N, unaligned bases) ---------------------------
// The matrix-pipe kernels want 16-byte rows.  Such a product runs on zero-padded copies instead: A
// to [M][Kp], B to [Kp][Np] (Kp, Np the next multiples of 16 bytes) and the kernel on those, which
// writes its [M][N] result element by element at C's own pitch.  The copies move A and B once more
// through HBM, a fraction of what element-wise loads lose (bf16 2047x895x4863: 197 -> 42 us).
// E: unsigned integer of the element size.  kNoSplit: not done (operands over the scratch
// limit, tiny products), the caller takes its other path.
constexpr int kNoSplit = -1001;  // not a DXH_ERR_* value
// out[b][r][c] = (r < rows_in && c < cols_in) ? in[b][r][c] : 0, one 16-byte chunk of out per lane
template <typename E>
__global__ __launch_bounds__(kBlock) void pad_rows_kernel(const E *__restrict__ in, E *__restrict__ out, int64_t rows_in, int64_t cols_in,
                                                          int64_t rows_out, int64_t chunks_out, int64_t total) {
    constexpr int V = kVecBytes / (int)sizeof(E);
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
        const int64_t ch = i % chunks_out, r = (i / chunks_out) % rows_out, b = i / (chunks_out * rows_out);
        const E *p = in + (b * rows_in + r) * cols_in + ch * V;
        vec_t<E, V> x;
#pragma unroll
        for (int e = 0; e < V; ++e) x.v[e] = (r < rows_in && ch * V + e < cols_in) ? p[e] : (E)0;
        *reinterpret_cast<vec_t<E, V> *>(out + i * V) = x;
    }
}
// The same for 2-byte elements, whose source chunks start on any 2-byte boundary: a lane reads
// the aligned dwords that cover its 8 elements (one 16-byte load that only needs 4-byte alignment,
// plus one dword when the chunk starts in the upper half of a dword) and shifts, instead of eight
// 2-byte loads.  Only dwords that hold at least one wanted element are read, so no load leaves
// the pages of the source.
inline unsigned copy_blocks(int64_t total);
typedef uint32_t u32x4_a4_t __attribute__((ext_vector_type(4), aligned(4)));
template <int UNUSED = 0>  // a template only so that the header can define it
__global__ __launch_bounds__(kBlock) void pad_rows16_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out, int64_t rows_in, int64_t cols_in,
                                                            int64_t rows_out, int64_t chunks_out, int64_t total) {
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
        const int64_t ch = i % chunks_out, r = (i / chunks_out) % rows_out, b = i / (chunks_out * rows_out);
        const int64_t left = cols_in - ch * 8;  // elements of the source row from this chunk on
        u32x4_t x = {0u, 0u, 0u, 0u};
        if (r < rows_in && left > 0) {
            const uint16_t *p = in + (b * rows_in + r) * cols_in + ch * 8;
            const bool odd = (reinterpret_cast<uintptr_t>(p) & 2) != 0;
            const uint32_t *q = reinterpret_cast<const uint32_t *>(p - (odd ? 1 : 0));  // the dword that holds p[0]
            uint32_t d[5] = {0u, 0u, 0u, 0u, 0u};
            if (left >= 8) {
                const u32x4_t v = *reinterpret_cast<const u32x4_a4_t *>(q);
                d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
                if (odd) d[4] = q[4];
            } else {
                const int dwords = ((odd ? 1 : 0) + (int)left + 1) / 2;
#pragma unroll
                for (int j = 0; j < 5; ++j)
                    if (j < dwords) d[j] = q[j];
            }
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                o[j] = odd ? (d[j] >> 16) | (d[j + 1] << 16) : d[j];
                if (left < 8) o[j] &= (2 * j < left ? 0xffffu : 0u) | (2 * j + 1 < left ? 0xffff0000u : 0u);
            }
            x = u32x4_t{o[0], o[1], o[2], o[3]};
        }
        *reinterpret_cast<u32x4_t *>(out + i * 8) = x;
    }
}
template <typename E>
inline void launch_pad_rows(const E *in, E *out, int64_t rows_in, int64_t cols_in, int64_t rows_out, int64_t chunks_out, int64_t total, hipStream_t st) {
    if constexpr (sizeof(E) == 2)
        pad_rows16_kernel<0><<<copy_blocks(total), kBlock, 0, st>>>((const uint16_t *)in, (uint16_t *)out, rows_in, cols_in, rows_out, chunks_out, total);
    else
        pad_rows_kernel<E><<<copy_blocks(total), kBlock, 0, st>>>(in, out, rows_in, cols_in, rows_out, chunks_out, total);
}
// out[r][c] = in[r][c] for c < cols (rows of in hold chunks_in 16-byte chunks)
template <typename E>
__global__ __launch_bounds__(kBlock) void unpad_rows_kernel(const E *__restrict__ in, E *__restrict__ out, int64_t cols, int64_t chunks_in, int64_t total) {
    constexpr int V = kVecBytes / (int)sizeof(E);
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
        const int64_t ch = i % chunks_in, r = i / chunks_in;
        const vec_t<E, V> x = *reinterpret_cast<const vec_t<E, V> *>(in + i * V);
        E *p = out + r * cols + ch * V;
#pragma unroll
        for (int e = 0; e < V; ++e)
            if (ch * V + e < cols) p[e] = x.v[e];
    }
}
inline unsigned copy_blocks(int64_t total) {
    const int64_t blocks = (total + kBlock - 1) / kBlock;
    return (unsigned)(blocks > 16384 ? 16384 : blocks);
}
// inner(a, b, c, k_padded, n_padded, ldc) launches the aligned product on the copies.  With enough
// output tiles that the product is never cut along K, C is written straight at its own pitch
// (ldc = n) and no copy of C exists; a product that may be cut (its partial tiles assume [M][Np])
// goes through a padded C' (ldc = -1) that is copied out afterwards.
template <typename E, typename Inner>
int launch_on_padded_copies(Inner inner, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    constexpr int V = kVecBytes / (int)sizeof(E);
    const int64_t kp = (k + V - 1) / V * V, np = (n + V - 1) / V * V;
    const bool direct = batch * ((m + 127) / 128) * ((np + 127) / 128) * 2 > compute_units() && tuning().matmul_splitk <= 1;
    const int64_t a_elems = (batch * m * kp + V - 1) / V * V, b_elems = batch * kp * np, c_elems = direct ? 0 : batch * m * np;  // each part starts 16-byte aligned
    const int64_t bytes = (a_elems + b_elems + c_elems) * (int64_t)sizeof(E);
    if (bytes > kWorkspaceMaxBytes || m * n * k < (1 << 16)) return kNoSplit;
    E *ws = (E *)sc.take((size_t)bytes);
    if (!ws) return DXH_ERR_WORKSPACE;
    E *ap = ws, *bp = ap + a_elems, *cp = bp + b_elems;
    int64_t total = batch * m * (kp / V);
    const bool a_as_is = k == kp && ((uintptr_t)a % kVecBytes) == 0;  // only B and C have short rows
    int rc = DXH_OK;
    if (!sc.planning) {
        if (!a_as_is) launch_pad_rows<E>((const E *)a, ap, m, k, m, kp / V, total, st);
        total = batch * kp * (np / V);
        launch_pad_rows<E>((const E *)b, bp, k, n, kp, np / V, total, st);
        rc = launch_status();
        if (rc != DXH_OK) return rc;
    }
    if (direct) return inner(a_as_is ? a : (const void *)ap, (const void *)bp, c, kp, np, n);
    rc = inner(a_as_is ? a : (const void *)ap, (const void *)bp, (void *)cp, kp, np, (int64_t)-1);
    if (rc != DXH_OK || sc.planning) return rc;
    total = batch * m * (np / V);
    unpad_rows_kernel<E><<<copy_blocks(total), kBlock, 0, st>>>(cp, (E *)c, n, np / V, total);
    return launch_status();
}

// entry points of the per-dtype translation units (matmul_half.hip, matmul_fp.hip) and of the
// few-rows kernel (matmul_skinny.hip; kNoSkinny = not a shape for it)
constexpr int kNoSkinny = -1002;  // not a DXH_ERR_* value
int launch_matmul_skinny(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc);
int launch_matmul_half(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc);
// Several products that share their left operand, C_j = A B_j for j < count, as one launch: the tile map's
// batch index selects the pair (count 0: an ordinary, possibly batched, product).
constexpr int kSharedAMax = 4;
// C of a 16-bit product leaves with write-through stores when it is small enough that the kernel which reads it next
// finds it in the last-level cache (the rule of use_nt_store), else with non-temporal ones
inline int c_store_through(int64_t batch, int64_t m, int64_t n, size_t esize) { return use_nt_store((size_t)(batch * m * n) * esize) ? 0 : 1; }
struct SharedA { const void *b[kSharedAMax]; void *c[kSharedAMax]; int count; };
constexpr int kNoShared = -1004;  // not a DXH_ERR_* value: no single launch for these products, the caller multiplies one by one
int launch_matmul_half_dma(int dtype, int shape, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, const SharedA &multi = SharedA{});
int launch_matmul_half_shared(int dtype, const void *a, const SharedA &multi, int64_t m, int64_t k, int64_t n, hipStream_t st, bool dry);
// 128x128 (wide: 128x256) tiles cut into two halves of K that are summed inside the launch: `part` holds
// dma_split_bytes(tiles), `cnt` one zeroed counter per output tile (finish_counters, reduce.hip)
inline int64_t dma_split_bytes(int64_t tiles, int wide) { return tiles * 2 * 128 * (wide ? 256 : 128) * (int64_t)sizeof(float); }
int launch_matmul_half_dma_split(int dtype, int wide, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, float *part, unsigned *cnt, hipStream_t st);
unsigned *finish_counters(hipStream_t st, int64_t need);
int launch_matmul_f32(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc);
int launch_matmul_f64(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc);

}  // namespace dxh
