// changeshape.hip — transpose, concat, broadcastTo, indexselect, repeat (gfx950).
//
// Semantics: executor/op-ompsimd/src/deepx/tensorfunc/changeshape_miaobyte.hpp:45-200 with the
// shape rules of executor/deepxcore/src/deepx/shape_changeshape.cpp.  The reference moves one
// element per callback through index vectors; every op here is pure byte movement, so the
// kernels are chosen by layout, not dtype:
//
//   gather_rows   the innermost run of the output is also contiguous in the input (transpose
//                 that keeps the last axis, broadcastTo, indexselect): one lane moves one
//                 16-byte unit (or the widest power of two that divides the run), the output
//                 is written fully contiguously, the input row start comes from a mixed-radix
//                 decomposition of the row number (strides may be 0 = broadcast).
//   tile_transpose the last axis moves: 64x64 tiles staged through padded LDS so that both the
//                 global read (along the input's last axis) and the global write (along the
//                 output's last axis) are coalesced.
//   concat        one launch for up to 8 sources; each source is a 2-D strided copy into the
//                 output rows.
// All are HBM-bound: algorithmic bytes = bytes read once + bytes written once.
#include "common.hpp"
#include <vector>

namespace dxh {

constexpr int kGatherUnroll = 1;  // one unit per lane, one tile per workgroup: fastest measured copy shape
constexpr int kMaxOuter = DXH_MAX_DIMS;

struct OuterDims {
    int n;                        // number of outer (row-indexing) dims
    uint32_t size[kMaxOuter];     // output extent of each
    int64_t stride[kMaxOuter];    // input stride of each, in units
    FastDiv fsize[kMaxOuter];     // divide-free division by size[d] (32-bit index path)
    FastDiv fLu;                  // ... and by the units per row
};

// widest power-of-two unit (<= 16 bytes) dividing `bytes` and every pointer in `ptrs`
inline int unit_bytes(int64_t run_bytes, std::initializer_list<const void *> ptrs) {
    int u = kVecBytes;
    while (u > 1 && run_bytes % u != 0) u >>= 1;
    for (const void *p : ptrs) while (u > 1 && !aligned(p, u)) u >>= 1;
    return u;
}

// ---- gather_rows -------------------------------------------------------------------------
// out is [rows, Lu] units, contiguous.  in row start = sum_i idx_i * stride_i (units) where idx
// is the mixed-radix decomposition of the row number over `od`.  SPLAT: the input contributes a
// single element of type E per row position (innermost axis broadcast) that fills the unit.
template <typename U, typename I, bool SPLAT, typename E, bool REUSE, bool NTS, int ND>
__global__ __launch_bounds__(kBlock) void gather_rows_kernel(const void *__restrict__ in_, U *__restrict__ out, I total,
                                                              I Lu, OuterDims od, int through) {
    const I tile = (I)kBlock * kGatherUnroll;
    const I stride = (I)gridDim.x * tile;
    for (I base = (I)blockIdx.x * tile; base < total; base += stride) {
        U x[kGatherUnroll];
        I g[kGatherUnroll];
#pragma unroll
        for (int u = 0; u < kGatherUnroll; ++u) {
            g[u] = base + (I)u * kBlock + threadIdx.x;
            if (g[u] < total) {
                I row, v;
                int64_t off = 0;
                if constexpr (sizeof(I) == 4 && ND >= 0) {
                    // ND outer dims, fully unrolled: every extent, stride and magic number sits in
                    // scalar registers loaded once, and the address chain has no memory access in it
                    row = fast_div(g[u], od.fLu);
                    v = g[u] - row * Lu;
#pragma unroll
                    for (int d = ND - 1; d >= 0; --d) {
                        uint32_t q = fast_div(row, od.fsize[d]);
                        off += (int64_t)(row - q * od.size[d]) * od.stride[d];
                        row = q;
                    }
                } else if constexpr (sizeof(I) == 4) {
                    row = fast_div(g[u], od.fLu);
                    v = g[u] - row * Lu;
                    for (int d = od.n - 1; d >= 0; --d) {
                        uint32_t q = fast_div(row, od.fsize[d]);
                        off += (int64_t)(row - q * od.size[d]) * od.stride[d];
                        row = q;
                    }
                } else {
                    row = g[u] / Lu;
                    v = g[u] - row * Lu;
                    for (int d = od.n - 1; d >= 0; --d) {
                        I q = row / od.size[d];
                        off += (int64_t)(row - q * od.size[d]) * od.stride[d];
                        row = q;
                    }
                }
                if constexpr (SPLAT) {
                    E e = reinterpret_cast<const E *>(in_)[off];
                    constexpr int N = sizeof(U) / sizeof(E);
                    vec_t<E, N> r;
#pragma unroll
                    for (int k = 0; k < N; ++k) r.v[k] = e;
                    x[u] = __builtin_bit_cast(U, r);
                } else {
                    // REUSE: input rows are read many times (broadcast) and should stay cached
                    if constexpr (REUSE) x[u] = reinterpret_cast<const U *>(in_)[off + (int64_t)v];
                    else x[u] = ld_nt(reinterpret_cast<const U *>(in_) + off + (int64_t)v);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kGatherUnroll; ++u)
            if (g[u] < total) {
                if constexpr (NTS) st_stream(&out[g[u]], x[u], through); else out[g[u]] = x[u];
            }
    }
}

template <int UB, bool SPLAT, typename E, bool REUSE = false>
int launch_gather_unit(const void *in, void *out, int64_t rows, int64_t Lu, const OuterDims &od_in, hipStream_t st) {
    using U = typename raw_of<UB>::type;
    const int64_t total = rows * Lu;
    OuterDims od = od_in;
    for (int d = 0; d < od.n; ++d) od.fsize[d] = make_fastdiv(od.size[d]);
    od.fLu = make_fastdiv((uint32_t)std::min<int64_t>(Lu, 0xffffffffLL));
    unsigned grid = stream_grid(total, (int64_t)kBlock * kGatherUnroll, 0);
    const int through = use_nt_store((size_t)total * UB) ? 0 : 1;
    if (total < (int64_t)1 << 31) {
#define DXH_G(ND) gather_rows_kernel<U, uint32_t, SPLAT, E, REUSE, true, ND><<<grid, kBlock, 0, st>>>(in, (U *)out, (uint32_t)total, (uint32_t)Lu, od, through)
        switch (od.n) {
        case 0: DXH_G(0); break;
        case 1: DXH_G(1); break;
        case 2: DXH_G(2); break;
        case 3: DXH_G(3); break;
        case 4: DXH_G(4); break;
        default: DXH_G(-1); break;
        }
#undef DXH_G
    } else {
        gather_rows_kernel<U, uint64_t, SPLAT, E, REUSE, true, -1><<<grid, kBlock, 0, st>>>(in, (U *)out, (uint64_t)total, (uint64_t)Lu, od, through);
    }
    return launch_status();
}

// rows x run_bytes bytes per row; od.stride in ELEMENT-of-esize units on entry, converted here
inline int launch_gather(const void *in, void *out, int64_t rows, int64_t run_elems, int esize, OuterDims od, hipStream_t st,
                         bool reuse = false) {
    if (rows * run_elems == 0) return DXH_OK;
    const int ub = unit_bytes(run_elems * esize, {in, out});
    const int64_t Lu = run_elems * esize / ub;
    for (int d = 0; d < od.n; ++d) od.stride[d] = od.stride[d] * esize / ub;  // strides are multiples of the run
    if (reuse) {
        switch (ub) {
        case 16: return launch_gather_unit<16, false, uint8_t, true>(in, out, rows, Lu, od, st);
        case 8: return launch_gather_unit<8, false, uint8_t, true>(in, out, rows, Lu, od, st);
        case 4: return launch_gather_unit<4, false, uint8_t, true>(in, out, rows, Lu, od, st);
        case 2: return launch_gather_unit<2, false, uint8_t, true>(in, out, rows, Lu, od, st);
        default: return launch_gather_unit<1, false, uint8_t, true>(in, out, rows, Lu, od, st);
        }
    }
    switch (ub) {
    case 16: return launch_gather_unit<16, false, uint8_t>(in, out, rows, Lu, od, st);
    case 8: return launch_gather_unit<8, false, uint8_t>(in, out, rows, Lu, od, st);
    case 4: return launch_gather_unit<4, false, uint8_t>(in, out, rows, Lu, od, st);
    case 2: return launch_gather_unit<2, false, uint8_t>(in, out, rows, Lu, od, st);
    default: return launch_gather_unit<1, false, uint8_t>(in, out, rows, Lu, od, st);
    }
}

// innermost axis broadcast: every output row of `run_elems` elements repeats one input element
template <typename E>
int launch_splat(const void *in, void *out, int64_t rows, int64_t run_elems, const OuterDims &od, hipStream_t st) {
    if (rows * run_elems == 0) return DXH_OK;
    int ub = unit_bytes(run_elems * (int64_t)sizeof(E), {out});
    if (ub < (int)sizeof(E)) ub = sizeof(E);
    const int64_t Lu = run_elems * sizeof(E) / ub;
    switch (ub) {
    case 16: return launch_gather_unit<16, true, E>(in, out, rows, Lu, od, st);
    case 8: if constexpr (sizeof(E) <= 8) return launch_gather_unit<8, true, E>(in, out, rows, Lu, od, st);
    case 4: if constexpr (sizeof(E) <= 4) return launch_gather_unit<4, true, E>(in, out, rows, Lu, od, st);
    case 2: if constexpr (sizeof(E) <= 2) return launch_gather_unit<2, true, E>(in, out, rows, Lu, od, st);
    default: if constexpr (sizeof(E) == 1) return launch_gather_unit<1, true, E>(in, out, rows, Lu, od, st);
    }
    return DXH_ERR_ARG;
}

// ---- tile_transpose ----------------------------------------------------------------------
// Input viewed through `bd` batch dims plus two tiled axes: axis A (size nA, input stride sA,
// contiguous in the OUTPUT) and axis C (size nC, contiguous in the INPUT, output stride oC).
struct BatchDims {
    int n;
    uint32_t size[kMaxOuter];
    int64_t istride[kMaxOuter];
    int64_t ostride[kMaxOuter];
};
constexpr int kTile = 64;

template <typename E>
__global__ __launch_bounds__(kBlock) void tile_transpose_kernel(const E *__restrict__ in, E *__restrict__ out, int64_t nA,
                                                                 int64_t sA, int64_t nC, int64_t oC, int tilesA, int tilesC,
                                                                 BatchDims bd) {
    __shared__ E tile[kTile][kTile + 1];
    int64_t b = blockIdx.x;  // diagonal order over the tile grid, see tile_transpose_vec_kernel
    const int tc = (int)(b % tilesC); b /= tilesC;
    const int ta = (int)((b % tilesA + tc) % tilesA); b /= tilesA;
    int64_t ioff = 0, ooff = 0;
    for (int d = bd.n - 1; d >= 0; --d) {
        int64_t q = b / bd.size[d];
        int64_t r = b - q * bd.size[d];
        ioff += r * bd.istride[d];
        ooff += r * bd.ostride[d];
        b = q;
    }
    const int tx = threadIdx.x % kTile, ty = threadIdx.x / kTile;  // 64 x 4
    const int64_t a0 = (int64_t)ta * kTile, c0 = (int64_t)tc * kTile;
    // read: rows along A, lanes along C (contiguous in the input)
#pragma unroll 4
    for (int r = ty; r < kTile; r += kBlock / kTile) {
        int64_t a = a0 + r, c = c0 + tx;
        if (a < nA && c < nC) tile[r][tx] = in[ioff + a * sA + c];
    }
    __syncthreads();
    // write: rows along C, lanes along A (contiguous in the output)
#pragma unroll 4
    for (int r = ty; r < kTile; r += kBlock / kTile) {
        int64_t c = c0 + r, a = a0 + tx;
        if (a < nA && c < nC) out[ooff + c * oC + a] = tile[tx][r];
    }
}

// ---- tile_transpose, 16-byte version ----------------------------------------------------
// Same (A, C) view, for elements of ES bytes with V = 16/ES of them per 16-byte vector; needs nA,
// nC and every stride to be multiples of V and 16-byte aligned bases.  Tile = (16 V) x (16 V)
// elements, so that both the input rows (along C) and the output rows (along A) are touched in
// 256-byte runs by 16 lanes.  Each lane owns one V x V block: it loads V input rows of 16 bytes,
// transposes the block in registers (relabelling for 4/8-byte elements, v_perm_b32 for 2/1-byte
// ones) into V output vectors, and passes them through LDS to the lane that stores them, so all
// global and LDS traffic is in 16-byte units.  The LDS slot of an a-block is XORed with the
// c-block, which keeps both the stores (16 lanes, same a-block) and the loads conflict free.
typedef uint32_t tt_u32x4 __attribute__((ext_vector_type(4)));

template <int ES> __device__ __forceinline__ void transpose_block(const tt_u32x4 (&rows)[16 / ES], tt_u32x4 (&cols)[16 / ES]) {
    constexpr int V = 16 / ES;
    if constexpr (ES == 16) {
        cols[0] = rows[0];
    } else if constexpr (ES == 8) {
#pragma unroll
        for (int j = 0; j < 2; ++j) cols[j] = tt_u32x4{rows[0][2 * j], rows[0][2 * j + 1], rows[1][2 * j], rows[1][2 * j + 1]};
    } else if constexpr (ES == 4) {
#pragma unroll
        for (int j = 0; j < 4; ++j) cols[j] = tt_u32x4{rows[0][j], rows[1][j], rows[2][j], rows[3][j]};
    } else if constexpr (ES == 2) {
#pragma unroll
        for (int j = 0; j < V; ++j)
#pragma unroll
            for (int d = 0; d < 4; ++d)
                cols[j][d] = __builtin_amdgcn_perm(rows[2 * d + 1][j / 2], rows[2 * d][j / 2], (j & 1) ? 0x07060302u : 0x05040100u);
    } else {
#pragma unroll
        for (int j = 0; j < V; ++j)
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t sel = 0x0c0c0000u | (uint32_t)((4 + (j & 3)) << 8) | (uint32_t)(j & 3);  // byte j%4 of two rows
                const uint32_t t0 = __builtin_amdgcn_perm(rows[4 * d + 1][j / 4], rows[4 * d][j / 4], sel);
                const uint32_t t1 = __builtin_amdgcn_perm(rows[4 * d + 3][j / 4], rows[4 * d + 2][j / 4], sel);
                cols[j][d] = __builtin_amdgcn_perm(t1, t0, 0x05040100u);
            }
    }
}

template <int ES>
__global__ __launch_bounds__(kBlock) void tile_transpose_vec_kernel(const char *__restrict__ in, char *__restrict__ out, int64_t nA,
                                                                     int64_t sA, int64_t nC, int64_t oC, int tilesA, int tilesC,
                                                                     BatchDims bd, int through) {
    constexpr int V = 16 / ES, T = 16 * V;
    __shared__ tt_u32x4 lds[kBlock * V];  // [c in tile][a-block ^ c-block]
    // Diagonal order: consecutive workgroups step along C and along A together, so that neither
    // the reads (tile rows sA apart) nor the writes (tile rows oC apart) of the workgroups in
    // flight fall on addresses that differ only in high bits (power-of-two pitches otherwise pile
    // onto a few memory channels).
    int64_t b = blockIdx.x;
    const int tc = (int)(b % tilesC); b /= tilesC;
    const int ta = (int)((b % tilesA + tc) % tilesA); b /= tilesA;
    int64_t ioff = 0, ooff = 0;
    for (int d = bd.n - 1; d >= 0; --d) {
        int64_t q = b / bd.size[d];
        int64_t r = b - q * bd.size[d];
        ioff += r * bd.istride[d];
        ooff += r * bd.ostride[d];
        b = q;
    }
    const int l = threadIdx.x;
    {   // lanes along C: V input rows of one V x V block each
        const int cblk = l & 15, ablk = l >> 4;
        const int64_t a0 = (int64_t)ta * T + ablk * V, c0 = (int64_t)tc * T + cblk * V;
        if (a0 < nA && c0 < nC) {
            tt_u32x4 rows[V], cols[V];
#pragma unroll
            for (int r = 0; r < V; ++r)
                rows[r] = __builtin_nontemporal_load(reinterpret_cast<const tt_u32x4 *>(in + (ioff + (a0 + r) * sA + c0) * ES));
            transpose_block<ES>(rows, cols);
#pragma unroll
            for (int j = 0; j < V; ++j) lds[(cblk * V + j) * 16 + (ablk ^ cblk)] = cols[j];
        }
    }
    __syncthreads();
    {   // lanes along A: 16 output rows (values of c) per pass, 256 contiguous bytes each
        const int ablk = l & 15, crow = l >> 4;
        const int64_t a0 = (int64_t)ta * T + ablk * V;
#pragma unroll
        for (int i = 0; i < V; ++i) {
            const int c = crow + 16 * i;
            const int64_t gc = (int64_t)tc * T + c;
            if (gc < nC && a0 < nA)
                st_stream(reinterpret_cast<tt_u32x4 *>(out + (ooff + gc * oC + a0) * ES), lds[c * 16 + (ablk ^ ((c / V) & 15))], through);
        }
    }
}

// ---- concat --------------------------------------------------------------------------------
constexpr int kConcatMax = 8;
struct ConcatSrcs {
    int n;
    const void *ptr[kConcatMax];
    int64_t run[kConcatMax];     // units per outer row of this source
    int64_t pref[kConcatMax];    // unit offset of this source inside an output row
    int64_t cum[kConcatMax + 1]; // units before this source in the flattened work list
    FastDiv frun[kConcatMax];    // divide-free division by run[i] when everything fits 32 bits
};

// blockIdx.y = source, so run / prefix / pointer are wave-uniform scalars and the only per-lane
// work before the data load is one divide-free division.
template <typename U, bool FAST>
__global__ __launch_bounds__(kBlock) void concat_kernel(ConcatSrcs s, U *__restrict__ out, int64_t out_row, int64_t outer, int through) {
    const int i = blockIdx.y;
    const U *__restrict__ src = nullptr;
    int64_t run = 1, pref = 0;
    FastDiv frun{1, 0, 0};
#pragma unroll
    for (int k = 0; k < kConcatMax; ++k)
        if (k == i) { src = reinterpret_cast<const U *>(s.ptr[k]); run = s.run[k]; pref = s.pref[k]; frun = s.frun[k]; }
    const int64_t total = run * outer;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x; g < total; g += stride) {
        int64_t o, v;
        if constexpr (FAST) {
            const uint32_t oo = fast_div((uint32_t)g, frun);
            o = oo;
            v = (uint32_t)g - oo * (uint32_t)run;
        } else {
            o = g / run;
            v = g - o * run;
        }
        st_stream(&out[o * out_row + pref + v], ld_nt(&src[g]), through);
    }
}

// ---- indexselect ---------------------------------------------------------------------------
template <typename U, typename IT>
__global__ __launch_bounds__(kBlock) void indexselect_kernel(const U *__restrict__ in, const IT *__restrict__ index,
                                                              U *__restrict__ out, int64_t total, int64_t Lu, int64_t M,
                                                              int64_t adim, FastDiv fLu, FastDiv fM, bool fast, int through) {
    const int64_t tile = (int64_t)kBlock * kGatherUnroll;
    const int64_t stride = (int64_t)gridDim.x * tile;
    for (int64_t base = (int64_t)blockIdx.x * tile; base < total; base += stride) {
        U x[kGatherUnroll];
        int64_t g[kGatherUnroll];
#pragma unroll
        for (int u = 0; u < kGatherUnroll; ++u) {
            g[u] = base + (int64_t)u * kBlock + threadIdx.x;
            if (g[u] < total) {
                int64_t row, v, p, j;
                if (fast) {  // everything fits 32 bits: divide-free
                    const uint32_t r32 = fast_div((uint32_t)g[u], fLu), p32 = fast_div(r32, fM);
                    row = r32; v = (uint32_t)g[u] - r32 * (uint32_t)Lu;
                    p = p32; j = r32 - p32 * (uint32_t)M;
                } else {
                    row = g[u] / Lu; v = g[u] - row * Lu;
                    p = row / M; j = row - p * M;
                }
                int64_t k = (int64_t)index[j];
                k = k < 0 ? 0 : (k >= adim ? adim - 1 : k);
                x[u] = in[(p * adim + k) * Lu + v];
            }
        }
#pragma unroll
        for (int u = 0; u < kGatherUnroll; ++u)
            if (g[u] < total) st_stream(&out[g[u]], x[u], through);
    }
}

// ---- repeat --------------------------------------------------------------------------------
struct RepeatDims {
    int n;
    uint32_t osize[kMaxOuter];
    uint32_t reps[kMaxOuter];
    int64_t istride[kMaxOuter];
};
template <typename E>
__global__ __launch_bounds__(kBlock) void repeat_kernel(const E *__restrict__ in, E *__restrict__ out, int64_t total, RepeatDims rd) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t g = (int64_t)blockIdx.x * kBlock + threadIdx.x; g < total; g += stride) {
        int64_t rem = g, off = 0;
        for (int d = rd.n - 1; d >= 0; --d) {
            int64_t q = rem / rd.osize[d];
            int64_t r = rem - q * rd.osize[d];
            off += (r / rd.reps[d]) * rd.istride[d];
            rem = q;
        }
        out[g] = in[off];
    }
}

inline bool valid_shape(const int32_t *shape, int ndim, int64_t *size) {
    if (!shape || ndim < 1 || ndim > DXH_MAX_DIMS) return false;
    int64_t n = 1;
    for (int i = 0; i < ndim; ++i) { if (shape[i] < 0) return false; n *= shape[i]; }
    *size = n;
    return true;
}

// Output axes given as (extent, input stride in elements; 0 = broadcast): drop extent-1 axes,
// merge neighbours that are both broadcast or adjacent in the input, then copy rows with the
// gather kernel (innermost run dense) or splat one element per row (innermost axis broadcast).
// Returns kTooManyAxes when more axes survive the merge than the kernels index.
constexpr int kTooManyAxes = -1000;
inline int launch_broadcast(const void *in, void *out, int es, int n_axes, const int64_t *extent, const int64_t *stride,
                            int64_t nout, hipStream_t st) {
    int64_t sz[2 * DXH_MAX_DIMS], sd[2 * DXH_MAX_DIMS];
    int nd = 0;
    for (int i = 0; i < n_axes; ++i) {
        if (extent[i] == 1) continue;
        if (nd > 0 && ((sd[nd - 1] == 0 && stride[i] == 0) || (stride[i] != 0 && sd[nd - 1] == stride[i] * extent[i]))) {
            sz[nd - 1] *= extent[i];
            sd[nd - 1] = stride[i];
        } else { sz[nd] = extent[i]; sd[nd] = stride[i]; ++nd; }
    }
    if (nd == 0 || (nd == 1 && sd[0] == 1)) {
        if (in == out) return DXH_OK;
        return (int)hipMemcpyAsync(out, in, (size_t)nout * es, hipMemcpyDeviceToDevice, st);
    }
    if (nd - 1 > kMaxOuter) return kTooManyAxes;
    for (int i = 0; i < nd; ++i) if (sz[i] > 0xffffffffLL) return DXH_ERR_SHAPE;
    OuterDims od{};
    od.n = nd - 1;
    int64_t rows = 1;
    for (int i = 0; i < nd - 1; ++i) { od.size[i] = (uint32_t)sz[i]; od.stride[i] = sd[i]; rows *= sz[i]; }
    if (sd[nd - 1] == 1) return launch_gather(in, out, rows, sz[nd - 1], es, od, st, /*reuse=*/true);
    switch (es) {  // innermost axis is broadcast: splat one element per row position
    case 8: return launch_splat<uint64_t>(in, out, rows, sz[nd - 1], od, st);
    case 4: return launch_splat<uint32_t>(in, out, rows, sz[nd - 1], od, st);
    case 2: return launch_splat<uint16_t>(in, out, rows, sz[nd - 1], od, st);
    default: return launch_splat<uint8_t>(in, out, rows, sz[nd - 1], od, st);
    }
}

}  // namespace dxh

using namespace dxh;

extern "C" {

int dxh_transpose(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *order, void *out, void *stream) {
    const int es = dtype_size(dtype);
    if (!es) return DXH_ERR_DTYPE;
    int64_t n;
    if (!valid_shape(shape, ndim, &n) || !order) return DXH_ERR_ARG;
    bool seen[DXH_MAX_DIMS] = {false};
    for (int i = 0; i < ndim; ++i) {
        if (order[i] < 0 || order[i] >= ndim || seen[order[i]]) return DXH_ERR_ARG;
        seen[order[i]] = true;
    }
    if (n == 0) return DXH_OK;
    if (!in || !out) return DXH_ERR_ARG;
    if (!aligned(in, es) || !aligned(out, es)) return DXH_ERR_ALIGN;
    hipStream_t st = as_stream(stream);
    // input strides (elements)
    int64_t istr[DXH_MAX_DIMS];
    { int64_t s = 1; for (int i = ndim - 1; i >= 0; --i) { istr[i] = s; s *= shape[i]; } }
    // output dims in output order: (size, input stride); drop size-1, merge input-adjacent runs
    int64_t osz[DXH_MAX_DIMS], ost[DXH_MAX_DIMS];
    int nd = 0;
    for (int i = 0; i < ndim; ++i) {
        int64_t sz = shape[order[i]], sd = istr[order[i]];
        if (sz == 1) continue;
        if (nd > 0 && ost[nd - 1] == sd * sz) { osz[nd - 1] *= sz; ost[nd - 1] = sd; }
        else { osz[nd] = sz; ost[nd] = sd; ++nd; }
    }
    if (nd <= 1) {  // identity permutation
        if (in == out) return DXH_OK;
        return (int)hipMemcpyAsync(out, in, (size_t)n * es, hipMemcpyDeviceToDevice, st);
    }
    for (int i = 0; i < nd; ++i) if (osz[i] > 0xffffffffLL) return DXH_ERR_SHAPE;
    int es_eff = es;  // element size the kernels move
    if (ost[nd - 1] == 1 && nd >= 3) {
        // A short innermost run (2..16 bytes, a power of two) that stays innermost is better moved
        // as one wide element by the tiled transpose than gathered 16 bytes at a time from
        // scattered rows: fold it into the element size.
        const int64_t run_bytes = osz[nd - 1] * es;
        const bool pow2 = (run_bytes & (run_bytes - 1)) == 0;
        if (pow2 && run_bytes <= 16 && run_bytes > es && aligned(in, (size_t)run_bytes) && aligned(out, (size_t)run_bytes)) {
            for (int i = 0; i < nd - 1; ++i) ost[i] /= osz[nd - 1];  // every other input stride is a multiple of the innermost size
            es_eff = (int)run_bytes;
            --nd;
        }
    }
    if (ost[nd - 1] == 1) {
        // the innermost output run is contiguous in the input too
        OuterDims od{};
        od.n = nd - 1;
        int64_t rows = 1;
        for (int i = 0; i < nd - 1; ++i) { od.size[i] = (uint32_t)osz[i]; od.stride[i] = ost[i]; rows *= osz[i]; }
        return launch_gather(in, out, rows, osz[nd - 1], es_eff, od, st);
    }
    // the last axis moves: tile over (A = output-last axis, C = input-last axis)
    int64_t ostr[DXH_MAX_DIMS];
    { int64_t s = 1; for (int i = nd - 1; i >= 0; --i) { ostr[i] = s; s *= osz[i]; } }
    int qc = -1;
    for (int i = 0; i < nd; ++i) if (ost[i] == 1) qc = i;
    if (qc < 0) return DXH_ERR_ARG;  // cannot happen: some merged dim holds the input's last axis
    const int64_t nA = osz[nd - 1], sA = ost[nd - 1], nC = osz[qc], oC = ostr[qc];
    BatchDims bd{};
    int64_t batch = 1;
    for (int i = 0; i < nd - 1; ++i) {
        if (i == qc) continue;
        bd.size[bd.n] = (uint32_t)osz[i]; bd.istride[bd.n] = ost[i]; bd.ostride[bd.n] = ostr[i]; ++bd.n;
        batch *= osz[i];
    }
    const int V = 16 / es_eff;
    bool vec = aligned(in, kVecBytes) && aligned(out, kVecBytes) && nA % V == 0 && nC % V == 0 && sA % V == 0 && oC % V == 0;
    for (int i = 0; i < bd.n; ++i) vec = vec && bd.istride[i] % V == 0 && bd.ostride[i] % V == 0;
    if (vec) {
        const int T = 16 * V;
        const int64_t tilesA = (nA + T - 1) / T, tilesC = (nC + T - 1) / T, blocks = batch * tilesA * tilesC;
        if (blocks > 0x7fffffff) return DXH_ERR_SHAPE;
        const int through = use_nt_store((size_t)(batch * nA * nC) * (size_t)es_eff) ? 0 : 1;
#define DXH_TT(ES) tile_transpose_vec_kernel<ES><<<(unsigned)blocks, kBlock, 0, st>>>((const char *)in, (char *)out, nA, sA, nC, oC, (int)tilesA, (int)tilesC, bd, through)
        switch (es_eff) {
        case 16: DXH_TT(16); break;
        case 8: DXH_TT(8); break;
        case 4: DXH_TT(4); break;
        case 2: DXH_TT(2); break;
        default: DXH_TT(1); break;
        }
#undef DXH_TT
        return launch_status();
    }
    const int64_t tilesA = (nA + kTile - 1) / kTile, tilesC = (nC + kTile - 1) / kTile;
    const int64_t blocks = batch * tilesA * tilesC;
    if (blocks > 0x7fffffff) return DXH_ERR_SHAPE;
    switch (es_eff) {
    case 16: tile_transpose_kernel<uint4><<<(unsigned)blocks, kBlock, 0, st>>>((const uint4 *)in, (uint4 *)out, nA, sA, nC, oC, (int)tilesA, (int)tilesC, bd); break;
    case 8: tile_transpose_kernel<uint64_t><<<(unsigned)blocks, kBlock, 0, st>>>((const uint64_t *)in, (uint64_t *)out, nA, sA, nC, oC, (int)tilesA, (int)tilesC, bd); break;
    case 4: tile_transpose_kernel<uint32_t><<<(unsigned)blocks, kBlock, 0, st>>>((const uint32_t *)in, (uint32_t *)out, nA, sA, nC, oC, (int)tilesA, (int)tilesC, bd); break;
    case 2: tile_transpose_kernel<uint16_t><<<(unsigned)blocks, kBlock, 0, st>>>((const uint16_t *)in, (uint16_t *)out, nA, sA, nC, oC, (int)tilesA, (int)tilesC, bd); break;
    default: tile_transpose_kernel<uint8_t><<<(unsigned)blocks, kBlock, 0, st>>>((const uint8_t *)in, (uint8_t *)out, nA, sA, nC, oC, (int)tilesA, (int)tilesC, bd); break;
    }
    return launch_status();
}

int dxh_concat(int dtype, const void *const *ins, int nins, const int32_t *axis_sizes, const int32_t *out_shape, int ndim,
               int axis, void *out, void *stream) {
    const int es = dtype_size(dtype);
    if (!es) return DXH_ERR_DTYPE;
    int64_t n;
    if (!valid_shape(out_shape, ndim, &n) || !ins || !axis_sizes || nins < 1 || axis < 0 || axis >= ndim) return DXH_ERR_ARG;
    int64_t total_axis = 0;
    for (int i = 0; i < nins; ++i) { if (axis_sizes[i] < 0) return DXH_ERR_ARG; total_axis += axis_sizes[i]; }
    if (total_axis != out_shape[axis]) return DXH_ERR_SHAPE;
    if (n == 0) return DXH_OK;
    if (!out) return DXH_ERR_ARG;
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < axis; ++i) outer *= out_shape[i];
    for (int i = axis + 1; i < ndim; ++i) inner *= out_shape[i];
    // unit: widest power of two dividing every run and every pointer
    int ub = unit_bytes(inner * es * total_axis, {out});
    for (int i = 0; i < nins; ++i) {
        if (axis_sizes[i] == 0) continue;
        if (!ins[i]) return DXH_ERR_ARG;
        ub = std::min(ub, unit_bytes((int64_t)axis_sizes[i] * inner * es, {ins[i]}));
    }
    if (ub < es && (!aligned(out, es))) return DXH_ERR_ALIGN;
    const int64_t out_row = total_axis * inner * es / ub;
    hipStream_t st = as_stream(stream);
    int64_t pref = 0;
    int i = 0;
    while (i < nins) {
        ConcatSrcs s{};
        int64_t cum = 0;
        while (i < nins && s.n < kConcatMax) {
            int64_t run = (int64_t)axis_sizes[i] * inner * es / ub;
            if (run > 0) {
                s.ptr[s.n] = ins[i]; s.run[s.n] = run; s.pref[s.n] = pref; s.cum[s.n] = cum;
                s.frun[s.n] = make_fastdiv((uint32_t)std::min<int64_t>(run, 0xffffffffLL));
                cum += run * outer;
                ++s.n;
            }
            pref += run;
            ++i;
        }
        s.cum[s.n] = cum;
        if (s.n == 0 || cum == 0) continue;
        int64_t max_units = 0;
        for (int k = 0; k < s.n; ++k) max_units = std::max(max_units, s.run[k] * outer);
        const bool fast = max_units < ((int64_t)1 << 32);
        const int through = use_nt_store((size_t)(out_row * outer) * (size_t)ub) ? 0 : 1;
        dim3 grid(stream_grid(max_units, kBlock, 0) > 0x7fffffffu ? 0x7fffffffu : stream_grid(max_units, kBlock, 0), (unsigned)s.n);
#define DXH_CC(U)                                                                           \
        if (fast) concat_kernel<U, true><<<grid, kBlock, 0, st>>>(s, (U *)out, out_row, outer, through); \
        else concat_kernel<U, false><<<grid, kBlock, 0, st>>>(s, (U *)out, out_row, outer, through);
        switch (ub) {
        case 16: DXH_CC(uint4) break;
        case 8: DXH_CC(uint64_t) break;
        case 4: DXH_CC(uint32_t) break;
        case 2: DXH_CC(uint16_t) break;
        default: DXH_CC(uint8_t) break;
        }
#undef DXH_CC
        int rc = launch_status();
        if (rc != DXH_OK) return rc;
    }
    return DXH_OK;
}

int dxh_broadcastTo(int dtype, const void *in, const int32_t *in_shape, int in_ndim, const int32_t *out_shape, int out_ndim,
                    void *out, void *stream) {
    const int es = dtype_size(dtype);
    if (!es) return DXH_ERR_DTYPE;
    int64_t nin, nout;
    if (!valid_shape(in_shape, in_ndim, &nin) || !valid_shape(out_shape, out_ndim, &nout)) return DXH_ERR_ARG;
    if (in_ndim > out_ndim) return DXH_ERR_SHAPE;
    const int shift = out_ndim - in_ndim;
    int64_t istr[DXH_MAX_DIMS];
    { int64_t s = 1; for (int i = in_ndim - 1; i >= 0; --i) { istr[i] = s; s *= in_shape[i]; } }
    // per output axis: input stride, 0 where the axis is broadcast (broadcastMap, shape_changeshape.cpp:79-104)
    int64_t extent[DXH_MAX_DIMS], stride[DXH_MAX_DIMS];
    for (int i = 0; i < out_ndim; ++i) {
        extent[i] = out_shape[i];
        stride[i] = 0;
        if (i >= shift) {
            if (in_shape[i - shift] == out_shape[i]) stride[i] = istr[i - shift];
            else if (in_shape[i - shift] != 1) return DXH_ERR_SHAPE;
        }
    }
    if (nout == 0) return DXH_OK;
    if (!in || !out) return DXH_ERR_ARG;
    if (!aligned(in, es) || !aligned(out, es)) return DXH_ERR_ALIGN;
    const int rc = launch_broadcast(in, out, es, out_ndim, extent, stride, nout, as_stream(stream));
    return rc == kTooManyAxes ? DXH_ERR_SHAPE : rc;
}

int dxh_indexselect(int dtype, const void *in, const int32_t *in_shape, int in_ndim, int index_dtype, const void *index,
                    const int32_t *index_shape, int index_ndim, int axis, void *out, void *stream) {
    const int es = dtype_size(dtype);
    if (!es) return DXH_ERR_DTYPE;
    if (index_dtype != DXH_I32 && index_dtype != DXH_I64) return DXH_ERR_DTYPE;
    int64_t nin, m;
    if (!valid_shape(in_shape, in_ndim, &nin) || !valid_shape(index_shape, index_ndim, &m)) return DXH_ERR_ARG;
    if (axis < 0) axis += in_ndim;
    if (axis < 0 || axis >= in_ndim) return DXH_ERR_ARG;
    int64_t pre = 1, post = 1;
    for (int i = 0; i < axis; ++i) pre *= in_shape[i];
    for (int i = axis + 1; i < in_ndim; ++i) post *= in_shape[i];
    const int64_t adim = in_shape[axis];
    if (pre * m * post == 0) return DXH_OK;
    if (adim == 0) return DXH_ERR_SHAPE;
    if (!in || !index || !out) return DXH_ERR_ARG;
    if (!aligned(in, es) || !aligned(out, es) || !aligned(index, index_dtype == DXH_I64 ? 8 : 4)) return DXH_ERR_ALIGN;
    const int ub = unit_bytes(post * es, {in, out});
    const int64_t Lu = post * es / ub;
    const int64_t total = pre * m * Lu;
    hipStream_t st = as_stream(stream);
    unsigned grid = stream_grid(total, (int64_t)kBlock * kGatherUnroll, 0);
    const bool fast = total < ((int64_t)1 << 32) && Lu < ((int64_t)1 << 32) && m < ((int64_t)1 << 32);
    const int through = use_nt_store((size_t)total * (size_t)ub) ? 0 : 1;
    const FastDiv fLu = make_fastdiv((uint32_t)std::min<int64_t>(Lu, 0xffffffffLL)), fM = make_fastdiv((uint32_t)std::min<int64_t>(m, 0xffffffffLL));
#define DXH_IS(U)                                                                                                      \
    if (index_dtype == DXH_I64)                                                                                        \
        indexselect_kernel<U, int64_t><<<grid, kBlock, 0, st>>>((const U *)in, (const int64_t *)index, (U *)out, total, Lu, m, adim, fLu, fM, fast, through); \
    else                                                                                                               \
        indexselect_kernel<U, int32_t><<<grid, kBlock, 0, st>>>((const U *)in, (const int32_t *)index, (U *)out, total, Lu, m, adim, fLu, fM, fast, through);
    switch (ub) {
    case 16: DXH_IS(uint4) break;
    case 8: DXH_IS(uint64_t) break;
    case 4: DXH_IS(uint32_t) break;
    case 2: DXH_IS(uint16_t) break;
    default: DXH_IS(uint8_t) break;
    }
#undef DXH_IS
    return launch_status();
}

int dxh_repeat(int dtype, const void *in, const int32_t *shape, int ndim, const int32_t *repeats, void *out, void *stream) {
    const int es = dtype_size(dtype);
    if (!es) return DXH_ERR_DTYPE;
    int64_t nin;
    if (!valid_shape(shape, ndim, &nin) || !repeats) return DXH_ERR_ARG;
    RepeatDims rd{};
    rd.n = ndim;
    int64_t total = 1, s = 1;
    for (int i = ndim - 1; i >= 0; --i) {
        if (repeats[i] < 1) return DXH_ERR_ARG;
        int64_t o = (int64_t)shape[i] * repeats[i];
        if (o > 0xffffffffLL) return DXH_ERR_SHAPE;
        rd.osize[i] = (uint32_t)o; rd.reps[i] = (uint32_t)repeats[i]; rd.istride[i] = s;
        s *= shape[i];
        total *= o;
    }
    if (total == 0) return DXH_OK;
    if (!in || !out) return DXH_ERR_ARG;
    if (!aligned(in, es) || !aligned(out, es)) return DXH_ERR_ALIGN;
    hipStream_t st = as_stream(stream);
    {   // repeat = broadcast of the input seen as [d0, 1, d1, 1, ...] to [d0, r0, d1, r1, ...]
        int64_t extent[2 * DXH_MAX_DIMS], stride[2 * DXH_MAX_DIMS];
        for (int i = 0; i < ndim; ++i) {
            extent[2 * i] = shape[i]; stride[2 * i] = rd.istride[i];
            extent[2 * i + 1] = repeats[i]; stride[2 * i + 1] = 0;
        }
        const int rc = launch_broadcast(in, out, es, 2 * ndim, extent, stride, total, st);
        if (rc != kTooManyAxes) return rc;
    }
    unsigned grid = stream_grid(total, kBlock, 16);
    switch (es) {
    case 8: repeat_kernel<uint64_t><<<grid, kBlock, 0, st>>>((const uint64_t *)in, (uint64_t *)out, total, rd); break;
    case 4: repeat_kernel<uint32_t><<<grid, kBlock, 0, st>>>((const uint32_t *)in, (uint32_t *)out, total, rd); break;
    case 2: repeat_kernel<uint16_t><<<grid, kBlock, 0, st>>>((const uint16_t *)in, (uint16_t *)out, total, rd); break;
    default: repeat_kernel<uint8_t><<<grid, kBlock, 0, st>>>((const uint8_t *)in, (uint8_t *)out, total, rd); break;
    }
    return launch_status();
}

}  // extern "C"
