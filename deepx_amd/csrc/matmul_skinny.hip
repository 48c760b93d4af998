// matmul_skinny.hip — float GEMM with at most 8 rows of A (one token, a few tokens): the product
// is a stream over B, so it is built like the strided-axis reduction and not on the matrix pipe,
// where a 64-row tile would spend 7/8 of its MFMAs on padding and, worse, read B through far
// fewer workgroups than the memory system needs.
//   C[m][n] = sum_k A[m][k] B[k][n],  m < MB <= 8
//   workgroup  32 column-lanes x 8 k-lanes; a column-lane owns V = 16 / sizeof(T) adjacent columns
//              (one 16-byte load per row of B), so a workgroup reads 512 contiguous bytes per row
//   K          cut into S slices (grid.y) while there is less than a workgroup per CU; a slice is
//              walked in sub-chunks of kSub rows whose A values are staged in LDS (every lane of a
//              k-lane reads the same A[m][k]: an LDS broadcast)
//   sums       fp32 (fp64 for fp64) fused multiply-adds per lane, the 8 k-lanes are added through
//              LDS; with S > 1 the slices go to the stream's split-K workspace and
//              splitk_reduce_kernel adds them in slice order and rounds once
#include "matmul_common.hpp"

namespace dxh {

constexpr int kSkinnyTX = 32, kSkinnyTY = 8, kSub = 512;

template <typename T> struct skinny_acc { using type = float; };
template <> struct skinny_acc<double> { using type = double; };
__device__ __forceinline__ float fma_acc(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_acc(double a, double b, double c) { return __builtin_fma(a, b, c); }

// AL: N is a multiple of V and B is 16-byte aligned, so row r of B splits into aligned 16-byte
// pieces that start at the same columns for every r.  Otherwise (any N, B aligned to its element
// size) the 16-byte grid of row r starts phase(r) = (address of B[r][0] / sizeof(T)) % V elements
// before column 0, and the loads follow that grid instead of the columns: a k-lane visits rows
// r = ty + 8 i, whose phase is the same for every i (8 N elements are a whole number of 16-byte
// pieces), so lane (tx, ty) owns the V columns from c0 - phase(ty) + V tx on, all its loads are
// aligned, and its accumulators stay with the same columns.  A workgroup then loads 32 pieces per
// row but answers for 31 V columns, the ones every k-lane covers whatever its phase; the sums over
// the k-lanes pick each column out of LDS at the k-lane's own offset.  Pieces that stick out of a
// row (before column 0, past N) bring in neighbouring elements, or bytes just outside the buffer
// within the same aligned 16 bytes; their sums belong to columns that are never stored.
template <typename T, int MB, typename TO, bool AL>
__global__ __launch_bounds__(kBlock) void matmul_skinny_kernel(const T *__restrict__ A, const T *__restrict__ B, TO *__restrict__ out,
                                                                int M, int K, int N, int S, int chunk) {
    using AT = typename skinny_acc<T>::type;
    constexpr int V = kVecBytes / (int)sizeof(T);
    using VT = vec_t<T, V>;
    __shared__ __attribute__((aligned(16))) AT a_lds[MB * kSub];  // [row of the sub-chunk][m]: the MB values of a row are one or a few 16-byte reads
    __shared__ AT red[kBlock * V];
    const int tx = threadIdx.x % kSkinnyTX, ty = threadIdx.x / kSkinnyTX;
    const int64_t batch = blockIdx.z;
    const int s = blockIdx.y;
    const int nv = N / V;                        // AL only
    const int cv = blockIdx.x * kSkinnyTX + tx;  // AL: vector column of this lane
    A += batch * (int64_t)M * K;
    B += batch * (int64_t)K * N;
    const int k0 = s * chunk, k1 = (k0 + chunk < K) ? k0 + chunk : K;
    constexpr int kCols = (AL ? kSkinnyTX : kSkinnyTX - 1) * V;  // columns a workgroup answers for
    auto phase = [&](int y) __attribute__((always_inline)) { return AL ? 0 : (int)((reinterpret_cast<uintptr_t>(B + (int64_t)(k0 + y) * N) / sizeof(T)) % V); };
    const int c0 = blockIdx.x * kCols;               // !AL: first column of the workgroup
    const int col0 = c0 - phase(ty) + V * tx;        // !AL: first column of this lane (may be -V + 1 .. -1)
    const bool active = AL ? cv < nv : col0 < N;
    AT acc[MB][V];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int v = 0; v < V; ++v) acc[m][v] = AT(0);
    const VT *Bv = reinterpret_cast<const VT *>(B) + cv;
    auto load_b = [&](int64_t row) __attribute__((always_inline)) -> VT {
        if constexpr (AL) return Bv[row * nv];
        else return *reinterpret_cast<const VT *>(B + row * N + col0);
    };
    for (int kb = k0; kb < k1; kb += kSub) {
        const int len = (kb + kSub < k1) ? kSub : k1 - kb;
        // The first four rows of B are requested before A is staged, so that their latency runs
        // under the staging; after that the next four are always in flight while four are used.
        constexpr int U = 4, STEP = U * kSkinnyTY;
        VT x[U];
        const bool batched = active && ty + (U - 1) * kSkinnyTY < len;
        if (batched) {
#pragma unroll
            for (int u = 0; u < U; ++u) x[u] = load_b(kb + ty + u * kSkinnyTY);
        }
        __syncthreads();  // the previous sub-chunk's A values are no longer read
#pragma unroll
        for (int m = 0; m < MB; ++m)
            for (int r = threadIdx.x; r < len; r += kBlock) a_lds[r * MB + m] = (m < M) ? AT(load_acc(A[(int64_t)m * K + kb + r])) : AT(0);
        __syncthreads();
        if (active) {
            auto use = [&](const VT(&b)[U], int r) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    AT a[MB];
#pragma unroll
                    for (int m = 0; m < MB; ++m) a[m] = a_lds[(r + u * kSkinnyTY) * MB + m];
#pragma unroll
                    for (int m = 0; m < MB; ++m)
#pragma unroll
                        for (int v = 0; v < V; ++v) acc[m][v] = fma_acc(a[m], AT(load_acc(b[u].v[v])), acc[m][v]);
                }
            };
            int r = ty;
            if (batched) {
                for (; r + STEP + (U - 1) * kSkinnyTY < len; r += STEP) {
                    VT y[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) y[u] = load_b(kb + r + STEP + u * kSkinnyTY);
                    use(x, r);
#pragma unroll
                    for (int u = 0; u < U; ++u) x[u] = y[u];
                }
                use(x, r);
                r += STEP;
            }
            for (; r < len; r += kSkinnyTY) {
                const VT b = load_b(kb + r);
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    const AT a = a_lds[r * MB + m];
#pragma unroll
                    for (int v = 0; v < V; ++v) acc[m][v] = fma_acc(a, AT(load_acc(b.v[v])), acc[m][v]);
                }
            }
        }
    }
    // add the 8 k-lanes of every column through LDS, one row of A at a time
    TO *o = out + ((batch * S + s) * (int64_t)M) * N;
#pragma unroll
    for (int m = 0; m < MB; ++m) {
        __syncthreads();
        if constexpr (!AL) {
            // red[y][q]: what k-lane y summed for column c0 - phase(y) + q
#pragma unroll
            for (int v = 0; v < V; ++v) red[ty * (kSkinnyTX * V) + V * tx + v] = active ? acc[m][v] : AT(0);
            __syncthreads();
            const int col = c0 + (int)threadIdx.x;
            if ((int)threadIdx.x < kCols && col < N && m < M) {
                AT t = red[threadIdx.x + phase(0)];
#pragma unroll
                for (int y = 1; y < kSkinnyTY; ++y) t += red[y * (kSkinnyTX * V) + threadIdx.x + phase(y)];
                if constexpr (std::is_same_v<TO, AT>) o[(int64_t)m * N + col] = t;
                else o[(int64_t)m * N + col] = store_acc<TO>(t);
            }
            continue;
        }
#pragma unroll
        for (int v = 0; v < V; ++v) red[(v * kSkinnyTY + ty) * kSkinnyTX + tx] = acc[m][v];
        __syncthreads();
        if (ty == 0 && active && m < M) {
#pragma unroll
            for (int v = 0; v < V; ++v) {
                AT t = red[(v * kSkinnyTY) * kSkinnyTX + tx];
#pragma unroll
                for (int y = 1; y < kSkinnyTY; ++y) t += red[(v * kSkinnyTY + y) * kSkinnyTX + tx];
                if constexpr (std::is_same_v<TO, AT>) o[(int64_t)m * N + (int64_t)cv * V + v] = t;
                else o[(int64_t)m * N + (int64_t)cv * V + v] = store_acc<TO>(t);
            }
        }
    }
}

template <typename T, int MB, bool AL>
int launch_skinny_mb(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    using AT = typename skinny_acc<T>::type;
    constexpr int V = kVecBytes / (int)sizeof(T);
    const int64_t cols = (AL ? kSkinnyTX : kSkinnyTX - 1) * V, ctiles = (n + cols - 1) / cols;
    // slices of K: about `per_cu` workgroups per CU, at least `min_rows` rows per slice
    const int64_t per_cu = tuning().skinny_per_cu, min_rows = tuning().skinny_min_rows;
    int64_t S = (per_cu * (int64_t)compute_units() + batch * ctiles - 1) / (batch * ctiles);
    if (S > k / min_rows) S = k / min_rows;
    if (S < 1 || tuning().matmul_splitk == 1) S = 1;
    const int64_t partial = batch * m * n * (int64_t)sizeof(AT);
    if (S > 1 && S * partial > kWorkspaceMaxBytes) S = 1;
    int64_t chunk = (k + S - 1) / S;
    chunk = (chunk + kSkinnyTY - 1) / kSkinnyTY * kSkinnyTY;
    S = (k + chunk - 1) / chunk;
    if (ctiles > 0x7fffffff || S > 65535 || batch > 65535) return kNoSkinny;
    const dim3 grid((unsigned)ctiles, (unsigned)S, (unsigned)batch);
    if (S == 1) {
        if (sc.planning) return DXH_OK;
        matmul_skinny_kernel<T, MB, T, AL><<<grid, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, 1, (int)chunk);
        return launch_status();
    }
    AT *ws = (AT *)sc.take((size_t)(partial * S));
    if (!ws) return DXH_ERR_WORKSPACE;
    if (sc.planning) return DXH_OK;
    matmul_skinny_kernel<T, MB, AT, AL><<<grid, kBlock, 0, st>>>((const T *)a, (const T *)b, ws, (int)m, (int)k, (int)n, (int)S, (int)chunk);
    const int rc = launch_status();
    return rc != DXH_OK ? rc : launch_splitk_reduce<AT, T>(ws, (T *)c, batch, m * n, (int)S, st);
}

// Returns kNoSkinny when the shape is not one for this kernel (the caller goes on to the matrix pipe).
template <typename T>
int launch_skinny_t(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    constexpr int V = kVecBytes / (int)sizeof(T);
    // 9..16 rows only for fp32 / fp64 whose rows of B are not 16-byte pieces, where the matrix pipe would need a
    // padded copy of B first (fp32 12x4096x4097: 43 us there, 30 here); 16-bit types: the conversions make that many rows vector-ALU-bound
    constexpr int kMaxRows = sizeof(T) >= 4 ? 16 : 8;
    if (m > kMaxRows || k < 256 || k > 0x7fffffff / 2 || n > 0x7fffffff / 2 || tuning().matmul_tile != 0) return kNoSkinny;
    if (n % V == 0 && aligned(b, kVecBytes)) {
        if (m == 1) return launch_skinny_mb<T, 1, true>(a, b, c, batch, m, k, n, st, sc);
        if (m == 2) return launch_skinny_mb<T, 2, true>(a, b, c, batch, m, k, n, st, sc);
        if (m <= 4) return launch_skinny_mb<T, 4, true>(a, b, c, batch, m, k, n, st, sc);
        if (m <= 8) return launch_skinny_mb<T, 8, true>(a, b, c, batch, m, k, n, st, sc);
        return kNoSkinny;  // 9..16 rows of 16-byte rows: the matrix pipe is as fast (fp32 16x4096x4096: 29.8 us there, 33.8 here)
    }
    if (!aligned(b, sizeof(T))) return kNoSkinny;
    if (m == 1) return launch_skinny_mb<T, 1, false>(a, b, c, batch, m, k, n, st, sc);
    if (m == 2) return launch_skinny_mb<T, 2, false>(a, b, c, batch, m, k, n, st, sc);
    if (m <= 4) return launch_skinny_mb<T, 4, false>(a, b, c, batch, m, k, n, st, sc);
    if (m <= 8) return launch_skinny_mb<T, 8, false>(a, b, c, batch, m, k, n, st, sc);
    if constexpr (kMaxRows == 16) return launch_skinny_mb<T, 16, false>(a, b, c, batch, m, k, n, st, sc);
    return kNoSkinny;
}

// fp32 and fp64 always.  For bf16 / f16 with 16-byte rows of B the 64x64 matrix-pipe tiles over K
// slices are as fast or faster (one row of [4096,4096] takes 12.3 us against 14.2 here, eight rows
// 12.7 against 24.4: eight conversions and multiply-adds per 2-byte element are vector-ALU-bound),
// so they come here only when the matrix pipe would need a padded copy of B first (one row of
// [768,50257]: 18.5 us against 39.7) or when DXH_TUNE_SKINNY_HALF asks for it.  fp32: 15 against
// 28.6 us for one row of [4096,4096], 93 against 153 us for [896,151936] (5.9 TB/s).
int launch_matmul_skinny(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    switch (dtype) {
    // 16-bit types: only where the matrix pipe would first have to copy B into 16-byte rows (or when asked for)
    case DXH_BF16: return (tuning().skinny_half || n % 8 != 0 || !aligned(b, kVecBytes)) ? launch_skinny_t<bf16_t>(a, b, c, batch, m, k, n, st, sc) : kNoSkinny;
    case DXH_F16: return (tuning().skinny_half || n % 8 != 0 || !aligned(b, kVecBytes)) ? launch_skinny_t<f16_t>(a, b, c, batch, m, k, n, st, sc) : kNoSkinny;
    case DXH_F32: return launch_skinny_t<float>(a, b, c, batch, m, k, n, st, sc);
    case DXH_F64: return launch_skinny_t<double>(a, b, c, batch, m, k, n, st, sc);
    default: return kNoSkinny;
    }
}

}  // namespace dxh
