// matmul_skinny.hip — float GEMM with at most 8 rows of A (one token, a few tokens): the product
// is a stream over B, so it is built like the strided-axis reduction and not on the matrix pipe,
// where a 64-row tile would spend 7/8 of its MFMAs on padding and, worse, read B through far
// fewer workgroups than the memory system needs.
//   C[m][n] = sum_k A[m][k] B[k][n],  m < MB <= 8
//   workgroup  32 column-lanes x 8 k-lanes; a column-lane owns V = 16 / sizeof(T) adjacent columns
//              (one 16-byte load per row of B), so a workgroup reads 512 contiguous bytes per row
//   K          cut into S slices (grid.y) so that a few workgroups per CU exist; a slice is
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

template <typename T, int MB, typename TO>
__global__ __launch_bounds__(kBlock) void matmul_skinny_kernel(const T *__restrict__ A, const T *__restrict__ B, TO *__restrict__ out,
                                                                int M, int K, int N, int S, int chunk) {
    using AT = typename skinny_acc<T>::type;
    constexpr int V = kVecBytes / (int)sizeof(T);
    using VT = vec_t<T, V>;
    __shared__ AT a_lds[MB * kSub];
    __shared__ AT red[kBlock * V];
    const int tx = threadIdx.x % kSkinnyTX, ty = threadIdx.x / kSkinnyTX;
    const int64_t batch = blockIdx.z;
    const int s = blockIdx.y;
    const int nv = N / V;                       // launcher guarantees N % V == 0
    const int cv = blockIdx.x * kSkinnyTX + tx;  // vector column of this lane
    const bool active = cv < nv;
    A += batch * (int64_t)M * K;
    B += batch * (int64_t)K * N;
    const int k0 = s * chunk, k1 = (k0 + chunk < K) ? k0 + chunk : K;
    AT acc[MB][V];
#pragma unroll
    for (int m = 0; m < MB; ++m)
#pragma unroll
        for (int v = 0; v < V; ++v) acc[m][v] = AT(0);
    const VT *Bv = reinterpret_cast<const VT *>(B) + cv;
    for (int kb = k0; kb < k1; kb += kSub) {
        const int len = (kb + kSub < k1) ? kSub : k1 - kb;
        // The first four rows of B are requested before A is staged, so that their latency runs
        // under the staging; after that the next four are always in flight while four are used.
        constexpr int U = 4, STEP = U * kSkinnyTY;
        VT x[U];
        const bool batched = active && ty + (U - 1) * kSkinnyTY < len;
        if (batched) {
#pragma unroll
            for (int u = 0; u < U; ++u) x[u] = Bv[(int64_t)(kb + ty + u * kSkinnyTY) * nv];
        }
        __syncthreads();  // the previous sub-chunk's A values are no longer read
#pragma unroll
        for (int m = 0; m < MB; ++m)
            for (int r = threadIdx.x; r < len; r += kBlock) a_lds[m * kSub + r] = (m < M) ? AT(load_acc(A[(int64_t)m * K + kb + r])) : AT(0);
        __syncthreads();
        if (active) {
            auto use = [&](const VT(&b)[U], int r) __attribute__((always_inline)) {
#pragma unroll
                for (int u = 0; u < U; ++u)
#pragma unroll
                    for (int m = 0; m < MB; ++m) {
                        const AT a = a_lds[m * kSub + r + u * kSkinnyTY];
#pragma unroll
                        for (int v = 0; v < V; ++v) acc[m][v] = fma_acc(a, AT(load_acc(b[u].v[v])), acc[m][v]);
                    }
            };
            int r = ty;
            if (batched) {
                for (; r + STEP + (U - 1) * kSkinnyTY < len; r += STEP) {
                    VT y[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) y[u] = Bv[(int64_t)(kb + r + STEP + u * kSkinnyTY) * nv];
                    use(x, r);
#pragma unroll
                    for (int u = 0; u < U; ++u) x[u] = y[u];
                }
                use(x, r);
                r += STEP;
            }
            for (; r < len; r += kSkinnyTY) {
                const VT b = Bv[(int64_t)(kb + r) * nv];
#pragma unroll
                for (int m = 0; m < MB; ++m) {
                    const AT a = a_lds[m * kSub + r];
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

template <typename T, int MB>
int launch_skinny_mb(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    using AT = typename skinny_acc<T>::type;
    constexpr int V = kVecBytes / (int)sizeof(T);
    const int64_t ctiles = (n / V + kSkinnyTX - 1) / kSkinnyTX;
    // slices of K: about `per_cu` workgroups per CU, at least `min_rows` rows per slice, none under capture
    const int64_t per_cu = tuning().skinny_per_cu, min_rows = tuning().skinny_min_rows;
    int64_t S = (per_cu * (int64_t)compute_units() + batch * ctiles - 1) / (batch * ctiles);
    if (S > k / min_rows) S = k / min_rows;
    if (S < 1 || tuning().matmul_splitk == 1) S = 1;
    const int64_t partial = batch * m * n * (int64_t)sizeof(AT);
    if (S > 1 && (S * partial > kWorkspaceMaxBytes || stream_is_capturing(st))) S = 1;
    int64_t chunk = (k + S - 1) / S;
    chunk = (chunk + kSkinnyTY - 1) / kSkinnyTY * kSkinnyTY;
    S = (k + chunk - 1) / chunk;
    if (ctiles > 0x7fffffff || S > 65535 || batch > 65535) return kNoSkinny;
    const dim3 grid((unsigned)ctiles, (unsigned)S, (unsigned)batch);
    if (S == 1) {
        matmul_skinny_kernel<T, MB, T><<<grid, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, 1, (int)chunk);
        return launch_status();
    }
    std::lock_guard<std::recursive_mutex> hold(workspace_launch_mutex());
    AT *ws = (AT *)stream_workspace(st, kWorkspaceSplitK, (size_t)(partial * S));
    if (!ws) return kNoSkinny;
    matmul_skinny_kernel<T, MB, AT><<<grid, kBlock, 0, st>>>((const T *)a, (const T *)b, ws, (int)m, (int)k, (int)n, (int)S, (int)chunk);
    const int rc = launch_status();
    return rc != DXH_OK ? rc : launch_splitk_reduce<AT, T>(ws, (T *)c, batch, m * n, (int)S, st);
}

// Returns kNoSkinny when the shape is not one for this kernel (the caller goes on to the matrix pipe).
template <typename T>
int launch_skinny_t(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    constexpr int V = kVecBytes / (int)sizeof(T);
    if (m > 8 || k < 256 || n % V != 0 || !aligned(b, kVecBytes) || k > 0x7fffffff / 2 || tuning().matmul_tile != 0) return kNoSkinny;
    if (m == 1) return launch_skinny_mb<T, 1>(a, b, c, batch, m, k, n, st);
    if (m == 2) return launch_skinny_mb<T, 2>(a, b, c, batch, m, k, n, st);
    if (m <= 4) return launch_skinny_mb<T, 4>(a, b, c, batch, m, k, n, st);
    return launch_skinny_mb<T, 8>(a, b, c, batch, m, k, n, st);
}

// fp32 and fp64 by default.  The kernel is correct for bf16 / f16 as well (DXH_TUNE_SKINNY_HALF),
// but there the 64x64 matrix-pipe tiles over K slices are as
// fast or faster: one row of [4096,4096] takes 12.3 us against 14.2 here, eight rows 12.7 against
// 24.4 (eight conversions and multiply-adds per 2-byte element are vector-ALU-bound).  fp32:
// 19.3 against 28.6 us for one row of [4096,4096], 93 against 153 us for [896,151936] (5.9 TB/s).
int launch_matmul_skinny(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    switch (dtype) {
    case DXH_BF16: return tuning().skinny_half ? launch_skinny_t<bf16_t>(a, b, c, batch, m, k, n, st) : kNoSkinny;
    case DXH_F16: return tuning().skinny_half ? launch_skinny_t<f16_t>(a, b, c, batch, m, k, n, st) : kNoSkinny;
    case DXH_F32: return launch_skinny_t<float>(a, b, c, batch, m, k, n, st);
    case DXH_F64: return launch_skinny_t<double>(a, b, c, batch, m, k, n, st);
    default: return kNoSkinny;
    }
}

}  // namespace dxh
