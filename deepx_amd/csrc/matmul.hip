// matmul.hip — batched row-major GEMM  C[b,m,n] = sum_k A[b,m,k] * B[b,k,n]  (gfx950).
//
// Replaces cublasSgemm(StridedBatched) of executor/op-cuda/src/deepx/tensorfunc/matmul_cublas.hpp:16-145
// and cblas_sgemm of executor/op-ompsimd/src/deepx/tensorfunc/matmul_cblas.hpp:11-60 (alpha=1, beta=0).
//
//   bf16 / f16   matmul_half.hip: MFMA v_mfma_f32_32x32x16_{bf16,f16}, fp32 accumulate, one RNE
//                rounding of C.
//   f32 / f64    matmul_fp.hip: MFMA v_mfma_f32_32x32x2_f32 / v_mfma_f64_16x16x4_f64.
//   M <= 8       matmul_skinny.hip (floats): vector-ALU stream over B, K cut into slices.
//   integers     here: LDS-tiled 64x64x16 multiply-add kernel, 4x4 outputs per lane; accumulate in
//                the storage type (integers wrap).  int8 with at least 8 output tiles of 128x128:
//                v_mfma_i32_32x32x16_i8, int32 accumulate, low 8 bits stored (the same value).
#include "matmul_common.hpp"
#include <algorithm>

namespace dxh {

// ---- integer kernel: LDS-tiled multiply-add ------------------------------------------------
constexpr int GT = 64, GK = 16;
template <typename T>
__global__ __launch_bounds__(kBlock) void matmul_tiled_kernel(const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C,
                                                               int M, int K, int N, int tiles_m, int tiles_n) {
    __shared__ T As[GK][GT + 1];  // [k][m]
    __shared__ T Bs[GK][GT + 1];  // [k][n]
    int64_t bid = blockIdx.x;
    const int tn = (int)(bid % tiles_n); bid /= tiles_n;
    const int tm = (int)(bid % tiles_m); bid /= tiles_m;
    A += bid * (int64_t)M * K;
    B += bid * (int64_t)K * N;
    C += bid * (int64_t)M * N;
    const int m0 = tm * GT, n0 = tn * GT;
    const int t = threadIdx.x, tx = t & 15, ty = t >> 4;
    T acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = T(0);
    // The next K step is fetched into registers while the current one is multiplied.  Loads are
    // from clamped addresses and masked when they move to LDS: a select right at the load would
    // make the loop wait for its own prefetch.
    T ra[4], rb[4];
    auto fetch = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int h = 0; h < 4; ++h) {  // A tile 64x16: lanes along k (contiguous), 4 rows per lane
            const int gm = m0 + (t >> 4) + h * 16, gk = k0 + (t & 15);
            ra[h] = A[(int64_t)(gm < M ? gm : M - 1) * K + (gk < K ? gk : K - 1)];
        }
#pragma unroll
        for (int h = 0; h < 4; ++h) {  // B tile 16x64: lanes along n (contiguous), 4 k-rows per lane
            const int gk = k0 + (t >> 6) + h * 4, gn = n0 + (t & 63);
            rb[h] = B[(int64_t)(gk < K ? gk : K - 1) * N + (gn < N ? gn : N - 1)];
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += GK) {
#pragma unroll
        for (int h = 0; h < 4; ++h) As[t & 15][(t >> 4) + h * 16] = (m0 + (t >> 4) + h * 16 < M && k0 + (t & 15) < K) ? ra[h] : T(0);
#pragma unroll
        for (int h = 0; h < 4; ++h) Bs[(t >> 6) + h * 4][t & 63] = (k0 + (t >> 6) + h * 4 < K && n0 + (t & 63) < N) ? rb[h] : T(0);
        __syncthreads();
        if (k0 + GK < K) fetch(k0 + GK);
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            T a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx + j * 16];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if constexpr (std::is_integral_v<T>) {
                        using U = std::conditional_t<(sizeof(T) < 4), uint32_t, std::make_unsigned_t<T>>;
                        acc[i][j] = T(U(U(acc[i][j]) + U(U(a[i]) * U(b[j]))));
                    } else {
                        acc[i][j] = __builtin_fma(a[i], b[j], acc[i][j]);
                    }
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = m0 + ty * 4 + i, col = n0 + tx + j * 16;
            if (row < M && col < N) C[(int64_t)row * N + col] = acc[i][j];
        }
}

// ---- int8 on the matrix pipe -------------------------------------------------------------
// v_mfma_i32_32x32x16_i8: lane L supplies 8 consecutive k (one 64-bit register) of row / column
// L % 32, k = 8 (L / 32) + j, and accumulates in int32; the result layout is that of the other
// 32x32 MFMAs (column L % 32, row 8 (v / 4) + 4 (L / 32) + v % 4).  int32 sums of int8 products
// are exact up to K = 2^17 and wrap modulo 2^32 beyond, so the low 8 bits always equal the
// reference's accumulation in the storage type (arithmetic modulo 2^8).
// Workgroup tile 128 x 128, K step 64 bytes, 4 waves 2 x 2 with 2 x 2 MFMA tiles each; A is kept
// [m][k] in LDS and B transposed to [n][k] while it is stored, so both operands are 8-byte reads.
constexpr int IM = 128, IN = 128, IK = 64, ILD = IK + 16;  // LDS row stride 80 bytes: 16-byte aligned rows
typedef int i32x16 __attribute__((ext_vector_type(16)));
template <bool VEC>
__global__ __launch_bounds__(kBlock) void matmul_i8_mfma_kernel(const int8_t *__restrict__ A, const int8_t *__restrict__ B, int8_t *__restrict__ C,
                                                                 int M, int K, int N, int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(16))) int8_t As[IM * ILD];
    __shared__ __attribute__((aligned(16))) int8_t Bs[IN * ILD];  // [n][k]
    int64_t bid = blockIdx.x;
    const int tn = (int)(bid % tiles_n); bid /= tiles_n;
    const int tm = (int)(bid % tiles_m); bid /= tiles_m;
    A += bid * (int64_t)M * K;
    B += bid * (int64_t)K * N;
    C += bid * (int64_t)M * N;
    const int m0 = tm * IM, n0 = tn * IN;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wm = w >> 1, wn = w & 1;
    i32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0;
    for (int k0 = 0; k0 < K; k0 += IK) {
        // A tile: 128 rows x 64 k, 16 bytes per lane and half
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int r = (t >> 2) + h * 64, kc = (t & 3) * 16, gm = m0 + r, gk = k0 + kc;
            vec_t<int8_t, 16> x;
            if (VEC && gm < M && gk + 16 <= K) {
                x = *reinterpret_cast<const vec_t<int8_t, 16> *>(A + (int64_t)gm * K + gk);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) x.v[e] = (gm < M && gk + e < K) ? A[(int64_t)gm * K + gk + e] : (int8_t)0;
            }
            *reinterpret_cast<vec_t<int8_t, 16> *>(&As[r * ILD + kc]) = x;
        }
        // B tile: 64 k x 128 n, 16 bytes (16 n) per lane and half, transposed into Bs[n][k]
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int kr = (t >> 3) + h * 32, nc = (t & 7) * 16, gk = k0 + kr, gn = n0 + nc;
            vec_t<int8_t, 16> x;
            if (VEC && gk < K && gn + 16 <= N) {
                x = *reinterpret_cast<const vec_t<int8_t, 16> *>(B + (int64_t)gk * N + gn);
            } else {
#pragma unroll
                for (int e = 0; e < 16; ++e) x.v[e] = (gk < K && gn + e < N) ? B[(int64_t)gk * N + gn + e] : (int8_t)0;
            }
#pragma unroll
            for (int e = 0; e < 16; ++e) Bs[(nc + e) * ILD + kr] = x.v[e];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < IK; kk += 16) {
            const int ko = kk + (lane >> 5) * 8;
            long af[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) af[i] = *reinterpret_cast<const long *>(&As[(wm * 64 + i * 32 + (lane & 31)) * ILD + ko]);
#pragma unroll
            for (int j = 0; j < 2; ++j) bf[j] = *reinterpret_cast<const long *>(&Bs[(wn * 64 + j * 32 + (lane & 31)) * ILD + ko]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x16_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * 64 + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                const int col = n0 + wn * 64 + j * 32 + (lane & 31);
                if (row < M && col < N) C[(int64_t)row * N + col] = (int8_t)acc[i][j][v];
            }
}
int launch_i8_mfma(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    const int64_t tiles_m = (m + IM - 1) / IM, tiles_n = (n + IN - 1) / IN;
    const int64_t blocks = batch * tiles_m * tiles_n;
    if (blocks > 0x7fffffff) return DXH_ERR_SHAPE;
    const bool vec = k % 16 == 0 && n % 16 == 0 && aligned(a, kVecBytes) && aligned(b, kVecBytes);
    if (vec) matmul_i8_mfma_kernel<true><<<(unsigned)blocks, kBlock, 0, st>>>((const int8_t *)a, (const int8_t *)b, (int8_t *)c, (int)m, (int)k, (int)n, (int)tiles_m, (int)tiles_n);
    else matmul_i8_mfma_kernel<false><<<(unsigned)blocks, kBlock, 0, st>>>((const int8_t *)a, (const int8_t *)b, (int8_t *)c, (int)m, (int)k, (int)n, (int)tiles_m, (int)tiles_n);
    return launch_status();
}

template <typename T>
int launch_tiled(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    const int64_t tiles_m = (m + GT - 1) / GT, tiles_n = (n + GT - 1) / GT;
    const int64_t blocks = batch * tiles_m * tiles_n;
    if (blocks > 0x7fffffff) return DXH_ERR_SHAPE;
    matmul_tiled_kernel<T><<<(unsigned)blocks, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, (int)tiles_m, (int)tiles_n);
    return launch_status();
}


}  // namespace dxh

using namespace dxh;

// One dispatcher for the real call and for the workspace query (sc.planning).
static int matmul_dispatch(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n,
                           void *stream, Scratch &sc) {
    if (batch < 0 || m < 0 || k < 0 || n < 0) return DXH_ERR_ARG;
    if (m > 0x7fffffff || k > 0x7fffffff || n > 0x7fffffff) return DXH_ERR_SHAPE;
    const int es = dtype_size(dtype);
    if (!es || dtype == DXH_BOOL) return DXH_ERR_DTYPE;
    if (batch * m * n == 0) return DXH_OK;
    if (!c) return DXH_ERR_ARG;
    hipStream_t st = as_stream(stream);
    if (k == 0) {  // empty sum: a fill kernel rather than a memset node, so the call stays graph-capturable
        if (sc.planning) return DXH_OK;
        dxh_scalar zero = {0.0, 0};
        return dxh_constant(dtype, c, batch * m * n, zero, stream);
    }
    if (!a || !b) return DXH_ERR_ARG;
    if (!aligned(a, es) || !aligned(b, es) || !aligned(c, es)) return DXH_ERR_ALIGN;
    if (m <= 16) {  // a few rows of A: a stream over B, not matrix-pipe work
        const int rc = launch_matmul_skinny(dtype, a, b, c, batch, m, k, n, st, sc);
        if (rc != kNoSkinny) return rc;
    }
    switch (dtype) {
    case DXH_BF16:
    case DXH_F16: return launch_matmul_half(dtype, a, b, c, batch, m, k, n, st, sc);
    case DXH_F32: return launch_matmul_f32(a, b, c, batch, m, k, n, st, sc);
    case DXH_F64: return launch_matmul_f64(a, b, c, batch, m, k, n, st, sc);
    default: break;
    }
    if (sc.planning) return DXH_OK;  // the integer kernels need no scratch
    switch (dtype) {
    case DXH_I64: return launch_tiled<int64_t>(a, b, c, batch, m, k, n, st);
    case DXH_I32: return launch_tiled<int32_t>(a, b, c, batch, m, k, n, st);
    case DXH_I16: return launch_tiled<int16_t>(a, b, c, batch, m, k, n, st);
    case DXH_I8:  // small products stay on the 64x64 kernel: a 128x128 tile would leave most CUs idle
        return (m >= 64 && n >= 64 && batch * ((m + 127) / 128) * ((n + 127) / 128) >= 8) ? launch_i8_mfma(a, b, c, batch, m, k, n, st)
                                                                                        : launch_tiled<int8_t>(a, b, c, batch, m, k, n, st);
    default: return DXH_ERR_DTYPE;
    }
}

extern "C" int dxh_matmul_workspace_bytes(int dtype, const void *a, const void *b, const void *c, int64_t batch, int64_t m,
                                          int64_t k, int64_t n, size_t *bytes) {
    if (!bytes) return DXH_ERR_ARG;
    *bytes = 0;
    Scratch sc;
    sc.planning = true;
    const int rc = matmul_dispatch(dtype, a, b, const_cast<void *>(c), batch, m, k, n, nullptr, sc);
    if (rc == DXH_OK) *bytes = sc.used;
    return rc;
}

// C_j = A B_j, j < count: one launch where the products take an LDS-direct tile uncut, else one after another
// (each with the whole workspace: launches of one stream run in order).
static int matmul_shared_dispatch(int dtype, const void *a, const void *const *bs, void *const *cs, int count, int64_t m, int64_t k, int64_t n,
                                  void *stream, Scratch &sc) {
    if (count < 1 || !bs || !cs || m < 0 || k < 0 || n < 0) return DXH_ERR_ARG;
    for (int j = 0; j < count; ++j) {
        if (!cs[j] && m * n > 0) return DXH_ERR_ARG;
        for (int i = 0; i < j; ++i)
            if (cs[i] == cs[j] && m * n > 0) return DXH_ERR_ARG;  // two products into one result
    }
    if ((dtype == DXH_BF16 || dtype == DXH_F16) && count >= 2 && m * n * k > 0 && a) {
        bool all = true;
        for (int j = 0; j < count; ++j) all = all && bs[j] && cs[j];
        auto group = [&](int at) {
            SharedA g{};
            g.count = std::min(count - at, kSharedAMax);
            for (int j = 0; j < g.count; ++j) { g.b[j] = bs[at + j]; g.c[j] = cs[at + j]; }
            return g;
        };
        // every group of pairs takes the same decision (same shape; the alignment of each pair is looked at)
        bool shared = all;
        for (int at = 0; shared && at < count; at += kSharedAMax) {
            const SharedA g = group(at);
            if (g.count >= 2) shared = launch_matmul_half_shared(dtype, a, g, m, k, n, nullptr, true) == DXH_OK;
        }
        if (shared) {
            for (int at = 0; at < count; at += kSharedAMax) {
                const SharedA g = group(at);
                int rc;
                if (g.count >= 2) rc = sc.planning ? DXH_OK : launch_matmul_half_shared(dtype, a, g, m, k, n, as_stream(stream), false);
                else rc = matmul_dispatch(dtype, a, bs[at], cs[at], 1, m, k, n, stream, sc);  // one pair left over
                if (rc != DXH_OK) return rc;
            }
            return DXH_OK;
        }
    }
    size_t most = 0;
    for (int j = 0; j < count; ++j) {
        Scratch one = sc;
        one.used = 0;
        const int rc = matmul_dispatch(dtype, a, bs[j], cs[j], 1, m, k, n, stream, one);
        if (rc != DXH_OK) return rc;
        most = std::max(most, one.used);
    }
    sc.used = most;
    return DXH_OK;
}

extern "C" int dxh_matmul_shared_a_workspace_bytes(int dtype, const void *a, const void *const *bs, void *const *cs, int count, int64_t m, int64_t k, int64_t n,
                                                   size_t *bytes) {
    if (!bytes) return DXH_ERR_ARG;
    *bytes = 0;
    Scratch sc;
    sc.planning = true;
    const int rc = matmul_shared_dispatch(dtype, a, bs, cs, count, m, k, n, nullptr, sc);
    if (rc == DXH_OK) *bytes = sc.used;
    return rc;
}

extern "C" int dxh_matmul_shared_a(int dtype, const void *a, const void *const *bs, void *const *cs, int count, int64_t m, int64_t k, int64_t n,
                                   void *workspace, size_t workspace_bytes, void *stream) {
    if (workspace && !aligned(workspace, 256)) return DXH_ERR_WORKSPACE;
    Scratch sc;
    sc.base = (char *)workspace;
    sc.bytes = workspace ? workspace_bytes : 0;
    return matmul_shared_dispatch(dtype, a, bs, cs, count, m, k, n, stream, sc);
}

extern "C" int dxh_matmul(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n,
                          void *workspace, size_t workspace_bytes, void *stream) {
    if (workspace && !aligned(workspace, 256)) return DXH_ERR_WORKSPACE;
    Scratch sc;
    sc.base = (char *)workspace;
    sc.bytes = workspace ? workspace_bytes : 0;
    return matmul_dispatch(dtype, a, b, c, batch, m, k, n, stream, sc);
}
