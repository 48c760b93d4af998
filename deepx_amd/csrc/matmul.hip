// matmul.hip — batched row-major GEMM  C[b,m,n] = sum_k A[b,m,k] * B[b,k,n]  (gfx950).
//
// Replaces cublasSgemm(StridedBatched) of executor/op-cuda/src/deepx/tensorfunc/matmul_cublas.hpp:16-145
// and cblas_sgemm of executor/op-ompsimd/src/deepx/tensorfunc/matmul_cblas.hpp:11-60 (alpha=1, beta=0).
//
//   bf16 / f16   matmul_half.hip: MFMA v_mfma_f32_32x32x16_{bf16,f16}, fp32 accumulate, one RNE
//                rounding of C.
//   f32 / f64    matmul_fp.hip: MFMA v_mfma_f32_32x32x2_f32 / v_mfma_f64_16x16x4_f64.
//   integers     here: LDS-tiled 64x64x16 multiply-add kernel, 4x4 outputs per lane; accumulate in
//                the storage type (integers wrap).
#include "matmul_common.hpp"

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
    for (int k0 = 0; k0 < K; k0 += GK) {
        // A tile 64x16: lanes along k (contiguous), 4 rows per lane
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const int r = (t >> 4) + h * 16, kc = t & 15;
            const int gm = m0 + r, gk = k0 + kc;
            As[kc][r] = (gm < M && gk < K) ? A[(int64_t)gm * K + gk] : T(0);
        }
        // B tile 16x64: lanes along n (contiguous), 4 k-rows per lane
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const int kr = (t >> 6) + h * 4, nc = t & 63;
            const int gk = k0 + kr, gn = n0 + nc;
            Bs[kr][nc] = (gk < K && gn < N) ? B[(int64_t)gk * N + gn] : T(0);
        }
        __syncthreads();
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

extern "C" int dxh_matmul(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n,
                          void *stream) {
    if (batch < 0 || m < 0 || k < 0 || n < 0) return DXH_ERR_ARG;
    if (m > 0x7fffffff || k > 0x7fffffff || n > 0x7fffffff) return DXH_ERR_SHAPE;
    const int es = dtype_size(dtype);
    if (!es || dtype == DXH_BOOL) return DXH_ERR_DTYPE;
    if (batch * m * n == 0) return DXH_OK;
    if (!c) return DXH_ERR_ARG;
    hipStream_t st = as_stream(stream);
    if (k == 0) {  // empty sum: a fill kernel rather than a memset node, so the call stays graph-capturable
        dxh_scalar zero = {0.0, 0};
        return dxh_constant(dtype, c, batch * m * n, zero, stream);
    }
    if (!a || !b) return DXH_ERR_ARG;
    if (!aligned(a, es) || !aligned(b, es) || !aligned(c, es)) return DXH_ERR_ALIGN;
    switch (dtype) {
    case DXH_BF16:
    case DXH_F16: return launch_matmul_half(dtype, a, b, c, batch, m, k, n, st);
    case DXH_F32: return launch_matmul_f32(a, b, c, batch, m, k, n, st);
    case DXH_F64: return launch_matmul_f64(a, b, c, batch, m, k, n, st);
    case DXH_I64: return launch_tiled<int64_t>(a, b, c, batch, m, k, n, st);
    case DXH_I32: return launch_tiled<int32_t>(a, b, c, batch, m, k, n, st);
    case DXH_I16: return launch_tiled<int16_t>(a, b, c, batch, m, k, n, st);
    case DXH_I8: return launch_tiled<int8_t>(a, b, c, batch, m, k, n, st);
    default: return DXH_ERR_DTYPE;
    }
}

