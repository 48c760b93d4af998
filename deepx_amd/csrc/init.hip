// init.hip — constant fill and arange (executor/op-cuda init_miaobyte.cuh:18-30; arithmetic
// of executor/op-ompsimd/src/deepx/tensorfunc/init_miaobyte.hpp:16-70).
#include "common.hpp"
#include <ctime>

namespace dxh {

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void constant_kernel(T *__restrict__ out, int64_t n, const T value) {
    using VT = vec_t<T, V>;
    const int64_t nv = n / V;
    VT r;
#pragma unroll
    for (int k = 0; k < V; ++k) r.v[k] = value;
    VT *vo = reinterpret_cast<VT *>(out);
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < nv; i += stride) st_mode<3>(&vo[i], r);
    if (blockIdx.x == 0) {
        int64_t j = nv * V + threadIdx.x;
        if (j < n) out[j] = value;
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void arange_kernel(T *__restrict__ out, int64_t n, const T start, const T step) {
    using A = acc_t<T>;
    const A s0 = load_acc(start), s1 = load_acc(step);
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        if constexpr (std::is_integral_v<A>) {
            using U = std::conditional_t<(sizeof(A) < 4), uint32_t, std::make_unsigned_t<A>>;
            out[i] = store_acc<T>(A(U(U(s0) + U(U(A(i)) * U(s1)))));
        } else {
            out[i] = store_acc<T>(s0 + A(i) * s1);
        }
    }
}

// ---- counter-based random numbers: splitmix64 of (seed, index) -------------------------------
__host__ __device__ inline uint64_t mix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__device__ inline double u01(uint64_t seed, uint64_t idx) {  // [0,1) with 53 random bits
    return double(mix64(mix64(seed) ^ idx) >> 11) * 0x1.0p-53;
}
template <typename T> __device__ inline T from_double(double v) {
    if constexpr (std::is_same_v<T, bf16_t>) return to_bf16(float(v));
    else if constexpr (std::is_same_v<T, f16_t>) return to_f16(float(v));
    else return T(v);  // integers truncate like static_cast<T>(distribution(generator))
}
enum RandKind { RAND_UNIFORM, RAND_NORMAL };
template <typename T, int KIND>
__global__ __launch_bounds__(kBlock) void random_kernel(T *__restrict__ out, int64_t n, double a, double b, uint64_t seed) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        double v;
        if constexpr (KIND == RAND_UNIFORM) {
            v = a + (b - a) * u01(seed, (uint64_t)i);
        } else {  // Box-Muller on two independent uniforms
            double u1 = 1.0 - u01(seed, 2 * (uint64_t)i), u2 = u01(seed, 2 * (uint64_t)i + 1);
            v = a + b * sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2);
        }
        out[i] = from_double<T>(v);
    }
}
template <typename R>
__global__ __launch_bounds__(kBlock) void dropout_kernel(R *__restrict__ data, int64_t n, float p, uint64_t seed) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride)
        if (u01(seed, (uint64_t)i) < (double)p) data[i] = R(0);
}
inline uint64_t pick_seed(uint32_t seed) {
    if (seed != 0) return seed;
    static uint64_t counter = 0;
    return mix64((uint64_t)(uintptr_t)&counter ^ (uint64_t)clock() ^ (++counter << 32)) | 1;
}
template <typename T, int KIND> int launch_random(void *out, int64_t n, double a, double b, uint32_t seed, hipStream_t st) {
    if (!aligned(out, sizeof(T))) return DXH_ERR_ALIGN;
    random_kernel<T, KIND><<<stream_grid(n, kBlock, 16), kBlock, 0, st>>>((T *)out, n, a, b, pick_seed(seed));
    return launch_status();
}
template <int KIND> int random_all(int dtype, void *out, int64_t n, dxh_scalar a, dxh_scalar b, uint32_t seed, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(out);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return launch_random<double, KIND>(out, n, a.f, b.f, seed, st);
    case DXH_F32: return launch_random<float, KIND>(out, n, a.f, b.f, seed, st);
    case DXH_F16: return launch_random<f16_t, KIND>(out, n, a.f, b.f, seed, st);
    case DXH_BF16: return launch_random<bf16_t, KIND>(out, n, a.f, b.f, seed, st);
    case DXH_I64: return launch_random<int64_t, KIND>(out, n, (double)a.i, (double)b.i, seed, st);
    case DXH_I32: return launch_random<int32_t, KIND>(out, n, (double)a.i, (double)b.i, seed, st);
    case DXH_I16: return launch_random<int16_t, KIND>(out, n, (double)a.i, (double)b.i, seed, st);
    case DXH_I8: return launch_random<int8_t, KIND>(out, n, (double)a.i, (double)b.i, seed, st);
    default: return DXH_ERR_DTYPE;
    }
}

template <typename T> int launch_constant(void *out, int64_t n, dxh_scalar v, hipStream_t st) {
    if (!aligned(out, sizeof(T))) return DXH_ERR_ALIGN;
    constexpr int V = vec_len<T>;
    T x;
    if constexpr (std::is_same_v<T, bool_t>) x = bool_t{uint8_t(v.i ? 1 : 0)}; else x = scalar_to<T>(v);
    if (aligned(out, kVecBytes)) {
        unsigned g = stream_grid(n / V + 1, kBlock, 0);
        constant_kernel<T, V><<<g, kBlock, 0, st>>>((T *)out, n, x);
    } else {
        unsigned g = stream_grid(n, kBlock, 16);
        constant_kernel<T, 1><<<g, kBlock, 0, st>>>((T *)out, n, x);
    }
    return launch_status();
}
template <typename T> int launch_arange(void *out, int64_t n, dxh_scalar s0, dxh_scalar s1, hipStream_t st) {
    if (!aligned(out, sizeof(T))) return DXH_ERR_ALIGN;
    unsigned g = stream_grid(n, kBlock, 16);
    arange_kernel<T><<<g, kBlock, 0, st>>>((T *)out, n, scalar_to<T>(s0), scalar_to<T>(s1));
    return launch_status();
}

}  // namespace dxh

using namespace dxh;

extern "C" {

int dxh_constant(int dtype, void *out, int64_t n, dxh_scalar value, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(out);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return launch_constant<double>(out, n, value, st);
    case DXH_F32: return launch_constant<float>(out, n, value, st);
    case DXH_F16: return launch_constant<f16_t>(out, n, value, st);
    case DXH_BF16: return launch_constant<bf16_t>(out, n, value, st);
    case DXH_I64: return launch_constant<int64_t>(out, n, value, st);
    case DXH_I32: return launch_constant<int32_t>(out, n, value, st);
    case DXH_I16: return launch_constant<int16_t>(out, n, value, st);
    case DXH_I8: return launch_constant<int8_t>(out, n, value, st);
    case DXH_BOOL: return launch_constant<bool_t>(out, n, value, st);
    default: return DXH_ERR_DTYPE;
    }
}

int dxh_arange(int dtype, void *out, int64_t n, dxh_scalar start, dxh_scalar step, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(out);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return launch_arange<double>(out, n, start, step, st);
    case DXH_F32: return launch_arange<float>(out, n, start, step, st);
    case DXH_F16: return launch_arange<f16_t>(out, n, start, step, st);
    case DXH_BF16: return launch_arange<bf16_t>(out, n, start, step, st);
    case DXH_I64: return launch_arange<int64_t>(out, n, start, step, st);
    case DXH_I32: return launch_arange<int32_t>(out, n, start, step, st);
    case DXH_I16: return launch_arange<int16_t>(out, n, start, step, st);
    case DXH_I8: return launch_arange<int8_t>(out, n, start, step, st);
    default: return DXH_ERR_DTYPE;
    }
}

int dxh_uniform(int dtype, void *out, int64_t n, dxh_scalar low, dxh_scalar high, uint32_t seed, void *stream) {
    return random_all<RAND_UNIFORM>(dtype, out, n, low, high, seed, stream);
}
int dxh_normal(int dtype, void *out, int64_t n, dxh_scalar mean, dxh_scalar stddev, uint32_t seed, void *stream) {
    return random_all<RAND_NORMAL>(dtype, out, n, mean, stddev, seed, stream);
}
int dxh_dropout(int dtype, void *inout, int64_t n, float p, uint32_t seed, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(inout);
    const int es = dtype_size(dtype);
    if (!es) return DXH_ERR_DTYPE;
    if (!aligned(inout, es)) return DXH_ERR_ALIGN;
    hipStream_t st = as_stream(stream);
    const uint64_t sd = pick_seed(seed);
    unsigned g = stream_grid(n, kBlock, 16);
    switch (es) {  // zero has the same bit pattern in every dtype
    case 8: dropout_kernel<uint64_t><<<g, kBlock, 0, st>>>((uint64_t *)inout, n, p, sd); break;
    case 4: dropout_kernel<uint32_t><<<g, kBlock, 0, st>>>((uint32_t *)inout, n, p, sd); break;
    case 2: dropout_kernel<uint16_t><<<g, kBlock, 0, st>>>((uint16_t *)inout, n, p, sd); break;
    default: dropout_kernel<uint8_t><<<g, kBlock, 0, st>>>((uint8_t *)inout, n, p, sd); break;
    }
    return launch_status();
}

}  // extern "C"
