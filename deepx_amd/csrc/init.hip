// init.hip — constant fill and arange (executor/op-cuda init_miaobyte.cuh:18-30; arithmetic
// of executor/op-ompsimd/src/deepx/tensorfunc/init_miaobyte.hpp:16-70).
#include "common.hpp"

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
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < nv; i += stride) st_nt(&vo[i], r);
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

}  // extern "C"
