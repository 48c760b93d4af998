// compare.hip — compare -> bool mask, switch (select) and todtype (cast) kernels.
//
// All HBM-bound streaming kernels: 16-byte loads on the widest operand, the narrow
// operand (1-byte masks, the smaller side of a cast) moves with proportionally smaller
// accesses so that every wave access stays contiguous.
// Semantics: executor/op-ompsimd/src/deepx/tensorfunc/elementwise_miaobyte.hpp:767-1027
// (compare, switch) and :103-112 (todtype).
#include "common.hpp"
#include <limits>

namespace dxh {

constexpr int kUnrollC = 1;
constexpr int kBlocksPerCUC = 0;

template <int U, typename Body> __device__ inline void tile_loop_c(int64_t nv, Body body) {
    const int64_t tile = (int64_t)kBlock * U;
    const int64_t stride = (int64_t)gridDim.x * tile;
    for (int64_t base = (int64_t)blockIdx.x * tile; base < nv; base += stride) {
        if (base + tile <= nv) body(base + threadIdx.x, std::true_type{});
        else body(base + threadIdx.x, std::false_type{});
    }
}

enum CmpKind { CMP_EQ, CMP_NE, CMP_LT, CMP_GT };

template <typename A> __device__ inline bool within_eps(A a, A b, float eps) {
    if constexpr (std::is_integral_v<A>) {
        // std::abs(a-b) <= epsilon on integers: the difference is converted to float
        uint64_t d = (uint64_t)(int64_t)a - (uint64_t)(int64_t)b;
        uint64_t ad = ((int64_t)d < 0) ? (uint64_t)0 - d : d;
        return float(ad) <= eps;
    } else if constexpr (std::is_same_v<A, double>) {
        return fabs(a - b) <= (double)eps;
    } else {
        return fabsf(a - b) <= eps;
    }
}
template <typename A> __device__ inline bool beyond_eps(A a, A b, float eps) {
    if constexpr (std::is_integral_v<A>) return !within_eps(a, b, eps);
    else if constexpr (std::is_same_v<A, double>) return fabs(a - b) > (double)eps;
    else return fabsf(a - b) > eps;
}
template <int K, typename A> __device__ inline uint8_t cmp_one(A a, A b, float eps) {
    bool r;
    if constexpr (K == CMP_EQ) r = (eps == 0.0f) ? (a == b) : within_eps<A>(a, b, eps);
    else if constexpr (K == CMP_NE) r = (eps == 0.0f) ? (a != b) : beyond_eps<A>(a, b, eps);
    else if constexpr (K == CMP_LT) r = a < b;
    else r = a > b;
    return r ? 1 : 0;
}

// SCALAR=true compares against `s`, otherwise against b[i].
// Vectors per lane and trip: a comparison with a scalar has one load stream, and a single 16-byte
// load per lane does not keep it busy (fp32 equalscalar, 64 / 256 MiB: 4.8 / 5.7 TB/s with one
// vector per lane, 5.6 / 6.0 with four); with two load streams, and for 1-byte elements, one
// vector per lane measured the same or better.
template <typename T, bool SCALAR> constexpr int compare_unroll = (SCALAR && sizeof(T) > 1) ? 4 : 1;
template <typename T, int V, int K, bool SCALAR, bool NTL>
__device__ __forceinline__ void compare_body(const T *__restrict__ a, const T *__restrict__ b, const T s,
                                                          float eps, uint8_t *__restrict__ m, int64_t n) {
    using VT = vec_t<T, V>;
    using MT = vec_t<uint8_t, V>;
    using A = acc_t<T>;
    constexpr int UC = compare_unroll<T, SCALAR>;
    const int64_t nv = n / V;
    const A sv = load_acc(s);
    const VT *va = reinterpret_cast<const VT *>(a);
    const VT *vb = reinterpret_cast<const VT *>(b);
    MT *vm = reinterpret_cast<MT *>(m);
    tile_loop_c<UC>(nv, [&](int64_t i, auto full) {
        VT x[UC], y[UC];
#pragma unroll
        for (int u = 0; u < UC; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) {
                x[u] = ld_sel<NTL>(&va[j]);
                if constexpr (!SCALAR) y[u] = ld_sel<NTL>(&vb[j]);
            }
        }
#pragma unroll
        for (int u = 0; u < UC; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) {
                MT r;
#pragma unroll
                for (int k = 0; k < V; ++k) {
                    A bb;
                    if constexpr (SCALAR) bb = sv; else bb = A(load_acc(y[u].v[k]));
                    r.v[k] = cmp_one<K, A>(A(load_acc(x[u].v[k])), bb, eps);
                }
                vm[j] = r;  // masks are a quarter or less of the traffic: plain stores
            }
        }
    });
    if (blockIdx.x == 0) {
        int64_t j = nv * V + threadIdx.x;
        if (j < n) {
            A bb;
            if constexpr (SCALAR) bb = sv; else bb = A(load_acc(b[j]));
            m[j] = cmp_one<K, A>(A(load_acc(a[j])), bb, eps);
        }
    }
}
template <typename T, int V, int K, bool SCALAR>
__global__ __launch_bounds__(kBlock) void compare_kernel(const T *__restrict__ a, const T *__restrict__ b, const T s, float eps, uint8_t *__restrict__ m, int64_t n, int ntl) {
    if (ntl) compare_body<T, V, K, SCALAR, true>(a, b, s, eps, m, n);
    else compare_body<T, V, K, SCALAR, false>(a, b, s, eps, m, n);
}

template <typename T, int K, bool SCALAR>
int launch_compare(const void *a, const void *b, dxh_scalar s, float eps, void *m, int64_t n, hipStream_t st) {
    if (!aligned(a, sizeof(T)) || (!SCALAR && !aligned(b, sizeof(T)))) return DXH_ERR_ALIGN;
    constexpr int V = vec_len<T>;
    const T sv = SCALAR ? scalar_to<T>(s) : T{};
    // a comparison reads 1..16 bytes per mask byte, a read-dominated stream: nt loads from 16 MiB up
    // (fp32 / bf16 equalscalar at 64 MiB: 4742 / 4764 GB/s with nt loads, 4658 / 3898 without)
    const int ntl = SCALAR ? nt_load_forced((size_t)n * sizeof(T) > ((size_t)16 << 20)) : nt_load_2r1w((size_t)n * (2 * sizeof(T) + 1));
    if (aligned(a, kVecBytes) && (SCALAR || aligned(b, kVecBytes)) && aligned(m, V)) {
        unsigned g = stream_grid(n / V + 1, (int64_t)kBlock * compare_unroll<T, SCALAR>, kBlocksPerCUC);
        compare_kernel<T, V, K, SCALAR><<<g, kBlock, 0, st>>>((const T *)a, (const T *)b, sv, eps, (uint8_t *)m, n, ntl);
    } else {
        unsigned g = stream_grid(n, (int64_t)kBlock * compare_unroll<T, SCALAR>, kBlocksPerCUC);
        compare_kernel<T, 1, K, SCALAR><<<g, kBlock, 0, st>>>((const T *)a, (const T *)b, sv, eps, (uint8_t *)m, n, ntl);
    }
    return launch_status();
}

template <int K, bool SCALAR>
int compare_all(int dtype, const void *a, const void *b, dxh_scalar s, float eps, void *m, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(m);
    if (!SCALAR) DXH_CHECK_PTR(b);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return launch_compare<double, K, SCALAR>(a, b, s, eps, m, n, st);
    case DXH_F32: return launch_compare<float, K, SCALAR>(a, b, s, eps, m, n, st);
    case DXH_F16: return launch_compare<f16_t, K, SCALAR>(a, b, s, eps, m, n, st);
    case DXH_BF16: return launch_compare<bf16_t, K, SCALAR>(a, b, s, eps, m, n, st);
    case DXH_I64: return launch_compare<int64_t, K, SCALAR>(a, b, s, eps, m, n, st);
    case DXH_I32: return launch_compare<int32_t, K, SCALAR>(a, b, s, eps, m, n, st);
    case DXH_I16: return launch_compare<int16_t, K, SCALAR>(a, b, s, eps, m, n, st);
    case DXH_I8: return launch_compare<int8_t, K, SCALAR>(a, b, s, eps, m, n, st);
    default: return DXH_ERR_DTYPE;
    }
}

// ---- switch ------------------------------------------------------------------------------
struct SwitchPtrs { const void *p[DXH_SWITCH_MAX]; };

// bool cases, two tensors: C[i] = cases[i] ? t1[i] : t0[i]; both sources stream.
template <typename R, int V, bool NTS, bool NTL>
__device__ __forceinline__ void switch_bool_body(const R *__restrict__ t0, const R *__restrict__ t1,
                                                              const uint8_t *__restrict__ cases, R *__restrict__ c, int64_t n) {
    using VT = vec_t<R, V>;
    using MT = vec_t<uint8_t, V>;
    const int64_t nv = n / V;
    const VT *v0 = reinterpret_cast<const VT *>(t0);
    const VT *v1 = reinterpret_cast<const VT *>(t1);
    const MT *vm = reinterpret_cast<const MT *>(cases);
    VT *vc = reinterpret_cast<VT *>(c);
    tile_loop_c<kUnrollC>(nv, [&](int64_t i, auto full) {
        VT x[kUnrollC], y[kUnrollC];
        MT w[kUnrollC];
#pragma unroll
        for (int u = 0; u < kUnrollC; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) { x[u] = ld_sel<NTL>(&v0[j]); y[u] = ld_sel<NTL>(&v1[j]); w[u] = ld_sel<NTL>(&vm[j]); }
        }
#pragma unroll
        for (int u = 0; u < kUnrollC; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) {
                VT r;
#pragma unroll
                for (int k = 0; k < V; ++k) r.v[k] = w[u].v[k] ? y[u].v[k] : x[u].v[k];
                st_sel<NTS>(&vc[j], r);
            }
        }
    });
    if (blockIdx.x == 0) {
        int64_t j = nv * V + threadIdx.x;
        if (j < n) c[j] = cases[j] ? t1[j] : t0[j];
    }
}
template <typename R, int V, bool NTS>
__global__ __launch_bounds__(kBlock) void switch_bool_kernel(const R *__restrict__ t0, const R *__restrict__ t1, const uint8_t *__restrict__ cases, R *__restrict__ c, int64_t n, int ntl) {
    if (ntl) switch_bool_body<R, V, NTS, true>(t0, t1, cases, c, n);
    else switch_bool_body<R, V, NTS, false>(t0, t1, cases, c, n);
}

// int32 cases, up to DXH_SWITCH_MAX tensors: only the selected source is read.
template <typename R>
__global__ __launch_bounds__(kBlock) void switch_i32_kernel(SwitchPtrs t, int nt, const int32_t *__restrict__ cases,
                                                             R *__restrict__ c, int64_t n) {
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        int32_t w = cases[i];
        R v = R(0);
#pragma unroll
        for (int k = 0; k < DXH_SWITCH_MAX; ++k)
            if (k < nt && w == k) v = reinterpret_cast<const R *>(t.p[k])[i];
        c[i] = v;
    }
}

template <typename R>
int launch_switch(const void *const *tensors, int nt, int cases_dtype, const void *cases, void *c, int64_t n, hipStream_t st) {
    for (int k = 0; k < nt; ++k) if (!tensors[k] || !aligned(tensors[k], sizeof(R))) return tensors[k] ? DXH_ERR_ALIGN : DXH_ERR_ARG;
    if (!aligned(c, sizeof(R))) return DXH_ERR_ALIGN;
    if (cases_dtype == DXH_BOOL) {
        if (nt != 2) return DXH_ERR_ARG;
        constexpr int V = kVecBytes / (int)sizeof(R);
        const int ntl = nt_load_2r1w((size_t)n * (3 * sizeof(R) + 1));
        if (aligned(tensors[0], kVecBytes) && aligned(tensors[1], kVecBytes) && aligned(c, kVecBytes) && aligned(cases, V)) {
            unsigned g = stream_grid(n / V + 1, (int64_t)kBlock * kUnrollC, kBlocksPerCUC);
            if (use_nt_store((size_t)n * sizeof(R))) switch_bool_kernel<R, V, true><<<g, kBlock, 0, st>>>((const R *)tensors[0], (const R *)tensors[1], (const uint8_t *)cases, (R *)c, n, ntl);
            else switch_bool_kernel<R, V, false><<<g, kBlock, 0, st>>>((const R *)tensors[0], (const R *)tensors[1], (const uint8_t *)cases, (R *)c, n, ntl);
        } else {
            unsigned g = stream_grid(n, (int64_t)kBlock * kUnrollC, kBlocksPerCUC);
            switch_bool_kernel<R, 1, false><<<g, kBlock, 0, st>>>((const R *)tensors[0], (const R *)tensors[1], (const uint8_t *)cases, (R *)c, n, ntl);
        }
    } else if (cases_dtype == DXH_I32) {
        if (!aligned(cases, 4)) return DXH_ERR_ALIGN;
        SwitchPtrs t{};
        for (int k = 0; k < nt; ++k) t.p[k] = tensors[k];
        unsigned g = stream_grid(n, kBlock, 16);
        switch_i32_kernel<R><<<g, kBlock, 0, st>>>(t, nt, (const int32_t *)cases, (R *)c, n);
    } else {
        return DXH_ERR_DTYPE;
    }
    return launch_status();
}

// ---- todtype -----------------------------------------------------------------------------
template <typename D, typename S> __device__ inline D cast_elem(S v) {
    if constexpr (std::is_same_v<S, bf16_t> || std::is_same_v<S, f16_t>) {
        return cast_elem<D, float>(load_acc(v));
    } else if constexpr (std::is_same_v<D, bf16_t> || std::is_same_v<D, f16_t>) {
        float f;
        if constexpr (std::is_same_v<S, float>) {
            f = v;
        } else {
            // double / integer sources: one rounding only.  Round to float toward zero,
            // then set the sticky bit (round-to-odd) so the final RNE sees the lost bits.
            double d = double(v);
            f = __double2float_rz(d);
            if (double(f) != d && !isinf(f) && !isnan(d)) f = bits_to_float(float_to_bits(f) | 1u);
        }
        if constexpr (std::is_same_v<D, bf16_t>) return to_bf16(f); else return to_f16(f);
    } else if constexpr (std::is_floating_point_v<S> && std::is_integral_v<D>) {
        if (v != v) return D(0);
        double d = trunc(double(v));
        const double lo = double(std::numeric_limits<D>::min());
        const double hi = double(std::numeric_limits<D>::max());
        if (d <= lo) return std::numeric_limits<D>::min();
        if (d >= hi) return std::numeric_limits<D>::max();
        return D(d);
    } else {
        return D(v);
    }
}

// Vectors per lane and trip: a narrowing cast is read-dominated and wants several loads in flight
// per lane (int32 -> int8 at 256 MiB: 5.1 TB/s with one vector per lane, 6.9 with four); a widening
// or same-size one is write-dominated and measured 5-8 % faster with one.
template <typename S, typename D> constexpr int cast_unroll = sizeof(D) < sizeof(S) ? 4 : 1;
template <typename S, typename D, int V, bool NTS, bool NTL>
__device__ __forceinline__ void cast_body(const S *__restrict__ a, D *__restrict__ c, int64_t n) {
    using VS = vec_t<S, V>;
    using VD = vec_t<D, V>;
    const int64_t nv = n / V;
    const VS *va = reinterpret_cast<const VS *>(a);
    VD *vc = reinterpret_cast<VD *>(c);
    tile_loop_c<cast_unroll<S, D>>(nv, [&](int64_t i, auto full) {
        VS x[cast_unroll<S, D>];
#pragma unroll
        for (int u = 0; u < cast_unroll<S, D>; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) x[u] = ld_sel<NTL>(&va[j]);
        }
#pragma unroll
        for (int u = 0; u < cast_unroll<S, D>; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) {
                VD r;
#pragma unroll
                for (int k = 0; k < V; ++k) r.v[k] = cast_elem<D, S>(x[u].v[k]);
                st_sel<NTS>(&vc[j], r);
            }
        }
    });
    if (blockIdx.x == 0) {
        int64_t j = nv * V + threadIdx.x;
        if (j < n) c[j] = cast_elem<D, S>(a[j]);
    }
}
template <typename S, typename D, int V, bool NTS>
__global__ __launch_bounds__(kBlock) void cast_kernel(const S *__restrict__ a, D *__restrict__ c, int64_t n, int ntl) {
    if (ntl) cast_body<S, D, V, NTS, true>(a, c, n);
    else cast_body<S, D, V, NTS, false>(a, c, n);
}

template <typename S, typename D> int launch_cast(const void *a, void *c, int64_t n, hipStream_t st) {
    if (!aligned(a, sizeof(S)) || !aligned(c, sizeof(D))) return DXH_ERR_ALIGN;
    constexpr int W = sizeof(S) > sizeof(D) ? sizeof(S) : sizeof(D);
    constexpr int V = kVecBytes / W;  // the wider side moves 16 bytes per lane
    const int ntl = nt_load_1r1w((size_t)n * sizeof(S), (size_t)n * sizeof(D));
    if (aligned(a, V * sizeof(S)) && aligned(c, V * sizeof(D))) {
        unsigned g = stream_grid(n / V + 1, (int64_t)kBlock * cast_unroll<S, D>, kBlocksPerCUC);
        if (use_nt_store((size_t)n * sizeof(D))) cast_kernel<S, D, V, true><<<g, kBlock, 0, st>>>((const S *)a, (D *)c, n, ntl);
        else cast_kernel<S, D, V, false><<<g, kBlock, 0, st>>>((const S *)a, (D *)c, n, ntl);
    } else {
        unsigned g = stream_grid(n, (int64_t)kBlock * cast_unroll<S, D>, kBlocksPerCUC);
        cast_kernel<S, D, 1, false><<<g, kBlock, 0, st>>>((const S *)a, (D *)c, n, ntl);
    }
    return launch_status();
}
template <typename S> int cast_from(const void *a, int dst, void *c, int64_t n, hipStream_t st) {
    switch (dst) {
    case DXH_F64: return launch_cast<S, double>(a, c, n, st);
    case DXH_F32: return launch_cast<S, float>(a, c, n, st);
    case DXH_F16: return launch_cast<S, f16_t>(a, c, n, st);
    case DXH_BF16: return launch_cast<S, bf16_t>(a, c, n, st);
    case DXH_I64: return launch_cast<S, int64_t>(a, c, n, st);
    case DXH_I32: return launch_cast<S, int32_t>(a, c, n, st);
    case DXH_I16: return launch_cast<S, int16_t>(a, c, n, st);
    case DXH_I8: return launch_cast<S, int8_t>(a, c, n, st);
    default: return DXH_ERR_DTYPE;
    }
}

}  // namespace dxh

using namespace dxh;

extern "C" {

static const dxh_scalar kNoScalar = {0.0, 0};

int dxh_equal(int dtype, const void *a, const void *b, float eps, void *m, int64_t n, void *stream) { return compare_all<CMP_EQ, false>(dtype, a, b, kNoScalar, eps, m, n, stream); }
int dxh_notequal(int dtype, const void *a, const void *b, float eps, void *m, int64_t n, void *stream) { return compare_all<CMP_NE, false>(dtype, a, b, kNoScalar, eps, m, n, stream); }
int dxh_equalscalar(int dtype, const void *a, dxh_scalar s, float eps, void *m, int64_t n, void *stream) { return compare_all<CMP_EQ, true>(dtype, a, nullptr, s, eps, m, n, stream); }
int dxh_notequalscalar(int dtype, const void *a, dxh_scalar s, float eps, void *m, int64_t n, void *stream) { return compare_all<CMP_NE, true>(dtype, a, nullptr, s, eps, m, n, stream); }
int dxh_less(int dtype, const void *a, const void *b, void *m, int64_t n, void *stream) { return compare_all<CMP_LT, false>(dtype, a, b, kNoScalar, 0.f, m, n, stream); }
int dxh_greater(int dtype, const void *a, const void *b, void *m, int64_t n, void *stream) { return compare_all<CMP_GT, false>(dtype, a, b, kNoScalar, 0.f, m, n, stream); }
int dxh_lessscalar(int dtype, const void *a, dxh_scalar s, void *m, int64_t n, void *stream) { return compare_all<CMP_LT, true>(dtype, a, nullptr, s, 0.f, m, n, stream); }
int dxh_greaterscalar(int dtype, const void *a, dxh_scalar s, void *m, int64_t n, void *stream) { return compare_all<CMP_GT, true>(dtype, a, nullptr, s, 0.f, m, n, stream); }

int dxh_switch(int dtype, const void *const *tensors, int ntensors, int cases_dtype, const void *cases, void *c,
               int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(tensors); DXH_CHECK_PTR(cases); DXH_CHECK_PTR(c);
    if (ntensors < 1 || ntensors > DXH_SWITCH_MAX) return DXH_ERR_ARG;
    hipStream_t st = as_stream(stream);
    switch (dtype_size(dtype)) {
    case 8: return launch_switch<uint64_t>(tensors, ntensors, cases_dtype, cases, c, n, st);
    case 4: return launch_switch<uint32_t>(tensors, ntensors, cases_dtype, cases, c, n, st);
    case 2: return launch_switch<uint16_t>(tensors, ntensors, cases_dtype, cases, c, n, st);
    case 1: return launch_switch<uint8_t>(tensors, ntensors, cases_dtype, cases, c, n, st);
    default: return DXH_ERR_DTYPE;
    }
}

int dxh_todtype(int src, const void *a, int dst, void *c, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(c);
    hipStream_t st = as_stream(stream);
    if (src == dst) {
        int es = dtype_size(src);
        if (!es) return DXH_ERR_DTYPE;
        if (a == c) return DXH_OK;
        return (int)hipMemcpyAsync(c, a, (size_t)n * es, hipMemcpyDeviceToDevice, st);
    }
    switch (src) {
    case DXH_F64: return cast_from<double>(a, dst, c, n, st);
    case DXH_F32: return cast_from<float>(a, dst, c, n, st);
    case DXH_F16: return cast_from<f16_t>(a, dst, c, n, st);
    case DXH_BF16: return cast_from<bf16_t>(a, dst, c, n, st);
    case DXH_I64: return cast_from<int64_t>(a, dst, c, n, st);
    case DXH_I32: return cast_from<int32_t>(a, dst, c, n, st);
    case DXH_I16: return cast_from<int16_t>(a, dst, c, n, st);
    case DXH_I8: return cast_from<int8_t>(a, dst, c, n, st);
    default: return DXH_ERR_DTYPE;
    }
}

}  // extern "C"
