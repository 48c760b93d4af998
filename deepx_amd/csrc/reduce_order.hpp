// reduce_order.hpp — the accumulate type, the combining step and the order in which the lanes of a
// row stage fold a row (reduce.hip).  Shared with the kernel that computes a row sum in the middle
// of a run of elementwise ops (elementwise.hip): calling the same code is what makes its sums the
// bits of dxh_sum.
#pragma once
#include "common.hpp"
#include <limits>

namespace dxh {

enum RedKind { R_SUM = 0, R_PROD = 1, R_MAX = 2, R_MIN = 3 };

template <typename T> struct racc_of { using type = T; };
template <> struct racc_of<bf16_t> { using type = float; };
template <> struct racc_of<f16_t> { using type = float; };
template <> struct racc_of<int16_t> { using type = int32_t; };
template <> struct racc_of<int8_t> { using type = int32_t; };
template <typename T> using racc_t = typename racc_of<T>::type;

template <typename A, typename T> __device__ inline A rload(T x) {
    if constexpr (std::is_same_v<T, bf16_t> || std::is_same_v<T, f16_t>) return load_acc(x);
    else return A(x);
}
template <typename T, typename A> __device__ inline T rstore(A v) {
    if constexpr (std::is_same_v<T, bf16_t>) return to_bf16(v);
    else if constexpr (std::is_same_v<T, f16_t>) return to_f16(v);
    else return T(v);  // integers truncate: wrap-around arithmetic is width independent
}

// identity element: 0 / 1 / lowest() / max() of the STORAGE type, as the reference
// pre-fills the result (reduce_miaobyte.hpp:24,101,191,274)
template <int K, typename A, typename TS> __host__ __device__ inline A rinit() {
    if constexpr (K == R_SUM) return A(0);
    else if constexpr (K == R_PROD) return A(1);
    else if constexpr (std::is_same_v<TS, bf16_t>) return K == R_MAX ? -3.3895313892515355e38f : 3.3895313892515355e38f;
    else if constexpr (std::is_same_v<TS, f16_t>) return K == R_MAX ? -65504.0f : 65504.0f;
    else return K == R_MAX ? A(std::numeric_limits<TS>::lowest()) : A(std::numeric_limits<TS>::max());
}
template <int K, typename A> __device__ inline A rop(A a, A b) {
    if constexpr (K == R_SUM) {
        if constexpr (std::is_integral_v<A>) { using U = std::make_unsigned_t<A>; return A(U(a) + U(b)); }
        else return a + b;
    } else if constexpr (K == R_PROD) {
        if constexpr (std::is_integral_v<A>) { using U = std::make_unsigned_t<A>; return A(U(a) * U(b)); }
        else return a * b;
    } else if constexpr (K == R_MAX) return (a < b) ? b : a;
    else return (b < a) ? b : a;
}

template <typename A> __device__ inline A shfl_xor_any(A v, int off) {
    if constexpr (sizeof(A) == 8) {
        uint64_t u = __builtin_bit_cast(uint64_t, v);
        uint32_t lo = __shfl_xor((int)(uint32_t)u, off, kWave);
        uint32_t hi = __shfl_xor((int)(uint32_t)(u >> 32), off, kWave);
        return __builtin_bit_cast(A, (uint64_t(hi) << 32) | lo);
    } else {
        return __builtin_bit_cast(A, __shfl_xor(__builtin_bit_cast(int, v), off, kWave));
    }
}

// What one lane of a G-lane group folds of a row of `lv` vectors: vectors lane, lane + G, ... in
// batches of 8 (a balanced tree per batch), then 4, then one by one, per vector component.
// `ld(i)` returns vector i of the row.
template <int K, typename A, int V, typename Load>
__device__ __forceinline__ void row_lane_fold(A (&acc)[V], int64_t lane, int64_t G, int64_t lv, Load ld) {
    int64_t i = lane;
    for (; i + 7 * G < lv; i += 8 * G) {
        decltype(ld(i)) x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) x[u] = ld(i + u * G);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            A t0 = rop<K, A>(rop<K, A>(rload<A>(x[0].v[k]), rload<A>(x[1].v[k])), rop<K, A>(rload<A>(x[2].v[k]), rload<A>(x[3].v[k])));
            A t1 = rop<K, A>(rop<K, A>(rload<A>(x[4].v[k]), rload<A>(x[5].v[k])), rop<K, A>(rload<A>(x[6].v[k]), rload<A>(x[7].v[k])));
            acc[k] = rop<K, A>(acc[k], rop<K, A>(t0, t1));
        }
    }
    for (; i + 3 * G < lv; i += 4 * G) {
        auto x0 = ld(i), x1 = ld(i + G), x2 = ld(i + 2 * G), x3 = ld(i + 3 * G);
#pragma unroll
        for (int k = 0; k < V; ++k) {
            A t0 = rop<K, A>(rload<A>(x0.v[k]), rload<A>(x1.v[k]));
            A t1 = rop<K, A>(rload<A>(x2.v[k]), rload<A>(x3.v[k]));
            acc[k] = rop<K, A>(acc[k], rop<K, A>(t0, t1));
        }
    }
    for (; i < lv; i += G) {
        auto x = ld(i);
#pragma unroll
        for (int k = 0; k < V; ++k) acc[k] = rop<K, A>(acc[k], rload<A>(x.v[k]));
    }
}
// The lane's V accumulators into one value, then across the lanes of the group (adjacent lanes of
// one wave, G a power of two up to 64): every lane ends up with the group's result.
template <int K, typename A, int V>
__device__ __forceinline__ A row_group_fold(const A (&acc)[V], int G) {
    A v = acc[0];
#pragma unroll
    for (int k = 1; k < V; ++k) v = rop<K, A>(v, acc[k]);
    const int gw = G < kWave ? G : kWave;
    for (int off = gw >> 1; off > 0; off >>= 1) v = rop<K, A>(v, shfl_xor_any<A>(v, off));
    return v;
}

// Lanes per row of the single row stage that dxh_sum runs on a 16-byte aligned fp32 [rows, cols]
// tensor over its last axis, or 0 when the plan is anything else (several stages, a split row, the
// whole workgroup on one row).
int sum_rows_group_f32(int64_t rows, int64_t cols);
// The same for sum / prod / reducemax / reducemin over the last axis of a 16-byte aligned [rows, cols]
// tensor of fp32 (esize 4) or 16-bit floats (esize 2, accumulated in fp32): all four take one plan.
int reduce_rows_group(int esize, int64_t rows, int64_t cols);

}  // namespace dxh
