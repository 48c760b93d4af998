// chain_static.hpp — runs of elementwise ops whose op list is known at compile time.
//
// dxh_chain and dxh_chain_rows walk an op table at run time (elementwise.hip): operands are picked by
// number out of LDS slots and every op goes through a switch, which costs more instructions than the
// arithmetic of a short op.  The sequences that the deepx front emits over and over (its RMSNorm, its
// SiLU gate, its softmax) are described here as types instead: a program is a list of inputs (dtype,
// extent) and a list of ops (code, operands, dtype, extent), the kernel is instantiated per program,
// every value lives in registers under a compile-time index, and only the scalars and pointers stay
// run-time arguments.  The arithmetic is the same functors (elementwise_ops.hpp), every result is
// rounded to its op's dtype before anything uses it, and a row reduction is folded in the order of
// the separate reduction kernel (reduce_order.hpp), so a compiled run stores the bits of the
// interpreted run and of the separate launches.
#pragma once
#include <tuple>
#include "matmul_common.hpp"
#include "reduce_order.hpp"
#include "elementwise_ops.hpp"

namespace dxh {

enum { kSF32 = 0, kSBF16 = 1, kSF16 = 2 };  // dtype codes of a program (those of the row-form op table)
constexpr int kNotStatic = -1003;           // not a DXH_ERR_* value: the run is none of the compiled programs

// entry points of chain_static.hip for dxh_chain / dxh_chain_rows, after they have validated a run
int static_chain_try(int dtype, const void *const *inputs, int n_inputs, const dxh_chain_op *ops, int n_ops, int64_t n, hipStream_t st);
int static_rows_try(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops, int64_t rows, int64_t cols, hipStream_t st, bool dry);
void chain_count_interpreted();

template <typename F, int... I>
inline void static_for_host_impl(F &f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F> inline void static_for_host(F f) { static_for_host_impl(f, std::make_integer_sequence<int, N>{}); }

template <int DT, int EXT> struct SIn { static constexpr int dt = DT, ext = EXT; };
// lhs / rhs: an input index, or DXH_CHAIN_RESULT + j for the result of op j (as in the C ABI); rhs is
// ignored by the scalar and unary forms
template <int CODE, int L, int R, int DT, int EXT> struct SOp { static constexpr int code = CODE, lhs = L, rhs = R, dt = DT, ext = EXT; };
template <typename... T> struct SList {
    static constexpr int size = sizeof...(T);
    template <int K> using at = std::tuple_element_t<K, std::tuple<T...>>;
};
template <typename Ins, typename Ops> struct SProg {
    using ins = Ins;
    using ops = Ops;
    static constexpr int n_in = Ins::size, n_ops = Ops::size, n_val = Ins::size + Ops::size;
    // value number of an operand reference: inputs first, then results
    static constexpr int value_of(int ref) { return ref < DXH_CHAIN_RESULT ? ref : n_in + (ref - DXH_CHAIN_RESULT); }
    template <int V> static constexpr int dt_of() {
        if constexpr (V < n_in) return Ins::template at<V>::dt; else return Ops::template at<V - n_in>::dt;
    }
    template <int V> static constexpr int ext_of() {
        if constexpr (V < n_in) return Ins::template at<V>::ext; else return Ops::template at<V - n_in>::ext;
    }
};
constexpr bool chain_code_is_binary(int code) { return code <= DXH_CHAIN_MIN; }
constexpr bool chain_code_is_rowred(int code) { return code == DXH_CHAIN_ROWSUM || code == DXH_CHAIN_ROWMAX || code == DXH_CHAIN_ROWMIN; }
constexpr int chain_dtype_bytes(int dt) { return dt == kSF32 ? 4 : 2; }

// Element size of the operands of a program's row reductions (they must agree: it fixes how the lanes
// share a row), 0 without one, -1 when they disagree.
template <typename Prog, int K = 0> constexpr int prog_reduce_esize() {
    if constexpr (K == Prog::n_ops) return 0;
    else {
        using Op = typename Prog::ops::template at<K>;
        constexpr int rest = prog_reduce_esize<Prog, K + 1>();
        if constexpr (!chain_code_is_rowred(Op::code)) return rest;
        else {
            constexpr int mine = chain_dtype_bytes(Prog::template dt_of<Prog::value_of(Op::lhs)>());
            return rest == 0 || rest == mine ? mine : -1;
        }
    }
}

// fp32 values -> their dtype's storage and back: what a store followed by a load would do
template <int DT, int N> __device__ __forceinline__ void round_in_place(float (&y)[N]) {
    if constexpr (DT == kSBF16) {
        vec_t<bf16_t, N> r;
        store_acc_vec<bf16_t, N>(r, y);
#pragma unroll
        for (int e = 0; e < N; ++e) y[e] = load_acc(r.v[e]);
    } else if constexpr (DT == kSF16) {
        vec_t<f16_t, N> r;
        store_acc_vec<f16_t, N>(r, y);
#pragma unroll
        for (int e = 0; e < N; ++e) y[e] = load_acc(r.v[e]);
    }
}
__device__ __forceinline__ float round_one(float y, int dt) {
    return dt == kSBF16 ? load_acc(to_bf16(y)) : dt == kSF16 ? load_acc(to_f16(y)) : y;
}
// N consecutive elements of dtype DT at `p` (element index `i`), as fp32 / from fp32 values that are
// already rounded to DT; accesses are 16 bytes wide where N elements are that long, else whole
template <int DT, int N> __device__ __forceinline__ void load_elems(const void *p, int64_t i, float (&y)[N]) {
    if constexpr (DT == kSF32) {
        static_assert(N % 4 == 0, "whole 16-byte pieces");
        typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
            const f4 x = reinterpret_cast<const f4 *>(reinterpret_cast<const float *>(p) + i)[q];
            y[4 * q] = x[0]; y[4 * q + 1] = x[1]; y[4 * q + 2] = x[2]; y[4 * q + 3] = x[3];
        }
    } else if constexpr (DT == kSBF16) {
        const vec_t<bf16_t, N> x = *reinterpret_cast<const vec_t<bf16_t, N> *>(reinterpret_cast<const bf16_t *>(p) + i);
#pragma unroll
        for (int e = 0; e < N; ++e) y[e] = load_acc(x.v[e]);
    } else {
        const vec_t<f16_t, N> x = *reinterpret_cast<const vec_t<f16_t, N> *>(reinterpret_cast<const f16_t *>(p) + i);
#pragma unroll
        for (int e = 0; e < N; ++e) y[e] = load_acc(x.v[e]);
    }
}
template <int DT, int N, bool NT> __device__ __forceinline__ void store_elems(void *p, int64_t i, const float (&y)[N]) {
    if constexpr (DT == kSF32) {
        typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
            const f4 x = {y[4 * q], y[4 * q + 1], y[4 * q + 2], y[4 * q + 3]};
            f4 *dst = reinterpret_cast<f4 *>(reinterpret_cast<float *>(p) + i) + q;
            if constexpr (NT) __builtin_nontemporal_store(x, dst); else *dst = x;
        }
    } else if constexpr (DT == kSBF16) {
        vec_t<bf16_t, N> r;
        store_acc_vec<bf16_t, N>(r, y);
        st_sel<NT>(reinterpret_cast<vec_t<bf16_t, N> *>(reinterpret_cast<bf16_t *>(p) + i), r);
    } else {
        vec_t<f16_t, N> r;
        store_acc_vec<f16_t, N>(r, y);
        st_sel<NT>(reinterpret_cast<vec_t<f16_t, N> *>(reinterpret_cast<f16_t *>(p) + i), r);
    }
}
// the same with the launch's store mode: non-temporal for a pure stream, write-through (sc0 sc1) for
// outputs small enough that the next kernel finds them in the last-level cache (use_nt_store)
template <int DT, int N> __device__ __forceinline__ void store_elems_sel(void *p, int64_t i, const float (&y)[N], bool nt) {
    if constexpr (DT == kSF32) {
        typedef float f4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int q = 0; q < N / 4; ++q) {
            const f4 x = {y[4 * q], y[4 * q + 1], y[4 * q + 2], y[4 * q + 3]};
            f4 *dst = reinterpret_cast<f4 *>(reinterpret_cast<float *>(p) + i) + q;
            if (nt) st_mode<1>(dst, x); else st_mode<2>(dst, x);
        }
    } else if constexpr (DT == kSBF16) {
        vec_t<bf16_t, N> r;
        store_acc_vec<bf16_t, N>(r, y);
        auto *dst = reinterpret_cast<vec_t<bf16_t, N> *>(reinterpret_cast<bf16_t *>(p) + i);
        if (nt) st_mode<1>(dst, r); else st_mode<2>(dst, r);
    } else {
        vec_t<f16_t, N> r;
        store_acc_vec<f16_t, N>(r, y);
        auto *dst = reinterpret_cast<vec_t<f16_t, N> *>(reinterpret_cast<f16_t *>(p) + i);
        if (nt) st_mode<1>(dst, r); else st_mode<2>(dst, r);
    }
}
template <int DT> __device__ __forceinline__ float load_one(const void *p, int64_t i) {
    if constexpr (DT == kSF32) return reinterpret_cast<const float *>(p)[i];
    else if constexpr (DT == kSBF16) return load_acc(reinterpret_cast<const bf16_t *>(p)[i]);
    else return load_acc(reinterpret_cast<const f16_t *>(p)[i]);
}
template <int DT> __device__ __forceinline__ void store_one(void *p, int64_t i, float y) {
    if constexpr (DT == kSF32) reinterpret_cast<float *>(p)[i] = y;
    else if constexpr (DT == kSBF16) reinterpret_cast<bf16_t *>(p)[i] = to_bf16(y);
    else reinterpret_cast<f16_t *>(p)[i] = to_f16(y);
}

// ---- one-extent programs on N elements per lane: the flat kernel and the matmul epilogue -----------
// in[j][e]: element e of input j (already fp32); res[k][e]: result of op k, rounded to dtype DT.
template <typename Prog, int DT, int N>
__device__ __forceinline__ void eval_flat(const float (&in)[Prog::n_in][N], float (&res)[Prog::n_ops][N], const float *scalar) {
    static_for<Prog::n_ops>([&](auto k_) __attribute__((always_inline)) {
        constexpr int k = decltype(k_)::value;
        using Op = typename Prog::ops::template at<k>;
        static_assert(!chain_code_is_rowred(Op::code), "no rows here");
        const float s = scalar[k];
#pragma unroll
        for (int e = 0; e < N; ++e) {
            float a, b = 0.f;
            if constexpr (Op::lhs < DXH_CHAIN_RESULT) a = in[Op::lhs][e]; else a = res[Op::lhs - DXH_CHAIN_RESULT][e];
            if constexpr (chain_code_is_binary(Op::code)) {
                if constexpr (Op::rhs < DXH_CHAIN_RESULT) b = in[Op::rhs][e]; else b = res[Op::rhs - DXH_CHAIN_RESULT][e];
            }
            res[k][e] = chain_apply<Op::code, DT != kSF32>(a, b, s);
        }
        round_in_place<DT, N>(res[k]);
    });
}

}  // namespace dxh
