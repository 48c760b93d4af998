// elementwise_ops.hpp — the arithmetic of the elementwise ops, one functor per op on the accumulate
// type (fp32 for 16-bit floats).  Shared by the streaming kernels (elementwise.hip), the runs of ops
// that go out as one launch (interpreted there, compiled in chain_static.hip) and the matmul
// epilogue: calling the same functor is what makes a fused result the bits of the separate launch.
// Arithmetic follows executor/op-ompsimd's tensorfunc/elementwise_miaobyte.hpp (cited per op in
// include/dxhip.h).
#pragma once
#include "common.hpp"

namespace dxh {

// ---- op functors on the accumulate type -----------------------------------------------
template <typename A> __device__ inline A wrap_add(A a, A b) { using U = std::make_unsigned_t<A>; return A(U(U(a) + U(b))); }
template <typename A> __device__ inline A wrap_sub(A a, A b) { using U = std::make_unsigned_t<A>; return A(U(U(a) - U(b))); }
template <typename A> __device__ inline A wrap_mul(A a, A b) {
    using U = std::conditional_t<(sizeof(A) < 4), uint32_t, std::make_unsigned_t<A>>;
    return A(U(U(a) * U(b)));
}
template <typename A> __device__ inline A wrap_div(A a, A b) {
    if (b == 0) return A(0);
    if (b == A(-1)) return wrap_sub<A>(A(0), a);
    return A(a / b);
}

struct OpAdd { template <typename A> __device__ static A f(A a, A b) { if constexpr (std::is_integral_v<A>) return wrap_add(a, b); else return a + b; } };
struct OpSub { template <typename A> __device__ static A f(A a, A b) { if constexpr (std::is_integral_v<A>) return wrap_sub(a, b); else return a - b; } };
struct OpRSub { template <typename A> __device__ static A f(A a, A b) { return OpSub::f(b, a); } };
struct OpMul { template <typename A> __device__ static A f(A a, A b) { if constexpr (std::is_integral_v<A>) return wrap_mul(a, b); else return a * b; } };
struct OpDiv { template <typename A> __device__ static A f(A a, A b) { if constexpr (std::is_integral_v<A>) return wrap_div(a, b); else return a / b; } };
struct OpRDiv { template <typename A> __device__ static A f(A a, A b) { return OpDiv::f(b, a); } };
// std::max / std::min of the reference: (a<b)?b:a and (b<a)?b:a
struct OpMax { template <typename A> __device__ static A f(A a, A b) { return (a < b) ? b : a; } };
struct OpMin { template <typename A> __device__ static A f(A a, A b) { return (b < a) ? b : a; } };
struct OpPow {
    __device__ static float f(float a, float b) { return powf(a, b); }
    __device__ static double f(double a, double b) { return pow(a, b); }
};
struct OpRPow { template <typename A> __device__ static A f(A a, A b) { return OpPow::f(b, a); } };
// pow(x, 2): the correctly rounded value is x*x (one rounding), including signed zeros, infinities and NaN
struct OpSquare { template <typename A> __device__ static A f(A a) { return a * a; } };

struct OpSqrt { __device__ static float f(float a) { return sqrtf(a); } __device__ static double f(double a) { return sqrt(a); } };
struct OpExp { __device__ static float f(float a) { return expf(a); } __device__ static double f(double a) { return exp(a); } };
struct OpLog { __device__ static float f(float a) { return logf(a); } __device__ static double f(double a) { return log(a); } };
struct OpSin { __device__ static float f(float a) { return sinf(a); } __device__ static double f(double a) { return sin(a); } };
struct OpCos { __device__ static float f(float a) { return cosf(a); } __device__ static double f(double a) { return cos(a); } };
struct OpTan { __device__ static float f(float a) { return tanf(a); } __device__ static double f(double a) { return tan(a); } };
struct OpInvert {
    template <typename A> __device__ static A f(A a) {
        if constexpr (std::is_same_v<A, bool_t>) return bool_t{uint8_t(a.v ? 0 : 1)};
        else return A(~a);
    }
};

// exp whose result is stored as a 16-bit float: 2^(a log2 e) on the hardware's exp2.  The product is rounded
// once (|a log2 e| < 150 in the finite range, so 2^-17 absolute) and v_exp_f32 is good to an ulp of fp32: the
// result is within 2^-17 of exp(a) relative, against half an ulp of 2^-9 (bf16) or 2^-12 (f16) for the one
// rounding that follows — a 16-bit result differs from the correctly rounded one in under 1 % (bf16) / 4 % (f16)
// of the cases, by one unit in the last place, at a third of the instructions of the fp32 expansion.  v_exp_f32
// flushes results under 2^-126; those are reached through a scaled second step, so denormal 16-bit results
// (bf16 has fp32's exponent range) come out as such.
__device__ __forceinline__ float exp_to_half(float a) {
    const float t = a * 1.44269504088896340736f;
    const bool tiny = t < -126.0f;
    const float r = __builtin_amdgcn_exp2f(tiny ? t + 64.0f : t);
    return tiny ? r * 0x1p-64f : r;
}
// f(a) of a unary op on a tensor of storage type T (the accumulate type's functor, but for the 16-bit exp)
template <typename Op, typename T> __device__ __forceinline__ acc_t<T> unary_apply(acc_t<T> a) {
    if constexpr (std::is_same_v<Op, OpExp> && (std::is_same_v<T, bf16_t> || std::is_same_v<T, f16_t>)) return exp_to_half(a);
    else return Op::f(a);
}

// the float ops of a run by their dxh_chain_code: y = f(a, b) for the two-tensor forms, f(a, s) for the
// scalar forms, f(a) for the unary ones (DXH_CHAIN_COPY: a itself; row reductions are not elementwise)
// HALF: the op's result is a 16-bit float
template <int CODE, bool HALF> __device__ __forceinline__ float chain_apply(float a, float b, float s) {
    if constexpr (CODE == DXH_CHAIN_ADD) return OpAdd::f(a, b);
    else if constexpr (CODE == DXH_CHAIN_SUB) return OpSub::f(a, b);
    else if constexpr (CODE == DXH_CHAIN_MUL) return OpMul::f(a, b);
    else if constexpr (CODE == DXH_CHAIN_DIV) return OpDiv::f(a, b);
    else if constexpr (CODE == DXH_CHAIN_MAX) return OpMax::f(a, b);
    else if constexpr (CODE == DXH_CHAIN_MIN) return OpMin::f(a, b);
    else if constexpr (CODE == DXH_CHAIN_ADDSCALAR) return OpAdd::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_SUBSCALAR) return OpSub::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_RSUBSCALAR) return OpRSub::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_MULSCALAR) return OpMul::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_DIVSCALAR) return OpDiv::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_RDIVSCALAR) return OpRDiv::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_MAXSCALAR) return OpMax::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_MINSCALAR) return OpMin::f(a, s);
    else if constexpr (CODE == DXH_CHAIN_SQRT) return OpSqrt::f(a);
    else if constexpr (CODE == DXH_CHAIN_EXP) return HALF ? exp_to_half(a) : OpExp::f(a);
    else if constexpr (CODE == DXH_CHAIN_LOG) return OpLog::f(a);
    else if constexpr (CODE == DXH_CHAIN_SQUARE) return OpSquare::f(a);
    else return a;
}

}  // namespace dxh
