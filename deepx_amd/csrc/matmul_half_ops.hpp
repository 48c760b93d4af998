// matmul_half_ops.hpp — device helpers shared by the bf16 / f16 matrix-pipe kernels
// (matmul_half.hip, matmul_half_dma.hip): the MFMA wrapper, packed conversion of results and the
// transposing LDS read.
#pragma once
#include "matmul_common.hpp"

namespace dxh {

template <typename T, typename V> __device__ inline f32x16 mfma32(V a, V b, f32x16 c) {
    if constexpr (std::is_same_v<T, bf16_t>)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
// two fp32 accumulators -> one dword of two bf16/f16, round to nearest even (v_cvt_pk_bf16_f32 /
// v_cvt_pk_f16_f32); element a in the low half
template <typename T> __device__ __forceinline__ uint32_t pack2(float a, float b) {
    if constexpr (std::is_same_v<T, bf16_t>) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
    else return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, f16x2));
}
// Within each group of 16 lanes, lane i passes the address of 4 consecutive 16-bit elements
// ("row i") and receives element i%4 of rows i/4, 4 + i/4, 8 + i/4, 12 + i/4.
__device__ __forceinline__ u32x2 lds_read_tr16(const uint16_t *p) {
    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *)p);
    return __builtin_bit_cast(u32x2, v);
}

}  // namespace dxh
