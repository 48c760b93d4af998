// matmul_common.hpp — pieces shared by the matrix-pipe GEMM kernels: vector typedefs, compile-time
// loops, the XCD-aware workgroup -> tile map and the launch-side helpers.
#pragma once
#include <utility>
#include "common.hpp"

namespace dxh {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // native vector: arrays of it stay in registers
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F> __device__ __forceinline__ void static_for(F f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }
template <int V> using ic = std::integral_constant<int, V>;


// ---- XCD-aware workgroup -> tile map (shared by the MFMA kernels) ---------------------------
// Workgroups are dealt round-robin to the 8 XCDs, each with a private L2.  XCD x takes the
// contiguous range [x*chunk, (x+1)*chunk) of a grouped tile order (group_m tile rows at a time,
// column-major inside a group), i.e. a compact, roughly square patch of C whose A and B panels
// fit its L2.  The grid is 8*chunk workgroups; those past the last tile exit at once.
struct TileMap { int tiles_m, tiles_n, total, chunk, group_m; };
struct TileCoord { int batch, tm, tn; bool valid; };
inline bool make_tile_map(int64_t batch, int64_t m, int64_t n, int tm, int tn, TileMap &map) {
    const int64_t tiles_m = (m + tm - 1) / tm, tiles_n = (n + tn - 1) / tn, total = batch * tiles_m * tiles_n;
    if (total > 0x0fffffff) return false;
    map.tiles_m = (int)tiles_m; map.tiles_n = (int)tiles_n; map.total = (int)total;
    map.chunk = (int)((total + 7) / 8);
    int group_m = 1;  // tile rows per group: the chunk of one XCD should cover a roughly square patch of C
    while ((int64_t)(group_m + 1) * (group_m + 1) * tm <= (int64_t)map.chunk * tn && group_m + 1 <= tiles_m) ++group_m;
    map.group_m = group_m;
    return true;
}
__device__ __forceinline__ TileCoord tile_of_block(const TileMap &map) {
    TileCoord c;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    int logical = xcd * map.chunk + slot;
    c.valid = logical < map.total;
    const int per_batch = map.tiles_m * map.tiles_n;
    c.batch = logical / per_batch;
    logical -= c.batch * per_batch;
    const int in_group = map.group_m * map.tiles_n;
    const int first_m = (logical / in_group) * map.group_m;
    const int size_m = (map.tiles_m - first_m < map.group_m) ? map.tiles_m - first_m : map.group_m;
    const int within = logical % in_group;
    c.tm = first_m + within % size_m;
    c.tn = within / size_m;
    return c;
}

inline int compute_units() {
    static const int cus = [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v <= 0) {
            (void)hipGetLastError();
            v = 256;
        }
        return v;
    }();
    return cus;
}


// entry points of the per-dtype translation units (matmul_half.hip, matmul_fp.hip)
int launch_matmul_half(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st);
int launch_matmul_f32(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st);
int launch_matmul_f64(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st);

}  // namespace dxh
