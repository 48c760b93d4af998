// common.hpp — shared device/host helpers of libdxhip (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "../../include/dxhip.h"

namespace dxh {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr int kBlock = 256;        // 4 waves per workgroup: one per SIMD of a CU
constexpr int kCUs = 256;          // MI355X: 8 XCDs x 32 CUs
constexpr int kVecBytes = 16;      // one global_load_dwordx4 per lane

// ---- storage types ---------------------------------------------------------------------
// 16-bit floats are carried as raw bits; arithmetic happens in fp32 and is rounded once
// (RNE) on store.
struct bf16_t { uint16_t bits; };
struct f16_t { uint16_t bits; };
struct bool_t { uint8_t v; };

template <typename T> struct acc_of { using type = T; };
template <> struct acc_of<bf16_t> { using type = float; };
template <> struct acc_of<f16_t> { using type = float; };
template <typename T> using acc_t = typename acc_of<T>::type;

__host__ __device__ inline float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__host__ __device__ inline uint32_t float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

__host__ __device__ inline float load_acc(bf16_t x) { return bits_to_float(uint32_t(x.bits) << 16); }
__host__ __device__ inline float load_acc(f16_t x) { return float(__builtin_bit_cast(_Float16, x.bits)); }
template <typename T> __host__ __device__ inline T load_acc(T x) { return x; }

// fp32 -> bf16, round to nearest even, NaN kept quiet.  The device has an instruction for it
// (v_cvt_pk_bf16_f32, two values at a time) whose result equals the arithmetic below for every one of
// the 2^32 inputs, NaN payloads included (checked exhaustively on the GPU); the host computes it.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__host__ __device__ inline bf16_t to_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return bf16_t{uint16_t(__builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{f, f}, bf16x2_t)))};
#else
    uint32_t u = float_to_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return bf16_t{uint16_t((u >> 16) | 0x0040u)};
    u += 0x7fffu + ((u >> 16) & 1u);
    return bf16_t{uint16_t(u >> 16)};
#endif
}
__host__ __device__ inline f16_t to_f16(float f) {
    return f16_t{__builtin_bit_cast(uint16_t, (_Float16)f)};  // v_cvt_f16_f32, RNE
}
template <typename T> __host__ __device__ inline T store_acc(acc_t<T> v) {
    if constexpr (std::is_same_v<T, bf16_t>) return to_bf16(v);
    else if constexpr (std::is_same_v<T, f16_t>) return to_f16(v);
    else return v;
}

// V results of an op -> one vector of the storage type.  16-bit floats are converted two at a time
// (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32, both round to nearest even): one instruction per dword of
// the vector instead of a conversion and a merge per element.
template <typename T, int V> struct alignas(sizeof(T) * V) vec_t;
template <typename T, int V> __device__ __forceinline__ void store_acc_vec(vec_t<T, V> &r, const acc_t<T> (&x)[V]);

// scalar operand -> storage type, mirroring T(std::stof(text)) upstream of the ABI
template <typename T> inline T scalar_to(const dxh_scalar &s) {
    if constexpr (std::is_same_v<T, bf16_t>) return to_bf16(float(s.f));
    else if constexpr (std::is_same_v<T, f16_t>) return to_f16(float(s.f));
    else if constexpr (std::is_floating_point_v<T>) return T(s.f);
    else return T(s.i);
}

// ---- 16-byte vectors -------------------------------------------------------------------
template <typename T, int N> struct alignas(sizeof(T) * N) vec_t { T v[N]; };
template <typename T, int V> __device__ __forceinline__ void store_acc_vec(vec_t<T, V> &r, const acc_t<T> (&x)[V]) {
    if constexpr ((std::is_same_v<T, bf16_t> || std::is_same_v<T, f16_t>) && V % 2 == 0) {
        uint32_t *w = reinterpret_cast<uint32_t *>(r.v);
#pragma unroll
        for (int k = 0; k < V / 2; ++k) {
            if constexpr (std::is_same_v<T, bf16_t>) w[k] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{x[2 * k], x[2 * k + 1]}, bf16x2_t));
            else w[k] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{x[2 * k], x[2 * k + 1]}, f16x2_t));
        }
    } else {
#pragma unroll
        for (int k = 0; k < V; ++k) r.v[k] = store_acc<T>(x[k]);
    }
}
template <typename T> constexpr int vec_len = kVecBytes / (int)sizeof(T);

template <int BYTES> struct raw_of;
template <> struct raw_of<1> { using type = uint8_t; };
template <> struct raw_of<2> { using type = uint16_t; };
template <> struct raw_of<4> { using type = uint32_t; };
template <> struct raw_of<8> { using type = uint64_t; };
template <> struct raw_of<16> { using type = uint4; };

// ---- streaming (non-temporal) global access ------------------------------------------------
// Every tensor of an elementwise / changeshape / reduce op is touched exactly once.  The `nt`
// hint lifted a streaming add from ~5.0 to ~6.5 TB/s on MI355X; which loads and stores carry it
// (or one of the scope bits) is decided per launch: nt_load_*, stream_policy_2r1w, st_mode below.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
template <int BYTES> struct nt_raw;
template <> struct nt_raw<1> { using type = uint8_t; };
template <> struct nt_raw<2> { using type = uint16_t; };
template <> struct nt_raw<4> { using type = uint32_t; };
template <> struct nt_raw<8> { using type = uint64_t; };
template <> struct nt_raw<16> { using type = u32x4_t; };
template <typename VT> __device__ inline VT ld_nt(const VT *p) {
    using R = typename nt_raw<sizeof(VT)>::type;
    return __builtin_bit_cast(VT, __builtin_nontemporal_load(reinterpret_cast<const R *>(p)));
}
template <typename VT> __device__ inline void st_nt(VT *p, const VT &v) {
    using R = typename nt_raw<sizeof(VT)>::type;
    __builtin_nontemporal_store(__builtin_bit_cast(R, v), reinterpret_cast<R *>(p));
}

// Store policy of a streaming kernel: 0 plain, 1 nt, 2 write-through at system scope (sc0 sc1; 4-, 8- and
// 16-byte stores), 3 nt at agent scope (sc1 nt; 16-byte stores only); widths a mode does not have fall back to
// nt.  2 is the fastest partner of nt loads when two tensors are read per tensor written (see
// stream_policy_2r1w); 3 is the fastest for write-dominated streams (fp32 broadcast of a row,
// GB/s at 64 / 128 / 256 MiB: nt 5997 / 6453 / 6798, sc1 nt 6163 / 6811 / 7308; bf16 transpose
// +4 %, concat +2 %).
template <int ST, typename VT> __device__ inline void st_mode(VT *p, const VT &v) {
    if constexpr (ST == 0) {
        *p = v;
    } else if constexpr (ST == 2 && sizeof(VT) == 16) {
        const u32x4_t r = __builtin_bit_cast(u32x4_t, v);
        // s_nop: a VALU write to the data registers of a 16-byte store needs a wait state after the
        // store, which the compiler inserts for its own stores but not behind inline assembly
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(r) : "memory");
    } else if constexpr (ST == 2 && sizeof(VT) == 8) {
        const uint64_t r = __builtin_bit_cast(uint64_t, v);
        asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(r) : "memory");
    } else if constexpr (ST == 2 && sizeof(VT) == 4) {
        const uint32_t r = __builtin_bit_cast(uint32_t, v);
        asm volatile("global_store_dword %0, %1, off sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(r) : "memory");
    } else if constexpr (ST == 3 && sizeof(VT) == 16) {
        const u32x4_t r = __builtin_bit_cast(u32x4_t, v);
        asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(r) : "memory");
    } else {
        st_nt(p, v);
    }
}
// store of a write-dominated stream (transposes, broadcasts, gathers, concat): write-through when the launch's output
// is small enough for the next kernel to find it in the last-level cache (!use_nt_store), else nt at agent scope
template <typename VT> __device__ inline void st_stream(VT *p, const VT &v, int through) {
    if (through) st_mode<2>(p, v); else st_mode<3>(p, v);
}
template <bool NTL, typename VT> __device__ inline VT ld_sel(const VT *p) {
    if constexpr (NTL) return ld_nt(p);
    else return *p;
}

// Stores carry the nt hint too.  A/B runs in one process on random data (the knob below): 64 MiB
// add 6.28 vs 6.10 TB/s, bf16 broadcast 5.9 vs 4.9 TB/s in favour of nt, at every size tried.
struct Tuning {
    int64_t nt_store_bytes = (int64_t)32 << 20;   // DXH_TUNE_NT_STORE_BYTES: a launch that stores more than this uses non-temporal stores
    int64_t reduce_target_blocks = 4 * 256;       // DXH_TUNE_REDUCE_TARGET_BLOCKS
    int64_t reduce_col_target_blocks = 256;       // strided-axis stages: about one workgroup per CU, each
                                                  // walking its rows with software-pipelined loads
    int64_t reduce_col_min_rows = 16;             // DXH_TUNE_REDUCE_COL_MIN_ROWS
    int64_t reduce_col_max_lanes = 128;           // DXH_TUNE_REDUCE_COL_MAX_LANES
    int64_t reduce_row_loads = 4;                 // DXH_TUNE_REDUCE_ROW_LOADS: vectors per lane a row group aims for
    int64_t matmul_tile = 0;                      // DXH_TUNE_MATMUL_TILE: 0 = chosen per shape
    int64_t matmul_splitk = 0;                    // DXH_TUNE_MATMUL_SPLITK: 0 = chosen per shape, 1 = never, n = n slices
    int64_t nt_load = 0;                          // DXH_TUNE_NT_LOAD: 0 = by op class and size, 1 = always, 2 = never
    int64_t skinny_per_cu = 1;                    // DXH_TUNE_SKINNY_PER_CU
    int64_t skinny_min_rows = 256;                // DXH_TUNE_SKINNY_MIN_ROWS
    int64_t skinny_half = 0;                      // DXH_TUNE_SKINNY_HALF
    int64_t reduce_fused_finish = 1;              // DXH_TUNE_REDUCE_FUSED_FINISH
    int64_t chain_static = 1;                     // DXH_TUNE_CHAIN_STATIC
};
Tuning &tuning();  // runtime.hip

inline bool stream_is_capturing(hipStream_t st) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cap) != hipSuccess) { (void)hipGetLastError(); return true; }  // unknown: assume the worst
    return cap != hipStreamCaptureStatusNone;
}
void reduce_stream_release(hipStream_t st);  // reduce.hip: gives back the stream's slice of finish counters
// reduce.hip: counters that launches recorded under capture took belong to the graph the capture ends in
// (nullptr: the capture failed) and return to the pool with it
void finish_capture_ended(hipStream_t st, const void *graph);
void finish_graph_destroyed(const void *graph);
void finish_capture_stats(int64_t *in_use, int64_t *capacity);
void reduce_device_init();  // reduce.hip: resolves the file-scope device arrays of the current device
void chain_device_init();   // elementwise.hip: raises the dynamic-LDS limit of the row-form chain kernels on the current device

// Whether the loads of a streaming kernel carry the nt hint.  Measured on MI355X with buffers
// rotated through 768 MB (fp32, GB/s with nt / without):
//   one read per write (scalar, unary)   16 MiB 4671/5528   64 MiB 5907/6657   128 MiB 6238/6898   256 MiB 6340/5905
//   two reads per write (binary)          4 MiB 2783/3209   16 MiB 5339/5174    64 MiB 6368/5878   256 MiB 6499/5832
//   read only (row reduction)            16 MiB 3263/3460   64 MiB 5751/5937   128 MiB 6577/6655   256 MiB 6834/5991
// i.e. plain loads win while the tensors of one launch fit the 256 MiB last-level cache, except
// for read-dominated streams of more than a few MiB.
inline bool nt_load_forced(bool by_rule) {
    const int64_t knob = tuning().nt_load;
    return knob == 1 ? true : knob == 2 ? false : by_rule;
}
inline bool nt_load_1r1w(size_t in_bytes, size_t out_bytes) { return nt_load_forced(in_bytes + out_bytes > ((size_t)256 << 20)); }
inline bool nt_load_2r1w(size_t total_bytes) { return nt_load_forced(total_bytes > ((size_t)24 << 20)); }
// Two reads per write, loads and stores together (fp32 add, GB/s, MiB per tensor):
//   loads nt, stores nt       32: 5869   64: 6367   128: 6593   256: 6451
//   loads nt, stores sc0 sc1  32: 6197   64: 6758   128: 7138   256: 6264
// 0 = plain loads + nt stores, 1 = nt loads + nt stores, 2 = nt loads + sc0 sc1 stores
inline int stream_policy_2r1w(size_t total_bytes) {
    if (!nt_load_2r1w(total_bytes)) return 0;
    return total_bytes <= ((size_t)512 << 20) ? 2 : 1;
}
inline bool nt_load_reduce(size_t in_bytes) { return nt_load_forced(in_bytes > ((size_t)128 << 20)); }
// Strided-axis stage: its rows are a pitch apart, and nt loads won at every size tried (fp32 [R,8192],
// nt / plain GB/s: 32 MiB 3174/3067, 128 MiB 5520/5270, 256 MiB 6190/5894; bf16 [8192,8192] 4574/2964,
// bf16 [64,512,2048] axis 1 5794/3239) except within noise at 7 MiB.
inline bool nt_load_reduce_col(size_t in_bytes) { return nt_load_forced(in_bytes >= ((size_t)8 << 20)); }
// Stores of the elementwise kernels, the fused runs and the 16-bit products: non-temporal for a launch that
// stores more than 32 MiB (a pure stream: measured fastest on buffers rotated past the last-level cache),
// write-through (sc0 sc1) below.  A deepx program reads an op's result in one of its next instructions, and a
// tensor of activation size that went out with write-through stores is in the 256 MiB last-level cache then
// without having filled the L2s with dirty lines.  The SiLU gate of config 5 (19.9 MB out) on its own / the whole
// block (RMSNorm, three products, gate) as four launches, same process: nt 12.0 / 90 us, plain 12.7-13.1 / 85.5,
// sc0 sc1 11.5 / 84; with the products' C written through as well 79-81 us.  Non-temporal stores at agent scope
// (sc1 nt) are the fastest for the producer alone (11.4) and leave nothing for the consumer (90).
inline bool use_nt_store(size_t out_bytes) { return (int64_t)out_bytes > tuning().nt_store_bytes; }
template <bool NT, typename VT> __device__ inline void st_sel(VT *p, const VT &v) {
    if constexpr (NT) st_nt(p, v); else st_mode<2>(p, v);
}

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

inline int dtype_size(int dtype) {
    switch (dtype) {
    case DXH_F64: case DXH_I64: return 8;
    case DXH_F32: case DXH_I32: return 4;
    case DXH_F16: case DXH_BF16: case DXH_I16: return 2;
    case DXH_I8: case DXH_BOOL: return 1;
    default: return 0;
    }
}

// ---- division by a run-time constant without a divide ----------------------------------------
// q = n / d for any 32-bit n, d >= 1: one v_mul_hi_u32, a subtract, two shifts, an add (round-up
// method with a 33-bit magic number).  Index decompositions in the changeshape kernels divide by
// shape extents several times per 16-byte unit; a hardware-free divide costs ~25 instructions each.
struct FastDiv { uint32_t d, magic, shift; };
inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f{d, 0, 0};
    if (d <= 1) return f;
    uint32_t L = 0;
    while ((1ull << L) < d) ++L;  // ceil(log2 d)
    f.magic = (uint32_t)(((1ull << 32) * ((1ull << L) - d)) / d + 1);
    f.shift = L - 1;
    return f;
}
__host__ __device__ inline uint32_t fast_div(uint32_t n, const FastDiv &f) {
    if (f.d <= 1) return n;
#if defined(__HIP_DEVICE_COMPILE__)
    uint32_t t = __umulhi(n, f.magic);
#else
    uint32_t t = (uint32_t)(((uint64_t)n * f.magic) >> 32);
#endif
    return (t + ((n - t) >> 1)) >> f.shift;
}

// ---- launch helpers --------------------------------------------------------------------
inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// Number of workgroups for a streaming kernel whose workgroup consumes `per_block` work
// items per loop trip: enough to cover the work, capped at `waves_per_cu` resident
// workgroups per CU so the grid-stride loop keeps every CU's queues full.
inline unsigned stream_grid(int64_t items, int64_t per_block, int blocks_per_cu) {
    int64_t need = (items + per_block - 1) / per_block;
    // blocks_per_cu == 0: one tile per workgroup, no grid-stride trips (the fastest shape measured
    // for pure streaming: the hardware dispatcher balances CUs better than a fixed-stride loop)
    int64_t cap = blocks_per_cu > 0 ? (int64_t)kCUs * blocks_per_cu : ((int64_t)1 << 30);
    if (need < 1) need = 1;
    return (unsigned)(need < cap ? need : cap);
}

inline int launch_status() {
    hipError_t e = hipGetLastError();
    return (int)e;
}

#define DXH_CHECK_N(n) do { if ((n) < 0) return DXH_ERR_ARG; if ((n) == 0) return DXH_OK; } while (0)
#define DXH_CHECK_PTR(p) do { if (!(p)) return DXH_ERR_ARG; } while (0)

}  // namespace dxh
