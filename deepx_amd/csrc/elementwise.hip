// elementwise.hip — streaming elementwise kernels of libdxhip (gfx950).
//
// Every op here is HBM-bound: 16-byte non-temporal global loads (global_load_dwordx4 ... nt),
// four per lane and operand issued back to back, 16-byte non-temporal stores, one tile of
// 4 x 256 vectors per workgroup and as many workgroups as tiles (measured fastest on MI355X
// against grid-stride variants that loop: 6.4 TB/s vs 5.0 TB/s for a 3-stream add).  Arithmetic follows executor/op-ompsimd's
// tensorfunc/elementwise_miaobyte.hpp (cited per op in include/dxhip.h); 16-bit floats
// compute in fp32 and round once.
#include "reduce_order.hpp"
#include "elementwise_ops.hpp"
#include "chain_static.hpp"
#include <mutex>

namespace dxh {

constexpr int kUnroll = 4;       // vectors in flight per lane and operand (3-stream add: 6.42 TB/s against 6.25 with 1)
constexpr int kBlocksPerCU = 0;  // 0 = one tile per workgroup (see stream_grid)

// ---- tile loop --------------------------------------------------------------------------
// Calls body(vector_index) for every vector index in [0, nv), UNROLL*256 per workgroup trip.
// `full` tiles run without bounds checks so the UNROLL loads issue back to back.
template <int U, typename Body> __device__ inline void tile_loop(int64_t nv, Body body) {
    const int64_t tile = (int64_t)kBlock * U;
    const int64_t stride = (int64_t)gridDim.x * tile;
    for (int64_t base = (int64_t)blockIdx.x * tile; base < nv; base += stride) {
        if (base + tile <= nv) {
            body(base + threadIdx.x, std::true_type{});
        } else {
            body(base + threadIdx.x, std::false_type{});
        }
    }
}

template <typename T, int V, typename Op, int ST, bool NTL>
__device__ __forceinline__ void binary_body(const T *__restrict__ a, const T *__restrict__ b,
                                                         T *__restrict__ c, int64_t n) {
    using VT = vec_t<T, V>;
    using A = acc_t<T>;
    const int64_t nv = n / V;
    const VT *va = reinterpret_cast<const VT *>(a);
    const VT *vb = reinterpret_cast<const VT *>(b);
    VT *vc = reinterpret_cast<VT *>(c);
    tile_loop<kUnroll>(nv, [&](int64_t i, auto full) {
        VT x[kUnroll], y[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) { x[u] = ld_sel<NTL>(&va[j]); y[u] = ld_sel<NTL>(&vb[j]); }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) {
                VT r;
                A t[V];
#pragma unroll
                for (int k = 0; k < V; ++k) t[k] = Op::f(A(load_acc(x[u].v[k])), A(load_acc(y[u].v[k])));
                store_acc_vec<T, V>(r, t);
                st_mode<ST>(&vc[j], r);
            }
        }
    });
    // scalar tail (n not a multiple of V)
    if (blockIdx.x == 0) {
        int64_t j = nv * V + threadIdx.x;
        if (j < n) c[j] = store_acc<T>(Op::f(A(load_acc(a[j])), A(load_acc(b[j]))));
    }
}
// ntl: loads carry the nt hint (chosen per launch, see nt_load_* in common.hpp)
template <typename T, int V, typename Op, bool NTS>
__global__ __launch_bounds__(kBlock) void binary_kernel(const T *__restrict__ a, const T *__restrict__ b, T *__restrict__ c, int64_t n, int ntl) {
    if constexpr (NTS) {  // ntl here: a stream_policy_2r1w value
        if (ntl == 2) binary_body<T, V, Op, 2, true>(a, b, c, n);
        else if (ntl == 1) binary_body<T, V, Op, 1, true>(a, b, c, n);
        else binary_body<T, V, Op, 1, false>(a, b, c, n);
    } else {
        if (ntl) binary_body<T, V, Op, 2, true>(a, b, c, n);
        else binary_body<T, V, Op, 2, false>(a, b, c, n);
    }
}

template <typename T, int V, typename Op, bool NTS, bool NTL>
__device__ __forceinline__ void scalar_body(const T *__restrict__ a, const T s, T *__restrict__ c, int64_t n) {
    using VT = vec_t<T, V>;
    using A = acc_t<T>;
    const int64_t nv = n / V;
    const A sv = load_acc(s);
    const VT *va = reinterpret_cast<const VT *>(a);
    VT *vc = reinterpret_cast<VT *>(c);
    tile_loop<kUnroll>(nv, [&](int64_t i, auto full) {
        VT x[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) x[u] = ld_sel<NTL>(&va[j]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) {
                VT r;
                A t[V];
#pragma unroll
                for (int k = 0; k < V; ++k) t[k] = Op::f(A(load_acc(x[u].v[k])), sv);
                store_acc_vec<T, V>(r, t);
                st_sel<NTS>(&vc[j], r);
            }
        }
    });
    if (blockIdx.x == 0) {
        int64_t j = nv * V + threadIdx.x;
        if (j < n) c[j] = store_acc<T>(Op::f(A(load_acc(a[j])), sv));
    }
}
// ntl: loads carry the nt hint (chosen per launch, see nt_load_* in common.hpp)
template <typename T, int V, typename Op, bool NTS>
__global__ __launch_bounds__(kBlock) void scalar_kernel(const T *__restrict__ a, const T s, T *__restrict__ c, int64_t n, int ntl) {
    if (ntl) scalar_body<T, V, Op, NTS, true>(a, s, c, n);
    else scalar_body<T, V, Op, NTS, false>(a, s, c, n);
}

template <typename T, int V, typename Op, bool NTS, bool NTL>
__device__ __forceinline__ void unary_body(const T *__restrict__ a, T *__restrict__ c, int64_t n) {
    using VT = vec_t<T, V>;
    const int64_t nv = n / V;
    const VT *va = reinterpret_cast<const VT *>(a);
    VT *vc = reinterpret_cast<VT *>(c);
    tile_loop<kUnroll>(nv, [&](int64_t i, auto full) {
        VT x[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) x[u] = ld_sel<NTL>(&va[j]);
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            int64_t j = i + u * kBlock;
            if (decltype(full)::value || j < nv) {
                VT r;
                acc_t<T> t[V];
#pragma unroll
                for (int k = 0; k < V; ++k) t[k] = unary_apply<Op, T>(load_acc(x[u].v[k]));
                store_acc_vec<T, V>(r, t);
                st_sel<NTS>(&vc[j], r);
            }
        }
    });
    if (blockIdx.x == 0) {
        int64_t j = nv * V + threadIdx.x;
        if (j < n) c[j] = store_acc<T>(unary_apply<Op, T>(load_acc(a[j])));
    }
}
// ntl: loads carry the nt hint (chosen per launch, see nt_load_* in common.hpp)
template <typename T, int V, typename Op, bool NTS>
__global__ __launch_bounds__(kBlock) void unary_kernel(const T *__restrict__ a, T *__restrict__ c, int64_t n, int ntl) {
    if (ntl) unary_body<T, V, Op, NTS, true>(a, c, n);
    else unary_body<T, V, Op, NTS, false>(a, c, n);
}

// ---- host launchers ---------------------------------------------------------------------
template <typename T, typename Op>
int launch_binary(const void *a, const void *b, void *c, int64_t n, hipStream_t st) {
    if (!aligned(a, sizeof(T)) || !aligned(b, sizeof(T)) || !aligned(c, sizeof(T))) return DXH_ERR_ALIGN;
    constexpr int V = vec_len<T>;
    const int ntl = stream_policy_2r1w((size_t)n * sizeof(T) * 3);
    if (aligned(a, kVecBytes) && aligned(b, kVecBytes) && aligned(c, kVecBytes)) {
        unsigned g = stream_grid(n / V + 1, (int64_t)kBlock * kUnroll, kBlocksPerCU);
        if (use_nt_store((size_t)n * sizeof(T))) binary_kernel<T, V, Op, true><<<g, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, n, ntl);
        else binary_kernel<T, V, Op, false><<<g, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, n, ntl);
    } else {
        unsigned g = stream_grid(n, (int64_t)kBlock * kUnroll, kBlocksPerCU);
        binary_kernel<T, 1, Op, false><<<g, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, n, ntl);
    }
    return launch_status();
}
template <typename T, typename Op>
int launch_scalar(const void *a, dxh_scalar s, void *c, int64_t n, hipStream_t st) {
    if (!aligned(a, sizeof(T)) || !aligned(c, sizeof(T))) return DXH_ERR_ALIGN;
    constexpr int V = vec_len<T>;
    const T sv = scalar_to<T>(s);
    const int ntl = nt_load_1r1w((size_t)n * sizeof(T), (size_t)n * sizeof(T));
    if (aligned(a, kVecBytes) && aligned(c, kVecBytes)) {
        unsigned g = stream_grid(n / V + 1, (int64_t)kBlock * kUnroll, kBlocksPerCU);
        if (use_nt_store((size_t)n * sizeof(T))) scalar_kernel<T, V, Op, true><<<g, kBlock, 0, st>>>((const T *)a, sv, (T *)c, n, ntl);
        else scalar_kernel<T, V, Op, false><<<g, kBlock, 0, st>>>((const T *)a, sv, (T *)c, n, ntl);
    } else {
        unsigned g = stream_grid(n, (int64_t)kBlock * kUnroll, kBlocksPerCU);
        scalar_kernel<T, 1, Op, false><<<g, kBlock, 0, st>>>((const T *)a, sv, (T *)c, n, ntl);
    }
    return launch_status();
}
template <typename T, typename Op>
int launch_unary(const void *a, void *c, int64_t n, hipStream_t st) {
    if (!aligned(a, sizeof(T)) || !aligned(c, sizeof(T))) return DXH_ERR_ALIGN;
    constexpr int V = vec_len<T>;
    const int ntl = nt_load_1r1w((size_t)n * sizeof(T), (size_t)n * sizeof(T));
    if (aligned(a, kVecBytes) && aligned(c, kVecBytes)) {
        unsigned g = stream_grid(n / V + 1, (int64_t)kBlock * kUnroll, kBlocksPerCU);
        if (use_nt_store((size_t)n * sizeof(T))) unary_kernel<T, V, Op, true><<<g, kBlock, 0, st>>>((const T *)a, (T *)c, n, ntl);
        else unary_kernel<T, V, Op, false><<<g, kBlock, 0, st>>>((const T *)a, (T *)c, n, ntl);
    } else {
        unsigned g = stream_grid(n, (int64_t)kBlock * kUnroll, kBlocksPerCU);
        unary_kernel<T, 1, Op, false><<<g, kBlock, 0, st>>>((const T *)a, (T *)c, n, ntl);
    }
    return launch_status();
}

template <typename Op> int binary_all(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(b); DXH_CHECK_PTR(c);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return launch_binary<double, Op>(a, b, c, n, st);
    case DXH_F32: return launch_binary<float, Op>(a, b, c, n, st);
    case DXH_F16: return launch_binary<f16_t, Op>(a, b, c, n, st);
    case DXH_BF16: return launch_binary<bf16_t, Op>(a, b, c, n, st);
    case DXH_I64: return launch_binary<int64_t, Op>(a, b, c, n, st);
    case DXH_I32: return launch_binary<int32_t, Op>(a, b, c, n, st);
    case DXH_I16: return launch_binary<int16_t, Op>(a, b, c, n, st);
    case DXH_I8: return launch_binary<int8_t, Op>(a, b, c, n, st);
    default: return DXH_ERR_DTYPE;
    }
}
template <typename Op> int scalar_all(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(c);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return launch_scalar<double, Op>(a, s, c, n, st);
    case DXH_F32: return launch_scalar<float, Op>(a, s, c, n, st);
    case DXH_F16: return launch_scalar<f16_t, Op>(a, s, c, n, st);
    case DXH_BF16: return launch_scalar<bf16_t, Op>(a, s, c, n, st);
    case DXH_I64: return launch_scalar<int64_t, Op>(a, s, c, n, st);
    case DXH_I32: return launch_scalar<int32_t, Op>(a, s, c, n, st);
    case DXH_I16: return launch_scalar<int16_t, Op>(a, s, c, n, st);
    case DXH_I8: return launch_scalar<int8_t, Op>(a, s, c, n, st);
    default: return DXH_ERR_DTYPE;
    }
}
template <typename Op> int binary_f32f64(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(b); DXH_CHECK_PTR(c);
    switch (dtype) {
    case DXH_F64: return launch_binary<double, Op>(a, b, c, n, as_stream(stream));
    case DXH_F32: return launch_binary<float, Op>(a, b, c, n, as_stream(stream));
    default: return DXH_ERR_DTYPE;
    }
}
template <typename Op> int scalar_f32f64(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(c);
    switch (dtype) {
    case DXH_F64: return launch_scalar<double, Op>(a, s, c, n, as_stream(stream));
    case DXH_F32: return launch_scalar<float, Op>(a, s, c, n, as_stream(stream));
    default: return DXH_ERR_DTYPE;
    }
}
template <typename Op, bool HALF> int unary_float(int dtype, const void *a, void *c, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(c);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_F64: return launch_unary<double, Op>(a, c, n, st);
    case DXH_F32: return launch_unary<float, Op>(a, c, n, st);
    case DXH_F16: if constexpr (HALF) return launch_unary<f16_t, Op>(a, c, n, st); else return DXH_ERR_DTYPE;
    case DXH_BF16: if constexpr (HALF) return launch_unary<bf16_t, Op>(a, c, n, st); else return DXH_ERR_DTYPE;
    default: return DXH_ERR_DTYPE;
    }
}


// ---- a run of elementwise ops in one launch ---------------------------------------------------
// Same arithmetic as the kernels above, op after op, each result rounded to T and stored before
// the next op uses it, so every output has the bits the separate launches give.  What is saved is
// the traffic: an operand that an earlier op of the run produced (or that was loaded for an
// earlier op) is not read from memory again.  A lane handles one 16-byte vector index: it loads
// that vector of every input up front (all loads in flight together) and walks the op list.  The
// result of the op before is at hand in registers; inputs, and results that a later op other
// than the next one uses, sit in LDS slots of the lane's own, addressed by operand number at run
// time (no barriers: no lane reads another lane's slots).  The launch asks for as many slots as
// the run needs (4 KiB each), so short runs keep the CU full of waves.
constexpr int kChainOps = DXH_CHAIN_MAX_OPS, kChainInputs = DXH_CHAIN_MAX_INPUTS;
struct ChainArgs {  // first kernel argument: sits at offset 0 of the kernel-argument segment
    const void *in[kChainInputs];
    void *out[kChainOps];
    double scalar[kChainOps];  // already rounded to T on the host
    uint32_t op[kChainOps];    // code | lhs << 8 | rhs << 16 | save << 24, the last three as int8 (filled by the launcher from the arrays below)
    int8_t code[kChainOps], lhs[kChainOps], rhs[kChainOps];  // operand: LDS slot, or kChainPrev = result of the op before
    int8_t save[kChainOps];                                  // LDS slot that keeps the result for later ops, or -1
    int n_in, n_ops;                                         // inputs occupy slots 0 .. n_in - 1
};
constexpr int kChainPrev = -1;
template <typename T, bool NTS>
__global__ __launch_bounds__(kBlock) void chain_kernel(const ChainArgs p, int64_t nv) {
    constexpr int V = vec_len<T>;
    using VT = vec_t<T, V>;
    using A = acc_t<T>;
    extern __shared__ __attribute__((aligned(16))) unsigned char chain_lds[];
    const int t = threadIdx.x;
    // The op table is indexed by a loop counter.  Out of the by-value kernel argument that would make
    // the compiler copy the whole table into per-lane scratch memory; read from the kernel-argument
    // segment itself it is a scalar load per op, with no set-up phase.
    typedef const ChainArgs __attribute__((address_space(4))) *ArgTable;
    const ArgTable tab = (ArgTable)__builtin_amdgcn_kernarg_segment_ptr();
    // registers and LDS hold raw 16-byte vectors (a select between two of them stays in registers)
    u32x4_t *raw = reinterpret_cast<u32x4_t *>(chain_lds);
    for (int64_t i = (int64_t)blockIdx.x * kBlock + t; i < nv; i += (int64_t)gridDim.x * kBlock) {
        u32x4_t x0 = {0u, 0u, 0u, 0u}, x1 = x0, x2 = x0, x3 = x0, x4 = x0, x5 = x0, x6 = x0, x7 = x0;
#define DXH_CH_LOAD(j) if (j < p.n_in) x##j = reinterpret_cast<const u32x4_t *>(p.in[j])[i]
        DXH_CH_LOAD(0); DXH_CH_LOAD(1); DXH_CH_LOAD(2); DXH_CH_LOAD(3); DXH_CH_LOAD(4); DXH_CH_LOAD(5); DXH_CH_LOAD(6); DXH_CH_LOAD(7);
#undef DXH_CH_LOAD
#define DXH_CH_KEEP(j) if (j < p.n_in) raw[j * kBlock + t] = x##j
        DXH_CH_KEEP(0); DXH_CH_KEEP(1); DXH_CH_KEEP(2); DXH_CH_KEEP(3); DXH_CH_KEEP(4); DXH_CH_KEEP(5); DXH_CH_KEEP(6); DXH_CH_KEEP(7);
#undef DXH_CH_KEEP
        u32x4_t prev = x0;
        for (int k = 0; k < p.n_ops; ++k) {
            const uint32_t d = tab->op[k];
            const int code = (int)(d & 0xff), l = (int)(int8_t)(d >> 8), q = (int)(int8_t)(d >> 16), save = (int)(int8_t)(d >> 24);
            void *out = tab->out[k];
            u32x4_t ra = prev, rb = prev;
            if (l != kChainPrev) ra = raw[l * kBlock + t];
            if (q != kChainPrev) rb = raw[q * kBlock + t];
            const VT a = __builtin_bit_cast(VT, ra), b = __builtin_bit_cast(VT, rb);
            const A s = A(tab->scalar[k]);
            VT r;
            A y[V];
#define DXH_CH_BIN(Op) _Pragma("unroll") for (int v = 0; v < V; ++v) y[v] = Op::f(A(load_acc(a.v[v])), A(load_acc(b.v[v]))); break
#define DXH_CH_SCALAR(Op) _Pragma("unroll") for (int v = 0; v < V; ++v) y[v] = Op::f(A(load_acc(a.v[v])), s); break
#define DXH_CH_UNARY(Op) _Pragma("unroll") for (int v = 0; v < V; ++v) y[v] = unary_apply<Op, T>(load_acc(a.v[v])); break
            switch (code) {
            case DXH_CHAIN_ADD: DXH_CH_BIN(OpAdd);
            case DXH_CHAIN_SUB: DXH_CH_BIN(OpSub);
            case DXH_CHAIN_MUL: DXH_CH_BIN(OpMul);
            case DXH_CHAIN_DIV: DXH_CH_BIN(OpDiv);
            case DXH_CHAIN_MAX: DXH_CH_BIN(OpMax);
            case DXH_CHAIN_MIN: DXH_CH_BIN(OpMin);
            case DXH_CHAIN_ADDSCALAR: DXH_CH_SCALAR(OpAdd);
            case DXH_CHAIN_SUBSCALAR: DXH_CH_SCALAR(OpSub);
            case DXH_CHAIN_RSUBSCALAR: DXH_CH_SCALAR(OpRSub);
            case DXH_CHAIN_MULSCALAR: DXH_CH_SCALAR(OpMul);
            case DXH_CHAIN_DIVSCALAR: DXH_CH_SCALAR(OpDiv);
            case DXH_CHAIN_RDIVSCALAR: DXH_CH_SCALAR(OpRDiv);
            case DXH_CHAIN_MAXSCALAR: DXH_CH_SCALAR(OpMax);
            case DXH_CHAIN_MINSCALAR: DXH_CH_SCALAR(OpMin);
            case DXH_CHAIN_SQRT: DXH_CH_UNARY(OpSqrt);
            case DXH_CHAIN_EXP: DXH_CH_UNARY(OpExp);
            default: DXH_CH_UNARY(OpLog);
            }
#undef DXH_CH_BIN
#undef DXH_CH_SCALAR
#undef DXH_CH_UNARY
            store_acc_vec<T, V>(r, y);
            prev = __builtin_bit_cast(u32x4_t, r);
            if (save >= 0) raw[save * kBlock + t] = prev;
            if (out) st_sel<NTS>(&reinterpret_cast<u32x4_t *>(out)[i], prev);
        }
    }
}

template <typename T>
int launch_chain(ChainArgs &p, const dxh_chain_op *ops, int64_t n, hipStream_t st) {
    constexpr int V = vec_len<T>;
    if (n % V != 0) return DXH_ERR_ALIGN;
    for (int k = 0; k < p.n_ops; ++k) {
        p.scalar[k] = (double)load_acc(scalar_to<T>(ops[k].scalar));
        p.op[k] = (uint32_t)(uint8_t)p.code[k] | (uint32_t)(uint8_t)p.lhs[k] << 8 | (uint32_t)(uint8_t)p.rhs[k] << 16 | (uint32_t)(uint8_t)p.save[k] << 24;
    }
    const int64_t nv = n / V, blocks = (nv + kBlock - 1) / kBlock;
    int slots = p.n_in;
    for (int k = 0; k < p.n_ops; ++k) slots = std::max(slots, p.save[k] + 1);
    size_t stored = 0;
    for (int k = 0; k < p.n_ops; ++k)
        if (p.out[k]) stored += (size_t)n * sizeof(T);
    const unsigned grid = (unsigned)std::min<int64_t>(blocks, 1 << 22);
    if (use_nt_store(stored)) chain_kernel<T, true><<<grid, kBlock, (size_t)slots * kBlock * kVecBytes, st>>>(p, nv);
    else chain_kernel<T, false><<<grid, kBlock, (size_t)slots * kBlock * kVecBytes, st>>>(p, nv);
    return launch_status();
}


// ---- a run of elementwise ops over a [rows, cols] view, with row / column vectors and casts ------
// The same interpreter for runs whose tensors differ in dtype (f32, bf16, f16) or in extent: besides
// [rows, cols] tensors a run may read and write row vectors [1, cols] and column vectors [rows, 1],
// and its ops include the cast (todtype), the copy of a vector into every row or column
// (broadcastTo) and the sum of every row (sum over the last axis).  A lane owns groups of four
// adjacent columns of one row.  Every value is carried as fp32 (a 16-bit float is exact in it) and
// every result is rounded to its op's dtype before anything uses it, so the stored bits are those
// of the separate launches.  An op on vectors is computed by every lane for its own row or columns
// and stored by the lanes of column 0 or row 0 only; a later op of the run that reads the vector
// has the value at hand, no lane waits for another.  That is also why a vector input must not be
// an output of the same run: lanes that read it race with the lane that overwrites it.
//
// Two lane layouts, one group of four columns per lane in both.  Without a row sum the groups are
// dealt out in memory order.  With one (BYROW) a row has P adjacent lanes of its own (P a power of
// two, lanes past the row's last group idle) and the sum is folded by the first G of them exactly as
// the G lanes of dxh_sum's row stage fold it (same code, reduce_order.hpp; the operand is read back
// from its LDS slot, where lane j of the row put group j), so it has the bits dxh_sum would store;
// two workgroup barriers per sum hand the operand over and the result back.
//
// The op table is read from the kernel-argument segment itself, through the scalar cache, with the
// op counter as index: indexing the by-value argument that way would make the compiler copy it to
// per-lane scratch memory, and a copy in LDS costs a set-up phase longer than the ops of a small run.
enum { kRowFull = 0, kRowVec = 1, kColVec = 2 };
enum { kRcF32 = 0, kRcBF16 = 1, kRcF16 = 2 };
constexpr int kRowOps = DXH_CHAIN_ROWS_MAX_OPS, kRowVecs = 4;
constexpr size_t kRowLdsMax = 156 * 1024, kRowLdsDefault = 64 * 1024;  // dynamic LDS: what the CU has beside the static part, what a launch gets unasked
struct RowChainArgs {  // first kernel argument: sits at offset 0 of the kernel-argument segment
    uint64_t op[kRowOps];  // code | lhs << 8 | rhs << 16 | save << 24 | dtype << 32 | extent << 40; lhs, rhs, save as int8
    float scalar[kRowOps];  // already rounded to the op's dtype on the host
    void *out[kRowOps];
    const void *in[kChainInputs];
    uint8_t in_dtype[kChainInputs], in_kind[kChainInputs];
    int n_in, n_ops;
};
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4_t rowchain_load(const void *p, int dt, int kind, int64_t row, int64_t c4, int64_t i) {
    if (kind == kColVec) {
        float v;
        if (dt == kRcF32) v = reinterpret_cast<const float *>(p)[row];
        else if (dt == kRcBF16) v = load_acc(reinterpret_cast<const bf16_t *>(p)[row]);
        else v = load_acc(reinterpret_cast<const f16_t *>(p)[row]);
        return f32x4_t{v, v, v, v};
    }
    const int64_t j = kind == kRowVec ? c4 : i;
    if (dt == kRcF32) return reinterpret_cast<const f32x4_t *>(p)[j];
    if (dt == kRcBF16) {
        const vec_t<bf16_t, 4> x = reinterpret_cast<const vec_t<bf16_t, 4> *>(p)[j];
        return f32x4_t{load_acc(x.v[0]), load_acc(x.v[1]), load_acc(x.v[2]), load_acc(x.v[3])};
    }
    const vec_t<f16_t, 4> x = reinterpret_cast<const vec_t<f16_t, 4> *>(p)[j];
    return f32x4_t{load_acc(x.v[0]), load_acc(x.v[1]), load_acc(x.v[2]), load_acc(x.v[3])};
}
// rounds y to the op's dtype (in place, as fp32 again) and, if this lane is the one to store it
// (`owner`: its group of columns exists), stores it where the op's extent says
__device__ __forceinline__ void rowchain_round_store(float (&y)[4], void *out, int dt, int kind, bool owner, int64_t row, int64_t c4, int64_t i) {
    const bool mine = out && owner && (kind == kRowFull || (kind == kRowVec ? row == 0 : c4 == 0));
    const int64_t j = kind == kRowVec ? c4 : i;
    if (dt == kRcF32) {
        if (mine) {
            if (kind == kColVec) reinterpret_cast<float *>(out)[row] = y[0];
            else reinterpret_cast<f32x4_t *>(out)[j] = f32x4_t{y[0], y[1], y[2], y[3]};
        }
    } else if (dt == kRcBF16) {
        vec_t<bf16_t, 4> r;
        store_acc_vec<bf16_t, 4>(r, y);
#pragma unroll
        for (int v = 0; v < 4; ++v) y[v] = load_acc(r.v[v]);
        if (mine) {
            if (kind == kColVec) reinterpret_cast<bf16_t *>(out)[row] = r.v[0];
            else reinterpret_cast<vec_t<bf16_t, 4> *>(out)[j] = r;
        }
    } else {
        vec_t<f16_t, 4> r;
        store_acc_vec<f16_t, 4>(r, y);
#pragma unroll
        for (int v = 0; v < 4; ++v) y[v] = load_acc(r.v[v]);
        if (mine) {
            if (kind == kColVec) reinterpret_cast<f16_t *>(out)[row] = r.v[0];
            else reinterpret_cast<vec_t<f16_t, 4> *>(out)[j] = r;
        }
    }
}
template <bool BYROW>
__global__ __launch_bounds__(kBlock) void chain_rows_kernel(const RowChainArgs p, int64_t rows, int64_t cq, int G, int P) {
    extern __shared__ __attribute__((aligned(16))) unsigned char chain_lds[];
    __shared__ float row_sums[kBlock];  // BYROW: one per row of the workgroup
    typedef const RowChainArgs __attribute__((address_space(4))) *ArgTable;
    const ArgTable tab = (ArgTable)__builtin_amdgcn_kernarg_segment_ptr();
    const int t = threadIdx.x;
    f32x4_t *slot = reinterpret_cast<f32x4_t *>(chain_lds);  // slot s of this lane: slot[s * kBlock + t]
    const int64_t total = rows * cq;
    const int64_t first = BYROW ? (int64_t)blockIdx.x : (int64_t)blockIdx.x * kBlock + t;
    const int64_t step = BYROW ? total : (int64_t)gridDim.x * kBlock;  // BYROW: one trip, the rows come from the block index
    const int n_in = p.n_in, n_ops = p.n_ops;
    for (int64_t i0 = first; i0 < total; i0 += step) {
        int64_t row, c4, idx;
        bool own = true;
        int lane = 0, row_in_block = 0;
        if constexpr (BYROW) {
            lane = t & (P - 1);
            row_in_block = t / P;
            const int64_t r = (int64_t)blockIdx.x * (kBlock / P) + row_in_block;
            // lanes past the last row or the row's last group go through the motions (barriers and shuffles
            // need them) on a clamped position and store nothing
            own = r < rows && lane < cq;
            row = r < rows ? r : rows - 1;
            c4 = lane < cq ? lane : cq - 1;
            idx = row * cq + c4;
        } else {
            if (total <= 0x7fffffff) { const uint32_t r32 = (uint32_t)i0 / (uint32_t)cq; row = r32; c4 = (uint32_t)i0 - r32 * (uint32_t)cq; }
            else { row = i0 / cq; c4 = i0 - row * cq; }
            idx = i0;
        }
        f32x4_t prev = {0.f, 0.f, 0.f, 0.f};
        for (int j = 0; j < n_in; ++j) slot[j * kBlock + t] = rowchain_load(tab->in[j], tab->in_dtype[j], tab->in_kind[j], row, c4, idx);
        for (int k = 0; k < n_ops; ++k) {
            const uint64_t d = tab->op[k];
            const int code = (int)(d & 0xff), l = (int)(int8_t)(d >> 8), q = (int)(int8_t)(d >> 16), save = (int)(int8_t)(d >> 24);
            const int dt = (int)((d >> 32) & 0xff), kind = (int)((d >> 40) & 0xff);
            const float s = tab->scalar[k];
            void *out = tab->out[k];
            f32x4_t a = prev, b = prev;
            if (l != kChainPrev) a = slot[l * kBlock + t];
            if (q != kChainPrev) b = slot[q * kBlock + t];
            float rowsum = 0.f;
            if constexpr (BYROW) {
                if (code >= DXH_CHAIN_ROWSUM) {  // sum, max or min of the row; the operand sits in slot l (the host sees to that), group j of the row at lane j
                    __syncthreads();
                    if (lane < G) {
                        const f32x4_t *src = slot + l * kBlock + row_in_block * P;
                        auto ld = [&](int64_t i) __attribute__((always_inline)) { return __builtin_bit_cast(vec_t<float, 4>, src[i]); };
                        float v;
                        if (code == DXH_CHAIN_ROWSUM) {
                            float acc[4] = {0.f, 0.f, 0.f, 0.f};
                            row_lane_fold<R_SUM, float, 4>(acc, lane, G, cq, ld);
                            v = row_group_fold<R_SUM, float, 4>(acc, G);
                        } else if (code == DXH_CHAIN_ROWMAX) {
                            float acc[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[e] = rinit<R_MAX, float, float>();
                            row_lane_fold<R_MAX, float, 4>(acc, lane, G, cq, ld);
                            v = row_group_fold<R_MAX, float, 4>(acc, G);
                        } else {
                            float acc[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[e] = rinit<R_MIN, float, float>();
                            row_lane_fold<R_MIN, float, 4>(acc, lane, G, cq, ld);
                            v = row_group_fold<R_MIN, float, 4>(acc, G);
                        }
                        if (lane == 0) row_sums[row_in_block] = v;
                    }
                    __syncthreads();
                    rowsum = row_sums[row_in_block];
                }
            }
            float y[4];
#define DXH_RC_BIN(Op) _Pragma("unroll") for (int v = 0; v < 4; ++v) y[v] = Op::f(a[v], b[v]); break
#define DXH_RC_SCALAR(Op) _Pragma("unroll") for (int v = 0; v < 4; ++v) y[v] = Op::f(a[v], s); break
#define DXH_RC_UNARY(Op) _Pragma("unroll") for (int v = 0; v < 4; ++v) y[v] = Op::f(a[v]); break
            switch (code) {
            case DXH_CHAIN_ADD: DXH_RC_BIN(OpAdd);
            case DXH_CHAIN_SUB: DXH_RC_BIN(OpSub);
            case DXH_CHAIN_MUL: DXH_RC_BIN(OpMul);
            case DXH_CHAIN_DIV: DXH_RC_BIN(OpDiv);
            case DXH_CHAIN_MAX: DXH_RC_BIN(OpMax);
            case DXH_CHAIN_MIN: DXH_RC_BIN(OpMin);
            case DXH_CHAIN_ADDSCALAR: DXH_RC_SCALAR(OpAdd);
            case DXH_CHAIN_SUBSCALAR: DXH_RC_SCALAR(OpSub);
            case DXH_CHAIN_RSUBSCALAR: DXH_RC_SCALAR(OpRSub);
            case DXH_CHAIN_MULSCALAR: DXH_RC_SCALAR(OpMul);
            case DXH_CHAIN_DIVSCALAR: DXH_RC_SCALAR(OpDiv);
            case DXH_CHAIN_RDIVSCALAR: DXH_RC_SCALAR(OpRDiv);
            case DXH_CHAIN_MAXSCALAR: DXH_RC_SCALAR(OpMax);
            case DXH_CHAIN_MINSCALAR: DXH_RC_SCALAR(OpMin);
            case DXH_CHAIN_SQRT: DXH_RC_UNARY(OpSqrt);
            case DXH_CHAIN_EXP:
                if (dt == kRcF32) { DXH_RC_UNARY(OpExp); }
                _Pragma("unroll") for (int v = 0; v < 4; ++v) y[v] = exp_to_half(a[v]);
                break;
            case DXH_CHAIN_LOG: DXH_RC_UNARY(OpLog);
            case DXH_CHAIN_SQUARE: DXH_RC_UNARY(OpSquare);
            case DXH_CHAIN_ROWSUM: case DXH_CHAIN_ROWMAX: case DXH_CHAIN_ROWMIN: _Pragma("unroll") for (int v = 0; v < 4; ++v) y[v] = rowsum; break;
            default: _Pragma("unroll") for (int v = 0; v < 4; ++v) y[v] = a[v]; break;  // DXH_CHAIN_COPY
            }
#undef DXH_RC_BIN
#undef DXH_RC_SCALAR
#undef DXH_RC_UNARY
            rowchain_round_store(y, out, dt, kind, own, row, c4, idx);
            prev = f32x4_t{y[0], y[1], y[2], y[3]};
            if (save >= 0) slot[save * kBlock + t] = prev;
        }
    }
}

// Launches with more dynamic LDS than a kernel gets unasked need the limit raised once per device.
// That is a call on the function, not on a stream: it is made at device set-up (dxh_set_device) or
// by the first launch that needs it, unless that one is being captured.
namespace {
std::mutex g_rows_mutex;
bool g_rows_lds_raised[64] = {};
}
int chain_rows_raise_lds(hipStream_t st, bool may_be_capturing) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { (void)hipGetLastError(); return (int)e; }
    if (dev < 0 || dev >= 64) return DXH_ERR_ARG;
    std::lock_guard<std::mutex> lock(g_rows_mutex);
    if (g_rows_lds_raised[dev]) return DXH_OK;
    if (may_be_capturing && stream_is_capturing(st)) return DXH_ERR_NOT_READY;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chain_rows_kernel<true>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kRowLdsMax);
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void *>(&chain_rows_kernel<false>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)kRowLdsMax);
    if (e != hipSuccess) { (void)hipGetLastError(); return (int)e; }
    g_rows_lds_raised[dev] = true;
    return DXH_OK;
}
void chain_device_init() { (void)chain_rows_raise_lds(nullptr, false); }

}  // namespace dxh

using namespace dxh;

extern "C" {

int dxh_add(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) { return binary_all<OpAdd>(dtype, a, b, c, n, stream); }
int dxh_sub(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) { return binary_all<OpSub>(dtype, a, b, c, n, stream); }
int dxh_mul(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) { return binary_all<OpMul>(dtype, a, b, c, n, stream); }
int dxh_div(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) { return binary_all<OpDiv>(dtype, a, b, c, n, stream); }
int dxh_max(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) { return binary_all<OpMax>(dtype, a, b, c, n, stream); }
int dxh_min(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) { return binary_all<OpMin>(dtype, a, b, c, n, stream); }
int dxh_pow(int dtype, const void *a, const void *b, void *c, int64_t n, void *stream) { return binary_f32f64<OpPow>(dtype, a, b, c, n, stream); }

int dxh_addscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) { return scalar_all<OpAdd>(dtype, a, s, c, n, stream); }
int dxh_subscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) { return scalar_all<OpSub>(dtype, a, s, c, n, stream); }
int dxh_rsubscalar(int dtype, dxh_scalar s, const void *a, void *c, int64_t n, void *stream) { return scalar_all<OpRSub>(dtype, a, s, c, n, stream); }
int dxh_mulscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) { return scalar_all<OpMul>(dtype, a, s, c, n, stream); }
int dxh_divscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) { return scalar_all<OpDiv>(dtype, a, s, c, n, stream); }
int dxh_rdivscalar(int dtype, dxh_scalar s, const void *a, void *c, int64_t n, void *stream) { return scalar_all<OpRDiv>(dtype, a, s, c, n, stream); }
int dxh_maxscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) { return scalar_all<OpMax>(dtype, a, s, c, n, stream); }
int dxh_minscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) { return scalar_all<OpMin>(dtype, a, s, c, n, stream); }
int dxh_powscalar(int dtype, const void *a, dxh_scalar s, void *c, int64_t n, void *stream) {
    // the square (RMSNorm's powscalar(x, 2)) skips the general powf/pow expansion: 1.8 M floats took
    // 11.5 us through it, a launch-bound 4 us as x*x
    if (s.f == 2.0 && (dtype == DXH_F32 || dtype == DXH_F64)) return unary_float<OpSquare, false>(dtype, a, c, n, stream);
    return scalar_f32f64<OpPow>(dtype, a, s, c, n, stream);
}
int dxh_rpowscalar(int dtype, dxh_scalar s, const void *a, void *c, int64_t n, void *stream) { return scalar_f32f64<OpRPow>(dtype, a, s, c, n, stream); }

int dxh_sqrt(int dtype, const void *a, void *c, int64_t n, void *stream) { return unary_float<OpSqrt, true>(dtype, a, c, n, stream); }
int dxh_exp(int dtype, const void *a, void *c, int64_t n, void *stream) { return unary_float<OpExp, true>(dtype, a, c, n, stream); }
int dxh_log(int dtype, const void *a, void *c, int64_t n, void *stream) { return unary_float<OpLog, true>(dtype, a, c, n, stream); }
int dxh_sin(int dtype, const void *a, void *c, int64_t n, void *stream) { return unary_float<OpSin, true>(dtype, a, c, n, stream); }
int dxh_cos(int dtype, const void *a, void *c, int64_t n, void *stream) { return unary_float<OpCos, true>(dtype, a, c, n, stream); }
int dxh_tan(int dtype, const void *a, void *c, int64_t n, void *stream) { return unary_float<OpTan, false>(dtype, a, c, n, stream); }

int dxh_invert(int dtype, const void *a, void *c, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    DXH_CHECK_PTR(a); DXH_CHECK_PTR(c);
    hipStream_t st = as_stream(stream);
    switch (dtype) {
    case DXH_I64: return launch_unary<int64_t, OpInvert>(a, c, n, st);
    case DXH_I32: return launch_unary<int32_t, OpInvert>(a, c, n, st);
    case DXH_I16: return launch_unary<int16_t, OpInvert>(a, c, n, st);
    case DXH_I8: return launch_unary<int8_t, OpInvert>(a, c, n, st);
    case DXH_BOOL: return launch_unary<bool_t, OpInvert>(a, c, n, st);
    default: return DXH_ERR_DTYPE;
    }
}

int dxh_chain(int dtype, const void *const *inputs, int n_inputs, const dxh_chain_op *ops, int n_ops, int64_t n, void *stream) {
    DXH_CHECK_N(n);
    if (n_ops < 1 || n_ops > kChainOps || n_inputs < 0 || n_inputs > kChainInputs || !ops || (n_inputs > 0 && !inputs)) return DXH_ERR_ARG;
    ChainArgs p{};
    p.n_in = n_inputs;
    p.n_ops = n_ops;
    for (int j = 0; j < n_inputs; ++j) {
        if (!inputs[j]) return DXH_ERR_ARG;
        if (!aligned(inputs[j], kVecBytes)) return DXH_ERR_ALIGN;
        p.in[j] = inputs[j];
    }
    // operand of op k: an input's slot, the registers (result of op k - 1), or the slot that the
    // producing op saves into (handed out here, on first use)
    int next_slot = n_inputs;
    for (int k = 0; k < n_ops; ++k) p.save[k] = -1;
    constexpr int kBad = -2;
    auto operand = [&](int ref, int k) {
        if (ref >= 0 && ref < n_inputs) return ref;
        if (ref < DXH_CHAIN_RESULT || ref >= DXH_CHAIN_RESULT + k) return kBad;
        const int j = ref - DXH_CHAIN_RESULT;
        if (j == k - 1) return kChainPrev;
        if (p.save[j] < 0) p.save[j] = (int8_t)next_slot++;
        return (int)p.save[j];
    };
    for (int k = 0; k < n_ops; ++k) {
        const dxh_chain_op &o = ops[k];
        if (o.code < DXH_CHAIN_ADD || o.code > DXH_CHAIN_LOG || (!o.out && k == n_ops - 1)) return DXH_ERR_ARG;
        if (o.out && !aligned(o.out, kVecBytes)) return DXH_ERR_ALIGN;
        const int l = operand(o.lhs, k), r = o.code <= DXH_CHAIN_MIN ? operand(o.rhs, k) : l;
        if (l == kBad || r == kBad) return DXH_ERR_ARG;
        p.code[k] = (int8_t)o.code; p.lhs[k] = (int8_t)l; p.rhs[k] = (int8_t)r; p.out[k] = o.out;
    }
    if (n == 0) return DXH_OK;
    hipStream_t st = as_stream(stream);
    if (dtype == DXH_F32 || dtype == DXH_F16 || dtype == DXH_BF16) {
        if (n % (kVecBytes / dtype_size(dtype)) != 0) return DXH_ERR_ALIGN;
        const int rc = static_chain_try(dtype, inputs, n_inputs, ops, n_ops, n, st);
        if (rc != kNotStatic) return rc;
    }
    chain_count_interpreted();
    switch (dtype) {
    case DXH_F64: return launch_chain<double>(p, ops, n, st);
    case DXH_F32: return launch_chain<float>(p, ops, n, st);
    case DXH_F16: return launch_chain<f16_t>(p, ops, n, st);
    case DXH_BF16: return launch_chain<bf16_t>(p, ops, n, st);
    default: return DXH_ERR_DTYPE;
    }
}


int dxh_chain_rows_can_sum(int64_t rows, int64_t cols) {
    if (rows < 1 || cols < 4 || cols % 4 != 0) return 0;
    const int g = sum_rows_group_f32(rows, cols);
    return g > 0 && cols / 4 <= (int64_t)g * kRowVecs;
}

// dry: every check of a real call and no launch
static int chain_rows_impl(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops, int64_t rows, int64_t cols, void *stream, bool dry) {
    if (rows < 0 || cols < 0 || n_ops < 1 || n_ops > kRowOps || n_inputs < 0 || n_inputs > kChainInputs || !ops || (n_inputs > 0 && !inputs)) return DXH_ERR_ARG;
    if (cols % 4 != 0) return DXH_ERR_ALIGN;
    if (rows > 0 && cols / 4 > INT64_MAX / rows) return DXH_ERR_SHAPE;
    auto dtype_code = [](int dtype) { return dtype == DXH_F32 ? (int)kRcF32 : dtype == DXH_BF16 ? (int)kRcBF16 : dtype == DXH_F16 ? (int)kRcF16 : -1; };
    // a [rows, cols] tensor or a row vector is touched four elements at a time, a column vector one
    auto align_of = [](int dt, int kind) { return (size_t)(kind == kColVec ? 1 : 4) * (dt == kRcF32 ? 4 : 2); };
    RowChainArgs p{};
    p.n_in = n_inputs;
    p.n_ops = n_ops;
    for (int j = 0; j < n_inputs; ++j) {
        const int dt = dtype_code(inputs[j].dtype);
        if (dt < 0) return DXH_ERR_DTYPE;
        if (!inputs[j].data || inputs[j].extent < DXH_CHAIN_FULL || inputs[j].extent > DXH_CHAIN_COLUMN) return DXH_ERR_ARG;
        if (!aligned(inputs[j].data, align_of(dt, inputs[j].extent))) return DXH_ERR_ALIGN;
        p.in[j] = inputs[j].data; p.in_dtype[j] = (uint8_t)dt; p.in_kind[j] = (uint8_t)inputs[j].extent;
    }
    int next_slot = n_inputs;
    bool by_row = false, half_reduction = false;
    int save_of[kRowOps], kind_of[kRowOps], dtype_of[kRowOps], code_of[kRowOps], lhs_of[kRowOps], rhs_of[kRowOps];
    for (int k = 0; k < n_ops; ++k) save_of[k] = -1;
    constexpr int kBad = -2;
    // operand of op k (see dxh_chain); `want` is the extent it must have, or -1 for any; `in_slot`: never
    // the registers, even when it is the result of the op before
    auto operand = [&](int ref, int k, int want, bool in_slot, int *dtype) {
        if (ref >= 0 && ref < n_inputs) {
            *dtype = p.in_dtype[ref];
            return want < 0 || p.in_kind[ref] == want ? ref : kBad;
        }
        if (ref < DXH_CHAIN_RESULT || ref >= DXH_CHAIN_RESULT + k) return kBad;
        const int j = ref - DXH_CHAIN_RESULT;
        *dtype = dtype_of[j];
        if (want >= 0 && kind_of[j] != want) return kBad;
        if (j == k - 1 && !in_slot) return kChainPrev;
        if (save_of[j] < 0) save_of[j] = next_slot++;
        return save_of[j];
    };
    for (int k = 0; k < n_ops; ++k) {
        const dxh_chain_rows_op &o = ops[k];
        const int dt = dtype_code(o.dtype);
        if (dt < 0) return DXH_ERR_DTYPE;
        if (o.code < DXH_CHAIN_ADD || o.code > DXH_CHAIN_ROWMIN || o.extent < DXH_CHAIN_FULL || o.extent > DXH_CHAIN_COLUMN || (!o.out && k == n_ops - 1)) return DXH_ERR_ARG;
        if (o.out && !aligned(o.out, align_of(dt, o.extent))) return DXH_ERR_ALIGN;
        kind_of[k] = o.extent;  // before operand(): a later op asks for it
        dtype_of[k] = dt;
        const bool rowsum = o.code >= DXH_CHAIN_ROWSUM;  // sum, max or min of every row
        // an op of full extent takes anything, an op on vectors only vectors of its own kind; a row
        // reduction turns a [rows, cols] operand into a column of the same dtype
        const int want = rowsum ? (int)kRowFull : o.extent == DXH_CHAIN_FULL ? -1 : o.extent;
        int ldt = 0, rdt = 0;
        const int l = operand(o.lhs, k, want, rowsum, &ldt), r = o.code <= DXH_CHAIN_MIN ? operand(o.rhs, k, want, false, &rdt) : l;
        if (l == kBad || r == kBad) return DXH_ERR_ARG;
        if (rowsum) {
            if (o.extent != DXH_CHAIN_COLUMN) return DXH_ERR_ARG;
            if (dt != ldt) return DXH_ERR_DTYPE;
            if (dt != kRcF32) half_reduction = true;  // compiled programs only
            by_row = true;
        }
        for (int j = 0; j < n_inputs; ++j)
            if (o.out && o.out == inputs[j].data && inputs[j].extent != DXH_CHAIN_FULL) return DXH_ERR_ARG;  // lanes would race for it
        code_of[k] = o.code; lhs_of[k] = l; rhs_of[k] = r; p.out[k] = o.out;
        const float sf = (float)o.scalar.f;
        p.scalar[k] = dt == kRcF32 ? sf : dt == kRcBF16 ? load_acc(to_bf16(sf)) : load_acc(to_f16(sf));
    }
    int slots = std::max(n_inputs, 1);
    for (int k = 0; k < n_ops; ++k) {  // save_of[k] is final only now: a later op may have asked for the slot
        slots = std::max(slots, save_of[k] + 1);
        p.op[k] = (uint64_t)(uint8_t)code_of[k] | (uint64_t)(uint8_t)(int8_t)lhs_of[k] << 8 | (uint64_t)(uint8_t)(int8_t)rhs_of[k] << 16 |
                  (uint64_t)(uint8_t)(int8_t)save_of[k] << 24 | (uint64_t)(uint8_t)dtype_of[k] << 32 | (uint64_t)(uint8_t)kind_of[k] << 40;
    }
    if (rows > 0 && cols > 0) {  // a run that the library holds a compiled kernel for
        const int rc = static_rows_try(inputs, n_inputs, ops, n_ops, rows, cols, as_stream(stream), dry);
        if (rc != kNotStatic) return rc;
    }
    if (half_reduction) return DXH_ERR_DTYPE;  // the interpreting kernel's lanes share a row the way the fp32 reduction does
    const int64_t cq = cols / 4;
    int group = 0, per_row = 1;
    if (by_row) {  // the first lanes of a row fold it as dxh_sum's row stage would, or the sums would not be its sums
        if (rows == 0 || cols == 0) return DXH_OK;
        group = sum_rows_group_f32(rows, cols);
        if (group <= 0 || cq > (int64_t)group * kRowVecs) return DXH_ERR_SHAPE;
        per_row = group;
        while (per_row < cq) per_row <<= 1;  // at most group * kRowVecs = kBlock lanes
    }
    const size_t lds = (size_t)slots * kBlock * kVecBytes;
    if (lds > kRowLdsMax) return DXH_ERR_SHAPE;
    if (rows == 0 || cols == 0 || dry) return DXH_OK;
    hipStream_t st = as_stream(stream);
    if (lds > kRowLdsDefault) {
        const int rc = chain_rows_raise_lds(st, true);
        if (rc != DXH_OK) return rc;
    }
    chain_count_interpreted();
    if (by_row) {
        const int64_t rows_per_block = kBlock / per_row, blocks = (rows + rows_per_block - 1) / rows_per_block;
        if (blocks > 0x7fffffff) return DXH_ERR_SHAPE;
        chain_rows_kernel<true><<<(unsigned)blocks, kBlock, lds, st>>>(p, rows, cq, group, per_row);
    } else {
        const int64_t blocks = (rows * cq + kBlock - 1) / kBlock;
        chain_rows_kernel<false><<<(unsigned)std::min<int64_t>(blocks, 1 << 22), kBlock, lds, st>>>(p, rows, cq, 1, 1);
    }
    return launch_status();
}

int dxh_chain_rows(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops, int64_t rows, int64_t cols, void *stream) {
    return chain_rows_impl(inputs, n_inputs, ops, n_ops, rows, cols, stream, false);
}
int dxh_chain_rows_check(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops, int64_t rows, int64_t cols) {
    return chain_rows_impl(inputs, n_inputs, ops, n_ops, rows, cols, nullptr, true);
}

}  // extern "C"
