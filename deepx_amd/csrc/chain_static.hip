// chain_static.hip — compiled instances of the runs of ops that the deepx front emits over and over
// (chain_static.hpp says how a run becomes a type).  dxh_chain and dxh_chain_rows hand every run to
// static_chain_try / static_rows_try first; a run that equals one of the programs below in codes,
// operand references, dtypes and extents is launched as that program's kernel, anything else (or
// DXH_TUNE_CHAIN_STATIC 0) goes to the interpreting kernels of elementwise.hip.  Scalars, pointers
// and which results are stored stay run-time values.
//
// Row form: a row belongs to G adjacent lanes, lane j holding the 16-byte vectors j, j + G, ... of
// the row in registers (NV of them at most) — G and that assignment are the separate reduction
// kernel's for the same [rows, cols] and element size (reduce.hip: build_plan, reduce_row_body), and
// the fold below visits a lane's vectors in that kernel's order (batches of 8, then 4, then singles,
// then the group's shuffles), so a row sum / max / min inside a run has the separate launch's bits
// without a trip through LDS.  Without a row reduction in the program G only shapes the loads.
#include "chain_static.hpp"
#include <atomic>

namespace dxh {

struct StaticArgs {
    const void *in[DXH_CHAIN_MAX_INPUTS];
    void *out[DXH_CHAIN_ROWS_MAX_OPS];
    float scalar[DXH_CHAIN_ROWS_MAX_OPS];  // already rounded to the op's dtype on the host
    int nt_store;  // use_nt_store on the bytes the launch stores: non-temporal stores, else write-through ones
};

// ---- row form ---------------------------------------------------------------------------------------
template <typename Prog, int VW, int NV>
__global__ __launch_bounds__(kBlock) void chain_static_rows_kernel(const StaticArgs p, int64_t rows, int lv, int G) {
    constexpr int NIN = Prog::n_in, NOPS = Prog::n_ops;
    const int t = threadIdx.x, lane = t & (G - 1), rows_per_block = kBlock / G;
    const int64_t row_raw = (int64_t)blockIdx.x * rows_per_block + t / G;
    const bool row_ok = row_raw < rows;
    const int64_t row = row_ok ? row_raw : rows - 1;  // lanes past the last row go through the motions (shuffles need them) and store nothing
    // vector u of this lane: number c[u] of the row, or past the row's end (then it is clamped for
    // loads and never stored or folded)
    int c[NV];
    bool own[NV];
#pragma unroll
    for (int u = 0; u < NV; ++u) {
        const int raw = lane + u * G;
        own[u] = raw < lv;
        c[u] = own[u] ? raw : lv - 1;
    }
    // values by number: inputs first, then results.  FULL and ROW values: [u][e]; a COLUMN value is one
    // number per row, kept in [0][0].  Every index below is a compile-time constant after unrolling.
    float val[Prog::n_val][NV][VW];
    static_for<NIN>([&](auto j_) __attribute__((always_inline)) {
        constexpr int j = decltype(j_)::value;
        using In = typename Prog::ins::template at<j>;
        if constexpr (In::ext == DXH_CHAIN_COLUMN) {
            val[j][0][0] = load_one<In::dt>(p.in[j], row);
        } else {
#pragma unroll
            for (int u = 0; u < NV; ++u)
                load_elems<In::dt, VW>(p.in[j], ((In::ext == DXH_CHAIN_ROW ? 0 : row * lv) + c[u]) * VW, val[j][u]);
        }
    });
    static_for<NOPS>([&](auto k_) __attribute__((always_inline)) {
        constexpr int k = decltype(k_)::value, me = NIN + k;
        using Op = typename Prog::ops::template at<k>;
        constexpr int L = Prog::value_of(Op::lhs), R = chain_code_is_binary(Op::code) ? Prog::value_of(Op::rhs) : L;
        constexpr int Lext = Prog::template ext_of<L>(), Rext = Prog::template ext_of<R>();
        const float s = p.scalar[k];
        void *out = p.out[k];
        if constexpr (chain_code_is_rowred(Op::code)) {
            // the lane's vectors of the operand, folded as reduce_row_body folds them
            constexpr int K = Op::code == DXH_CHAIN_ROWSUM ? R_SUM : Op::code == DXH_CHAIN_ROWMAX ? R_MAX : R_MIN;
            constexpr int Ldt = Prog::template dt_of<L>();
            static_assert(Lext == DXH_CHAIN_FULL && Op::ext == DXH_CHAIN_COLUMN && Ldt == Op::dt, "a row reduction takes a full operand of its own dtype");
            float acc[VW];
#pragma unroll
            for (int e = 0; e < VW; ++e) {
                if constexpr (Ldt == kSBF16) acc[e] = rinit<K, float, bf16_t>();
                else if constexpr (Ldt == kSF16) acc[e] = rinit<K, float, f16_t>();
                else acc[e] = rinit<K, float, float>();
            }
            auto tree8 = [&](auto u0) __attribute__((always_inline)) {
                constexpr int u = decltype(u0)::value;
                if constexpr (u + 8 <= NV) {
#pragma unroll
                    for (int e = 0; e < VW; ++e) {
                        const float t0 = rop<K, float>(rop<K, float>(val[L][u][e], val[L][u + 1][e]), rop<K, float>(val[L][u + 2][e], val[L][u + 3][e]));
                        const float t1 = rop<K, float>(rop<K, float>(val[L][u + 4][e], val[L][u + 5][e]), rop<K, float>(val[L][u + 6][e], val[L][u + 7][e]));
                        acc[e] = rop<K, float>(acc[e], rop<K, float>(t0, t1));
                    }
                }
            };
            auto tree4 = [&](auto u0) __attribute__((always_inline)) {
                constexpr int u = decltype(u0)::value;
                if constexpr (u + 4 <= NV) {
#pragma unroll
                    for (int e = 0; e < VW; ++e) {
                        const float t0 = rop<K, float>(val[L][u][e], val[L][u + 1][e]);
                        const float t1 = rop<K, float>(val[L][u + 2][e], val[L][u + 3][e]);
                        acc[e] = rop<K, float>(acc[e], rop<K, float>(t0, t1));
                    }
                }
            };
            auto singles = [&](auto u0) __attribute__((always_inline)) {  // at most three are left at that point
                static_for<3>([&](auto d_) __attribute__((always_inline)) {
                    constexpr int u = decltype(u0)::value + decltype(d_)::value;
                    if constexpr (u < NV) {
                        if (lane + u * G < lv) {
#pragma unroll
                            for (int e = 0; e < VW; ++e) acc[e] = rop<K, float>(acc[e], val[L][u][e]);
                        }
                    }
                });
            };
            // NV <= 8: one batch of 8 takes everything; else at most one batch of 4, then singles
            static_assert(NV <= 8, "the fold below covers eight vectors per lane");
            if (NV >= 8 && lane + 7 * G < lv) {
                tree8(ic<0>{});
            } else if (NV >= 4 && lane + 3 * G < lv) {
                tree4(ic<0>{});
                singles(ic<4>{});
            } else {
                singles(ic<0>{});
            }
            float v = row_group_fold<K, float, VW>(acc, G);
            v = round_one(v, Op::dt);
            val[me][0][0] = v;
            if (out && row_ok && lane == 0) store_one<Op::dt>(out, row, v);
        } else if constexpr (Op::ext == DXH_CHAIN_COLUMN) {
            static_assert(Lext == DXH_CHAIN_COLUMN && Rext == DXH_CHAIN_COLUMN, "an op on column vectors takes column vectors");
            float v = chain_apply<Op::code, Op::dt != kSF32>(val[L][0][0], val[R][0][0], s);
            v = round_one(v, Op::dt);
            val[me][0][0] = v;
            if (out && row_ok && lane == 0) store_one<Op::dt>(out, row, v);
        } else {
            static_assert(Op::ext == DXH_CHAIN_FULL || (Lext == DXH_CHAIN_ROW && Rext == DXH_CHAIN_ROW), "an op on row vectors takes row vectors");
#pragma unroll
            for (int u = 0; u < NV; ++u) {
#pragma unroll
                for (int e = 0; e < VW; ++e) {
                    const float a = Lext == DXH_CHAIN_COLUMN ? val[L][0][0] : val[L][u][e];
                    const float b = Rext == DXH_CHAIN_COLUMN ? val[R][0][0] : val[R][u][e];
                    val[me][u][e] = chain_apply<Op::code, Op::dt != kSF32>(a, b, s);
                }
                round_in_place<Op::dt, VW>(val[me][u]);
                if (out && own[u]) {
                    if constexpr (Op::ext == DXH_CHAIN_FULL) {
                        if (row_ok) store_elems_sel<Op::dt, VW>(out, (row * lv + c[u]) * VW, val[me][u], p.nt_store != 0);
                    } else {
                        if (row_raw == 0) store_elems<Op::dt, VW, false>(out, (int64_t)c[u] * VW, val[me][u]);
                    }
                }
            }
        }
    });
}

// ---- flat form: one dtype, every tensor of the same n elements --------------------------------------
template <typename Prog, int DT>
__global__ __launch_bounds__(kBlock) void chain_static_flat_kernel(const StaticArgs p, int64_t nv) {
    constexpr int N = 16 / chain_dtype_bytes(DT);
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= nv) return;
    float in[Prog::n_in][N], res[Prog::n_ops][N];
    static_for<Prog::n_in>([&](auto j_) __attribute__((always_inline)) { load_elems<DT, N>(p.in[decltype(j_)::value], i * N, in[decltype(j_)::value]); });
    eval_flat<Prog, DT, N>(in, res, p.scalar);
    static_for<Prog::n_ops>([&](auto k_) __attribute__((always_inline)) {
        constexpr int k = decltype(k_)::value;
        if (p.out[k]) store_elems_sel<DT, N>(p.out[k], i * N, res[k], p.nt_store != 0);
    });
}

// ---- the programs -------------------------------------------------------------------------------------
namespace {
constexpr int RES = DXH_CHAIN_RESULT, FULL = DXH_CHAIN_FULL, ROW = DXH_CHAIN_ROW, COL = DXH_CHAIN_COLUMN;

// RMSNorm of a 16-bit (or fp32) activation in fp32 with a weight row of the same type, as the batch path sees the front's
// T5LayerNorm (front/py/deepx/nn/modules/norm/t5layernorm.py:17-22) once its tensors exist:
//   xf = todtype(x)  sq = xf^2  var = sum(sq, -1)  var /= cols  var += eps  var = sqrt(var)  var = 1 / var
//   rs = broadcastTo(var)  xn = xf * rs  wf1 = todtype(w)  wf = broadcastTo(wf1)  xn = wf * xn  h = todtype(xn)
template <int HALF>
using RmsNormProg = SProg<SList<SIn<HALF, FULL>, SIn<HALF, ROW>>,
                          SList<SOp<DXH_CHAIN_COPY, 0, 0, kSF32, FULL>, SOp<DXH_CHAIN_SQUARE, RES + 0, 0, kSF32, FULL>, SOp<DXH_CHAIN_ROWSUM, RES + 1, 0, kSF32, COL>,
                                SOp<DXH_CHAIN_DIVSCALAR, RES + 2, 0, kSF32, COL>, SOp<DXH_CHAIN_ADDSCALAR, RES + 3, 0, kSF32, COL>, SOp<DXH_CHAIN_SQRT, RES + 4, 0, kSF32, COL>,
                                SOp<DXH_CHAIN_RDIVSCALAR, RES + 5, 0, kSF32, COL>, SOp<DXH_CHAIN_COPY, RES + 6, 0, kSF32, FULL>, SOp<DXH_CHAIN_MUL, RES + 0, RES + 7, kSF32, FULL>,
                                SOp<DXH_CHAIN_COPY, 1, 0, kSF32, ROW>, SOp<DXH_CHAIN_COPY, RES + 9, 0, kSF32, FULL>, SOp<DXH_CHAIN_MUL, RES + 10, RES + 8, kSF32, FULL>,
                                SOp<DXH_CHAIN_COPY, RES + 11, 0, HALF, FULL>>>;

// softmax over the last axis as the front spells it (front/py/deepx/nn/functional/normalization.py:4-17):
//   m = reducemax(t, -1)  mb = broadcastTo(m)  d = t - mb  e = exp(d)  s = sum(e, -1)  e2 = exp(d)
//   sb = broadcastTo(s)  y = e2 / sb
template <int DT>
using SoftmaxProg = SProg<SList<SIn<DT, FULL>>,
                          SList<SOp<DXH_CHAIN_ROWMAX, 0, 0, DT, COL>, SOp<DXH_CHAIN_COPY, RES + 0, 0, DT, FULL>, SOp<DXH_CHAIN_SUB, 0, RES + 1, DT, FULL>,
                                SOp<DXH_CHAIN_EXP, RES + 2, 0, DT, FULL>, SOp<DXH_CHAIN_ROWSUM, RES + 3, 0, DT, COL>, SOp<DXH_CHAIN_EXP, RES + 2, 0, DT, FULL>,
                                SOp<DXH_CHAIN_COPY, RES + 4, 0, DT, FULL>, SOp<DXH_CHAIN_DIV, RES + 5, RES + 6, DT, FULL>>>;
// the same when the caller reuses the first exp (five lines and two broadcasts)
template <int DT>
using SoftmaxShortProg = SProg<SList<SIn<DT, FULL>>,
                               SList<SOp<DXH_CHAIN_ROWMAX, 0, 0, DT, COL>, SOp<DXH_CHAIN_COPY, RES + 0, 0, DT, FULL>, SOp<DXH_CHAIN_SUB, 0, RES + 1, DT, FULL>,
                                     SOp<DXH_CHAIN_EXP, RES + 2, 0, DT, FULL>, SOp<DXH_CHAIN_ROWSUM, RES + 3, 0, DT, COL>, SOp<DXH_CHAIN_COPY, RES + 4, 0, DT, FULL>,
                                     SOp<DXH_CHAIN_DIV, RES + 3, RES + 5, DT, FULL>>>;

// attention weights as the front computes them (front/py/deepx/nn/modules/transformer/attention.py:15,24): the scores times the
// scaling factor, then the softmax above on the product — one more line in front, a = t * scaling
template <int DT>
using ScaledSoftmaxProg = SProg<SList<SIn<DT, FULL>>,
                                SList<SOp<DXH_CHAIN_MULSCALAR, 0, 0, DT, FULL>, SOp<DXH_CHAIN_ROWMAX, RES + 0, 0, DT, COL>, SOp<DXH_CHAIN_COPY, RES + 1, 0, DT, FULL>,
                                      SOp<DXH_CHAIN_SUB, RES + 0, RES + 2, DT, FULL>, SOp<DXH_CHAIN_EXP, RES + 3, 0, DT, FULL>, SOp<DXH_CHAIN_ROWSUM, RES + 4, 0, DT, COL>,
                                      SOp<DXH_CHAIN_EXP, RES + 3, 0, DT, FULL>, SOp<DXH_CHAIN_COPY, RES + 5, 0, DT, FULL>, SOp<DXH_CHAIN_DIV, RES + 6, RES + 7, DT, FULL>>>;

// SiLU gate of the front's gated MLP (front/py/deepx/nn/functional/activite.py:11-18,
// front/py/deepx/nn/modules/mlp/gatedmlp.py:20-26): sg = -g  sg = exp(sg)  sg += 1  sg = 1 / sg  sg = g * sg  sg *= u
using SiluGateProg = SProg<SList<SIn<0, FULL>, SIn<0, FULL>>,
                           SList<SOp<DXH_CHAIN_MULSCALAR, 0, 0, 0, FULL>, SOp<DXH_CHAIN_EXP, RES + 0, 0, 0, FULL>, SOp<DXH_CHAIN_ADDSCALAR, RES + 1, 0, 0, FULL>,
                                 SOp<DXH_CHAIN_RDIVSCALAR, RES + 2, 0, 0, FULL>, SOp<DXH_CHAIN_MUL, 0, RES + 3, 0, FULL>, SOp<DXH_CHAIN_MUL, RES + 4, 1, 0, FULL>>>;
// SiLU alone: the first five lines of the above
using SiluProg = SProg<SList<SIn<0, FULL>>,
                       SList<SOp<DXH_CHAIN_MULSCALAR, 0, 0, 0, FULL>, SOp<DXH_CHAIN_EXP, RES + 0, 0, 0, FULL>, SOp<DXH_CHAIN_ADDSCALAR, RES + 1, 0, 0, FULL>,
                             SOp<DXH_CHAIN_RDIVSCALAR, RES + 2, 0, 0, FULL>, SOp<DXH_CHAIN_MUL, 0, RES + 3, 0, FULL>>>;
// The same two as swish(x, beta) spells them (activite.py:15-16: x * sigmoid(x * beta), sigmoid(t) = 1 / (exp(t * -1) + 1)):
// one more line in front, t = x * beta
using SwishGateProg = SProg<SList<SIn<0, FULL>, SIn<0, FULL>>,
                            SList<SOp<DXH_CHAIN_MULSCALAR, 0, 0, 0, FULL>, SOp<DXH_CHAIN_MULSCALAR, RES + 0, 0, 0, FULL>, SOp<DXH_CHAIN_EXP, RES + 1, 0, 0, FULL>,
                                  SOp<DXH_CHAIN_ADDSCALAR, RES + 2, 0, 0, FULL>, SOp<DXH_CHAIN_RDIVSCALAR, RES + 3, 0, 0, FULL>, SOp<DXH_CHAIN_MUL, 0, RES + 4, 0, FULL>,
                                  SOp<DXH_CHAIN_MUL, RES + 5, 1, 0, FULL>>>;
using SwishProg = SProg<SList<SIn<0, FULL>>,
                        SList<SOp<DXH_CHAIN_MULSCALAR, 0, 0, 0, FULL>, SOp<DXH_CHAIN_MULSCALAR, RES + 0, 0, 0, FULL>, SOp<DXH_CHAIN_EXP, RES + 1, 0, 0, FULL>,
                              SOp<DXH_CHAIN_ADDSCALAR, RES + 2, 0, 0, FULL>, SOp<DXH_CHAIN_RDIVSCALAR, RES + 3, 0, 0, FULL>, SOp<DXH_CHAIN_MUL, 0, RES + 4, 0, FULL>>>;

// sigmoid on its own (activite.py:10-12): the first four lines of SiluProg
using SigmoidProg = SProg<SList<SIn<0, FULL>>,
                          SList<SOp<DXH_CHAIN_MULSCALAR, 0, 0, 0, FULL>, SOp<DXH_CHAIN_EXP, RES + 0, 0, 0, FULL>, SOp<DXH_CHAIN_ADDSCALAR, RES + 1, 0, 0, FULL>,
                                SOp<DXH_CHAIN_RDIVSCALAR, RES + 2, 0, 0, FULL>>>;

std::atomic<int64_t> g_static_launches{0}, g_interpreted_launches{0};

int dtype_code(int dtype) { return dtype == DXH_F32 ? (int)kSF32 : dtype == DXH_BF16 ? (int)kSBF16 : dtype == DXH_F16 ? (int)kSF16 : -1; }

// does the run-time table spell program Prog?
template <typename Prog>
bool rows_match(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops) {
    if (n_inputs != Prog::n_in || n_ops != Prog::n_ops) return false;
    bool same = true;
    static_for_host<Prog::n_in>([&](auto j_) {
        constexpr int j = decltype(j_)::value;
        using In = typename Prog::ins::template at<j>;
        same = same && dtype_code(inputs[j].dtype) == In::dt && inputs[j].extent == In::ext;
    });
    static_for_host<Prog::n_ops>([&](auto k_) {
        constexpr int k = decltype(k_)::value;
        using Op = typename Prog::ops::template at<k>;
        same = same && ops[k].code == Op::code && ops[k].lhs == Op::lhs && (!chain_code_is_binary(Op::code) || ops[k].rhs == Op::rhs) &&
               dtype_code(ops[k].dtype) == Op::dt && ops[k].extent == Op::ext;
    });
    return same;
}
template <typename Prog>
bool flat_match(int n_inputs, const dxh_chain_op *ops, int n_ops) {
    if (n_inputs != Prog::n_in || n_ops != Prog::n_ops) return false;
    bool same = true;
    static_for_host<Prog::n_ops>([&](auto k_) {
        constexpr int k = decltype(k_)::value;
        using Op = typename Prog::ops::template at<k>;
        same = same && ops[k].code == Op::code && ops[k].lhs == Op::lhs && (!chain_code_is_binary(Op::code) || ops[k].rhs == Op::rhs);
    });
    return same;
}

template <typename Prog, int VW>
int launch_rows(const StaticArgs &a, int64_t rows, int64_t cols, hipStream_t st, bool dry) {
    constexpr int es = prog_reduce_esize<Prog>();
    static_assert(es >= 0, "the row reductions of a program share one element size");
    const int64_t lv = cols / VW;
    int G;
    if (es > 0) {
        G = reduce_rows_group(es, rows, cols);  // the lanes share a row as the separate reduction would
        if (G <= 0) return kNotStatic;
    } else {
        G = 1;
        while (G < kWave && G * 2 <= lv) G <<= 1;
    }
    const int64_t need = (lv + G - 1) / G;
    if (need > 8 || lv > INT32_MAX) return kNotStatic;
    const int rows_per_block = kBlock / G;
    const int64_t blocks = (rows + rows_per_block - 1) / rows_per_block;
    if (blocks > 0x7fffffff) return kNotStatic;
    const unsigned grid = (unsigned)blocks;
    if (dry) return DXH_OK;
    if (need <= 1) chain_static_rows_kernel<Prog, VW, 1><<<grid, kBlock, 0, st>>>(a, rows, (int)lv, G);
    else if (need <= 2) chain_static_rows_kernel<Prog, VW, 2><<<grid, kBlock, 0, st>>>(a, rows, (int)lv, G);
    else if (need <= 4) chain_static_rows_kernel<Prog, VW, 4><<<grid, kBlock, 0, st>>>(a, rows, (int)lv, G);
    else chain_static_rows_kernel<Prog, VW, 8><<<grid, kBlock, 0, st>>>(a, rows, (int)lv, G);
    return launch_status();
}
}  // namespace

void chain_count_interpreted() { g_interpreted_launches.fetch_add(1, std::memory_order_relaxed); }

// The caller (dxh_chain_rows) has validated the table.  Returns kNotStatic when no program fits.
int static_rows_try(const dxh_chain_tensor *inputs, int n_inputs, const dxh_chain_rows_op *ops, int n_ops, int64_t rows, int64_t cols, hipStream_t st, bool dry) {
    if (!tuning().chain_static || rows < 1 || cols < 1) return kNotStatic;
    StaticArgs a{};
    size_t stored = 0;
    for (int j = 0; j < n_inputs; ++j) a.in[j] = inputs[j].data;
    for (int k = 0; k < n_ops; ++k) {
        a.out[k] = ops[k].out;
        if (ops[k].out && ops[k].extent == DXH_CHAIN_FULL) stored += (size_t)rows * (size_t)cols * (ops[k].dtype == DXH_F32 ? 4 : 2);
        const float sf = (float)ops[k].scalar.f;
        a.scalar[k] = ops[k].dtype == DXH_F32 ? sf : ops[k].dtype == DXH_BF16 ? load_acc(to_bf16(sf)) : load_acc(to_f16(sf));
    }
    a.nt_store = use_nt_store(stored);
    // VW elements per lane vector: pointers of [rows, cols] tensors and row vectors must be aligned to it
    auto aligned_to = [&](int vw) {
        if (cols % vw != 0) return false;
        for (int j = 0; j < n_inputs; ++j)
            if (inputs[j].extent != DXH_CHAIN_COLUMN && !aligned(inputs[j].data, (size_t)vw * (inputs[j].dtype == DXH_F32 ? 4 : 2))) return false;
        for (int k = 0; k < n_ops; ++k)
            if (ops[k].out && ops[k].extent != DXH_CHAIN_COLUMN && !aligned(ops[k].out, (size_t)vw * (ops[k].dtype == DXH_F32 ? 4 : 2))) return false;
        return true;
    };
    int rc = kNotStatic;
#define DXH_TRY_ROWS(PROG, VW) if (rc == kNotStatic && rows_match<PROG>(inputs, n_inputs, ops, n_ops) && aligned_to(VW)) rc = launch_rows<PROG, VW>(a, rows, cols, st, dry)
    DXH_TRY_ROWS(RmsNormProg<kSBF16>, 4);
    DXH_TRY_ROWS(RmsNormProg<kSF16>, 4);
    DXH_TRY_ROWS(RmsNormProg<kSF32>, 4);  // a model kept in fp32: the two casts are copies
    DXH_TRY_ROWS(SoftmaxProg<kSF32>, 4);
    DXH_TRY_ROWS(SoftmaxProg<kSBF16>, 8);
    DXH_TRY_ROWS(SoftmaxProg<kSF16>, 8);
    DXH_TRY_ROWS(ScaledSoftmaxProg<kSF32>, 4);
    DXH_TRY_ROWS(ScaledSoftmaxProg<kSBF16>, 8);
    DXH_TRY_ROWS(ScaledSoftmaxProg<kSF16>, 8);
    DXH_TRY_ROWS(SoftmaxShortProg<kSF32>, 4);
    DXH_TRY_ROWS(SoftmaxShortProg<kSBF16>, 8);
    DXH_TRY_ROWS(SoftmaxShortProg<kSF16>, 8);
#undef DXH_TRY_ROWS
    if (rc == DXH_OK && !dry) g_static_launches.fetch_add(1, std::memory_order_relaxed);
    return rc;
}

// The caller (dxh_chain) has validated the table: n a whole number of 16-byte vectors, pointers aligned.
int static_chain_try(int dtype, const void *const *inputs, int n_inputs, const dxh_chain_op *ops, int n_ops, int64_t n, hipStream_t st) {
    const int dt = dtype_code(dtype);
    if (!tuning().chain_static || dt < 0 || n < 1) return kNotStatic;
    StaticArgs a{};
    size_t stored = 0;
    for (int j = 0; j < n_inputs; ++j) a.in[j] = inputs[j];
    for (int k = 0; k < n_ops; ++k) {
        a.out[k] = ops[k].out;
        if (ops[k].out) stored += (size_t)n * chain_dtype_bytes(dt);
        const float sf = (float)ops[k].scalar.f;
        a.scalar[k] = dt == kSF32 ? sf : dt == kSBF16 ? load_acc(to_bf16(sf)) : load_acc(to_f16(sf));
    }
    a.nt_store = use_nt_store(stored);
    const int64_t nv = n / (16 / chain_dtype_bytes(dt)), blocks = (nv + kBlock - 1) / kBlock;
    if (blocks > 0x7fffffff) return kNotStatic;
    int rc = kNotStatic;
#define DXH_TRY_FLAT(PROG)                                                                                                   \
    if (rc == kNotStatic && flat_match<PROG>(n_inputs, ops, n_ops)) {                                                        \
        if (dt == kSF32) chain_static_flat_kernel<PROG, kSF32><<<(unsigned)blocks, kBlock, 0, st>>>(a, nv);                  \
        else if (dt == kSBF16) chain_static_flat_kernel<PROG, kSBF16><<<(unsigned)blocks, kBlock, 0, st>>>(a, nv);           \
        else chain_static_flat_kernel<PROG, kSF16><<<(unsigned)blocks, kBlock, 0, st>>>(a, nv);                              \
        rc = launch_status();                                                                                                \
    }
    DXH_TRY_FLAT(SiluGateProg);
    DXH_TRY_FLAT(SiluProg);
    DXH_TRY_FLAT(SwishGateProg);
    DXH_TRY_FLAT(SwishProg);
    DXH_TRY_FLAT(SigmoidProg);
#undef DXH_TRY_FLAT
    if (rc == DXH_OK) g_static_launches.fetch_add(1, std::memory_order_relaxed);
    return rc;
}

}  // namespace dxh

extern "C" int dxh_chain_stats(int64_t *compiled, int64_t *interpreted) {
    if (!compiled || !interpreted) return DXH_ERR_ARG;
    *compiled = dxh::g_static_launches.load(std::memory_order_relaxed);
    *interpreted = dxh::g_interpreted_launches.load(std::memory_order_relaxed);
    return DXH_OK;
}
