// matmul_fp.hip — fp32 and fp64 GEMM on the matrix pipe: v_mfma_f32_32x32x2_f32 and
// v_mfma_f64_16x16x4_f64, operands and accumulators in the storage type.
#include "matmul_common.hpp"

namespace dxh {

// ---- fp32 MFMA kernel ------------------------------------------------------------------------
// v_mfma_f32_32x32x2_f32 (fp32 operands, fp32 accumulate: 157 TFLOP/s peak, 64 cycles each).  A
// fp32 GEMM on the matrix pipe is compute bound by a wide margin (8x fewer flops per operand
// byte than bf16 at 1/16 of the rate): workgroup tile (64 FM) x (64 FN), K step FK, 4 waves 2x2,
// each wave FM x FN MFMA tiles, two LDS stages, PD K steps held in registers ahead of the stage
// being multiplied.  What keeps the pipe full is the issue order: MFMA operands are read from LDS
// one group (8 k) ahead into a second register buffer, and LDS stores, global loads and those
// reads are pinned between the MFMAs (sched_group_barrier); left alone the compiler reads each
// operand right before its MFMA and the pipe idles for an LDS latency every fourth MFMA.
//   A      LDS [m][FK k] with rows padded by 4 floats; a lane reads the FK/2 consecutive k of its
//          row half with ds_read_b128 (the k order inside a K step is a free permutation as
//          long as both operands use it: MFMA e of lane half h multiplies k = (FK/2) h + e).
//   B      LDS [FK k][n] as loaded, rows padded by 4 floats; one ds_read_b32 per lane and k.
//   roles  MFMA on (B^T, A^T): a result lane holds 4 consecutive n of one row m -> 16-byte stores.
//   MODE   0: element-wise accesses with bounds checks.  1 (VEC): K % 4 == 0, N % 4 == 0 and 16-byte
//          aligned pointers.  2: A and B as in 1, but C has its own pitch ldc and n_store <= N columns
//          (B was zero-padded to N columns) and is stored element by element.
//   VEC    K % 4 == 0, N % 4 == 0 and 16-byte aligned pointers: 16-byte loads and stores with
//          clamped rows/columns; otherwise element-wise accesses with bounds checks.
template <int FM, int FN, int FK, int PD, int MODE>
__global__ __launch_bounds__(kBlock, 2) void matmul_mfma_f32_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                                    float *__restrict__ C, int M, int lda, int N, TileMap map, KSplit ks, int ldc, int n_store) {
    constexpr bool VEC = MODE != 0, EDGE = MODE == 2;
    constexpr int TM = 64 * FM, TN = 64 * FN, FA_ROW = FK + 4, FB_ROW = TN + 4;
    constexpr int STAGE = TM * FA_ROW + FK * FB_ROW;  // floats
    constexpr int CA = FK / 4, CB = TN / 4;           // 16-byte chunks per A row / B row
    constexpr int A_LD = TM * CA / kBlock, B_LD = FK * CB / kBlock;
    constexpr int HK = FK / 2;                        // k values per lane half
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    constexpr int LDS_FLOATS = 2 * STAGE > TM * (TN + 4) ? 2 * STAGE : TM * (TN + 4);  // K-loop stages, then the result tile
    __shared__ __attribute__((aligned(16))) float lds[LDS_FLOATS];
    const TileCoord tc = tile_of_block(map);
    if (!tc.valid) return;
    const int tm = tc.tm, tn = tc.tn;
    // K slice of this workgroup: rows of A keep their pitch lda, K is the length of the slice
    const int slice = tc.batch % ks.splits, kbase = slice * ks.ksub, K = lda - kbase < ks.ksub ? lda - kbase : ks.ksub;
    A += (tc.batch / ks.splits) * (int64_t)M * lda + kbase;
    B += ((tc.batch / ks.splits) * (int64_t)lda + kbase) * N;
    C += tc.batch * (int64_t)M * ldc;
    const int m0 = tm * TM, n0 = tn * TN;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wm = w >> 1, wn = w & 1;

    // per-lane chunks: A (row = id / CA, c = id % CA), B (krow = id / CB, c = id % CB), id = t + 256 i
    f32x4 ra[PD][A_LD], rb[PD][B_LD];
    auto load_global = [&](auto set, int k0) __attribute__((always_inline)) {
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, row = id / CA, kk = k0 + (id % CA) * 4, gm = m0 + row;
            if constexpr (VEC) {
                ra[set][i] = *reinterpret_cast<const f32x4 *>(A + (int64_t)(gm < M ? gm : M - 1) * lda + (kk < K ? kk : 0));
            } else {
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (gm < M && kk + e < K) ? A[(int64_t)gm * lda + kk + e] : 0.f;
                ra[set][i] = v;
            }
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, krow = id / CB, gk = k0 + krow, gn = n0 + (id % CB) * 4;
            if constexpr (VEC) {
                rb[set][i] = *reinterpret_cast<const f32x4 *>(B + (int64_t)(gk < K ? gk : 0) * N + (gn < N ? gn : N - 4));
            } else {
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (gk < K && gn + e < N) ? B[(int64_t)gk * N + gn + e] : 0.f;
                rb[set][i] = v;
            }
        });
    };
    // k0: the K step that register set `set` holds.  MASKED (only the store of a partial last K
    // step): chunks past K were loaded from a clamped address and are zeroed here.  The common
    // path has no select on loaded values: the scheduler would move it to the top of the K step
    // and every step would wait out the full latency of its own prefetch.
    auto store_lds = [&](auto set, auto stage, auto masked, int k0) __attribute__((always_inline)) {
        float *As = lds + decltype(stage)::value * STAGE, *Bs = As + TM * FA_ROW;
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            const bool keep = !decltype(masked)::value || k0 + (id % CA) * 4 < K;
            *reinterpret_cast<f32x4 *>(As + (id / CA) * FA_ROW + (id % CA) * 4) = keep ? ra[set][i] : f32x4{0.f, 0.f, 0.f, 0.f};
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            const bool keep = !decltype(masked)::value || k0 + id / CB < K;
            *reinterpret_cast<f32x4 *>(Bs + (id / CB) * FB_ROW + (id % CB) * 4) = keep ? rb[set][i] : f32x4{0.f, 0.f, 0.f, 0.f};
        });
    };

    f32x16 acc[FM][FN];
    static_for<FM>([&](auto i) __attribute__((always_inline)) {
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
        });
    });
    const int h = lane >> 5, l32 = lane & 31;
    // A K step is multiplied in Q groups of 8 k per lane half (MFMA e of lane half h multiplies
    // k = HK*h + 8q + e; both operands use this order).  The operands of a group sit in one of
    // two register buffers, read from LDS while the previous group is being multiplied.
    constexpr int Q = HK / 8, NMG = FM * FN * 8, NRG = 2 * FM + 8 * FN, NLD = A_LD + B_LD;
    f32x4 fa[2][FM][2];
    float fb[2][FN][8];
    auto read_frags = [&](auto buf, auto stage, auto q) __attribute__((always_inline)) {
        const float *As = lds + decltype(stage)::value * STAGE, *Bs = As + TM * FA_ROW;
        static_for<FM>([&](auto i) __attribute__((always_inline)) {
            const float *p = As + (wm * 32 * FM + 32 * i + l32) * FA_ROW + HK * h + 8 * decltype(q)::value;
            fa[buf][i][0] = *reinterpret_cast<const f32x4 *>(p);
            fa[buf][i][1] = *reinterpret_cast<const f32x4 *>(p + 4);
        });
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int e = 0; e < 8; ++e) fb[buf][j][e] = Bs[(HK * h + 8 * decltype(q)::value + e) * FB_ROW + wn * 32 * FN + 32 * j + l32];
        });
    };
    auto mma = [&](auto buf, auto lo, auto hi) __attribute__((always_inline)) {
        static_for<decltype(hi)::value - decltype(lo)::value>([&](auto x) __attribute__((always_inline)) {
            constexpr int idx = decltype(lo)::value + decltype(x)::value, e = idx / (FM * FN), i = idx % (FM * FN) / FN, j = idx % FN;
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[buf][j][e], fa[buf][i][e >> 2][e & 3], acc[i][j], 0, 0, 0);
        });
    };

    // One K step: LDS stage S is multiplied (its group 0 is already in a fragment buffer); register
    // set R (K step k_store) moves into stage S^1 and is refilled with K step k_load.  The LDS
    // stores and global loads are dealt out between the first half of the last group's MFMAs; the
    // second half runs after the barrier, under the reads of the next stage's group 0.
    auto step = [&](auto S, auto masked, int k_store, int k_load) __attribute__((always_inline)) {
        constexpr int sv = decltype(S)::value;
        const auto R = ic<(PD == 1) ? 0 : sv ^ 1>{};  // register set (kt + 1) % PD
        static_for<Q>([&](auto q) __attribute__((always_inline)) {
            constexpr int qv = decltype(q)::value, cur = (sv * Q + qv) & 1;
            if constexpr (qv + 1 < Q) {
                read_frags(ic<cur ^ 1>{}, S, ic<qv + 1>{});
                mma(ic<cur>{}, ic<0>{}, ic<NMG>{});
                interleave(ic<NMG>{}, ic<NRG>{}, ic<0>{}, ic<0>{});
            } else {
                store_lds(R, ic<sv ^ 1>{}, masked, k_store);
                load_global(R, k_load);
                mma(ic<cur>{}, ic<0>{}, ic<NMG / 2>{});
                interleave(ic<NMG / 2>{}, ic<0>{}, ic<NLD>{}, ic<NLD>{});
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                read_frags(ic<cur ^ 1>{}, ic<sv ^ 1>{}, ic<0>{});
                mma(ic<cur>{}, ic<NMG / 2>{}, ic<NMG>{});
                interleave(ic<NMG - NMG / 2>{}, ic<NRG>{}, ic<0>{}, ic<0>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto last_step = [&](auto S) __attribute__((always_inline)) {  // nothing left to load
        constexpr int sv = decltype(S)::value;
        static_for<Q>([&](auto q) __attribute__((always_inline)) {
            constexpr int qv = decltype(q)::value, cur = (sv * Q + qv) & 1;
            if constexpr (qv + 1 < Q) {
                read_frags(ic<cur ^ 1>{}, S, ic<qv + 1>{});
                mma(ic<cur>{}, ic<0>{}, ic<NMG>{});
                interleave(ic<NMG>{}, ic<NRG>{}, ic<0>{}, ic<0>{});
            } else {
                mma(ic<cur>{}, ic<0>{}, ic<NMG>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // LDS stage (kt & 1) holds K step kt, register set (kt + 1) % PD holds step kt + 1 and is
    // refilled with step kt + 1 + PD once it has moved to LDS.  Steps past the end are clamped
    // onto the last one (loaded, never stored).  Only the store of a partial last K step is masked.
    const int KT = (K + FK - 1) / FK;
    const bool tail = VEC && K % FK != 0;
    auto k_of = [&](int stepno) { return (stepno < KT ? stepno : KT - 1) * FK; };
    load_global(ic<0>{}, 0);
    if (tail && KT == 1) store_lds(ic<0>{}, ic<0>{}, std::true_type{}, 0);
    else store_lds(ic<0>{}, ic<0>{}, std::false_type{}, 0);
    static_for<PD>([&](auto d) __attribute__((always_inline)) { load_global(ic<(decltype(d)::value + 1) % PD>{}, k_of(decltype(d)::value + 1)); });
    __syncthreads();
    read_frags(ic<0>{}, ic<0>{}, ic<0>{});
    const int plain = tail ? KT - 2 : KT - 1;  // steps kt < plain store a full K step
    int kt = 0;
    for (; kt + 1 < plain; kt += 2) {
        step(ic<0>{}, std::false_type{}, (kt + 1) * FK, k_of(kt + 1 + PD));
        step(ic<1>{}, std::false_type{}, (kt + 2) * FK, k_of(kt + 2 + PD));
    }
    if (kt < plain) {
        step(ic<0>{}, std::false_type{}, (kt + 1) * FK, k_of(kt + 1 + PD));
        ++kt;
    }
    if (tail && KT >= 2) {
        if (kt & 1) step(ic<1>{}, std::true_type{}, (kt + 1) * FK, k_of(kt + 1 + PD));
        else step(ic<0>{}, std::true_type{}, (kt + 1) * FK, k_of(kt + 1 + PD));
        ++kt;
    }
    if (kt & 1) last_step(ic<1>{});
    else last_step(ic<0>{});

    // Result lane: row m = lane%32 of its MFMA tile; register group g holds columns 8g + 4h .. +3.
    // The tile goes through LDS (rows padded by 4 floats: the 16 lanes of a ds_write_b128 phase
    // hit 16 different bank quads) so that every global store instruction writes whole rows of
    // the tile: a short-K product is bound by this store stream.
    constexpr int LDC = TN + 4;
    __syncthreads();
    static_for<FM>([&](auto i) __attribute__((always_inline)) {
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
            float *p = lds + (wm * 32 * FM + 32 * i + l32) * LDC + wn * 32 * FN + 32 * j + 4 * h;
#pragma unroll
            for (int g = 0; g < 4; ++g)
                *reinterpret_cast<f32x4 *>(p + 8 * g) = f32x4{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
        });
    });
    __syncthreads();
    if constexpr (VEC && !EDGE) {
#pragma unroll
        for (int i = 0; i < TM * CB / kBlock; ++i) {
            const int id = t + kBlock * i, row = id / CB, col = (id % CB) * 4, gm = m0 + row, gn = n0 + col;
            if (gm < M && gn < N)
                __builtin_nontemporal_store(*reinterpret_cast<const f32x4 *>(lds + row * LDC + col),
                                            reinterpret_cast<f32x4 *>(C + (int64_t)gm * N + gn));
        }
    } else {
#pragma unroll 4
        for (int i = 0; i < TM * TN / kBlock; ++i) {
            const int id = t + kBlock * i, row = id / TN, col = id % TN, gm = m0 + row, gn = n0 + col;
            if (gm < M && gn < n_store) C[(int64_t)gm * ldc + gn] = lds[row * LDC + col];
        }
    }
}

// ---- fp64 MFMA kernel ------------------------------------------------------------------------
// v_mfma_f64_16x16x4_f64 (78.6 TFLOP/s peak, 64 cycles each): lane L supplies A[row L%16][k L/16]
// and B[k L/16][col L%16]; the result lane holds D[4v + L/16][L%16] in register v.  Same plan as
// the fp32 kernel: workgroup tile (64 FM) x (64 FN), K step 16, 4 waves 2x2, each wave
// (2 FM) x (2 FN) MFMA tiles, double-buffered LDS with one K step prefetched in registers.  MFMA e
// of lane class q = L/16 multiplies k = 4q + e, so a lane reads its four A values of a K step as
// two 16-byte LDS loads.  Result rows are contiguous over 16 lanes: plain 8-byte stores coalesce.
typedef double f64x4 __attribute__((ext_vector_type(4)));
typedef double f64x2 __attribute__((ext_vector_type(2)));
template <int FM, int FN, bool VEC>
__global__ __launch_bounds__(kBlock, 2) void matmul_mfma_f64_kernel(const double *__restrict__ A, const double *__restrict__ B,
                                                                    double *__restrict__ C, int M, int lda, int N, TileMap map, KSplit ks, int ldc, int n_store) {
    constexpr int DK = 16, TM = 64 * FM, TN = 64 * FN, DA_ROW = DK + 2, DB_ROW = TN + 4;
    constexpr int STAGE = TM * DA_ROW + DK * DB_ROW;  // doubles
    constexpr int CA = DK / 2, CB = TN / 2;           // 16-byte chunks per A row / B row
    constexpr int A_LD = TM * CA / kBlock, B_LD = DK * CB / kBlock;
    constexpr int RT = 2 * FM, CT = 2 * FN;           // 16x16 MFMA tiles per wave along m and n
    __shared__ __attribute__((aligned(16))) double lds[2 * STAGE];
    const TileCoord tc = tile_of_block(map);
    if (!tc.valid) return;
    const int tm = tc.tm, tn = tc.tn;
    const int slice = tc.batch % ks.splits, kbase = slice * ks.ksub, K = lda - kbase < ks.ksub ? lda - kbase : ks.ksub;  // K slice, as in the fp32 kernel
    A += (tc.batch / ks.splits) * (int64_t)M * lda + kbase;
    B += ((tc.batch / ks.splits) * (int64_t)lda + kbase) * N;
    C += tc.batch * (int64_t)M * ldc;  // ldc = N, n_store = N unless B was zero-padded to N columns for a C of n_store columns
    const int m0 = tm * TM, n0 = tn * TN;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wm = w >> 1, wn = w & 1;

    f64x2 ra[A_LD], rb[B_LD];
    auto load_global = [&](int k0) __attribute__((always_inline)) {
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, row = id / CA, kk = k0 + (id % CA) * 2, gm = m0 + row;
            if constexpr (VEC) {
                ra[i] = *reinterpret_cast<const f64x2 *>(A + (int64_t)(gm < M ? gm : M - 1) * lda + (kk < K ? kk : 0));
            } else {
                f64x2 v;
#pragma unroll
                for (int e = 0; e < 2; ++e) v[e] = (gm < M && kk + e < K) ? A[(int64_t)gm * lda + kk + e] : 0.0;
                ra[i] = v;
            }
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, krow = id / CB, gk = k0 + krow, gn = n0 + (id % CB) * 2;
            if constexpr (VEC) {
                rb[i] = *reinterpret_cast<const f64x2 *>(B + (int64_t)(gk < K ? gk : 0) * N + (gn < N ? gn : N - 2));
            } else {
                f64x2 v;
#pragma unroll
                for (int e = 0; e < 2; ++e) v[e] = (gk < K && gn + e < N) ? B[(int64_t)gk * N + gn + e] : 0.0;
                rb[i] = v;
            }
        });
    };
    // MASKED (only the store of a partial last K step): chunks past K are zeroed (see the fp32 kernel)
    auto store_lds = [&](auto stage, auto masked, int k0) __attribute__((always_inline)) {
        double *As = lds + decltype(stage)::value * STAGE, *Bs = As + TM * DA_ROW;
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            const bool keep = !decltype(masked)::value || k0 + (id % CA) * 2 < K;
            *reinterpret_cast<f64x2 *>(As + (id / CA) * DA_ROW + (id % CA) * 2) = keep ? ra[i] : f64x2{0.0, 0.0};
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            const bool keep = !decltype(masked)::value || k0 + id / CB < K;
            *reinterpret_cast<f64x2 *>(Bs + (id / CB) * DB_ROW + (id % CB) * 2) = keep ? rb[i] : f64x2{0.0, 0.0};
        });
    };

    f64x4 acc[RT][CT];
    static_for<RT>([&](auto i) __attribute__((always_inline)) {
        static_for<CT>([&](auto j) __attribute__((always_inline)) { acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0}; });
    });
    const int q = lane >> 4, l16 = lane & 15;
    // MFMA e of lane quarter q multiplies k = 4q + e.  A K step is multiplied in Q groups of GE
    // e (one e for the 128x128 tile, whose 128 accumulator registers leave room for no more);
    // the operands of a group are read from LDS into one of two register buffers while the
    // previous group is multiplied, and LDS stores / global loads are pinned between the MFMAs, as
    // in the fp32 kernel.
    constexpr int GE = (FM * FN == 4) ? 1 : 2, Q = 4 / GE;
    constexpr int NMG = RT * CT * GE, NRG = RT + GE * CT, NLD = A_LD + B_LD;
    double fa[2][RT][GE], fb[2][CT][GE];
    auto read_frags = [&](auto buf, auto stage, auto g) __attribute__((always_inline)) {
        const double *As = lds + decltype(stage)::value * STAGE, *Bs = As + TM * DA_ROW;
        static_for<RT>([&](auto i) __attribute__((always_inline)) {
            const double *p = As + (wm * 32 * FM + 16 * i + l16) * DA_ROW + 4 * q + GE * decltype(g)::value;
            if constexpr (GE == 2) {
                const f64x2 v = *reinterpret_cast<const f64x2 *>(p);
                fa[buf][i][0] = v[0];
                fa[buf][i][GE - 1] = v[1];
            } else {
                fa[buf][i][0] = *p;
            }
        });
        static_for<CT>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int e = 0; e < GE; ++e) fb[buf][j][e] = Bs[(4 * q + GE * decltype(g)::value + e) * DB_ROW + wn * 32 * FN + 16 * j + l16];
        });
    };
    auto mma = [&](auto buf, auto lo, auto hi) __attribute__((always_inline)) {
        static_for<decltype(hi)::value - decltype(lo)::value>([&](auto x) __attribute__((always_inline)) {
            constexpr int idx = decltype(lo)::value + decltype(x)::value, e = idx / (RT * CT), i = idx % (RT * CT) / CT, j = idx % CT;
            acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[buf][i][e], fb[buf][j][e], acc[i][j], 0, 0, 0);
        });
    };
    // One K step: stage S is multiplied (its group 0 already sits in fragment buffer 0); the
    // register set (K step k_store) moves into stage S^1 and is refilled with K step k_load.
    auto step = [&](auto S, auto masked, int k_store, int k_load) __attribute__((always_inline)) {
        constexpr int sv = decltype(S)::value;
        static_for<Q>([&](auto g) __attribute__((always_inline)) {
            constexpr int gv = decltype(g)::value, cur = gv & 1;  // Q is even
            if constexpr (gv + 1 < Q) {
                read_frags(ic<cur ^ 1>{}, S, ic<gv + 1>{});
                mma(ic<cur>{}, ic<0>{}, ic<NMG>{});
                interleave(ic<NMG>{}, ic<NRG>{}, ic<0>{}, ic<0>{});
            } else {
                store_lds(ic<sv ^ 1>{}, masked, k_store);
                load_global(k_load);
                mma(ic<cur>{}, ic<0>{}, ic<NMG / 2>{});
                interleave(ic<NMG / 2>{}, ic<0>{}, ic<NLD>{}, ic<NLD>{});
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                read_frags(ic<cur ^ 1>{}, ic<sv ^ 1>{}, ic<0>{});
                mma(ic<cur>{}, ic<NMG / 2>{}, ic<NMG>{});
                interleave(ic<NMG - NMG / 2>{}, ic<NRG>{}, ic<0>{}, ic<0>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto last_step = [&](auto S) __attribute__((always_inline)) {
        static_for<Q>([&](auto g) __attribute__((always_inline)) {
            constexpr int gv = decltype(g)::value, cur = gv & 1;
            if constexpr (gv + 1 < Q) {
                read_frags(ic<cur ^ 1>{}, S, ic<gv + 1>{});
                mma(ic<cur>{}, ic<0>{}, ic<NMG>{});
                interleave(ic<NMG>{}, ic<NRG>{}, ic<0>{}, ic<0>{});
            } else {
                mma(ic<cur>{}, ic<0>{}, ic<NMG>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // Stage (kt & 1) holds K step kt and the register set holds step kt + 1, refilled with step
    // kt + 2 once it has moved to LDS (steps past the end are clamped onto the last one: loaded,
    // never stored).  Only the store of a partial last K step is masked.
    const int KT = (K + DK - 1) / DK;
    const bool tail = VEC && K % DK != 0;
    auto k_of = [&](int stepno) { return (stepno < KT ? stepno : KT - 1) * DK; };
    load_global(0);
    if (tail && KT == 1) store_lds(ic<0>{}, std::true_type{}, 0);
    else store_lds(ic<0>{}, std::false_type{}, 0);
    load_global(k_of(1));
    __syncthreads();
    read_frags(ic<0>{}, ic<0>{}, ic<0>{});
    const int plain = tail ? KT - 2 : KT - 1;  // steps kt < plain store a full K step
    int kt = 0;
    for (; kt + 1 < plain; kt += 2) {
        step(ic<0>{}, std::false_type{}, (kt + 1) * DK, k_of(kt + 2));
        step(ic<1>{}, std::false_type{}, (kt + 2) * DK, k_of(kt + 3));
    }
    if (kt < plain) {
        step(ic<0>{}, std::false_type{}, (kt + 1) * DK, k_of(kt + 2));
        ++kt;
    }
    if (tail && KT >= 2) {
        if (kt & 1) step(ic<1>{}, std::true_type{}, (kt + 1) * DK, k_of(kt + 2));
        else step(ic<0>{}, std::true_type{}, (kt + 1) * DK, k_of(kt + 2));
        ++kt;
    }
    if (kt & 1) last_step(ic<1>{});
    else last_step(ic<0>{});

    static_for<RT>([&](auto i) __attribute__((always_inline)) {
        static_for<CT>([&](auto j) __attribute__((always_inline)) {
            const int gn = n0 + wn * 32 * FN + 16 * j + l16;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int gm = m0 + wm * 32 * FM + 16 * i + 4 * v + q;
                if (gm < M && gn < n_store) __builtin_nontemporal_store(acc[i][j][v], C + (int64_t)gm * ldc + gn);
            }
        });
    });
}

// Launch of one tile shape, cut along K when choose_ksplit says so: the slices then write fp32 /
// fp64 partial tiles into the call's scratch and splitk_reduce_kernel adds them up.
// may_split = false: C has a pitch of its own (the slices' partial tiles and their sum assume [M][N]).
template <typename T, typename Launch>
int launch_fp_tile(Launch launch, int tm, int tn, int kstep, int64_t min_k, T *c, int64_t batch, int64_t m, int64_t k, int64_t n, bool may_split, hipStream_t st, Scratch &sc) {
    const int64_t tiles = batch * ((m + tm - 1) / tm) * ((n + tn - 1) / tn), partial = batch * m * n * (int64_t)sizeof(T);
    const KSplit ks = may_split ? choose_ksplit(tiles, k, kstep, min_k, partial) : KSplit{1, (int)k};
    TileMap map;
    if (!make_tile_map(batch * ks.splits, m, n, tm, tn, map)) return DXH_ERR_SHAPE;
    const unsigned blocks = (unsigned)(8 * map.chunk);
    if (ks.splits == 1) {
        if (sc.planning) return DXH_OK;
        launch(blocks, c, map, ks);
        return launch_status();
    }
    T *ws = (T *)sc.take((size_t)(partial * ks.splits));
    if (!ws) return DXH_ERR_WORKSPACE;
    if (sc.planning) return DXH_OK;
    launch(blocks, ws, map, ks);
    const int rc = launch_status();
    return rc != DXH_OK ? rc : launch_splitk_reduce<T, T>(ws, c, batch, m * n, ks.splits, st);
}

// ldc < 0: C is [M][N].  ldc >= 0 (vec only): C has ldc columns at pitch ldc, B was zero-padded to N columns.
template <int FM, int FN, int FK, int PD>
int launch_f32_tile(const float *a, const float *b, float *c, int64_t batch, int64_t m, int64_t k, int64_t n, bool vec, int64_t ldc, hipStream_t st, Scratch &sc) {
    return launch_fp_tile<float>([&](unsigned blocks, float *out, const TileMap &map, KSplit ks) {
        if (ldc >= 0) matmul_mfma_f32_kernel<FM, FN, FK, PD, 2><<<blocks, kBlock, 0, st>>>(a, b, out, (int)m, (int)k, (int)n, map, ks, (int)ldc, (int)ldc);
        else if (vec) matmul_mfma_f32_kernel<FM, FN, FK, PD, 1><<<blocks, kBlock, 0, st>>>(a, b, out, (int)m, (int)k, (int)n, map, ks, (int)n, (int)n);
        else matmul_mfma_f32_kernel<FM, FN, FK, PD, 0><<<blocks, kBlock, 0, st>>>(a, b, out, (int)m, (int)k, (int)n, map, ks, (int)n, (int)n);
    }, 64 * FM, 64 * FN, FK, 1024, c, batch, m, k, n, ldc < 0, st, sc);
}

// fp32: the matrix pipe is the bound, so the tile is chosen for CU balance.  Cost model per tile
// shape, in microseconds: two workgroups share a CU, a round of two workgroups per CU takes a fixed
// 3 us (first loads, result stores) plus K times the tile's time per k (0.118 us for 128x128 on
// 4096^3; 128x64 and 64x64 run at 0.96 and 0.90 of that rate per flop), and a last round that
// leaves at most one workgroup per CU counts 0.5 (a lone workgroup has the matrix pipe to itself).
// Small tiles take longer K steps and a deeper prefetch: with few MFMAs per step only that hides
// the global-load latency.
static int launch_matmul_f32_at(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, int64_t ldc, hipStream_t st, Scratch &sc);
int launch_matmul_f32(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    return launch_matmul_f32_at(a, b, c, batch, m, k, n, -1, st, sc);
}
// ldc >= 0: called on zero-padded copies of A and B; C then has ldc columns at pitch ldc
static int launch_matmul_f32_at(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, int64_t ldc, hipStream_t st, Scratch &sc) {
    const bool vec = k % 4 == 0 && n % 4 == 0 && n >= 4 && aligned(a, kVecBytes) && aligned(b, kVecBytes) && (ldc >= 0 || aligned(c, kVecBytes));
    if (ldc >= 0 && !vec) return DXH_ERR_ALIGN;
    const int64_t cus = compute_units();
    auto cost = [&](int tm, int tn, double eff) {
        const int64_t tiles = batch * ((m + tm - 1) / tm) * ((n + tn - 1) / tn);
        const int64_t full = tiles / (2 * cus), rem = tiles % (2 * cus);
        const double rounds = (double)full + (rem > cus ? 1.0 : rem > 0 ? 0.5 : 0.0);
        return rounds * (3.0 + (double)k * 0.1183 * (double)(tm * tn) / (128.0 * 128.0) / eff);
    };
    if (!vec && tuning().matmul_tile == 0) {  // odd K / N or unaligned bases: the vector path on zero-padded copies
        const int rc = launch_on_padded_copies<uint32_t>(
            [&](const void *pa, const void *pb, void *pc, int64_t pk, int64_t pn, int64_t pitch) { return launch_matmul_f32_at(pa, pb, pc, batch, m, pk, pn, pitch, st, sc); },
            a, b, c, batch, m, k, n, st, sc);
        if (rc != kNoSplit) return rc;
    }
    const float *af = (const float *)a, *bf = (const float *)b;
    float *cf = (float *)c;
    int64_t choice = tuning().matmul_tile;
    if (choice == 0) {
        const double c1 = cost(128, 128, 1.0), c2 = cost(128, 64, 0.957), c3 = cost(64, 64, 0.897);
        choice = (c1 <= c2 && c1 <= c3) ? 1 : (c2 <= c3) ? 2 : 3;
    }
    switch (choice) {
    case 1: return launch_f32_tile<2, 2, 32, 1>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    case 2: return launch_f32_tile<2, 1, 32, 2>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    case 3: return launch_f32_tile<1, 1, 64, 2>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    case 4: return launch_f32_tile<2, 2, 16, 1>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    default: return launch_f32_tile<1, 1, 64, 2>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    }
}

template <int FM, int FN>
int launch_f64_tile(const double *a, const double *b, double *c, int64_t batch, int64_t m, int64_t k, int64_t n, bool vec, int64_t ldc, hipStream_t st, Scratch &sc) {
    const int pitch = (int)(ldc >= 0 ? ldc : n);
    return launch_fp_tile<double>([&](unsigned blocks, double *out, const TileMap &map, KSplit ks) {
        if (vec) matmul_mfma_f64_kernel<FM, FN, true><<<blocks, kBlock, 0, st>>>(a, b, out, (int)m, (int)k, (int)n, map, ks, pitch, pitch);
        else matmul_mfma_f64_kernel<FM, FN, false><<<blocks, kBlock, 0, st>>>(a, b, out, (int)m, (int)k, (int)n, map, ks, pitch, pitch);
    }, 64 * FM, 64 * FN, 16, 512, c, batch, m, k, n, ldc < 0, st, sc);
}

// fp64 on the matrix pipe; tile chosen for CU balance with the fp32 cost model (0.116 us per k for
// a round of 128x64 tiles on 4096^3, 64x64 at 0.94 of that rate per flop).  The 128x128 tile is
// not chosen: its 128 accumulator registers leave too few for the operand buffers and it runs
// behind 128x64 on every shape tried; the tuning knob still selects it.
static int launch_matmul_f64_at(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, int64_t ldc, hipStream_t st, Scratch &sc);
int launch_matmul_f64(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    return launch_matmul_f64_at(a, b, c, batch, m, k, n, -1, st, sc);
}
static int launch_matmul_f64_at(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, int64_t ldc, hipStream_t st, Scratch &sc) {
    const bool vec = k % 2 == 0 && n % 2 == 0 && n >= 2 && aligned(a, kVecBytes) && aligned(b, kVecBytes);
    if (ldc >= 0 && !vec) return DXH_ERR_ALIGN;
    const int64_t cus = compute_units();
    auto cost = [&](int tm, int tn, double eff) {
        const int64_t tiles = batch * ((m + tm - 1) / tm) * ((n + tn - 1) / tn);
        const int64_t full = tiles / (2 * cus), rem = tiles % (2 * cus);
        const double rounds = (double)full + (rem > cus ? 1.0 : rem > 0 ? 0.5 : 0.0);
        return rounds * (3.0 + (double)k * 0.1163 * (double)(tm * tn) / (128.0 * 64.0) / eff);
    };
    if (!vec && tuning().matmul_tile == 0) {  // odd K / N or unaligned bases: the vector path on zero-padded copies
        const int rc = launch_on_padded_copies<uint64_t>(
            [&](const void *pa, const void *pb, void *pc, int64_t pk, int64_t pn, int64_t pitch) { return launch_matmul_f64_at(pa, pb, pc, batch, m, pk, pn, pitch, st, sc); },
            a, b, c, batch, m, k, n, st, sc);
        if (rc != kNoSplit) return rc;
    }
    const double *af = (const double *)a, *bf = (const double *)b;
    double *cf = (double *)c;
    int64_t choice = tuning().matmul_tile;
    if (choice == 0) {
        choice = cost(128, 64, 1.0) <= cost(64, 64, 0.941) ? 2 : 3;
    }
    switch (choice) {
    case 1: return launch_f64_tile<2, 2>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    case 2: return launch_f64_tile<2, 1>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    default: return launch_f64_tile<1, 1>(af, bf, cf, batch, m, k, n, vec, ldc, st, sc);
    }
}

}  // namespace dxh
