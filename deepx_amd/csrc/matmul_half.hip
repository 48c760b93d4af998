// matmul_half.hip — bf16 / f16 GEMM on the matrix pipe (v_mfma_f32_32x32x16_{bf16,f16}, fp32
// accumulate, one RNE rounding of C).  Aligned shapes (K % 8 == 0, N % 8 == 0) take
// matmul_mfma_tile_kernel, 64x64 to 256x256 workgroup tiles, software-pipelined over K, cut along
// K when the output has few tiles; other shapes run the same kernel on zero-padded copies, or,
// when those would not fit the scratch limit, matmul_mfma_kernel, a plain 128x128x32 tile with
// element-wise edge handling.
#include "matmul_half_ops.hpp"

namespace dxh {

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int LDK = BK + 8;  // padded k-stride (elements) of both LDS tiles: 80 bytes, keeps 16-byte alignment


// VEC_A: rows of A are 16-byte aligned (K % 8 == 0, base aligned); VEC_B likewise for B (N % 8 == 0).
template <typename T, bool VEC_A, bool VEC_B>
__global__ __launch_bounds__(kBlock) void matmul_mfma_kernel(const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C,
                                                              int M, int K, int N, int tiles_m, int tiles_n) {
    __shared__ __attribute__((aligned(16))) uint16_t As[BM * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[BN * LDK];  // transposed: [n][k]
    int64_t bid = blockIdx.x;
    const int tn = (int)(bid % tiles_n); bid /= tiles_n;
    const int tm = (int)(bid % tiles_m); bid /= tiles_m;
    const int64_t batch = bid;
    A += batch * (int64_t)M * K;
    B += batch * (int64_t)K * N;
    C += batch * (int64_t)M * N;
    const int m0 = tm * BM, n0 = tn * BN;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6;
    const int wm = w >> 1, wn = w & 1;
    const uint16_t *Ar = reinterpret_cast<const uint16_t *>(A);
    const uint16_t *Br = reinterpret_cast<const uint16_t *>(B);

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    for (int k0 = 0; k0 < K; k0 += BK) {
        // ---- A tile: 128 rows x 32 k, 16 bytes (8 k) per lane, two rows per lane
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int r = (t >> 2) + h * 64, kc = (t & 3) * 8;
            const int gm = m0 + r, gk = k0 + kc;
            vec_t<uint16_t, 8> x;
            if (VEC_A && gm < M && gk + 8 <= K) {
                x = *reinterpret_cast<const vec_t<uint16_t, 8> *>(Ar + (int64_t)gm * K + gk);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) x.v[j] = (gm < M && gk + j < K) ? Ar[(int64_t)gm * K + gk + j] : (uint16_t)0;
            }
            *reinterpret_cast<vec_t<uint16_t, 8> *>(&As[r * LDK + kc]) = x;
        }
        // ---- B tile: 32 k x 128 n, 16 bytes (8 n) per lane, transposed into Bs[n][k]
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int kr = (t >> 4) + h * 16, nc = (t & 15) * 8;
            const int gk = k0 + kr, gn = n0 + nc;
            vec_t<uint16_t, 8> x;
            if (VEC_B && gk < K && gn + 8 <= N) {
                x = *reinterpret_cast<const vec_t<uint16_t, 8> *>(Br + (int64_t)gk * N + gn);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j) x.v[j] = (gk < K && gn + j < N) ? Br[(int64_t)gk * N + gn + j] : (uint16_t)0;
            }
#pragma unroll
            for (int j = 0; j < 8; ++j) Bs[(nc + j) * LDK + kr] = x.v[j];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            uint4 af[2], bf[2];
            const int ko = kk + (lane >> 5) * 8;
#pragma unroll
            for (int i = 0; i < 2; ++i) af[i] = *reinterpret_cast<const uint4 *>(&As[(wm * 64 + i * 32 + (lane & 31)) * LDK + ko]);
#pragma unroll
            for (int j = 0; j < 2; ++j) bf[j] = *reinterpret_cast<const uint4 *>(&Bs[(wn * 64 + j * 32 + (lane & 31)) * LDK + ko]);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = mfma32<T>(af[i], bf[j], acc[i][j]);
        }
        __syncthreads();
    }
    // ---- epilogue: D[row][col], col = lane%32, row = 8*(v/4) + 4*(lane/32) + v%4
    uint16_t *Cr = reinterpret_cast<uint16_t *>(C);
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * 64 + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                const int col = n0 + wn * 64 + j * 32 + (lane & 31);
                if (row < M && col < N) Cr[(int64_t)row * N + col] = store_acc<T>(acc[i][j][v]).bits;
            }
}

constexpr int PK = 64;  // K step of the MFMA tile kernel
__device__ inline int swz(int row, int chunk) { return chunk ^ ((row ^ (row >> 3)) & 7); }

// ---- MFMA kernel with the B transposition done by the LDS read ------------------------------
// Workgroup tile TM x TN (TM a multiple of 64, TN 64, 128 or 256), K step 64, 4 waves in a 2x2 grid, each wave a
// (TM/2) x (TN/2) patch of 32x32x16 MFMAs.  Requirements (checked by the launcher): K % 8 == 0,
// N % 8 == 0, 16-byte aligned A, B, C.  KTAIL (K % 64 != 0): chunks of A and rows of B at k >= K
// are read from clamped addresses and replaced by zeros.
//   loads  every global load is 16 bytes per lane (a wave instruction occupies the vector cache for
//          the same 16 cycles whatever its width, so 8-byte loads halve its throughput).
//   A      [TM m][64 k] in LDS, 128-byte rows, 16-byte chunk c of row r at chunk c ^ swizzle(r).
//   B      stays n-contiguous in LDS, [64 k][TN n] with rows padded by 64 bytes; the MFMA operand
//          (8 consecutive k of one column per lane) is assembled by two ds_read_b64_tr_b16.
//   pipe   PD (1 or 2) K steps in flight in registers, two LDS stages, one barrier per K step; the stores
//          into the next stage and the global loads are spread over the four k-substeps.
//   roles  the MFMA runs on (B^T, A^T): a lane of the result then holds 4 consecutive n of one row
//          m, which packs into 8-byte LDS stores for the epilogue.
//   map    blockIdx -> tile through tile_of_block (XCD-aware, above).
// the `count` loads of a K step are dealt out over its four k-substeps
constexpr int part_first(int count, int part) { return count * part / 4; }
constexpr int part_count(int count, int part) { return count * (part + 1) / 4 - count * part / 4; }

template <typename T, int TM, int TN, int PD, bool KTAIL, int MODE>
__global__ __launch_bounds__(kBlock, (TM * TN <= 128 * 128) ? 2 : 1) void matmul_mfma_tile_kernel(
    const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C, float *__restrict__ partial, int M, int lda, int N, TileMap map, KSplit ks,
    int ldc, int n_store, int c_through) {
    // MODE 0: C[M][N] in 16-byte row pieces.  1 (SPLIT): fp32 partial tile of a K slice.  2 (EDGE): C has
    // its own pitch ldc and n_store <= N columns (B was zero-padded to N columns): rows of C are not
    // 16-byte aligned, so the tile is stored element by element.
    constexpr bool SPLIT = MODE == 1, EDGE = MODE == 2;
    static_assert(TM % 64 == 0 && (TN == 64 || TN == 128 || TN == 256), "B rows must split evenly over the 256 lanes");
    constexpr int FM = TM / 64, FN = TN / 64;      // 32x32 MFMA tiles per wave along m and n
    constexpr int A_LD = TM / 32, B_LD = TN / 32;  // 16-byte global loads per lane per K step
    constexpr int CB = TN / 8;                     // 16-byte chunks per B row
    constexpr int KR = kBlock / CB;                // B rows covered by one load of the workgroup
    constexpr int B_ROW = TN + 32;                 // elements per k-row of the B stage (64-byte pad)
    constexpr int A_STAGE = TM * PK, STAGE = A_STAGE + PK * B_ROW;
    constexpr int LDC = TN + 8;
    constexpr int LDS_ELEMS = (2 * STAGE > TM * LDC) ? 2 * STAGE : TM * LDC;
    __shared__ __attribute__((aligned(16))) uint16_t lds[LDS_ELEMS];

    const TileCoord tc = tile_of_block(map);
    if (!tc.valid) return;
    // SPLIT: the workgroup multiplies K slice tc.batch % splits of batch tc.batch / splits (rows of
    // A keep their pitch lda, K is the slice length) and stores an fp32 partial tile.
    const int batch = SPLIT ? tc.batch / ks.splits : tc.batch, tm = tc.tm, tn = tc.tn;
    const int kbase = SPLIT ? (tc.batch % ks.splits) * ks.ksub : 0, K = SPLIT ? (lda - kbase < ks.ksub ? lda - kbase : ks.ksub) : lda;
    const int m0 = tm * TM, n0 = tn * TN;

    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wm = w >> 1, wn = w & 1;
    const uint16_t *Ab = reinterpret_cast<const uint16_t *>(A) + ((int64_t)batch * M + m0) * lda + kbase;
    const uint16_t *Bb = reinterpret_cast<const uint16_t *>(B) + ((int64_t)batch * lda + kbase) * N + n0;

    // Branch-free loads: rows past M and columns past N are clamped onto valid memory; their
    // products land in accumulator rows/columns that the epilogue never stores.
    const int arow = t >> 3, ach = t & 7;
    int a_off[A_LD], a_lds[A_LD];
    static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
        const int r = arow + 32 * i;
        a_off[i] = (m0 + r < M ? r : M - 1 - m0) * lda + ach * 8;
        a_lds[i] = r * PK + swz(r, ach) * 8;
    });
    const int brow = t / CB, bch = t % CB;
    const int b_col = n0 + bch * 8 < N ? bch * 8 : N - 8 - n0, b_off = brow * N + b_col;
    const int b_lds = brow * B_ROW + bch * 8;

    u32x4 ra[PD][A_LD], rb[PD][B_LD];
    auto load_part = [&](auto set, auto part, int k0) __attribute__((always_inline)) {
        static_for<part_count(A_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(A_LD, decltype(part)::value) + decltype(q)::value;
            if constexpr (KTAIL) {
                ra[set][i] = *reinterpret_cast<const u32x4 *>(Ab + a_off[i] + (k0 + ach * 8 < K ? k0 : K - 8 - ach * 8));
            } else {
                ra[set][i] = *reinterpret_cast<const u32x4 *>(Ab + a_off[i] + k0);
            }
        });
        static_for<part_count(B_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(B_LD, decltype(part)::value) + decltype(q)::value;
            if constexpr (KTAIL) {
                const int gk = k0 + brow + i * KR;
                rb[set][i] = *reinterpret_cast<const u32x4 *>(Bb + (int64_t)(gk < K ? gk : K - 1) * N + b_col);
            } else {
                rb[set][i] = *reinterpret_cast<const u32x4 *>(Bb + (int64_t)(k0 + i * KR) * N + b_off);
            }
        });
    };
    // k0: the K step that register set `set` holds.  The zero fill of a partial K step happens
    // here and not at the load, so that nothing waits for a load right after issuing it.
    auto store_part = [&](auto set, auto part, auto stage, auto masked, int k0) __attribute__((always_inline)) {
        uint16_t *As = lds + decltype(stage)::value * STAGE, *Bs = As + A_STAGE;
        static_for<part_count(A_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(A_LD, decltype(part)::value) + decltype(q)::value;
            if constexpr (KTAIL && decltype(masked)::value)
                *reinterpret_cast<u32x4 *>(As + a_lds[i]) = k0 + ach * 8 < K ? ra[set][i] : u32x4{0u, 0u, 0u, 0u};
            else
                *reinterpret_cast<u32x4 *>(As + a_lds[i]) = ra[set][i];
        });
        static_for<part_count(B_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(B_LD, decltype(part)::value) + decltype(q)::value;
            if constexpr (KTAIL && decltype(masked)::value)
                *reinterpret_cast<u32x4 *>(Bs + b_lds + i * KR * B_ROW) = k0 + brow + i * KR < K ? rb[set][i] : u32x4{0u, 0u, 0u, 0u};
            else
                *reinterpret_cast<u32x4 *>(Bs + b_lds + i * KR * B_ROW) = rb[set][i];
        });
    };

    // fragment registers, double-buffered over the k-substeps
    u32x4 fa[2][FM], fb[2][FN];
    const int fa_row = wm * (TM / 2) + (lane & 31), fch = lane >> 5;
    const int fb_off = (8 * fch + ((lane & 15) >> 2)) * B_ROW + wn * (TN / 2) + (lane & 16) + 4 * (lane & 3);
    auto read_frags = [&](auto buf, auto stage, auto ks) __attribute__((always_inline)) {
        const uint16_t *As = lds + decltype(stage)::value * STAGE, *Bs = As + A_STAGE;
        static_for<FM>([&](auto i) __attribute__((always_inline)) {
            const int row = fa_row + 32 * i, ch = decltype(ks)::value * 2 + fch;
            fa[buf][i] = *reinterpret_cast<const u32x4 *>(As + row * PK + swz(row, ch) * 8);
        });
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
            const uint16_t *p = Bs + fb_off + decltype(ks)::value * 16 * B_ROW + 32 * j;
            const u32x2 lo = lds_read_tr16(p), hi = lds_read_tr16(p + 4 * B_ROW);
            fb[buf][j] = u32x4{lo.x, lo.y, hi.x, hi.y};
        });
    };

    f32x16 acc[FM][FN];
    static_for<FM>([&](auto i) __attribute__((always_inline)) {
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
        });
    });
    constexpr int NM = FM * FN;                                 // MFMAs per k-substep
    constexpr int ND = FM + 2 * FN;                             // LDS fragment reads per substep
    auto mma = [&](auto buf, auto lo, auto hi) __attribute__((always_inline)) {
        static_for<decltype(hi)::value - decltype(lo)::value>([&](auto x) __attribute__((always_inline)) {
            constexpr int idx = decltype(lo)::value + decltype(x)::value, i = idx / FN, j = idx % FN;
            acc[i][j] = mfma32<T>(fb[buf][j], fa[buf][i], acc[i][j]);
        });
    };

    // One K step: LDS stage S is multiplied; register set R (the next K step) moves into stage
    // S^1 and is refilled with the K step PD further on.  Fragment buffer 0 holds substep 0 on
    // entry.  The last substep straddles the barrier: half of its MFMAs are queued before it and
    // the other half runs under the first fragment reads of stage S^1.
    auto step = [&](auto S, auto masked, int k_store, int k_load) __attribute__((always_inline)) {
        constexpr int s = decltype(S)::value;
        const auto R = ic<(PD == 1) ? 0 : s ^ 1>{};  // register set (kt + 1) % PD
        static_for<4>([&](auto ks) __attribute__((always_inline)) {
            constexpr int cur = decltype(ks)::value & 1;
            constexpr int NW = part_count(A_LD, decltype(ks)::value) + part_count(B_LD, decltype(ks)::value);  // LDS writes = global loads
            if constexpr (decltype(ks)::value < 3) {
                read_frags(ic<cur ^ 1>{}, S, ic<decltype(ks)::value + 1>{});
                store_part(R, ks, ic<s ^ 1>{}, masked, k_store);
                load_part(R, ks, k_load);
                mma(ic<cur>{}, ic<0>{}, ic<NM>{});
                interleave(ic<NM>{}, ic<ND>{}, ic<NW>{}, ic<NW>{});
            } else {
                store_part(R, ks, ic<s ^ 1>{}, masked, k_store);
                load_part(R, ks, k_load);
                mma(ic<cur>{}, ic<0>{}, ic<NM / 2>{});
                interleave(ic<NM / 2>{}, ic<0>{}, ic<NW>{}, ic<NW>{});
                __builtin_amdgcn_sched_barrier(0);
                __syncthreads();
                read_frags(ic<cur ^ 1>{}, ic<s ^ 1>{}, ic<0>{});
                mma(ic<cur>{}, ic<NM / 2>{}, ic<NM>{});
                interleave(ic<NM - NM / 2>{}, ic<ND>{}, ic<0>{}, ic<0>{});
            }
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    const int KT = (K + PK - 1) / PK;
    // c_through bit 1: the K steps are walked from a starting step of the tile's own, wrapping round (see launch_tile)
    int rot = 0;
    if constexpr (!KTAIL && !SPLIT) rot = (c_through & 2) ? (int)(((int64_t)batch * map.tiles_m + tm) % KT) : 0;
    auto k_of = [&](int stepno) __attribute__((always_inline)) {
        int s = (stepno < KT ? stepno : KT - 1) + rot;
        return (s >= KT ? s - KT : s) * PK;
    };
    static_for<4>([&](auto part) __attribute__((always_inline)) { load_part(ic<0>{}, part, k_of(0)); });
    static_for<4>([&](auto part) __attribute__((always_inline)) { store_part(ic<0>{}, part, ic<0>{}, std::true_type{}, 0); });
    static_for<PD>([&](auto d) __attribute__((always_inline)) { static_for<4>([&](auto part) __attribute__((always_inline)) { load_part(ic<(decltype(d)::value + 1) % PD>{}, part, k_of(decltype(d)::value + 1)); }); });
    __syncthreads();
    read_frags(ic<0>{}, ic<0>{}, ic<0>{});
    // KTAIL kernels mask every store: peeling the two steps that need it costs more registers
    // than the tile sizes with 128 and more accumulator registers have left.
    const auto masked = std::integral_constant<bool, KTAIL>{};
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
        step(ic<0>{}, masked, k_of(kt + 1), k_of(kt + 1 + PD));
        step(ic<1>{}, masked, k_of(kt + 2), k_of(kt + 2 + PD));
    }
    if (kt < KT) step(ic<0>{}, masked, k_of(kt + 1), k_of(kt + 1 + PD));
    if constexpr (SPLIT) {
        // fp32 partial tile straight from the accumulators: 16 bytes (4 consecutive n) per store
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        float *P = partial + (int64_t)tc.batch * M * N;
        static_for<FM>([&](auto i) __attribute__((always_inline)) {
            static_for<FN>([&](auto j) __attribute__((always_inline)) {
                const int gm = m0 + wm * (TM / 2) + 32 * i + (lane & 31);
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int gn = n0 + wn * (TN / 2) + 32 * j + 8 * g + 4 * (lane >> 5);
                    if (gm < M && gn < N)  // N % 8 == 0: four columns are inside or outside together
                        *reinterpret_cast<f32x4 *>(P + (int64_t)gm * N + gn) = f32x4{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
                }
            });
        });
        return;
    }
    __syncthreads();

    // ---- epilogue: result lane holds row m = lane%32 of its MFMA tile and, per group g of 4
    // registers, columns 8g + 4*(lane/32) .. +3: one 8-byte LDS store each, then 16-byte row stores
    uint16_t *Cs = lds;
    static_for<FM>([&](auto i) __attribute__((always_inline)) {
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int row = wm * (TM / 2) + 32 * i + (lane & 31);
                const int col = wn * (TN / 2) + 32 * j + 8 * g + 4 * (lane >> 5);
                *reinterpret_cast<u32x2 *>(Cs + row * LDC + col) =
                    u32x2{pack2<T>(acc[i][j][4 * g], acc[i][j][4 * g + 1]), pack2<T>(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3])};
            }
        });
    });
    __syncthreads();
    uint16_t *Cr = reinterpret_cast<uint16_t *>(C) + (int64_t)batch * M * (EDGE ? ldc : N);
    if constexpr (EDGE) {
        // consecutive lanes along a row, one element each: every store instruction writes runs of
        // contiguous bytes whatever the alignment of the row
#pragma unroll 8
        for (int i = 0; i < TM * TN / kBlock; ++i) {
            const int c = t + i * kBlock, row = c / TN, col = c % TN;
            const int gm = m0 + row, gn = n0 + col;
            if (gm < M && gn < n_store) Cr[(int64_t)gm * ldc + gn] = Cs[row * LDC + col];
        }
    } else {
#pragma unroll
        for (int i = 0; i < TM * CB / kBlock; ++i) {
            const int c = t + i * kBlock, row = c / CB, ch = c % CB;
            const int gm = m0 + row, gn = n0 + ch * 8;
            if (gm < M && gn < N) {  // N % 8 == 0: a chunk is either fully inside or fully outside
                uint4 *dst = reinterpret_cast<uint4 *>(Cr + (int64_t)gm * N + gn);
                const uint4 piece = *reinterpret_cast<const uint4 *>(Cs + row * LDC + ch * 8);
                if (c_through & 1) st_mode<2>(dst, piece); else st_nt(dst, piece);
            }
        }
    }
}

// ldc < 0: C is [M][N] and 16-byte aligned.  ldc >= 0 (needs K % 64 == 0): C has pitch ldc and ldc columns.
template <typename T, int TM, int TN, int PD>
int launch_tile(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, int64_t ldc, hipStream_t st, Scratch &sc) {
    if (sc.planning) return DXH_OK;  // needs no scratch
    TileMap map;
    if (!make_tile_map(batch, m, n, TM, TN, map)) return DXH_ERR_SHAPE;
    const KSplit one{1, (int)k};
    if (ldc >= 0)
        matmul_mfma_tile_kernel<T, TM, TN, PD, false, 2><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, nullptr, (int)m, (int)k, (int)n, map, one, (int)ldc, (int)ldc, 0);
    else if (k % PK == 0) {
        // One tile across N and rows of A a multiple of 4 KiB apart (attention weights times values: [.., 2048, 2048] x
        // [.., 2048, 64]): A is streamed from memory exactly once, every tile asks for the same 128 bytes of 64 or 128 rows
        // at a time, and with all tiles at the same K step those pieces meet on the same memory channels (4.2 TB/s at a
        // pitch of 4096 bytes, 4.8 at 4224).  Each tile then starts at a K step of its own and wraps round: 30.0 -> 26.7 us
        // on that shape, 48.9 -> 44.3 us with K = 4096.  Not for other pitches, where the walk in step is the faster
        // one (K = 4160: 46 against 53 us); the sum of a row is the same up to fp32 rounding order.
        const int rotate = (map.tiles_n == 1 && k / PK >= 8 && ((size_t)k * sizeof(T)) % 4096 == 0) ? 2 : 0;
        matmul_mfma_tile_kernel<T, TM, TN, PD, false, 0><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, nullptr, (int)m, (int)k, (int)n, map, one, (int)n, (int)n, c_store_through(batch, m, n, sizeof(T)) | rotate);
    }
    else
        matmul_mfma_tile_kernel<T, TM, TN, PD, true, 0><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, nullptr, (int)m, (int)k, (int)n, map, one, (int)n, (int)n, c_store_through(batch, m, n, sizeof(T)));
    return launch_status();
}

// Few output tiles and a long K: 64x64 tiles over K slices, fp32 partial tiles in the call's
// scratch, then one pass that adds the slices in order and rounds once.  Returns kNoSplit when the
// product should not be cut (the caller then launches the ordinary way).
template <typename T>
int launch_split(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    constexpr int TM = 64, TN = 64, SPD = 1;  // two K steps in flight were measured slower here (64x8192x4096: 21.4 vs 19.0 us)
    const int64_t tiles = batch * ((m + TM - 1) / TM) * ((n + TN - 1) / TN), partial = batch * m * n * (int64_t)sizeof(float);
    const KSplit ks = choose_ksplit(tiles, k, PK, 2048, partial);
    TileMap map;
    if (ks.splits < 2 || !make_tile_map(batch * ks.splits, m, n, TM, TN, map)) return kNoSplit;
    float *ws = (float *)sc.take((size_t)(partial * ks.splits));
    if (!ws) return DXH_ERR_WORKSPACE;
    if (sc.planning) return DXH_OK;
    if (k % PK == 0)
        matmul_mfma_tile_kernel<T, TM, TN, SPD, false, 1><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, nullptr, ws, (int)m, (int)k, (int)n, map, ks, (int)n, (int)n, 0);
    else
        matmul_mfma_tile_kernel<T, TM, TN, SPD, true, 1><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, nullptr, ws, (int)m, (int)k, (int)n, map, ks, (int)n, (int)n, 0);
    const int rc = launch_status();
    return rc != DXH_OK ? rc : launch_splitk_reduce<float, T>(ws, (T *)c, batch, m * n, ks.splits, st);
}

// Rows that are not 16-byte aligned (odd K or N, unaligned bases): A and B are copied, zero-padded
// to K64 (next multiple of 64) and N8 columns, into the call's scratch, the tile kernel runs on
// the copies and stores C directly at its own pitch, element by element (EDGE).  Returns kNoSplit
// when that is not possible (operands over the scratch limit, tiny products).
template <typename T> int launch_mfma(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc, int64_t ldc = -1);
template <typename T>
int launch_padded(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    const int64_t kp = (k + PK - 1) / PK * PK, np = (n + 7) / 8 * 8;
    const bool a_as_is = k == kp && aligned(a, kVecBytes);
    const int64_t a_elems = a_as_is ? 0 : (batch * m * kp + 7) / 8 * 8, b_elems = batch * kp * np;
    const int64_t bytes = (a_elems + b_elems) * 2;
    if (bytes > kWorkspaceMaxBytes || m * n * k < (1 << 16) || kp > (1 << 22) || np > (1 << 24)) return kNoSplit;
    uint16_t *ws = (uint16_t *)sc.take((size_t)bytes);
    if (!ws) return DXH_ERR_WORKSPACE;
    if (sc.planning) return DXH_OK;  // the tile kernel on the copies needs no more
    uint16_t *ap = ws, *bp = ws + a_elems;
    if (!a_as_is) {
        const int64_t total = batch * m * (kp / 8);
        launch_pad_rows<uint16_t>((const uint16_t *)a, ap, m, k, m, kp / 8, total, st);
    }
    const int64_t total = batch * kp * (np / 8);
    launch_pad_rows<uint16_t>((const uint16_t *)b, bp, k, n, kp, np / 8, total, st);
    const int rc = launch_status();
    return rc != DXH_OK ? rc : launch_mfma<T>(a_as_is ? a : (const void *)ap, bp, c, batch, m, kp, np, st, sc, n);
}

// The workgroup tile of an aligned bf16 / f16 product that is not cut along K (DXH_TUNE_MATMUL_TILE numbering).
// dma_ok: the LDS-direct kernels can take it (K a multiple of 64, C at its own [M][N]).
static int64_t choose_uncut_tile(int64_t batch, int64_t m, int64_t k, int64_t n, int64_t ldc, bool dma_ok) {
    int64_t choice = 0;
    // 256x256 tiles halve the bytes every CU pulls through its vector cache per flop, but need
    // about one tile per CU to pay off.  Below that, 128x128 tiles (two workgroups per CU) as
    // long as they still give every CU a workgroup and a half; skinny outputs go to 128x64 or
    // 64x64 tiles so that all CUs (and their vector caches) take part.
    const int64_t cus = compute_units();
    auto tiles = [&](int tm, int tn) { return batch * ((m + tm - 1) / tm) * ((n + tn - 1) / tn); };
    if (m <= 64) choice = 5;  // one tile row: anything taller multiplies padding (bf16 [1,896]x[896,151936]: 53 vs 75 us)
    else if (tiles(128, 64) * 4 >= cus * 3) {
        // Enough output for tiles of 128x64 and up: estimated time in us of the candidates.  The two
        // one-workgroup-per-CU tiles run in rounds of `cus` tiles, each round paying its own
        // prologue and its own burst of C stores (nothing else runs on the CU to hide them); K
        // steps get faster when only part of the CUs is busy.  128x128 tiles run two to a CU: a
        // pair of tiles takes 1.08 us per K step, a tile that has the CU to itself 0.53 us.
        const double ksteps = (double)((k + PK - 1) / PK);
        auto one_per_cu = [&](int tm, int tn, double step, double overhead) {
            const int64_t t = tiles(tm, tn), rounds = (t + cus - 1) / cus;
            const double busy = rounds > 1 ? 1.0 : (double)t / (double)cus;
            return (double)rounds * (ksteps * step * (0.65 + 0.35 * busy) + overhead);
        };
        const int64_t t1 = tiles(128, 128), full = t1 / (2 * cus), rem = t1 % (2 * cus);
        const double c1 = ksteps * (1.08 * (double)full + (rem == 0 ? 0.0 : rem <= cus ? 0.53 : 1.08)) + 2.0;
        const double edge = ldc >= 0 ? 5.0 : 0.0;  // element-wise C stores make the burst at the end of a round longer
        const double c4 = one_per_cu(256, 256, 1.645, 3.5 + edge), c6 = one_per_cu(192, 256, 1.21, 6.0 + edge);
        // 128x64 tiles, two to a CU as well: 0.33 us per K step and tile (2048x4864x896: 224 tiles, 27 us)
        const double c2 = ksteps * 0.33 * (double)((tiles(128, 64) + cus - 1) / cus) + 2.0;
        choice = (c1 <= c4 && c1 <= c6) ? 1 : (c4 <= c6) ? 4 : 6;
        if (c2 < (choice == 1 ? c1 : choice == 4 ? c4 : c6)) choice = 2;
        // Lower tiles of the same width, one wave per 64 columns (matmul_half_dma.hip only): when a
        // lower tile still fits the output into one round, every CU's K loop gets shorter
        // (2048x896x4864: 18.2 us with 160 rows, 19.8 with 192; 2048x4096x4096: 56.9 us with 128
        // rows, 63.4 with 192, hipBLASLt 70.9).  Both run three LDS stages of K 64 (against five of
        // K 32: 2048x4096x4096 58.4 -> 55.7 us, 3072^3 with 160 rows 51.6 -> 48.8 us).
        // And a tile half as wide for an N that 256 columns divide badly (8192x4864x896, where 256-wide
        // tiles compute 1024 columns: 58.5 us against 66.5 with 128 rows x 256).
        // All three are taken for a single round only: over several rounds the square tile's lower
        // traffic through L2 wins again (8192^3: 843 us with 256x128, 790 with 256x256).
        if (dma_ok) {
            const double c11 = one_per_cu(160, 256, 0.96, 5.5), c12 = one_per_cu(128, 256, 0.85, 5.0), c13 = one_per_cu(256, 128, 0.76, 3.5) - (tiles(256, 128) <= cus / 2 ? ksteps * 0.09 : 0.0);  // 0.52 us per step up to half the CUs
            double best = choice == 1 ? c1 : choice == 2 ? c2 : choice == 4 ? c4 : c6;
            // ... except on a short K (up to 16 steps), where a round is mostly its prologue and its C burst and the
            // operands are small: there the estimate holds over several rounds too (8192x896x4864: 73 us with 160
            // rows, 86 with 128x128 two to a CU, 79 with 256x256; 4096x896x4864: 36.7 against 43.5)
            const bool any_rounds = ksteps <= 16.0;
            if (c11 < best && (any_rounds || tiles(160, 256) <= cus)) { best = c11; choice = 11; }
            if (c12 < best && (any_rounds || tiles(128, 256) <= cus)) { best = c12; choice = 12; }
            if (c13 < best && (any_rounds || tiles(256, 128) <= cus)) { best = c13; choice = 13; }
        }
    }
    else choice = 5;  // 1024x8192x1024 as 128 tiles of 128x64: 38 us, 31 us with 256 64x64 tiles
    return choice;
}

// ldc >= 0: called by launch_padded on its copies; C then has ldc columns at pitch ldc
template <typename T>
int launch_mfma(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc, int64_t ldc) {
    const bool fast = k % 8 == 0 && n % 8 == 0 && aligned(a, kVecBytes) && aligned(b, kVecBytes) && (ldc >= 0 || aligned(c, kVecBytes)) &&
                      k <= (1 << 22) && n <= (1 << 24);
    int64_t choice = tuning().matmul_tile;
    if (ldc >= 0 && (!fast || k % PK != 0)) return DXH_ERR_ALIGN;  // launch_padded hands over aligned copies only
    const bool dma_ok = fast && ldc < 0 && k % 64 == 0;
    // A long K over few output tiles: 128x128 tiles whose K is cut in two inside one launch (the halves
    // meet in the caller's scratch; matmul_half_dma.hip).  Measured against what would run otherwise on
    // 17 such shapes: 0.57-0.93 of its time from K = 4096 up and 48 to 128 tiles (2048x4864x896: 25.8 ->
    // 23.7 us, 1536x8192x768: 48 -> 27 us), slower with K = 2048 or under 20 tiles.
    if (dma_ok && choice == 0 && tuning().matmul_splitk != 1 && m > 128 && k >= 4096) {
        const int64_t t14 = batch * ((m + 127) / 128) * ((n + 127) / 128), t15 = batch * ((m + 127) / 128) * ((n + 255) / 256);
        if (t14 >= 40 && 2 * t14 <= compute_units()) choice = 14;
        // the same with 128x256 tiles (four waves side by side) for outputs twice that size: 0.87-0.94 of
        // the uncut time from K = 6144 up, or from K = 4096 with under 100 tiles (1024x4096x3072: 36.9 ->
        // 32.2 us; 2048x8192x2048: 70.5 -> 65.6 us, hipBLASLt 85; 2048x4096x2048 with 128 tiles loses)
        else if (t15 >= 40 && 2 * t15 <= compute_units() && (k >= 6144 || t15 <= 100)) choice = 15;
    }
    if (fast && ldc < 0 && (choice == 0 || choice == 5)) {
        const int rc = launch_split<T>(a, b, c, batch, m, k, n, st, sc);
        if (rc != kNoSplit) return rc;
    }
    if (fast && choice == 0) choice = choose_uncut_tile(batch, m, k, n, ldc, dma_ok);
    // The two one-workgroup-per-CU tiles have a twin whose operands travel straight into LDS
    // (matmul_half_dma.hip: less power, no LDS store traffic, deeper prefetch; 8192^3 830 -> 782 us,
    // 4096^3 109 -> 102 us); it needs whole K steps of 64 and C at its own [M][N].  Its 256x256 tile
    // runs two LDS stages of K 64 when K is long (whole cache lines of A, half the barriers) and four
    // of K 32 when it is short (2048x896x4864: 21.2 against 22.6 us with the shallow pipeline).
    if (dma_ok && tuning().matmul_tile == 0 && (choice == 4 || choice == 6)) choice = choice == 6 ? 8 : k >= 2048 ? 10 : 7;
    if (dma_ok && (choice == 14 || choice == 15)) {
        const int wide = choice == 15;
        const int64_t t14 = batch * ((m + 127) / 128) * ((n + (wide ? 255 : 127)) / (wide ? 256 : 128));
        if (t14 <= 1024 && k >= 64 * 2) {
            float *part = (float *)sc.take((size_t)dma_split_bytes(t14, wide));
            if (!part) return DXH_ERR_WORKSPACE;
            if (sc.planning) return DXH_OK;
            if (unsigned *cnt = finish_counters(st, t14))
                return launch_matmul_half_dma_split(std::is_same_v<T, bf16_t> ? DXH_BF16 : DXH_F16, wide, a, b, c, batch, m, k, n, part, cnt, st);
        }
        choice = wide ? 12 : 1;  // no counters to be had (or too many tiles): the same tile, uncut
    }
    if (dma_ok && choice >= 7 && choice <= 13) {
        if (sc.planning) return DXH_OK;
        return launch_matmul_half_dma(std::is_same_v<T, bf16_t> ? DXH_BF16 : DXH_F16, (int)choice - 7, a, b, c, batch, m, k, n, st);
    }
    if (fast) {
        switch (choice) {
        case 2: case 9: return launch_tile<T, 128, 64, 2>(a, b, c, batch, m, k, n, ldc, st, sc);
        case 3: return launch_tile<T, 64, 128, 2>(a, b, c, batch, m, k, n, ldc, st, sc);
        case 4: return launch_tile<T, 256, 256, 1>(a, b, c, batch, m, k, n, ldc, st, sc);
        case 5: return launch_tile<T, 64, 64, 2>(a, b, c, batch, m, k, n, ldc, st, sc);
        case 6: case 8: case 11: case 12: return launch_tile<T, 192, 256, 1>(a, b, c, batch, m, k, n, ldc, st, sc);
        case 7: case 10: case 13: return launch_tile<T, 256, 256, 1>(a, b, c, batch, m, k, n, ldc, st, sc);
        case 14: case 15: default: return launch_tile<T, 128, 128, 1>(a, b, c, batch, m, k, n, ldc, st, sc);
        }
    }
    if (!fast && tuning().matmul_tile == 0 && k <= (1 << 22) && n <= (1 << 24)) {
        const int rc = launch_padded<T>(a, b, c, batch, m, k, n, st, sc);
        if (rc != kNoSplit) return rc;
    }
    if (sc.planning) return DXH_OK;
    const int64_t tiles_m = (m + BM - 1) / BM, tiles_n = (n + BN - 1) / BN;
    const int64_t blocks = batch * tiles_m * tiles_n;
    if (blocks > 0x7fffffff) return DXH_ERR_SHAPE;
    const bool va = (k % 8 == 0) && aligned(a, kVecBytes);
    const bool vb = (n % 8 == 0) && aligned(b, kVecBytes);
#define DXH_MM(VA, VB) matmul_mfma_kernel<T, VA, VB><<<(unsigned)blocks, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, (int)tiles_m, (int)tiles_n)
    if (va && vb) DXH_MM(true, true);
    else if (va) DXH_MM(true, false);
    else if (vb) DXH_MM(false, true);
    else DXH_MM(false, false);
#undef DXH_MM
    return launch_status();
}
// C_j = A B_j for the pairs of `multi` as ONE launch of an LDS-direct tile: the tile that one of the products
// alone would take, over a tile map with one batch entry per pair, so the second product's tiles start as
// the first's finish (one prologue for the lot, the stores of C_0 run under the K loops of C_1).  Only for
// products that take such a tile uncut; kNoShared otherwise, and the caller multiplies one by one.  dry: the
// decision without the launch.
int launch_matmul_half_shared(int dtype, const void *a, const SharedA &multi, int64_t m, int64_t k, int64_t n, hipStream_t st, bool dry) {
    if (multi.count < 2 || multi.count > kSharedAMax || tuning().matmul_tile != 0) return kNoShared;
    bool ok = m > 64 && k % 64 == 0 && n % 8 == 0 && aligned(a, kVecBytes) && k <= (1 << 22) && n <= (1 << 24);
    for (int j = 0; j < multi.count; ++j) ok = ok && aligned(multi.b[j], kVecBytes) && aligned(multi.c[j], kVecBytes);
    if (!ok) return kNoShared;
    const int64_t cus = compute_units();
    // a long K over few tiles is cut along K when multiplied alone (scratch, counters): not here
    const int64_t t64 = ((m + 63) / 64) * ((n + 63) / 64), t128 = ((m + 127) / 128) * ((n + 127) / 128);
    if (k >= 2048 && tuning().matmul_splitk != 1 && (t64 * 2 <= cus || (k >= 4096 && t128 >= 40 && 2 * t128 <= cus))) return kNoShared;
    if (tuning().matmul_splitk >= 2) return kNoShared;
    int64_t choice = choose_uncut_tile(1, m, k, n, -1, true);
    if (choice == 4 || choice == 6) choice = choice == 6 ? 8 : k >= 2048 ? 10 : 7;  // their LDS-direct twins, as in launch_mfma
    if (choice < 7 || choice > 13) return kNoShared;
    if (dry) return DXH_OK;
    return launch_matmul_half_dma(dtype, (int)choice - 7, a, nullptr, nullptr, 1, m, k, n, st, multi);
}

int launch_matmul_half(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, Scratch &sc) {
    return dtype == DXH_BF16 ? launch_mfma<bf16_t>(a, b, c, batch, m, k, n, st, sc) : launch_mfma<f16_t>(a, b, c, batch, m, k, n, st, sc);
}

}  // namespace dxh
