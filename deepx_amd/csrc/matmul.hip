// matmul.hip — batched row-major GEMM  C[b,m,n] = sum_k A[b,m,k] * B[b,k,n]  (gfx950).
//
// Replaces cublasSgemm(StridedBatched) of executor/op-cuda/src/deepx/tensorfunc/matmul_cublas.hpp:16-145
// and cblas_sgemm of executor/op-ompsimd/src/deepx/tensorfunc/matmul_cblas.hpp:11-60 (alpha=1, beta=0).
//
//   bf16 / f16   MFMA v_mfma_f32_32x32x16_{bf16,f16}, fp32 accumulate, one RNE rounding of C.
//                Aligned shapes (K % 64 == 0, N % 8 == 0): matmul_mfma_tile_kernel, 64x64 to
//                256x256 workgroup tiles, software-pipelined over K.  Anything else:
//                matmul_mfma_kernel, a plain 128x128x32 tile with element-wise edge handling.
//   f32          MFMA v_mfma_f32_32x32x2_f32 (fp32 operands and accumulate): matmul_mfma_f32_kernel.
//   f64          MFMA v_mfma_f64_16x16x4_f64: matmul_mfma_f64_kernel.
//   integers     LDS-tiled 64x64x16 multiply-add kernel, 4x4 outputs per lane; accumulate in the
//                storage type (integers wrap).
#include "common.hpp"

namespace dxh {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int BM = 128, BN = 128, BK = 32;
constexpr int LDK = BK + 8;  // padded k-stride (elements) of both LDS tiles: 80 bytes, keeps 16-byte alignment

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));  // native vector: arrays of it stay in registers
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T, typename V> __device__ inline f32x16 mfma32(V a, V b, f32x16 c) {
    if constexpr (std::is_same_v<T, bf16_t>)
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

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

// ---- MFMA kernel with the B transposition done by the LDS read ------------------------------
// Workgroup tile TM x TN (64, 128 or 256 each), K step 64, 4 waves in a 2x2 grid, each wave a
// (TM/2) x (TN/2) patch of 32x32x16 MFMAs.  Requirements (checked by the launcher): K % 64 == 0,
// N % 8 == 0, 16-byte aligned A, B, C.
//   loads  every global load is 16 bytes per lane (a wave instruction occupies the vector cache for
//          the same 16 cycles whatever its width, so 8-byte loads halve its throughput).
//   A      [TM m][64 k] in LDS, 128-byte rows, 16-byte chunk c of row r at chunk c ^ swizzle(r).
//   B      stays n-contiguous in LDS, [64 k][TN n] with rows padded by 64 bytes; the MFMA operand
//          (8 consecutive k of one column per lane) is assembled by two ds_read_b64_tr_b16.
//   pipe   PD K steps in flight in registers, two LDS stages, one barrier per K step; the stores
//          into the next stage and the global loads are spread over the four k-substeps.
//   roles  the MFMA runs on (B^T, A^T): a lane of the result then holds 4 consecutive n of one row
//          m, which packs into 8-byte LDS stores for the epilogue.
//   map    blockIdx -> tile through tile_of_block (XCD-aware, above).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &f, std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F> __device__ __forceinline__ void static_for(F f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }
template <int V> using ic = std::integral_constant<int, V>;

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

// the `count` loads of a K step are dealt out over its four k-substeps
constexpr int part_first(int count, int part) { return count * part / 4; }
constexpr int part_count(int count, int part) { return count * (part + 1) / 4 - count * part / 4; }

template <typename T, int TM, int TN, int PD>
__global__ __launch_bounds__(kBlock, (TM * TN <= 128 * 128) ? 2 : 1) void matmul_mfma_tile_kernel(
    const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C, int M, int K, int N, TileMap map) {
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
    const int batch = tc.batch, tm = tc.tm, tn = tc.tn;
    const int m0 = tm * TM, n0 = tn * TN;

    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wm = w >> 1, wn = w & 1;
    const uint16_t *Ab = reinterpret_cast<const uint16_t *>(A) + ((int64_t)batch * M + m0) * K;
    const uint16_t *Bb = reinterpret_cast<const uint16_t *>(B) + (int64_t)batch * K * N + n0;

    // Branch-free loads: rows past M and columns past N are clamped onto valid memory; their
    // products land in accumulator rows/columns that the epilogue never stores.
    const int arow = t >> 3, ach = t & 7;
    int a_off[A_LD], a_lds[A_LD];
    static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
        const int r = arow + 32 * i;
        a_off[i] = (m0 + r < M ? r : M - 1 - m0) * K + ach * 8;
        a_lds[i] = r * PK + swz(r, ach) * 8;
    });
    const int brow = t / CB, bch = t % CB;
    const int b_off = brow * N + (n0 + bch * 8 < N ? bch * 8 : N - 8 - n0);
    const int b_lds = brow * B_ROW + bch * 8;

    u32x4 ra[PD][A_LD], rb[PD][B_LD];
    auto load_part = [&](auto set, auto part, int k0) __attribute__((always_inline)) {
        static_for<part_count(A_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(A_LD, decltype(part)::value) + decltype(q)::value;
            ra[set][i] = *reinterpret_cast<const u32x4 *>(Ab + a_off[i] + k0);
        });
        static_for<part_count(B_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(B_LD, decltype(part)::value) + decltype(q)::value;
            rb[set][i] = *reinterpret_cast<const u32x4 *>(Bb + (int64_t)(k0 + i * KR) * N + b_off);
        });
    };
    auto store_part = [&](auto set, auto part, auto stage) __attribute__((always_inline)) {
        uint16_t *As = lds + decltype(stage)::value * STAGE, *Bs = As + A_STAGE;
        static_for<part_count(A_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(A_LD, decltype(part)::value) + decltype(q)::value;
            *reinterpret_cast<u32x4 *>(As + a_lds[i]) = ra[set][i];
        });
        static_for<part_count(B_LD, decltype(part)::value)>([&](auto q) __attribute__((always_inline)) {
            constexpr int i = part_first(B_LD, decltype(part)::value) + decltype(q)::value;
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
    // Issue order inside a scheduling region: after each of `mfmas` MFMAs an even share of the
    // region's LDS reads, LDS writes and global loads, so that the matrix pipe always has the next
    // MFMA queued while the memory instructions are issued underneath it.
    auto interleave = [&](auto mfmas, auto reads, auto writes, auto loads) __attribute__((always_inline)) {
        constexpr int nm = decltype(mfmas)::value, nr = decltype(reads)::value, nw = decltype(writes)::value, nl = decltype(loads)::value;
        static_for<nm>([&](auto x) __attribute__((always_inline)) {
            constexpr int m = decltype(x)::value;
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            constexpr int r = nr * (m + 1) / nm - nr * m / nm, wr = nw * (m + 1) / nm - nw * m / nm, l = nl * (m + 1) / nm - nl * m / nm;
            if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);
            if constexpr (wr > 0) __builtin_amdgcn_sched_group_barrier(0x200, wr, 0);
            if constexpr (l > 0) __builtin_amdgcn_sched_group_barrier(0x020, l, 0);
        });
    };

    // One K step: LDS stage S is multiplied; register set R (the next K step) moves into stage
    // S^1 and is refilled with the K step PD further on.  Fragment buffer 0 holds substep 0 on
    // entry.  The last substep straddles the barrier: half of its MFMAs are queued before it and
    // the other half runs under the first fragment reads of stage S^1.
    auto step = [&](auto S, auto R, int k_load) __attribute__((always_inline)) {
        constexpr int s = decltype(S)::value;
        static_for<4>([&](auto ks) __attribute__((always_inline)) {
            constexpr int cur = decltype(ks)::value & 1;
            constexpr int NW = part_count(A_LD, decltype(ks)::value) + part_count(B_LD, decltype(ks)::value);  // LDS writes = global loads
            if constexpr (decltype(ks)::value < 3) {
                read_frags(ic<cur ^ 1>{}, S, ic<decltype(ks)::value + 1>{});
                store_part(R, ks, ic<s ^ 1>{});
                load_part(R, ks, k_load);
                mma(ic<cur>{}, ic<0>{}, ic<NM>{});
                interleave(ic<NM>{}, ic<ND>{}, ic<NW>{}, ic<NW>{});
            } else {
                store_part(R, ks, ic<s ^ 1>{});
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

    const int KT = K / PK;
    auto k_of = [&](int stepno) __attribute__((always_inline)) { return (stepno < KT ? stepno : KT - 1) * PK; };
    static_for<4>([&](auto part) __attribute__((always_inline)) { load_part(ic<0>{}, part, k_of(0)); });
    static_for<4>([&](auto part) __attribute__((always_inline)) { store_part(ic<0>{}, part, ic<0>{}); });
    static_for<PD>([&](auto d) __attribute__((always_inline)) { static_for<4>([&](auto part) __attribute__((always_inline)) { load_part(ic<(decltype(d)::value + 1) % PD>{}, part, k_of(decltype(d)::value + 1)); }); });
    __syncthreads();
    read_frags(ic<0>{}, ic<0>{}, ic<0>{});
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
        step(ic<0>{}, ic<1 % PD>{}, k_of(kt + 1 + PD));
        step(ic<1>{}, ic<2 % PD>{}, k_of(kt + 2 + PD));
    }
    if (kt < KT) step(ic<0>{}, ic<1 % PD>{}, k_of(kt + 1 + PD));
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
    uint16_t *Cr = reinterpret_cast<uint16_t *>(C) + (int64_t)batch * M * N;
#pragma unroll
    for (int i = 0; i < TM * CB / kBlock; ++i) {
        const int c = t + i * kBlock, row = c / CB, ch = c % CB;
        const int gm = m0 + row, gn = n0 + ch * 8;
        if (gm < M && gn < N)  // N % 8 == 0: a chunk is either fully inside or fully outside
            st_nt(reinterpret_cast<uint4 *>(Cr + (int64_t)gm * N + gn), *reinterpret_cast<const uint4 *>(Cs + row * LDC + ch * 8));
    }
}

// ---- fp32 MFMA kernel ------------------------------------------------------------------------
// v_mfma_f32_32x32x2_f32 (fp32 operands, fp32 accumulate: 157 TFLOP/s peak, 64 cycles each).  A
// fp32 GEMM on the matrix pipe is compute bound by a wide margin (8x fewer flops per operand
// byte than bf16 at 1/16 of the rate), so this kernel is a plain double-buffered one: workgroup
// tile (64 FM) x (64 FN), K step FK, 4 waves 2x2, each wave FM x FN MFMA tiles, PD K steps held
// in registers ahead of the LDS stage being multiplied.
//   A      LDS [m][FK k] with rows padded by 4 floats; a lane reads the FK/2 consecutive k of its
//          row half with ds_read_b128 (the k order inside a K step is a free permutation as
//          long as both operands use it: MFMA e of lane half h multiplies k = (FK/2) h + e).
//   B      LDS [FK k][n] as loaded, rows padded by 4 floats; one ds_read_b32 per lane and k.
//   roles  MFMA on (B^T, A^T): a result lane holds 4 consecutive n of one row m -> 16-byte stores.
//   VEC    K % 4 == 0, N % 4 == 0 and 16-byte aligned pointers: 16-byte loads and stores with
//          clamped rows/columns; otherwise element-wise accesses with bounds checks.
template <int FM, int FN, int FK, int PD, bool VEC>
__global__ __launch_bounds__(kBlock, 2) void matmul_mfma_f32_kernel(const float *__restrict__ A, const float *__restrict__ B,
                                                                    float *__restrict__ C, int M, int K, int N, TileMap map) {
    constexpr int TM = 64 * FM, TN = 64 * FN, FA_ROW = FK + 4, FB_ROW = TN + 4;
    constexpr int STAGE = TM * FA_ROW + FK * FB_ROW;  // floats
    constexpr int CA = FK / 4, CB = TN / 4;           // 16-byte chunks per A row / B row
    constexpr int A_LD = TM * CA / kBlock, B_LD = FK * CB / kBlock;
    constexpr int HK = FK / 2;                        // k values per lane half
    typedef float f32x4 __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) float lds[2 * STAGE];
    const TileCoord tc = tile_of_block(map);
    if (!tc.valid) return;
    const int tm = tc.tm, tn = tc.tn;
    A += tc.batch * (int64_t)M * K;
    B += tc.batch * (int64_t)K * N;
    C += tc.batch * (int64_t)M * N;
    const int m0 = tm * TM, n0 = tn * TN;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wm = w >> 1, wn = w & 1;

    // per-lane chunks: A (row = id / CA, c = id % CA), B (krow = id / CB, c = id % CB), id = t + 256 i
    f32x4 ra[PD][A_LD], rb[PD][B_LD];
    auto load_global = [&](auto set, int k0) __attribute__((always_inline)) {
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, row = id / CA, kk = k0 + (id % CA) * 4, gm = m0 + row;
            if constexpr (VEC) {
                const float *p = A + (int64_t)(gm < M ? gm : M - 1) * K + (kk < K ? kk : 0);
                f32x4 v = *reinterpret_cast<const f32x4 *>(p);
                ra[set][i] = (kk < K) ? v : f32x4{0.f, 0.f, 0.f, 0.f};
            } else {
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (gm < M && kk + e < K) ? A[(int64_t)gm * K + kk + e] : 0.f;
                ra[set][i] = v;
            }
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, krow = id / CB, gk = k0 + krow, gn = n0 + (id % CB) * 4;
            if constexpr (VEC) {
                const float *p = B + (int64_t)(gk < K ? gk : 0) * N + (gn < N ? gn : N - 4);
                f32x4 v = *reinterpret_cast<const f32x4 *>(p);
                rb[set][i] = (gk < K) ? v : f32x4{0.f, 0.f, 0.f, 0.f};
            } else {
                f32x4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = (gk < K && gn + e < N) ? B[(int64_t)gk * N + gn + e] : 0.f;
                rb[set][i] = v;
            }
        });
    };
    auto store_lds = [&](auto set, auto stage) __attribute__((always_inline)) {
        float *As = lds + decltype(stage)::value * STAGE, *Bs = As + TM * FA_ROW;
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            *reinterpret_cast<f32x4 *>(As + (id / CA) * FA_ROW + (id % CA) * 4) = ra[set][i];
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            *reinterpret_cast<f32x4 *>(Bs + (id / CB) * FB_ROW + (id % CB) * 4) = rb[set][i];
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
    // MFMA e of lane half h multiplies k = HK*h + e of the K step (both operands use this order)
    auto compute = [&](auto stage) __attribute__((always_inline)) {
        const float *As = lds + decltype(stage)::value * STAGE, *Bs = As + TM * FA_ROW;
        static_for<HK / 8>([&](auto q) __attribute__((always_inline)) {  // 8 k per lane half at a time
            f32x4 fa[FM][2];
            float fb[FN][8];
            static_for<FM>([&](auto i) __attribute__((always_inline)) {
                const float *p = As + (wm * 32 * FM + 32 * i + l32) * FA_ROW + HK * h + 8 * decltype(q)::value;
                fa[i][0] = *reinterpret_cast<const f32x4 *>(p);
                fa[i][1] = *reinterpret_cast<const f32x4 *>(p + 4);
            });
            static_for<FN>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
                for (int e = 0; e < 8; ++e) fb[j][e] = Bs[(HK * h + 8 * decltype(q)::value + e) * FB_ROW + wn * 32 * FN + 32 * j + l32];
            });
#pragma unroll
            for (int e = 0; e < 8; ++e)
                static_for<FM>([&](auto i) __attribute__((always_inline)) {
                    static_for<FN>([&](auto j) __attribute__((always_inline)) {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][e], fa[i][e >> 2][e & 3], acc[i][j], 0, 0, 0);
                    });
                });
        });
    };

    // LDS stage (kt & 1) holds K step kt, register set (kt + 1) % PD holds step kt + 1 and is
    // refilled with step kt + 1 + PD once it has moved to LDS.  Steps past the end are clamped
    // onto the last one (loaded, never multiplied).
    const int KT = (K + FK - 1) / FK;
    auto k_of = [&](int stepno) { return (stepno < KT ? stepno : KT - 1) * FK; };
    auto step = [&](auto S, auto R, int k_load) __attribute__((always_inline)) {
        compute(S);
        store_lds(R, ic<decltype(S)::value ^ 1>{});
        load_global(R, k_load);
        __syncthreads();
    };
    load_global(ic<0>{}, 0);
    store_lds(ic<0>{}, ic<0>{});
    static_for<PD>([&](auto d) __attribute__((always_inline)) { load_global(ic<(decltype(d)::value + 1) % PD>{}, k_of(decltype(d)::value + 1)); });
    __syncthreads();
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
        step(ic<0>{}, ic<1 % PD>{}, k_of(kt + 1 + PD));
        step(ic<1>{}, ic<2 % PD>{}, k_of(kt + 2 + PD));
    }
    if (kt < KT) compute(ic<0>{});

    // result lane: row m = lane%32 of its MFMA tile; register group g holds columns 8g + 4h .. +3
    static_for<FM>([&](auto i) __attribute__((always_inline)) {
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
            const int gm = m0 + wm * 32 * FM + 32 * i + l32;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int gn = n0 + wn * 32 * FN + 32 * j + 8 * g + 4 * h;
                if constexpr (VEC) {
                    if (gm < M && gn < N)
                        __builtin_nontemporal_store(f32x4{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]},
                                                    reinterpret_cast<f32x4 *>(C + (int64_t)gm * N + gn));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (gm < M && gn + e < N) C[(int64_t)gm * N + gn + e] = acc[i][j][4 * g + e];
                }
            }
        });
    });
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
                                                                    double *__restrict__ C, int M, int K, int N, TileMap map) {
    constexpr int DK = 16, TM = 64 * FM, TN = 64 * FN, DA_ROW = DK + 2, DB_ROW = TN + 4;
    constexpr int STAGE = TM * DA_ROW + DK * DB_ROW;  // doubles
    constexpr int CA = DK / 2, CB = TN / 2;           // 16-byte chunks per A row / B row
    constexpr int A_LD = TM * CA / kBlock, B_LD = DK * CB / kBlock;
    constexpr int RT = 2 * FM, CT = 2 * FN;           // 16x16 MFMA tiles per wave along m and n
    __shared__ __attribute__((aligned(16))) double lds[2 * STAGE];
    const TileCoord tc = tile_of_block(map);
    if (!tc.valid) return;
    const int tm = tc.tm, tn = tc.tn;
    A += tc.batch * (int64_t)M * K;
    B += tc.batch * (int64_t)K * N;
    C += tc.batch * (int64_t)M * N;
    const int m0 = tm * TM, n0 = tn * TN;
    const int t = threadIdx.x, lane = t & 63, w = t >> 6, wm = w >> 1, wn = w & 1;

    f64x2 ra[A_LD], rb[B_LD];
    auto load_global = [&](int k0) __attribute__((always_inline)) {
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, row = id / CA, kk = k0 + (id % CA) * 2, gm = m0 + row;
            if constexpr (VEC) {
                const double *p = A + (int64_t)(gm < M ? gm : M - 1) * K + (kk < K ? kk : 0);
                f64x2 v = *reinterpret_cast<const f64x2 *>(p);
                ra[i] = (kk < K) ? v : f64x2{0.0, 0.0};
            } else {
                f64x2 v;
#pragma unroll
                for (int e = 0; e < 2; ++e) v[e] = (gm < M && kk + e < K) ? A[(int64_t)gm * K + kk + e] : 0.0;
                ra[i] = v;
            }
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i, krow = id / CB, gk = k0 + krow, gn = n0 + (id % CB) * 2;
            if constexpr (VEC) {
                const double *p = B + (int64_t)(gk < K ? gk : 0) * N + (gn < N ? gn : N - 2);
                f64x2 v = *reinterpret_cast<const f64x2 *>(p);
                rb[i] = (gk < K) ? v : f64x2{0.0, 0.0};
            } else {
                f64x2 v;
#pragma unroll
                for (int e = 0; e < 2; ++e) v[e] = (gk < K && gn + e < N) ? B[(int64_t)gk * N + gn + e] : 0.0;
                rb[i] = v;
            }
        });
    };
    auto store_lds = [&](int stage) __attribute__((always_inline)) {
        double *As = lds + stage * STAGE, *Bs = As + TM * DA_ROW;
        static_for<A_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            *reinterpret_cast<f64x2 *>(As + (id / CA) * DA_ROW + (id % CA) * 2) = ra[i];
        });
        static_for<B_LD>([&](auto i) __attribute__((always_inline)) {
            const int id = t + kBlock * i;
            *reinterpret_cast<f64x2 *>(Bs + (id / CB) * DB_ROW + (id % CB) * 2) = rb[i];
        });
    };

    f64x4 acc[RT][CT];
    static_for<RT>([&](auto i) __attribute__((always_inline)) {
        static_for<CT>([&](auto j) __attribute__((always_inline)) { acc[i][j] = f64x4{0.0, 0.0, 0.0, 0.0}; });
    });
    const int q = lane >> 4, l16 = lane & 15;
    auto compute = [&](int stage) __attribute__((always_inline)) {
        const double *As = lds + stage * STAGE, *Bs = As + TM * DA_ROW;
        f64x2 fa[RT][2];
        double fb[CT][4];
        static_for<RT>([&](auto i) __attribute__((always_inline)) {
            const double *p = As + (wm * 32 * FM + 16 * i + l16) * DA_ROW + 4 * q;
            fa[i][0] = *reinterpret_cast<const f64x2 *>(p);
            fa[i][1] = *reinterpret_cast<const f64x2 *>(p + 2);
        });
        static_for<CT>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int e = 0; e < 4; ++e) fb[j][e] = Bs[(4 * q + e) * DB_ROW + wn * 32 * FN + 16 * j + l16];
        });
#pragma unroll
        for (int e = 0; e < 4; ++e)
            static_for<RT>([&](auto i) __attribute__((always_inline)) {
                static_for<CT>([&](auto j) __attribute__((always_inline)) {
                    acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(fa[i][e >> 1][e & 1], fb[j][e], acc[i][j], 0, 0, 0);
                });
            });
    };

    const int KT = (K + DK - 1) / DK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
        const bool more = kt + 1 < KT;
        if (more) load_global((kt + 1) * DK);
        compute(kt & 1);
        if (more) store_lds((kt + 1) & 1);
        __syncthreads();
    }

    static_for<RT>([&](auto i) __attribute__((always_inline)) {
        static_for<CT>([&](auto j) __attribute__((always_inline)) {
            const int gn = n0 + wn * 32 * FN + 16 * j + l16;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int gm = m0 + wm * 32 * FM + 16 * i + 4 * v + q;
                if (gm < M && gn < N) __builtin_nontemporal_store(acc[i][j][v], C + (int64_t)gm * N + gn);
            }
        });
    });
}

// ---- generic tiled kernel (f32, f64, integers) ------------------------------------------
constexpr int GT = 64, GK = 16;
template <typename T>
__global__ __launch_bounds__(kBlock) void matmul_tiled_kernel(const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C,
                                                               int M, int K, int N, int tiles_m, int tiles_n) {
    __shared__ T As[GK][GT + 1];  // [k][m]
    __shared__ T Bs[GK][GT + 1];  // [k][n]
    int64_t bid = blockIdx.x;
    const int tn = (int)(bid % tiles_n); bid /= tiles_n;
    const int tm = (int)(bid % tiles_m); bid /= tiles_m;
    A += bid * (int64_t)M * K;
    B += bid * (int64_t)K * N;
    C += bid * (int64_t)M * N;
    const int m0 = tm * GT, n0 = tn * GT;
    const int t = threadIdx.x, tx = t & 15, ty = t >> 4;
    T acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = T(0);
    for (int k0 = 0; k0 < K; k0 += GK) {
        // A tile 64x16: lanes along k (contiguous), 4 rows per lane
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const int r = (t >> 4) + h * 16, kc = t & 15;
            const int gm = m0 + r, gk = k0 + kc;
            As[kc][r] = (gm < M && gk < K) ? A[(int64_t)gm * K + gk] : T(0);
        }
        // B tile 16x64: lanes along n (contiguous), 4 k-rows per lane
#pragma unroll
        for (int h = 0; h < 4; ++h) {
            const int kr = (t >> 6) + h * 4, nc = t & 63;
            const int gk = k0 + kr, gn = n0 + nc;
            Bs[kr][nc] = (gk < K && gn < N) ? B[(int64_t)gk * N + gn] : T(0);
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < GK; ++kk) {
            T a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Bs[kk][tx + j * 16];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if constexpr (std::is_integral_v<T>) {
                        using U = std::conditional_t<(sizeof(T) < 4), uint32_t, std::make_unsigned_t<T>>;
                        acc[i][j] = T(U(U(acc[i][j]) + U(U(a[i]) * U(b[j]))));
                    } else {
                        acc[i][j] = __builtin_fma(a[i], b[j], acc[i][j]);
                    }
                }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = m0 + ty * 4 + i, col = n0 + tx + j * 16;
            if (row < M && col < N) C[(int64_t)row * N + col] = acc[i][j];
        }
}

template <typename T, int TM, int TN, int PD>
int launch_tile(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    TileMap map;
    if (!make_tile_map(batch, m, n, TM, TN, map)) return DXH_ERR_SHAPE;
    matmul_mfma_tile_kernel<T, TM, TN, PD><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, map);
    return launch_status();
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

template <typename T>
int launch_mfma(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    const bool fast = k % PK == 0 && n % 8 == 0 && aligned(a, kVecBytes) && aligned(b, kVecBytes) && aligned(c, kVecBytes) &&
                      k <= (1 << 22) && n <= (1 << 24);
    int64_t choice = tuning().matmul_tile;
    if (fast && choice == 0) {
        // 256x256 tiles halve the bytes every CU pulls through its vector cache per flop, but need
        // about one tile per CU to pay off.  Below that, 128x128 tiles (two workgroups per CU) as
        // long as they still give every CU a workgroup and a half; skinny outputs go to 128x64 or
        // 64x64 tiles so that all CUs (and their vector caches) take part.
        const int64_t cus = compute_units();
        auto tiles = [&](int tm, int tn) { return batch * ((m + tm - 1) / tm) * ((n + tn - 1) / tn); };
        if (tiles(256, 256) * 10 >= cus * 9) choice = 4;
        else if (tiles(128, 128) * 2 >= cus * 3) choice = 1;
        else if (tiles(128, 64) * 2 >= cus) choice = 2;
        else choice = 5;
    }
    if (fast) {
        switch (choice) {
        case 2: return launch_tile<T, 128, 64, 1>(a, b, c, batch, m, k, n, st);
        case 3: return launch_tile<T, 64, 128, 1>(a, b, c, batch, m, k, n, st);
        case 4: return launch_tile<T, 256, 256, 1>(a, b, c, batch, m, k, n, st);
        case 5: return launch_tile<T, 64, 64, 1>(a, b, c, batch, m, k, n, st);
        default: return launch_tile<T, 128, 128, 1>(a, b, c, batch, m, k, n, st);
        }
    }
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
template <typename T>
int launch_tiled(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    const int64_t tiles_m = (m + GT - 1) / GT, tiles_n = (n + GT - 1) / GT;
    const int64_t blocks = batch * tiles_m * tiles_n;
    if (blocks > 0x7fffffff) return DXH_ERR_SHAPE;
    matmul_tiled_kernel<T><<<(unsigned)blocks, kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, (int)tiles_m, (int)tiles_n);
    return launch_status();
}

template <int FM, int FN, int FK, int PD>
int launch_f32_tile(const float *a, const float *b, float *c, int64_t batch, int64_t m, int64_t k, int64_t n, bool vec, hipStream_t st) {
    TileMap map;
    if (!make_tile_map(batch, m, n, 64 * FM, 64 * FN, map)) return DXH_ERR_SHAPE;
    const unsigned blocks = (unsigned)(8 * map.chunk);
    if (vec) matmul_mfma_f32_kernel<FM, FN, FK, PD, true><<<blocks, kBlock, 0, st>>>(a, b, c, (int)m, (int)k, (int)n, map);
    else matmul_mfma_f32_kernel<FM, FN, FK, PD, false><<<blocks, kBlock, 0, st>>>(a, b, c, (int)m, (int)k, (int)n, map);
    return launch_status();
}

// fp32: the matrix pipe is the bound, so the tile is chosen for CU balance.  Cost model per tile
// shape: two workgroups share a CU; a CU's time is (rounds of two tiles) x tile flops / efficiency,
// where a last round that leaves at most one workgroup per CU counts 0.6 (a lone workgroup runs
// faster than two that share the pipe) and the efficiencies are the measured large-square rates
// relative to the 128x128 tile.  Small tiles take longer K steps and a deeper prefetch: with few
// MFMAs per step only that hides the global-load latency.
inline int launch_f32(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    const bool vec = k % 4 == 0 && n % 4 == 0 && n >= 4 && aligned(a, kVecBytes) && aligned(b, kVecBytes) && aligned(c, kVecBytes);
    const int64_t cus = compute_units();
    auto cost = [&](int tm, int tn, double eff) {
        const int64_t tiles = batch * ((m + tm - 1) / tm) * ((n + tn - 1) / tn);
        const int64_t full = tiles / (2 * cus), rem = tiles % (2 * cus);
        const double rounds = (double)full + (rem > cus ? 1.0 : rem > 0 ? 0.6 : 0.0);
        return rounds * (double)tm * (double)tn / eff;
    };
    const float *af = (const float *)a, *bf = (const float *)b;
    float *cf = (float *)c;
    int64_t choice = tuning().matmul_tile;
    if (choice == 0) {
        const double c1 = cost(128, 128, 1.0), c2 = cost(128, 64, 0.95), c3 = cost(64, 64, 0.86);
        choice = (c1 <= c2 && c1 <= c3) ? 1 : (c2 <= c3) ? 2 : 3;
    }
    switch (choice) {
    case 1: return launch_f32_tile<2, 2, 32, 1>(af, bf, cf, batch, m, k, n, vec, st);
    case 2: return launch_f32_tile<2, 1, 32, 2>(af, bf, cf, batch, m, k, n, vec, st);
    case 3: return launch_f32_tile<1, 1, 64, 2>(af, bf, cf, batch, m, k, n, vec, st);
    case 4: return launch_f32_tile<2, 2, 16, 1>(af, bf, cf, batch, m, k, n, vec, st);
    default: return launch_f32_tile<1, 1, 64, 2>(af, bf, cf, batch, m, k, n, vec, st);
    }
}

template <int FM, int FN>
int launch_f64_tile(const double *a, const double *b, double *c, int64_t batch, int64_t m, int64_t k, int64_t n, bool vec, hipStream_t st) {
    TileMap map;
    if (!make_tile_map(batch, m, n, 64 * FM, 64 * FN, map)) return DXH_ERR_SHAPE;
    const unsigned blocks = (unsigned)(8 * map.chunk);
    if (vec) matmul_mfma_f64_kernel<FM, FN, true><<<blocks, kBlock, 0, st>>>(a, b, c, (int)m, (int)k, (int)n, map);
    else matmul_mfma_f64_kernel<FM, FN, false><<<blocks, kBlock, 0, st>>>(a, b, c, (int)m, (int)k, (int)n, map);
    return launch_status();
}

// fp64 on the matrix pipe; tile chosen for CU balance like fp32 (efficiencies measured on 4096^3)
inline int launch_f64(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st) {
    const bool vec = k % 2 == 0 && n % 2 == 0 && n >= 2 && aligned(a, kVecBytes) && aligned(b, kVecBytes);
    const int64_t cus = compute_units();
    auto cost = [&](int tm, int tn, double eff) {
        const int64_t tiles = batch * ((m + tm - 1) / tm) * ((n + tn - 1) / tn);
        const int64_t full = tiles / (2 * cus), rem = tiles % (2 * cus);
        const double rounds = (double)full + (rem > cus ? 1.0 : rem > 0 ? 0.6 : 0.0);
        return rounds * (double)tm * (double)tn / eff;
    };
    const double *af = (const double *)a, *bf = (const double *)b;
    double *cf = (double *)c;
    int64_t choice = tuning().matmul_tile;
    if (choice == 0) {
        const double c1 = cost(128, 128, 1.0), c2 = cost(128, 64, 0.86), c3 = cost(64, 64, 0.95);
        choice = (c1 <= c2 && c1 <= c3) ? 1 : (c2 <= c3) ? 2 : 3;
    }
    switch (choice) {
    case 1: return launch_f64_tile<2, 2>(af, bf, cf, batch, m, k, n, vec, st);
    case 2: return launch_f64_tile<2, 1>(af, bf, cf, batch, m, k, n, vec, st);
    default: return launch_f64_tile<1, 1>(af, bf, cf, batch, m, k, n, vec, st);
    }
}

}  // namespace dxh

using namespace dxh;

extern "C" int dxh_matmul(int dtype, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n,
                          void *stream) {
    if (batch < 0 || m < 0 || k < 0 || n < 0) return DXH_ERR_ARG;
    if (m > 0x7fffffff || k > 0x7fffffff || n > 0x7fffffff) return DXH_ERR_SHAPE;
    const int es = dtype_size(dtype);
    if (!es || dtype == DXH_BOOL) return DXH_ERR_DTYPE;
    if (batch * m * n == 0) return DXH_OK;
    if (!c) return DXH_ERR_ARG;
    hipStream_t st = as_stream(stream);
    if (k == 0) {  // empty sum: a fill kernel rather than a memset node, so the call stays graph-capturable
        dxh_scalar zero = {0.0, 0};
        return dxh_constant(dtype, c, batch * m * n, zero, stream);
    }
    if (!a || !b) return DXH_ERR_ARG;
    if (!aligned(a, es) || !aligned(b, es) || !aligned(c, es)) return DXH_ERR_ALIGN;
    switch (dtype) {
    case DXH_BF16: return launch_mfma<bf16_t>(a, b, c, batch, m, k, n, st);
    case DXH_F16: return launch_mfma<f16_t>(a, b, c, batch, m, k, n, st);
    case DXH_F32: return launch_f32(a, b, c, batch, m, k, n, st);
    case DXH_F64: return launch_f64(a, b, c, batch, m, k, n, st);
    case DXH_I64: return launch_tiled<int64_t>(a, b, c, batch, m, k, n, st);
    case DXH_I32: return launch_tiled<int32_t>(a, b, c, batch, m, k, n, st);
    case DXH_I16: return launch_tiled<int16_t>(a, b, c, batch, m, k, n, st);
    case DXH_I8: return launch_tiled<int8_t>(a, b, c, batch, m, k, n, st);
    default: return DXH_ERR_DTYPE;
    }
}
