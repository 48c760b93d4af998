// matmul_half_dma.hip — bf16 / f16 GEMM on the matrix pipe with operands that travel from global
// memory straight into LDS (global_load_lds_dwordx4), never through vector registers.
//
// Same tiling idea as matmul_mfma_tile_kernel (matmul_half.hip): workgroup tile TM x TN, 4 waves in
// a 2 x 2 grid, v_mfma_f32_32x32x16_{bf16,f16} on (B^T, A^T), B transposed by the LDS read.  What
// differs is the pipeline.  The tile keeps NS K steps of DK (32 or 64) in LDS; the loads of K step
// t + NS - 1 are issued, one between every few MFMAs, while step t is multiplied, so NS - 1 steps
// of global latency are hidden without a register or an LDS store per 16 bytes.  LDS-direct loads
// fill LDS at the vector cache's 64 bytes per clock without taking read bandwidth from the
// fragment reads (ds_write_b128 at that rate leaves them 93 of 132 bytes per clock), and the
// kernel draws less power: 8192^3 ran at 1.97 GHz against 1.83 GHz for the register-staged one.
// One workgroup barrier per K step.
//
// LDS-direct loads write lane L's 16 bytes to (M0 base) + 16 L, a contiguous KiB per wave
// instruction, so the LDS image is chosen by which global address each lane fetches:
//   A stage  [TM rows][DK k]; 16-byte chunk c of row r sits at chunk c ^ ((r >> 2) & 3) in 64-byte
//            rows (DK 32) and at c ^ ((r >> 1) & 7) in 128-byte rows (DK 64): the 16 lanes of one
//            pass of a ds_read_b128 then cover 16 different bank groups.  DK 64 fetches whole
//            128-byte cache lines of A; DK 32 half lines, twice.
//   B stage  [DK k][TN n], rows of TN * 2 bytes; 64-byte group g of row k sits at group g ^ (k & 3)
//            (g ^ ((k >> 1) & 1) in the 128-byte rows of TN 64): the transposing read
//            (ds_read_b64_tr_b16) fetches 64 bytes of 4 consecutive rows per half wave, which then
//            fall on different banks.
// Requirements (checked by the launcher): K % DK == 0, N % 8 == 0, 16-byte aligned A, B, C.
#include "matmul_half_ops.hpp"

namespace dxh {

// One LDS-direct load: lane's 16 bytes from `base + off` land at LDS byte address lds + 16 * lane.
// The statement writes M0 and says so: the clobber puts a definition of M0 on the statement, which
// keeps the compiler's own M0 set-ups (dynamically indexed registers, its LDS-direct accesses) from
// being shared across it.  M0 is a reserved register, so the compiler remarks that it will not save
// it around the statement; nothing here needs that, hence the diagnostic is switched off for this
// one function.  No "memory" clobber: ordering against the LDS reads comes from the workgroup
// barriers around it, and the statement is volatile, so it stays between them.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void dma16(const void *base, uint32_t off, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds) : "m0");
}
#pragma clang diagnostic pop
template <int N> __device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N)); }

// NSPLIT = 2: the tile map holds two entries per output tile, each the same tile over one half of
// K.  A half stores its fp32 accumulators to `part` (its own 4 * TM * TN bytes, element e of lane t
// at [e * 256 + t]) and counts itself in `cnt[tile]`; the half that finds it is the second adds the
// other's partial tile to its own accumulators (a + b == b + a in fp32: the sum does not depend on
// which half came last), puts the counter back to zero and stores C.  The partials travel with
// device-scope stores and loads and the count follows a wait for the stores' acknowledgement, as in
// reduce_col_fused_kernel (reduce.hip).
template <typename T, int TM, int TN, int DK, int NS, int WN = 2, int NSPLIT = 0>
__global__ __launch_bounds__(kBlock, 1) void matmul_dma_kernel(const T *__restrict__ A, const T *__restrict__ B, T *__restrict__ C, int M, int K, int N,
                                                                TileMap map, float *part, unsigned *cnt, const SharedA multi, const int c_through) {
    // the four waves form a WM x WN grid over the tile: 2 x 2, or 1 x 4 for a tile height that is
    // a multiple of 32 but not of 64
    constexpr int WM = 4 / WN, WTM = TM / WM, WTN = TN / WN;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && (TN == 64 || TN == 128 || TN == 256) && (DK == 32 || DK == 64), "tile shape");
    constexpr int FM = WTM / 32, FN = WTN / 32;  // 32x32 MFMA tiles per wave along m and n
    constexpr int KS = DK / 16;                  // k-substeps (one MFMA depth each) per K step
    constexpr int A_ROWB = DK * 2;               // bytes of an A row in LDS
    // LDS-direct loads per lane and K step.  A tile whose KiB blocks do not divide by four waves is
    // rounded up: the waves left over fetch the last block once more (same data to the same place),
    // so that every wave has the same number of loads in flight and one vmcnt value fits all.
    constexpr int A_BLOCKS = TM * A_ROWB / 1024, A_INS = (A_BLOCKS + 3) / 4, B_INS = DK * TN * 2 / 4096;
    constexpr int NLD = A_INS + B_INS;
    constexpr int A_BYTES = TM * A_ROWB, B_ROWB = TN * 2, STAGE = A_BYTES + DK * B_ROWB;
    constexpr int LDC = TN + 8;
    constexpr int LDS_BYTES = (NS * STAGE > TM * LDC * 2) ? NS * STAGE : TM * LDC * 2;
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
    static_assert((NS - 2) * NLD <= 63, "vmcnt field");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];

    const TileCoord tc = tile_of_block(map);
    if (!tc.valid) return;
    const int m0 = tc.tm * TM, n0 = tc.tn * TN;
    const int t = threadIdx.x, lane = t & 63, w = __builtin_amdgcn_readfirstlane(t >> 6), wm = w / WN, wn = w % WN;
    int zb = tc.batch, slice = 0, kbeg = 0, KT = K / DK;
    if constexpr (NSPLIT > 0) {
        static_assert(NSPLIT == 0 || NSPLIT == 2, "two halves: their sum is the same in either order");
        zb = tc.batch / NSPLIT;
        slice = tc.batch - zb * NSPLIT;
        const int base = KT / NSPLIT, rem = KT - base * NSPLIT;  // K steps dealt out evenly; the launcher makes sure that base >= 1
        kbeg = slice * base + (slice < rem ? slice : rem);
        KT = base + (slice < rem ? 1 : 0);
    }
    // multi.count > 0: the tile map's batch index picks one of several B / C pairs that share the one A
    // (selected with compares: an index into the by-value argument would send it to per-lane memory)
    if (multi.count > 0) {
        B = reinterpret_cast<const T *>(zb == 0 ? multi.b[0] : zb == 1 ? multi.b[1] : zb == 2 ? multi.b[2] : multi.b[3]);
        C = reinterpret_cast<T *>(zb == 0 ? multi.c[0] : zb == 1 ? multi.c[1] : zb == 2 ? multi.c[2] : multi.c[3]);
        zb = 0;
    }
    const uint16_t *Ab = reinterpret_cast<const uint16_t *>(A) + ((int64_t)zb * M + m0) * K + (int64_t)kbeg * DK;
    const uint16_t *Bb = reinterpret_cast<const uint16_t *>(B) + ((int64_t)zb * K + (int64_t)kbeg * DK) * N + n0;
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;

    // ---- which 16 bytes each lane fetches (byte offsets from the tile's A / B origin at k = 0) ----
    // Rows past M and columns past N are clamped onto valid memory; their products land in
    // accumulator rows / columns that the epilogue never stores.
    uint32_t a_off[A_INS], b_off[B_INS];
    // A rows of 64 bytes (K step 32): a wave instruction covers 16 rows, chunk c of row r sits at
    // c ^ ((r >> 2) & 3).  Rows of 128 bytes (K step 64): 8 rows, chunk c at c ^ ((r >> 1) & 7).
    // Either way the 16 lanes of one pass of a ds_read_b128 fall on 16 different bank groups.
    uint32_t a_lds[A_INS];  // byte offset of the load's KiB block inside the A stage
    static_for<A_INS>([&](auto q) __attribute__((always_inline)) {
        const int blk = 4 * decltype(q)::value + w < A_BLOCKS ? 4 * decltype(q)::value + w : A_BLOCKS - 1;
        int r, c;
        if constexpr (DK == 32) { r = 16 * blk + (lane >> 2); c = (lane & 3) ^ ((r >> 2) & 3); }
        else { r = 8 * blk + (lane >> 3); c = (lane & 7) ^ ((r >> 1) & 7); }
        a_off[q] = ((uint32_t)(m0 + r < M ? r : M - 1 - m0) * (uint32_t)K + (uint32_t)c * 8u) * 2u;
        a_lds[q] = (uint32_t)blk * 1024u;
    });
    constexpr int LPR = TN / 8, RPB = 64 / LPR;  // lanes per B row, B rows per wave instruction
    // B rows of 256 bytes and more hold four 64-byte groups or a multiple: group g of row k sits at
    // g ^ (k & 3).  A 128-byte row (TN 64) has two: g ^ ((k >> 1) & 1), which still spreads the four
    // rows of a transposing read over all banks (rows k and k + 2 are 256 bytes apart).
    auto bswz = [](int k) __attribute__((always_inline)) { return TN >= 128 ? (k & 3) : ((k >> 1) & 1); };
    static_for<B_INS>([&](auto q) __attribute__((always_inline)) {
        const int r = RPB * (4 * decltype(q)::value + w) + lane / LPR, p = lane % LPR;
        const int col = (((p >> 2) ^ bswz(r)) * 4 + (p & 3)) * 8;
        b_off[q] = ((uint32_t)r * (uint32_t)N + (uint32_t)(n0 + col < N ? col : N - 8 - n0)) * 2u;
    });
    // load q of a K step: q < A_INS moves 16 rows of A, the others RPB rows of B
    auto issue_one = [&](auto q, uint32_t sa, const uint16_t *ag, const uint16_t *bg) __attribute__((always_inline)) {
        constexpr int i = decltype(q)::value;
        if constexpr (i < A_INS) dma16(ag, a_off[i], sa + a_lds[i]);
        else dma16(bg, b_off[i - A_INS], sa + w * 1024 + A_BYTES + (i - A_INS) * 4096);
    };
    auto issue = [&](int stage, int kstep) __attribute__((always_inline)) {
        const uint32_t sa = lds0 + stage * STAGE;
        const uint16_t *ag = Ab + kstep * DK, *bg = Bb + (int64_t)kstep * DK * N;
        static_for<NLD>([&](auto q) __attribute__((always_inline)) { issue_one(q, sa, ag, bg); });
    };

    // ---- fragment reads -----------------------------------------------------------------------
    const int sw = (lane >> 2) & 3, fch = lane >> 5;
    const int fa_base = (wm * WTM + (lane & 31)) * A_ROWB;
    const int swa = DK == 32 ? sw : (lane >> 1) & 7;  // the A row's swizzle term: rows of a wave tile start at multiples of 32
    int fa_ch[KS];  // byte offset of the lane's chunk in each substep
    static_for<KS>([&](auto ks) __attribute__((always_inline)) { fa_ch[ks] = ((2 * decltype(ks)::value + fch) ^ swa) * 16; });
    const int fb_base = A_BYTES + (8 * fch + sw) * B_ROWB + ((lane & 16) + 4 * (lane & 3)) * 2;
    int fb_g[FN];
    static_for<FN>([&](auto j) __attribute__((always_inline)) { fb_g[j] = ((wn * (WTN / 32) + decltype(j)::value) ^ bswz(sw)) * 64; });

    // fragment read r of a substep: r < FM is the A fragment of MFMA row r, the others are the low
    // and high half (k 0-3 and 4-7 of the lane's eight) of a B fragment
    u32x4 fa[2][FM], fb[2][FN];
    auto read_one = [&](auto buf, auto ks, const unsigned char *S, auto r) __attribute__((always_inline)) {
        constexpr int i = decltype(r)::value;
        if constexpr (i < FM) {
            fa[buf][i] = *reinterpret_cast<const u32x4 *>(S + fa_base + fa_ch[decltype(ks)::value] + i * 32 * A_ROWB);
        } else {
            constexpr int j = (i - FM) / 2, h = (i - FM) % 2;
            const uint16_t *p = reinterpret_cast<const uint16_t *>(S + fb_base + fb_g[j] + decltype(ks)::value * 16 * B_ROWB) + h * 4 * TN;
            const u32x2 v = lds_read_tr16(p);
            if constexpr (h == 0) { fb[buf][j].x = v.x; fb[buf][j].y = v.y; }
            else { fb[buf][j].z = v.x; fb[buf][j].w = v.y; }
        }
    };

    f32x16 acc[FM][FN];
    static_for<FM>([&](auto i) __attribute__((always_inline)) {
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;
        });
    });
    constexpr int NM = FM * FN, ND = FM + 2 * FN;
    auto mma = [&](auto buf, auto lo, auto hi) __attribute__((always_inline)) {
        static_for<decltype(hi)::value - decltype(lo)::value>([&](auto x) __attribute__((always_inline)) {
            constexpr int idx = decltype(lo)::value + decltype(x)::value, i = idx / FN, j = idx % FN;
            acc[i][j] = mfma32<T>(fb[buf][j], fa[buf][i], acc[i][j]);
        });
    };

    auto k_of = [&](int s) __attribute__((always_inline)) { return s < KT ? s : KT - 1; };
    // steps past the end fetch the last step again: the count of loads in flight stays the same
    // on every trip, and the copies land in stages that nobody reads any more
#pragma unroll
    for (int s = 0; s < NS - 1; ++s) issue(s, k_of(s));

    // K step t: its stage is complete once at most (NS - 2) steps' loads are still in flight; the
    // barrier makes every wave's part of it visible and tells that all waves are done with stage
    // t - 1, which the loads of step t + NS - 1 then overwrite.  Substep 1 of step t - 1 straddles
    // the barrier: its second half of MFMAs runs under the first fragment reads of step t.
    //
    // A phase of the K step: `nm` MFMAs of fragment buffer `mb` starting at `m0`, `nr` fragment
    // reads into buffer `rb` for substep `rks` starting at read `r0`, `nd` loads starting at load
    // `d0`, cut into groups of (one load, a few MFMAs, their share of the reads) whose order is
    // pinned.  Spreading the loads matters: four waves that issue all their loads at once right
    // after the barrier wait on the vector memory queue instead of feeding the matrix pipe
    // (8192^3: matrix pipe 62 % busy with the loads in one burst, 870 -> 785 us spread out).
    int stage = 0, fill = NS - 1;
    uint32_t sa_fill = 0;
    const uint16_t *ag_fill = Ab, *bg_fill = Bb;
    const unsigned char *S_cur = lds;
    auto phase = [&](auto mb, auto m0_, auto nm_, auto rb, auto rks, auto r0_, auto nr_, auto d0_, auto nd_) __attribute__((always_inline)) {
        constexpr int m0 = decltype(m0_)::value, nm = decltype(nm_)::value, r0 = decltype(r0_)::value, nr = decltype(nr_)::value;
        constexpr int d0 = decltype(d0_)::value, nd = decltype(nd_)::value;
        constexpr int G = nd > 0 ? nd : 1;  // groups
        static_for<G>([&](auto g_) __attribute__((always_inline)) {
            constexpr int g = decltype(g_)::value;
            constexpr int ma = nm * g / G, mz = nm * (g + 1) / G, ra = nr * g / G, rz = nr * (g + 1) / G;
            if constexpr (nd > 0) issue_one(ic<d0 + g>{}, sa_fill, ag_fill, bg_fill);
            static_for<rz - ra>([&](auto x) __attribute__((always_inline)) { read_one(rb, rks, S_cur, ic<r0 + ra + decltype(x)::value>{}); });
            mma(mb, ic<m0 + ma>{}, ic<m0 + mz>{});
            if constexpr (mz > ma) interleave(ic<mz - ma>{}, ic<rz - ra>{}, ic<0>{}, ic<0>{});
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    // The K step as phases: [second half of the previous step's last substep | first reads of this
    // step], then one phase per substep but the last [its MFMAs | the next substep's reads], then
    // [first half of the last substep].  Loads are dealt out in proportion to the MFMAs of a phase.
    constexpr int TOTAL = KS * NM;                                      // MFMAs per K step
    constexpr auto load_at = [](int mfmas_before) { return NLD * mfmas_before / TOTAL; };
    constexpr int H = NM / 2;                                           // MFMAs after the barrier of the straddling substep
    auto enter = [&](int kt) __attribute__((always_inline)) {
        wait_loads<(NS - 2) * NLD>();
        __syncthreads();
        const int ks = k_of(kt + NS - 1);
        sa_fill = lds0 + fill * STAGE;
        ag_fill = Ab + ks * DK;
        bg_fill = Bb + (int64_t)ks * DK * N;
        S_cur = lds + stage * STAGE;
    };
    auto rest = [&]() __attribute__((always_inline)) {
        static_for<KS - 1>([&](auto ks_) __attribute__((always_inline)) {
            constexpr int ks = decltype(ks_)::value, before = (NM - H) + ks * NM;
            phase(ic<ks & 1>{}, ic<0>{}, ic<NM>{}, ic<(ks + 1) & 1>{}, ic<ks + 1>{}, ic<0>{}, ic<ND>{}, ic<load_at(before)>{},
                  ic<load_at(before + NM) - load_at(before)>{});
        });
        constexpr int before = (NM - H) + (KS - 1) * NM;
        phase(ic<(KS - 1) & 1>{}, ic<0>{}, ic<H>{}, ic<0>{}, ic<0>{}, ic<0>{}, ic<0>{}, ic<load_at(before)>{}, ic<NLD - load_at(before)>{});
        stage = stage + 1 == NS ? 0 : stage + 1;
        fill = fill + 1 == NS ? 0 : fill + 1;
    };
    enter(0);
    // first step: nothing to multiply yet under the first fragment reads
    phase(ic<1>{}, ic<0>{}, ic<0>{}, ic<0>{}, ic<0>{}, ic<0>{}, ic<ND>{}, ic<0>{}, ic<load_at(NM - H)>{});
    rest();
    for (int kt = 1; kt < KT; ++kt) {
        enter(kt);
        phase(ic<(KS - 1) & 1>{}, ic<H>{}, ic<NM - H>{}, ic<0>{}, ic<0>{}, ic<0>{}, ic<ND>{}, ic<0>{}, ic<load_at(NM - H)>{});
        rest();
    }
    mma(ic<(KS - 1) & 1>{}, ic<H>{}, ic<NM>{});
    wait_loads<0>();  // the refetched tail steps must have landed before the C tile reuses the LDS
    __syncthreads();

    if constexpr (NSPLIT > 0) {
        __shared__ int is_last;
        constexpr int E = NM * 16;  // accumulators per lane
        const int tile = (zb * map.tiles_m + tc.tm) * map.tiles_n + tc.tn;
        float *P = part + (int64_t)tile * NSPLIT * E * kBlock + t;
        float *mine = P + (int64_t)slice * E * kBlock;
        const float *other = P + (int64_t)(1 - slice) * E * kBlock;
        static_for<NM>([&](auto x) __attribute__((always_inline)) {
            constexpr int i = decltype(x)::value / FN, j = decltype(x)::value % FN;
#pragma unroll
            for (int v = 0; v < 16; ++v)
                __hip_atomic_store(mine + (decltype(x)::value * 16 + v) * kBlock, acc[i][j][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        });
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stores are in memory before the barrier, hence before the count
        __syncthreads();
        if (t == 0) {
            const unsigned old = __hip_atomic_fetch_add(cnt + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const int last = old == (unsigned)(NSPLIT - 1);
            if (last) __hip_atomic_store(cnt + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            is_last = last;
        }
        __syncthreads();
        if (!is_last) return;
        __atomic_signal_fence(__ATOMIC_SEQ_CST);  // the loads below stay below the count
        float got[NM][16];  // every load is issued before the first is used: one memory round trip, not NM
        static_for<NM>([&](auto x) __attribute__((always_inline)) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
                got[decltype(x)::value][v] = __hip_atomic_load(other + (decltype(x)::value * 16 + v) * kBlock, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        });
        static_for<NM>([&](auto x) __attribute__((always_inline)) {
            constexpr int i = decltype(x)::value / FN, j = decltype(x)::value % FN;
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] += got[decltype(x)::value][v];
        });
    }

    // ---- epilogue: result lane holds row m = lane%32 of its MFMA tile and, per group g of 4
    // registers, columns 8g + 4*(lane/32) .. +3: one 8-byte LDS store each, then 16-byte row stores
    uint16_t *Cs = reinterpret_cast<uint16_t *>(lds);
    static_for<FM>([&](auto i) __attribute__((always_inline)) {
        static_for<FN>([&](auto j) __attribute__((always_inline)) {
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int row = wm * WTM + 32 * i + (lane & 31);
                const int col = wn * WTN + 32 * j + 8 * g + 4 * (lane >> 5);
                *reinterpret_cast<u32x2 *>(Cs + row * LDC + col) =
                    u32x2{pack2<T>(acc[i][j][4 * g], acc[i][j][4 * g + 1]), pack2<T>(acc[i][j][4 * g + 2], acc[i][j][4 * g + 3])};
            }
        });
    });
    __syncthreads();
    uint16_t *Cr = reinterpret_cast<uint16_t *>(C) + (int64_t)zb * M * N;
    constexpr int CB = TN / 8;
#pragma unroll
    for (int i = 0; i < TM * CB / kBlock; ++i) {
        const int c = t + i * kBlock, row = c / CB, ch = c % CB;
        const int gm = m0 + row, gn = n0 + ch * 8;
        if (gm < M && gn < N) {  // N % 8 == 0: a chunk is either fully inside or fully outside
            uint4 *dst = reinterpret_cast<uint4 *>(Cr + (int64_t)gm * N + gn);
            const uint4 piece = *reinterpret_cast<const uint4 *>(Cs + row * LDC + ch * 8);
            if (c_through) st_mode<2>(dst, piece); else st_nt(dst, piece);  // c_store_through: will the next kernel find C in the last-level cache
        }
    }
}

template <typename T, int TM, int TN, int DK, int NS, int WN = 2>
static int launch_dma_tile(const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, const SharedA &multi) {
    TileMap map;
    if (!make_tile_map(multi.count > 0 ? multi.count : batch, m, n, TM, TN, map)) return DXH_ERR_SHAPE;
    matmul_dma_kernel<T, TM, TN, DK, NS, WN><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, map, nullptr, nullptr, multi, c_store_through(multi.count > 0 ? multi.count : batch, m, n, sizeof(T)));
    return launch_status();
}

// 128x128 (wide: 128x256) tiles, each cut into two halves of K that meet in `part` (dma_split_bytes) and `cnt` (one
// zeroed counter per output tile, left zero).
template <typename T>
static int launch_dma_split(int wide, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, float *part, unsigned *cnt, hipStream_t st) {
    TileMap map;
    if (!make_tile_map(batch * 2, m, n, 128, wide ? 256 : 128, map)) return DXH_ERR_SHAPE;
    if (wide) matmul_dma_kernel<T, 128, 256, 64, 3, 4, 2><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, map, part, cnt, SharedA{}, c_store_through(batch, m, n, sizeof(T)));
    else matmul_dma_kernel<T, 128, 128, 64, 3, 2, 2><<<(unsigned)(8 * map.chunk), kBlock, 0, st>>>((const T *)a, (const T *)b, (T *)c, (int)m, (int)k, (int)n, map, part, cnt, SharedA{}, c_store_through(batch, m, n, sizeof(T)));
    return launch_status();
}

// shape: 0 = 256x256 in K steps of 32, 1 = 192x256 / 32, 2 = 128x64 / 64, 3 = 256x256 / 64, 4 = 160x256 / 64 and
// 5 = 128x256 / 64 with the waves side by side, 6 = 256x128 / 64.  The caller has
// checked K % 64 == 0, N % 8 == 0, the alignment of a, b, c and that every byte offset inside a tile
// fits 32 bits.
template <typename T>
static int launch_dma_shape(int shape, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, const SharedA &multi) {
    switch (shape) {
    case 0: return launch_dma_tile<T, 256, 256, 32, 4>(a, b, c, batch, m, k, n, st, multi);
    case 1: return launch_dma_tile<T, 192, 256, 32, 5>(a, b, c, batch, m, k, n, st, multi);
    case 3: return launch_dma_tile<T, 256, 256, 64, 2>(a, b, c, batch, m, k, n, st, multi);
    case 4: return launch_dma_tile<T, 160, 256, 64, 3, 4>(a, b, c, batch, m, k, n, st, multi);
    case 5: return launch_dma_tile<T, 128, 256, 64, 3, 4>(a, b, c, batch, m, k, n, st, multi);
    case 6: return launch_dma_tile<T, 256, 128, 64, 3>(a, b, c, batch, m, k, n, st, multi);
    default: return launch_dma_tile<T, 128, 64, 64, 5>(a, b, c, batch, m, k, n, st, multi);
    }
}
int launch_matmul_half_dma_split(int dtype, int wide, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, float *part, unsigned *cnt, hipStream_t st) {
    return dtype == DXH_BF16 ? launch_dma_split<bf16_t>(wide, a, b, c, batch, m, k, n, part, cnt, st) : launch_dma_split<f16_t>(wide, a, b, c, batch, m, k, n, part, cnt, st);
}
int launch_matmul_half_dma(int dtype, int shape, const void *a, const void *b, void *c, int64_t batch, int64_t m, int64_t k, int64_t n, hipStream_t st, const SharedA &multi) {
    return dtype == DXH_BF16 ? launch_dma_shape<bf16_t>(shape, a, b, c, batch, m, k, n, st, multi) : launch_dma_shape<f16_t>(shape, a, b, c, batch, m, k, n, st, multi);
}

}  // namespace dxh
