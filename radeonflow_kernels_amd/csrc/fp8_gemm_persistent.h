// Persistent form of gemm_fp8_blockscale_tile: one workgroup per compute unit walks its tiles (id, id + grid,
// id + 2*grid, ...) and runs ONE software pipeline over the concatenated K blocks of all of them.
//
// What it buys: in the one-workgroup-per-tile kernel every tile pays for a cold start (first stage loaded with
// nothing to overlap, ~2 us), for two redundant prefetches at its end and for a workgroup launch. Here the loads of
// the next tile's first two K blocks are simply the next loads of the pipeline: they are in flight while the last
// K blocks of the current tile compute, its first fragments are fetched in the last slots of the current tile, and
// the bf16 store of the finished tile runs from a private LDS region while the next stage is already resident.
// Tiles with few K blocks (K = 256: two per tile) gain the most.
//
// Restrictions (checked by the host): M >= BM, M % 16 == 0 and N % BN == 0 (per-lane load offsets are
// tile-independent, the tile origin lives in the scalar base pointers: every tile is a whole tile), K/128 even (a
// tile starts on LDS stage 0). When M is not a multiple of BM the last row of tiles starts at row M - BM instead of
// tiles_m * BM - BM: it overlaps the row of tiles before it, both compute the rows they share from the same operands
// with the same instructions and store the same values. M_store <= M is the number of rows of C that exist (a caller
// whose M is not a multiple of 16 passes A and a_scale padded to M rows and its own C). Numerics and the per-tile
// instruction schedule are those of tile_mainloop.
#pragma once
#include "fp8_gemm_kernels.h"

namespace rf {

template <int BM, int BN, int WAVES_M, int WAVES_N>
struct PersistentGeom {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    static constexpr int STORE_PASSES = G::TM;           // one m-tile (16 rows) per pass: 2.25 KiB per wave
    using S = StoreGeom<BM, BN, WAVES_M, WAVES_N, STORE_PASSES>;
    static constexpr int STAGING_OFF = 2 * G::STAGE + 16;
    static constexpr int LDS_BYTES = STAGING_OFF + G::NW * S::REGION;
    static_assert(LDS_BYTES <= 160 * 1024, "stages + private store regions fit the CU's LDS");
};

// HALF_TAIL (256 x 256 tiles): the grid's workgroups take the whole rounds only (the first T - T % grid tiles), and the
// T % grid tiles that are left are finished as 128 x 256 half tiles, one per workgroup, by the three-stage loop of
// tile_mainloop: a last round that is at most half full then takes about half a tile's time instead of a whole one
// (8192 x 4608 x 7168 is 576 tiles on 256 CUs: 2.25 rounds). Left-over tile i (0 <= i < R) is split between workgroups
// i and i + R8, R8 = R rounded up to a multiple of 8, so that both run on the XCD whose region the tile belongs to;
// the host checks 0 < R and R8 + R <= grid.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool HALF_TAIL = false>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_fp8_blockscale_persistent(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, uint16_t *__restrict__ C, int M, int N, int K, int tiles_m, int tiles_n,
    int group_m, int M_store) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    using P = PersistentGeom<BM, BN, WAVES_M, WAVES_N>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    constexpr int NW = G::NW, WM = G::WM, WN = G::WN, TM = G::TM, TN = G::TN;
    constexpr int STAGE_A = G::STAGE_A, STAGE_B = G::STAGE_B, STAGE_S = G::STAGE_S;
    constexpr int OFF_B = 2 * STAGE_A, OFF_S = 2 * STAGE_A + 2 * STAGE_B, OFF_SB = BM * 4;
    static_assert(STAGE_A + 3 * 8 * BM + 16 * (BM / 16) < 65536 && STAGE_B + 3 * 8 * BN + 16 * (BN / 16) < 65536,
                  "stage offsets must fit the immediate offset of an LDS read");
    constexpr int INST_A = STAGE_A / 1024 / NW, INST_B = STAGE_B / 1024 / NW;
    constexpr int NSC = BM / 64;
    static_assert(STAGE_A % (1024 * NW) == 0 && STAGE_B % (1024 * NW) == 0, "loads must divide evenly over waves");
    static_assert(NSC <= NW && WN <= 128 && 128 % WN == 0 && TM % 4 == 0, "same tile constraints as tile_mainloop");
    constexpr int CPR_A = BM / 16, CPR_B = BN / 16, RPI_A = 1024 / BM, RPI_B = 1024 / BN;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int L = lane & 15, g = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const int QK = K / BK, QN = (N + 127) / 128;
    const int T = tiles_m * tiles_n;
    const int my_tiles = HALF_TAIL ? T / (int)gridDim.x :                               // >= 1: grid <= T
        __builtin_amdgcn_readfirstlane((T - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x);

    // Origin of this workgroup's r-th tile; past the end it repeats the last one (prefetches that nobody uses). The map
    // from tile ordinal to tile costs a handful of integer divisions on the vector unit, and the two load cursors and
    // the store each need it once per tile: with two K blocks per tile that was a tenth of the launch (6144 x 7168 x
    // 256: 25.4 -> 23.2 us). So lane r works out the origin of tile r once, before the loop, and a tile boundary only
    // reads that lane.
    int m0_of_lane, n0_of_lane;
    {
        int tm, tn;
        const int r = lane < my_tiles - 1 ? lane : my_tiles - 1;
        tile_of_block(blockIdx.x + r * gridDim.x, T, tiles_m, tiles_n, group_m, true, tm, tn);
        m0_of_lane = tm * BM < M - BM ? tm * BM : M - BM;
        n0_of_lane = tn * BN;
    }
    auto tile_origin = [&](int r, int &m0, int &n0) {
        if (r > my_tiles - 1) r = my_tiles - 1;
        if (r < 64) {
            m0 = __builtin_amdgcn_readlane(m0_of_lane, r);
            n0 = __builtin_amdgcn_readlane(n0_of_lane, r);
        } else {
            int tm, tn;
            tile_of_block(blockIdx.x + r * gridDim.x, T, tiles_m, tiles_n, group_m, true, tm, tn);
            m0 = __builtin_amdgcn_readfirstlane(tm * BM < M - BM ? tm * BM : M - BM);
            n0 = __builtin_amdgcn_readfirstlane(tn * BN);
        }
    };

    // ---- global -> LDS: per-lane offsets inside a K block, relative to the tile origin (see tile_mainloop) ----
    constexpr int PER_A = (8 / RPI_A) > 0 ? (8 / RPI_A) : 1, PER_B = (8 / RPI_B) > 0 ? (8 / RPI_B) : 1;
    constexpr int GRP_A = (INST_A * RPI_A + 31) / 32, GRP_B = (INST_B * RPI_B + 31) / 32;
    constexpr int NCLS_A = (PER_A < INST_A ? PER_A : INST_A) * GRP_A, NCLS_B = (PER_B < INST_B ? PER_B : INST_B) * GRP_B;
    static_assert((INST_A * RPI_A) % 32 == 0 || INST_A * RPI_A < 32, "a wave's rows cover whole 32-row groups");
    static_assert((INST_B * RPI_B) % 32 == 0 || INST_B * RPI_B < 32, "a wave's rows cover whole 32-row groups");
    auto cls_a = [](int i) { return i % PER_A + PER_A * (i * RPI_A / 32); };
    auto rep_a = [](int c) { return c % PER_A + (c / PER_A) * (32 / RPI_A); };
    auto cls_b = [](int i) { return i % PER_B + PER_B * (i * RPI_B / 32); };
    auto rep_b = [](int c) { return c % PER_B + (c / PER_B) * (32 / RPI_B); };
    uint32_t goff_a[NCLS_A], goff_b[NCLS_B], goff_s, goff_sb;
#pragma unroll
    for (int c_ = 0; c_ < NCLS_A; c_++) {
        const int kl = (wave * INST_A + rep_a(c_)) * RPI_A + lane / CPR_A;
        const int c = (lane % CPR_A) ^ swizzle_of_row<BM>(kl);
        goff_a[c_] = (uint32_t)(lane / CPR_A) * (uint32_t)M + (uint32_t)(c * 16);
    }
#pragma unroll
    for (int c_ = 0; c_ < NCLS_B; c_++) {
        const int kl = (wave * INST_B + rep_b(c_)) * RPI_B + lane / CPR_B;
        const int c = (lane % CPR_B) ^ swizzle_of_row<BN>(kl);
        goff_b[c_] = (uint32_t)(lane / CPR_B) * (uint32_t)N + (uint32_t)(c * 16);
    }
    {
        const int sl = (wave < NSC ? wave : 0) * 64 + lane, r = sl % WM;
        goff_s = (uint32_t)((sl / WM) * WM + 16 * (r % TM) + r / TM) * 4u;
        // b_scale slots: the tile's column blocks (N is a multiple of BN here, so they all exist); the other lanes
        // repeat the last one
        constexpr int NBLK = BN / 128 > 0 ? BN / 128 : 1;
        goff_sb = (uint32_t)(lane < NBLK ? lane : NBLK - 1) * 4u;
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)(RF_LDS uint8_t *)lds;
    constexpr int D_SA = INST_A + INST_B, D_SB = D_SA + 1, NDMA = D_SB + 1;
    const uint32_t lds_dst_a = lds_base + wave * (INST_A * 1024), lds_dst_b = lds_base + OFF_B + wave * (INST_B * 1024),
                   lds_dst_s = lds_base + OFF_S + wave * 256, lds_dst_sb = lds_base + OFF_S + OFF_SB;
    auto dma_src = [&](int d, int m0, int n0, int kb) -> const uint8_t * {
        if (d < INST_A) return A + ((size_t)kb * BK + (size_t)(wave * INST_A + d) * RPI_A) * M + m0;
        if (d < D_SA) return B + ((size_t)kb * BK + (size_t)(wave * INST_B + (d - INST_A)) * RPI_B) * N + n0;
        if (d == D_SA) return (const uint8_t *)(SA + (size_t)kb * M + m0);
        return (const uint8_t *)(SB + (size_t)kb * QN + (n0 >> 7));
    };
    auto dma_step = [&](int d) -> size_t {
        return d < INST_A ? (size_t)BK * M : d < D_SA ? (size_t)BK * N : d == D_SA ? (size_t)M * 4 : (size_t)QN * 4;
    };
    auto issue_dma = [&](int d, int stage, const uint8_t *src) {
        if (d < INST_A) {
            asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :: "v"(goff_a[cls_a(d < INST_A ? d : 0)]), "s"(src), "s"(lds_dst_a), "n"(d * 1024 + stage * STAGE_A)
                         : "memory", "scc");
        } else if (d < D_SA) {
            const int e = d - INST_A < INST_B ? d - INST_A : 0;
            asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :: "v"(goff_b[cls_b(e >= 0 ? e : 0)]), "s"(src), "s"(lds_dst_b), "n"(e * 1024 + stage * STAGE_B)
                         : "memory", "scc");
        } else if (d == D_SA) {
            if (wave < NSC)
                asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                             :: "v"(goff_s), "s"(src), "s"(lds_dst_s), "n"(stage * STAGE_S) : "memory", "scc");
        } else if (wave == 0) {
            asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                         :: "v"(goff_sb), "s"(src), "s"(lds_dst_sb), "n"(stage * STAGE_S) : "memory", "scc");
        }
    };
    // Two stages: the wait before the barrier is for every load this wave has issued (the three-stage form of
    // tile_mainloop, which waits for all but the newest block's loads, has no persistent counterpart: a tile would
    // have to start on any of three stages).
    auto wait_for_stage = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

    // ---- LDS -> MFMA operands (see tile_mainloop) ----
    const int krow = 32 * g + (L >> 1);
    static_assert((TM & (TM - 1)) == 0 && (TN & (TN - 1)) == 0, "tile counts are powers of two");
    const uint32_t aoff_base = krow * BM + (((wm * TM) ^ swizzle_of_row<BM>(krow)) << 4) + 8 * (L & 1);
    const uint32_t boff_base = OFF_B + krow * BN + (((wn * TN) ^ swizzle_of_row<BN>(krow)) << 4) + 8 * (L & 1);
    const uint32_t soff = OFF_S + (wm * WM + L * TM) * 4;
    const uint32_t sboff = OFF_S + OFF_SB + (((wn * WN) >> 7) << 2);    // n0 is a multiple of BN: block inside the tile

    constexpr int PR = 4, LAG = 3, NMFMA = TM * TN, BAR_SLOT = (TM - 1) * TN;
    static_assert(LAG < TN && LAG < PR && TM % 2 == 0 && NDMA - TN <= BAR_SLOT, "same schedule as tile_mainloop");

    f32x4 acc[TM][TN];
    i32x8 bfrag[TN], afrag[2];
    f32x4 pring[PR];
    float s[TM], sraw[TM], sb_raw = 0.f;
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
        for (int i = 0; i < TN; i++) acc[j][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < PR; r++) pring[r] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < TM; j++) s[j] = 0.f;

    auto rd = [&](uint32_t stage_base, uint32_t off) {
        return __builtin_amdgcn_ds_read_tr8_b64_v2i32((RF_LDS i32x2 *)(lds + stage_base + off));
    };
    auto read_bfrag = [&](int i, int stage) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            i32x2 v = rd(stage * STAGE_B, (boff_base ^ (i << 4)) + t * 8 * BN);
            bfrag[i][2 * t] = v[0];
            bfrag[i][2 * t + 1] = v[1];
        }
    };
    auto read_afrag = [&](int buf, int j, int stage) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            i32x2 v = rd(stage * STAGE_A, (aoff_base ^ (j << 4)) + t * 8 * BM);
            afrag[buf][2 * t] = v[0];
            afrag[buf][2 * t + 1] = v[1];
        }
    };
    auto read_scales = [&](int stage) {
#pragma unroll
        for (int q = 0; q < TM / 4; q++) {
            f32x4 v = *(RF_LDS f32x4 *)(lds + stage * STAGE_S + soff + q * 16);
#pragma unroll
            for (int e = 0; e < 4; e++) sraw[4 * q + e] = v[e];
        }
        sb_raw = *(RF_LDS float *)(lds + stage * STAGE_S + sboff);
    };

    // ---- two load cursors run ahead of the compute position ----
    // cursor 1 = the K block after the current one (DMA instructions d >= TN, issued in the first slots of a step);
    // cursor 2 = two blocks ahead (instructions d < TN, issued after the barrier). Each holds its tile ordinal, K block
    // and the source pointers of its instructions; crossing into the next tile recomputes the pointers from that
    // tile's origin.
    // BY_OPERAND: the cursors split the instructions by operand (cursor 2 = the A rows, cursor 1 = the B rows and the
    // scales), so each per-lane offset register belongs to one cursor and can carry that cursor's K position: a step
    // is then a handful of 32-bit vector adds beside the MFMAs, the scalar pointers stay at the tile's first K block,
    // and the ten 64-bit scalar additions per K block (a burst of scalar work after the last slot) are gone. The
    // offsets stay below K * M and K * N, which the host keeps under 2^32 for this kernel.
    constexpr bool BY_OPERAND = TN == INST_A;
    const uint32_t step_a = (uint32_t)BK * (uint32_t)M, step_b = (uint32_t)BK * (uint32_t)N, step_s = (uint32_t)M * 4u,
                   step_sb = (uint32_t)QN * 4u;
    const uint8_t *dsrc[NDMA];
    int c1_r = 0, c1_kb = 0, c2_r = 0, c2_kb = 0;     // set below
    auto shift_offsets = [&](int which, int blocks) {  // BY_OPERAND: move a cursor's per-lane offsets by `blocks` K blocks
        if (which == 2) {
#pragma unroll
            for (int c_ = 0; c_ < NCLS_A; c_++) goff_a[c_] += (uint32_t)blocks * step_a;
        } else {
#pragma unroll
            for (int c_ = 0; c_ < NCLS_B; c_++) goff_b[c_] += (uint32_t)blocks * step_b;
            goff_s += (uint32_t)blocks * step_s;
            goff_sb += (uint32_t)blocks * step_sb;
        }
    };
    // point a cursor's instructions at (tile r, block kb); from_kb = the block its offsets stand at (BY_OPERAND)
    auto seek = [&](int which, int r, int kb, int from_kb) {
        int m0, n0;
        tile_origin(r, m0, n0);
#pragma unroll
        for (int d = 0; d < NDMA; d++)
            if ((d >= TN) == (which == 1)) dsrc[d] = dma_src(d, m0, n0, BY_OPERAND ? 0 : kb);
        if constexpr (BY_OPERAND) shift_offsets(which, kb - from_kb);
    };
    auto advance = [&](int which, int &r, int &kb) {   // move a cursor one K block on
        if (kb + 1 < QK) {
            kb += 1;
            if constexpr (BY_OPERAND) {
                shift_offsets(which, 1);
            } else {
#pragma unroll
                for (int d = 0; d < NDMA; d++)
                    if ((d >= TN) == (which == 1)) dsrc[d] += dma_step(d);
            }
        } else {
            r += 1;
            seek(which, r, 0, kb);
            kb = 0;
        }
    };

    int m0_cur, n0_cur;
    tile_origin(0, m0_cur, n0_cur);
    {
        // cold start: stage 0 <- block 0 of the first tile, then its first operands; stage 1 <- start of block 1
#pragma unroll
        for (int d = 0; d < NDMA; d++) issue_dma(d, 0, dma_src(d, m0_cur, n0_cur, 0));
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        read_bfrag(0, 0);
        read_afrag(0, 0, 0);
        read_scales(0);
#pragma unroll
        for (int i = 1; i < TN; i++) read_bfrag(i, 0);
        // cursor 2 issues its part of block 1 here and moves on to block 2 (or the next tile); cursor 1 stands at
        // block 1 (QK >= 2)
        c2_r = 0; c2_kb = 1;
        seek(2, 0, 1, 0);
#pragma unroll
        for (int d = 0; d < TN && d < NDMA; d++) issue_dma(d, 1, dsrc[d]);
        advance(2, c2_r, c2_kb);
        c1_r = 0; c1_kb = 1;
        seek(1, 0, 1, 0);
        // like every first K block of a tile, the one that follows finds cursor 1's loads already issued
#pragma unroll
        for (int d = TN; d < NDMA; d++) issue_dma(d, 1, dsrc[d]);
    }

    // store instructions per wave of an unmasked tile store (store_whole_tile_bf16: one m-tile per pass, whole rows)
    constexpr int NST = whole_tile_store_instructions<BM, BN, WAVES_M, WAVES_N>();
    static_assert(NST <= 48, "the count must fit the wait instruction's field with room for the loads");
    bool stores_behind = false;          // the newest NST vector memory instructions of this wave are a tile's stores

    // one K block of the current tile; cur = the LDS stage it reads
    // first_c: the first K block of a tile, whose cursor-1 loads have been issued already (before the previous tile's
    // store, see below)
    auto k_block = [&](auto cur_c, auto first_c) {
        constexpr int cur = decltype(cur_c)::value, nxt = 1 - cur;
        constexpr bool first = decltype(first_c)::value != 0;
        const float s_last = s[TM - 1];
#pragma unroll
        for (int j = 0; j < TM; j++) s[j] = sraw[j] * sb_raw;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NMFMA; t++) {
            const int j = t / TN, i = t % TN;
            if (t == BAR_SLOT) {
                // The first K block of a tile that follows a stored tile: the loads it waits for were all issued
                // before that tile's stores, a wave's vector memory instructions complete in the order it issued
                // them (loads and stores alike), so "all but the newest NST" are exactly the loads. The stores'
                // acknowledgements (written through: about a microsecond under load) then have until the next K
                // block's wait.
                if (first && stores_behind) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NST) : "memory");
                else wait_for_stage();
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            pring[t % PR] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                bfrag[i], afrag[j & 1], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            asm volatile("" : "+v"(pring[t % PR]));
            __builtin_amdgcn_sched_barrier(0);
            if (!first && t + TN < NDMA) issue_dma(t + TN, nxt, dsrc[t + TN]);             // cursor 1
            if (t >= BAR_SLOT && t - BAR_SLOT < NDMA && t - BAR_SLOT < TN)
                issue_dma(t - BAR_SLOT, cur, dsrc[t - BAR_SLOT]);                          // cursor 2
            if (j + 1 < TM) {
                if (i == 0) read_afrag((j + 1) & 1, j + 1, cur);
            } else {
                read_bfrag(i, nxt);
                if (i == 0) {
                    read_afrag(0, 0, nxt);
                    read_scales(nxt);
                }
            }
            if (t >= LAG) {
                const int u = t - LAG, ju = u / TN, iu = u % TN;
#pragma unroll
                for (int e = 0; e < 4; e++) acc[ju][iu][e] = __builtin_fmaf(s[ju], pring[u % PR][e], acc[ju][iu][e]);
                asm volatile("" : "+v"(acc[ju][iu]));
            } else {
                const int u = NMFMA + t - LAG, ju = u / TN, iu = u % TN;
#pragma unroll
                for (int e = 0; e < 4; e++) acc[ju][iu][e] = __builtin_fmaf(s_last, pring[u % PR][e], acc[ju][iu][e]);
                asm volatile("" : "+v"(acc[ju][iu]));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        advance(1, c1_r, c1_kb);
        advance(2, c2_r, c2_kb);
    };

    for (int r = 0; r < my_tiles; r++) {
        k_block(IntTag<0>{}, IntTag<1>{});
        k_block(IntTag<1>{}, IntTag<0>{});
        for (int kb = 2; kb < QK; kb += 2) {
            k_block(IntTag<0>{}, IntTag<0>{});
            k_block(IntTag<1>{}, IntTag<0>{});
        }
        // the tile is complete: fold what the last K block still owes, store, start the next tile from zero. The
        // operands of the next tile's first K block are already in registers, its second block is on its way.
#pragma unroll
        for (int t = 0; t < LAG; t++) {
            const int u = NMFMA + t - LAG, ju = u / TN, iu = u % TN;
#pragma unroll
            for (int e = 0; e < 4; e++) acc[ju][iu][e] = __builtin_fmaf(s[TM - 1], pring[u % PR][e], acc[ju][iu][e]);
        }
        // The rest of the next tile's second K block (cursor 1; stage 1 is free since the last barrier) is asked for
        // before this tile's stores and not in the first slots of the next K block: the memory pipeline of the CU
        // takes instructions in order, and loads queued behind 128 KB of stores held up every wave at the start of
        // the next tile (with two K blocks per tile: 0.7 us of each tile's 4.4).
#pragma unroll
        for (int d = TN; d < NDMA; d++) issue_dma(d, 1, dsrc[d]);
        if (m0_cur + BM <= M_store) {
            store_whole_tile_bf16<BM, BN, WAVES_M, WAVES_N>(acc, C, N, m0_cur, n0_cur, lds + P::STAGING_OFF);
            stores_behind = true;
        } else {                                          // the last rows of A are padding: C does not have them
            store_whole_tile_bf16<BM, BN, WAVES_M, WAVES_N, true>(acc, C, N, m0_cur, n0_cur, lds + P::STAGING_OFF,
                                                                  M_store - m0_cur);
            stores_behind = false;                        // masked stores: how many were issued is not known here
        }
#pragma unroll
        for (int j = 0; j < TM; j++)
#pragma unroll
            for (int i = 0; i < TN; i++) acc[j][i] = (f32x4){0.f, 0.f, 0.f, 0.f};
        // the first LAG folds of the next K block add s[TM-1] * (ring entries of this tile): make that 0 * 0
#pragma unroll
        for (int q = 0; q < PR; q++) pring[q] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < TM; j++) s[j] = 0.f;
        tile_origin(r + 1, m0_cur, n0_cur);
    }
    // prefetches past the last tile must land before the LDS is handed on
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (HALF_TAIL) {
        static_assert(BM == 256 && BN == 256 && WAVES_M == 2 && WAVES_N == 4, "half tiles of the 256 x 256 tile");
        const int grid = (int)gridDim.x, R = T % grid, R8 = (R + 7) / 8 * 8;
        const int b = (int)blockIdx.x;
        const int half = b < R ? 0 : (b >= R8 && b < R8 + R) ? 1 : -1;
        if (half < 0) return;                               // uniform over the workgroup
        int tm, tn;
        tile_of_block(T - R + (half ? b - R8 : b), T, tiles_m, tiles_n, group_m, true, tm, tn);
        const int m0 = (tm * BM < M - BM ? tm * BM : M - BM) + 128 * half, n0 = tn * BN;
        __syncthreads();                                    // every wave is done with its store staging region
        using H = TileGeom<128, 256, 2, 4, 3>;
        static_assert(H::LDS_BYTES <= P::LDS_BYTES, "the half tile's stages fit this kernel's LDS");
        f32x4 acc2[H::TM][H::TN];
        tile_mainloop<128, 256, 2, 4, 3>(A, B, SA, SB, M, M, N, m0, n0, 0, QK, lds, acc2);
        store_tile_bf16<128, 256, 2, 4>(acc2, C, M_store, N, m0, n0, lds);
    }
}

}  // namespace rf
