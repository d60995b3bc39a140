// Second tile family of the FP8 blockwise-scaled GEMM for gfx950: tiles whose sides are not powers of two.
//
// Why it exists: with 256 compute units, a shape is fastest when its tile count is a multiple of 256. The headline
// shape M=6144 N=4608 has 432 tiles of 256x256 (two rounds, the second one 69 % full) but exactly 512 tiles of
// 192x288. Such tiles need a different inner loop from fp8_gemm_kernels.h:
//   * 8 waves as 4 (m) x 2 (n); a wave owns WM = BM/4 rows (TM = 3 or 4 m-tiles of 16) and WN = BN/2 columns
//     (TN up to 9 n-tiles). The A-matrix fragments of all TM m-tiles stay in registers for the whole K block and
//     the B-matrix fragments stream through a small ring, one n-tile per TM MFMAs (the other family holds B and
//     streams A);
//   * WN may exceed 128 and need not divide it, so a wave's columns straddle two b_scale blocks: both products
//     sa*sb0 and sa*sb1 are kept and each fold picks one by the (wave-uniform) position of its n-tile;
//   * LDS rows are BM / BN bytes with BM/16, BN/16 not powers of two: the chunk swizzle only touches the low
//     1-2 bits of the chunk index (see swizzle_of_row), and per-lane base registers replace the XOR addressing.
// Everything else (LDS-DMA loads issued by hand, transpose reads, lagged scale folds, barrier placement,
// numerics) follows the same scheme as tile_mainloop.
#pragma once
#include "fp8_gemm_kernels.h"

namespace rf {

template <int BM_, int BN_, int WAVES_M_, int WAVES_N_>
struct HoldAGeom {
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
    static constexpr int NW = WAVES_M * WAVES_N, NT = NW * 64;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 16, TN = WN / 16;
    static constexpr int STAGE_A = BK * BM, STAGE_B = BK * BN;
    static constexpr int STAGE_S = WAVES_M * 256;                 // per wave row: 16 lanes x 4 a_scale floats
    static constexpr int STAGE = STAGE_A + STAGE_B + STAGE_S;
    static constexpr int LDS_BYTES = 2 * STAGE;
    static constexpr int OUT_ROW = WN * 2 + 16;                   // staged bf16 row of a wave, padded
    static_assert(BM % (16 * WAVES_M) == 0 && BN % (16 * WAVES_N) == 0, "whole 16x16 tiles per wave");
    static_assert(TM <= 4, "a lane's a_scale values are one 16-byte LDS read");
    static_assert(WN <= 144, "a wave's columns touch at most two b_scale blocks");
    static_assert(STAGE_A % 1024 == 0 && STAGE_B % 1024 == 0, "whole 1 KiB load instructions");
    static_assert(NW * WM * OUT_ROW <= LDS_BYTES, "the output staging fits in the stage buffers");
};

template <int BM, int BN, int WAVES_M, int WAVES_N>
__device__ __forceinline__ void tile_mainloop_hold_a(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, int M, int N, int m0, int n0, int kb_begin, int kb_end, uint8_t *lds,
    f32x4 (&acc)[BM / WAVES_M / 16][BN / WAVES_N / 16]) {
    using G = HoldAGeom<BM, BN, WAVES_M, WAVES_N>;
    constexpr int NW = G::NW, WM = G::WM, WN = G::WN, TM = G::TM, TN = G::TN;
    constexpr int STAGE_A = G::STAGE_A, STAGE_B = G::STAGE_B, STAGE = G::STAGE;
    constexpr int CPR_A = BM / 16, CPR_B = BN / 16;              // 16-byte chunks per LDS row
    // 1 KiB load instructions of a stage: NA for A, NB for B, dealt to the waves in contiguous runs of IA / IB; the
    // remainders RA / RB go one each to the first waves.
    constexpr int NA = STAGE_A / 1024, NB = STAGE_B / 1024;
    constexpr int IA = NA / NW, RA = NA % NW, IB = NB / NW, RB = NB % NW;
    constexpr int D_RA = IA + IB, D_RB = D_RA + (RA ? 1 : 0), D_S = D_RB + (RB ? 1 : 0), NDMA = D_S + 1;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int L = lane & 15, g = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    const int QN = (N + 127) / 128;

    // ---- global -> LDS ----
    // DMA instruction d of this wave: d < IA -> A instruction wave*IA + d; d < IA+IB -> B instruction wave*IB + ..;
    // D_RA / D_RB -> the remainder instructions (first RA / RB waves only); D_S -> a_scale (first WAVES_M waves).
    // LDS chunk q = 64*instruction + lane of the A (B) region is row q / CPR, position q % CPR; it holds the source
    // chunk (position ^ swizzle_of_row(row)). The per-lane source offset inside a K block is row*ld + column.
    uint32_t goff[NDMA];
    uint32_t ldst[NDMA];                                          // LDS destination inside a stage (scalar)
    const uint32_t lds_base = (uint32_t)(uintptr_t)(RF_LDS uint8_t *)lds;
#pragma unroll
    for (int d = 0; d < D_S; d++) {
        const bool is_a = d < IA || (RA && d == D_RA);
        const int inst = d < IA ? wave * IA + d : d < IA + IB ? wave * IB + (d - IA)
                       : is_a ? NW * IA + (wave < RA ? wave : 0) : NW * IB + (wave < RB ? wave : 0);
        const int q = inst * 64 + lane;
        if (is_a) {
            const int kl = q / CPR_A, c = (q % CPR_A) ^ swizzle_of_row<BM>(kl);
            int m = m0 + c * 16;
            if (m + 16 > M) m = M - 16;                           // columns past M: any valid bytes will do
            goff[d] = (uint32_t)kl * (uint32_t)M + (uint32_t)m;
            ldst[d] = lds_base + inst * 1024;
        } else {
            const int kl = q / CPR_B, c = (q % CPR_B) ^ swizzle_of_row<BN>(kl);
            int n = n0 + c * 16;
            if (n + 16 > N) n = N - 16;
            goff[d] = (uint32_t)kl * (uint32_t)N + (uint32_t)n;
            ldst[d] = lds_base + STAGE_A + inst * 1024;
        }
    }
    {
        // a_scale slot 4*L + j of wave row w holds the scale of tile row w*WM + 16*j + L: the TM scales a lane needs
        // (its column L of every m-tile of its wave) are one 16-byte read
        const int w = wave < WAVES_M ? wave : 0, j = (lane & 3) < TM ? (lane & 3) : TM - 1;
        int m = m0 + w * WM + 16 * j + (lane >> 2);
        if (m > M - 1) m = M - 1;
        goff[D_S] = (uint32_t)m * 4u;
        ldst[D_S] = lds_base + STAGE_A + STAGE_B + w * 256;
    }
    // issued through inline asm so that the kernel, not the compiler, owns the wait for these loads
    auto issue_dma = [&](int d, uint32_t stage_off, const uint8_t *src_a, const uint8_t *src_b, const uint8_t *src_s) {
        const bool is_a = d < IA || (RA && d == D_RA);
        if (d == D_S) {
            if (wave < WAVES_M)
                asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                             :: "v"(goff[D_S]), "s"(src_s), "s"(stage_off + ldst[D_S]) : "memory");
        } else if (d < D_RA || (is_a ? wave < RA : wave < RB)) {
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :: "v"(goff[d]), "s"(is_a ? src_a : src_b), "s"(stage_off + ldst[d]) : "memory");
        }
    };

    // ---- LDS -> MFMA operands ----
    // lane (L,g) of transpose read t points at row k = 32g + 8t + L/2, half (L&1) of a 16-byte chunk. The swizzle
    // of that row does not depend on t. A side: one offset register per m-tile. B side: the swizzle flips only the
    // low SWB bits of the chunk index, so n-tile i is at base[i % 2^SWB] + 16*i.
    const int krow = 32 * g + (L >> 1);
    constexpr int SWB = swizzle_bits<BN>();
    static_assert(SWB <= 2, "B rows with a wide swizzle need the XOR addressing of the other tile family");
    constexpr int NRES = (1 << SWB) < TN ? (1 << SWB) : TN;
    uint32_t aoff[TM], boff[NRES];
#pragma unroll
    for (int j = 0; j < TM; j++)
        aoff[j] = krow * BM + 8 * (L & 1) + (((wm * TM + j) ^ swizzle_of_row<BM>(krow)) << 4);
#pragma unroll
    for (int r = 0; r < NRES; r++)
        boff[r] = STAGE_A + krow * BN + 8 * (L & 1) + 16 * ((((wn * TN + r) ^ swizzle_of_row<BN>(krow))) - r);
    const uint32_t soff = STAGE_A + STAGE_B + wm * 256 + L * 16;

    // b_scale blocks of this wave's columns: n-tiles i < ib use block nb0, the others nb1
    const int ncol0 = n0 + wn * WN;
    int nb0 = ncol0 >> 7, nb1 = nb0 + 1;
    int ib = ((nb0 + 1) * 128 - ncol0) >> 4;
    if (ib > TN) ib = TN;
    if (nb0 > QN - 1) nb0 = QN - 1;
    if (nb1 > QN - 1) nb1 = QN - 1;

#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
        for (int i = 0; i < TN; i++) acc[j][i] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // b_scale is wave-uniform but fetched with vector loads: see tile_mainloop
    int vzero;
    asm volatile("v_mov_b32 %0, 0" : "=v"(vzero));

    // ---- main loop ----
    // MFMA slot t = (n-tile i, m-tile j), n-tile-major. The B fragment of n-tile i+AHEAD is fetched while n-tile i
    // computes (ring of NBUF = AHEAD+1 fragments; TN is a multiple of NBUF, so ring positions repeat per K block).
    // The barrier that publishes the next stage sits at BAR_SLOT, the first slot whose fetch belongs to the next K
    // block. In the last n-tile row each A fragment is dead once its MFMA has issued and is refilled from the
    // next stage. After the barrier the stage just consumed is free: the LDS-DMA loads of K block kb+2 start
    // there, one per slot, and run on into the first slots of the next iteration.
    constexpr int NBUF = (TN % 3 == 0) ? 3 : 2, AHEAD = NBUF - 1;
    static_assert(TN % NBUF == 0, "ring positions must repeat per K block");
    // The partial sum of slot t goes to ring entry t % PR and is folded LAG slots later, also across the K block
    // boundary: the ring position only carries over if the slot count is a multiple of PR.
    constexpr int NMFMA = TM * TN, PR = (NMFMA % 4 == 0) ? 4 : 3, LAG = PR - 1;
    constexpr int BAR_SLOT = (TN - AHEAD) * TM, NPOST = NMFMA - BAR_SLOT;
    static_assert(NMFMA % PR == 0, "ring positions must repeat per K block");
    static_assert(LAG <= TM && LAG < PR, "lagged folds of a K block stay inside its last n-tile row");
    static_assert(NDMA - NPOST <= BAR_SLOT, "the DMA batch finishes well before the barrier that needs it");
    const int kb_last = kb_end - 1;
    auto clamp_kb = [&](int kb) { return kb < kb_last ? kb : kb_last; };   // past the end: re-fetch the last block
    auto src_a_of = [&](int kb) { return A + (size_t)kb * BK * M; };
    auto src_b_of = [&](int kb) { return B + (size_t)kb * BK * N; };
    auto src_s_of = [&](int kb) { return (const uint8_t *)(SA + (size_t)kb * M); };

    i32x8 afrag[TM], bfrag[NBUF];
    f32x4 pring[PR];
    // sc: the scales the folds use right now (sa*sb of the b_scale block the current n-tile row lies in); s1: the
    // scales of the wave's second b_scale block, swapped in when the folds reach n-tile ib
    float sc[TM], s1[TM], sraw[4], sb0_cur = 0.f, sb1_cur = 0.f, sb0_next = 0.f, sb1_next = 0.f;
#pragma unroll
    for (int r = 0; r < PR; r++) pring[r] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < TM; j++) sc[j] = s1[j] = 0.f;

    auto rd = [&](uint32_t off) { return __builtin_amdgcn_ds_read_tr8_b64_v2i32((RF_LDS i32x2 *)(lds + off)); };
    auto read_b_part = [&](int buf, int i, uint32_t stage_base, int t) {
        i32x2 v = rd(stage_base + boff[i % NRES] + 16 * i + t * 8 * BN);
        bfrag[buf][2 * t] = v[0];
        bfrag[buf][2 * t + 1] = v[1];
    };
    auto read_a = [&](int j, uint32_t stage_base) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            i32x2 v = rd(stage_base + aoff[j] + t * 8 * BM);
            afrag[j][2 * t] = v[0];
            afrag[j][2 * t + 1] = v[1];
        }
    };
    auto read_scales = [&](uint32_t stage_base) {
        f32x4 v = *(RF_LDS f32x4 *)(lds + stage_base + soff);
#pragma unroll
        for (int e = 0; e < 4; e++) sraw[e] = v[e];
    };

    if (kb_begin < kb_end) {
        // prologue: stage 0 <- first K block, then its first operands; stage 1 <- start of the second K block
#pragma unroll
        for (int d = 0; d < NDMA; d++) issue_dma(d, 0, src_a_of(kb_begin), src_b_of(kb_begin), src_s_of(kb_begin));
        sb0_cur = SB[(size_t)kb_begin * QN + nb0 + vzero];
        sb1_cur = SB[(size_t)kb_begin * QN + nb1 + vzero];
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        asm volatile("" : "+v"(sb0_cur), "+v"(sb1_cur));
        __syncthreads();
#pragma unroll
        for (int j = 0; j < TM; j++) read_a(j, 0);
        read_scales(0);
#pragma unroll
        for (int i = 0; i < AHEAD; i++)
#pragma unroll
            for (int t = 0; t < 4; t++) read_b_part(i, i, 0, t);
        const int k1 = clamp_kb(kb_begin + 1);
#pragma unroll
        for (int d = 0; d < NPOST && d < NDMA; d++) issue_dma(d, STAGE, src_a_of(k1), src_b_of(k1), src_s_of(k1));
    }
    for (int kb = kb_begin, it = 0; kb < kb_end; ++kb, ++it) {
        const uint32_t cur = (it & 1) * STAGE, nxt = ((it + 1) & 1) * STAGE;
        const int kn1 = clamp_kb(kb + 1), kn2 = clamp_kb(kb + 2);
        const uint8_t *a1 = src_a_of(kn1), *b1 = src_b_of(kn1), *q1 = src_s_of(kn1);
        const uint8_t *a2 = src_a_of(kn2), *b2 = src_b_of(kn2), *q2 = src_s_of(kn2);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NMFMA; t++) {
            const int i = t / TM, j = t % TM;
            if (t == BAR_SLOT) {
                // my DMA loads of the next stage have landed; after the barrier everyone's have, and everyone has
                // finished reading the current stage
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                asm volatile("" : "+v"(sb0_next), "+v"(sb1_next));   // covered by the wait above
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            if (t == 0) {
                sb0_next = SB[(size_t)kn1 * QN + nb0 + vzero];
                sb1_next = SB[(size_t)kn1 * QN + nb1 + vzero];
            }
            pring[t % PR] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                bfrag[i % NBUF], afrag[j], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            asm volatile("" : "+v"(pring[t % PR]));          // anchor: the MFMA is issued here, not later
            __builtin_amdgcn_sched_barrier(0);
            // LDS-DMA: the batch for block kb+1 (started in the previous iteration) continues in the first slots;
            // the batch for block kb+2 starts right after the barrier
            if (t + NPOST < NDMA) issue_dma(t + NPOST, nxt, a1, b1, q1);
            if (t >= BAR_SLOT && t - BAR_SLOT < NDMA) issue_dma(t - BAR_SLOT, cur, a2, b2, q2);
            // LDS -> registers: the four reads of n-tile i+AHEAD are spread over the TM slots of n-tile i
            {
                const int ii = i + AHEAD;
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (r * TM / 4 == j) read_b_part(ii % NBUF, ii < TN ? ii : ii - TN, ii < TN ? cur : nxt, r);
            }
            if (i == TN - 1) {
                read_a(j, nxt);                                    // afrag[j] is dead: refill for block kb+1
                if (j == 0) read_scales(nxt);
            }
            // lagged fold. The first LAG slots fold the tail of the previous K block with the scales it left in
            // sc; when the folds reach n-tile 0 of this block sc is recomputed, when they reach n-tile ib (if the
            // wave has a second b_scale block) s1 is swapped in: a wave-uniform branch around TM moves.
            {
                const bool tail = t < LAG;
                const int u = tail ? NMFMA + t - LAG : t - LAG, iu = u / TM, ju = u % TM;
                if (!tail && ju == 0) {
                    if (iu == 0) {
#pragma unroll
                        for (int j2 = 0; j2 < TM; j2++) {
                            sc[j2] = sraw[j2] * sb0_cur;
                            s1[j2] = sraw[j2] * sb1_cur;
                        }
                    } else if (iu == ib) {
                        // moves written as asm so that they stay behind a scalar branch (taken once per K block)
                        // instead of becoming TM selects in every n-tile row
#pragma unroll
                        for (int j2 = 0; j2 < TM; j2++) asm volatile("v_mov_b32 %0, %1" : "+v"(sc[j2]) : "v"(s1[j2]));
                    }
                }
#pragma unroll
                for (int e = 0; e < 4; e++) acc[ju][iu][e] = __builtin_fmaf(sc[ju], pring[u % PR][e], acc[ju][iu][e]);
                asm volatile("" : "+v"(acc[ju][iu]));        // anchor: the fold happens in this slot
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        sb0_cur = sb0_next;
        sb1_cur = sb1_next;
    }
    // folds still owed by the last K block
#pragma unroll
    for (int t = 0; t < LAG; t++) {
        const int u = NMFMA + t - LAG, iu = u / TM, ju = u % TM;
#pragma unroll
        for (int e = 0; e < 4; e++) acc[ju][iu][e] = __builtin_fmaf(sc[ju], pring[u % PR][e], acc[ju][iu][e]);
    }
    // LDS-DMA writes of the last (redundant) prefetches must land before this workgroup's LDS can be handed on
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Stores a wave's accumulators as bf16 into C, masked at the M and N edges: each wave stages its whole WM x WN tile
// in its own LDS region (rows padded by 16 bytes) and writes it out 16 bytes per lane, consecutive lanes along a row.
// All waves must call it together: it starts with a barrier, because LDS-DMA loads of other waves may still be
// landing in the stage buffers that are reused here.
template <int BM, int BN, int WAVES_M, int WAVES_N>
__device__ __forceinline__ void store_tile_bf16_hold_a(const f32x4 (&acc)[BM / WAVES_M / 16][BN / WAVES_N / 16],
                                                       uint16_t *__restrict__ C, int M, int N, int m0, int n0,
                                                       uint8_t *lds) {
    using G = HoldAGeom<BM, BN, WAVES_M, WAVES_N>;
    constexpr int ROW = G::OUT_ROW, CPR = G::WN / 8, TOTAL = G::WM * CPR;   // 16-byte chunks per row / per wave tile
    int vz;                                  // keeps this address arithmetic below the main loop (see store_tile_bf16)
    asm volatile("v_mov_b32 %0, 0" : "=v"(vz));
    const int lane = (threadIdx.x & 63) + vz, wave = threadIdx.x >> 6, L = lane & 15, g = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    uint8_t *region = lds + wave * (G::WM * ROW);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < G::TM; j++)
#pragma unroll
        for (int i = 0; i < G::TN; i++) {                // lane holds C[16j + L][16i + 4g .. +3]
            uint2 v;
            v.x = pack_bf16x2(acc[j][i][0], acc[j][i][1]);
            v.y = pack_bf16x2(acc[j][i][2], acc[j][i][3]);
            *(uint2 *)(region + (16 * j + L) * ROW + (16 * i + 4 * g) * 2) = v;
        }
    // same wave writes and reads its region: program order is enough, the compiler inserts the LDS wait
#pragma unroll
    for (int q0 = 0; q0 < TOTAL; q0 += 64) {
        const int q = q0 + lane;
        if (q < TOTAL) {
            const int r = q / CPR, cb = (q % CPR) * 16;                 // row of the wave tile, byte column
            const uint4 v = *(const uint4 *)(region + r * ROW + cb);
            const int m = m0 + wm * G::WM + r;
            const int n = n0 + wn * G::WN + cb / 2;
            if (m < M && n < N) *(uint4 *)(C + (size_t)m * N + n) = v;
        }
    }
}

// One workgroup per (tile, K split); same contract as gemm_fp8_blockscale_tile.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool PARTIAL>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_fp8_blockscale_tile_hold_a(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, void *__restrict__ Cout, int M, int N, int K, int kb_per_split,
    int tiles_m, int tiles_n, int group_m) {
    using G = HoldAGeom<BM, BN, WAVES_M, WAVES_N>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, tiles_m * tiles_n, tiles_m, tiles_n, group_m, true, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int QK = K / BK;
    const int kb_begin = blockIdx.y * kb_per_split;
    const int kb_end = kb_begin + kb_per_split < QK ? kb_begin + kb_per_split : QK;
    f32x4 acc[G::TM][G::TN];
    tile_mainloop_hold_a<BM, BN, WAVES_M, WAVES_N>(A, B, SA, SB, M, N, m0, n0, kb_begin, kb_end, lds, acc);
    if constexpr (PARTIAL)
        store_tile_f32<BM, BN, WAVES_M, WAVES_N>(acc, (float *)Cout + ((size_t)blockIdx.y * M + m0) * N + n0, N, M - m0,
                                                 N - n0);
    else
        store_tile_bf16_hold_a<BM, BN, WAVES_M, WAVES_N>(acc, (uint16_t *)Cout, M, N, m0, n0, lds);
}

}  // namespace rf
