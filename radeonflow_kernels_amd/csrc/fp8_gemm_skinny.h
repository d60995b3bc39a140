// Skinny-K form of the block-scaled fp8 GEMM: K = 128 ... 512 (one to four scale blocks).
//
// With so little K the GEMM is a streaming store of C (6144 x 7168 x 256: 88 MB of bf16 against 3.4 MB of operands and
// 4.5 us of matrix work), and what decides its time is how early the first store leaves and whether stores keep
// leaving. The tiled kernels finish a whole 256 x 256 tile before its first store: a compute unit alternates between a
// K loop with nothing to store and a burst of 128 KB. Here the roles are turned round:
//   * a workgroup owns a strip of 256 columns and a range of rows of it. The strip's B operand (256 columns x K) is
//     loaded once, at the start, and then lives in REGISTERS as ready MFMA fragments (K/128 x 4 fragments per wave: 64
//     registers at K = 256);
//   * A is streamed through a ring of four LDS slots in items of 128 rows, three items ahead of the compute position
//     (an item's loads take about 2 us to come back on a busy chip, its compute a fraction of that);
//   * each wave walks the 16-row m-tiles of its 64 x 64 share of the item: 4 transpose reads per K block, K/128 x 4
//     MFMAs, the block-scale folds, bf16 conversion, staging through a private 2.25 KiB LDS region, two 1 KiB stores
//     (whole 128-byte lines). The first store leaves after 8 MFMAs, and stores are spread evenly over the item.
// With three or four K blocks an item is 64 rows (wave share 32 x 64, two m-tiles), so that four item slots and the
// strip's fragments (up to 128 registers) still fit; B then passes through the whole ring before the first item is
// loaded, and a wave works through an m-tile K block by K block (one A fragment and four partial tiles live at a time).
// Numerics are those of the tiled kernels: per K block the products are summed inside the MFMA from zero and folded
// with acc = fma(a_scale * b_scale, partial, acc), K blocks in order; one bf16 rounding.
//
// Requirements checked by the host: K = 128 * QK, M % 16 == 0, M >= 16, N % 64 == 0, a / b / c 16-byte aligned, grid =
// strips * per_strip. M_store <= M is the number of rows of C that exist (a caller whose M is not a multiple of 16 pads
// A and a_scale).
#pragma once
#include "fp8_gemm_kernels.h"

namespace rf {

template <int QK>
struct SkinnyGeom {
    static constexpr int BN = 256, NW = 8, TN = 4;                    // strip width, waves (2 x 4), n-tiles per wave
    static constexpr int IM = QK <= 2 ? 128 : 64, TM = IM / 32;       // rows per item; wave share IM/2 x 64 = TM m-tiles
    static constexpr int RING = 4;                                    // item slots: three items in flight beside the current one
    static constexpr int B_KB = BK * BN, A_KB = BK * IM;              // bytes of one K block of a strip / of an item
    static constexpr int B_BYTES = QK * B_KB, A_SLOT = QK * A_KB, S_SLOT = QK * IM * 4;
    // The strip's B operand passes through the slots behind the first item's once, on its way into registers: all of it
    // at once with 128-row items (two slots hold it), B_KPP K blocks at a time with 64-row items (three slots)
    static constexpr int OFF_B = IM == 128 ? 2 * A_SLOT : A_SLOT;
    static constexpr int B_KPP = (RING * A_SLOT - OFF_B) / B_KB < QK ? (RING * A_SLOT - OFF_B) / B_KB : QK;
    static constexpr int B_PHASES = (QK + B_KPP - 1) / B_KPP;
    static constexpr int OFF_S = RING * A_SLOT, OFF_SB = OFF_S + RING * S_SLOT, OFF_STAGE = OFF_SB + 256;
    static constexpr int STAGE_ROW = 64 * 2 + 16, STAGE_REGION = 16 * STAGE_ROW;     // one m-tile of a wave, rows padded
    static constexpr int LDS_BYTES = OFF_STAGE + NW * STAGE_REGION;
    static constexpr int CPR_A = IM / 16, RPI_A = 64 / CPR_A;         // 16-byte chunks per LDS row of A, rows per 1 KiB load
    static constexpr int INST_A = QK * IM / 64, INST_B = 32 / NW;     // 1 KiB load instructions per wave: an item, a K block of B
    static constexpr int NSA = QK * IM / 64;                          // a_scale loads per item (64 rows each), one per wave
    static constexpr int STORES = TM * 2;                             // store instructions per wave and unmasked item
    static_assert(QK >= 1 && QK <= 4, "one to four K blocks");
    static_assert(B_KPP >= 1, "at least one K block of B fits behind the first item");
    static_assert(NSA <= NW, "one scale load per wave at most");
    static_assert(LDS_BYTES <= 160 * 1024, "item ring + scales + store staging fit the CU's LDS");
    static_assert((RING - 1) * STORES + (RING - 2) * INST_A <= 63, "the largest wait count fits the instruction's field");
};

template <int QK>
__global__ __launch_bounds__(512) void gemm_fp8_blockscale_skinny(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, uint16_t *__restrict__ C, int M, int N, int per_strip, int M_store) {
    using G = SkinnyGeom<QK>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int L = lane & 15, g = lane >> 4, wm = wave & 1, wn = wave >> 1;
    const int QN = (N + 127) / 128;
    // this workgroup: strip blockIdx.x / per_strip, and of its rows (in units of 64) the share blockIdx.x % per_strip
    const int strip = (int)blockIdx.x / per_strip, part = (int)blockIdx.x - strip * per_strip;
    const int units = (M + 63) / 64;
    const int m_begin = 64 * (int)((long)part * units / per_strip);
    int m_end = 64 * (int)((long)(part + 1) * units / per_strip);
    if (m_end > M) m_end = M;
    if (m_begin >= m_end) return;
    const int n_items = (m_end - m_begin + G::IM - 1) / G::IM;
    const int row_lim = m_end < M_store ? m_end : M_store;             // rows of C this workgroup may write end here
    const int n0 = strip * G::BN;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(RF_LDS uint8_t *)lds;

    // LDS-DMA loads through inline asm (the kernel owns the vmcnt waits, see tile_mainloop): 64-bit scalar base +
    // per-lane 32-bit offset, M0 = LDS destination of the instruction (lane l lands at M0 + 16 l, or M0 + 4 l).
    auto dma16 = [&](uint32_t voff, const uint8_t *sbase, uint32_t dst) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane(dst)) : "memory");
    };
    auto dma4 = [&](uint32_t voff, const uint8_t *sbase, uint32_t dst) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1"
                     :: "v"(voff), "s"(sbase), "s"(__builtin_amdgcn_readfirstlane(dst)) : "memory");
    };
    // LDS rows are the operands' own rows (128 bytes of A, 256 of B per K row), their 16-byte chunks XOR-swizzled by
    // row on the source side so that the transpose reads are free of bank conflicts.
    auto issue_b = [&](int kb, int at) {                             // K block kb of the strip into staging position at
#pragma unroll
        for (int d = 0; d < G::INST_B; d++) {
            const int q = wave * G::INST_B + d;                      // K rows 4q .. 4q+3 of the block
            const int rl = lane >> 4, ch = lane & 15, kl = 4 * q + rl;
            int n = n0 + ((ch ^ swizzle_of_row<G::BN>(kl)) << 4);
            if (n + 16 > N) n = N - 16;                              // columns past N: any valid bytes will do
            dma16((uint32_t)rl * (uint32_t)N + (uint32_t)n, B + (size_t)(kb * BK + 4 * q) * N,
                  lds_base + G::OFF_B + at * G::B_KB + q * 1024);
        }
    };
    auto issue_b_scales = [&]() {
        if (wave == G::NW - 1) {                                     // b_scale slot 2 kb + blk <- block n0/128 + blk of K block kb
            const int kb = (lane >> 1) < QK ? (lane >> 1) : QK - 1;
            int nb = (n0 >> 7) + (lane & 1);
            if (nb > QN - 1) nb = QN - 1;
            dma4((uint32_t)(kb * QN + nb) * 4u, (const uint8_t *)SB, lds_base + G::OFF_SB);
        }
    };
    auto issue_a = [&](int item) {                                   // rows m_begin + IM item .. of A into slot item % RING
        const int slot = item & (G::RING - 1), m0 = m_begin + item * G::IM;
#pragma unroll
        for (int d = 0; d < G::INST_A; d++) {
            const int q = wave * G::INST_A + d;                      // K rows RPI_A q .. of the item
            const int rl = lane / G::CPR_A, ch = lane % G::CPR_A, kl = (G::RPI_A * q + rl) & 127;
            int m = m0 + ((ch ^ swizzle_of_row<G::IM>(kl)) << 4);
            if (m + 16 > M) m = M - 16;                              // rows past M: any valid bytes will do
            dma16((uint32_t)rl * (uint32_t)M + (uint32_t)m, A + (size_t)(G::RPI_A * q) * M,
                  lds_base + slot * G::A_SLOT + q * 1024);
        }
        if (wave < G::NSA) {
            // a_scale position (IM/2) h + TM l + j of a K block holds the scale of item row (IM/2) h + 16 j + l, so that
            // the TM scales a lane needs (row l of each of its wave's m-tiles) are contiguous
            constexpr int PER_KB = G::IM / 64;                       // loads per K block
            const int kb = wave / PER_KB, pos = (wave % PER_KB) * 64 + lane;
            const int h = pos / (G::IM / 2), r = pos % (G::IM / 2);
            int m = m0 + (G::IM / 2) * h + 16 * (r % G::TM) + r / G::TM;
            if (m > M - 1) m = M - 1;
            dma4((uint32_t)m * 4u, (const uint8_t *)(SA + (size_t)kb * M),
                 lds_base + G::OFF_S + slot * G::S_SLOT + (kb * G::IM + (wave % PER_KB) * 64) * 4);
        }
    };

    // per-lane LDS offsets of the transpose reads (see tile_mainloop): row 32 g + 8 t + L/2 of a K block, half L&1 of
    // the 16-byte chunk of the n-tile / m-tile
    const int krow = 32 * g + (L >> 1);
    const uint32_t boff = G::OFF_B + krow * G::BN + (((wn * G::TN) ^ swizzle_of_row<G::BN>(krow)) << 4) + 8 * (L & 1);
    const uint32_t aoff = krow * G::IM + (((wm * G::TM) ^ swizzle_of_row<G::IM>(krow)) << 4) + 8 * (L & 1);
    const uint32_t soff = G::OFF_S + (wm * (G::IM / 2) + L * G::TM) * 4;
    uint8_t *region = lds + G::OFF_STAGE + wave * G::STAGE_REGION;
    auto rd = [&](uint32_t off) { return __builtin_amdgcn_ds_read_tr8_b64_v2i32((RF_LDS i32x2 *)(lds + off)); };
    const bool active = n0 + 64 * wn < N;                            // a wave whose columns lie past N only loads

    // start: the first item and the strip's B operand; B goes from LDS into registers, where it stays
    issue_a(0);
    issue_b_scales();
    i32x8 bfrag[QK][G::TN];
    float sbv[QK];
#pragma unroll
    for (int ph = 0; ph < G::B_PHASES; ph++) {
#pragma unroll
        for (int kb = ph * G::B_KPP; kb < (ph + 1) * G::B_KPP && kb < QK; kb++) issue_b(kb, kb - ph * G::B_KPP);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
#pragma unroll
        for (int kb = ph * G::B_KPP; kb < (ph + 1) * G::B_KPP && kb < QK; kb++) {
#pragma unroll
            for (int i = 0; i < G::TN; i++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const i32x2 v = rd((kb - ph * G::B_KPP) * G::B_KB + (boff ^ (i << 4)) + q * 8 * G::BN);
                    bfrag[kb][i][2 * q] = v[0];
                    bfrag[kb][i][2 * q + 1] = v[1];
                }
            sbv[kb] = *(RF_LDS float *)(lds + G::OFF_SB + (kb * 2 + (wn >> 1)) * 4);
        }
        __syncthreads();                 // everyone holds these fragments: the staging space is free again
    }
    // Waiting for an item's loads. A wave's vector memory instructions complete in the order it issued them, loads and
    // stores alike, so "all but the newest n" have landed once at least n instructions were issued after them. `issued`
    // counts instructions this wave has issued for certain (the A loads; an item's stores only when none of them is
    // masked), mark1..mark3 are its values right after the loads of the next three items.
    int issued = 0, mark1 = 0, mark2 = 0, mark3 = 0;
#pragma unroll
    for (int i = 1; i < G::RING; i++) {
        if (i < n_items) {
            issue_a(i);
            issued += G::INST_A;
        }
        if (i == 1) mark1 = issued; else if (i == 2) mark2 = issued; else mark3 = issued;
    }
    // wait until at most `younger` (rounded down to a multiple of four) of this wave's instructions are outstanding
    auto wait_all_but = [&](int younger) {
        if (younger >= 32) asm volatile("s_waitcnt vmcnt(32)" ::: "memory");
        else if (younger >= 28) asm volatile("s_waitcnt vmcnt(28)" ::: "memory");
        else if (younger >= 24) asm volatile("s_waitcnt vmcnt(24)" ::: "memory");
        else if (younger >= 20) asm volatile("s_waitcnt vmcnt(20)" ::: "memory");
        else if (younger >= 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else if (younger >= 12) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
        else if (younger >= 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else if (younger >= 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    auto wait_for_next_item = [&]() { wait_all_but(issued - mark1); };

    // one item; full_c: no row of it is masked
    auto compute_item = [&](int t, auto full_c) {
        constexpr bool full = decltype(full_c)::value != 0;
        const int slot = t & (G::RING - 1), m0 = m_begin + t * G::IM;
        float sv[QK][G::TM];                                         // a_scale of row L of each m-tile, per K block
#pragma unroll
        for (int kb = 0; kb < QK; kb++) {
            if constexpr (G::TM == 4) {
                const f32x4 x = *(RF_LDS f32x4 *)(lds + slot * G::S_SLOT + soff + kb * G::IM * 4);
#pragma unroll
                for (int jj = 0; jj < 4; jj++) sv[kb][jj] = x[jj];
            } else {
                const f32x2 x = *(RF_LDS f32x2 *)(lds + slot * G::S_SLOT + soff + kb * G::IM * 4);
                sv[kb][0] = x[0];
                sv[kb][1] = x[1];
            }
        }
        uint16_t *out = C + (size_t)(m0 + wm * (G::IM / 2) + (lane >> 3)) * N + n0 + wn * 64 + (lane & 7) * 8;
        const int row = m0 + wm * (G::IM / 2) + (lane >> 3);
        staged_u32x4 v[2][2];
        auto store_rows = [&](int j) {                               // m-tile j's two store instructions (8 rows each)
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const staged_u32x4 x = v[j & 1][q];
                if (full || row + 16 * j + 8 * q < row_lim)
                    store_c16(out + (size_t)(16 * j + 8 * q) * N, make_uint4(x[0], x[1], x[2], x[3]));
            }
        };
        // lane holds C[16 j + L][16 i + 4 g .. + 3]: staged by row, read back 16 bytes per lane, 8 lanes per row
        auto stage_tile = [&](int j, const f32x4 (&acc)[G::TN]) {
#pragma unroll
            for (int i = 0; i < G::TN; i++) {
                const staged_u32x2 w = {pack_bf16x2(acc[i][0], acc[i][1]), pack_bf16x2(acc[i][2], acc[i][3])};
                *(staged_u32x2 *)(region + L * G::STAGE_ROW + (16 * i + 4 * g) * 2) = w;
            }
#pragma unroll
            for (int q = 0; q < 2; q++)
                v[j & 1][q] = *(const staged_u32x4 *)(region + (q * 8 + (lane >> 3)) * G::STAGE_ROW + (lane & 7) * 16);
        };
        if constexpr (QK <= 2) {
            // all K blocks of an m-tile at once: its fragments are fetched while the previous m-tile's MFMAs issue
            i32x8 afrag[2][QK];
            auto read_afrag = [&](int buf, int j) {
#pragma unroll
                for (int kb = 0; kb < QK; kb++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const i32x2 x = rd(slot * G::A_SLOT + kb * G::A_KB + (aoff ^ (j << 4)) + q * 8 * G::IM);
                        afrag[buf][kb][2 * q] = x[0];
                        afrag[buf][kb][2 * q + 1] = x[1];
                    }
            };
            read_afrag(0, 0);
#pragma unroll
            for (int j = 0; j < G::TM; j++) {
                if (j + 1 < G::TM) read_afrag((j + 1) & 1, j + 1);
                f32x4 p[QK][G::TN];
#pragma unroll
                for (int kb = 0; kb < QK; kb++)
#pragma unroll
                    for (int i = 0; i < G::TN; i++)
                        p[kb][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            bfrag[kb][i], afrag[j & 1][kb], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                f32x4 acc[G::TN];
#pragma unroll
                for (int i = 0; i < G::TN; i++) {
                    acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kb = 0; kb < QK; kb++) {
                        const float sc = sv[kb][j] * sbv[kb];
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[i][e] = __builtin_fmaf(sc, p[kb][i][e], acc[i][e]);
                    }
                }
                if (j > 0) store_rows(j - 1);
                stage_tile(j, acc);
            }
        } else {
            // K block by K block: step u = (m-tile u / QK, K block u % QK); the fragment of step u + 1 is fetched while
            // the MFMAs of step u issue, and the folds of step u follow the MFMAs of step u + 1
            i32x8 afrag[2];
            auto read_afrag = [&](int buf, int u) {
                const int j = u / QK, kb = u % QK;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const i32x2 x = rd(slot * G::A_SLOT + kb * G::A_KB + (aoff ^ (j << 4)) + q * 8 * G::IM);
                    afrag[buf][2 * q] = x[0];
                    afrag[buf][2 * q + 1] = x[1];
                }
            };
            f32x4 p[2][G::TN], acc[G::TN];
            auto fold = [&](int u) {
                const int j = u / QK, kb = u % QK;
                const float sc = sv[kb][j] * sbv[kb];
#pragma unroll
                for (int i = 0; i < G::TN; i++) {
                    if (kb == 0) acc[i] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[i][e] = __builtin_fmaf(sc, p[u & 1][i][e], acc[i][e]);
                }
                if (kb == QK - 1) {
                    if (j > 0) store_rows(j - 1);
                    stage_tile(j, acc);
                }
            };
            read_afrag(0, 0);
#pragma unroll
            for (int u = 0; u < G::TM * QK; u++) {
                if (u + 1 < G::TM * QK) read_afrag((u + 1) & 1, u + 1);
#pragma unroll
                for (int i = 0; i < G::TN; i++)
                    p[u & 1][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                        bfrag[u % QK][i], afrag[u & 1], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                if (u > 0) fold(u - 1);
            }
            fold(G::TM * QK - 1);
        }
        store_rows(G::TM - 1);
    };

    for (int t = 0; t < n_items; t++) {
        if (t > 0) {
            wait_for_next_item();
            __syncthreads();             // everyone's loads of item t have landed, and everyone has left item t - 1
            if (t + G::RING - 1 < n_items) {                          // into the slot of item t - 1
                issue_a(t + G::RING - 1);
                issued += G::INST_A;
            }
            mark1 = mark2;
            mark2 = mark3;
            mark3 = issued;
        }
        if (active) {
            if (m_begin + (t + 1) * G::IM <= row_lim) {
                compute_item(t, IntTag<1>{});
                issued += G::STORES;
            } else {
                compute_item(t, IntTag<0>{});
            }
        }
    }
}

}  // namespace rf
