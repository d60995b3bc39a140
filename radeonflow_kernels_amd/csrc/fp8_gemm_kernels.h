// Device kernels of the FP8 (OCP e4m3fn) blockwise-scaled GEMM for gfx950 (MI355X).
//
// Replaces the reference's transpose + rocWMMA pipeline (src/gemm/transpose_kernel.cpp:17-63,
// src/gemm/gemm_kernel.cpp:306-562, src/gemm/gemm_kernel.cpp:288-303) with a design built on
// three gfx950 features:
//   * global_load_lds_dwordx4  - 16 B per lane straight from HBM/L2 into LDS, no VGPR staging;
//   * ds_read_b64_tr_b8        - LDS transpose read: a 16-lane group that points at 8 k-rows x 16
//                                bytes gets back, per lane, 8 consecutive k for one m (or n). The
//                                operands arrive M-/N-contiguous ([K][M], [K][N]) and MFMA wants
//                                K-contiguous bytes per lane, so this removes the reference's two
//                                transpose pre-passes entirely;
//   * v_mfma_f32_16x16x128_f8f6f4 - one MFMA consumes exactly one 128-wide scale block.
//
// Data flow per workgroup: a BM x BN output tile, K walked in blocks of 128. Each K block is one
// LDS stage holding A[k0:k0+128][m0:m0+BM] and B[k0:k0+128][n0:n0+BN] exactly as they lie in
// memory (rows of BM / BN bytes), with the 16-byte chunks of every row XOR-swizzled so that the
// transpose reads are bank-conflict free. Two stages are double-buffered.
//
// MFMA orientation: the B-matrix fragment is the MFMA "A" operand (rows = n) and the A-matrix
// fragment is the MFMA "B" operand (columns = m). A lane (L = lane%16, g = lane/16) then holds
// D[n = 4g..4g+3][m = L]: four consecutive n of one row m, i.e. 8 contiguous bytes of bf16 C, and
// needs a single scale a_scale[m,kb]*b_scale[nb,kb] per 16x16 tile.
//
// Numerics (what the reference's kernel does, src/gemm/gemm_kernel.cpp:138-208): the products of a
// 128-K block are summed inside the MFMA in fp32 starting from zero, then acc = fma(sa*sb, partial, acc).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rf {

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int BK = 128;        // K per stage == the quantisation block
template <int V> struct IntTag { static constexpr int value = V; };
constexpr int NUM_XCD = 8;

#define RF_LDS __attribute__((address_space(3)))
#define RF_GLOBAL __attribute__((address_space(1)))

// XOR applied to the 16-byte-chunk index of LDS row k (row width W bytes). Chosen so that the 32
// lanes the LDS serves together in a transpose read (two 16-lane groups: 8 k-rows x 2 half-chunks
// each, the groups 32 rows apart) touch all 64 banks exactly once. Row k starts W/16 * k chunks into
// the 16-chunk bank period; with W/16 = 2^e * odd, rows 2^(4-e) apart (and rows 32 apart) start on
// the same chunk, and the XOR spreads exactly those over the low e bits of the chunk index. It never
// leaves an aligned group of 2^e chunks, so it also works for rows of 12, 14 or 18 chunks.
template <int W>
constexpr int swizzle_bits() {
    static_assert(W % 32 == 0, "tile row width");
    constexpr int q = W / 16;
    return (q % 16 == 0) ? 4 : (q % 8 == 0) ? 3 : (q % 4 == 0) ? 2 : 1;
}
template <int W>
__device__ __forceinline__ int swizzle_of_row(int k) {
    constexpr int r = 4 - swizzle_bits<W>();                 // log2(rows per bank period)
    return ((k & 7) >> r) | (((k >> 5) & 1) << (3 - r));
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    f32x2 v = {lo, hi};
    bf16x2 h = __builtin_convertvector(v, bf16x2);           // v_cvt_pk_bf16_f32: RNE, NaN-safe
    return __builtin_bit_cast(uint32_t, h);
}

// Workgroup id -> (tile_m, tile_n). Workgroups are dealt round-robin to the 8 XCDs (each with its own L2), so
// id%8 is the XCD. Whatever an XCD's workgroups read, its L2 has to fetch once: a band of full tile rows makes
// every XCD read all of B. So, when the tile grid divides, the XCDs are laid out as a 4x2 (or 2x4, 8x1, 1x8) grid
// of rectangular regions, as square as possible, and the workgroups of an XCD walk their region down the rows
// first, so that the ~32 tiles in flight on the XCD form a compact patch sharing A rows and B columns. Otherwise
// each XCD gets a contiguous range of tile ids, ordered in groups of `group_m` tile rows.
__device__ __forceinline__ void tile_of_block(int bid, int nblocks, int tiles_m, int tiles_n, int group_m,
                                              bool xcd_remap, int &tile_m, int &tile_n) {
    int id = bid;
    if (xcd_remap) {
        const int xcd = bid % NUM_XCD, idx = bid / NUM_XCD;
        int xm = 0, xn = 0;                                   // XCD grid
        if (tiles_m % 4 == 0 && tiles_n % 2 == 0 && tiles_m >= 2 * tiles_n / 2) { xm = 4; xn = 2; }
        else if (tiles_m % 2 == 0 && tiles_n % 4 == 0) { xm = 2; xn = 4; }
        else if (tiles_m % 4 == 0 && tiles_n % 2 == 0) { xm = 4; xn = 2; }
        else if (tiles_m % 8 == 0) { xm = 8; xn = 1; }
        else if (tiles_n % 8 == 0) { xm = 1; xn = 8; }
        if (xm) {
            const int rm = tiles_m / xm, rn = tiles_n / xn;   // region size in tiles; rm*rn workgroups per XCD
            tile_m = (xcd % xm) * rm + idx % rm;
            tile_n = (xcd / xm) * rn + idx / rm;
            return;
        }
        const int per = nblocks / NUM_XCD, rem = nblocks % NUM_XCD;
        id = xcd * per + (xcd < rem ? xcd : rem) + idx;
    }
    int group_sz = group_m * tiles_n;
    int grp = id / group_sz;
    int first_m = grp * group_m;
    int rows = tiles_m - first_m < group_m ? tiles_m - first_m : group_m;
    int in_grp = id - grp * group_sz;
    tile_m = first_m + in_grp % rows;
    tile_n = in_grp / rows;
}

// Geometry of one kernel variant. NS = number of LDS stages (K blocks resident or in flight).
template <int BM_, int BN_, int WAVES_M_, int WAVES_N_, int NS_ = 2>
struct TileGeom {
    static constexpr int BM = BM_, BN = BN_, WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, NS = NS_;
    static constexpr int NW = WAVES_M * WAVES_N, NT = NW * 64;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 16, TN = WN / 16;
    static constexpr int STAGE_A = BK * BM, STAGE_B = BK * BN;
    static constexpr int STAGE_S = BM * 4 + 256;                  // a_scale of the tile rows + 64 b_scale slots
    static constexpr int STAGE = STAGE_A + STAGE_B + STAGE_S;
    static constexpr int LDS_BYTES = NS * STAGE + 16;             // the stages + a 16-byte mailbox
    static_assert(LDS_BYTES <= 160 * 1024, "stages fit the CU's LDS");
};

// Accumulates into acc the contribution of K blocks [kb_begin, kb_end) to the BM x BN tile at (m0, n0).
// M is the number of rows of A (and of a_scale) that may be touched, ldm the distance in elements between two
// K rows of A and of a_scale (ldm == M for a plain GEMM, ldm > M when A is a row range of a larger matrix).
// All waves of the workgroup call it together. On return every LDS-DMA load has landed, but other waves may still
// be reading LDS: a barrier is needed before LDS is written again.
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS = 2>
__device__ __forceinline__ void tile_mainloop(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, int M, int ldm, int N, int m0, int n0, int kb_begin, int kb_end, uint8_t *lds,
    f32x4 (&acc)[BM / WAVES_M / 16][BN / WAVES_N / 16], int opaque_zero = 0) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N, NS>;
    constexpr int NW = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 16, TN = WN / 16;
    // one LDS stage: A[128][BM] bytes, B[128][BN] bytes, BM fp32 a_scale values and the b_scale values of the
    // tile's columns. The stages are interleaved by operand (A0 A1 .. B0 B1 .. S0 S1 ..), so that a transpose read
    // of any stage is "per-lane base register + immediate": no address arithmetic in the loop.
    constexpr int STAGE_A = G::STAGE_A, STAGE_B = G::STAGE_B, STAGE_S = G::STAGE_S;
    constexpr int OFF_B = NS * STAGE_A, OFF_S = NS * (STAGE_A + STAGE_B), OFF_SB = BM * 4;   // OFF_SB inside an S region
    static_assert(NS == 2 || NS == 3, "two stages (one K block in flight) or three (two in flight)");
    constexpr int INST_A = STAGE_A / 1024 / NW, INST_B = STAGE_B / 1024 / NW;   // 1 KiB per wave instruction
    constexpr int NSC = BM / 64;                                                // scale loads: 64 floats each
    static_assert(STAGE_A % (1024 * NW) == 0 && STAGE_B % (1024 * NW) == 0, "loads must divide evenly over waves");
    static_assert(NSC <= NW, "one scale load per wave at most");
    // ONE_SB: the wave's columns lie inside one 128-column b_scale block. Otherwise (tile sides that are not powers
    // of two) they may straddle two: n-tiles below a wave-uniform split use the first block's scale, the others the
    // second's, and the K loop is instantiated once per possible split.
    constexpr bool ONE_SB = WN <= 128 && 128 % WN == 0;
    static_assert(ONE_SB || (TN == 3 && WN < 128), "straddling waves: three n-tiles, split before n-tile 1 or 2");
    static_assert(TM % 2 == 0, "scales are read back two or four at a time");
    constexpr int CPR_A = BM / 16, CPR_B = BN / 16;          // 16-byte chunks per LDS row
    // EVEN: a 1 KiB load instruction covers whole rows (RPI of them). Otherwise instruction q covers the 64 chunks
    // from linear chunk 64q of the stage, a wave's instructions together cover whole rows (ROWS_W of them).
    constexpr bool EVEN_A = 1024 % BM == 0, EVEN_B = 1024 % BN == 0;
    constexpr int RPI_A = EVEN_A ? 1024 / BM : 0, RPI_B = EVEN_B ? 1024 / BN : 0;      // rows per load instruction
    constexpr int ROWS_W_A = INST_A * 64 / CPR_A, ROWS_W_B = INST_B * 64 / CPR_B;      // rows per wave
    static_assert((INST_A * 64) % CPR_A == 0 && (INST_B * 64) % CPR_B == 0, "a wave's loads cover whole rows");

    // (opaque_zero: a caller that runs several instantiations of this loop inside a loop of its own passes a zero the
    // compiler cannot see through, made inside its loop; otherwise every instantiation's per-lane offsets are computed
    // once before the caller's loop and stay in registers through all of it)
    const int tid = threadIdx.x + opaque_zero;
    const int lane = tid & 63;
    // (a workgroup may hold several wave groups of NW waves, each running this loop on its own tile of LDS: the wave's
    // index inside its group)
    const int wave = __builtin_amdgcn_readfirstlane((tid >> 6) % NW);
    const int L = lane & 15, g = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;

    const int QN = (N + 127) / 128;

    // ---- global -> LDS: per-lane source offsets inside one K block (rows k_local, swizzled chunk) ----
    // Load instruction i of this wave covers rows (wave*INST + i)*RPI .. +RPI-1. Its per-lane offset differs from
    // that of another instruction only by a wave-uniform amount when both see the same row swizzle, i.e. the same
    // (k & 7) and (k >> 5) & 1 for every lane. So only one VGPR per swizzle class is kept; the rest is scalar.
    // (Rows that are not a power of two wide: every instruction of a wave keeps its own offset register.)
    constexpr int PER_A = !EVEN_A ? 1 : (8 / RPI_A) > 0 ? (8 / RPI_A) : 1, PER_B = !EVEN_B ? 1 : (8 / RPI_B) > 0 ? (8 / RPI_B) : 1;
    constexpr int GRP_A = (INST_A * RPI_A + 31) / 32, GRP_B = (INST_B * RPI_B + 31) / 32;   // 32-row groups per wave
    constexpr int NCLS_A = !EVEN_A ? INST_A : (PER_A < INST_A ? PER_A : INST_A) * GRP_A;
    constexpr int NCLS_B = !EVEN_B ? INST_B : (PER_B < INST_B ? PER_B : INST_B) * GRP_B;
    static_assert(!EVEN_A || (INST_A * RPI_A) % 32 == 0 || INST_A * RPI_A < 32, "a wave's rows cover whole 32-row groups");
    static_assert(!EVEN_B || (INST_B * RPI_B) % 32 == 0 || INST_B * RPI_B < 32, "a wave's rows cover whole 32-row groups");
    auto cls_a = [](int i) { return !EVEN_A ? i : i % PER_A + PER_A * (i * RPI_A / 32); };   // class of instruction i
    auto rep_a = [](int c) { return !EVEN_A ? c : c % PER_A + (c / PER_A) * (32 / (EVEN_A ? RPI_A : 1)); };   // first instruction of class c
    auto cls_b = [](int i) { return !EVEN_B ? i : i % PER_B + PER_B * (i * RPI_B / 32); };
    auto rep_b = [](int c) { return !EVEN_B ? c : c % PER_B + (c / PER_B) * (32 / (EVEN_B ? RPI_B : 1)); };
    uint32_t goff_a[NCLS_A], goff_b[NCLS_B], goff_s, goff_sb;
#pragma unroll
    for (int c_ = 0; c_ < NCLS_A; c_++) {
        int rl, ch, kl;                                       // row relative to the instruction's scalar base, chunk, stage row
        if constexpr (EVEN_A) {
            rl = lane / CPR_A, ch = lane % CPR_A, kl = (wave * INST_A + rep_a(c_)) * RPI_A + rl;
        } else {
            const int ql = rep_a(c_) * 64 + lane;
            rl = ql / CPR_A, ch = ql % CPR_A, kl = wave * ROWS_W_A + rl;
        }
        int c = ch ^ swizzle_of_row<BM>(kl);
        int m = m0 + c * 16;
        if (m + 16 > M) m = M - 16;                           // rows past M: any valid bytes will do
        goff_a[c_] = (uint32_t)rl * (uint32_t)ldm + (uint32_t)m;
    }
#pragma unroll
    for (int c_ = 0; c_ < NCLS_B; c_++) {
        int rl, ch, kl;
        if constexpr (EVEN_B) {
            rl = lane / CPR_B, ch = lane % CPR_B, kl = (wave * INST_B + rep_b(c_)) * RPI_B + rl;
        } else {
            const int ql = rep_b(c_) * 64 + lane;
            rl = ql / CPR_B, ch = ql % CPR_B, kl = wave * ROWS_W_B + rl;
        }
        int c = ch ^ swizzle_of_row<BN>(kl);
        int n = n0 + c * 16;
        if (n + 16 > N) n = N - 16;
        goff_b[c_] = (uint32_t)rl * (uint32_t)N + (uint32_t)n;
    }
    {
        // a_scale slot s of the stage holds the scale of row (s/WM)*WM + 16*(s%TM) + (s%WM)/TM of the tile, so that
        // the TM scales a lane needs (its column L of every m-tile of its wave) are contiguous in LDS.
        int sl = (wave < NSC ? wave : 0) * 64 + lane;
        int r = sl % WM;
        int m = m0 + (sl / WM) * WM + 16 * (r % TM) + r / TM;
        if (m > M - 1) m = M - 1;
        goff_s = (uint32_t)m * 4u;
        // b_scale slot l of the stage holds the scale of the l-th 128-column block the tile touches (clamped)
        int nbq = (n0 >> 7) + lane;
        if (nbq > QN - 1) nbq = QN - 1;
        goff_sb = (uint32_t)nbq * 4u;
    }
    // The LDS-DMA loads are issued through inline asm on purpose: the compiler cannot tell which stage a
    // transpose read touches, so for builtin LDS-DMA loads it waits for vmcnt(0) before the first LDS read
    // that follows them, which serialises the prefetch with the compute it is meant to overlap. Here the
    // kernel owns the wait: one s_waitcnt vmcnt before the barrier of each iteration. For the same reason the loop
    // contains no other vector memory load at all (the b_scale values come through LDS like the a_scale ones): the
    // compiler then never emits a vmcnt wait of its own inside it.
    // Addressing: 64-bit SGPR base (advances by 128 rows per K block) + per-lane 32-bit offset; M0 holds
    // the LDS destination of the instruction (lane l lands at M0 + 16*l, or M0 + 4*l for the dword form).
    const uint32_t lds_base = (uint32_t)(uintptr_t)(RF_LDS uint8_t *)lds;
    constexpr int D_SA = INST_A + INST_B, D_SB = D_SA + 1, NDMA = D_SB + 1;
    // DMA instruction d of this wave: A rows (d < INST_A), then B rows, then the a_scales (first NSC waves), then the
    // b_scales (wave 0). Its global source for K block kb is dma_src(d, kb); its LDS destination inside a stage is
    // fixed. In the loop each instruction keeps a running source pointer (one 64-bit scalar add per K block).
    const uint32_t lds_dst_a = lds_base + wave * (INST_A * 1024), lds_dst_b = lds_base + OFF_B + wave * (INST_B * 1024),
                   lds_dst_s = lds_base + OFF_S + wave * 256, lds_dst_sb = lds_base + OFF_S + OFF_SB;
    auto dma_src = [&](int d, int kb) -> const uint8_t * {
        if (d < INST_A) return A + ((size_t)kb * BK + (size_t)(EVEN_A ? (wave * INST_A + d) * RPI_A : wave * ROWS_W_A)) * ldm;
        if (d < D_SA)
            return B + ((size_t)kb * BK + (size_t)(EVEN_B ? (wave * INST_B + (d - INST_A)) * RPI_B : wave * ROWS_W_B)) * N;
        if (d == D_SA) return (const uint8_t *)(SA + (size_t)kb * ldm);
        return (const uint8_t *)(SB + (size_t)kb * QN);
    };
    auto dma_step = [&](int d) -> size_t {       // bytes from one K block to the next
        return d < INST_A ? (size_t)BK * ldm : d < D_SA ? (size_t)BK * N : d == D_SA ? (size_t)ldm * 4 : (size_t)QN * 4;
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
    // Wait until the loads of the stage that is read next have landed. Two stages: every load this wave has issued.
    // Three stages: all but the loads of the newest block; a wave's loads complete in the order it issued them, every
    // wave issues at least INST_A + INST_B per block (those with scale loads one or two more, whose oldest then have
    // to land as well), so "all but the newest INST_A + INST_B" covers it.
    auto wait_for_stage = [&]() {
        if constexpr (NS == 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" :: "n"(INST_A + INST_B) : "memory");
    };

    // ---- LDS -> MFMA operands: per-lane byte offsets of the transpose reads (stage 0, t = 0) ----
    // lane (L,g) of read t points at row k = 32g + 8t + L/2, half (L&1) of 16-byte chunk c.
    const int krow = 32 * g + (L >> 1);
    // chunk index of m-tile j is (wm*TM + j) ^ sw = ((wm*TM) ^ sw) ^ j when j < TM and wm*TM is a multiple of TM
    // (TM, TN powers of two): one base register per operand, the tile index is XORed in at the use. Other tile counts
    // keep one offset register per tile.
    constexpr bool POW2_T = (TM & (TM - 1)) == 0 && (TN & (TN - 1)) == 0;
    const uint32_t aoff_base = krow * BM + (((wm * TM) ^ swizzle_of_row<BM>(krow)) << 4) + 8 * (L & 1);
    // (OFF_B has no low bits set, so it passes through the XOR with the tile index unchanged)
    const uint32_t boff_base = OFF_B + krow * BN + (((wn * TN) ^ swizzle_of_row<BN>(krow)) << 4) + 8 * (L & 1);
    uint32_t aoff_tile[POW2_T ? 1 : TM], boff_tile[POW2_T ? 1 : TN];
    if constexpr (!POW2_T) {
#pragma unroll
        for (int j = 0; j < TM; j++)
            aoff_tile[j] = krow * BM + (((wm * TM + j) ^ swizzle_of_row<BM>(krow)) << 4) + 8 * (L & 1);
#pragma unroll
        for (int i = 0; i < TN; i++)
            boff_tile[i] = OFF_B + krow * BN + (((wn * TN + i) ^ swizzle_of_row<BN>(krow)) << 4) + 8 * (L & 1);
    }
    const uint32_t soff = OFF_S + (wm * WM + L * TM) * 4;               // this lane's TM scales
    // this wave's b_scale slots (slot = 128-column block - first block of the tile): n-tiles i < sb_split lie in the
    // block of slot 0, the others in the next one
    const int ncol0 = n0 + wn * WN;
    const int sb_split_raw = (((ncol0 >> 7) + 1) * 128 - ncol0) >> 4;
    const int sb_split = __builtin_amdgcn_readfirstlane(sb_split_raw < TN ? sb_split_raw : TN);
    const uint32_t sboff = OFF_S + OFF_SB + (((ncol0 >> 7) - (n0 >> 7)) << 2);
    const uint32_t sboff1 = sboff + (sb_split < TN ? 4 : 0);

#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
        for (int i = 0; i < TN; i++) acc[j][i] = (f32x4){0.f, 0.f, 0.f, 0.f};

    // ---- main loop: one K block per iteration, software-pipelined by hand across iterations ----
    // MFMA slot t = (m-tile j, n-tile i), row-major. In steady state the matrix pipe never waits for a K-block
    // boundary:
    //   * the partial sum of slot t goes to a ring of PR register tiles and is folded into the accumulator LAG
    //     slots later (the last LAG folds of a K block run in the first slots of the next one);
    //   * the A-matrix fragment of m-tile j+1 is fetched from LDS while the MFMAs of m-tile j issue;
    //   * the barrier that publishes the next stage sits before the LAST m-tile's slots (slot BAR_SLOT). In those
    //     slots each B-matrix fragment is dead as soon as its MFMA has issued and is refilled from the next
    //     stage, together with the first A fragment and the scales of the next K block;
    //   * after that barrier the stage just consumed is free: the LDS-DMA loads of K block kb+NS start there, one
    //     per slot, and run on into the first slots of the next iteration.
    // An empty volatile asm after each MFMA / fold anchors it in its slot, sched_barrier(0) keeps the slots apart;
    // the compiler still places the LDS waits and hazard nops.
    constexpr int NMFMA = TM * TN, PR = (NMFMA % 4 == 0 && TN > 3) ? 4 : 3, LAG = PR - 1, BAR_SLOT = (TM - 1) * TN;
    static_assert(NMFMA % PR == 0, "ring positions repeat per K block");
    static_assert(LAG < TN && LAG < PR, "lagged folds of a K block stay inside its last m-tile row");
    static_assert(TM % 2 == 0, "the last m-tile uses afrag[1], so afrag[0] is free for the next block");
    static_assert(NDMA - TN <= BAR_SLOT, "the DMA batch finishes well before the barrier that needs it");
    const int kb_last = kb_end - 1;
    auto clamp_kb = [&](int kb) { return kb < kb_last ? kb : kb_last; };   // past the end: re-fetch the last block

    i32x8 bfrag[TN], afrag[2];
    f32x4 pring[PR];
    float s[TM], s1[ONE_SB ? 1 : TM], sraw[TM], sb_raw = 0.f, sb_raw1 = 0.f;   // s1: scales of the second b_scale block
#pragma unroll
    for (int r = 0; r < PR; r++) pring[r] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < TM; j++) s[j] = 0.f;
#pragma unroll
    for (int j = 0; j < (ONE_SB ? 1 : TM); j++) s1[j] = 0.f;

    auto rd = [&](uint32_t stage_base, uint32_t off) {
        return __builtin_amdgcn_ds_read_tr8_b64_v2i32((RF_LDS i32x2 *)(lds + stage_base + off));
    };
    auto read_bfrag = [&](int i, int stage) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            i32x2 v = rd(stage * STAGE_B, (POW2_T ? boff_base ^ (i << 4) : boff_tile[POW2_T ? 0 : i]) + t * 8 * BN);
            bfrag[i][2 * t] = v[0];
            bfrag[i][2 * t + 1] = v[1];
        }
    };
    auto read_afrag = [&](int buf, int j, int stage) {
#pragma unroll
        for (int t = 0; t < 4; t++) {
            i32x2 v = rd(stage * STAGE_A, (POW2_T ? aoff_base ^ (j << 4) : aoff_tile[POW2_T ? 0 : j]) + t * 8 * BM);
            afrag[buf][2 * t] = v[0];
            afrag[buf][2 * t + 1] = v[1];
        }
    };
    auto read_scales = [&](int stage) {
        if constexpr (TM % 4 == 0) {
#pragma unroll
            for (int q = 0; q < TM / 4; q++) {
                f32x4 v = *(RF_LDS f32x4 *)(lds + stage * STAGE_S + soff + q * 16);
#pragma unroll
                for (int e = 0; e < 4; e++) sraw[4 * q + e] = v[e];
            }
        } else {
#pragma unroll
            for (int q = 0; q < TM / 2; q++) {
                f32x2 v = *(RF_LDS f32x2 *)(lds + stage * STAGE_S + soff + q * 8);
                sraw[2 * q] = v[0];
                sraw[2 * q + 1] = v[1];
            }
        }
        sb_raw = *(RF_LDS float *)(lds + stage * STAGE_S + sboff);
        if constexpr (!ONE_SB) sb_raw1 = *(RF_LDS float *)(lds + stage * STAGE_S + sboff1);
    };

    if (kb_begin < kb_end) {
        // prologue: stages 0..NS-2 <- the first K blocks, then the first operands; stage NS-1 <- start of the next
#pragma unroll
        for (int st = 0; st < NS - 1; st++)
#pragma unroll
            for (int d = 0; d < NDMA; d++) issue_dma(d, st, dma_src(d, clamp_kb(kb_begin + st)));
        wait_for_stage();
        __syncthreads();
        read_bfrag(0, 0);
        read_afrag(0, 0, 0);
        read_scales(0);
#pragma unroll
        for (int i = 1; i < TN; i++) read_bfrag(i, 0);
#pragma unroll
        for (int d = 0; d < TN && d < NDMA; d++) issue_dma(d, NS - 1, dma_src(d, clamp_kb(kb_begin + NS - 1)));
    }
    // running DMA sources: instructions d >= TN are issued for block kb+NS-1 in the first slots of iteration kb,
    // instructions d < TN for block kb+NS in its last slots (blocks past the end are clamped to the last one)
    const uint8_t *dsrc[NDMA];
#pragma unroll
    for (int d = 0; d < NDMA; d++) dsrc[d] = dma_src(d, clamp_kb(kb_begin + (d < TN ? NS : NS - 1)));
    // one K block; cur is the stage it reads (compile-time: the loop below is unrolled NS times)
    // split (compile-time): n-tiles i < split fold with s, the others with s1
    auto k_block = [&](auto cur_c, auto split_c, int kb) {
        constexpr int cur = decltype(cur_c)::value, nxt = (cur + 1) % NS, prv = (cur + NS - 1) % NS;
        constexpr int split = decltype(split_c)::value;
        const bool adv1 = kb + NS <= kb_last, adv2 = kb + NS + 1 <= kb_last;   // does the next iteration move on a block?
        // scales of the previous block's last m-tile (lagged folds)
        const float s_last = s[TM - 1], s1_last = s1[ONE_SB ? 0 : TM - 1];
#pragma unroll
        for (int j = 0; j < TM; j++) s[j] = sraw[j] * sb_raw;
        if constexpr (!ONE_SB)
#pragma unroll
            for (int j = 0; j < TM; j++) s1[j] = sraw[j] * sb_raw1;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NMFMA; t++) {
            const int j = t / TN, i = t % TN;
            if (t == BAR_SLOT) {
                // my DMA loads of the next stage have landed; after the barrier everyone's have, and everyone has
                // finished reading the current stage (its last fragment was fetched one m-tile ago)
                wait_for_stage();
                __syncthreads();
                __builtin_amdgcn_sched_barrier(0);
            }
            pring[t % PR] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                bfrag[i], afrag[j & 1], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
            asm volatile("" : "+v"(pring[t % PR]));          // anchor: the MFMA is issued here, not later
            __builtin_amdgcn_sched_barrier(0);
            // LDS-DMA: the batch for block kb+NS-1 (started in the previous iteration) continues in the first slots;
            // the batch for block kb+NS starts right after the barrier, into the stage this iteration has consumed
            if (t + TN < NDMA) {
                issue_dma(t + TN, prv, dsrc[t + TN]);
                dsrc[t + TN] += adv1 ? dma_step(t + TN) : 0;
            }
            if (t >= BAR_SLOT && t - BAR_SLOT < NDMA && t - BAR_SLOT < TN) {
                issue_dma(t - BAR_SLOT, cur, dsrc[t - BAR_SLOT]);
                dsrc[t - BAR_SLOT] += adv2 ? dma_step(t - BAR_SLOT) : 0;
            }
            // LDS -> registers
            if (j + 1 < TM) {
                if (i == 0) read_afrag((j + 1) & 1, j + 1, cur);      // a whole m-tile ahead of its use
            } else {
                read_bfrag(i, nxt);                                    // bfrag[i] is dead: refill for block kb+1
                if (i == 0) {
                    read_afrag(0, 0, nxt);
                    read_scales(nxt);
                }
            }
            // lagged fold
            if (t >= LAG) {
                const int u = t - LAG, ju = u / TN, iu = u % TN;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[ju][iu][e] = __builtin_fmaf(iu < split ? s[ju] : s1[ONE_SB ? 0 : ju], pring[u % PR][e], acc[ju][iu][e]);
                asm volatile("" : "+v"(acc[ju][iu]));        // anchor: the fold happens in this slot
            } else {
                const int u = NMFMA + t - LAG, ju = u / TN, iu = u % TN;   // tail of the previous K block
#pragma unroll
                for (int e = 0; e < 4; e++)
                    acc[ju][iu][e] = __builtin_fmaf(iu < split ? s_last : s1_last, pring[u % PR][e], acc[ju][iu][e]);
                asm volatile("" : "+v"(acc[ju][iu]));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto k_loop = [&](auto split_c) {
        constexpr int split = decltype(split_c)::value;
        int kb = kb_begin;
        if constexpr (NS == 2) {
            for (; kb + 1 < kb_end; kb += 2) {
                k_block(IntTag<0>{}, split_c, kb);
                k_block(IntTag<1>{}, split_c, kb + 1);
            }
            if (kb < kb_end) k_block(IntTag<0>{}, split_c, kb);
        } else {
            for (; kb + 2 < kb_end; kb += 3) {
                k_block(IntTag<0>{}, split_c, kb);
                k_block(IntTag<1>{}, split_c, kb + 1);
                k_block(IntTag<2>{}, split_c, kb + 2);
            }
            if (kb < kb_end) k_block(IntTag<0>{}, split_c, kb);
            if (kb + 1 < kb_end) k_block(IntTag<1>{}, split_c, kb + 1);
        }
        // folds still owed by the last K block
#pragma unroll
        for (int t = 0; t < LAG; t++) {
            const int u = NMFMA + t - LAG, ju = u / TN, iu = u % TN;
#pragma unroll
            for (int e = 0; e < 4; e++)
                acc[ju][iu][e] = __builtin_fmaf(iu < split ? s[TM - 1] : s1[ONE_SB ? 0 : TM - 1], pring[u % PR][e], acc[ju][iu][e]);
        }
    };
    if constexpr (ONE_SB) {
        k_loop(IntTag<TN>{});
    } else {
        // a wave whose columns lie in one block reads the same slot twice (sboff1 == sboff) and takes either path
        if (sb_split == 1) k_loop(IntTag<1>{});
        else k_loop(IntTag<2>{});
    }
    // LDS-DMA writes of the last (redundant) prefetches must land before this workgroup's LDS can be handed on
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes of C or of a split-K partial sum. The store carries device scope (sc1): the line is written through to
// memory instead of staying dirty in the XCD's L2 until the end of the kernel. C is written once and not read again,
// and with 56 to 88 MB of it the write-back at the end of the kernel was time that nothing overlapped (6144 x 7168 x
// 2048: 89.4 -> 87.2 us; non-temporal hints measured slower than either). The fp32 partial sums of a K split are read
// next by the reduction kernel, on whatever XCD its workgroups land, so they have to leave this L2 anyway
// (1024 x 1536 x 7168 with 4 splits: 24.2 -> 23.5 us, 1024 x 576 x 7168 with 8: 17.9 -> 17.0 us).
__device__ __forceinline__ void store_c16(void *p, const uint4 &v) {
    const u32x4 w = {v.x, v.y, v.z, v.w};
    // A store of more than 8 bytes reads its data registers a little after it has been issued; the compiler keeps
    // vector instructions that overwrite them away from its own stores, but it does not look inside this statement.
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" :: "v"(p), "v"(w) : "memory");
}

// Stores a wave's accumulators as bf16 into C, masked at the M and N edges. In the MFMA layout a lane owns 4
// consecutive n of one row, so a direct store instruction would touch 16 rows with 32-byte pieces. Instead each wave
// stages its tile, TM/PASSES m-tiles at a time, through its own LDS region (row = WN bf16 + 16 bytes of padding) and
// writes it back out with 16 bytes per lane, 8 lanes per row: every store instruction covers whole 128-byte lines.
// `staging` is the start of NW regions of StoreGeom::REGION bytes. BARRIER: the regions overlay the stage buffers,
// so all waves must call together and a barrier comes first (LDS-DMA loads of other waves may still be landing
// there). Without it the regions are private memory of the waves and nothing is synchronised.
template <int BM, int BN, int WAVES_M, int WAVES_N, int PASSES>
struct StoreGeom {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    static constexpr int ROW = G::WN * 2 + 16;           // bytes per staged row
    static constexpr int ROWS = G::TM / PASSES * 16;     // rows staged per pass
    static constexpr int REGION = ROWS * ROW;            // bytes per wave
    static_assert(G::TM % PASSES == 0, "whole m-tiles per pass");
};
// Passes used when the staging overlays the stage buffers: the fewest that give whole store instructions.
template <int BM, int WAVES_M>
constexpr int default_store_passes() { return (BM / WAVES_M / 16) % 3 == 0 ? 3 : 2; }
template <int BM, int BN, int WAVES_M, int WAVES_N, int PASSES = default_store_passes<BM, WAVES_M>(), bool BARRIER = true>
__device__ __forceinline__ void store_tile_bf16(const f32x4 (&acc)[BM / WAVES_M / 16][BN / WAVES_N / 16],
                                                uint16_t *__restrict__ C, int M, int N, int m0, int n0,
                                                uint8_t *staging) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    using S = StoreGeom<BM, BN, WAVES_M, WAVES_N, PASSES>;
    constexpr int ROW = S::ROW, ROWS = S::ROWS, TMP = G::TM / PASSES;
    constexpr int LPR = G::WN * 2 / 16;                  // lanes per row on the way out (16 bytes each)
    constexpr bool WHOLE_ROWS = 64 % LPR == 0;           // a store instruction covers whole rows
    constexpr int RPI = WHOLE_ROWS ? 64 / LPR : 1;       // rows per store instruction
    static_assert(!BARRIER || G::NW * S::REGION <= 2 * G::STAGE, "staging fits in the stage buffers");
    static_assert(WHOLE_ROWS ? ROWS % RPI == 0 : (ROWS * LPR) % 64 == 0, "whole store instructions");
    // the opaque zero keeps this address arithmetic below the main loop: hoisted above it, it would cost the
    // loop dozens of registers
    int vz;
    asm volatile("v_mov_b32 %0, 0" : "=v"(vz));
    const int lane = (threadIdx.x & 63) + vz, wave = threadIdx.x >> 6, L = lane & 15, g = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    uint8_t *region = staging + wave * S::REGION;
    if constexpr (BARRIER) __syncthreads();
#pragma unroll
    for (int h = 0; h < PASSES; h++) {
#pragma unroll
        for (int jj = 0; jj < TMP; jj++) {
            const int j = h * TMP + jj;
#pragma unroll
            for (int i = 0; i < G::TN; i++) {            // lane holds C[16j + L][16i + 4g .. +3]
                uint2 v;
                v.x = pack_bf16x2(acc[j][i][0], acc[j][i][1]);
                v.y = pack_bf16x2(acc[j][i][2], acc[j][i][3]);
                *(uint2 *)(region + (16 * jj + L) * ROW + (16 * i + 4 * g) * 2) = v;
            }
        }
        // same wave writes and reads its region: program order is enough, the compiler inserts the LDS wait
        if constexpr (WHOLE_ROWS) {
#pragma unroll
            for (int r0 = 0; r0 < ROWS; r0 += RPI) {
                const int r = r0 + lane / LPR, cb = (lane % LPR) * 16;          // row in the pass, byte column
                const uint4 v = *(const uint4 *)(region + r * ROW + cb);
                const int m = m0 + wm * G::WM + h * ROWS + r;
                const int n = n0 + wn * G::WN + cb / 2;
                if (m < M && n < N) store_c16(C + (size_t)m * N + n, v);
            }
        } else {
            // rows of LPR chunks with 64 % LPR != 0: the pass's chunks in row-major order, 64 per instruction
#pragma unroll
            for (int q0 = 0; q0 < ROWS * LPR; q0 += 64) {
                const int q = q0 + lane, r = q / LPR, cb = (q % LPR) * 16;
                const uint4 v = *(const uint4 *)(region + r * ROW + cb);
                const int m = m0 + wm * G::WM + h * ROWS + r;
                const int n = n0 + wn * G::WN + cb / 2;
                if (m < M && n < N) store_c16(C + (size_t)m * N + n, v);
            }
        }
    }
}

// The same for whole tiles (no edge masks) with the passes overlapped: one m-tile per pass through a private region
// of the wave, and the global stores of a pass are issued only after the next pass's LDS traffic. LDS executes a
// wave's instructions in order, so a pass may overwrite the region as soon as the previous pass's reads have been
// issued; only the stores wait for read data, and by then a later pass's conversions and LDS instructions have
// covered that latency. (With read -> store -> next write in program order a 256 x 256 tile's epilogue took 1.6 us
// on an otherwise idle chip, nearly all of it eight LDS round trips.)
// The staging region is written 8 bytes and read 16 bytes at a time: both through types that may alias anything, so
// that the compiler keeps the writes (to its type rules an 8-byte vector store is never read by a 16-byte vector
// load) and keeps them in order with the reads.
// Store instructions a wave issues for one unmasked tile (one m-tile per pass, 64 / LPR rows per instruction).
template <int BM, int BN, int WAVES_M, int WAVES_N>
constexpr int whole_tile_store_instructions() {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    return G::TM * (16 / (64 / (G::WN * 2 / 16)));
}
typedef uint32_t staged_u32x2 __attribute__((ext_vector_type(2), may_alias));
typedef uint32_t staged_u32x4 __attribute__((ext_vector_type(4), may_alias));
// MASKED: only the tile's first row_lim rows exist in C (a caller whose M is not a multiple of 16 has padded A and
// a_scale, not C); whole columns always.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool MASKED = false>
__device__ __forceinline__ void store_whole_tile_bf16(const f32x4 (&acc)[BM / WAVES_M / 16][BN / WAVES_N / 16],
                                                      uint16_t *__restrict__ C, int N, int m0, int n0, uint8_t *staging,
                                                      int row_lim = BM) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    constexpr int ROW = G::WN * 2 + 16;                  // bytes per staged row
    constexpr int LPR = G::WN * 2 / 16;                  // lanes per row on the way out (16 bytes each)
    static_assert(64 % LPR == 0 && 16 % (64 / LPR) == 0, "a store instruction covers whole rows of one m-tile");
    constexpr int RPI = 64 / LPR, NI = 16 / RPI;         // rows per store instruction, instructions per m-tile
    static_assert(G::TM * NI == whole_tile_store_instructions<BM, BN, WAVES_M, WAVES_N>(), "the persistent kernel counts on it");
    int vz;                                              // see store_tile_bf16
    asm volatile("v_mov_b32 %0, 0" : "=v"(vz));
    const int lane = (threadIdx.x & 63) + vz, wave = threadIdx.x >> 6, L = lane & 15, g = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    uint8_t *region = staging + wave * (16 * ROW);
    uint16_t *out = C + (size_t)(m0 + wm * G::WM + lane / LPR) * N + n0 + wn * G::WN + (lane % LPR) * 8;
    staged_u32x4 v[2][NI];
#pragma unroll
    for (int j = 0; j <= G::TM; j++) {
        if (j < G::TM) {
#pragma unroll
            for (int i = 0; i < G::TN; i++) {            // lane holds C[16j + L][16i + 4g .. +3]
                const staged_u32x2 w = {pack_bf16x2(acc[j][i][0], acc[j][i][1]), pack_bf16x2(acc[j][i][2], acc[j][i][3])};
                *(staged_u32x2 *)(region + L * ROW + (16 * i + 4 * g) * 2) = w;
            }
#pragma unroll
            for (int q = 0; q < NI; q++)
                v[j & 1][q] = *(const staged_u32x4 *)(region + (q * RPI + lane / LPR) * ROW + (lane % LPR) * 16);
        }
        if (j > 0) {
#pragma unroll
            for (int q = 0; q < NI; q++) {
                const staged_u32x4 x = v[(j - 1) & 1][q];
                if (!MASKED || wm * G::WM + (j - 1) * 16 + q * RPI + lane / LPR < row_lim)
                    store_c16(out + (size_t)((j - 1) * 16 + q * RPI) * N, make_uint4(x[0], x[1], x[2], x[3]));
            }
        }
    }
}

// fp32 tile with leading dimension ld; rows < m_lim and cols < n_lim are written (limits relative to the tile).
// Through LDS, one m-tile (16 rows) of every wave per pass, written out 16 bytes per lane with neighbouring lanes along
// a row: each store instruction covers whole rows of the wave tile (256 contiguous bytes for 64 columns) instead of
// sixteen 64-byte pieces. Starts with a barrier like store_tile_bf16 (the regions overlay the stages).
template <int BM, int BN, int WAVES_M, int WAVES_N>
__device__ __forceinline__ void store_tile_f32_staged(const f32x4 (&acc)[BM / WAVES_M / 16][BN / WAVES_N / 16],
                                                      float *__restrict__ t, size_t ld, int m_lim, int n_lim,
                                                      uint8_t *staging) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    constexpr int ROW = G::WN * 4 + 16, REGION = 16 * ROW;
    constexpr int LPR = G::WN / 4;                        // lanes per row (16 bytes each)
    constexpr bool WHOLE_ROWS = 64 % LPR == 0;            // a store instruction covers whole rows
    constexpr int RPI = WHOLE_ROWS ? 64 / LPR : 1;        // rows per store instruction
    static_assert(G::NW * REGION <= 2 * G::STAGE && (WHOLE_ROWS ? 16 % RPI == 0 : (16 * LPR) % 64 == 0), "staging geometry");
    int vz;                                  // see store_tile_bf16
    asm volatile("v_mov_b32 %0, 0" : "=v"(vz));
    const int lane = (threadIdx.x & 63) + vz, wave = threadIdx.x >> 6, L = lane & 15, g = lane >> 4;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    uint8_t *region = staging + wave * REGION;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < G::TM; j++) {
#pragma unroll
        for (int i = 0; i < G::TN; i++) *(f32x4 *)(region + L * ROW + (16 * i + 4 * g) * 4) = acc[j][i];
        if constexpr (WHOLE_ROWS) {
#pragma unroll
            for (int r0 = 0; r0 < 16; r0 += RPI) {
                const int r = r0 + lane / LPR, cb = (lane % LPR) * 16;
                const uint4 v = *(const uint4 *)(region + r * ROW + cb);
                const int m = wm * G::WM + 16 * j + r, n = wn * G::WN + cb / 4;
                if (m < m_lim && n < n_lim) store_c16(t + (size_t)m * ld + n, v);
            }
        } else {
            // rows of LPR chunks with 64 % LPR != 0: the m-tile's chunks in row-major order, 64 per instruction
#pragma unroll
            for (int q0 = 0; q0 < 16 * LPR; q0 += 64) {
                const int q = q0 + lane, r = q / LPR, cb = (q % LPR) * 16;
                const uint4 v = *(const uint4 *)(region + r * ROW + cb);
                const int m = wm * G::WM + 16 * j + r, n = wn * G::WN + cb / 4;
                if (m < m_lim && n < n_lim) store_c16(t + (size_t)m * ld + n, v);
            }
        }
    }
}

// Partial tiles exchanged between workgroups of the stream-K grid. The two workgroups may sit on different XCDs,
// whose L2 caches are not coherent with each other. Instead of device-wide fences (which write back and invalidate
// a whole L2, throwing away the A/B tiles every other workgroup on the XCD is re-using), each access carries system
// scope itself: relaxed 64-bit atomic stores write through to memory, relaxed atomic loads bypass the caches.
// Layout is register order (tile (j,i) of wave w at ((w*TM + j)*TN + i)*256 floats, lane l at +4l): every store
// instruction covers 1 KiB of contiguous memory; the only reader is a workgroup with the same thread mapping.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool ACCUMULATE_FROM>
__device__ __forceinline__ void exchange_tile_f32(f32x4 (&acc)[BM / WAVES_M / 16][BN / WAVES_N / 16], float *t) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    int vz;                                  // see store_tile_bf16
    asm volatile("v_mov_b32 %0, 0" : "=v"(vz));
    uint64_t *q = (uint64_t *)(t + ((size_t)(threadIdx.x >> 6) * (G::TM * G::TN) * 64 + (threadIdx.x & 63) + vz) * 4);
#pragma unroll
    for (int j = 0; j < G::TM; j++) {
#pragma unroll
        for (int i = 0; i < G::TN; i++) {
            if constexpr (ACCUMULATE_FROM) {
                f32x2 lo = __builtin_bit_cast(f32x2, __hip_atomic_load(q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM));
                f32x2 hi = __builtin_bit_cast(f32x2, __hip_atomic_load(q + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM));
                acc[j][i][0] += lo[0]; acc[j][i][1] += lo[1]; acc[j][i][2] += hi[0]; acc[j][i][3] += hi[1];
            } else {
                f32x2 lo = {acc[j][i][0], acc[j][i][1]}, hi = {acc[j][i][2], acc[j][i][3]};
                __hip_atomic_store(q, __builtin_bit_cast(uint64_t, lo), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                __hip_atomic_store(q + 1, __builtin_bit_cast(uint64_t, hi), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            q += 128;                        // next tile: 64 lanes x 16 bytes further
        }
    }
}

// ---------------------------------------------------------------------------------------------
// One workgroup per (tile, K split). PARTIAL=false: writes bf16 C. PARTIAL=true: writes the fp32 partial sums of
// the K range of split blockIdx.y to ws[split][M][N] (summed by reduce_splitk_bf16). M_store <= M is the number of
// rows of bf16 C that exist (a caller whose M is not a multiple of 16 passes A padded to M rows and its own C).
// Requirements checked by the host: M%16==0, N%16==0, M>=16, N>=16, a/b 16-byte aligned,
// c 16-byte aligned, K%128==0.
// ---------------------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, bool PARTIAL, int NS = 2>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_fp8_blockscale_tile(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, void *__restrict__ Cout, int M, int N, int K, int kb_per_split,
    int tiles_m, int tiles_n, int group_m, int M_store) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N, NS>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, tiles_m * tiles_n, tiles_m, tiles_n, group_m, true, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int QK = K / BK;
    const int kb_begin = blockIdx.y * kb_per_split;
    const int kb_end = kb_begin + kb_per_split < QK ? kb_begin + kb_per_split : QK;
    f32x4 acc[G::TM][G::TN];
    tile_mainloop<BM, BN, WAVES_M, WAVES_N, NS>(A, B, SA, SB, M, M, N, m0, n0, kb_begin, kb_end, lds, acc);
    if constexpr (PARTIAL)
        store_tile_f32_staged<BM, BN, WAVES_M, WAVES_N>(acc, (float *)Cout + ((size_t)blockIdx.y * M + m0) * N + n0, N,
                                                        M - m0, N - n0, lds);
    else
        store_tile_bf16<BM, BN, WAVES_M, WAVES_N>(acc, (uint16_t *)Cout, M_store, N, m0, n0, lds);
}

// ---------------------------------------------------------------------------------------------
// K split inside one workgroup. GROUPS wave groups (NW waves each) compute the same BM x BN tile, group g over K blocks
// [g * QK / GROUPS, (g + 1) * QK / GROUPS) with LDS stages of its own; then groups 1.. hand their fp32 accumulators to
// group 0 through LDS, which adds them in group order and stores bf16: the bits of the two-launch form with GROUPS equal
// K parts (PARTIAL kernel + reduce_splitk_bf16), without the partial sums' trip through memory and without the second
// launch. Every wave of the workgroup runs the same number of loop iterations (each holds a workgroup-wide barrier), so
// the host launches it only when QK % GROUPS == 0; the kernel returns at once otherwise.
// Same argument list as gemm_fp8_blockscale_tile (kb_per_split is not used).
// ---------------------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, int GROUPS>
struct InWgSplitGeom {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N, NS>;
    static constexpr int GROUP_LDS = (G::LDS_BYTES + 1023) / 1024 * 1024;
    static constexpr int LDS_BYTES = GROUPS * GROUP_LDS;
    static_assert(LDS_BYTES <= 160 * 1024, "every group's stages fit the CU's LDS");
    static_assert(G::TM * G::TN * G::NT * 16 <= GROUP_LDS, "a group's accumulators fit its own LDS region");
    static_assert(G::NT * GROUPS <= 1024, "one workgroup");
};
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS, int GROUPS>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64 * GROUPS) void gemm_fp8_blockscale_tile_ksplit_in_wg(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, void *__restrict__ Cout, int M, int N, int K, int kb_per_split,
    int tiles_m, int tiles_n, int group_m, int M_store) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N, NS>;
    using W = InWgSplitGeom<BM, BN, WAVES_M, WAVES_N, NS, GROUPS>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int QK = K / BK;
    if (QK % GROUPS != 0) return;                           // never launched so: unequal K parts would not meet at the barriers
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, tiles_m * tiles_n, tiles_m, tiles_n, group_m, true, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int grp = __builtin_amdgcn_readfirstlane((int)threadIdx.x / G::NT), len = QK / GROUPS;
    uint8_t *my_lds = lds + grp * W::GROUP_LDS;
    f32x4 acc[G::TM][G::TN];
    tile_mainloop<BM, BN, WAVES_M, WAVES_N, NS>(A, B, SA, SB, M, M, N, m0, n0, grp * len, (grp + 1) * len, my_lds, acc);
    __syncthreads();                                        // every group is done with its stages
    // accumulators in register order: tile (j, i) of thread t of the group at ((j * TN + i) * NT + t) * 16 bytes
    f32x4 *mine = (f32x4 *)my_lds + (int)threadIdx.x % G::NT;
    if (grp > 0) {
#pragma unroll
        for (int j = 0; j < G::TM; j++)
#pragma unroll
            for (int i = 0; i < G::TN; i++) mine[(j * G::TN + i) * G::NT] = acc[j][i];
    }
    __syncthreads();
    if (grp == 0) {
#pragma unroll
        for (int q = 1; q < GROUPS; q++) {
            const f32x4 *theirs = (const f32x4 *)(lds + q * W::GROUP_LDS) + (int)threadIdx.x % G::NT;
#pragma unroll
            for (int j = 0; j < G::TM; j++)
#pragma unroll
                for (int i = 0; i < G::TN; i++) {
                    const f32x4 v = theirs[(j * G::TN + i) * G::NT];
                    acc[j][i][0] += v[0]; acc[j][i][1] += v[1]; acc[j][i][2] += v[2]; acc[j][i][3] += v[3];
                }
        }
        // staging in group 0's own region, which nobody else touches any more: no barrier (the other groups are gone)
        store_tile_bf16<BM, BN, WAVES_M, WAVES_N, default_store_passes<BM, WAVES_M>(), false>(acc, (uint16_t *)Cout, M_store, N,
                                                                                              m0, n0, lds);
    }
}

// ---------------------------------------------------------------------------------------------
// Stream-K: a persistent grid of P workgroups (one per CU). The T tiles x QK K-blocks are laid out as one line of
// work units and cut into P equal contiguous ranges, so every CU gets the same number of MFMAs whatever T is
// (432 tiles on 256 CUs is 1.69 tiles each, not 2). A workgroup walks its range tile by tile. A tile whose K
// range is shared by several workgroups is finished by whichever of them arrives last: each one stores its fp32
// partial tile to its workspace slot with write-through stores and bumps the tile's counter; the one that
// reads count == parts-1 adds the other partials and writes bf16. Nobody waits for anybody, so there is nothing to
// deadlock, and the last arriver resets the counter: the counters are zero again when the kernel ends.
// Used only when every range is at least QK units long (T >= P), so a split tile has exactly 2 contributors.
// ws: tile_count[T] (unsigned, zero on entry), then at byte offset ws_slots_off 2*P slots of BM*BN floats.
// ---------------------------------------------------------------------------------------------
template <int BM, int BN, int WAVES_M, int WAVES_N>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_fp8_blockscale_streamk(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, uint16_t *__restrict__ C, int M, int N, int K, int tiles_m, int tiles_n, int group_m,
    unsigned *__restrict__ tile_count, float *__restrict__ slots) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    volatile unsigned *mailbox = (volatile unsigned *)(lds + 2 * G::STAGE);
    const int P = gridDim.x, QK = K / BK;
    const long long U = (long long)tiles_m * tiles_n * QK;
    // workgroups are dealt round-robin to the XCDs: give each XCD a contiguous band of the unit line
    const int xcd = blockIdx.x % NUM_XCD, idx = blockIdx.x / NUM_XCD, per = P / NUM_XCD, rem = P % NUM_XCD;
    const int slot = xcd * per + (xcd < rem ? xcd : rem) + idx;
    auto lo_of = [&](int s) { return (long long)s * U / P; };
    auto slot_of = [&](long long u) { return (int)((((u + 1) * P) - 1) / U); };   // largest s with lo_of(s) <= u
    const long long lo = lo_of(slot), hi = lo_of(slot + 1);
    for (long long u = lo; u < hi;) {
        const int tile = (int)(u / QK);
        const long long tq = (long long)tile * QK;
        const int kb0 = (int)(u - tq);
        const int kb1 = hi - tq < QK ? (int)(hi - tq) : QK;
        int tile_m, tile_n;
        tile_of_block(tile, tiles_m * tiles_n, tiles_m, tiles_n, group_m, false, tile_m, tile_n);
        const int m0 = tile_m * BM, n0 = tile_n * BN;
        f32x4 acc[G::TM][G::TN];
        __syncthreads();                     // every wave is done with LDS (previous segment, or the mailbox)
        tile_mainloop<BM, BN, WAVES_M, WAVES_N>(A, B, SA, SB, M, M, N, m0, n0, kb0, kb1, lds, acc);
        bool write_c = (kb0 == 0 && kb1 == QK);
        if (!write_c) {
            // the host only launches this kernel with T >= P, so a tile has exactly two contributors: the workgroup
            // whose range ends inside it and the next one
            const int s_first = slot_of(tq);
            const int other = slot == s_first ? slot + 1 : slot - 1;
            // a contributor's slot: 2*s for the first segment of its range, 2*s+1 when the tile starts before its range
            auto slot_ptr = [&](int s) { return slots + (size_t)(2 * s + (lo_of(s) < tq ? 1 : 0)) * (BM * BN); };
            exchange_tile_f32<BM, BN, WAVES_M, WAVES_N, false>(acc, slot_ptr(slot));
            // the write-through stores are acknowledged (vmcnt) once they are at the coherence point; only then may
            // the counter move
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
            if (threadIdx.x == 0)
                *mailbox = __hip_atomic_fetch_add(tile_count + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __syncthreads();
            if (*mailbox == 1u) {            // the other contributor arrived first: I finish the tile
                exchange_tile_f32<BM, BN, WAVES_M, WAVES_N, true>(acc, slot_ptr(other));
                if (threadIdx.x == 0)        // ready for the next launch
                    __hip_atomic_store(tile_count + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                write_c = true;
            }
        }
        if (write_c) store_tile_bf16<BM, BN, WAVES_M, WAVES_N>(acc, C, M, N, m0, n0, lds);
        u = tq + kb1;
    }
}

// Sum of split-K partials in split order 0..S-1, then one bf16 rounding
// (the reference's reduce_kernel, src/gemm/gemm_kernel.cpp:288-303). 4 outputs per thread.
// mn: elements of C; split_stride: elements between two splits in ws (>= mn: the partials may have more rows than C).
__global__ __launch_bounds__(256) void reduce_splitk_bf16(const float *__restrict__ ws, uint16_t *__restrict__ C,
                                                          size_t mn, int splits, size_t split_stride) {
    size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= mn) return;
    const float *p = ws + i;
    f32x4 s = *(const f32x4 *)p;
    // The partials of up to 8 splits are fetched together and then added in split order: with one load per loop
    // iteration a small output (few threads, nothing else to run) pays the memory latency once per split.
    constexpr int BATCH = 8;
    int q0 = 1;
    for (; q0 + BATCH <= splits; q0 += BATCH) {
        f32x4 v[BATCH];
#pragma unroll
        for (int q = 0; q < BATCH; q++) v[q] = *(const f32x4 *)(p + (size_t)(q0 + q) * split_stride);
#pragma unroll
        for (int q = 0; q < BATCH; q++) {
            s[0] += v[q][0]; s[1] += v[q][1]; s[2] += v[q][2]; s[3] += v[q][3];
        }
    }
    if (q0 < splits) {
        f32x4 v[BATCH - 1];
#pragma unroll
        for (int q = 0; q < BATCH - 1; q++)
            if (q0 + q < splits) v[q] = *(const f32x4 *)(p + (size_t)(q0 + q) * split_stride);
#pragma unroll
        for (int q = 0; q < BATCH - 1; q++)
            if (q0 + q < splits) {
                s[0] += v[q][0]; s[1] += v[q][1]; s[2] += v[q][2]; s[3] += v[q][3];
            }
    }
    uint2 o;
    o.x = pack_bf16x2(s[0], s[1]);
    o.y = pack_bf16x2(s[2], s[3]);
    *(uint2 *)(C + i) = o;
}

// ---------------------------------------------------------------------------------------------
// Grouped form: `groups` independent GEMMs that share N and K, one launch. A (and a_scale, C) hold the rows of all
// groups back to back (group g owns rows row_start[g] .. row_start[g+1]-1 of an M_total-row matrix), B and b_scale
// hold one [K][N] / [K/128][QN] block per group. This is the layout of expert GEMMs after tokens have been sorted by
// expert (the reference's consumer is LaunchGroupGEMM over first_token_offset, src/moe/moe.cpp:213-248, which runs
// fp16 hipBLASLt there). One workgroup per (group, tile): the table is small enough to travel as a kernel argument.
// Requirements checked by the host: every row_start a multiple of 16 (and so M_total), N % 16 == 0, K % 128 == 0.
// C may pack the groups more tightly than A does: group g writes out_row_start[g+1] - out_row_start[g] rows from row
// out_row_start[g] of C, any counts, while its A rows start at row_start[g] and are padded to a multiple of 16 (the
// host stages A that way when the caller's group sizes are not multiples of 16).
//
// Which workgroup computes what. The expert weights are the bulk of the bytes (one [K][N] block per group, read by
// the few row tiles the group has), and what an XCD's workgroups read its own L2 has to fetch: with a group's tiles
// dealt round-robin over the 8 XCDs every L2 fetches the group's A rows and several L2s the same weight tile (32
// uneven groups, 8192 x 4096 x 7168: 2.06 GB fetched for 1.0 GB of operands; 1.28 GB with the map below). So the work
// items are put in one line, group by group, a group's column tiles one after the other and the row tiles of a
// column tile side by side, and the line is cut into 8 contiguous pieces with the same number of items, one per XCD.
// An XCD then works through a few whole groups: a weight tile is fetched by one L2 and serves all row tiles of its
// group there, and a group's A rows are fetched once (twice for a group cut by a piece boundary). Workgroup b runs
// on XCD b % 8 and takes item number b / 8 of that XCD's piece. Equal counts, not equal estimated cost: workgroups
// are handed out in the order of their ids, and when the XCD whose turn it is has no free CU the others wait with
// it, so all XCDs move through their pieces at the same pace; pieces of equal estimated cost but different lengths
// (a 128-row tile counted as 0.6 of a 256-row one) measured 12 % slower than equal counts on uneven groups.
// ---------------------------------------------------------------------------------------------
constexpr int kMaxGroups = 256;
struct GroupTable {
    int row_start[kMaxGroups + 1];      // first row of each group in A and a_scale (multiples of 16)
    int out_row_start[kMaxGroups + 1];  // first row of each group in C; the differences are the true row counts
    int tile_start[kMaxGroups + 1];     // prefix of work items (one per tile); tile_start[groups] is their number
};
// Work item of this workgroup: its group and its index among the group's items. False: nothing to do (the grid is
// 8 x the longest piece).
__device__ __forceinline__ bool grouped_work_item(const GroupTable &table, int groups, int &grp, int &local) {
    const int xcd = blockIdx.x % NUM_XCD;
    const long items = table.tile_start[groups];
    const int item = (int)(items * xcd / NUM_XCD) + (int)(blockIdx.x / NUM_XCD);
    if (item >= (int)(items * (xcd + 1) / NUM_XCD)) return false;
    // the last g with tile_start[g] <= item (empty groups own no item)
    int lo = 0, hi = groups;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (table.tile_start[mid] <= item) lo = mid; else hi = mid;
    }
    grp = lo;
    local = item - table.tile_start[lo];
    return true;
}
template <int BM, int BN, int WAVES_M, int WAVES_N, int NS = 2>
__global__ __launch_bounds__(WAVES_M *WAVES_N * 64) void gemm_fp8_blockscale_grouped(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, uint16_t *__restrict__ C, int M_total, int N, int K, int groups,
    const GroupTable table) {
    using G = TileGeom<BM, BN, WAVES_M, WAVES_N>;
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    int grp, local;
    if (!grouped_work_item(table, groups, grp, local)) return;
    const int row0 = table.row_start[grp], rows = table.row_start[grp + 1] - row0;
    const int out0 = table.out_row_start[grp], out_rows = table.out_row_start[grp + 1] - out0;
    const int tiles_m = (rows + BM - 1) / BM;
    const int m0 = (local % tiles_m) * BM, n0 = (local / tiles_m) * BN;
    const int QK = K / BK, QN = (N + 127) / 128;
    f32x4 acc[G::TM][G::TN];
    tile_mainloop<BM, BN, WAVES_M, WAVES_N, NS>(A + row0, B + (size_t)grp * K * N, SA + row0,
                                                SB + (size_t)grp * QK * QN, rows, M_total, N, m0, n0, 0, QK, lds, acc);
    store_tile_bf16<BM, BN, WAVES_M, WAVES_N>(acc, C + (size_t)out0 * N, out_rows, N, m0, n0, lds);
}

// The same with two tile heights in one launch: a group's rows are cut into 256-row tiles, and what is left over
// goes to a 128 x 256 tile when it is at most 128 rows (otherwise to one more 256-row tile). With uneven groups half
// of the left-overs are that small, and a 128-row tile costs little more than half a 256-row one. A column tile of a
// group has one work item per row tile, the 128-row one last. Both paths are 8 waves and share the LDS allocation;
// the branch is uniform over the workgroup.
__global__ __launch_bounds__(512) void gemm_fp8_blockscale_grouped_mixed(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, uint16_t *__restrict__ C, int M_total, int N, int K, int groups,
    const GroupTable table) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    int grp, local;
    if (!grouped_work_item(table, groups, grp, local)) return;
    const int row0 = table.row_start[grp], rows = table.row_start[grp + 1] - row0;
    const int out0 = table.out_row_start[grp], out_rows = table.out_row_start[grp + 1] - out0;
    const int big_m = rows / 256 + (rows % 256 > 128 ? 1 : 0);       // 256-row tiles of this group
    const int tiles_m = rows / 256 + (rows % 256 > 0 ? 1 : 0);       // row tiles of either height
    const int tile_m = local % tiles_m, n0 = (local / tiles_m) * 256;
    const int QK = K / BK, QN = (N + 127) / 128;
    const uint8_t *Bg = B + (size_t)grp * K * N;
    const float *SBg = SB + (size_t)grp * QK * QN;
    if (tile_m < big_m) {
        const int m0 = tile_m * 256;
        f32x4 acc[TileGeom<256, 256, 2, 4>::TM][TileGeom<256, 256, 2, 4>::TN];
        tile_mainloop<256, 256, 2, 4>(A + row0, Bg, SA + row0, SBg, rows, M_total, N, m0, n0, 0, QK, lds, acc);
        store_tile_bf16<256, 256, 2, 4>(acc, C + (size_t)out0 * N, out_rows, N, m0, n0, lds);
    } else {
        const int r1 = row0 + big_m * 256, rest = rows - big_m * 256;  // 16..128 rows
        f32x4 acc[TileGeom<128, 256, 2, 4>::TM][TileGeom<128, 256, 2, 4>::TN];
        tile_mainloop<128, 256, 2, 4, 3>(A + r1, Bg, SA + r1, SBg, rest, M_total, N, 0, n0, 0, QK, lds, acc);
        store_tile_bf16<128, 256, 2, 4>(acc, C + (size_t)(out0 + big_m * 256) * N, out_rows - big_m * 256, N, 0, n0, lds);
    }
}

// The grouped GEMM with tiles of four heights and work queues. A group's rows are cut into 256-row tiles and one last
// tile of 64, 128, 192 or 256 rows (the smallest that holds what is left), all 256 columns wide and all run by eight
// waves: uneven groups pad their rows to a multiple of 64 instead of 128 or 256 (32 groups of 16..816 rows: 9088 rows
// of MFMA work instead of 10240), and a short tile spends its time on what it has to do anyway, streaming its column
// tile of the group's weights. Tiles of different heights take different times, so the work is not dealt out by the
// hardware's dispatcher (which hands out workgroups in id order and makes all XCDs wait for the slowest): one
// workgroup per CU stays resident and takes items from queues, one queue per XCD. The host puts the items in one
// line (group after group in an order of its choice; inside a group column tile by column tile, the row tiles of one
// column tile next to each other) and cuts the line into eight pieces, one per queue: whole groups per queue where
// there are enough of them, the longest first, so that a group's activations and each of its weight tiles are
// fetched by one L2 and the short tiles fill the end of the launch. (Column tiles dealt out over the XCDs instead,
// every queue with the same mix: 6 % slower, every XCD then fetches every group's activations.) A workgroup whose
// own queue is empty helps with the others' in turn. A queue is one counter in device memory: atomicInc with a wrap
// value of (items + workgroups - 1). Every workgroup draws from a queue until it draws a number that is no item,
// exactly once per queue, so the counter's last draw wraps it back to zero: the counters need no clearing between
// launches (launches that share counters must not overlap).
// In the table of this kernel tile_start[p] counts the items of the first p groups of the line.
// ---------------------------------------------------------------------------------------------
struct GroupQueues {
    int piece_start[NUM_XCD + 1];        // queue x holds items piece_start[x] .. piece_start[x + 1] - 1 of the line
    int workgroups;                      // of the launch
    uint8_t order[kMaxGroups];           // order[p]: the group at position p of the line
};
constexpr int kQueueTileLds =
    TileGeom<256, 256, 2, 4>::LDS_BYTES > TileGeom<128, 256, 2, 4, 3>::LDS_BYTES ? TileGeom<256, 256, 2, 4>::LDS_BYTES
                                                                                 : TileGeom<128, 256, 2, 4, 3>::LDS_BYTES;
static_assert(TileGeom<192, 256, 2, 4>::LDS_BYTES <= kQueueTileLds && TileGeom<64, 256, 2, 4, 3>::LDS_BYTES <= kQueueTileLds,
              "the 256- and 128-row tiles are the largest");
constexpr int kQueueLds = kQueueTileLds + 16;                    // + the slot through which a draw reaches all waves
template <int BM, int NS>
__device__ __forceinline__ void grouped_queue_tile(const uint8_t *A, const uint8_t *B, const float *SA, const float *SB,
                                                   uint16_t *C, int rows, int out_rows, int M_total, int N, int n0, int QK,
                                                   uint8_t *lds) {
    f32x4 acc[TileGeom<BM, 256, 2, 4>::TM][TileGeom<BM, 256, 2, 4>::TN];
    int vz;
    asm volatile("v_mov_b32 %0, 0" : "=v"(vz));
    tile_mainloop<BM, 256, 2, 4, NS>(A, B, SA, SB, rows, M_total, N, 0, n0, 0, QK, lds, acc, vz);
    store_tile_bf16<BM, 256, 2, 4>(acc, C, out_rows, N, 0, n0, lds);
}
__global__ __launch_bounds__(512) void gemm_fp8_blockscale_grouped_queue(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, uint16_t *__restrict__ C, int M_total, int N, int K, int groups,
    const GroupTable table, const GroupQueues queues, unsigned *__restrict__ counters) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    volatile int *drawn = (volatile int *)(lds + kQueueTileLds);
    const int QK = K / BK, QN = (N + 127) / 128;
    const int xcd = blockIdx.x % NUM_XCD;
    for (int turn = 0; turn < NUM_XCD; turn++) {
        const int qx = (xcd + turn) % NUM_XCD;
        const int first = queues.piece_start[qx], count = queues.piece_start[qx + 1] - first;
        for (;;) {
            __syncthreads();             // the previous item's staged stores and the previous draw have been read
            if (threadIdx.x == 0)
                *drawn = (int)atomicInc(counters + qx, (unsigned)(count + queues.workgroups - 1));
            __syncthreads();
            const int got = __builtin_amdgcn_readfirstlane(*drawn);
            if (got >= count) break;
            const int item = first + got;
            int lo = 0, hi = groups;     // the last p with tile_start[p] <= item (empty groups own no item)
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (table.tile_start[mid] <= item) lo = mid; else hi = mid;
            }
            const int grp = queues.order[lo], local = item - table.tile_start[lo];
            const int row0 = table.row_start[grp], rows = table.row_start[grp + 1] - row0;
            const int out0 = table.out_row_start[grp], out_rows = table.out_row_start[grp + 1] - out0;
            const int full = rows / 256, rest = rows - full * 256;
            const int tiles_m = full + (rest > 0 ? 1 : 0);
            const int tile_m = local % tiles_m, n0 = (local / tiles_m) * 256, m0 = tile_m * 256;
            const int height = tile_m < full ? 4 : (rest + 63) / 64;           // in units of 64 rows
            const uint8_t *Ai = A + row0 + m0, *Bg = B + (size_t)grp * K * N;
            const float *SAi = SA + row0 + m0, *SBg = SB + (size_t)grp * QK * QN;
            uint16_t *Ci = C + (size_t)(out0 + m0) * N;
            const int r = rows - m0, o = out_rows - m0;
            if (height == 4) grouped_queue_tile<256, 2>(Ai, Bg, SAi, SBg, Ci, r, o, M_total, N, n0, QK, lds);
            else if (height == 3) grouped_queue_tile<192, 2>(Ai, Bg, SAi, SBg, Ci, r, o, M_total, N, n0, QK, lds);
            else if (height == 2) grouped_queue_tile<128, 3>(Ai, Bg, SAi, SBg, Ci, r, o, M_total, N, n0, QK, lds);
            else grouped_queue_tile<64, 3>(Ai, Bg, SAi, SBg, Ci, r, o, M_total, N, n0, QK, lds);
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Bounds-checked kernel for shapes or alignments the tiled kernel does not take (M or N not a
// multiple of 16, unaligned pointers). One wave per 16x16 output tile, bytes gathered directly
// from global memory; out-of-range rows/columns contribute zeros and are not stored.
// ---------------------------------------------------------------------------------------------
__global__ __launch_bounds__(64) void gemm_fp8_blockscale_checked(
    const uint8_t *__restrict__ A, const uint8_t *__restrict__ B, const float *__restrict__ SA,
    const float *__restrict__ SB, uint16_t *__restrict__ C, int M, int ldm, int N, int K) {
    const int lane = threadIdx.x, L = lane & 15, g = lane >> 4;
    const int m0 = blockIdx.y * 16, n0 = blockIdx.x * 16;
    const int QK = K / BK, QN = (N + 127) / 128;
    const int m_ld = m0 + L, n_ld = n0 + L;                  // operand rows this lane gathers
    const bool m_ok = m_ld < M, n_ok = n_ld < N;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int kb = 0; kb < QK; kb++) {
        union { i32x8 v; uint8_t b[32]; } fa, fb;
#pragma unroll
        for (int j = 0; j < 32; j++) {
            size_t k = (size_t)kb * BK + 32 * g + j;
            fa.b[j] = m_ok ? A[k * ldm + m_ld] : (uint8_t)0;
            fb.b[j] = n_ok ? B[k * N + n_ld] : (uint8_t)0;
        }
        f32x4 p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fb.v, fa.v, (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
        // lane holds D[n = n0+4g+e][m = m0+L]
        float sa = m_ok ? SA[(size_t)kb * ldm + m_ld] : 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int n = n0 + 4 * g + e;
            float sb = n < N ? SB[(size_t)kb * QN + (n >> 7)] : 0.f;
            acc[e] = __builtin_fmaf(sa * sb, p[e], acc[e]);
        }
    }
    if (m_ok) {
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int n = n0 + 4 * g + e;
            if (n < N) C[(size_t)m_ld * N + n] = (uint16_t)(pack_bf16x2(acc[e], 0.f) & 0xffff);
        }
    }
}

}  // namespace rf
