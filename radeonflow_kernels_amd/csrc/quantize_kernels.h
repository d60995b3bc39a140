// Block quantisers that produce the GEMM's operands on the GPU, in the launcher's layouts.
//
// The reference has no quantiser: its harness draws fp8 bytes and scales directly
// (tests/gemm/gemm_test.cpp:64-99), and the recipe that real callers use is only stated in words: per
// (row, 128-wide K block) for activations and per 128x128 block for weights, scale = amax / 448, value =
// e4m3fn(x / scale) with round-to-nearest-even. These kernels implement exactly that recipe and write
//   a[k*M + m]  (fp8, the [K][M] layout of the launcher),  as[kb*M + m]
//   b[k*N + n]  (fp8, [K][N]),                             bs[kb*QN + nb]
// so the step before the GEMM needs no host work and no transpose pass: the transposition happens in LDS on the
// way out. Both are pure streaming kernels (4 or 2 bytes read, 1 byte written per element): HBM-bound.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rf {

typedef unsigned quant_u32x4 __attribute__((ext_vector_type(4)));
// 16 bytes of output, written through to memory (sc1) instead of left dirty in the XCD's L2: the GEMM that reads them
// runs on all XCDs, so they have to leave this L2 anyway, and written through they do so while the kernel still runs
// (6144 x 7168 from bf16: 26.2-27.0 -> 25.1-25.2 us, from fp32 36.0 -> 35.7 us).
// (The statement carries its own wait states: a store of more than 8 bytes reads its data registers a little after it
// has been issued, and the compiler's hazard check does not look inside it.)
__device__ __forceinline__ void store16_through(void *p, const uint4 &v) {
    const quant_u32x4 w = {v.x, v.y, v.z, v.w};
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" :: "v"(p), "v"(w) : "memory");
}

template <int V> struct IntConst { static constexpr int value = V; };
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

// fp32 -> OCP e4m3fn code, round to nearest even, anything that rounds above 448 (and NaN) becomes NaN (0x7F).
// Integer/exact-float arithmetic only, so that it agrees bit for bit with a CPU implementation; no branches.
__device__ __forceinline__ uint32_t f32_to_e4m3fn_code(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    const uint32_t sign = (u >> 24) & 0x80u, abits = u & 0x7fffffffu;
    const int e = (int)(abits >> 23) - 127;                   // floor(log2 |f|) for normal inputs
    int q = e - 3;                                            // exponent of the rounding quantum: 3 mantissa bits
    q = q < -9 ? -9 : q;                                      // subnormal range of e4m3: quantum 2^-9
    q = q > 120 ? 120 : q;                                    // Inf / NaN: keep the factor below finite
    const float inv_quantum = __builtin_bit_cast(float, (uint32_t)(127 - q) << 23);
    const float r = __builtin_rintf(__builtin_bit_cast(float, abits) * inv_quantum);   // exact product, RNE to integer
    // r is in [0,16] for finite inputs; code = exponent field (q+10) and mantissa r-8, which also covers the subnormal
    // codes (q = -9) and the carry r == 16 into the next exponent
    const bool finite = abits < 0x7f800000u;
    const int code = ((q + 10) << 3) + (int)(finite ? r : 0.f) - 8;
    return sign | (uint32_t)((code > 126 || !finite) ? 0x7F : code);
}

// Four fp32 values -> four e4m3fn codes packed in one word (value j in byte j), same results as f32_to_e4m3fn_code.
// Uses the conversion instruction of gfx950 (v_cvt_pk_fp8_f32: OCP e4m3fn, round to nearest even, values that round
// above 448 and infinities become NaN). Compared over all 2^32 inputs it differs from the integer encoder only for
// NaNs with a clear sign bit (it returns 0xFF, the encoder keeps the sign: 0x7F), so a group that contains a NaN goes
// through the integer encoder.
__device__ __forceinline__ uint32_t f32x4_to_e4m3fn_codes(float x0, float x1, float x2, float x3) {
    int w = __builtin_amdgcn_cvt_pk_fp8_f32(x0, x1, 0, false);
    w = __builtin_amdgcn_cvt_pk_fp8_f32(x2, x3, w, true);
    if (x0 != x0 || x1 != x1 || x2 != x2 || x3 != x3)
        w = (int)(f32_to_e4m3fn_code(x0) | (f32_to_e4m3fn_code(x1) << 8) | (f32_to_e4m3fn_code(x2) << 16) |
                  (f32_to_e4m3fn_code(x3) << 24));
    return (uint32_t)w;
}

// Plain elementwise cast fp32 -> e4m3fn (no scaling), four values per thread.
__global__ __launch_bounds__(256) void cast_f32_to_e4m3fn(const float *__restrict__ x, uint8_t *__restrict__ out, size_t n) {
    const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i + 4 <= n) {
        const float4 v = *(const float4 *)(x + i);
        *(uint32_t *)(out + i) = f32x4_to_e4m3fn_codes(v.x, v.y, v.z, v.w);
    } else {
        for (size_t j = i; j < n; j++) out[j] = (uint8_t)f32_to_e4m3fn_code(x[j]);
    }
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

// Maximum over each aligned group of 16 lanes, left in all of them, for N unsigned values at once: four DPP steps
// (swap within pairs, within quads, rotate the 16-lane row by 4 and by 8) instead of LDS-crossbar shuffles, each one
// v_max_u32 with a DPP operand. Written as asm because the compiler emits move + max for the builtin form. A DPP
// operand must not be read within two instructions of the VALU write that produced it, and the compiler's hazard
// recogniser does not look inside asm statements (it may also place a register copy right in front of one): every
// step carries its own two wait states.
template <int N>
__device__ __forceinline__ void max_over_16_lanes(uint32_t (&a)[N]) {
#pragma unroll
    for (int i = 0; i < N; i++)
        asm volatile("s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(a[i]));
#pragma unroll
    for (int i = 0; i < N; i++)
        asm volatile("s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "+v"(a[i]));
#pragma unroll
    for (int i = 0; i < N; i++)
        asm volatile("s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf" : "+v"(a[i]));
#pragma unroll
    for (int i = 0; i < N; i++)
        asm volatile("s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf" : "+v"(a[i]));
    asm volatile("s_nop 1" ::: "memory");     // the compiler may follow up with a DPP or lane-crossing read of a[N-1]
}

// The same for one float with "a NaN never wins" comparisons (the rare path of rows that contain a NaN).
__device__ __forceinline__ float max_over_16_lanes_nan_safe(float a) {
    auto step = [&](auto ctrl) {
        const float o = __builtin_bit_cast(
            float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, a), decltype(ctrl)::value, 0xf, 0xf, false));
        a = o > a ? o : a;
    };
    step(IntConst<0xB1>{});      // quad_perm [1,0,3,2]
    step(IntConst<0x4E>{});      // quad_perm [2,3,0,1]
    step(IntConst<0x124>{});     // row_ror 4
    step(IntConst<0x128>{});     // row_ror 8
    return a;
}

// a / 448 for a in [2^-100, FLT_MAX]: product with RN(1/448) plus one correction step through the exact remainder.
// Compared with the IEEE division over every float in that range on the CPU: identical (below 2^-100 the remainder
// underflows and it is not).
__device__ __forceinline__ float div_by_448(float a) {
    constexpr float C = 1.0f / 448.0f;
    const float q = a * C;
    const float r = __builtin_fmaf(-q, 448.0f, a);
    return __builtin_fmaf(r, C, q);
}

// One workgroup (256 threads) per 128 x 128 block: rows r0.. of X (ld = K elements), K block kb.
// PER_ROW: one scale per row (activations). Otherwise one scale for the whole block (weights).
// IN_BF16: X holds bf16 instead of fp32.
// A thread loads 16 bytes at a time: KPT = 4 (fp32) or 8 (bf16) consecutive k of one row, so a row is spread over
// LPR = 32 (16) neighbouring lanes; it holds RPT = 16 (8) rows, in runs of four consecutive rows (a run becomes one
// 32-bit LDS store per k): run g of thread t starts at row g * (128 / NG) + 4 * (t / LPR).
//
// GROUPED (activations of several groups, for the grouped GEMM): the R rows written are the rows of a padded layout in
// which group g starts at row pad_start[g], a multiple of 16, and holds src_start[g+1] - src_start[g] rows of X (from
// row src_start[g]) followed by rows of zeros with scale 1 up to the next group's start. Group starts are multiples
// of 16 and a thread's rows come in runs of four from a multiple of four, so a run lies in one group.
constexpr int kQuantMaxGroups = 256;
struct QuantGroups {
    int pad_start[kQuantMaxGroups + 1];     // first row of each group in the padded layout; [groups] = R
    int src_start[kQuantMaxGroups + 1];     // first row of each group in X; [groups] = rows of X
    int groups;
    // the group that holds the first row of each 128-row block of the padded layout, for the first kQuantBlockTable
    // blocks (later blocks search the table): a search is eight dependent scalar loads, about as long as a block's work
    unsigned short block_group[512];
};
constexpr int kQuantBlockTable = 512;
template <bool PER_ROW, bool IN_BF16, bool GROUPED>
__device__ __forceinline__ void quantize_block128_body(const void *__restrict__ X, int R, int K,
                                                       uint8_t *__restrict__ out, float *__restrict__ scales,
                                                       int scale_ld, bool vector_store, const QuantGroups &tab) {
    constexpr int KPT = IN_BF16 ? 8 : 4, LPR = 128 / KPT, RPT = 64 / KPT, NG = RPT / 4;
    constexpr int PITCH = 128 + 4;                            // LDS row (one k, 128 rows of X), padded against conflicts
    __shared__ __attribute__((aligned(16))) uint8_t tile[128 * PITCH];
    __shared__ float wave_max[4];
    const int t = threadIdx.x, lane_k = t % LPR, rsub = t / LPR;
    auto row_of = [&](int i) { return (i >> 2) * (128 / NG) + 4 * rsub + (i & 3); };
    // K blocks vary fastest over the grid: workgroups that run together read neighbouring pieces of the same rows
    const int rb = blockIdx.y, r0 = rb * 128, kb = blockIdx.x, k0 = kb * 128;
    // All loads are issued before the first one is used: rows past R read row R-1 again (their results are never
    // stored, and they are kept out of a block-wide maximum below) instead of sitting behind a branch each.
    // GROUPED: source row of each run of four rows and the first padded row past its group's true rows. The groups
    // that reach into this block are found with table reads that are the same for all lanes (the block starts in
    // group g0; at most 8 more groups of at least 16 padded rows follow inside it).
    int run_shift[NG], run_limit[NG];
    if constexpr (GROUPED) {
        int lo = 0, hi = tab.groups;                          // last g with pad_start[g] <= r0 (uniform)
        if (rb < kQuantBlockTable) {
            lo = tab.block_group[rb];
        } else {
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (tab.pad_start[mid] <= r0) lo = mid; else hi = mid;
            }
        }
#pragma unroll
        for (int u = 0; u < NG; u++) { run_shift[u] = 0; run_limit[u] = 0; }
        for (int g = lo; g < tab.groups && tab.pad_start[g] < r0 + 128; g++) {
            const int ps = tab.pad_start[g], ss = tab.src_start[g], rows = tab.src_start[g + 1] - ss;
#pragma unroll
            for (int u = 0; u < NG; u++)
                if (r0 + row_of(4 * u) >= ps) { run_shift[u] = ss - ps; run_limit[u] = ps + rows; }
        }
    }
    const int src_rows = GROUPED ? tab.src_start[tab.groups] : R;
    uint4 raw[RPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        const int r = r0 + row_of(i);
        int rc = r < R ? r : R - 1;
        if constexpr (GROUPED) {
            rc = r + run_shift[i >> 2];
            rc = rc < src_rows ? rc : src_rows - 1;
            rc = rc > 0 ? rc : 0;
        }
        const size_t off = (size_t)rc * K + k0 + KPT * lane_k;
        raw[i] = IN_BF16 ? *(const uint4 *)((const uint16_t *)X + off) : *(const uint4 *)((const float *)X + off);
        if constexpr (GROUPED) {
            if (r >= run_limit[i >> 2]) raw[i] = make_uint4(0u, 0u, 0u, 0u);      // padding row: zeros, scale 1
        }
    }
    float v[RPT][KPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        const uint32_t q[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if constexpr (IN_BF16) {
                v[i][2 * e] = bf16_bits_to_f32(q[e] & 0xffffu);
                v[i][2 * e + 1] = bf16_bits_to_f32(q[e] >> 16);
            } else {
                v[i][e] = __builtin_bit_cast(float, q[e]);
            }
        }
    }
    // amax: NaNs never win a comparison, like a scalar "if (|x| > amax)" loop. For everything but NaNs the order of
    // |x| is the order of its bit pattern as an unsigned integer, and NaN patterns lie above infinity: the maximum is
    // taken on the raw bits (two bf16 per instruction), and a row whose maximum lands above infinity contains a NaN
    // and takes the comparison loop instead.
    uint32_t amax_bits[RPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        const uint32_t q[4] = {raw[i].x, raw[i].y, raw[i].z, raw[i].w};
        if constexpr (IN_BF16) {
            u16x2 m = {0, 0};
#pragma unroll
            for (int e = 0; e < 4; e++) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, q[e] & 0x7fff7fffu));
            amax_bits[i] = (uint32_t)(m[0] > m[1] ? m[0] : m[1]) << 16;
        } else {
            uint32_t m = 0;
#pragma unroll
            for (int e = 0; e < 4; e++) { const uint32_t x = q[e] & 0x7fffffffu; m = x > m ? x : m; }
            amax_bits[i] = m;
        }
    }
    max_over_16_lanes(amax_bits);                             // all 16 lanes of a row group hold it
    float amax[RPT];
    bool has_nan[RPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        if constexpr (LPR == 32) { const uint32_t o = __shfl_xor(amax_bits[i], 16, 64); amax_bits[i] = o > amax_bits[i] ? o : amax_bits[i]; }
        amax[i] = __builtin_bit_cast(float, amax_bits[i]);
        has_nan[i] = amax_bits[i] > 0x7f800000u;              // the same in all lanes of the row
        if (__builtin_expect(has_nan[i], 0)) {
            float a = 0.f;
#pragma unroll
            for (int e = 0; e < KPT; e++) { const float x = __builtin_fabsf(v[i][e]); a = x > a ? x : a; }
            a = max_over_16_lanes_nan_safe(a);
            if constexpr (LPR == 32) { const float o = __shfl_xor(a, 16, 64); a = o > a ? o : a; }
            amax[i] = a;
        }
    }
    // scale = amax / 448, exactly as the IEEE division gives it
    auto scale_of = [](float a) {
        float sc = a > 0.f ? div_by_448(a) : 1.0f;
        if (__builtin_expect(a > 0.f && !(a >= 0x1p-100f && a <= 0x1.fffffep127f), 0)) sc = a / 448.0f;
        return sc;
    };
    float s[RPT];
    if constexpr (PER_ROW) {
#pragma unroll
        for (int i = 0; i < RPT; i++) {
            s[i] = scale_of(amax[i]);
            const int r = r0 + row_of(i);
            if (lane_k == 0 && r < R) scales[(size_t)kb * scale_ld + r] = s[i];
        }
    } else {
        float a = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; i++) a = (amax[i] > a && r0 + row_of(i) < R) ? amax[i] : a;
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1) { const float o = __shfl_xor(a, off, 64); a = o > a ? o : a; }
        if ((t & 63) == 0) wave_max[t >> 6] = a;
        __syncthreads();
        a = wave_max[0];
#pragma unroll
        for (int w = 1; w < 4; w++) a = wave_max[w] > a ? wave_max[w] : a;
        const float sb = scale_of(a);
#pragma unroll
        for (int i = 0; i < RPT; i++) s[i] = sb;
        if (t == 0) scales[(size_t)kb * scale_ld + rb] = sb;
    }
    // quantise and transpose through LDS: tile[k][row]. The value to encode is fl32(x / scale). A correctly rounded
    // division costs ~11 instructions per element. Instead, with r = rcp(scale) (the hardware reciprocal, within a few
    // ulp of 1 / scale), x * (r * (1 + 2^-20)) and x * (r * (1 - 2^-20)) are, in magnitude, above and below the exact
    // quotient and its fp32 rounding (the factors' rounding errors and the reciprocal's error are below 2^-21
    // together). The fp8 conversion is monotonic, so if the two products convert to the same code, fl32(x / scale)
    // converts to that code too. When they differ (a rounding boundary is that close: about 1 element in 10^5 for
    // fp32 sources, far more often for bf16 ones) the group of four is redone with the exact quotient; when a row
    // contains a NaN or an infinity, or its scale lies outside (2^-60, 2^60), with the IEEE division and the
    // NaN-aware encoder.
    float rup[RPT], rdown[RPT];
    bool fast[RPT / 4];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        const float rinv = __builtin_amdgcn_rcpf(s[i]);
        rup[i] = rinv * (1.0f + 0x1p-20f);
        rdown[i] = rinv * (1.0f - 0x1p-20f);
    }
#pragma unroll
    for (int g = 0; g < NG; g++) {
        fast[g] = true;
#pragma unroll
        for (int j = 0; j < 4; j++)
            fast[g] = fast[g] && s[4 * g + j] > 0x1p-60f && s[4 * g + j] < 0x1p60f && !has_nan[4 * g + j];
    }
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
        for (int e = 0; e < KPT; e++) {
            // bf16 sources go straight to the exact quotient: x and amax have 8-bit mantissas, so x / scale often IS
            // a rounding boundary, one such lane in 64 sends the whole wave to the exact path, and with 256 values per
            // wave and group that is nearly every time; the bracket would only be computed on top of it.
            int hi = 0, lo = 1;
            if constexpr (!IN_BF16) {
                float yu[4], yd[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    yu[j] = v[4 * g + j][e] * rup[4 * g + j];
                    yd[j] = v[4 * g + j][e] * rdown[4 * g + j];
                }
                // (the first conversion of a word keeps the upper half of its old value, which the second one
                // overwrites: any register will do as the old value)
                hi = __builtin_amdgcn_cvt_pk_fp8_f32(yu[0], yu[1], __builtin_bit_cast(int, yu[0]), false);
                hi = __builtin_amdgcn_cvt_pk_fp8_f32(yu[2], yu[3], hi, true);
                lo = __builtin_amdgcn_cvt_pk_fp8_f32(yd[0], yd[1], __builtin_bit_cast(int, yd[0]), false);
                lo = __builtin_amdgcn_cvt_pk_fp8_f32(yd[2], yd[3], lo, true);
            }
            uint32_t w = (uint32_t)hi;
            if (__builtin_expect(!fast[g], 0)) {
                w = f32x4_to_e4m3fn_codes(v[4 * g][e] / s[4 * g], v[4 * g + 1][e] / s[4 * g + 1],
                                          v[4 * g + 2][e] / s[4 * g + 2], v[4 * g + 3][e] / s[4 * g + 3]);
            } else if (__builtin_expect(hi != lo, 0)) {
                // A rounding boundary lies inside the bracket. With bf16 sources that is common, not rare: x and amax
                // have 8-bit mantissas, so x / scale often IS a boundary (a tie) and one lane in 64 is enough to send
                // the wave here. The exact quotient decides: the refinement steps of the f32 division expansion
                // without its range scaling, which the limits on the scale make unnecessary (identical to the IEEE
                // quotient on 2.9e9 CPU cases, ties of bf16-like operands and reciprocals off by an ulp included).
                float q[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const float x = v[4 * g + j][e], d = s[4 * g + j];
                    float r = __builtin_amdgcn_rcpf(d);
                    r = __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
                    float t = x * r;
                    t = __builtin_fmaf(__builtin_fmaf(-d, t, x), r, t);
                    q[j] = __builtin_copysignf(__builtin_fmaf(__builtin_fmaf(-d, t, x), r, t), x);   // -0 / d stays -0
                }
                int c = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], __builtin_bit_cast(int, q[0]), false);
                w = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], c, true);
            }
            *(uint32_t *)(tile + (KPT * lane_k + e) * PITCH + row_of(4 * g)) = w;
        }
    __syncthreads();
    // out[(k0 + k) * R + r0 + ..]: 128 bytes per k. 8 threads x 16 bytes per k row when the rows allow it.
    if (vector_store) {
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const int k = p * 32 + (t >> 3), c = (t & 7) * 16;
            const uint32_t *src = (const uint32_t *)(tile + k * PITCH + c);
            const uint4 w = {src[0], src[1], src[2], src[3]};
            if (r0 + c < R) {
                // whole 128-byte lines (R a multiple of 128) are written through; pieces of lines are left to L2 to
                // merge (written through, the grouped layout's rows, which start at multiples of 16, took 8 % longer)
                if (!GROUPED && R % 128 == 0) store16_through(out + (size_t)(k0 + k) * R + r0 + c, w);
                else *(uint4 *)(out + (size_t)(k0 + k) * R + r0 + c) = w;
            }
        }
    } else {
        for (int idx = t; idx < 128 * 128; idx += 256) {
            const int k = idx >> 7, c = idx & 127;
            if (r0 + c < R) out[(size_t)(k0 + k) * R + r0 + c] = tile[k * PITCH + c];
        }
    }
}

template <bool PER_ROW, bool IN_BF16>
__global__ __launch_bounds__(256) void quantize_block128(const void *__restrict__ X, int R, int K,
                                                         uint8_t *__restrict__ out, float *__restrict__ scales,
                                                         int scale_ld, bool vector_store) {
    QuantGroups none;                                         // not read
    quantize_block128_body<PER_ROW, IN_BF16, false>(X, R, K, out, scales, scale_ld, vector_store, none);
}
template <bool IN_BF16>
__global__ __launch_bounds__(256) void quantize_block128_grouped(const void *__restrict__ X, int R, int K,
                                                                 uint8_t *__restrict__ out, float *__restrict__ scales,
                                                                 const QuantGroups tab) {
    quantize_block128_body<true, IN_BF16, true>(X, R, K, out, scales, R, true, tab);
}

}  // namespace rf
