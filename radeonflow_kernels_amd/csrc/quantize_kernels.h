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

template <int V> struct IntConst { static constexpr int value = V; };

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

// Maximum over each aligned group of 16 lanes, left in all of them: four DPP steps (swap within pairs, within
// quads, rotate the 16-lane row by 4 and by 8) instead of LDS-crossbar shuffles. x > a ? x : a, so a NaN never wins.
__device__ __forceinline__ float max_over_16_lanes(float a) {
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

// One workgroup (256 threads) per 128 x 128 block: rows r0.. of X (ld = K elements), K block kb.
// PER_ROW: one scale per row (activations). Otherwise one scale for the whole block (weights).
// IN_BF16: X holds bf16 instead of fp32.
// A thread loads 16 bytes at a time: KPT = 4 (fp32) or 8 (bf16) consecutive k of one row, so a row is spread over
// LPR = 32 (16) neighbouring lanes; it holds RPT = 16 (8) rows, in runs of four consecutive rows (a run becomes one
// 32-bit LDS store per k): run g of thread t starts at row g * (128 / NG) + 4 * (t / LPR).
template <bool PER_ROW, bool IN_BF16>
__global__ __launch_bounds__(256) void quantize_block128(const void *__restrict__ X, int R, int K,
                                                         uint8_t *__restrict__ out, float *__restrict__ scales,
                                                         int scale_ld, bool vector_store) {
    constexpr int KPT = IN_BF16 ? 8 : 4, LPR = 128 / KPT, RPT = 64 / KPT, NG = RPT / 4;
    constexpr int PITCH = 128 + 4;                            // LDS row (one k, 128 rows of X), padded against conflicts
    __shared__ __attribute__((aligned(16))) uint8_t tile[128 * PITCH];
    __shared__ float wave_max[4];
    const int t = threadIdx.x, lane_k = t % LPR, rsub = t / LPR;
    auto row_of = [&](int i) { return (i >> 2) * (128 / NG) + 4 * rsub + (i & 3); };
    // K blocks vary fastest over the grid: workgroups that run together read neighbouring pieces of the same rows
    const int rb = blockIdx.y, r0 = rb * 128, kb = blockIdx.x, k0 = kb * 128;
    float v[RPT][KPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        const int r = r0 + row_of(i);
        if (r < R) {
            if constexpr (IN_BF16) {
                const uint4 w = *(const uint4 *)((const uint16_t *)X + (size_t)r * K + k0 + KPT * lane_k);
                const uint32_t q[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    v[i][2 * e] = bf16_bits_to_f32(q[e] & 0xffffu);
                    v[i][2 * e + 1] = bf16_bits_to_f32(q[e] >> 16);
                }
            } else {
                const float4 w = *(const float4 *)((const float *)X + (size_t)r * K + k0 + KPT * lane_k);
                v[i][0] = w.x; v[i][1] = w.y; v[i][2] = w.z; v[i][3] = w.w;
            }
        } else {
#pragma unroll
            for (int e = 0; e < KPT; e++) v[i][e] = 0.f;
        }
    }
    // amax: NaNs never win a comparison, like a scalar "if (|x| > amax)" loop
    float amax[RPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        float a = 0.f;
#pragma unroll
        for (int e = 0; e < KPT; e++) { const float x = __builtin_fabsf(v[i][e]); a = x > a ? x : a; }
        a = max_over_16_lanes(a);
        if constexpr (LPR == 32) { const float o = __shfl_xor(a, 16, 64); a = o > a ? o : a; }
        amax[i] = a;                                          // all LPR lanes of the row hold it
    }
    float s[RPT];
    if constexpr (PER_ROW) {
#pragma unroll
        for (int i = 0; i < RPT; i++) {
            s[i] = amax[i] > 0.f ? amax[i] / 448.0f : 1.0f;
            const int r = r0 + row_of(i);
            if (lane_k == 0 && r < R) scales[(size_t)kb * scale_ld + r] = s[i];
        }
    } else {
        float a = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; i++) a = amax[i] > a ? amax[i] : a;
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1) { const float o = __shfl_xor(a, off, 64); a = o > a ? o : a; }
        if ((t & 63) == 0) wave_max[t >> 6] = a;
        __syncthreads();
        a = wave_max[0];
#pragma unroll
        for (int w = 1; w < 4; w++) a = wave_max[w] > a ? wave_max[w] : a;
        const float sb = a > 0.f ? a / 448.0f : 1.0f;
#pragma unroll
        for (int i = 0; i < RPT; i++) s[i] = sb;
        if (t == 0) scales[(size_t)kb * scale_ld + rb] = sb;
    }
    // quantise and transpose through LDS: tile[k][row]. The value to encode is fl32(x / scale). A correctly rounded
    // division costs ~15 instructions; instead y = x * (1 / scale) is used, which is within 2^-22 (relative) of that
    // quotient. The fp8 conversion is monotonic, so if y * (1 - 2^-21) and y * (1 + 2^-21) convert to the same code,
    // the exact quotient (which lies between them) converts to that code too. Only when the two differ (a rounding
    // boundary is that close: about 1 element in 10^5), or a NaN is involved, or the scale is so far from 1 that its
    // reciprocal is not a normal number, the group of four is redone with the division.
    float rinv[RPT];
    bool fast[RPT];
#pragma unroll
    for (int i = 0; i < RPT; i++) {
        rinv[i] = 1.0f / s[i];
        fast[i] = s[i] > 0x1p-100f && s[i] < 0x1p100f;
    }
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
        for (int e = 0; e < KPT; e++) {
            float y[4];
            bool ok = true;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                y[j] = v[4 * g + j][e] * rinv[4 * g + j];
                ok = ok && fast[4 * g + j] && y[j] == y[j];
            }
            constexpr float UP = 1.0f + 0x1p-21f, DOWN = 1.0f - 0x1p-21f;
            int hi = __builtin_amdgcn_cvt_pk_fp8_f32(y[0] * UP, y[1] * UP, 0, false);
            hi = __builtin_amdgcn_cvt_pk_fp8_f32(y[2] * UP, y[3] * UP, hi, true);
            int lo = __builtin_amdgcn_cvt_pk_fp8_f32(y[0] * DOWN, y[1] * DOWN, 0, false);
            lo = __builtin_amdgcn_cvt_pk_fp8_f32(y[2] * DOWN, y[3] * DOWN, lo, true);
            uint32_t w = (uint32_t)hi;
            if (!ok || hi != lo)
                w = f32x4_to_e4m3fn_codes(v[4 * g][e] / s[4 * g], v[4 * g + 1][e] / s[4 * g + 1],
                                          v[4 * g + 2][e] / s[4 * g + 2], v[4 * g + 3][e] / s[4 * g + 3]);
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
            if (r0 + c < R) *(uint4 *)(out + (size_t)(k0 + k) * R + r0 + c) = w;
        }
    } else {
        for (int idx = t; idx < 128 * 128; idx += 256) {
            const int k = idx >> 7, c = idx & 127;
            if (r0 + c < R) out[(size_t)(k0 + k) * R + r0 + c] = tile[k * PITCH + c];
        }
    }
}

}  // namespace rf
