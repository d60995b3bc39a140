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

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __builtin_bit_cast(float, h << 16); }

// One workgroup (256 threads) per 128 x 128 block: rows r0.. of X (ld = K elements), K block kb.
// PER_ROW: one scale per row (activations). Otherwise one scale for the whole block (weights).
// IN_BF16: X holds bf16 instead of fp32.
// Thread t holds 4 consecutive k (4*(t%32)..) of the 16 rows 32*(i/4) + 4*(t/32) + i%4, i = 0..15: a row is spread
// over the 32 lanes of a half wave, and a thread's rows come in runs of four, which become one 32-bit LDS store.
template <bool PER_ROW, bool IN_BF16>
__global__ __launch_bounds__(256) void quantize_block128(const void *__restrict__ X, int R, int K,
                                                         uint8_t *__restrict__ out, float *__restrict__ scales,
                                                         int scale_ld, bool vector_store) {
    constexpr int PITCH = 128 + 4;                            // LDS row (one k, 128 rows of X), padded against conflicts
    __shared__ __attribute__((aligned(16))) uint8_t tile[128 * PITCH];
    auto row_of = [&](int i) { return 32 * (i >> 2) + 4 * (int)(threadIdx.x >> 5) + (i & 3); };
    __shared__ float wave_max[4];
    const int t = threadIdx.x, lane32 = t & 31;
    // K blocks vary fastest over the grid: workgroups that run together read neighbouring 512-byte (256-byte) pieces
    // of the same source rows
    const int rb = blockIdx.y, r0 = rb * 128, kb = blockIdx.x, k0 = kb * 128;
    float v[16][4];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        const int r = r0 + row_of(i);
        if (r < R) {
            if constexpr (IN_BF16) {
                const uint2 w = *(const uint2 *)((const uint16_t *)X + (size_t)r * K + k0 + 4 * lane32);
                v[i][0] = bf16_bits_to_f32(w.x & 0xffffu); v[i][1] = bf16_bits_to_f32(w.x >> 16);
                v[i][2] = bf16_bits_to_f32(w.y & 0xffffu); v[i][3] = bf16_bits_to_f32(w.y >> 16);
            } else {
                const float4 w = *(const float4 *)((const float *)X + (size_t)r * K + k0 + 4 * lane32);
                v[i][0] = w.x; v[i][1] = w.y; v[i][2] = w.z; v[i][3] = w.w;
            }
        } else {
            v[i][0] = v[i][1] = v[i][2] = v[i][3] = 0.f;
        }
    }
    // amax: NaNs never win a comparison, like a scalar "if (|x| > amax)" loop
    float amax[16];
#pragma unroll
    for (int i = 0; i < 16; i++) {
        float a = 0.f;
#pragma unroll
        for (int e = 0; e < 4; e++) { const float x = __builtin_fabsf(v[i][e]); a = x > a ? x : a; }
#pragma unroll
        for (int off = 16; off >= 1; off >>= 1) { const float o = __shfl_xor(a, off, 64); a = o > a ? o : a; }
        amax[i] = a;                                          // all 32 lanes of the row hold it
    }
    float s[16];
    if constexpr (PER_ROW) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            s[i] = amax[i] > 0.f ? amax[i] / 448.0f : 1.0f;
            const int r = r0 + row_of(i);
            if (lane32 == 0 && r < R) scales[(size_t)kb * scale_ld + r] = s[i];
        }
    } else {
        float a = 0.f;
#pragma unroll
        for (int i = 0; i < 16; i++) a = amax[i] > a ? amax[i] : a;
        { const float o = __shfl_xor(a, 32, 64); a = o > a ? o : a; }
        if ((t & 63) == 0) wave_max[t >> 6] = a;
        __syncthreads();
        a = wave_max[0];
#pragma unroll
        for (int w = 1; w < 4; w++) a = wave_max[w] > a ? wave_max[w] : a;
        const float sb = a > 0.f ? a / 448.0f : 1.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = sb;
        if (t == 0) scales[(size_t)kb * scale_ld + rb] = sb;
    }
    // quantise and transpose through LDS: tile[k][row]. (Replacing the 64 divisions per thread by a multiplication
    // with 1/scale plus an exact fallback near rounding boundaries was tried and is bit-exact, but no faster: the
    // kernel is bound by its memory access pattern, not by the ALU.)
#pragma unroll
    for (int i4 = 0; i4 < 4; i4++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            uint32_t w = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) w |= f32_to_e4m3fn_code(v[4 * i4 + j][e] / s[4 * i4 + j]) << (8 * j);
            *(uint32_t *)(tile + (4 * lane32 + e) * PITCH + row_of(4 * i4)) = w;
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
