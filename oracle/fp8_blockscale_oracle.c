/*
 * CPU oracle for the FP8 (OCP e4m3fn) blockwise-scaled GEMM.
 *
 * THIS FILE IS TEST INFRASTRUCTURE. It is the checker the GPU path is compared
 * against; nothing in the shipped library links or calls it. Only tests, the
 * smoke check and the benchmark's cpu_baseline leg may load it.
 *
 * What it restates (paths relative to the reference tree):
 *   - rfo_ref_gemm_*          scripts/problems/gemm/reference.py:40-85  (ref_kernel:
 *                             dequantise A and B with expanded scales, fp32 matmul,
 *                             cast to bf16) and its libtorch twin
 *                             tests/gemm/gemm_test.cpp:106-164.
 *   - operand memory layout   tests/gemm/gemm_test.cpp:82-98 (a is [K][M], b is [K][N],
 *                             a_scale is [QK][M], b_scale is [QK][QN]).
 *   - rfo_ref_gemm_blockfold  src/gemm/gemm_kernel.cpp:138-208 (per-128-K partial sum,
 *                             then acc += (sa*sb)*partial) and :610-632 (cpu_gemm's
 *                             scale indexing sa[k/128][m]*sb[k/128][n/128]).
 *   - rfo_f32_to_bf16_fast    src/gemm/gemm_kernel.cpp:210-218 (fast_f32tob16).
 *   - rfo_allclose            tests/checker/checker.cpp:10-105 (verbose_allclose:
 *                             |got-exp| <= atol + rtol*|exp| plus NaN/+-Inf position match).
 *
 * Pinning (each function has a check that does not retype its formula):
 *   - e4m3fn decode/encode, bf16 rounding: exhaustive / randomised comparison with the
 *     float8_e4m3fn and bfloat16 conversions of the installed PyTorch CPU library.
 *   - rfo_ref_gemm_f32 / _f64: fp64 brute force in numpy on tiny shapes, linearity and
 *     block-removal invariants, index-coded scales, and agreement with the torch-CPU
 *     restatement in oracle/ref_kernel.py.
 *   - rfo_randn: moments and a committed golden prefix (its integer hash is also
 *     restated in numpy and compared bit for bit).
 * Parity unpinned at bit level: the summation order inside torch.matmul (reference.py:84)
 * and inside the reference's MFMA path is not fixed by any reference test; parity is
 * pinned at the reference's own tolerance (rtol 2e-2, atol 1e-3), not bit for bit.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QBLK 128

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa; no Inf; 0x7F/0xFF are NaN ---- */
float rfo_e4m3fn_to_f32(uint8_t v) {
    int s = v >> 7, e = (v >> 3) & 15, m = v & 7;
    float r;
    if (e == 15 && m == 7) r = NAN;
    else if (e == 0) r = ldexpf((float)m, -9);             /* subnormal: m/8 * 2^-6 */
    else r = ldexpf((float)(8 + m), e - 10);               /* (1+m/8) * 2^(e-7) */
    return s ? -r : r;
}

/* Round-to-nearest-even fp32 -> e4m3fn. Magnitudes that round above 448 become NaN
 * (no saturation), which is what PyTorch's float8_e4m3fn cast does. */
uint8_t rfo_f32_to_e4m3fn(float f) {
    uint32_t u = f2u(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80);
    float a = fabsf(f);
    if (!(a == a)) return (uint8_t)(sign | 0x7F);
    if (a == 0.0f) return sign;
    /* quantum: 2^-9 below 2^-6, else 2^(floor(log2 a) - 3) */
    int ex;
    (void)frexpf(a, &ex);            /* a = fr * 2^ex, fr in [0.5,1) -> floor(log2 a) = ex-1 */
    int q = (ex - 1) - 3;
    if (q < -9) q = -9;
    float scaled = ldexpf(a, -q);    /* exact: power-of-two scaling */
    float r = nearbyintf(scaled);    /* default rounding mode: nearest even */
    float val = ldexpf(r, q);
    if (val > 448.0f) return (uint8_t)(sign | 0x7F);
    if (val == 0.0f) return sign;
    /* encode val (exactly representable now) */
    int e2;
    float fr = frexpf(val, &e2);     /* val = fr*2^e2, fr in [0.5,1) */
    int E = e2 - 1 + 7;
    uint8_t code;
    if (E <= 0) {
        code = (uint8_t)lrintf(ldexpf(val, 9));            /* subnormal mantissa (may be 8 -> 0x08 = min normal) */
    } else {
        int m = (int)lrintf(ldexpf(fr, 4)) - 8;            /* fr*16 in [8,16) */
        code = (uint8_t)((E << 3) | m);
    }
    return (uint8_t)(sign | code);
}

/* ---- bf16 ---- */
uint16_t rfo_f32_to_bf16(float f) {
    uint32_t u = f2u(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040); /* quiet NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
/* the reference's integer-add rounding, no NaN special case */
uint16_t rfo_f32_to_bf16_fast(float f) {
    uint32_t u = f2u(f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float rfo_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

void rfo_e4m3fn_to_f32_array(const uint8_t *in, float *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = rfo_e4m3fn_to_f32(in[i]); }
void rfo_f32_to_e4m3fn_array(const float *in, uint8_t *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = rfo_f32_to_e4m3fn(in[i]); }
void rfo_f32_to_bf16_array(const float *in, uint16_t *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = rfo_f32_to_bf16(in[i]); }
void rfo_f32_to_bf16_fast_array(const float *in, uint16_t *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = rfo_f32_to_bf16_fast(in[i]); }
void rfo_bf16_to_f32_array(const uint16_t *in, float *out, size_t n) { for (size_t i = 0; i < n; i++) out[i] = rfo_bf16_to_f32(in[i]); }

/* ---- counter-based N(0,1): element i of stream `seed` depends only on (seed, i) ---- */
uint64_t rfo_hash64(uint64_t seed, uint64_t i) {
    uint64_t z = seed * 0x9E3779B97F4A7C15ull + i * 0xD1B54A32D192ED03ull + 0x2545F4914F6CDD1Dull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
void rfo_randn(uint64_t seed, uint64_t offset, size_t n, float *out) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) {
        uint64_t h = rfo_hash64(seed, offset + i);
        /* two 24-bit uniforms; u1 in (0,1], u2 in [0,1) */
        double u1 = ((double)((h >> 40) & 0xFFFFFF) + 1.0) / 16777216.0;
        double u2 = (double)((h >> 8) & 0xFFFFFF) / 16777216.0;
        out[i] = (float)(sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2));
    }
}

/* ---- quantisers of the benchmark's synthetic inputs ----
 * A32 is [M][K] row-major. a_scale[m,kb] = amax(A32[m, kb*128:(kb+1)*128]) / 448 (1 when the block is all zero);
 * A8 = e4m3fn_rne(A32 / a_scale). Outputs in the launcher's layouts: a_km[k*M+m], as_qm[kb*M+m]. */
void rfo_quantize_a(const float *A32, int M, int K, uint8_t *a_km, float *as_qm) {
    int QK = K / QBLK;
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        for (int kb = 0; kb < QK; kb++) {
            const float *p = A32 + (size_t)m * K + (size_t)kb * QBLK;
            float amax = 0.f;
            for (int j = 0; j < QBLK; j++) { float a = fabsf(p[j]); if (a > amax) amax = a; }
            float s = amax > 0.f ? amax / 448.0f : 1.0f;
            as_qm[(size_t)kb * M + m] = s;
            for (int j = 0; j < QBLK; j++) a_km[(size_t)(kb * QBLK + j) * M + m] = rfo_f32_to_e4m3fn(p[j] / s);
        }
    }
}
/* B32 is [N][K] row-major; one scale per 128x128 block (last N block may be partial).
 * Outputs: b_kn[k*N+n], bs_qq[kb*QN+nb]. */
void rfo_quantize_b(const float *B32, int N, int K, uint8_t *b_kn, float *bs_qq) {
    int QK = K / QBLK, QN = (N + QBLK - 1) / QBLK;
#pragma omp parallel for schedule(static) collapse(2)
    for (int nb = 0; nb < QN; nb++) {
        for (int kb = 0; kb < QK; kb++) {
            int n1 = (nb + 1) * QBLK < N ? (nb + 1) * QBLK : N;
            float amax = 0.f;
            for (int n = nb * QBLK; n < n1; n++)
                for (int j = 0; j < QBLK; j++) { float a = fabsf(B32[(size_t)n * K + kb * QBLK + j]); if (a > amax) amax = a; }
            float s = amax > 0.f ? amax / 448.0f : 1.0f;
            bs_qq[(size_t)kb * QN + nb] = s;
            for (int n = nb * QBLK; n < n1; n++)
                for (int j = 0; j < QBLK; j++)
                    b_kn[(size_t)(kb * QBLK + j) * N + n] = rfo_f32_to_e4m3fn(B32[(size_t)n * K + kb * QBLK + j] / s);
        }
    }
}

/* ---- the oracle GEMM: dequantise every element, multiply, accumulate over the full K ----
 * rows == NULL -> all M rows, else only the listed rows (output is [nrows][N]).
 * acc in fp32, k ascending (reference.py:68,81,84). */
static void ref_rows_f32(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                         int M, int N, int K, const int *rows, int nrows, float *out) {
    int QN = (N + QBLK - 1) / QBLK;
    float lut[256];
    for (int i = 0; i < 256; i++) lut[i] = rfo_e4m3fn_to_f32((uint8_t)i);
#pragma omp parallel
    {
        float *arow = (float *)malloc(sizeof(float) * (size_t)K);
        float *brow = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(dynamic, 1)
        for (int r = 0; r < nrows; r++) {
            int m = rows ? rows[r] : r;
            for (int k = 0; k < K; k++) arow[k] = lut[a[(size_t)k * M + m]] * as[(size_t)(k / QBLK) * M + m];
            for (int n = 0; n < N; n++) {
                for (int k = 0; k < K; k++) brow[k] = lut[b[(size_t)k * N + n]] * bs[(size_t)(k / QBLK) * QN + n / QBLK];
                float acc = 0.f;
                for (int k = 0; k < K; k++) acc += arow[k] * brow[k];
                out[(size_t)r * N + n] = acc;
            }
        }
        free(arow); free(brow);
    }
}
void rfo_ref_gemm_f32(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                      int M, int N, int K, const int *rows, int nrows, float *out_f32, uint16_t *out_bf16) {
    if (!rows) nrows = M;
    float *tmp = out_f32 ? out_f32 : (float *)malloc(sizeof(float) * (size_t)nrows * N);
    ref_rows_f32(a, b, as, bs, M, N, K, rows, nrows, tmp);
    if (out_bf16) for (size_t i = 0; i < (size_t)nrows * N; i++) out_bf16[i] = rfo_f32_to_bf16(tmp[i]);
    if (!out_f32) free(tmp);
}
/* fp64 "truth": exact products, fp64 accumulation, no intermediate rounding of the dequantised values */
void rfo_ref_gemm_f64(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                      int M, int N, int K, const int *rows, int nrows, double *out) {
    int QN = (N + QBLK - 1) / QBLK, QK = K / QBLK;
    if (!rows) nrows = M;
    float lut[256];
    for (int i = 0; i < 256; i++) lut[i] = rfo_e4m3fn_to_f32((uint8_t)i);
#pragma omp parallel
    {
        float *bcol = (float *)malloc(sizeof(float) * (size_t)K);
#pragma omp for schedule(dynamic, 1)
        for (int n = 0; n < N; n++) {
            for (int k = 0; k < K; k++) bcol[k] = lut[b[(size_t)k * N + n]];
            for (int r = 0; r < nrows; r++) {
                int m = rows ? rows[r] : r;
                double acc = 0.0;
                for (int kb = 0; kb < QK; kb++) {
                    double p = 0.0;
                    for (int j = 0; j < QBLK; j++) { int k = kb * QBLK + j; p += (double)lut[a[(size_t)k * M + m]] * (double)bcol[k]; }
                    acc += p * (double)as[(size_t)kb * M + m] * (double)bs[(size_t)kb * QN + n / QBLK];
                }
                out[(size_t)r * N + n] = acc;
            }
        }
        free(bcol);
    }
}
/* the reference device kernel's own order: exact fp32 partial per 128-K block, s = sa*sb (fp32),
 * acc = fma(s, partial, acc); bf16 at the end */
void rfo_ref_gemm_blockfold(const uint8_t *a, const uint8_t *b, const float *as, const float *bs,
                            int M, int N, int K, const int *rows, int nrows, float *out_f32, uint16_t *out_bf16) {
    int QN = (N + QBLK - 1) / QBLK, QK = K / QBLK;
    if (!rows) nrows = M;
    float lut[256];
    for (int i = 0; i < 256; i++) lut[i] = rfo_e4m3fn_to_f32((uint8_t)i);
#pragma omp parallel for schedule(dynamic, 1)
    for (int n = 0; n < N; n++) {
        for (int r = 0; r < nrows; r++) {
            int m = rows ? rows[r] : r;
            float acc = 0.f;
            for (int kb = 0; kb < QK; kb++) {
                float p = 0.f;
                for (int j = 0; j < QBLK; j++) { int k = kb * QBLK + j; p += lut[a[(size_t)k * M + m]] * lut[b[(size_t)k * N + n]]; }
                float s = as[(size_t)kb * M + m] * bs[(size_t)kb * QN + n / QBLK];
                acc = fmaf(s, p, acc);
            }
            if (out_f32) out_f32[(size_t)r * N + n] = acc;
            if (out_bf16) out_bf16[(size_t)r * N + n] = rfo_f32_to_bf16(acc);
        }
    }
}

/* ---- allclose in the reference checker's form; returns the number of mismatches ---- */
long rfo_allclose(const uint16_t *got_bf16, const uint16_t *exp_bf16, size_t n, float rtol, float atol,
                  float *max_abs_err, long *first_bad) {
    long bad = 0; float mx = 0.f; long first = -1;
    for (size_t i = 0; i < n; i++) {
        float g = rfo_bf16_to_f32(got_bf16[i]), e = rfo_bf16_to_f32(exp_bf16[i]);
        int mism;
        if (isnan(g) || isnan(e)) mism = (isnan(g) != isnan(e));
        else if (isinf(g) || isinf(e)) mism = !(g == e);
        else { float d = fabsf(g - e); if (d > mx) mx = d; mism = d > atol + rtol * fabsf(e); }
        if (mism) { if (first < 0) first = (long)i; bad++; }
    }
    if (max_abs_err) *max_abs_err = mx;
    if (first_bad) *first_bad = first;
    return bad;
}
