// Measures what the whole gfx950 chip sustains on the fp8 MFMA the GEMM is built on when nothing else runs, and what
// the other register-level work of the GEMM's inner loop takes away from it:
//   mfma        8 waves per compute unit issue v_mfma_f32_16x16x128_f8f6f4 back to back from registers (32 per loop
//               iteration over 4 x 2 operand fragments, accumulating in the matrix unit; no memory, no LDS);
//   +folds      every MFMA starts from zero and its result is folded into one of 32 accumulator tiles with four
//               fp32 FMAs three slots later, as the block-scaled GEMM must (scale * partial + acc);
//   +lds_reads  in addition the operand fragments are re-read from LDS with ds_read_b64_tr_b8 at the GEMM's rate
//               (28 + 16 transpose reads per 32 MFMAs, conflict-free layout), still without any global memory traffic;
//   +b128_reads the same fragments read from a K-contiguous LDS layout instead (a row = one m or n, 128 bytes of K, 16-byte
//               chunks XOR-swizzled by row): two ds_read_b128 per fragment, half as many LDS instructions for the same
//               bytes. Prices operands that arrive K-contiguous (prepacked weights, a quantiser that writes them so).
// The published peak (5.0 PFLOP/s dense) assumes 2.4 GHz; under load the chip lowers its clock to stay inside its
// power limit, and how far depends on how many bits toggle in the operands and on what else the loop executes.
// The "+lds_reads" figure for realistic operands is the ceiling a block-scaled fp8 GEMM with fp32 folds on the vector
// unit can approach on this chip before it has loaded a single byte from memory.
//
//   mfma_ceiling [seconds per mode] [compute units]     prints one JSON line:
//   {"zeros": T, "normal": T, "random_bits": T, "normal_with_folds": T, "normal_with_folds_and_lds_reads": T,
//    "normal_with_folds_and_b128_reads": T, "zeros_with_folds_and_lds_reads": T, "unit": "TFLOP/s", "cus": n,
//    "implied_clock_ghz": {...}}
// zeros: all operand bytes 0. normal: e4m3fn codes of N(0,1) samples scaled so that 4.5 sigma maps to 448 (what a
// blockwise quantiser produces). random_bits: uniformly random finite e4m3fn codes. With fewer compute units than the
// chip has (second argument) the power limit is out of the picture and the figures show the cost in cycles alone.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
#define RF_LDS __attribute__((address_space(3)))

constexpr int kWords = 4096, kSlots = 32, kLdsBytes = 32768;

// MODE 0: acc = mfma(a, b, acc). MODE 1: p = mfma(a, b, 0); acc[t] = fma(s, p three slots ago, acc[t]).
// MODE 2: MODE 1 + the fragments re-read from LDS (a 128-row K block of 256-byte rows, 16-byte chunks XOR-swizzled by
// row like the GEMM's stages, so that the transpose reads are free of bank conflicts).
// MODE 3: MODE 1 + the fragments re-read with ds_read_b128 from a K-contiguous layout (256 rows of 128 bytes; lane (L, g)
// takes bytes 32 g .. 32 g + 31 of row L of the fragment's 16 rows; chunk index XORed with (row >> 1) & 7, so that the
// 16 lanes the LDS serves together touch 16 different 16-byte bank groups).
template <int MODE>
__global__ __launch_bounds__(512) void inner_loop(const int *__restrict__ src, float *out, int iters, float sc) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    for (int i = threadIdx.x; i < kLdsBytes / 4; i += 512) ((int *)lds)[i] = src[i % kWords];
    __syncthreads();
    // 2 + 4 operand fragments, as a wave of the GEMM holds them: consecutive MFMAs see different operand bits
    i32x8 a[2], b[4];
#pragma unroll
    for (int f = 0; f < 2; f++)
#pragma unroll
        for (int e = 0; e < 8; e++) a[f][e] = src[(threadIdx.x * 8 + e + f * 517) % kWords];
#pragma unroll
    for (int f = 0; f < 4; f++)
#pragma unroll
        for (int e = 0; e < 8; e++) b[f][e] = src[(threadIdx.x * 8 + e + kWords / 2 + f * 1031) % kWords];
    const int lane = threadIdx.x & 63, L = lane & 15, g = lane >> 4;
    const int krow = 32 * g + (L >> 1), swz = (krow & 7) | (((krow >> 5) & 1) << 3);
    const uint32_t off = krow * 256 + 8 * (L & 1);
    auto rd = [&](int chunk, int t) {
        return __builtin_amdgcn_ds_read_tr8_b64_v2i32((RF_LDS i32x2 *)(lds + off + (((chunk & 15) ^ swz) << 4) + t * 2048));
    };
    typedef int i32x4 __attribute__((ext_vector_type(4)));
    auto rd128 = [&](int frag, int h) {
        const int row = (16 * frag + L) & 255, chunk = (2 * g + h) ^ ((L >> 1) & 7);
        return *(RF_LDS i32x4 *)(lds + row * 128 + chunk * 16);
    };
    auto reread128 = [&](int t) {        // the same fragments at the same slots, two 16-byte reads each
        if (t % 4 == 0 && t < 28) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const i32x4 v = rd128(t / 4, h);
#pragma unroll
                for (int e = 0; e < 4; e++) a[((t / 4) + 1) & 1][4 * h + e] = v[e];
            }
        } else if (t >= 28) {
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const i32x4 v = rd128(8 + t, h);
#pragma unroll
                for (int e = 0; e < 4; e++) b[t - 28][4 * h + e] = v[e];
            }
        }
    };
    auto reread = [&](int t) {           // the GEMM's pattern: next m-tile's fragment, then the next block's fragments
        if (t % 4 == 0 && t < 28) {
#pragma unroll
            for (int q = 0; q < 4; q++) { i32x2 v = rd(t / 4, q); a[((t / 4) + 1) & 1][2 * q] = v[0]; a[((t / 4) + 1) & 1][2 * q + 1] = v[1]; }
        } else if (t >= 28) {
#pragma unroll
            for (int q = 0; q < 4; q++) { i32x2 v = rd(8 + t, q); b[t - 28][2 * q] = v[0]; b[t - 28][2 * q + 1] = v[1]; }
        }
    };
    if constexpr (MODE == 0) {
        f32x4 acc[8];
#pragma unroll
        for (int r = 0; r < 8; r++) acc[r] = (f32x4){0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int t = 0; t < kSlots; t++) {
                asm volatile("" : "+v"(b[t % 4]), "+v"(a[(t / 4) & 1]));      // no two MFMAs are the same to the compiler
                acc[t % 8] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[t % 4], a[(t / 4) & 1], acc[t % 8], 0, 0, 0, 0, 0, 0);
                asm volatile("" : "+v"(acc[t % 8]));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        float s = 0.f;
#pragma unroll
        for (int r = 0; r < 8; r++) s += acc[r][0] + acc[r][1] + acc[r][2] + acc[r][3];
        if (s == 1.2345f) out[threadIdx.x] = s;     // keeps the loop alive, practically never true
    } else {
        f32x4 acc[kSlots], pr[4];
#pragma unroll
        for (int r = 0; r < kSlots; r++) acc[r] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; r++) pr[r] = (f32x4){0.f, 0.f, 0.f, 0.f};
        float s[8];
#pragma unroll
        for (int j = 0; j < 8; j++) s[j] = sc * (j + 1);
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int t = 0; t < kSlots; t++) {
                asm volatile("" : "+v"(b[t % 4]), "+v"(a[(t / 4) & 1]));
                pr[t % 4] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b[t % 4], a[(t / 4) & 1], (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0, 0, 0, 0);
                asm volatile("" : "+v"(pr[t % 4]));
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (MODE == 2) reread(t);
                if constexpr (MODE == 3) reread128(t);
                const int u = (t + kSlots - 3) % kSlots;
#pragma unroll
                for (int e = 0; e < 4; e++) acc[u][e] = __builtin_fmaf(s[u / 4], pr[u % 4][e], acc[u][e]);
                asm volatile("" : "+v"(acc[u]));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        float r = 0.f;
#pragma unroll
        for (int q = 0; q < kSlots; q++) r += acc[q][0] + acc[q][1] + acc[q][2] + acc[q][3];
        if (r == 1.2345f) out[threadIdx.x] = r;
    }
}

// round-to-nearest-even e4m3fn code of a finite float, saturating at +-448
static uint8_t e4m3fn_code(float x) {
    const uint8_t sign = std::signbit(x) ? 0x80 : 0;
    float v = std::fabs(x);
    if (!(v < 448.f)) return sign | 0x7e;
    if (v < 0.0009765625f) return sign;                                   // below half the smallest subnormal
    int e;
    std::frexp(v, &e);                                                    // v = f * 2^e, f in [0.5, 1)
    int exp = e - 1 < -6 ? -6 : e - 1;                                    // subnormals share exponent -6
    const float q = std::nearbyint(std::ldexp(v, 3 - exp));               // multiples of 2^(exp-3), ties to even
    int m = (int)q;                                                       // 8..16 for normals, 0..8 for subnormals
    if (m == 16) { m = 8; exp++; }
    if (m < 8) return sign | (uint8_t)m;                                  // subnormal (exp == -6)
    return sign | (uint8_t)(((exp + 7) << 3) | (m - 8));
}

#define CHECK(e)                                                                              \
    do {                                                                                      \
        hipError_t r_ = (e);                                                                  \
        if (r_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #e, hipGetErrorString(r_)); return 1; } \
    } while (0)

typedef void (*kernel_t)(const int *, float *, int, float);

int main(int argc, char **argv) {
    const double seconds = argc > 1 ? atof(argv[1]) : 0.25;
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = argc > 2 && atoi(argv[2]) > 0 ? atoi(argv[2]) : prop.multiProcessorCount;
    int *d = nullptr;
    float *o = nullptr;
    CHECK(hipMalloc(&d, kWords * 4));
    CHECK(hipMalloc(&o, 512 * 4));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    std::mt19937 rng(1);
    std::normal_distribution<float> normal(0.f, 1.f);
    // (operand bits, loop form): the three operand kinds on the bare MFMA loop, then the GEMM's extra work
    const struct { int data, loop; const char *key; } runs[] = {
        {0, 0, "zeros"}, {1, 0, "normal"}, {2, 0, "random_bits"}, {1, 1, "normal_with_folds"},
        {1, 2, "normal_with_folds_and_lds_reads"}, {1, 3, "normal_with_folds_and_b128_reads"},
        {0, 2, "zeros_with_folds_and_lds_reads"}};
    constexpr int kRuns = sizeof(runs) / sizeof(runs[0]);
    const kernel_t kernels[4] = {inner_loop<0>, inner_loop<1>, inner_loop<2>, inner_loop<3>};
    double tflops[kRuns], ghz[kRuns];
    for (int r = 0; r < kRuns; r++) {
        std::mt19937 data_rng(1);
        std::vector<uint8_t> h(kWords * 4, 0);
        for (auto &byte : h) {
            if (runs[r].data == 1) byte = e4m3fn_code(normal(data_rng) * (448.f / 4.5f));
            if (runs[r].data == 2) do byte = (uint8_t)(data_rng() & 0xff); while ((byte & 0x7f) == 0x7f);
        }
        CHECK(hipMemcpy(d, h.data(), h.size(), hipMemcpyHostToDevice));
        const int iters = 1000;                                           // about 1 ms per launch
        // clocks settle over tens of milliseconds of load: run for `seconds`, report the last fifth
        const double flop = (double)cus * 8 * iters * kSlots * 2.0 * 16 * 16 * 128;
        double elapsed = 0, last = 0;
        int launches = 0, last_launches = 0;
        while (elapsed < seconds) {
            CHECK(hipEventRecord(e0));
            for (int q = 0; q < 10; q++)
                hipLaunchKernelGGL(kernels[runs[r].loop], dim3(cus), dim3(512), kLdsBytes, 0, d, o, iters, 0.001f);
            CHECK(hipEventRecord(e1));
            CHECK(hipEventSynchronize(e1));
            float ms;
            CHECK(hipEventElapsedTime(&ms, e0, e1));
            elapsed += ms * 1e-3;
            launches += 10;
            if (elapsed >= 0.8 * seconds) { last += ms * 1e-3; last_launches += 10; }
        }
        if (last_launches == 0) { last = elapsed; last_launches = launches; }
        tflops[r] = flop * last_launches / last * 1e-12;
        // two waves per SIMD, 32 cycles per instruction: the clock at which the matrix unit would be busy all the time
        ghz[r] = (double)iters * kSlots * 2 * 32 * last_launches / last * 1e-9;
    }
    printf("{");
    for (int r = 0; r < kRuns; r++) printf("\"%s\": %.1f, ", runs[r].key, tflops[r]);
    printf("\"unit\": \"TFLOP/s\", \"cus\": %d, \"implied_clock_ghz\": {", cus);
    for (int r = 0; r < kRuns; r++) printf("\"%s\": %.3f%s", runs[r].key, ghz[r], r + 1 < kRuns ? ", " : "");
    printf("}}\n");
    return 0;
}
