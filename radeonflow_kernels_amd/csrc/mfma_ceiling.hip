// Measures what the whole gfx950 chip sustains on the fp8 MFMA the GEMM is built on when nothing else runs:
// 8 waves per compute unit issue v_mfma_f32_16x16x128_f8f6f4 back to back from registers (8 independent
// accumulators per wave over 4 x 2 operand fragments, no memory, no LDS). The published peak (5.0 PFLOP/s dense) assumes 2.4 GHz; under load the
// chip lowers its clock to stay inside its power limit, and how far depends on how many bits toggle in the operands.
// The figure for realistic operands is the ceiling any fp8 GEMM on this chip can approach.
//
//   mfma_ceiling [seconds per mode]      prints one JSON line:
//   {"zeros": TFLOP/s, "normal": TFLOP/s, "random_bits": TFLOP/s, "unit": "TFLOP/s", "cus": n, "implied_clock_ghz": {...}}
// zeros: all operand bytes 0. normal: e4m3fn codes of N(0,1) samples scaled so that 4.5 sigma maps to 448 (what a
// blockwise quantiser produces). random_bits: uniformly random finite e4m3fn codes.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

typedef int i32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kAcc = 8, kWords = 4096;

__global__ __launch_bounds__(512) void mfma_from_registers(const int *__restrict__ src, float *out, int iters) {
    // 4 x 2 operand fragments, as a wave tile of a GEMM holds them: consecutive MFMAs see different operand bits
    i32x8 a[4], b[2];
#pragma unroll
    for (int f = 0; f < 4; f++)
#pragma unroll
        for (int e = 0; e < 8; e++) a[f][e] = src[(threadIdx.x * 8 + e + f * 517) % kWords];
#pragma unroll
    for (int f = 0; f < 2; f++)
#pragma unroll
        for (int e = 0; e < 8; e++) b[f][e] = src[(threadIdx.x * 8 + e + kWords / 2 + f * 1031) % kWords];
    f32x4 acc[kAcc];
#pragma unroll
    for (int r = 0; r < kAcc; r++) acc[r] = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < kAcc; r++)
            acc[r] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[r % 4], b[r / 4], acc[r], 0, 0, 0, 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int r = 0; r < kAcc; r++) s += acc[r][0] + acc[r][1] + acc[r][2] + acc[r][3];
    if (s == 1.2345f) out[threadIdx.x] = s;     // keeps the loop alive, practically never true
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

int main(int argc, char **argv) {
    const double seconds = argc > 1 ? atof(argv[1]) : 0.25;
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    int *d = nullptr;
    float *o = nullptr;
    CHECK(hipMalloc(&d, kWords * 4));
    CHECK(hipMalloc(&o, 512 * 4));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    std::mt19937 rng(1);
    std::normal_distribution<float> normal(0.f, 1.f);
    double tflops[3], ghz[3];
    for (int mode = 0; mode < 3; mode++) {
        std::vector<uint8_t> h(kWords * 4, 0);
        for (auto &byte : h) {
            if (mode == 1) byte = e4m3fn_code(normal(rng) * (448.f / 4.5f));
            if (mode == 2) do byte = (uint8_t)(rng() & 0xff); while ((byte & 0x7f) == 0x7f);
        }
        CHECK(hipMemcpy(d, h.data(), h.size(), hipMemcpyHostToDevice));
        const int iters = 4000;                                           // about 1 ms per launch
        // clocks settle over tens of milliseconds of load: run for `seconds`, report the last fifth
        const double flop = (double)cus * 8 * iters * kAcc * 2.0 * 16 * 16 * 128;
        double elapsed = 0, last = 0;
        int launches = 0, last_launches = 0;
        while (elapsed < seconds) {
            CHECK(hipEventRecord(e0));
            for (int r = 0; r < 10; r++) hipLaunchKernelGGL(mfma_from_registers, dim3(cus), dim3(512), 0, 0, d, o, iters);
            CHECK(hipEventRecord(e1));
            CHECK(hipEventSynchronize(e1));
            float ms;
            CHECK(hipEventElapsedTime(&ms, e0, e1));
            elapsed += ms * 1e-3;
            launches += 10;
            if (elapsed >= 0.8 * seconds) { last += ms * 1e-3; last_launches += 10; }
        }
        if (last_launches == 0) { last = elapsed; last_launches = launches; }
        tflops[mode] = flop * last_launches / last * 1e-12;
        // two waves per SIMD, 32 cycles per instruction
        ghz[mode] = (double)iters * kAcc * 2 * 32 * last_launches / last * 1e-9;
    }
    printf("{\"zeros\": %.1f, \"normal\": %.1f, \"random_bits\": %.1f, \"unit\": \"TFLOP/s\", \"cus\": %d, "
           "\"implied_clock_ghz\": {\"zeros\": %.3f, \"normal\": %.3f, \"random_bits\": %.3f}}\n",
           tflops[0], tflops[1], tflops[2], cus, ghz[0], ghz[1], ghz[2]);
    return 0;
}
