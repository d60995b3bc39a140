// Test infrastructure: do the vector memory instructions of one wave complete in issue order? Each iteration a wave
// issues NA LDS-DMA loads (global_load_lds_dwordx4) from a 1 GiB buffer (L2 misses: the addresses change every
// iteration) and then NB younger instructions that finish sooner: loads from a small hot buffer (L2 hits, 16 or 4 bytes
// per lane), or stores of 16 bytes per lane to hot lines (plain, or written through with sc1). It waits with
// s_waitcnt vmcnt(NB) and checks that the NA older loads have landed in LDS (the buffer's content is a function of the
// address). The GEMM kernels rely on this twice: the three-stage loop waits for "all but the newest K block's loads",
// and the persistent kernel's first wait of a tile for "all but the previous tile's stores". Prints one line per case;
// the last field of each line is the number of stale dwords (expected 0).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#include <vector>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s at %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
__device__ __host__ inline uint32_t pat(uint64_t dword_index) { return (uint32_t)(dword_index * 2654435761u) ^ 0x5bd1e995u; }
template <int NA, int NB, int WIDE_B>
__global__ __launch_bounds__(512) void probe(const uint32_t *big, size_t big_dwords, const uint32_t *hot, int iters,
                                             unsigned long long *bad, unsigned long long *checked) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
    const uint32_t my = lds_base + wave * (NA + NB) * 1024;
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;
    uint32_t rng = blockIdx.x * 977 + wave * 131 + 7;
    unsigned long long nbad = 0, nchk = 0;
    for (int it = 0; it < iters; it++) {
        // poison the NA destination slots
        for (int q = 0; q < NA; q++) *(uint4 *)(lds + wave * (NA + NB) * 1024 + q * 1024 + lane * 16) = make_uint4(0xdeadbeef, 0xdeadbeef, 0xdeadbeef, 0xdeadbeef);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        uint64_t base_dw[NA];
#pragma unroll
        for (int q = 0; q < NA; q++) {
            rng = rng * 1664525u + 1013904223u;
            base_dw[q] = ((uint64_t)(rng >> 4) * 256) % (big_dwords - 256);     // 1 KiB chunk start (dwords), wave-uniform
            base_dw[q] = __builtin_amdgcn_readfirstlane((uint32_t)base_dw[q]) | ((uint64_t)__builtin_amdgcn_readfirstlane((uint32_t)(base_dw[q] >> 32)) << 32);
            const uint32_t *src = big + base_dw[q];
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(lane16), "s"(src), "s"(my + q * 1024) : "memory");
        }
#pragma unroll
        for (int q = 0; q < NB; q++) {
            if (WIDE_B == 2 || WIDE_B == 3) {
                typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
                const u32x4_t w = {1u, 2u, 3u, (unsigned)it};
                uint32_t *dst = (uint32_t *)hot + 4096 + ((blockIdx.x * 8 + wave) % 64) * 2048 + q * 256 + lane * 4;
                if (WIDE_B == 2) asm volatile("global_store_dwordx4 %0, %1, off\n\ts_nop 1" :: "v"(dst), "v"(w) : "memory");
                else asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" :: "v"(dst), "v"(w) : "memory");
            } else if (WIDE_B)
                asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(lane16), "s"(hot + q * 256), "s"(my + (NA + q) * 1024) : "memory");
            else
                asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" :: "v"(lane4), "s"(hot + q * 256), "s"(my + (NA + q) * 1024) : "memory");
        }
        if (NB == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else if (NB == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
        else if (NB == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else if (NB == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if (NB == 7) asm volatile("s_waitcnt vmcnt(7)" ::: "memory");
        else if (NB == 16) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        else if (NB == 8) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
#pragma unroll
        for (int q = 0; q < NA; q++) {
            volatile uint32_t *vp = (volatile uint32_t *)(lds + wave * (NA + NB) * 1024 + q * 1024 + lane * 16);
            uint4 v = make_uint4(vp[0], vp[1], vp[2], vp[3]);
            const uint64_t dw = base_dw[q] + lane * 4;
            nbad += (v.x != pat(dw)) + (v.y != pat(dw + 1)) + (v.z != pat(dw + 2)) + (v.w != pat(dw + 3));
            nchk += 4;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    atomicAdd(bad, nbad);
    atomicAdd(checked, nchk);
}
template <int NA, int NB, int WIDE_B>
void run(const uint32_t *big, size_t n, const uint32_t *hot, int iters, unsigned long long *d) {
    CK(hipMemset(d, 0, 16));
    CK(hipFuncSetAttribute((const void *)probe<NA, NB, WIDE_B>, hipFuncAttributeMaxDynamicSharedMemorySize, 8 * (NA + NB) * 1024));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    CK(hipEventRecord(e0));
    hipLaunchKernelGGL((probe<NA, NB, WIDE_B>), dim3(1024), dim3(512), 8 * (NA + NB) * 1024, 0, big, n, hot, iters, d, d + 1);
    CK(hipEventRecord(e1));
    CK(hipDeviceSynchronize());
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    printf("[%.1f ms, %.2f TB/s of misses] ", ms, 1024.0 * 8 * iters * NA * 1024 / (ms * 1e-3) / 1e12);
    unsigned long long h[2]; CK(hipMemcpy(h, d, 16, hipMemcpyDeviceToHost));
    printf("older %d dwordx4 loads (L2 misses), then %d %s, wait vmcnt(%d): checked %llu stale %llu\n", NA, NB, WIDE_B == 2 ? "dwordx4 stores (L2 hits)" : WIDE_B == 3 ? "dwordx4 stores written through (sc1)" : WIDE_B ? "dwordx4 loads (L2 hits)" : "dword loads (L2 hits)", NB, h[1], h[0]);
    fflush(stdout);
}
int main(int argc, char **argv) {
    const int iters = argc > 1 ? atoi(argv[1]) : 2000;
    const size_t n = (size_t)1 << 28;   // 1 GiB of dwords: far larger than L2 + MALL
    uint32_t *big, *hot; unsigned long long *d;
    CK(hipMalloc(&big, n * 4)); CK(hipMalloc(&hot, 16 * 1024 + 64 * 2048 * 4 + 4096 * 4)); CK(hipMalloc(&d, 16));
    { std::vector<uint32_t> h(1 << 20); for (size_t c = 0; c < n; c += h.size()) { for (size_t i = 0; i < h.size(); i++) h[i] = pat(c + i); CK(hipMemcpy(big + c, h.data(), h.size() * 4, hipMemcpyHostToDevice)); } }
    CK(hipMemset(hot, 0x11, 16 * 1024));
    run<4, 0, 1>(big, n, hot, iters, d);     // control: vmcnt(0)
    run<4, 4, 1>(big, n, hot, iters, d);
    run<7, 7, 1>(big, n, hot, iters, d);
    run<4, 1, 1>(big, n, hot, iters, d);
    run<4, 1, 0>(big, n, hot, iters, d);     // the mixed-width case
    run<4, 4, 0>(big, n, hot, iters, d);
    run<4, 4, 2>(big, n, hot, iters, d);     // younger stores that hit in L2
    run<4, 16, 2>(big, n, hot, iters, d);
    run<7, 8, 2>(big, n, hot, iters, d);
    run<4, 16, 3>(big, n, hot, iters, d);    // younger stores written through to memory
    run<7, 8, 3>(big, n, hot, iters, d);
    return 0;
}
