// Host side of libgemm.so: the C ABI declared in include/rf_gemm.h.
//
// Takes the place of the reference's launcher (src/gemm/gemm_launcher.cpp): `run` keeps its
// signature and abort-on-error behaviour; dispatch is shape-generic (a heuristic over a small
// variant table tuned for gfx950) instead of a switch over 29 hard-coded shapes, and no transpose
// pre-pass or transposed copies exist.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cmath>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/rf_gemm.h"
#include "fp8_gemm_kernels.h"
#include "fp8_gemm_persistent.h"
#include "fp8_gemm_skinny.h"
#include "quantize_kernels.h"

// Scratch memory of rf_fp8_gemm_static, the entry point that allocates nothing: split-K partial sums and staging
// copies live here instead of in buffers from hipMalloc. Every device the library runs on holds its own copy at its
// own address until the process ends; host code never uses this name as an address (see ensure_device_info).
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

namespace {

thread_local std::string g_last_error;

int fail(int code, const std::string &msg) {
    g_last_error = msg;
    return code;
}
#define RF_HIP(expr)                                                                                   \
    do {                                                                                               \
        hipError_t e_ = (expr);                                                                        \
        if (e_ != hipSuccess)                                                                          \
            return fail(RF_ERR_HIP, std::string(#expr) + ": " + hipGetErrorString(e_));               \
    } while (0)

// ---- variant table -------------------------------------------------------------------------
typedef void (*tile_kernel_t)(const uint8_t *, const uint8_t *, const float *, const float *, void *, int, int, int,
                              int, int, int, int, int);
typedef void (*streamk_kernel_t)(const uint8_t *, const uint8_t *, const float *, const float *, uint16_t *, int, int,
                                 int, int, int, int, unsigned *, float *);
typedef void (*persistent_kernel_t)(const uint8_t *, const uint8_t *, const float *, const float *, uint16_t *, int, int,
                                    int, int, int, int, int);
struct Variant {
    int bm, bn, waves_m, waves_n, lds;
    tile_kernel_t direct, partial;
    streamk_kernel_t streamk;            // null: the variant has no stream-K form
    persistent_kernel_t persistent;      // null: no persistent form
    int lds_persistent;
    persistent_kernel_t persistent_half_tail = nullptr;   // null: no form that ends with half tiles
    int k_groups = 1;                    // > 1: wave groups of one workgroup split K between them (needs K/128 % k_groups == 0)
    int lds_bytes() const { return lds; }
    int threads() const { return waves_m * waves_n * 64 * k_groups; }
};
#define RF_VARIANT(BM, BN, WM, WN)                                                         \
    Variant { BM, BN, WM, WN, rf::TileGeom<BM, BN, WM, WN>::LDS_BYTES,                     \
              rf::gemm_fp8_blockscale_tile<BM, BN, WM, WN, false>,                         \
              rf::gemm_fp8_blockscale_tile<BM, BN, WM, WN, true>,                          \
              rf::gemm_fp8_blockscale_streamk<BM, BN, WM, WN>,                             \
              rf::gemm_fp8_blockscale_persistent<BM, BN, WM, WN>,                          \
              rf::PersistentGeom<BM, BN, WM, WN>::LDS_BYTES }
// tiles with sides that are not powers of two, same inner loop: one workgroup per tile only
#define RF_VARIANT_TILE_ONLY(BM, BN, WM, WN)                                               \
    Variant { BM, BN, WM, WN, rf::TileGeom<BM, BN, WM, WN>::LDS_BYTES,                     \
              rf::gemm_fp8_blockscale_tile<BM, BN, WM, WN, false>,                         \
              rf::gemm_fp8_blockscale_tile<BM, BN, WM, WN, true>, nullptr, nullptr, 0 }
// the same with three LDS stages: two K blocks in flight instead of one. A K block of these tiles is 0.4 us of MFMAs,
// less than a load takes to come back from L2 or the Infinity Cache on a busy chip, so with two stages the loop ran at
// the latency of its loads: 1024 x 4608 x 7168 45.6 -> 39.0 us, 256 x 7168 x 2304 15.6 -> 13.1 us; the best plan of 86
// of the 163 tabled shapes. The two-stage forms stay: they fit more workgroups per CU (64 x 128: three instead of
// two), which the smallest problems prefer. (128 x 128 with three stages never won and is not built.)
#define RF_VARIANT_TILE_ONLY_NS3(BM, BN, WM, WN)                                           \
    Variant { BM, BN, WM, WN, rf::TileGeom<BM, BN, WM, WN, 3>::LDS_BYTES,                  \
              rf::gemm_fp8_blockscale_tile<BM, BN, WM, WN, false, 3>,                      \
              rf::gemm_fp8_blockscale_tile<BM, BN, WM, WN, true, 3>, nullptr, nullptr, 0 }
const Variant kVariants[] = {
    Variant{256, 256, 2, 4, rf::TileGeom<256, 256, 2, 4>::LDS_BYTES, rf::gemm_fp8_blockscale_tile<256, 256, 2, 4, false>,
            rf::gemm_fp8_blockscale_tile<256, 256, 2, 4, true>, rf::gemm_fp8_blockscale_streamk<256, 256, 2, 4>,
            rf::gemm_fp8_blockscale_persistent<256, 256, 2, 4>, rf::PersistentGeom<256, 256, 2, 4>::LDS_BYTES,
            rf::gemm_fp8_blockscale_persistent<256, 256, 2, 4, true>},   // 0: 8 waves, wave tile 128(m) x 64(n), 128 KiB LDS
    RF_VARIANT(128, 128, 2, 2),   // 1: 4 waves, wave tile 64 x 64, 64 KiB LDS (2 workgroups per CU)
    RF_VARIANT(256, 128, 2, 2),   // 2: 4 waves, wave tile 128 x 64, 96 KiB LDS
    RF_VARIANT(128, 256, 2, 4),   // 3: 8 waves, wave tile 64 x 64, 96 KiB LDS
    RF_VARIANT(128, 64, 2, 1),    // 4: 2 waves, wave tile 64 x 64, 48 KiB LDS (3 workgroups per CU)
    RF_VARIANT_TILE_ONLY(192, 192, 2, 4),   // 5: 8 waves, wave tile 96 x 48, 98 KiB LDS (6144 x 4608 = 768 tiles = 3 x 256)
    RF_VARIANT_TILE_ONLY(128, 192, 2, 4),   // 6: 8 waves, wave tile 64 x 48, 82 KiB LDS (N = 576, 1536: no padded columns)
    RF_VARIANT_TILE_ONLY(64, 128, 2, 2),    // 7: 4 waves, wave tile 32 x 64, 49 KiB LDS (3 workgroups per CU; short M)
    RF_VARIANT_TILE_ONLY_NS3(128, 192, 2, 4),   // 8: variant 6 with three stages, 123 KiB LDS
    RF_VARIANT_TILE_ONLY_NS3(64, 128, 2, 2),    // 9: variant 7 with three stages, 74 KiB LDS (2 workgroups per CU)
    RF_VARIANT_TILE_ONLY_NS3(128, 256, 2, 4),   // 10: variant 3 with three stages, 149 KiB LDS
    RF_VARIANT_TILE_ONLY_NS3(192, 192, 2, 4),   // 11: variant 5 with three stages, 147 KiB LDS
    // 12: the 64 x 128 three-stage tile with K split between two wave groups of one workgroup (8 waves, 150 KiB LDS):
    // the split-K plan of a short, wide-K shape in one launch, with no partial sums in memory
    Variant{64, 128, 2, 2, rf::InWgSplitGeom<64, 128, 2, 2, 3, 2>::LDS_BYTES,
            rf::gemm_fp8_blockscale_tile_ksplit_in_wg<64, 128, 2, 2, 3, 2>, nullptr, nullptr, nullptr, 0, nullptr, 2},
    // 13: the 128 x 128 two-stage tile with K split between two wave groups (8 waves, 130 KiB LDS)
    Variant{128, 128, 2, 2, rf::InWgSplitGeom<128, 128, 2, 2, 2, 2>::LDS_BYTES,
            rf::gemm_fp8_blockscale_tile_ksplit_in_wg<128, 128, 2, 2, 2, 2>, nullptr, nullptr, nullptr, 0, nullptr, 2},
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

// ---- process-wide state ---------------------------------------------------------------------
struct TunedPlan {
    int m, n, k, variant, split_k, group_m, stream_k;
};

// Buffers, counters and kernel attributes belong to a device: one State per device, chosen by the device that is
// current at the call. Plans and the lock are shared by the process.
//
// Temporary device memory (split-K partial sums, stream-K slots and counters, staging copies of ragged operands) is
// kept per (device, stream): two launches on different streams of one device never share a buffer, so they may overlap,
// and launches on one stream are ordered by the stream. A buffer that has to grow is replaced, and the old one is kept
// until rf_gemm_destroy: work enqueued earlier may still use it, and waiting for that work here would block the host
// (and, with a timing callback of run() pending, deadlock against it).
struct StreamBuffers {
    hipStream_t stream = nullptr;
    uint8_t *pad = nullptr;              // staging for shapes the tiled kernels do not take as they are (see launch_padded)
    size_t pad_bytes = 0;
    float *ws = nullptr;                 // split-K partial sums / stream-K slots
    size_t ws_bytes = 0;
    unsigned *tile_count = nullptr;      // stream-K arrival counters, zero between launches
    bool tile_count_zeroed = false;
    uint64_t last_use = 0;
};
constexpr int kMaxStreamBuffers = 32;    // per device; one more stream takes over the least recently used set
struct State {
    std::vector<StreamBuffers> buffers;
    std::vector<void *> retired;         // outgrown buffers, freed by rf_gemm_destroy
    uint64_t tick = 0;
    bool attrs_set = false, grouped_attrs_set = false;
    int num_cu = 0;
    uint8_t *static_scratch = nullptr;   // this device's copy of the file-scope scratch array (rf_fp8_gemm_static)
    std::mutex ev_mu;                    // guards free_events only: the timing callback takes no other lock
    std::vector<std::pair<hipEvent_t, hipEvent_t>> free_events;
};
struct Shared {
    std::mutex mu;
    std::vector<TunedPlan> user_plans;   // rf_gemm_load_plans / RF_GEMM_PLANS: looked up before the built-in table
    bool env_plans_checked = false;
};
constexpr int kMaxDevices = 64;
Shared &shared() {
    static Shared s;
    return s;
}
State &state() {
    static State states[kMaxDevices];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) dev = 0;
    return states[dev];
}

// Plan file: one plan per line, "M N K variant split_k group_m stream_k"; braces and commas count as blanks (so a
// tuned_plans.inc written by the tuner is a plan file too), '#' and "//" start a comment. Appends to `out`.
int parse_plans(const char *path, std::vector<TunedPlan> &out) {
    FILE *f = fopen(path, "r");
    if (!f) return fail(RF_ERR_BAD_CONFIG, std::string("cannot open plan file ") + path);
    char line[512];
    int lineno = 0;
    std::vector<TunedPlan> plans;
    while (fgets(line, sizeof line, f)) {
        lineno++;
        if (char *c = strstr(line, "//")) *c = 0;
        if (char *c = strchr(line, '#')) *c = 0;
        for (char *c = line; *c; c++)
            if (*c == '{' || *c == '}' || *c == ',') *c = ' ';
        TunedPlan p;
        char extra;
        const int got = sscanf(line, " %d %d %d %d %d %d %d %c", &p.m, &p.n, &p.k, &p.variant, &p.split_k, &p.group_m,
                               &p.stream_k, &extra);
        if (got <= 0) continue;                       // blank or comment line
        if (got != 7 || p.m < 1 || p.n < 1 || p.k < rf::BK || p.k % rf::BK != 0 || p.variant < 0 ||
            p.variant >= kNumVariants || p.split_k < 1 || p.group_m < 1 || p.stream_k < RF_SCHEDULE_TILES ||
            p.stream_k > RF_SCHEDULE_SKINNY_K || (p.stream_k != RF_SCHEDULE_TILES && p.split_k != 1)) {
            fclose(f);
            return fail(RF_ERR_BAD_CONFIG, std::string(path) + ":" + std::to_string(lineno) +
                                               ": expected \"M N K variant split_k group_m stream_k\" with valid values");
        }
        plans.push_back(p);
    }
    fclose(f);
    out.insert(out.end(), plans.begin(), plans.end());
    return RF_OK;
}

int ensure_device_info(State &s) {
    if (s.attrs_set) return RF_OK;
    if (!shared().env_plans_checked) {
        // a file named by RF_GEMM_PLANS is loaded once, before the first plan is chosen; a bad file is an error
        if (const char *path = getenv("RF_GEMM_PLANS")) {
            int rc = parse_plans(path, shared().user_plans);
            if (rc != RF_OK) return rc;
        }
        shared().env_plans_checked = true;
    }
    int dev = 0;
    RF_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    RF_HIP(hipGetDeviceProperties(&prop, dev));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(RF_ERR_HIP, std::string("libgemm.so is built for gfx950 only, device is ") + prop.gcnArchName);
    s.num_cu = prop.multiProcessorCount;
    for (const Variant &v : kVariants) {
        RF_HIP(hipFuncSetAttribute((const void *)v.direct, hipFuncAttributeMaxDynamicSharedMemorySize, v.lds_bytes()));
        if (v.partial)
            RF_HIP(hipFuncSetAttribute((const void *)v.partial, hipFuncAttributeMaxDynamicSharedMemorySize, v.lds_bytes()));
        if (v.streamk)
            RF_HIP(hipFuncSetAttribute((const void *)v.streamk, hipFuncAttributeMaxDynamicSharedMemorySize, v.lds_bytes()));
        if (v.persistent)
            RF_HIP(hipFuncSetAttribute((const void *)v.persistent, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       v.lds_persistent));
        if (v.persistent_half_tail)
            RF_HIP(hipFuncSetAttribute((const void *)v.persistent_half_tail, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       v.lds_persistent));
    }
    RF_HIP(hipFuncSetAttribute((const void *)rf::gemm_fp8_blockscale_skinny<1>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               rf::SkinnyGeom<1>::LDS_BYTES));
    RF_HIP(hipFuncSetAttribute((const void *)rf::gemm_fp8_blockscale_skinny<2>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               rf::SkinnyGeom<2>::LDS_BYTES));
    RF_HIP(hipFuncSetAttribute((const void *)rf::gemm_fp8_blockscale_skinny<3>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               rf::SkinnyGeom<3>::LDS_BYTES));
    RF_HIP(hipFuncSetAttribute((const void *)rf::gemm_fp8_blockscale_skinny<4>, hipFuncAttributeMaxDynamicSharedMemorySize,
                               rf::SkinnyGeom<4>::LDS_BYTES));
    // the device address of this device's copy of the scratch array (the array's name is only a host-side handle)
    void *scratch_ptr = nullptr;
    RF_HIP(hipGetSymbolAddress(&scratch_ptr, HIP_SYMBOL(scratch)));
    s.static_scratch = (uint8_t *)scratch_ptr;
    s.attrs_set = true;
    return RF_OK;
}

constexpr int kMaxStreamKTiles = 16384;

__global__ void zero_words(unsigned *p) { p[blockIdx.x * 256 + threadIdx.x] = 0u; }

// hipMalloc that also works while the calling thread records a stream into a HIP graph: an allocation is not part
// of the recorded work, so the capture mode is relaxed around it (under the default mode the call would fail and
// invalidate the capture).
hipError_t device_malloc(void **p, size_t bytes) {
    hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
    hipError_t e = hipThreadExchangeStreamCaptureMode(&mode);
    if (e != hipSuccess) return e;
    e = hipMalloc(p, bytes);
    (void)hipThreadExchangeStreamCaptureMode(&mode);
    return e;
}

// Where a launch finds its temporary device memory: the growable buffers of its (device, stream), or, for
// rf_fp8_gemm_static, consecutive pieces of the device's static scratch array (nothing is allocated; a launch that
// needs more than the array holds fails).
int buffers_of(State &s, hipStream_t stream, StreamBuffers **out);
struct Mem {
    State &s;
    StreamBuffers *sb = nullptr;         // growable buffers of `stream`, bound at the first use (never in static mode)
    uint8_t *fixed = nullptr;            // static mode: this device's scratch array
    size_t fixed_used = 0;
    hipStream_t stream = nullptr;
    // Most launches need no temporary memory at all (one kernel, no K split, no staging): the stream's buffer set is
    // looked up, and past kMaxStreamBuffers streams taken over from another stream, only when a buffer is asked for.
    int bind() { return sb ? RF_OK : buffers_of(s, stream, &sb); }

    template <typename T>
    int grow(T *&buf, size_t &have, size_t need) {
        if (need <= have) return RF_OK;
        // the old buffer may still be read by launches enqueued earlier: keep it until rf_gemm_destroy
        if (buf) s.retired.push_back(buf);
        const size_t want = need > have + have / 2 ? need : have + have / 2;
        buf = nullptr;
        have = 0;
        RF_HIP(device_malloc((void **)&buf, want));
        have = want;
        return RF_OK;
    }
    int take_fixed(size_t bytes, void **out, const char *what) {
        const size_t at = (fixed_used + 255) / 256 * 256;
        if (at + bytes > kStaticScratchBytes)
            return fail(RF_ERR_BAD_CONFIG, std::string("rf_fp8_gemm_static: this shape needs ") + std::to_string(at + bytes) +
                                               " bytes of scratch memory (" + what + "), the static array holds " +
                                               std::to_string(kStaticScratchBytes));
        *out = fixed + at;
        fixed_used = at + bytes;
        return RF_OK;
    }
    // bytes the static array still has to give (after rounding the next piece up to 256)
    size_t fixed_left() const {
        const size_t at = (fixed_used + 255) / 256 * 256;
        return at < kStaticScratchBytes ? kStaticScratchBytes - at : 0;
    }
    int pad(size_t bytes, uint8_t **out) {
        if (fixed) return take_fixed(bytes, (void **)out, "staging copy of ragged or unaligned operands");
        int rc = bind();
        if (rc != RF_OK) return rc;
        rc = grow(sb->pad, sb->pad_bytes, bytes);
        *out = sb->pad;
        return rc;
    }
    int workspace(size_t bytes, float **out) {
        if (fixed) return take_fixed(bytes, (void **)out, "split-K partial sums");
        int rc = bind();
        if (rc != RF_OK) return rc;
        rc = grow(sb->ws, sb->ws_bytes, bytes);
        *out = sb->ws;
        return rc;
    }
    int tile_counters(unsigned **out) {
        if (fixed) return fail(RF_ERR_BAD_CONFIG, "rf_fp8_gemm_static: the stream-K schedule is not available");
        int rc = bind();
        if (rc != RF_OK) return rc;
        if (!sb->tile_count) RF_HIP(device_malloc((void **)&sb->tile_count, kMaxStreamKTiles * sizeof(unsigned)));
        if (!sb->tile_count_zeroed) {
            // zeroed on the stream of the launch that follows (the kernels leave the counters at zero afterwards);
            // a kernel and not a memset, so that the call may be recorded into a HIP graph. A recorded fill has not
            // run yet, so it does not count: launches keep filling first until one has done so for real.
            // (on the legacy null stream the query itself is refused while another thread captures in global mode:
            // that counts as "capturing", so the fill is issued and the flag stays false)
            hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
            const hipError_t qe = hipStreamIsCapturing(sb->stream, &st);
            if (qe == hipErrorStreamCaptureImplicit || qe == hipErrorStreamCaptureUnsupported) {
                (void)hipGetLastError();
                st = hipStreamCaptureStatusActive;
            } else if (qe != hipSuccess) {
                return fail(RF_ERR_HIP, std::string("hipStreamIsCapturing: ") + hipGetErrorString(qe));
            }
            hipLaunchKernelGGL(zero_words, dim3(kMaxStreamKTiles / 256), dim3(256), 0, sb->stream, sb->tile_count);
            RF_HIP(hipGetLastError());
            sb->tile_count_zeroed = st == hipStreamCaptureStatusNone;
        }
        *out = sb->tile_count;
        return RF_OK;
    }
};

// The buffer set of (current device, stream); the caller holds the lock. A set prepared by rf_gemm_init and not yet
// bound to a stream is taken first. Past kMaxStreamBuffers streams the least recently used set changes hands: the new
// stream is made to wait (on the device, through an event) for what the old stream has enqueued so far, so the host
// does not wait. A stream that is being captured into a graph cannot take a set over (the wait would become part of
// the graph, and the old stream's later work would not be ordered against the graph's replays): RF_ERR_BAD_CONFIG.
constexpr uintptr_t kUnboundStream = 1;  // not a valid stream handle
int buffers_of(State &s, hipStream_t stream, StreamBuffers **out) {
    StreamBuffers *unbound = nullptr, *lru = nullptr;
    for (StreamBuffers &b : s.buffers) {
        if (b.stream == stream) {
            b.last_use = ++s.tick;
            *out = &b;
            return RF_OK;
        }
        if ((uintptr_t)b.stream == kUnboundStream) unbound = &b;
        if (!lru || b.last_use < lru->last_use) lru = &b;
    }
    StreamBuffers *b = unbound;
    if (!b && (int)s.buffers.size() < kMaxStreamBuffers) {
        if (s.buffers.capacity() < (size_t)kMaxStreamBuffers) s.buffers.reserve(kMaxStreamBuffers);
        s.buffers.emplace_back();
        b = &s.buffers.back();
    }
    if (!b) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        const hipError_t qe = hipStreamIsCapturing(stream, &st);
        if (qe != hipSuccess || st != hipStreamCaptureStatusNone) {
            if (qe != hipSuccess) (void)hipGetLastError();
            return fail(RF_ERR_BAD_CONFIG, "more than " + std::to_string(kMaxStreamBuffers) + " streams have used temporary "
                        "device memory on this device, and a stream that is being captured cannot take over another "
                        "stream's buffers: use rf_fp8_gemm_static under capture, or fewer streams");
        }
        hipEvent_t ev = nullptr;
        RF_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        hipError_t e = hipEventRecord(ev, lru->stream);
        if (e == hipSuccess) e = hipStreamWaitEvent(stream, ev, 0);
        (void)hipEventDestroy(ev);                               // released once the wait has been satisfied
        if (e != hipSuccess) {
            // the old stream no longer exists (or is being captured): wait for the device instead
            (void)hipGetLastError();
            RF_HIP(hipDeviceSynchronize());
        }
        b = lru;
    }
    b->stream = stream;
    b->last_use = ++s.tick;
    *out = b;
    return RF_OK;
}

inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

struct Variant;
bool persistent_ok(const Variant &v, int m, int n, int k);

bool tiled_path_ok(const void *a, const void *b, const void *c, int m, int n) {
    return m >= 16 && n >= 16 && m % 16 == 0 && n % 16 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0 &&
           ((uintptr_t)c % 16) == 0;
}

// (K * M and K * N below 2^32: the persistent kernel keeps a load cursor's K position in 32-bit per-lane offsets)
bool persistent_ok(const Variant &v, int m, int n, int k) {
    return v.persistent && m >= v.bm && m % 16 == 0 && n % v.bn == 0 && (k / rf::BK) % 2 == 0 &&
           (unsigned long long)k * m < (1ull << 32) && (unsigned long long)k * n < (1ull << 32);
}

// Persistent schedule that finishes the last, partial round with half tiles: one workgroup per CU, at least one whole
// round, and a last round that two half tiles per left-over tile still fit into (see the kernel).
bool half_tail_ok(const Variant &v, int m, int n, int k, int num_cu) {
    if (!v.persistent_half_tail || !persistent_ok(v, m, n, k)) return false;
    const long t = (long)ceil_div(m, v.bm) * ceil_div(n, v.bn);
    const long r = t % num_cu;
    return t >= num_cu && r > 0 && (r + 7) / 8 * 8 + r <= num_cu;
}

// Skinny-K schedule (fp8_gemm_skinny.h): one to four K blocks, whole 16-row m-tiles and whole 64-column wave tiles.
bool skinny_ok(int m, int n, int k) {
    return k >= rf::BK && k <= 4 * rf::BK && k % rf::BK == 0 && m >= 16 && m % 16 == 0 && n >= 64 && n % 64 == 0;
}

// Stream-K: at least one tile per workgroup (then a split tile has exactly two contributors, which is all the kernel
// handles) and no more tiles than arrival counters.
bool stream_k_ok(const Variant &v, int m, int n, int num_cu) {
    const long t = (long)ceil_div(m, v.bm) * ceil_div(n, v.bn);
    return v.streamk && t >= num_cu && t <= kMaxStreamKTiles;
}

// Plans measured on one MI355X by the tuner (python -m radeonflow_kernels_amd.tuner.gemm_tuner --all --emit).
// The role of the reference's DISPATCH_GEMM table (src/gemm/gemm_launcher.cpp:229-259), except that a shape
// outside the table is not an error: it gets the heuristic below.
const TunedPlan kTunedPlans[] = {
    {0, 0, 0, 0, 1, 1, 0},
#include "tuned_plans.inc"
};

constexpr int kTunedOnCUs = 256;

// Heuristic plan for shapes without a measured entry. Inputs: shape and CU count.
void select_config(int m, int n, int k, int num_cu, bool tiled_ok, const std::vector<TunedPlan> &user_plans,
                   rf_gemm_config *out) {
    out->split_k = 1;
    out->group_m = 8;
    out->stream_k = 0;
    if (!tiled_ok) {
        out->variant = -1;
        return;
    }
    auto usable = [&](const TunedPlan &p) {
        return p.m == m && p.n == n && p.k == k && p.variant < kNumVariants && p.split_k <= k / rf::BK &&
               (kVariants[p.variant].k_groups == 1 || (p.split_k == 1 && (k / rf::BK) % kVariants[p.variant].k_groups == 0)) &&
               (p.stream_k != RF_SCHEDULE_PERSISTENT || persistent_ok(kVariants[p.variant], m, n, k)) &&
               (p.stream_k != RF_SCHEDULE_STREAM_K || stream_k_ok(kVariants[p.variant], m, n, num_cu)) &&
               (p.stream_k != RF_SCHEDULE_PERSISTENT_HALF_TAIL || half_tail_ok(kVariants[p.variant], m, n, k, num_cu)) &&
               (p.stream_k != RF_SCHEDULE_SKINNY_K || skinny_ok(m, n, k));
    };
    const TunedPlan *hit = nullptr;
    for (const TunedPlan &p : user_plans)
        if (!hit && usable(p)) hit = &p;
    // the compiled-in table was measured on a device with kTunedOnCUs compute units: round counts, and with them the
    // best tile and split, change with the unit count, so another device takes the cost model below (which counts
    // rounds for the device at hand) unless the caller has loaded plans measured there
    if (num_cu == kTunedOnCUs)
        for (const TunedPlan &p : kTunedPlans)
            if (!hit && usable(p)) hit = &p;
    if (hit) {
        out->variant = hit->variant;
        out->split_k = hit->split_k;
        out->group_m = hit->group_m;
        out->stream_k = hit->stream_k;
        return;
    }
    // Up to four K blocks and a large C: the launch is a streaming store, which the skinny-K schedule does best
    // (measured against the best tiled plan at N = 7168, K = 256: 1024 rows 6.5 against 6.9 us, 2048 rows 7.8 against
    // 10.3, 6144 rows 18.2 against 22.1; below about six million outputs the 64 x 128 tiles win, e.g. 2048 x 2048: 6.5
    // against 5.6 us). Three and four K blocks (items of 64 rows): from two million outputs on; N = 4096, K = 512: 1024
    // rows 5.9 against 6.8 us, 4096 rows 12.3 against 13.8, 8192 rows 22.5 against 24.0; N = 7168, K = 384: 512 rows
    // 4.9 against 6.0, 6144 rows 25.7 against 31.8. With K = 512 and more than sixteen strips the tiled plans are as
    // fast or faster (N = 7168: 2048 rows 15.1 against 13.1 us, 6144 rows 30.6 against 30.4).
    if (skinny_ok(m, n, k) &&
        (k <= 2 * rf::BK ? (double)m * n >= 6.0e6
                         : (double)m * n >= 2.0e6 && (k == 3 * rf::BK || ceil_div(n, 256) <= 16))) {
        out->variant = 0;
        out->stream_k = RF_SCHEDULE_SKINNY_K;
        return;
    }
    // No measured entry: a cost model whose constants were searched on the tuner's measurements of the tabled shapes so
    // that its plan comes close to the best measured one. Searched on 213 shapes (the 163 of the table and 50 others,
    // 36 of them drawn at random with M = 16 ... 8192, N = 512 ... 8192, K = 128 ... 8192): 0.8 % slower than the best
    // measured plan on average, 10 % at worst. On shapes a search had not seen its constants were 1.7 to 1.9 % behind
    // on average and 8 to 16 % at worst (14, 60 and 36 shapes). The constants rank plans, they are not measured times.
    // Time in microseconds of a plan =
    //   rounds * (K blocks per workgroup * c + f)           one workgroup per tile and K split
    //   rounds * K blocks * c + f + (rounds - 1) * f_next   persistent: only the first tile starts cold
    //   the same over the whole rounds + f_next + K blocks * c + f of the three-stage 128x256 tile
    //                                                       persistent with a last round of half tiles (the half
    //                                                       tiles start cold: at K = 512 the plain persistent
    //                                                       schedule of 128x256 tiles is 15-20 % faster)
    //   + reduction cost when K is split
    // with rounds = ceil(workgroups / CUs). Candidates: the 256x256 tile and the 128x256, 192x192, 128x192 and 64x128
    // tiles with two and with three stages (192-wide tiles win where they divide the shape into fuller rounds or leave
    // no padded columns, e.g. N = 576, 1536 or 3072; the 64x128 tile where M is short or the whole problem is a few
    // microseconds); the others never won by more than a few percent.
    struct Candidate { int variant; double c, f; };
    // (variants 12 and 13 split K between two wave groups of one workgroup: half the K blocks per group, one launch, no
    // reduction term. Variant 12, the 64 x 128 tile: the best plan of short shapes, M <= 512, with K = 512 ... 2304.
    // Variant 13, the 128 x 128 tile: the best plan where 128 x 128 tiles fill one round, e.g. 1024 x 3072 x 1536,
    // 512 x 7168 x 2048)
    const Candidate cands[] = {{0, 0.905, 5.96}, {3, 0.679, 3.61}, {5, 0.80, 5.8},  {6, 0.74, 4.3},  {7, 0.85, 0.3},
                               {8, 0.52, 4.2},   {9, 0.73, 0.5},   {10, 0.53, 5.9}, {11, 0.71, 7.0}, {12, 0.93, 1.4},
                               {13, 1.06, 3.3}};
    const double f_next = 3.3, reduce_fixed = 6.03, reduce_per_elem = 1.27e-6, c_half_tile = 0.47, f_half_tile = 5.2;
    const int splits_tried[] = {1, 2, 3, 4, 6, 8, 12, 16};
    const int qk = k / rf::BK;
    double best_cost = 1e30;
    for (const Candidate &cd : cands) {
        const Variant &v = kVariants[cd.variant];
        const long tiles = (long)ceil_div(m, v.bm) * ceil_div(n, v.bn);
        for (int sp : splits_tried) {
            if (sp > qk) break;
            if (v.k_groups > 1) {
                if (sp != 1 || qk % v.k_groups != 0) continue;
                const double t = (double)((tiles + num_cu - 1) / num_cu) * (qk / v.k_groups * cd.c + cd.f);
                if (t < best_cost) {
                    best_cost = t;
                    out->variant = cd.variant;
                    out->split_k = 1;
                    out->stream_k = RF_SCHEDULE_TILES;
                }
                continue;
            }
            const int kb_per = ceil_div(qk, sp), splits = ceil_div(qk, kb_per);
            const long rounds = (tiles * splits + num_cu - 1) / num_cu;
            for (int sched : {RF_SCHEDULE_TILES, RF_SCHEDULE_PERSISTENT}) {
                if (sched == RF_SCHEDULE_PERSISTENT && (splits != 1 || !persistent_ok(v, m, n, k))) continue;
                double t = sched == RF_SCHEDULE_PERSISTENT ? rounds * kb_per * cd.c + cd.f + (rounds - 1) * f_next
                                                           : rounds * (kb_per * cd.c + cd.f);
                if (splits > 1) t += reduce_fixed + reduce_per_elem * splits * (double)m * n;
                if (t < best_cost) {
                    best_cost = t;
                    out->variant = cd.variant;
                    out->split_k = sp;
                    out->stream_k = sched;
                }
                if (sched == RF_SCHEDULE_PERSISTENT && half_tail_ok(v, m, n, k, num_cu)) {
                    t = (rounds - 1) * kb_per * cd.c + cd.f + (rounds - 1) * f_next + kb_per * c_half_tile + f_half_tile;
                    if (t < best_cost) {
                        best_cost = t;
                        out->variant = cd.variant;
                        out->split_k = 1;
                        out->stream_k = RF_SCHEDULE_PERSISTENT_HALF_TAIL;
                    }
                }
            }
        }
    }
}

// The launch proper; the caller holds the lock and has checked shape and pointers. m_store >= 0: c has only m_store
// (<= m) rows, the rest of the m rows of the operands are padding (one workgroup per tile schedules only).
int launch_locked(State &s, Mem &mem, const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n,
                  int k, const rf_gemm_config *user_cfg, hipStream_t stream, int m_store = -1) {
    int rc = RF_OK;
    if (m_store < 0) m_store = m;
    const bool tiled_ok = tiled_path_ok(a, b, c, m, n);
    rf_gemm_config cfg;
    if (user_cfg) {
        cfg = *user_cfg;
        if (cfg.variant >= kNumVariants || cfg.variant < -1 || cfg.split_k < 1 || cfg.group_m < 1 ||
            cfg.split_k > k / rf::BK || (cfg.variant >= 0 && !tiled_ok) || (cfg.variant < 0 && cfg.split_k != 1) ||
            (cfg.stream_k != 0 && (cfg.variant < 0 || cfg.split_k != 1)))
            return fail(RF_ERR_BAD_CONFIG, "configuration not usable for this shape");
        if (cfg.variant >= 0 && kVariants[cfg.variant].k_groups > 1 &&
            (cfg.split_k != 1 || cfg.stream_k != RF_SCHEDULE_TILES || (k / rf::BK) % kVariants[cfg.variant].k_groups != 0))
            return fail(RF_ERR_BAD_CONFIG, "this variant splits K inside the workgroup: it needs split_k == 1, the tile "
                                           "schedule and a number of K blocks that its wave groups divide");
        if (cfg.stream_k == RF_SCHEDULE_STREAM_K) {
            const Variant &sv = kVariants[cfg.variant];
            if (!sv.streamk) return fail(RF_ERR_BAD_CONFIG, "this variant has no stream_k form");
            if (!stream_k_ok(sv, m, n, s.num_cu))
                return fail(RF_ERR_BAD_CONFIG, "stream_k needs at least as many tiles as compute units");
        } else if (cfg.stream_k == RF_SCHEDULE_PERSISTENT) {
            if (!persistent_ok(kVariants[cfg.variant], m, n, k))
                return fail(RF_ERR_BAD_CONFIG, "the persistent schedule needs M >= the tile height, M % 16 == 0, N a multiple of the tile width and K/128 even");
        } else if (cfg.stream_k == RF_SCHEDULE_PERSISTENT_HALF_TAIL) {
            if (!half_tail_ok(kVariants[cfg.variant], m, n, k, s.num_cu))
                return fail(RF_ERR_BAD_CONFIG, "the half-tile schedule needs the 256x256 tile, the persistent schedule's "
                                               "shape rules, at least one tile per compute unit and a last round that "
                                               "is at most half full");
        } else if (cfg.stream_k == RF_SCHEDULE_SKINNY_K) {
            if (cfg.variant != 0 || !skinny_ok(m, n, k))
                return fail(RF_ERR_BAD_CONFIG, "the skinny-K schedule needs variant 0, K = 128 ... 512, M a multiple of 16 and N a multiple of 64");
        } else if (cfg.stream_k != RF_SCHEDULE_TILES) {
            return fail(RF_ERR_BAD_CONFIG, "unknown schedule");
        }
    } else {
        select_config(m, n, k, s.num_cu, tiled_ok, shared().user_plans, &cfg);
    }

    if (mem.fixed && cfg.variant >= 0) {
        // rf_fp8_gemm_static: the plan has to live inside what is left of the static array. A stream-K plan (only a
        // plan file can name one) is replaced by the cost model's plan; a K split whose partial sums do not fit is cut
        // down to the number of parts that do, a single part needing no scratch memory at all.
        if (cfg.stream_k == RF_SCHEDULE_STREAM_K) select_config(m, n, k, s.num_cu, true, std::vector<TunedPlan>(), &cfg);
        if (cfg.stream_k == RF_SCHEDULE_STREAM_K) cfg.stream_k = RF_SCHEDULE_TILES;
        if (cfg.split_k > 1) {
            const size_t per_part = (size_t)m * n * sizeof(float);
            const int qk_ = k / rf::BK, kb_per = ceil_div(qk_, cfg.split_k), parts = ceil_div(qk_, kb_per);
            const size_t fit = mem.fixed_left() / per_part;
            if ((size_t)parts > fit) cfg.split_k = fit < 2 ? 1 : (int)fit;
        }
    }
    if (m_store != m && (cfg.variant < 0 || cfg.stream_k == RF_SCHEDULE_STREAM_K))
        return fail(RF_ERR_BAD_CONFIG, "internal: this schedule cannot write fewer rows than it computes");
    if (cfg.variant < 0) {
        dim3 grid(ceil_div(n, 16), ceil_div(m, 16));
        hipLaunchKernelGGL(rf::gemm_fp8_blockscale_checked, grid, dim3(64), 0, stream, (const uint8_t *)a,
                           (const uint8_t *)b, as, bs, (uint16_t *)c, m, m, n, k);
        RF_HIP(hipGetLastError());
        return RF_OK;
    }

    const Variant &v = kVariants[cfg.variant];
    const int tiles_m = ceil_div(m, v.bm), tiles_n = ceil_div(n, v.bn);
    const int qk = k / rf::BK;
    const int kb_per_split = ceil_div(qk, cfg.split_k);
    const int splits = ceil_div(qk, kb_per_split);          // every split owns at least one K block
    dim3 grid(tiles_m * tiles_n, splits);
    dim3 block(v.threads());
    if (cfg.stream_k == RF_SCHEDULE_PERSISTENT) {
        // as many resident workgroups as the LDS of a CU holds (small tiles: two or three per CU, so that one's
        // store drain overlaps another's compute)
        const int T = tiles_m * tiles_n;
        int per_cu = (160 * 1024) / v.lds_persistent;
        if (per_cu > 2048 / v.threads()) per_cu = 2048 / v.threads();
        const int P = s.num_cu * (per_cu < 1 ? 1 : per_cu);
        hipLaunchKernelGGL(v.persistent, dim3(T < P ? T : P), block, v.lds_persistent, stream,
                           (const uint8_t *)a, (const uint8_t *)b, as, bs, (uint16_t *)c, m, n, k, tiles_m, tiles_n,
                           cfg.group_m, m_store);
        RF_HIP(hipGetLastError());
        return RF_OK;
    }
    if (cfg.stream_k == RF_SCHEDULE_SKINNY_K) {
        // one strip of 256 columns per workgroup, and as many workgroups per strip as fill the chip once (each takes a
        // share of the strip's rows, in units of 64)
        const int strips = ceil_div(n, 256), units = ceil_div(m, 64);
        int per_strip = s.num_cu / strips;
        per_strip = per_strip < 1 ? 1 : per_strip > units ? units : per_strip;
#define RF_LAUNCH_SKINNY(QK)                                                                                            \
    hipLaunchKernelGGL(rf::gemm_fp8_blockscale_skinny<QK>, dim3(strips * per_strip), dim3(512),                         \
                       rf::SkinnyGeom<QK>::LDS_BYTES, stream, (const uint8_t *)a, (const uint8_t *)b, as, bs,           \
                       (uint16_t *)c, m, n, per_strip, m_store)
        if (qk == 1) RF_LAUNCH_SKINNY(1);
        else if (qk == 2) RF_LAUNCH_SKINNY(2);
        else if (qk == 3) RF_LAUNCH_SKINNY(3);
        else RF_LAUNCH_SKINNY(4);
#undef RF_LAUNCH_SKINNY
        RF_HIP(hipGetLastError());
        return RF_OK;
    }
    if (cfg.stream_k == RF_SCHEDULE_PERSISTENT_HALF_TAIL) {
        hipLaunchKernelGGL(v.persistent_half_tail, dim3(s.num_cu), block, v.lds_persistent, stream, (const uint8_t *)a,
                           (const uint8_t *)b, as, bs, (uint16_t *)c, m, n, k, tiles_m, tiles_n, cfg.group_m, m_store);
        RF_HIP(hipGetLastError());
        return RF_OK;
    }
    if (cfg.stream_k == RF_SCHEDULE_STREAM_K) {
        const int P = s.num_cu;
        unsigned *tile_count = nullptr;
        float *ws = nullptr;
        rc = mem.tile_counters(&tile_count);
        if (rc != RF_OK) return rc;
        rc = mem.workspace((size_t)2 * P * v.bm * v.bn * sizeof(float), &ws);
        if (rc != RF_OK) return rc;
        hipLaunchKernelGGL(v.streamk, dim3(P), block, v.lds_bytes(), stream, (const uint8_t *)a, (const uint8_t *)b, as,
                           bs, (uint16_t *)c, m, n, k, tiles_m, tiles_n, cfg.group_m, tile_count, ws);
        RF_HIP(hipGetLastError());
        return RF_OK;
    }
    if (splits == 1) {
        hipLaunchKernelGGL(v.direct, grid, block, v.lds_bytes(), stream, (const uint8_t *)a, (const uint8_t *)b, as, bs,
                           c, m, n, k, kb_per_split, tiles_m, tiles_n, cfg.group_m, m_store);
        RF_HIP(hipGetLastError());
    } else {
        const size_t mn = (size_t)m * n;
        float *ws = nullptr;
        rc = mem.workspace(mn * splits * sizeof(float), &ws);
        if (rc != RF_OK) return rc;
        hipLaunchKernelGGL(v.partial, grid, block, v.lds_bytes(), stream, (const uint8_t *)a, (const uint8_t *)b, as,
                           bs, (void *)ws, m, n, k, kb_per_split, tiles_m, tiles_n, cfg.group_m, m);
        RF_HIP(hipGetLastError());
        const size_t mn_store = (size_t)m_store * n;
        hipLaunchKernelGGL(rf::reduce_splitk_bf16, dim3((unsigned)((mn_store / 4 + 255) / 256)), dim3(256), 0, stream,
                           (const float *)ws, (uint16_t *)c, mn_store, splits, mn);
        RF_HIP(hipGetLastError());
    }
    return RF_OK;
}

// ---- shapes and pointers the tiled kernels do not take as they are ----
// M or N not a multiple of 16 (or below 16), or operands that are not 16-byte aligned, would leave the whole GEMM to
// the bounds-checked kernel, which is 7 to 35 times slower (M = 100, N = 4096, K = 7168: 129 us against 17 us for
// M = 112). Token counts are arbitrary in practice, so for anything but tiny problems the operands that need it are
// copied into a staging buffer with rows padded to a multiple of 16 (zeros: padded rows and columns produce values
// nobody reads), the tiled kernels run on the padded shape under the automatic plan, and C is copied back without the
// padding. b_scale needs no copy: ceil(N/128) does not change. The copies cost K*M (+ K*N when N is ragged) bytes.
constexpr double kPadThresholdMacs = 2097152.0;            // below this the bounds-checked kernel is as fast

// The grouped GEMM's staging copy: the caller's [rows][m_total] matrix (A with T = bytes, a_scale with T = float), in
// which group g owns columns out_row_start[g] .. out_row_start[g+1]-1, is copied to [rows][m_pad] with group g starting
// at column row_start[g], a multiple of 16; the columns between a group's end and the next start become zero.
// A workgroup writes 256 consecutive 16-byte pieces of kPadRows consecutive rows, whatever groups they belong to, so
// both sides of the copy move whole cache lines even when the groups are a few rows each. The groups that overlap the
// workgroup's columns are found with uniform (scalar) reads of the table; each thread then keeps the last one that
// starts at or before its column. Bytes are fetched as the aligned words that hold them and shifted into place: a
// source piece starts at any byte.
constexpr int kPadRows = 4;
template <typename T>
__device__ __forceinline__ void pad_group_rows_body(const T *__restrict__ src, int m_total, int m_pad, int rows, int groups,
                                                    T *__restrict__ dst, const rf::GroupTable &table, int block_row,
                                                    int block_chunk) {
    constexpr int PER = 16 / sizeof(T);
    if (block_chunk * 256 * PER >= m_pad) return;
    const int c_lo = block_chunk * 256 * PER, c_hi = (c_lo + 256 * PER < m_pad ? c_lo + 256 * PER : m_pad) - 1;
    auto last_group_starting_by = [&](int c) {                       // uniform binary search
        int lo = 0, hi = groups;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (table.row_start[mid] <= c) lo = mid; else hi = mid;
        }
        return lo;
    };
    const int g_lo = last_group_starting_by(c_lo), g_hi = last_group_starting_by(c_hi);
    const int col = c_lo + (int)threadIdx.x * PER;
    int start = table.row_start[g_lo], from = table.out_row_start[g_lo], count = table.out_row_start[g_lo + 1] - from;
    for (int g = g_lo + 1; g <= g_hi; g++) {
        const int s2 = table.row_start[g], f2 = table.out_row_start[g], n2 = table.out_row_start[g + 1] - f2;
        if (col >= s2) { start = s2; from = f2; count = n2; }
    }
    if (col >= m_pad) return;
    int valid = count - (col - start);                                 // columns of this piece that exist in the source
    valid = valid < 0 ? 0 : valid > PER ? PER : valid;
    const int r_first = block_row * kPadRows;
    const T *p0 = src + (size_t)r_first * m_total + from + (col - start);
    uint32_t w[kPadRows][5];
    int shift[kPadRows];
#pragma unroll
    for (int u = 0; u < kPadRows; u++) {
        const T *p = p0 + (size_t)u * m_total;
        shift[u] = 0;
        if (r_first + u < rows) {
            if constexpr (sizeof(T) == 4) {
#pragma unroll
                for (int e = 0; e < 4; e++) w[u][e] = e < valid ? ((const uint32_t *)p)[e] : 0u;
            } else {
                shift[u] = (int)((uintptr_t)p & 3);
                const int need = valid ? shift[u] + valid : 0;
                const uint32_t *q = (const uint32_t *)((const uint8_t *)p - shift[u]);
#pragma unroll
                for (int e = 0; e < 5; e++) w[u][e] = 4 * e < need ? q[e] : 0u;   // only words that hold a wanted byte
            }
        }
    }
#pragma unroll
    for (int u = 0; u < kPadRows; u++) {
        if (r_first + u >= rows) continue;
        uint32_t out[4];
        if constexpr (sizeof(T) == 4) {
#pragma unroll
            for (int e = 0; e < 4; e++) out[e] = w[u][e];
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                out[e] = __builtin_amdgcn_alignbyte(w[u][e + 1], w[u][e], shift[u]);
                const int nv = valid - 4 * e;
                if (nv < 4) out[e] = nv <= 0 ? 0u : out[e] & ((1u << (8 * nv)) - 1u);
            }
        }
        *(uint4 *)(dst + (size_t)(r_first + u) * m_pad + col) = make_uint4(out[0], out[1], out[2], out[3]);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void pad_group_rows(const T *__restrict__ src, int m_total, int m_pad, int rows,
                                                      int groups, T *__restrict__ dst, const rf::GroupTable table) {
    pad_group_rows_body<T>(src, m_total, m_pad, rows, groups, dst, table, blockIdx.x, blockIdx.y);
}

// A and a_scale in one launch (they are staged together whenever M or the group sizes are ragged): the first
// blocks_a workgroups along x copy the bytes of A, the others the floats of a_scale.
__global__ __launch_bounds__(256) void pad_group_rows_a_and_scales(const uint8_t *__restrict__ a, const float *__restrict__ as,
                                                                   int m_total, int m_pad, int k, int groups,
                                                                   uint8_t *__restrict__ a_dst, float *__restrict__ as_dst,
                                                                   int blocks_a, const rf::GroupTable table) {
    if ((int)blockIdx.x < blocks_a)
        pad_group_rows_body<uint8_t>(a, m_total, m_pad, k, groups, a_dst, table, blockIdx.x, blockIdx.y);
    else
        pad_group_rows_body<float>(as, m_total, m_pad, k / rf::BK, groups, as_dst, table, blockIdx.x - blocks_a, blockIdx.y);
}

// grid of pad_group_rows for `rows` rows of m_pad elements of `size` bytes
dim3 pad_grid(int m_pad, int size, int rows) {
    const int pieces = m_pad / (16 / size);
    return dim3((unsigned)((rows + kPadRows - 1) / kPadRows), (unsigned)((pieces + 255) / 256));     // rows on x: no 65535 limit
}

// Stages A and a_scale with one launch.
void launch_pad_a_and_scales(const void *a, const float *as, int m_total, int m_pad, int k, int groups, uint8_t *a_dst,
                             float *as_dst, const rf::GroupTable &table, hipStream_t stream) {
    const dim3 ga = pad_grid(m_pad, 1, k), gs = pad_grid(m_pad, 4, k / rf::BK);
    hipLaunchKernelGGL(pad_group_rows_a_and_scales, dim3(ga.x + gs.x, ga.y > gs.y ? ga.y : gs.y), dim3(256), 0, stream,
                       (const uint8_t *)a, as, m_total, m_pad, k, groups, a_dst, as_dst, (int)ga.x, table);
}

// table of one group of `cols` columns padded to `cols_pad`
rf::GroupTable one_group(int cols, int cols_pad) {
    rf::GroupTable t;
    t.row_start[0] = t.out_row_start[0] = t.tile_start[0] = 0;
    for (int g = 1; g <= rf::kMaxGroups; g++) {
        t.row_start[g] = cols_pad;
        t.out_row_start[g] = cols;
        t.tile_start[g] = 0;
    }
    return t;
}

// rf_fp8_gemm_static on a ragged or unaligned shape whose staging copies do not fit the static array as a whole: the
// rows of the problem are cut into pieces (row ranges of A, a_scale and C are independent GEMMs), each piece is staged,
// computed and, where C is staged too, copied back before the next one re-uses the same memory; the stream orders them.
// The staged copy of B (ragged N or an unaligned b) is shared by all pieces and has to fit beside them: when it takes
// more than half of the array, the bounds-checked kernel computes the whole problem in place instead.
int launch_padded_in_pieces(State &s, Mem &mem, const void *a, const void *b, const float *as, const float *bs, void *c,
                            int m, int n, int k, hipStream_t stream) {
    auto pad16 = [](int x) { return x < 16 ? 16 : (x + 15) / 16 * 16; };
    auto align = [](size_t x) { return (x + 255) / 256 * 256; };
    const int np = pad16(n), qk = k / rf::BK;
    const bool copy_b = np != n || (uintptr_t)b % 16 != 0;
    const bool copy_c = np != n || (uintptr_t)c % 16 != 0;
    const size_t b_bytes = copy_b ? align((size_t)k * np) : 0;
    // per row of a piece: its bytes of A, of a_scale and (when C is staged) of C; a quarter of what is left after B is
    // kept for the piece's split-K partial sums (launch_locked cuts the split down to what fits)
    const size_t per_row = (size_t)k + (size_t)qk * sizeof(float) + (copy_c ? (size_t)np * 2 : 0);
    const size_t left = mem.fixed_left() > b_bytes ? mem.fixed_left() - b_bytes : 0;
    long rows_fit = (long)((left - left / 4) / per_row) / 16 * 16 - 16;
    if (b_bytes > mem.fixed_left() / 2 || rows_fit < 16) {
        hipLaunchKernelGGL(rf::gemm_fp8_blockscale_checked, dim3(ceil_div(n, 16), ceil_div(m, 16)), dim3(64), 0, stream,
                           (const uint8_t *)a, (const uint8_t *)b, as, bs, (uint16_t *)c, m, m, n, k);
        RF_HIP(hipGetLastError());
        return RF_OK;
    }
    int rc = RF_OK;
    const void *b2 = b;
    if (copy_b) {
        uint8_t *pb = nullptr;
        rc = mem.pad(b_bytes, &pb);
        if (rc != RF_OK) return rc;
        hipLaunchKernelGGL(pad_group_rows<uint8_t>, pad_grid(np, 1, k), dim3(256), 0, stream, (const uint8_t *)b, n, np, k, 1,
                           pb, one_group(n, np));
        RF_HIP(hipGetLastError());
        b2 = pb;
    }
    const size_t base = mem.fixed_used;
    const int pieces = ceil_div(m, (int)(rows_fit < m ? rows_fit : m));
    const int rows_per = (ceil_div(m, pieces) + 15) / 16 * 16;           // even pieces, whole m-tiles
    for (int r0 = 0; r0 < m; r0 += rows_per) {
        const int rows = m - r0 < rows_per ? m - r0 : rows_per, rp = pad16(rows);
        mem.fixed_used = base;                                            // the pieces take turns in the same memory
        uint8_t *pa = nullptr, *psa = nullptr, *pc = nullptr;
        if ((rc = mem.pad(align((size_t)k * rp), &pa)) != RF_OK) return rc;
        if ((rc = mem.pad(align((size_t)qk * rp * sizeof(float)), &psa)) != RF_OK) return rc;
        if (copy_c && (rc = mem.pad(align((size_t)rp * np * 2), &pc)) != RF_OK) return rc;
        // columns r0 .. r0 + rows - 1 of the caller's [K][m] matrices, padded to rp columns
        launch_pad_a_and_scales((const uint8_t *)a + r0, as + r0, m, rp, k, 1, pa, (float *)psa, one_group(rows, rp), stream);
        RF_HIP(hipGetLastError());
        rf_gemm_config cfg;
        select_config(rp, np, k, s.num_cu, true, shared().user_plans, &cfg);
        void *c_piece = copy_c ? (void *)pc : (void *)((uint16_t *)c + (size_t)r0 * n);
        rc = launch_locked(s, mem, pa, b2, (const float *)psa, bs, c_piece, rp, np, k, &cfg, stream, copy_c ? rp : rows);
        if (rc != RF_OK) return rc;
        if (copy_c)
            RF_HIP(hipMemcpy2DAsync((uint16_t *)c + (size_t)r0 * n, (size_t)n * 2, pc, (size_t)np * 2, (size_t)n * 2, rows,
                                    hipMemcpyDeviceToDevice, stream));
    }
    return RF_OK;
}

int launch_padded(State &s, Mem &mem, const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n,
                  int k, hipStream_t stream) {
    auto pad16 = [](int x) { return x < 16 ? 16 : (x + 15) / 16 * 16; };
    auto align = [](size_t x) { return (x + 255) / 256 * 256; };
    const int mp = pad16(m), np = pad16(n), qk = k / rf::BK;
    const bool copy_a = mp != m || (uintptr_t)a % 16 != 0, copy_b = np != n || (uintptr_t)b % 16 != 0;
    const bool copy_sa = mp != m;
    // The plan of the padded shape. With whole columns and an aligned c, the whole-tile schedules (one workgroup per
    // tile, persistent) write the m true rows straight into c (their stores are masked by row); otherwise C is staged
    // and copied back.
    rf_gemm_config cfg;
    select_config(mp, np, k, s.num_cu, true, shared().user_plans, &cfg);
    const bool copy_c = np != n || (uintptr_t)c % 16 != 0 || (mp != m && cfg.stream_k == RF_SCHEDULE_STREAM_K);
    size_t off = 0;
    const size_t off_a = off;  off += copy_a ? align((size_t)k * mp) : 0;
    const size_t off_b = off;  off += copy_b ? align((size_t)k * np) : 0;
    const size_t off_sa = off; off += copy_sa ? align((size_t)qk * mp * sizeof(float)) : 0;
    const size_t off_c = off;  off += copy_c ? align((size_t)mp * np * 2) : 0;
    if (mem.fixed && off > mem.fixed_left()) return launch_padded_in_pieces(s, mem, a, b, as, bs, c, m, n, k, stream);
    uint8_t *pad = nullptr;
    int rc = mem.pad(off, &pad);
    if (rc != RF_OK) return rc;
    const void *a2 = a, *b2 = b;
    const float *as2 = as;
    void *c2 = c;
    if (copy_a && copy_sa) {
        launch_pad_a_and_scales(a, as, m, mp, k, 1, pad + off_a, (float *)(pad + off_sa), one_group(m, mp), stream);
        a2 = pad + off_a;
        as2 = (const float *)(pad + off_sa);
    } else if (copy_a) {                                   // M is fine, only the pointer is not aligned
        hipLaunchKernelGGL(pad_group_rows<uint8_t>, pad_grid(mp, 1, k), dim3(256), 0, stream, (const uint8_t *)a, m, mp, k, 1,
                           pad + off_a, one_group(m, mp));
        a2 = pad + off_a;
    }
    if (copy_b) {
        hipLaunchKernelGGL(pad_group_rows<uint8_t>, pad_grid(np, 1, k), dim3(256), 0, stream, (const uint8_t *)b, n, np, k, 1,
                           pad + off_b, one_group(n, np));
        b2 = pad + off_b;
    }
    if (copy_c) c2 = pad + off_c;
    RF_HIP(hipGetLastError());
    rc = launch_locked(s, mem, a2, b2, as2, bs, c2, mp, np, k, &cfg, stream, copy_c ? mp : m);
    if (rc != RF_OK) return rc;
    if (copy_c)
        RF_HIP(hipMemcpy2DAsync(c, (size_t)n * 2, c2, (size_t)np * 2, (size_t)n * 2, m, hipMemcpyDeviceToDevice, stream));
    return RF_OK;
}

int launch(const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n, int k,
           const rf_gemm_config *user_cfg, hipStream_t stream, bool static_memory = false) {
    g_last_error.clear();
    if (m < 1 || n < 1 || k < rf::BK || k % rf::BK != 0)
        return fail(RF_ERR_BAD_SHAPE, "unsupported shape M=" + std::to_string(m) + " N=" + std::to_string(n) +
                                          " K=" + std::to_string(k) + " (need M,N>=1, K a positive multiple of 128)");
    if (!a || !b || !as || !bs || !c) return fail(RF_ERR_NULL_POINTER, "null device pointer");
    State &s = state();
    std::lock_guard<std::mutex> lock(shared().mu);
    int rc = ensure_device_info(s);
    if (rc != RF_OK) return rc;
    Mem mem{s};
    mem.stream = stream;
    if (static_memory) mem.fixed = s.static_scratch;
    if (!user_cfg && !tiled_path_ok(a, b, c, m, n) && (double)m * n * k >= kPadThresholdMacs)
        return launch_padded(s, mem, a, b, as, bs, c, m, n, k, stream);
    return launch_locked(s, mem, a, b, as, bs, c, m, n, k, user_cfg, stream);
}

// ---- timing record for run() ----------------------------------------------------------------
struct TimerJob {
    hipEvent_t start, stop;
    double flop;
    float *time_ms, *gflops;
    State *owner;                        // the device state whose event pool the pair came from
};
void timer_callback(hipStream_t, hipError_t status, void *user) {
    TimerJob *job = static_cast<TimerJob *>(user);
    if (status == hipSuccess) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, job->start, job->stop) == hipSuccess) {
            if (job->time_ms) *job->time_ms = ms;
            if (job->gflops) *job->gflops = (float)(job->flop / (ms * 1e-3) / 1e9);
        }
    }
    State &s = *job->owner;               // the callback thread has no current device of its own
    {
        // the pool has a lock of its own: the launch path may hold the library lock while it waits for the device,
        // and the device may be waiting for this callback
        std::lock_guard<std::mutex> lock(s.ev_mu);
        s.free_events.emplace_back(job->start, job->stop);   // recycled, unlike the reference's growing list
    }
    delete job;
}

}  // namespace

extern "C" {

int rf_fp8_gemm(const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n, int k,
                hipStream_t stream) {
    return launch(a, b, as, bs, c, m, n, k, nullptr, stream);
}

int rf_fp8_gemm_static(const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n, int k,
                       hipStream_t stream) {
    return launch(a, b, as, bs, c, m, n, k, nullptr, stream, /*static_memory=*/true);
}

size_t rf_gemm_static_scratch_bytes(void) { return kStaticScratchBytes; }

int rf_fp8_gemm_ex(const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n, int k,
                   const rf_gemm_config *cfg, hipStream_t stream) {
    return launch(a, b, as, bs, c, m, n, k, cfg, stream);
}

int rf_fp8_gemm_time(const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n, int k,
                     const rf_gemm_config *cfg, int warmup, int iters, float *us_per_launch, hipStream_t stream) {
    if (!us_per_launch || iters < 1 || warmup < 0) {
        g_last_error.clear();
        return fail(RF_ERR_BAD_CONFIG, "rf_fp8_gemm_time needs iters >= 1, warmup >= 0 and a result pointer");
    }
    for (int i = 0; i < warmup; i++) {
        int rc = launch(a, b, as, bs, c, m, n, k, cfg, stream);
        if (rc != RF_OK) return rc;
    }
    hipEvent_t e0, e1;
    RF_HIP(hipEventCreate(&e0));
    RF_HIP(hipEventCreate(&e1));
    int rc = RF_OK;
    hipError_t err = hipEventRecord(e0, stream);
    for (int i = 0; i < iters && rc == RF_OK && err == hipSuccess; i++) rc = launch(a, b, as, bs, c, m, n, k, cfg, stream);
    if (err == hipSuccess) err = hipEventRecord(e1, stream);
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    float ms = 0.f;
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (rc != RF_OK) return rc;
    if (err != hipSuccess) return fail(RF_ERR_HIP, std::string("rf_fp8_gemm_time: ") + hipGetErrorString(err));
    *us_per_launch = ms * 1e3f / iters;
    return RF_OK;
}

int rf_gemm_select_config(int m, int n, int k, rf_gemm_config *out) {
    g_last_error.clear();
    if (!out) return fail(RF_ERR_NULL_POINTER, "out is null");
    if (m < 1 || n < 1 || k < rf::BK || k % rf::BK != 0) return fail(RF_ERR_BAD_SHAPE, "unsupported shape");
    State &s = state();
    std::lock_guard<std::mutex> lock(shared().mu);
    int rc = ensure_device_info(s);
    if (rc != RF_OK) return rc;
    const bool tiled = m >= 16 && n >= 16 && m % 16 == 0 && n % 16 == 0;
    if (!tiled && (double)m * n * k >= kPadThresholdMacs) {
        // the launch pads such a shape to multiples of 16 and plans for the padded shape (see launch_padded)
        m = m < 16 ? 16 : (m + 15) / 16 * 16;
        n = n < 16 ? 16 : (n + 15) / 16 * 16;
        select_config(m, n, k, s.num_cu, true, shared().user_plans, out);
        return RF_OK;
    }
    select_config(m, n, k, s.num_cu, tiled, shared().user_plans, out);
    return RF_OK;
}

int rf_gemm_plan_for(int m, int n, int k, int num_cu, rf_gemm_config *out) {
    g_last_error.clear();
    if (!out) return fail(RF_ERR_NULL_POINTER, "out is null");
    if (m < 1 || n < 1 || k < rf::BK || k % rf::BK != 0 || num_cu < 1) return fail(RF_ERR_BAD_SHAPE, "unsupported shape");
    std::lock_guard<std::mutex> lock(shared().mu);
    const bool tiled = m >= 16 && n >= 16 && m % 16 == 0 && n % 16 == 0;
    if (!tiled && (double)m * n * k >= kPadThresholdMacs) {
        m = m < 16 ? 16 : (m + 15) / 16 * 16;
        n = n < 16 ? 16 : (n + 15) / 16 * 16;
        select_config(m, n, k, num_cu, true, shared().user_plans, out);
        return RF_OK;
    }
    select_config(m, n, k, num_cu, tiled, shared().user_plans, out);
    return RF_OK;
}

int rf_gemm_load_plans(const char *path, int *count) {
    g_last_error.clear();
    if (!path) return fail(RF_ERR_NULL_POINTER, "path is null");
    std::lock_guard<std::mutex> lock(shared().mu);
    const size_t before = shared().user_plans.size();
    int rc = parse_plans(path, shared().user_plans);
    if (rc != RF_OK) return rc;
    if (count) *count = (int)(shared().user_plans.size() - before);
    return RF_OK;
}

void rf_gemm_clear_plans(void) {
    std::lock_guard<std::mutex> lock(shared().mu);
    shared().user_plans.clear();
}

int rf_gemm_num_variants(void) { return kNumVariants; }

int rf_gemm_variant_info(int variant, int *block_m, int *block_n, int *waves_m, int *waves_n, int *lds_bytes) {
    if (variant < 0 || variant >= kNumVariants) return RF_ERR_BAD_CONFIG;
    const Variant &v = kVariants[variant];
    if (block_m) *block_m = v.bm;
    if (block_n) *block_n = v.bn;
    if (waves_m) *waves_m = v.waves_m;
    if (waves_n) *waves_n = v.waves_n;
    if (lds_bytes) *lds_bytes = v.lds_bytes();
    return RF_OK;
}

int rf_gemm_variant_k_groups(int variant) {
    return variant >= 0 && variant < kNumVariants ? kVariants[variant].k_groups : 0;
}

int rf_gemm_variant_has_persistent(int variant) {
    return variant >= 0 && variant < kNumVariants && kVariants[variant].persistent != nullptr;
}

int rf_gemm_variant_has_stream_k(int variant) {
    return variant >= 0 && variant < kNumVariants && kVariants[variant].streamk != nullptr;
}

size_t rf_gemm_workspace_bytes(int m, int n, int k) {
    rf_gemm_config cfg;
    if (rf_gemm_select_config(m, n, k, &cfg) != RF_OK || cfg.variant < 0) return 0;
    // a ragged shape runs (and splits K) at its padded size; its staging copies live in a buffer of their own
    m = m < 16 ? 16 : (m + 15) / 16 * 16;
    n = n < 16 ? 16 : (n + 15) / 16 * 16;
    if (cfg.stream_k == RF_SCHEDULE_STREAM_K) {
        State &s = state();
        return (size_t)2 * s.num_cu * kVariants[cfg.variant].bm * kVariants[cfg.variant].bn * sizeof(float);
    }
    if (cfg.split_k <= 1) return 0;
    const int qk = k / rf::BK;
    const int kb_per_split = ceil_div(qk, cfg.split_k);
    return (size_t)m * n * sizeof(float) * ceil_div(qk, kb_per_split);
}

int rf_gemm_init(size_t workspace_bytes) {
    g_last_error.clear();
    State &s = state();
    std::lock_guard<std::mutex> lock(shared().mu);
    int rc = ensure_device_info(s);
    if (rc != RF_OK) return rc;
    if (workspace_bytes == 0) return RF_OK;
    // a buffer set that belongs to no stream yet: the first stream that needs one takes it over
    StreamBuffers *sb = nullptr;
    rc = buffers_of(s, (hipStream_t)kUnboundStream, &sb);
    if (rc != RF_OK) return rc;
    Mem mem{s, sb};
    float *ws = nullptr;
    return mem.workspace(workspace_bytes, &ws);
}

void rf_gemm_destroy(void) {
    State &s = state();
    std::lock_guard<std::mutex> lock(shared().mu);
    if (!s.buffers.empty() || !s.retired.empty()) (void)hipDeviceSynchronize();   // launches may still use them
    for (StreamBuffers &b : s.buffers) {
        if (b.ws) (void)hipFree(b.ws);
        if (b.pad) (void)hipFree(b.pad);
        if (b.tile_count) (void)hipFree(b.tile_count);
    }
    s.buffers.clear();
    for (void *p : s.retired) (void)hipFree(p);
    s.retired.clear();
    std::lock_guard<std::mutex> ev_lock(s.ev_mu);
    for (auto &p : s.free_events) {
        (void)hipEventDestroy(p.first);
        (void)hipEventDestroy(p.second);
    }
    s.free_events.clear();
}

const char *rf_gemm_last_error(void) { return g_last_error.c_str(); }

}  // extern "C"

namespace {
// rows x K source (row-major, K contiguous) -> fp8 [K][rows] + scales; see quantize_kernels.h
template <bool PER_ROW, bool IN_BF16>
int launch_quantize(const void *x, int rows, int k, void *out, float *scales, hipStream_t stream) {
    g_last_error.clear();
    if (rows < 1 || k < rf::BK || k % rf::BK != 0)
        return fail(RF_ERR_BAD_SHAPE, "unsupported shape rows=" + std::to_string(rows) + " K=" + std::to_string(k) +
                                          " (need rows>=1, K a positive multiple of 128)");
    if (!x || !out || !scales) return fail(RF_ERR_NULL_POINTER, "null device pointer");
    if ((uintptr_t)x % 16 != 0 || (uintptr_t)scales % 4 != 0)
        return fail(RF_ERR_BAD_CONFIG, "source must be 16-byte aligned, scales 4-byte aligned");
    State &s = state();
    {
        std::lock_guard<std::mutex> lock(shared().mu);
        int rc = ensure_device_info(s);
        if (rc != RF_OK) return rc;
    }
    const bool vector_store = rows % 16 == 0 && (uintptr_t)out % 16 == 0;
    const int row_blocks = ceil_div(rows, 128);
    dim3 grid(k / rf::BK, row_blocks);
    hipLaunchKernelGGL((rf::quantize_block128<PER_ROW, IN_BF16>), grid, dim3(256), 0, stream, x, rows, k, (uint8_t *)out,
                       scales, PER_ROW ? rows : row_blocks, vector_store);
    RF_HIP(hipGetLastError());
    return RF_OK;
}
}  // namespace

namespace {
typedef void (*grouped_kernel_t)(const uint8_t *, const uint8_t *, const float *, const float *, uint16_t *, int, int, int,
                                 int, const rf::GroupTable);
struct GroupedVariant {
    int bm, bn, threads, lds;
    grouped_kernel_t kernel;
    bool mixed;          // 256-row tiles plus one shorter tile for what is left over (one 128-row tile for at most 128
                         // rows; the queue form: 64, 128, 192 or 256 rows)
    bool queue = false;  // resident workgroups that take tiles from per-XCD queues (gemm_fp8_blockscale_grouped_queue)
    // row tiles of a group of `rows` rows
    int tiles_m(int rows) const {
        if (!mixed) return ceil_div(rows, bm);
        return rows / 256 + (rows % 256 > 0 ? 1 : 0);
    }
};

#define RF_GROUPED(BM, BN, WM, WN, NS) \
    GroupedVariant { BM, BN, WM *WN * 64, rf::TileGeom<BM, BN, WM, WN, NS>::LDS_BYTES, rf::gemm_fp8_blockscale_grouped<BM, BN, WM, WN, NS>, false }
constexpr int kMixedLds = rf::TileGeom<256, 256, 2, 4>::LDS_BYTES > rf::TileGeom<128, 256, 2, 4, 3>::LDS_BYTES
                              ? rf::TileGeom<256, 256, 2, 4>::LDS_BYTES : rf::TileGeom<128, 256, 2, 4, 3>::LDS_BYTES;
const GroupedVariant kGroupedVariants[] = {
    RF_GROUPED(256, 256, 2, 4, 2), RF_GROUPED(128, 256, 2, 4, 3), RF_GROUPED(128, 128, 2, 2, 2), RF_GROUPED(128, 64, 2, 1, 2),
    GroupedVariant{256, 256, 512, kMixedLds, rf::gemm_fp8_blockscale_grouped_mixed, true},
    GroupedVariant{256, 256, 512, rf::kQueueLds, nullptr, true, true}};
constexpr int kGroupedMixed = 4, kGroupedQueue = 5;
// Estimated time of a 256-column tile of the queue form by its height in units of 64 rows, relative to a 256-row tile
constexpr double kQueueTileCost[5] = {0.0, 0.68, 0.75, 0.97, 1.0};
constexpr int kNumGroupedVariants = sizeof(kGroupedVariants) / sizeof(kGroupedVariants[0]);

long grouped_tiles(const GroupedVariant &v, const int *row_offsets, int groups, int n) {
    long t = 0;
    for (int g = 0; g < groups; g++) t += (long)v.tiles_m(row_offsets[g + 1] - row_offsets[g]) * ceil_div(n, v.bn);
    return t;
}
}  // namespace

namespace {
// The automatic choice of rf_fp8_gemm_grouped (variant = -1) for groups of these sizes on a device with num_cu compute units.
int choose_grouped_variant(const int *row_offsets, int groups, int n, int k, int num_cu) {
    // the largest tile that still gives every CU a workgroup; failing that, the one with the most workgroups
    int variant = -1;
    long most = -1;
    int most_v = 0;
    for (int v = 0; v < kNumGroupedVariants && variant < 0; v++) {
        const long t = grouped_tiles(kGroupedVariants[v], row_offsets, groups, n);
        if (t >= num_cu) variant = v;
        if (t > most) { most = t; most_v = v; }
    }
    if (variant < 0) variant = most_v;
    if (variant == 1) variant = 0;      // 128-row tiles fill the chip: the 256-wide family, chosen below
    // Enough tiles for the 256-wide family (128-row tiles would give every CU one): 256-row tiles, 128-row tiles
    // (three stages) or the mixed form, by a
    // small model of what was measured (N = 4096, K = 7168, twelve group layouts). A tile costs its compute
    // (91 for 256 rows, 52 for 128, arbitrary units) plus a share of streaming its column tile of the group's
    // weights (36, divided among the row tiles that use it: they run side by side on one XCD); the launch takes
    // as many rounds of one tile per CU as the tile count needs, a last partial round counting 0.6 + 0.4 x its
    // fill. Round counts decide most cases: 32 uneven groups of 16..816 rows are 816 mixed tiles (3.19 rounds,
    // 369 us) or 1280 tiles of 128 rows (5.00 rounds, 342 us); 20 groups of 384 rows 287 against 246 us; 64 groups
    // of 16..176 rows 408 against 447 us. On the twelve layouts the choice is 0.9 % slower than the best of the
    // three on average, 8 % at worst (always taking the mixed form: 2.6 % and 17 %).
    if (variant == 0) {
        const int tiles_n256 = ceil_div(n, 256);
        double best_t = 0;
        for (int cand : {0, 1, kGroupedMixed}) {
            double cost = 0;
            long items = 0;
            for (int g = 0; g < groups; g++) {
                const int rows = row_offsets[g + 1] - row_offsets[g];
                if (rows == 0) continue;
                int big, small;
                if (cand == 0) { big = ceil_div(rows, 256); small = 0; }
                else if (cand == 1) { big = 0; small = ceil_div(rows, 128); }
                else { big = rows / 256 + (rows % 256 > 128 ? 1 : 0); small = rows % 256 > 0 && rows % 256 <= 128 ? 1 : 0; }
                cost += tiles_n256 * (91.0 * big + 52.0 * small + 36.0);      // 36 / t for each of the t row tiles
                items += (long)tiles_n256 * (big + small);
            }
            const double rounds_exact = (double)items / num_cu;
            const double full = std::floor(rounds_exact), frac = rounds_exact - full;
            const double t = (full + (frac > 0 ? 0.6 + 0.4 * frac : 0.0)) * cost / (double)items;
            if (best_t == 0 || t < best_t) { best_t = t; variant = cand; }
        }
        // The queue form (tiles of 64 to 256 rows, resident workgroups): where its shorter last tiles save at least
        // 7 % of the rows the chosen tiles compute and it has enough items to go round (1.5 per CU; 2.5 when K is
        // below 4096 and an item is short against the cost of drawing it). Measured on 68 layouts (8 to 128 groups of
        // uniform, exponential or equal sizes; N x K = 4096 x 7168, 7168 x 2048, 2048 x 7168, 4096 x 2048) against
        // the best of the four 256-wide forms: this rule 0.8 % behind on average, 11 % at worst; never the queue form
        // 4.6 % and 16 %; the queue form on row savings alone 2.2 % and 41 % (16 groups of 16..384 rows at
        // N = 2048: 170 items for 256 CUs, 91 against 65 us with 128-row tiles).
        long rows_chosen = 0, rows_queue = 0, items_queue = 0;
        for (int g = 0; g < groups; g++) {
            const int rows = row_offsets[g + 1] - row_offsets[g];
            rows_queue += ceil_div(rows, 64) * 64;
            items_queue += (long)ceil_div(rows, 256) * tiles_n256;
            rows_chosen += variant == 0 ? ceil_div(rows, 256) * 256 : variant == 1 ? ceil_div(rows, 128) * 128
                           : rows / 256 * 256 + (rows % 256 == 0 ? 0 : rows % 256 <= 128 ? 128 : 256);
        }
        const long items_needed = k >= 4096 ? 3L * num_cu / 2 : 5L * num_cu / 2;
        if (rows_queue * 100 <= rows_chosen * 93 && items_queue >= items_needed) variant = kGroupedQueue;
    }
    return variant;
}
// prepadded: a and as already hold every group from a multiple of 16 rows on (the layout rf_quantize_a_grouped_* writes
// and rf_grouped_padded_offsets describes); otherwise they hold the groups back to back as row_offsets says.
int grouped_gemm(const void *a, const void *b, const float *as, const float *bs, void *c, const int *row_offsets,
                 int groups, int n, int k, int variant, hipStream_t stream, bool prepadded) {
    g_last_error.clear();
    if (!row_offsets) return fail(RF_ERR_NULL_POINTER, "row_offsets is null");
    if (groups < 1 || groups > rf::kMaxGroups)
        return fail(RF_ERR_BAD_SHAPE, "groups must be between 1 and " + std::to_string(rf::kMaxGroups));
    if (n < 1 || k < rf::BK || k % rf::BK != 0 || row_offsets[0] != 0)
        return fail(RF_ERR_BAD_SHAPE, "unsupported shape (need N>=1, K a positive multiple of 128, row_offsets[0] == 0)");
    for (int g = 0; g < groups; g++)
        if (row_offsets[g + 1] < row_offsets[g]) return fail(RF_ERR_BAD_SHAPE, "row_offsets must not decrease");
    const int m_total = row_offsets[groups];
    if (m_total == 0) return RF_OK;
    if (!a || !b || !as || !bs || !c) return fail(RF_ERR_NULL_POINTER, "null device pointer");
    if (variant >= kNumGroupedVariants || variant < -1) return fail(RF_ERR_BAD_CONFIG, "no such grouped variant");
    State &s = state();
    std::lock_guard<std::mutex> lock(shared().mu);
    int rc = ensure_device_info(s);
    if (rc != RF_OK) return rc;
    if (!s.grouped_attrs_set) {
        for (const GroupedVariant &v : kGroupedVariants)
            if (v.kernel)
                RF_HIP(hipFuncSetAttribute((const void *)v.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, v.lds));
        RF_HIP(hipFuncSetAttribute((const void *)rf::gemm_fp8_blockscale_grouped_queue,
                                   hipFuncAttributeMaxDynamicSharedMemorySize, rf::kQueueLds));
        s.grouped_attrs_set = true;
    }
    const int qk = k / rf::BK, qn = ceil_div(n, 128);
    const bool direct = n % 16 == 0 && ((uintptr_t)b % 16) == 0 && ((uintptr_t)c % 16) == 0;
    bool stage = ((uintptr_t)a % 16) != 0;
    for (int g = 0; g <= groups; g++) stage = stage || row_offsets[g] % 16 != 0;
    if (prepadded) {
        if (!direct || ((uintptr_t)a % 16) != 0)
            return fail(RF_ERR_BAD_CONFIG, "the padded layout needs N % 16 == 0 and 16-byte aligned a, b and c");
        stage = false;
    }
    if (!direct || (stage && (double)m_total * n * k < kPadThresholdMacs)) {
        // ragged N, unaligned weights or output, or next to no work: the bounds-checked kernel, one launch per
        // non-empty group
        for (int g = 0; g < groups; g++) {
            const int r0 = row_offsets[g], rows = row_offsets[g + 1] - r0;
            if (rows == 0) continue;
            dim3 grid(ceil_div(n, 16), ceil_div(rows, 16));
            hipLaunchKernelGGL(rf::gemm_fp8_blockscale_checked, grid, dim3(64), 0, stream, (const uint8_t *)a + r0,
                               (const uint8_t *)b + (size_t)g * k * n, as + r0, bs + (size_t)g * qk * qn,
                               (uint16_t *)c + (size_t)r0 * n, rows, m_total, n, k);
            RF_HIP(hipGetLastError());
        }
        return RF_OK;
    }
    rf::GroupTable table;
    int m_rows = m_total;                      // rows of the A matrix the kernel reads
    if (stage) {
        // Group sizes that are not multiples of 16 (token counts per expert never are): A and a_scale are copied
        // into the staging buffer with every group starting at a multiple of 16, the kernel reads those and writes
        // each group's true rows straight into the caller's C. Costs one pass over A; the bounds-checked kernel
        // per group would be 10 to 30 times slower than the tiled one.
        int at = 0;
        for (int g = 0; g < groups; g++) {
            table.row_start[g] = at;
            const int pr = (row_offsets[g + 1] - row_offsets[g] + 15) / 16 * 16;
            at += pr;
        }
        for (int g = groups; g <= rf::kMaxGroups; g++) table.row_start[g] = at;
        for (int g = 0; g <= rf::kMaxGroups; g++) table.out_row_start[g] = row_offsets[g < groups ? g : groups];
        m_rows = at;
        const size_t a_bytes = ((size_t)k * m_rows + 255) / 256 * 256;
        Mem mem{s};
        mem.stream = stream;
        uint8_t *pad = nullptr;
        rc = mem.pad(a_bytes + (size_t)qk * m_rows * sizeof(float), &pad);
        if (rc != RF_OK) return rc;
        launch_pad_a_and_scales(a, as, m_total, m_rows, k, groups, pad, (float *)(pad + a_bytes), table, stream);
        RF_HIP(hipGetLastError());
        a = pad;
        as = (const float *)(pad + a_bytes);
    } else if (prepadded) {
        int at = 0;
        for (int g = 0; g < groups; g++) {
            table.row_start[g] = at;
            at += (row_offsets[g + 1] - row_offsets[g] + 15) / 16 * 16;
        }
        for (int g = groups; g <= rf::kMaxGroups; g++) table.row_start[g] = at;
        for (int g = 0; g <= rf::kMaxGroups; g++) table.out_row_start[g] = row_offsets[g < groups ? g : groups];
        m_rows = at;
    } else {
        for (int g = 0; g <= rf::kMaxGroups; g++)
            table.row_start[g] = table.out_row_start[g] = row_offsets[g < groups ? g : groups];
    }
    if (variant < 0) variant = choose_grouped_variant(row_offsets, groups, n, k, s.num_cu);
    const GroupedVariant &v = kGroupedVariants[variant];
    const int tiles_n = ceil_div(n, v.bn);
    int tiles = 0;
    for (int g = 0; g < groups; g++) {
        table.tile_start[g] = tiles;
        tiles += v.tiles_m(row_offsets[g + 1] - row_offsets[g]) * tiles_n;
    }
    for (int g = groups; g <= rf::kMaxGroups; g++) table.tile_start[g] = tiles;
    if (v.queue) {
        // The line of items and its eight pieces. Estimated time of a group = column tiles x (256-row tiles + what
        // its last, shorter tile costs relative to one). With at least two groups per XCD: whole groups per queue,
        // each group to the queue with the least work so far, the longest group first (so every queue's groups are in
        // falling order). Fewer groups: the groups as they come, cut where the estimated time reaches each eighth.
        auto rows_of = [&](int g) { return row_offsets[g + 1] - row_offsets[g]; };
        auto cost_of_tile = [&](int rows, int i) { return i < rows / 256 ? 1.0 : kQueueTileCost[(rows % 256 + 63) / 64]; };
        auto cost_of = [&](int g) {
            return tiles_n * (rows_of(g) / 256 + kQueueTileCost[(rows_of(g) % 256 + 63) / 64]);
        };
        rf::GroupQueues queues;
        std::vector<int> order(groups);
        for (int g = 0; g < groups; g++) order[g] = g;
        int piece_groups[rf::NUM_XCD + 1] = {0};          // positions of the line where the pieces start, if whole groups
        const bool whole_groups = groups >= 2 * rf::NUM_XCD;
        if (whole_groups) {
            std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return cost_of(x) > cost_of(y); });
            std::vector<int> lists[rf::NUM_XCD];
            double load[rf::NUM_XCD] = {0};
            for (int g : order) {
                int least = 0;
                for (int x = 1; x < rf::NUM_XCD; x++)
                    if (load[x] < load[least]) least = x;
                lists[least].push_back(g);
                load[least] += cost_of(g);
            }
            int p = 0;
            for (int x = 0; x < rf::NUM_XCD; x++) {
                piece_groups[x] = p;
                for (int g : lists[x]) order[p++] = g;
            }
            piece_groups[rf::NUM_XCD] = p;
        }
        int items = 0;
        for (int p = 0; p < groups; p++) {
            queues.order[p] = (uint8_t)order[p];
            table.tile_start[p] = items;
            items += v.tiles_m(rows_of(order[p])) * tiles_n;
        }
        for (int p = groups; p <= rf::kMaxGroups; p++) table.tile_start[p] = items;
        for (int p = groups; p < rf::kMaxGroups; p++) queues.order[p] = 0;
        if (whole_groups) {
            for (int x = 0; x <= rf::NUM_XCD; x++) queues.piece_start[x] = table.tile_start[piece_groups[x]];
        } else {
            double total = 0, before = 0;
            for (int g = 0; g < groups; g++) total += cost_of(g);
            queues.piece_start[0] = 0;
            int piece = 1, item = 0;
            for (int g = 0; g < groups; g++) {
                const int tm = v.tiles_m(rows_of(g));
                for (int tn = 0; tn < tiles_n && tm > 0; tn++)
                    for (int i = 0; i < tm; i++, item++) {
                        while (piece < rf::NUM_XCD && before >= total * piece / rf::NUM_XCD) queues.piece_start[piece++] = item;
                        before += cost_of_tile(rows_of(g), i);
                    }
            }
            while (piece <= rf::NUM_XCD) queues.piece_start[piece++] = items;
        }
        queues.workgroups = s.num_cu >= rf::NUM_XCD ? s.num_cu / rf::NUM_XCD * rf::NUM_XCD : rf::NUM_XCD;
        if (tiles < queues.workgroups) queues.workgroups = ceil_div(tiles, rf::NUM_XCD) * rf::NUM_XCD;
        Mem mem{s};
        mem.stream = stream;
        unsigned *counters = nullptr;
        rc = mem.tile_counters(&counters);
        if (rc != RF_OK) return rc;
        hipLaunchKernelGGL(rf::gemm_fp8_blockscale_grouped_queue, dim3(queues.workgroups), dim3(v.threads), v.lds, stream,
                           (const uint8_t *)a, (const uint8_t *)b, as, bs, (uint16_t *)c, m_rows, n, k, groups, table,
                           queues, counters);
        RF_HIP(hipGetLastError());
        return RF_OK;
    }
    const int longest = ceil_div(tiles, rf::NUM_XCD);          // every XCD takes an eighth of the tiles, rounded
    hipLaunchKernelGGL(v.kernel, dim3(longest * rf::NUM_XCD), dim3(v.threads), v.lds, stream, (const uint8_t *)a,
                       (const uint8_t *)b, as, bs, (uint16_t *)c, m_rows, n, k, groups, table);
    RF_HIP(hipGetLastError());
    return RF_OK;
}

template <bool IN_BF16>
int quantize_a_grouped(const void *x, const int *row_offsets, int groups, int k, void *a, float *as, hipStream_t stream) {
    g_last_error.clear();
    if (!row_offsets) return fail(RF_ERR_NULL_POINTER, "row_offsets is null");
    if (groups < 1 || groups > rf::kQuantMaxGroups || k < rf::BK || k % rf::BK != 0 || row_offsets[0] != 0)
        return fail(RF_ERR_BAD_SHAPE, "unsupported shape (need 1 <= groups <= 256, K a positive multiple of 128, row_offsets[0] == 0)");
    rf::QuantGroups tab;
    int at = 0;
    for (int g = 0; g < groups; g++) {
        if (row_offsets[g + 1] < row_offsets[g]) return fail(RF_ERR_BAD_SHAPE, "row_offsets must not decrease");
        tab.pad_start[g] = at;
        tab.src_start[g] = row_offsets[g];
        at += (row_offsets[g + 1] - row_offsets[g] + 15) / 16 * 16;
    }
    for (int g = groups; g <= rf::kQuantMaxGroups; g++) { tab.pad_start[g] = at; tab.src_start[g] = row_offsets[groups]; }
    tab.groups = groups;
    for (int blk = 0, g = 0; blk < rf::kQuantBlockTable; blk++) {        // last g with pad_start[g] <= 128 * blk
        while (g + 1 < groups && tab.pad_start[g + 1] <= 128 * blk) g++;
        tab.block_group[blk] = (unsigned short)g;
    }
    if (at == 0) return RF_OK;
    if (!x || !a || !as) return fail(RF_ERR_NULL_POINTER, "null device pointer");
    if ((uintptr_t)x % 16 != 0 || (uintptr_t)a % 16 != 0 || (uintptr_t)as % 4 != 0)
        return fail(RF_ERR_BAD_CONFIG, "source and a must be 16-byte aligned, scales 4-byte aligned");
    State &s = state();
    {
        std::lock_guard<std::mutex> lock(shared().mu);
        int rc = ensure_device_info(s);
        if (rc != RF_OK) return rc;
    }
    hipLaunchKernelGGL((rf::quantize_block128_grouped<IN_BF16>), dim3(k / rf::BK, ceil_div(at, 128)), dim3(256), 0, stream, x,
                       at, k, (uint8_t *)a, as, tab);
    RF_HIP(hipGetLastError());
    return RF_OK;
}
}  // namespace

extern "C" {

int rf_fp8_gemm_grouped(const void *a, const void *b, const float *as, const float *bs, void *c, const int *row_offsets,
                        int groups, int n, int k, int variant, hipStream_t stream) {
    return grouped_gemm(a, b, as, bs, c, row_offsets, groups, n, k, variant, stream, false);
}

int rf_fp8_gemm_grouped_padded(const void *a, const void *b, const float *as, const float *bs, void *c,
                               const int *row_offsets, int groups, int n, int k, int variant, hipStream_t stream) {
    return grouped_gemm(a, b, as, bs, c, row_offsets, groups, n, k, variant, stream, true);
}

int rf_grouped_variant_for(const int *row_offsets, int groups, int n, int k, int num_cu, int *variant) {
    g_last_error.clear();
    if (!row_offsets || !variant) return fail(RF_ERR_NULL_POINTER, "row_offsets or variant is null");
    if (groups < 1 || groups > rf::kMaxGroups || n < 1 || k < rf::BK || k % rf::BK != 0 || num_cu < 1 || row_offsets[0] != 0)
        return fail(RF_ERR_BAD_SHAPE, "unsupported shape (need 1 <= groups <= 256, N >= 1, K a positive multiple of 128, "
                                      "a compute unit count, row_offsets[0] == 0)");
    for (int g = 0; g < groups; g++)
        if (row_offsets[g + 1] < row_offsets[g]) return fail(RF_ERR_BAD_SHAPE, "row_offsets must not decrease");
    *variant = choose_grouped_variant(row_offsets, groups, n, k, num_cu);
    return RF_OK;
}

int rf_grouped_padded_offsets(const int *row_offsets, int groups, int *padded_offsets) {
    g_last_error.clear();
    if (!row_offsets || !padded_offsets) return fail(RF_ERR_NULL_POINTER, "null pointer");
    if (groups < 1 || groups > rf::kMaxGroups || row_offsets[0] != 0) return fail(RF_ERR_BAD_SHAPE, "unsupported groups");
    int at = 0;
    for (int g = 0; g < groups; g++) {
        if (row_offsets[g + 1] < row_offsets[g]) return fail(RF_ERR_BAD_SHAPE, "row_offsets must not decrease");
        padded_offsets[g] = at;
        at += (row_offsets[g + 1] - row_offsets[g] + 15) / 16 * 16;
    }
    padded_offsets[groups] = at;
    return RF_OK;
}

int rf_quantize_a_grouped_f32(const float *x, const int *row_offsets, int groups, int k, void *a, float *as,
                              hipStream_t stream) {
    return quantize_a_grouped<false>(x, row_offsets, groups, k, a, as, stream);
}
int rf_quantize_a_grouped_bf16(const void *x, const int *row_offsets, int groups, int k, void *a, float *as,
                               hipStream_t stream) {
    return quantize_a_grouped<true>(x, row_offsets, groups, k, a, as, stream);
}

int rf_cast_f32_to_e4m3fn(const float *x, size_t count, void *out, hipStream_t stream) {
    g_last_error.clear();
    if (count == 0) return RF_OK;
    if (!x || !out) return fail(RF_ERR_NULL_POINTER, "null device pointer");
    if ((uintptr_t)x % 16 != 0 || (uintptr_t)out % 4 != 0)
        return fail(RF_ERR_BAD_CONFIG, "source must be 16-byte aligned, destination 4-byte aligned");
    hipLaunchKernelGGL(rf::cast_f32_to_e4m3fn, dim3((unsigned)((count + 1023) / 1024)), dim3(256), 0, stream, x,
                       (uint8_t *)out, count);
    RF_HIP(hipGetLastError());
    return RF_OK;
}

int rf_quantize_a_f32(const float *x, int m, int k, void *a, float *as, hipStream_t stream) {
    return launch_quantize<true, false>(x, m, k, a, as, stream);
}
int rf_quantize_a_bf16(const void *x, int m, int k, void *a, float *as, hipStream_t stream) {
    return launch_quantize<true, true>(x, m, k, a, as, stream);
}
int rf_quantize_b_f32(const float *w, int n, int k, void *b, float *bs, hipStream_t stream) {
    return launch_quantize<false, false>(w, n, k, b, bs, stream);
}
int rf_quantize_b_bf16(const void *w, int n, int k, void *b, float *bs, hipStream_t stream) {
    return launch_quantize<false, true>(w, n, k, b, bs, stream);
}

void run(void *a, void *b, void *as, void *bs, void *c, int m, int n, int k, PerfMetrics *metrics,
         hipStream_t job_stream0) {
    TimerJob *job = nullptr;
    if (metrics) {
        job = new TimerJob();
        State &s = state();
        job->owner = &s;
        {
            std::lock_guard<std::mutex> lock(s.ev_mu);
            if (!s.free_events.empty()) {
                job->start = s.free_events.back().first;
                job->stop = s.free_events.back().second;
                s.free_events.pop_back();
            } else {
                job->start = job->stop = nullptr;
            }
        }
        if (!job->start && (hipEventCreate(&job->start) != hipSuccess || hipEventCreate(&job->stop) != hipSuccess)) {
            fprintf(stderr, "run: hipEventCreate failed\n");
            abort();
        }
        job->flop = 2.0 * m * n * k;
        job->time_ms = &metrics->entries[0].time;
        job->gflops = &metrics->entries[0].gflops;
        if (hipEventRecord(job->start, job_stream0) != hipSuccess) {
            fprintf(stderr, "run: hipEventRecord failed\n");
            abort();
        }
    }
    int rc = launch(a, b, (const float *)as, (const float *)bs, c, m, n, k, nullptr, job_stream0);
    if (rc != RF_OK) {
        if (rc == RF_ERR_BAD_SHAPE) printf("Error: Unsupported shape M=%d, K=%d, N=%d\n", m, k, n);
        fprintf(stderr, "Kernel execution failed.\n%s\n", g_last_error.c_str());
        fflush(stdout);
        abort();
    }
    if (job) {
        if (hipEventRecord(job->stop, job_stream0) != hipSuccess ||
            hipStreamAddCallback(job_stream0, timer_callback, job, 0) != hipSuccess) {
            fprintf(stderr, "run: could not enqueue the timing callback\n");
            abort();
        }
    }
}

}  // extern "C"
