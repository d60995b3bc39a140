/*
 * C ABI of libgemm.so: FP8 (OCP e4m3fn) blockwise-scaled GEMM for MI355X (gfx950).
 *
 *   C[m,n] = bf16( sum_kb  a_scale[m,kb] * b_scale[n/128,kb] * sum_{k in block kb} A[m,k] * B[n,k] )
 *
 * Memory layouts are the reference launcher's (tests/gemm/gemm_test.cpp:82-98, task.yml:22-27):
 *   a   fp8 e4m3fn bytes, [K][M]   (element (m,k) at a[k*M + m])
 *   b   fp8 e4m3fn bytes, [K][N]   (element (n,k) at b[k*N + n])
 *   as  fp32,             [K/128][M]
 *   bs  fp32,             [K/128][ceil(N/128)]
 *   c   bf16,             [M][N] row-major, fully overwritten
 * All pointers are device pointers. K must be a positive multiple of 128; M, N >= 1.
 * Shapes with M%16==0, N%16==0 and 16-byte aligned a/b/c take the tiled MFMA path as they are. Anything else is
 * staged: the operands that need it are copied with rows padded to a multiple of 16 (zeros) into an internal buffer
 * grown on demand, the tiled path runs on the padded shape, and c receives the result without the padding (cost: one
 * pass over a; when N is ragged or c unaligned also one over b and a staged copy of c). Problems below 2^21 multiply-adds, and explicit plans with
 * variant = -1, take a bounds-checked kernel instead (the role of the reference's legacy kernel,
 * src/gemm/gemm_kernel_legacy.cpp:237-374).
 * Temporary device memory (split-K partial sums, staging copies, stream-K counters) is kept per (device, stream), for
 * the device that is current at the call: launches on different streams of one device may overlap, launches on one
 * stream are ordered by the stream. Calls are serialised by one lock only while they enqueue. A buffer that has to grow
 * is replaced and the old one freed by rf_gemm_destroy, so no call waits for the device. A stream gets a buffer set only
 * when a launch on it needs temporary memory (most plans need none); up to 32 streams per device have a set of their
 * own, and when one more asks, the least recently used set changes hands: the new stream waits on the device for the
 * old stream's work enqueued so far (an event, no host wait). A stream that is being captured into a HIP graph cannot
 * take a set over and gets RF_ERR_BAD_CONFIG (its first 32 streams capture fine; rf_fp8_gemm_static never needs a set).
 * HIP graphs captured through this library refer to these buffers: destroy them before rf_gemm_destroy, and do not
 * replay a graph captured on a stream whose set has since changed hands.
 */
#ifndef RF_GEMM_H
#define RF_GEMM_H

#include <stddef.h>
#include "metrics.h"

#ifdef __cplusplus
extern "C" {
#endif

#ifndef HIP_INCLUDE_HIP_HIP_RUNTIME_API_H
typedef struct ihipStream_t *hipStream_t;
#endif

/* Status codes of the rf_* entry points. */
enum {
    RF_OK = 0,
    RF_ERR_BAD_SHAPE = 1,      /* m<1, n<1, k<128 or k%128 != 0 */
    RF_ERR_NULL_POINTER = 2,
    RF_ERR_HIP = 3,            /* a HIP call failed; see rf_gemm_last_error() */
    RF_ERR_BAD_CONFIG = 4      /* explicit config not available for this shape */
};

enum { RF_SCHEDULE_TILES = 0, RF_SCHEDULE_STREAM_K = 1, RF_SCHEDULE_PERSISTENT = 2, RF_SCHEDULE_PERSISTENT_HALF_TAIL = 3,
       RF_SCHEDULE_SKINNY_K = 4 };

/* One launch plan: which kernel variant and how K is split.
 * Replaces a DISPATCH_GEMM(...) line of the reference (src/gemm/gemm_launcher.cpp:158-162,229-259). */
typedef struct rf_gemm_config {
    int variant;      /* index into the variant table, see rf_gemm_variant_info(); -1 = bounds-checked kernel */
    int split_k;      /* >= 1; K blocks are divided over this many partial sums */
    int group_m;      /* tile-order grouping along M for L2 reuse (>=1) */
    int stream_k;     /* schedule, one of RF_SCHEDULE_*:
                         0 TILES      one workgroup per tile (and per K split);
                         1 STREAM_K   persistent grid, one workgroup per CU, equal shares of the tile x K-block work
                                      line; needs split_k == 1 and at least as many tiles as CUs;
                         2 PERSISTENT persistent grid, whole tiles, one load/compute pipeline running across the
                                      tiles of a workgroup; needs split_k == 1, M a multiple of 16 and at least the
                                      tile height, N a multiple of the tile width, K/128 even;
                         3 PERSISTENT_HALF_TAIL  the persistent schedule for the whole rounds of one tile per CU, the
                                      left-over tiles finished as 128-row half tiles, one per CU; 256x256 tile only,
                                      needs the persistent schedule's shape rules, at least one tile per CU and a
                                      last round that is at most half full;
                         4 SKINNY_K   K = 128 ... 512 only: persistent grid, a workgroup keeps the B operand of a strip of
                                      256 columns in registers and streams A in items of 128 (K > 256: 64) rows, storing each
                                      16-row piece of C as soon as it is complete (the launch is a streaming store of
                                      C); needs variant == 0, split_k == 1, M a multiple of 16, N a multiple of 64 */
} rf_gemm_config;

/* Drop-in for the reference's launcher entry (src/gemm/gemm_launcher.cpp:182-184):
 * same name, argument order and behaviour: enqueues on job_stream0 and returns; on any error prints a
 * message and abort()s (src/gemm/gemm_launcher.cpp:96-100,261-264). metrics may be NULL; if not,
 * entries[0].time (ms) and entries[0].gflops are written from a stream callback once the work has
 * finished (src/utils/timer.cpp:12-60). Like the reference's, the callback reads the two events with
 * hipEventElapsedTime, a call HIP does not promise to allow inside a stream callback (the ROCm runtime this library is
 * built for does); it is the only way to have the figures written before a hipDeviceSynchronize() that follows run()
 * returns, which is what the reference's checker relies on (tests/checker/checker.cpp:286-336). Pass metrics = NULL
 * (or call rf_fp8_gemm) to keep callbacks out of the stream altogether. */
void run(void *a, void *b, void *as, void *bs, void *c, int m, int n, int k, PerfMetrics *metrics,
         hipStream_t job_stream0);

/* Same computation, returns a status instead of aborting. Replaces launch_gemm / launch_gemm_legacy
 * (src/gemm/gemm_launcher.cpp:43-101,104-148) with shape-generic dispatch. */
int rf_fp8_gemm(const void *a, const void *b, const float *as, const float *bs, void *c,
                int m, int n, int k, hipStream_t stream);

/* rf_fp8_gemm for callers that cannot allocate device memory: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc. No counterpart in the reference (its launcher allocates a fixed workspace with
 * hipMalloc on first use, src/gemm/gemm_launcher.cpp:30-36). Same arguments as rf_fp8_gemm, but split-K partial sums
 * and the staging copies of ragged or unaligned operands live in a static device array of
 * rf_gemm_static_scratch_bytes() bytes (32 MiB; every GPU the library has run on holds one until the process ends),
 * and the call allocates and frees nothing. The plan is rf_fp8_gemm's, and so are the result bits, whenever that plan
 * fits the array. Otherwise the plan is fitted to it: a K split is cut down to as many parts as fit (one part needs no
 * scratch memory), a stream-K plan from a plan file is replaced by the automatic plan, and a ragged or unaligned shape
 * whose staging copies do not fit as a whole is computed in row ranges that take turns in the array (M = 6001, N = 4608,
 * K = 7168: two ranges); such results agree with rf_fp8_gemm's within the rounding of another K split, and bit for bit
 * on data whose sums are exact. Only when the staged copy of B (ragged N or an unaligned b) alone takes more than half
 * of the array does the much slower bounds-checked kernel compute the shape, in place. All calls on one GPU share that
 * GPU's array: two calls that overlap in time (different streams, or graph replays beside eager launches) race; calls on
 * one stream are ordered by the stream. */
int rf_fp8_gemm_static(const void *a, const void *b, const float *as, const float *bs, void *c,
                       int m, int n, int k, hipStream_t stream);
size_t rf_gemm_static_scratch_bytes(void);

/* As rf_fp8_gemm with an explicit plan (cfg == NULL selects automatically). This is what the tuner
 * drives instead of recompiling a template per configuration (tuner/template/gemm_perf.cpp:21-38). */
int rf_fp8_gemm_ex(const void *a, const void *b, const float *as, const float *bs, void *c,
                   int m, int n, int k, const rf_gemm_config *cfg, hipStream_t stream);

/* The same launch `iters` times back to back on `stream`, after `warmup` untimed launches, bracketed by one pair of
 * events: *us_per_launch receives the average microseconds per launch. For the tuner (the reference's counterpart times
 * each generated binary with its KernelTimer, tuner/template/gemm_perf.cpp): a host language that needs several
 * microseconds per call cannot time launches shorter than that from outside. Blocks until the last launch is done. */
int rf_fp8_gemm_time(const void *a, const void *b, const float *as, const float *bs, void *c, int m, int n, int k,
                     const rf_gemm_config *cfg, int warmup, int iters, float *us_per_launch, hipStream_t stream);

/* The plan rf_fp8_gemm would use for (m,n,k) on the current device: the gfx950 replacement of the
 * per-shape table in src/gemm/gemm_launcher.cpp:229-259 / tuner/gemm_tuner.py. */
int rf_gemm_select_config(int m, int n, int k, rf_gemm_config *out);

/* The plan for (m,n,k) on a device with num_cu compute units, worked out on the host alone (no device is touched, the
 * file named by RF_GEMM_PLANS is not read; plans loaded with rf_gemm_load_plans count). The built-in table was measured
 * on 256 compute units and is consulted only for that count; any other count gets the cost model, which counts rounds
 * of workgroups for the count given. For capacity planning and for tests of the planner's arithmetic. */
int rf_gemm_plan_for(int m, int n, int k, int num_cu, rf_gemm_config *out);

/* Measured plans from a file, looked up before the built-in table (the role of pasting DISPATCH_GEMM lines into the
 * reference's launcher, src/gemm/gemm_launcher.cpp:229-259, tuner/gemm_batch.py:196-200, without a rebuild). One plan
 * per line: "M N K variant split_k group_m stream_k"; braces and commas are blanks, '#' and "//" start a comment, so
 * the tuner's --emit-file output and csrc/tuned_plans.inc are both valid files. *count receives the number of plans
 * added (may be NULL). A line that does not parse or names a variant or schedule that does not exist fails the whole
 * file with RF_ERR_BAD_CONFIG (nothing is added). A plan that cannot run for its shape (e.g. the persistent schedule on
 * a ragged shape) is skipped at lookup. The file named by the environment variable RF_GEMM_PLANS is loaded the same
 * way before the first plan is chosen. rf_gemm_clear_plans forgets all loaded plans. */
int rf_gemm_load_plans(const char *path, int *count);
void rf_gemm_clear_plans(void);

/* Variant table introspection (for the tuner and tests). Returns RF_ERR_BAD_CONFIG past the end. */
int rf_gemm_num_variants(void);
int rf_gemm_variant_info(int variant, int *block_m, int *block_n, int *waves_m, int *waves_n, int *lds_bytes);
/* 1 if the variant can run with rf_gemm_config.stream_k = RF_SCHEDULE_STREAM_K / RF_SCHEDULE_PERSISTENT, 0 if not
 * (or if the index is out of range). */
int rf_gemm_variant_has_stream_k(int variant);
int rf_gemm_variant_has_persistent(int variant);
/* Number of wave groups of one workgroup that split K between them (0 if the index is out of range). 1 for the ordinary
 * variants. A variant with more computes a tile's K parts side by side in one workgroup and sums them through LDS in part
 * order (the bits of split_k = that many equal parts, in one launch, no partial sums in memory): it takes split_k == 1 and
 * the tile schedule only, and K/128 must be a multiple of the count (RF_ERR_BAD_CONFIG otherwise). */
int rf_gemm_variant_k_groups(int variant);

/* Device workspace (split-K partial sums) needed for a shape under the automatic plan, in bytes. The staging copies
 * of ragged or unaligned operands are not part of it: that buffer grows on the first such call. */
size_t rf_gemm_workspace_bytes(int m, int n, int k);

/* Optional explicit set-up / tear-down of the current device's workspace. run() and
 * rf_fp8_gemm() grow it lazily on first use (the reference's init_workspace, src/gemm/gemm_launcher.cpp:30-36,50-53,
 * allocates a fixed 1.5 GB instead). rf_gemm_init(bytes) pre-allocates so that later calls allocate nothing. */
int rf_gemm_init(size_t workspace_bytes);
void rf_gemm_destroy(void);

/* Grouped form: `groups` independent GEMMs sharing N and K in one launch, for expert layers whose tokens have been
 * sorted by expert. The reference's consumer of such a call is LaunchGroupGEMM(..., h_IDX, ...) over the host array
 * first_token_offset (src/moe/moe.cpp:204,213-221,244-248; fp16 hipBLASLt there); this is its fp8 block-scaled form.
 *   a   fp8  [K][M_total]           rows of all groups back to back, M_total = row_offsets[groups]
 *   as  fp32 [K/128][M_total]
 *   b   fp8  [groups][K][N]         one weight matrix per group
 *   bs  fp32 [groups][K/128][ceil(N/128)]
 *   c   bf16 [M_total][N]
 *   row_offsets  HOST array of groups+1 ints, row_offsets[0] == 0, non-decreasing; group g owns rows
 *                row_offsets[g] .. row_offsets[g+1]-1 (empty groups allowed); read before the call returns.
 * groups <= 256. One launch of the tiled kernel when N % 16 == 0 and b, c are 16-byte aligned. Offsets may be any
 * numbers (token counts per expert are): when one is not a multiple of 16, or a is not 16-byte aligned, a and as are
 * first copied into the internal staging buffer with every group starting at a multiple of 16 (one pass over a;
 * c is written in place, rows of neighbouring groups are not touched). Ragged N, unaligned b or c, and problems below
 * 2^21 multiply-adds run the bounds-checked kernel once per group.
 * variant: -1 = automatic, else an index into {256x256, 128x256, 128x128, 128x64} tiles, or 4 = 256-row tiles with a
 * 128 x 256 tile for a group's last rows when at most 128 are left, or 5 = 256-row tiles with a last tile of 64, 128,
 * 192 or 256 rows, run by one resident workgroup per CU that takes tiles from a queue per XCD (the automatic choice
 * for groups of uneven size; its queues are counters in the stream's buffer set, like the stream-K schedule's). */
int rf_fp8_gemm_grouped(const void *a, const void *b, const float *as, const float *bs, void *c, const int *row_offsets,
                        int groups, int n, int k, int variant, hipStream_t stream);

/* The tile form rf_fp8_gemm_grouped takes with variant = -1 for groups of these sizes on a device with num_cu compute
 * units (an index as described above); host arithmetic only, no device needed. For launches that take the tiled
 * kernels (N % 16 == 0, aligned b and c, not a tiny problem). No counterpart in the reference, whose grouped GEMM is
 * hipBLASLt's (src/moe/moe.cpp:213-221). */
int rf_grouped_variant_for(const int *row_offsets, int groups, int n, int k, int num_cu, int *variant);

/* The grouped form without the staging copy: a and as already hold every group from a multiple of 16 rows on.
 *   padded_offsets[g] = sum over earlier groups of their row counts rounded up to 16 (rf_grouped_padded_offsets writes
 *   groups + 1 of them on the host; M_pad = padded_offsets[groups]);
 *   a  fp8 [K][M_pad], as fp32 [K/128][M_pad]: group g's rows from column padded_offsets[g] on, anything in the padding
 *   (rf_quantize_a_grouped_* writes zeros with scale 1); b, bs, c and row_offsets as for rf_fp8_gemm_grouped (c holds
 *   the true rows back to back). Needs N % 16 == 0 and 16-byte aligned a, b, c (RF_ERR_BAD_CONFIG otherwise).
 * rf_quantize_a_grouped_*: x is [M_total][K] row-major (the groups' rows back to back, row_offsets on the host);
 * writes a and as in that padded layout in one pass, so that token counts per expert that are not multiples of 16
 * cost no extra pass over A (the staging copy of rf_fp8_gemm_grouped is 25-40 us for 57 MB of A). The reference has
 * no counterpart: its expert GEMMs are fp16 (src/moe/moe.cpp:213-248). */
int rf_grouped_padded_offsets(const int *row_offsets, int groups, int *padded_offsets);
int rf_quantize_a_grouped_f32(const float *x, const int *row_offsets, int groups, int k, void *a, float *as,
                              hipStream_t stream);
int rf_quantize_a_grouped_bf16(const void *x, const int *row_offsets, int groups, int k, void *a, float *as,
                               hipStream_t stream);
int rf_fp8_gemm_grouped_padded(const void *a, const void *b, const float *as, const float *bs, void *c,
                               const int *row_offsets, int groups, int n, int k, int variant, hipStream_t stream);

/* Block quantisers: the step before the GEMM, on the GPU. No counterpart in the reference, whose harness draws
 * fp8 bytes and scales directly (tests/gemm/gemm_test.cpp:64-99); they implement the recipe its callers use:
 * scale = amax/448 over a block (1 if the block is all zero), value = e4m3fn_rne(x / scale).
 *   rf_quantize_a_*: x is [m][k] row-major (fp32 or bf16), one scale per (row, 128-wide K block);
 *                    writes a ([K][M] fp8, the layout `run` takes) and as ([K/128][M] fp32).
 *   rf_quantize_b_*: w is [n][k] row-major, one scale per 128x128 block (the last N block may be partial);
 *                    writes b ([K][N] fp8) and bs ([K/128][ceil(N/128)] fp32).
 * k must be a positive multiple of 128; sources 16-byte aligned. Enqueued on `stream`. */
int rf_quantize_a_f32(const float *x, int m, int k, void *a, float *as, hipStream_t stream);
int rf_quantize_a_bf16(const void *x, int m, int k, void *a, float *as, hipStream_t stream);
int rf_quantize_b_f32(const float *w, int n, int k, void *b, float *bs, hipStream_t stream);
int rf_quantize_b_bf16(const void *w, int n, int k, void *b, float *bs, hipStream_t stream);

/* Elementwise cast fp32 -> OCP e4m3fn (round to nearest even; |x| that rounds above 448, infinities and NaN become
 * NaN with the sign kept), the conversion the quantisers apply after scaling. No counterpart in the reference. */
int rf_cast_f32_to_e4m3fn(const float *x, size_t count, void *out, hipStream_t stream);

/* Text of the last failure on this thread's most recent rf_* call ("" if none). */
const char *rf_gemm_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
