/*
 * Timing record handed to run(). Bit-compatible with the reference harness's struct
 * (tests/checker/metrics.h:4-13 in the reference tree): 4 + 20*28 = 564 bytes, C layout.
 * For the GEMM only entries[0].time (milliseconds) and entries[0].gflops are written and
 * `count` is left untouched, as the reference launcher does (src/gemm/gemm_launcher.cpp:191-193).
 */
#ifndef RF_METRICS_H
#define RF_METRICS_H

#ifdef __cplusplus
extern "C" {
#endif

typedef struct PerfMetricEntry {
    char name[20];
    float time;
    float gflops;
} PerfMetricEntry;

typedef struct PerfMetrics {
    int count;
    PerfMetricEntry entries[20];
} PerfMetrics;

#ifdef __cplusplus
}
#endif
#endif
