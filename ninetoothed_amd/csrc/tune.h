// Tuned choices: which kernel variant to run for a problem, found by timing the candidates once.
//
// Stands in for the reference's Triton autotuner (src/ninetoothed/generation.py:372-516), which times every
// block-size configuration of a generated kernel on the first call with a new problem.  Here the candidates
// are the hand-written variants of a program -- GEMM instances, attention loop forms, conv2d paths -- and the
// winners live in one per-process table keyed by (device, program, problem), behind a shared_mutex (the
// counterpart of the reference's per-context handle map, templates/thread_safe_unordered_map.h:10-30).
#pragma once

#include <hip/hip_runtime.h>

namespace nt {

enum TuneKind { kTuneGemm = 0, kTuneAttention = 1, kTuneConv2d = 2, kTuneKinds };
constexpr int kTuneMaxValues = 12;

// the recorded choice for a problem of the current device, or -1
int tune_lookup(int kind, const int *values, int count);
// (`extra`: up to three descriptive integers kept with the choice and written after it to the cache file)
void tune_record(int kind, const int *values, int count, int choice, const int *extra = nullptr, int extras = 0);

// Times candidates 0 .. candidates - 1 on `stream` with device events: 2 warm-up launches and `iters` timed ones
// each (a candidate whose `iters` launches take less than 0.5 ms is timed again over about 0.75 ms, at most 256 launches).  `launch(i)` returns 0, NINETOOTHED_NO_KERNEL (the candidate does not take the problem: skipped) or an
// error (returned).  *best receives the fastest candidate (-1 when none ran); with a `margin`, a later candidate
// replaces an earlier one only when it is faster by more than that fraction (candidates in order of preference).
// The first candidate is preceded by an untimed warm-up of about 20 ms.
// Synchronises; returns without timing anything (*best = -1, result 0) when the stream is being captured into a graph.
template <typename Launch>
int tune_time(hipStream_t stream, int candidates, int iters, Launch launch, int *best, float *best_ms, float margin = 0.0f) {
    *best = -1;
    *best_ms = 0.0f;
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (status != hipStreamCaptureStatusNone) return 0;
    if (iters <= 0) iters = 5;
    hipEvent_t start, stop;
    hipError_t err;
    if ((err = hipEventCreate(&start)) != hipSuccess) return (int)err;
    if ((err = hipEventCreate(&stop)) != hipSuccess) {
        (void)hipEventDestroy(start);
        return (int)err;
    }
    int result = 0;
    bool warm = false;
    for (int i = 0; i < candidates && result == 0; ++i) {
        int rc = launch(i);
        if (rc == 1) continue;  // NINETOOTHED_NO_KERNEL
        if (rc == 0) rc = launch(i);
        if (rc != 0) {
            result = rc;
            break;
        }
        // The first candidate that runs would otherwise be timed on an idle part whose clocks are still ramping up,
        // and lose to a slower one timed later: it first runs untimed for about 20 ms (at most 64 rounds).
        float warmed_ms = 0.0f;
        for (int round = 0; !warm && round < 64 && warmed_ms < 20.0f && rc == 0; ++round) {
            (void)hipEventRecord(start, stream);
            for (int r = 0; r < iters && rc == 0; ++r) rc = launch(i);
            (void)hipEventRecord(stop, stream);
            if (rc == 0 && (err = hipEventSynchronize(stop)) != hipSuccess) rc = (int)err;
            float ms = 0.0f;
            if (rc == 0) (void)hipEventElapsedTime(&ms, start, stop);
            warmed_ms += ms;
        }
        warm = true;
        if (rc != 0) {
            result = rc;
            break;
        }
        // short kernels are timed over more launches: a timed region of a few microseconds says little
        float ms = 0.0f;
        int timed = iters;
        for (int attempt = 0; attempt < 2 && rc == 0; ++attempt) {
            (void)hipEventRecord(start, stream);
            for (int r = 0; r < timed && rc == 0; ++r) rc = launch(i);
            (void)hipEventRecord(stop, stream);
            if (rc == 0 && (err = hipEventSynchronize(stop)) != hipSuccess) rc = (int)err;
            if (rc != 0) break;
            (void)hipEventElapsedTime(&ms, start, stop);
            if (ms >= 0.5f || timed >= 256) break;
            const int wanted = ms > 0.0f ? (int)(0.75f * (float)timed / ms) + 1 : 256;  // about 0.75 ms
            if (attempt == 0) timed = wanted < 256 ? (wanted > timed ? wanted : timed) : 256;
        }
        if (rc != 0) {
            result = rc;
            break;
        }
        ms /= (float)timed;
        if (*best < 0 || ms < *best_ms * (1.0f - margin)) {
            *best = i;
            *best_ms = ms;
        }
    }
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    return result;
}

}  // namespace nt
