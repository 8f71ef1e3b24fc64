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

// A choice read from a file is taken over only if the program's own source still knows it: each program registers,
// from a static initialiser, a function that says whether (index, descriptive integers) names one of its variants
// as this build numbers them.  Programs without such a function accept any index >= 0.
typedef bool (*TuneChoiceCheck)(int index, const int *extra, int extras);
bool tune_register_check(int kind, TuneChoiceCheck check);

// Written into the default pair of a saved file and compared on load: raised whenever the numbering of the GEMM
// instances, attention variants or conv2d paths changes, so that a file from another numbering is ignored whole.
constexpr int kTuneFileFormat = 4;

// Which kernel served the latest launch_nt_* call of the calling host thread: the launch functions leave a note
// (three thread-local stores), nt_last_launch formats it.  `name` must point to a string that lives as long as
// the library (a literal or an instance table entry).
enum LaunchProgram { kLaunchNone = 0, kLaunchGemm, kLaunchAttention, kLaunchConv2d, kLaunchSoftmax, kLaunchMap };
void note_launch(int program, int choice, const char *name);

// Times candidates 0 .. candidates - 1 on `stream` with device events and reports the fastest.  `launch(i)` returns 0,
// NINETOOTHED_NO_KERNEL (the candidate does not take the problem: skipped) or an error (returned).
//
// A choice made from one short timed region per candidate is a matter of luck on a part whose clock moves with
// load and temperature: a dip during one candidate's few milliseconds decides the variant for the rest of the
// process.  So (as triton.testing.do_bench, which the reference's autotuner uses, runs every configuration for a
// fixed time): the first candidate that runs is launched untimed for about 20 ms, every candidate's launch time is
// estimated over `iters` launches, and then the candidates take turns over several rounds -- each round times
// every candidate over a region of about 3 ms (at least one launch, at most 256) -- and a candidate's figure is the
// minimum of its rounds, so that a slow spell has to hit the same candidate in every round to mislead.
// Candidates are in order of preference: with a `margin`, a later candidate replaces an earlier one only when it
// is faster by more than that fraction.  *best = -1 when none ran.
// Synchronises; returns without timing anything (*best = -1, result 0) when the stream is being captured into a graph.
constexpr int kTuneMaxCandidates = 64;

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
    if (candidates > kTuneMaxCandidates) candidates = kTuneMaxCandidates;
    hipEvent_t start, stop;
    hipError_t err;
    if ((err = hipEventCreate(&start)) != hipSuccess) return (int)err;
    if ((err = hipEventCreate(&stop)) != hipSuccess) {
        (void)hipEventDestroy(start);
        return (int)err;
    }
    // milliseconds that `count` launches of candidate i take (negative: an error code, negated)
    auto region = [&](int i, int count, float *ms) -> int {
        int rc = 0;
        (void)hipEventRecord(start, stream);
        for (int r = 0; r < count && rc == 0; ++r) rc = launch(i);
        (void)hipEventRecord(stop, stream);
        const hipError_t waited = hipEventSynchronize(stop);
        if (rc == 0 && waited != hipSuccess) rc = (int)waited;
        *ms = 0.0f;
        if (rc == 0) (void)hipEventElapsedTime(ms, start, stop);
        return rc;
    };
    int live[kTuneMaxCandidates], launches[kTuneMaxCandidates];
    float fastest[kTuneMaxCandidates];
    int alive = 0, result = 0;
    for (int i = 0; i < candidates && result == 0; ++i) {  // which candidates take the problem
        int rc = launch(i);
        if (rc == 1) continue;  // NINETOOTHED_NO_KERNEL
        if (rc == 0) rc = launch(i);
        if (rc != 0) result = rc;
        else live[alive++] = i;
    }
    if (result == 0 && alive > 0) {
        float ms = 0.0f, warmed_ms = 0.0f;
        for (int round = 0; round < 64 && warmed_ms < 20.0f && result == 0; ++round) {  // let the part raise its clocks
            result = region(live[0], iters, &ms);
            warmed_ms += ms;
        }
        float round_ms = 0.0f;
        for (int c = 0; c < alive && result == 0; ++c) {  // how many launches make a region of about 3 ms
            result = region(live[c], iters, &ms);
            const float one = ms > 0.0f ? ms / (float)iters : 0.01f;
            const int wanted = (int)(3.0f / one) + 1;
            launches[c] = wanted > 256 ? 256 : wanted;
            fastest[c] = one;
            round_ms += one * (float)launches[c];
        }
        // long kernels get fewer rounds: a choice between candidates of 100 ms each is not worth seconds
        const int rounds = round_ms <= 100.0f ? 5 : (round_ms <= 400.0f ? 3 : 1);
        for (int round = 0; round < rounds && result == 0; ++round) {
            for (int c = 0; c < alive && result == 0; ++c) {
                result = region(live[c], launches[c], &ms);
                const float one = ms / (float)launches[c];
                if (result == 0 && (round == 0 || one < fastest[c])) fastest[c] = one;
            }
        }
        for (int c = 0; c < alive && result == 0; ++c) {
            if (*best < 0 || fastest[c] < *best_ms * (1.0f - margin)) {
                *best = live[c];
                *best_ms = fastest[c];
            }
        }
        if (result != 0) {
            *best = -1;
            *best_ms = 0.0f;
        }
    }
    (void)hipEventDestroy(start);
    (void)hipEventDestroy(stop);
    return result;
}

}  // namespace nt
