// Batches whose tensors reach 2^31 bytes.
//
// The fast convolution kernels address their operands through buffer descriptors with 32-bit byte
// offsets, so a tensor they read or write must stay below 2^31 bytes.  Convolution is independent per
// sample (fprop, dgrad) or a sum over samples (wgrad), so a larger batch is cut into runs of whole
// samples, each run a launch of its own on tensors that start at the run's first sample: the 64-bit
// part of every address is in the run's base pointers, the offsets inside a run stay 32-bit.  Runs are
// about 1.5 GiB, far beyond the size at which a launch reaches its full rate.
//
// Plain arithmetic without HIP calls, so that it can be checked on the host.
#pragma once

#include <stdint.h>

namespace aeth {

struct SampleRuns {
    int runs;   // 1: the call goes out as it is
    int per;    // samples per run (the last run may be shorter)
};

constexpr int64_t kRunTriggerBytes = ((int64_t)1 << 31) - ((int64_t)1 << 24);   // tensors from here on are cut
constexpr int64_t kRunTargetBytes = ((int64_t)3 << 29);                          // 1.5 GiB per tensor and run

// `a` and `b`: bytes per sample of the two batch-sized tensors of the call.
static inline SampleRuns plan_sample_runs(int S, int64_t a, int64_t b) {
    const int64_t big = a > b ? a : b;
    SampleRuns r{1, S};
    if (S <= 1 || big <= 0 || (int64_t)S * big < kRunTriggerBytes) return r;
    if (big > kRunTargetBytes) {
        // single samples beyond the target: one sample per run while a sample still fits a descriptor,
        // else the call stays whole (and takes the kernels with 64-bit addressing)
        if (big >= kRunTriggerBytes) return r;
        r.runs = S;
        r.per = 1;
        return r;
    }
    int per = (int)(kRunTargetBytes / big);
    if (per < 1) per = 1;
    const int runs = (int)(((int64_t)S + per - 1) / per);
    r.runs = runs;
    r.per = (int)(((int64_t)S + runs - 1) / runs);          // runs of equal length (the last at most runs - 1 shorter)
    r.runs = (int)(((int64_t)S + r.per - 1) / r.per);
    return r;
}

}  // namespace aeth
