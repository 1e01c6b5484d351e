// Bookkeeping of the library's scratch workspace (packed filters, split partial sums,
// batch-norm partials).  Kept free of HIP calls, with the allocator passed in, so that
// the rules below can be exercised on the host without a GPU.
//
// The workspace grows on demand.  A recorded step (HIP graph) has the address of the
// workspace it was recorded with baked into its kernel arguments, so a buffer that a
// live recording may still replay into must not be freed when a later, larger request
// replaces it: it is retired instead and freed when the last recording is destroyed.
// Nothing in the workspace carries state from one call to the next, so a replay that
// keeps using its retired buffer while eager calls use the new one stays correct.
#pragma once

#include <stdint.h>
#include <vector>

namespace aeth {

struct WorkspaceLedger {
    void* cur = nullptr;
    int64_t cur_bytes = 0;
    int64_t generation = 0;        // bumped every time the workspace is replaced
    int live_recordings = 0;       // recordings ended successfully and not yet destroyed
    bool recording_open = false;   // a recording is being captured right now
    std::vector<void*> retired;    // replaced buffers that live recordings may still use

    enum Result { kOk = 0, kWhileRecording = 1, kAllocFailed = 2 };

    static int64_t grown_size(int64_t bytes) {
        const int64_t want = bytes + bytes / 4;                   // 25 % slack
        const int64_t mb = (int64_t)1 << 20;
        return (want + mb - 1) / mb * mb;
    }

    // Returns a buffer of at least `bytes`.  alloc(size) -> pointer or nullptr;
    // release(pointer) frees one (the caller makes sure the device is idle first
    // through `before_release`, called once and only when something is freed).
    template <typename Alloc, typename Release, typename Quiesce>
    Result acquire(int64_t bytes, void** out, Alloc alloc, Release release, Quiesce before_release) {
        if (bytes <= cur_bytes) {
            *out = cur;
            return kOk;
        }
        if (recording_open) return kWhileRecording;               // its address would change under the capture
        const int64_t want = grown_size(bytes);
        if (cur != nullptr) {
            if (live_recordings > 0) {
                retired.push_back(cur);
            } else {
                before_release();
                release(cur);
            }
            cur = nullptr;
            cur_bytes = 0;
        }
        void* p = alloc(want);
        ++generation;
        if (p == nullptr) return kAllocFailed;
        cur = p;
        cur_bytes = want;
        *out = cur;
        return kOk;
    }

    void recording_ended_ok() { ++live_recordings; }

    // A recording was destroyed (the caller has made the device idle).
    template <typename Release>
    void recording_destroyed(Release release) {
        if (live_recordings > 0) --live_recordings;
        if (live_recordings == 0) {
            for (void* p : retired) release(p);
            retired.clear();
        }
    }

    template <typename Release>
    void reset(Release release) {
        for (void* p : retired) release(p);
        retired.clear();
        if (cur != nullptr) release(cur);
        cur = nullptr;
        cur_bytes = 0;
        live_recordings = 0;
        recording_open = false;
    }
};

}  // namespace aeth
