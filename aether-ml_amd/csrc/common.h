// Shared host-side plumbing of libaether_hip.so: the process-wide context,
// error reporting, the scratch workspace and small device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/aether_hip.h"

namespace aeth {

struct Context {
    bool ready = false;
    int device = -1;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop;
    // small always-present buffer for counters used by single-pass reductions
    unsigned int* counters = nullptr;
};

Context& ctx();
int fail(int code, const char* fmt, ...);
// Returns a pointer to at least `bytes` of library-owned scratch (packed filters, split
// partial sums); grows the buffer when needed.  A buffer that a recorded step may still
// replay into is kept until the last recording is destroyed; otherwise the old one is
// freed after the stream has drained.  Fails with AETH_E_STATE while a step is being recorded.
int workspace(int64_t bytes, void** out);
// While a prefix is set, workspace() hands out the bytes BEHIND the first `bytes` of the buffer (and makes the buffer large
// enough for both): the launch that owns the prefix is held back until a second one has been planned (pair_launch.h).
// workspace_base() is the start of the current buffer, i.e. of the prefix, after whatever growth the later calls caused.
void workspace_prefix(int64_t bytes);
void* workspace_base();
// Resolves the device address of the fixed scratch array of the entry point that
// allocates nothing (gather_f32.hip); called by aeth_init with the device current.
int conv_scratch_init(int device);

#define AETH_REQUIRE_INIT()                                                     \
    do {                                                                        \
        if (!aeth::ctx().ready) return aeth::fail(AETH_E_STATE, "%s: aeth_init has not been called", __func__); \
    } while (0)

#define AETH_CHECK_ARG(cond)                                                    \
    do {                                                                        \
        if (!(cond)) return aeth::fail(AETH_E_INVALID, "%s: argument check failed: %s", __func__, #cond); \
    } while (0)

#define AETH_HIP(call)                                                          \
    do {                                                                        \
        hipError_t e__ = (call);                                                \
        if (e__ != hipSuccess)                                                  \
            return aeth::fail(e__ == hipErrorOutOfMemory ? AETH_E_NOMEM : AETH_E_HIP, \
                              "%s: %s -> %s", __func__, #call, hipGetErrorString(e__)); \
    } while (0)

#define AETH_LAUNCH_CHECK()                                                     \
    do {                                                                        \
        hipError_t e__ = hipGetLastError();                                     \
        if (e__ != hipSuccess)                                                  \
            return aeth::fail(AETH_E_HIP, "%s: kernel launch -> %s", __func__, hipGetErrorString(e__)); \
    } while (0)

// Division by a runtime-constant positive divisor for 0 <= n < 2^31:
// q = umulhi(n, mul) >> shr.  d == 1 has no 32-bit multiplier; it is handled by a
// bit mask instead of a branch so that callers stay straight-line code.
struct FastDiv {
    unsigned int d, mul, shr, one;   // one = ~0u when d == 1
    FastDiv() : d(1), mul(0), shr(0), one(~0u) {}
    explicit FastDiv(int div) : d((unsigned)div), mul(0), shr(0), one(div == 1 ? ~0u : 0u) {
        if (div > 1) {
            unsigned l = 0;
            while ((1u << l) < (unsigned)div) ++l;           // ceil(log2 d)
            unsigned p = 31 + l;
            mul = (unsigned)(((1ull << p) + (unsigned)div - 1) / (unsigned)div);
            shr = p - 32;
        }
    }
    __host__ __device__ __forceinline__ unsigned div(unsigned n) const {
#if defined(__HIP_DEVICE_COMPILE__)
        unsigned q = __umulhi(n, mul) >> shr;
#else
        unsigned q = (unsigned)(((unsigned long long)n * mul) >> 32) >> shr;
#endif
        return (q & ~one) | (n & one);
    }
    __host__ __device__ __forceinline__ void divmod(unsigned n, unsigned& q, unsigned& r) const {
        q = div(n);
        r = n - q * d;
    }
};

static inline int cdiv(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }
static inline int64_t round_up(int64_t a, int64_t b) { return (a + b - 1) / b * b; }

}  // namespace aeth
