// One launch for the weight gradient and the input gradient of a layer.
//
// The two products of a layer's backward pass read the same upstream gradient and do not depend on each other.  On the
// layers of a small network neither fills the GPU (a few hundred workgroups of one long loop each), so run one after the
// other they cost two kernel durations where the hardware could overlap them.  An entry point that computes both arms
// `PairCtl`, calls the two ordinary dispatchers, and the dispatch leaves that a paired kernel exists for put their launch
// here instead of on the stream; `pair_flush` (pair_f32.hip) then launches one grid whose first workgroups run the wgrad
// kernel's body and whose other workgroups run the dgrad kernel's body, and one more grid for the two fixed-order sums
// where both products were split.  Every workgroup executes the code it would execute in a launch of its own kernel:
// the results are bit-identical to the separate launches.
#pragma once
#include "conv_common.h"

namespace aeth {

struct WgradParams;
struct DirectParams;

// Arguments of one reduce_splits4 launch.
struct HeldSum {
    int on = 0;
    const float* part = nullptr;
    float* out = nullptr;
    float* dbias = nullptr;
    int n_out = 0, n = 0, stride = 0, splits = 0;
};

enum { kHeldNone = 0, kHeldWgrad128 = 1, kHeldWgrad192 = 2 };              // wgrad_gemm_dma, wgrad_gemm_dma192
enum { kHeldGather128x32 = 1, kHeldGather64x64 = 2, kHeldDirect333 = 3 };   // dgrad kernels

struct PairCtl {
    bool armed = false;         // an entry point is collecting the two launches of one layer
    bool dgrad_ok = false;      // the dgrad in progress is one launch (unit stride)
    int wgrad_kind = kHeldNone;
    int dgrad_kind = kHeldNone;
    unsigned wgrad_blocks = 0;
    bool wgrad_in_ws = false;   // the held wgrad writes its partial sums at the start of the workspace
    unsigned dgrad_gx = 0, dgrad_gy = 0;
    GatherParams gather;        // kHeldGather*
    HeldSum wgrad_sum, dgrad_sum;
    void reset() { *this = PairCtl(); }
};

PairCtl& pair_ctl();
WgradParams& held_wgrad_params();
DirectParams& held_direct_params();
// Launches what is held (as a pair, or the wgrad alone when no dgrad joined it) and disarms.
int pair_flush(const char* fn);

}  // namespace aeth
