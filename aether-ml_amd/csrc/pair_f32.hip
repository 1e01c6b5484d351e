// A layer's weight gradient and input gradient in one launch (pair_launch.h), and the fp32 entry points that
// compute both: aeth_conv_bwd_f32, aeth_dense_bwd_f32.
#include "gather_kernels.h"
#include "wgrad_kernels.h"
#include "narrow_kernels.h"
#include "pair_launch.h"
#include "sample_runs.h"
#include "tuning.h"

namespace aeth {

static PairCtl g_pair;
static WgradParams g_held_wgrad;
static DirectParams g_held_direct;
PairCtl& pair_ctl() { return g_pair; }
WgradParams& held_wgrad_params() { return g_held_wgrad; }
DirectParams& held_direct_params() { return g_held_direct; }

template <int DK> struct DgradArg { typedef GatherParams type; };
template <> struct DgradArg<kHeldDirect333> { typedef DirectParams type; };

constexpr int pair_wgrad_row(int wk) { return wk == kHeldWgrad192 ? 192 : kWgBK; }              // floats per x slab row
constexpr int pair_wgrad_lds(int wk) { return (2 * kWgBR * pair_wgrad_row(wk) + 2 * kWgBR * kWgBN) * 4; }
constexpr int pair_dgrad_lds(int dk) {
    return dk == kHeldGather128x32 ? (2 * 128 + 2 * 32) * 8 * 16 : dk == kHeldGather64x64 ? 4 * 64 * 8 * 16 : kDirectMaxW * 4;
}
constexpr int pair_max(int a, int b) { return a > b ? a : b; }

// One grid for both kernels: the workgroups of the wgrad kernel first, rounded up to a whole number of XCDs, then those of
// the dgrad kernel.  The hardware hands workgroups to the XCDs round-robin, so inside its kernel a workgroup has the
// number it would have in a launch of that kernel alone and sits on the XCD it would sit on there: tiles that share
// operands keep sharing an L2.  The workgroups that pad the first kernel do nothing.  The two bodies use the same LDS.
// (Alternating the kernels in groups of one workgroup per XCD was measured too: 36 and 42 us against 32 and 32 on the
// second and third layer of a three-block CNN at batch 128, where the kernels alone take 22 + 17 and 22 + 12.)
template <int WK, int DK>
static __global__ __launch_bounds__(kThreads, 2) void bwd_pair(const WgradParams pw, const typename DgradArg<DK>::type pd,
                                                              const unsigned wgrad_blocks, const unsigned wgrad_padded,
                                                              const unsigned dgrad_gx, const FastDiv div_gx) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[pair_max(pair_wgrad_lds(WK), pair_dgrad_lds(DK))];
    const unsigned b = blockIdx.x;
    const bool is_w = b < wgrad_padded;
    const unsigned idx = is_w ? b : b - wgrad_padded;      // the workgroup's number inside its kernel
    if (is_w) {
        if (idx >= wgrad_blocks) return;
        constexpr int RS = pair_wgrad_row(WK);
        float* a0 = reinterpret_cast<float*>(lds);
        float* a1 = a0 + kWgBR * RS;
        float* y0 = a1 + kWgBR * RS;
        float* y1 = y0 + kWgBR * kWgBN;
        const BlockId blk{(int)idx, 0, (int)wgrad_blocks};
        if constexpr (WK == kHeldWgrad192) {
            wgrad_dma_body<6>(pw, a0, a1, y0, y1, blk);
        } else {
            if (pw.cw == 1) wgrad_dma_body<1>(pw, a0, a1, y0, y1, blk);
            else if (pw.cw == 2) wgrad_dma_body<2>(pw, a0, a1, y0, y1, blk);
            else wgrad_dma_body<4>(pw, a0, a1, y0, y1, blk);
        }
        return;
    }
    if constexpr (DK == kHeldDirect333) {
        direct_dgrad_body<float, 3, 3, 3, 2>(pd, idx, reinterpret_cast<float*>(lds));
    } else {
        unsigned y, x;
        div_gx.divmod(idx, y, x);
        const BlockId blk{(int)x, (int)y, (int)dgrad_gx};
        f4* l = reinterpret_cast<f4*>(lds);
        if constexpr (DK == kHeldGather128x32)
            gather_gemm_dma_body<float, 128, 32, 32, 32, true, 8, false, true>(pd, blk, l, l + 128 * 8, l + 2 * 128 * 8, l + 2 * 128 * 8 + 32 * 8);
        else
            gather_gemm_dma_body<float, 64, 64, 32, 32, true, 8, false, true>(pd, blk, l, l + 64 * 8, l + 2 * 64 * 8, l + 3 * 64 * 8);
    }
}

// The fixed-order sums of two split products in one launch: workgroups [0, a_blocks) are reduce_splits4 on `a`, the rest on `b`.
static __global__ __launch_bounds__(kThreads) void sums_pair(const HeldSum a, const HeldSum b, const unsigned a_blocks) {
    if (blockIdx.x < a_blocks)
        reduce_splits4_body(blockIdx.x, a.part, a.out, a.dbias, a.n_out, a.n, a.stride, a.splits, 0, nullptr, 0.f);
    else
        reduce_splits4_body(blockIdx.x - a_blocks, b.part, b.out, b.dbias, b.n_out, b.n, b.stride, b.splits, 0, nullptr, 0.f);
}

template <int WK, int DK>
static void launch_pair(const PairCtl& pc, const WgradParams& pw, hipStream_t st) {
    const unsigned padded = (unsigned)round_up(pc.wgrad_blocks, kXcds);
    const unsigned dblocks = pc.dgrad_gx * pc.dgrad_gy;
    if constexpr (DK == kHeldDirect333)
        hipLaunchKernelGGL((bwd_pair<WK, DK>), dim3(padded + dblocks), dim3(kThreads), 0, st, pw, held_direct_params(), pc.wgrad_blocks,
                           padded, pc.dgrad_gx, FastDiv((int)pc.dgrad_gx));
    else
        hipLaunchKernelGGL((bwd_pair<WK, DK>), dim3(padded + dblocks), dim3(kThreads), 0, st, pw, pc.gather, pc.wgrad_blocks, padded,
                           pc.dgrad_gx, FastDiv((int)pc.dgrad_gx));
}

int pair_flush(const char* fn) {
    const PairCtl pc = g_pair;
    g_pair.reset();
    workspace_prefix(0);
    if (pc.wgrad_kind == kHeldNone) return AETH_OK;                 // (a dgrad is only ever held behind a wgrad)
    WgradParams pw = g_held_wgrad;
    HeldSum wsum = pc.wgrad_sum;
    if (pc.wgrad_in_ws) {
        // the dgrad's plan may have grown the workspace since the wgrad was planned: its partial sums are the first bytes of the current one
        pw.out = static_cast<float*>(workspace_base());
        wsum.part = pw.out;
    }
    hipStream_t st = ctx().stream;
    if (pc.dgrad_kind == kHeldNone) {
        if (pc.wgrad_kind == kHeldWgrad192) hipLaunchKernelGGL(wgrad_gemm_dma192, dim3(pc.wgrad_blocks), dim3(kThreads), 0, st, pw);
        else hipLaunchKernelGGL(wgrad_gemm_dma, dim3(pc.wgrad_blocks), dim3(kThreads), 0, st, pw);
    } else if (pc.wgrad_kind == kHeldWgrad192) {
        if (pc.dgrad_kind == kHeldGather128x32) launch_pair<kHeldWgrad192, kHeldGather128x32>(pc, pw, st);
        else if (pc.dgrad_kind == kHeldGather64x64) launch_pair<kHeldWgrad192, kHeldGather64x64>(pc, pw, st);
        else launch_pair<kHeldWgrad192, kHeldDirect333>(pc, pw, st);
    } else {
        if (pc.dgrad_kind == kHeldGather128x32) launch_pair<kHeldWgrad128, kHeldGather128x32>(pc, pw, st);
        else if (pc.dgrad_kind == kHeldGather64x64) launch_pair<kHeldWgrad128, kHeldGather64x64>(pc, pw, st);
        else launch_pair<kHeldWgrad128, kHeldDirect333>(pc, pw, st);
    }
    if (hipGetLastError() != hipSuccess) return fail(AETH_E_HIP, "%s: kernel launch failed", fn);
    const HeldSum& dsum = pc.dgrad_sum;
    const bool d_on = pc.dgrad_kind != kHeldNone && dsum.on;
    if (wsum.on && d_on) {
        const unsigned wb = (unsigned)cdiv(wsum.n, 64), db = (unsigned)cdiv(dsum.n, 64);
        hipLaunchKernelGGL(sums_pair, dim3(wb + db), dim3(kThreads), 0, st, wsum, dsum, wb);
    } else if (wsum.on || d_on) {
        const HeldSum& s = wsum.on ? wsum : dsum;
        hipLaunchKernelGGL(reduce_splits4, dim3(cdiv(s.n, 64)), dim3(kThreads), 0, st, s.part, s.out, s.dbias, s.n_out, s.n, s.stride,
                           s.splits, 0, (float*)nullptr, 0.f);
    }
    if (hipGetLastError() != hipSuccess) return fail(AETH_E_HIP, "%s: kernel launch failed", fn);
    return AETH_OK;
}

// Arms the collection of a layer's two launches when both products go out whole (no runs of samples).
static void pair_arm(int S, int64_t x_sample_bytes, int64_t dy_sample_bytes) {
    g_pair.reset();
    workspace_prefix(0);
    g_pair.armed = tuning().pair_bwd != 0 && plan_sample_runs(S, x_sample_bytes, dy_sample_bytes).runs == 1;
}

static void pair_drop() {
    g_pair.reset();
    workspace_prefix(0);
}

}  // namespace aeth

using namespace aeth;

extern "C" {

int aeth_conv_bwd_f32(const float* x, const float* dy, const float* w, float* dw, float* dbias, float* dx,
                      int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && dy != nullptr && w != nullptr && dw != nullptr && dx != nullptr);
    int Ho, Wo;
    int rc = check_conv_dims(__func__, S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    pair_arm(S, (int64_t)H * W * C * 4, (int64_t)Ho * Wo * D * 4);
    rc = aeth_conv_wgrad_f32(x, dy, dw, dbias, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
    if (rc == AETH_OK) rc = aeth_conv_dgrad_f32(dy, w, dx, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
    if (rc != AETH_OK) {
        pair_drop();
        return rc;
    }
    return pair_flush(__func__);
}

int aeth_dense_bwd_f32(const float* x, const float* dy, const float* w, float* dw, float* dbias, float* dx,
                       const float* act_in, float* act_dx, float alpha, int M, int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && dy != nullptr && w != nullptr && dw != nullptr && dx != nullptr);
    AETH_CHECK_ARG((act_in == nullptr) == (act_dx == nullptr));
    AETH_CHECK_ARG(M > 0 && n_in > 0 && n_out > 0);
    const int64_t total = (int64_t)M * n_in;
    if (narrow_shape(n_out, 1, 1, 1, 1, 0, 0) && M <= 1024 && total < ((int64_t)1 << 31) &&
        (int64_t)(n_in + 1) * 16 < ((int64_t)1 << 31)) {
        // a classifier head: weight gradient, bias gradient, input gradient and the activation's backward pass in one launch
        NarrowParams pw, pd;
        pw.a = x; pw.b = dy; pw.bias = nullptr; pw.out = dw; pw.out2 = dbias; pw.M = M; pw.K = n_in; pw.N = n_out;
        pd.a = dy; pd.b = w; pd.bias = nullptr; pd.out = dx; pd.out2 = nullptr; pd.M = M; pd.K = n_in; pd.N = n_out;
        const unsigned wb = (unsigned)cdiv((int64_t)(n_in + 1) * 16, kThreads), db = (unsigned)cdiv(total, kThreads);
        hipLaunchKernelGGL(narrow_bwd, dim3(wb + db), dim3(kThreads), 0, ctx().stream, pw, pd, wb, (unsigned)total, act_in, act_dx,
                           alpha);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    pair_arm(M, (int64_t)n_in * 4, (int64_t)n_out * 4);
    int rc = aeth_dense_wgrad_f32(x, dy, dw, dbias, M, n_in, n_out);
    if (rc == AETH_OK) rc = aeth_dense_dgrad_f32(dy, w, dx, M, n_in, n_out);
    if (rc != AETH_OK) {
        pair_drop();
        return rc;
    }
    rc = pair_flush(__func__);
    if (rc == AETH_OK && act_in != nullptr) rc = aeth_relu_bwd_f32(act_in, dx, act_dx, alpha, total);
    return rc;
}

}  // extern "C"
