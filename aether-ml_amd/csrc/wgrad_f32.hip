// fp32 entry points of wgrad: the convolution's filter / bias gradient and the dense layer's
// weight / bias gradient (its 1x1 case).
#include "wgrad_dispatch.h"

using namespace aeth;

extern "C" {

int aeth_conv_wgrad_f32(const float* x, const float* dy, float* dw, float* dbias,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && dy != nullptr && dw != nullptr);
    return conv_wgrad_impl<float>(__func__, x, dy, dw, dbias, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

int aeth_dense_wgrad_f32(const float* x, const float* dy, float* dw, float* dbias, int M, int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && dy != nullptr && dw != nullptr);
    return conv_wgrad_impl<float>(__func__, x, dy, dw, dbias, M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0);
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
    int rc = aeth_dense_wgrad_f32(x, dy, dw, dbias, M, n_in, n_out);
    if (rc == AETH_OK) rc = aeth_dense_dgrad_f32(dy, w, dx, M, n_in, n_out);
    if (rc == AETH_OK && act_in != nullptr) rc = aeth_relu_bwd_f32(act_in, dx, act_dx, alpha, total);
    return rc;
}

}  // extern "C"
