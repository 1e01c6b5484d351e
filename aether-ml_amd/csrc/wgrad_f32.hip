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

}  // extern "C"
