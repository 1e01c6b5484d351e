// bf16-input / fp32-accumulate / fp32-output entry points of the gather-GEMM path
// (fprop and dgrad on v_mfma_f32_32x32x16_bf16).
#include "gather_dispatch.h"

using namespace aeth;

extern "C" {

int aeth_conv_fprop_bf16(const uint16_t* x, const uint16_t* w, const float* bias, float* y,
                         int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && w != nullptr && y != nullptr);
    return conv_fprop_impl<uint16_t>(__func__, x, w, bias, y, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

int aeth_conv_dgrad_bf16(const uint16_t* dy, const uint16_t* w, float* dx,
                         int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy != nullptr && w != nullptr && dx != nullptr);
    return conv_dgrad_impl<uint16_t>(__func__, dy, w, dx, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

}  // extern "C"
