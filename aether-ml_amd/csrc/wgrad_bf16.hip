// bf16-input / fp32-accumulate entry point of wgrad (v_mfma_f32_32x32x16_bf16 reducing over
// pixels; shapes the bf16 kernels reject widen to fp32 on the way into LDS, which is exact).
#include "wgrad_dispatch.h"

using namespace aeth;

extern "C" {

int aeth_conv_wgrad_bf16(const uint16_t* x, const uint16_t* dy, float* dw, float* dbias,
                         int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && dy != nullptr && dw != nullptr);
    return conv_wgrad_impl<uint16_t>(__func__, x, dy, dw, dbias, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

}  // extern "C"
