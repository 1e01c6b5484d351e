// bf16-input / fp32-accumulate convolution (placeholder until the MFMA bf16
// kernels land: every entry point reports that it is unavailable).
#include "common.h"

using namespace aeth;

extern "C" {

int aeth_conv_fprop_bf16(const uint16_t*, const uint16_t*, const float*, float*, int, int, int, int, int, int, int,
                         int, int, int, int) {
    return fail(AETH_E_INVALID, "aeth_conv_fprop_bf16: not built");
}
int aeth_conv_dgrad_bf16(const uint16_t*, const uint16_t*, float*, int, int, int, int, int, int, int, int, int, int,
                         int) {
    return fail(AETH_E_INVALID, "aeth_conv_dgrad_bf16: not built");
}
int aeth_conv_wgrad_bf16(const uint16_t*, const uint16_t*, float*, float*, int, int, int, int, int, int, int, int,
                         int, int, int) {
    return fail(AETH_E_INVALID, "aeth_conv_wgrad_bf16: not built");
}

}  // extern "C"
