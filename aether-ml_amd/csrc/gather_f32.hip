// fp32 entry points of the gather-GEMM path: convolution fprop / dgrad and the dense layer's
// forward and input-gradient products (the 1x1 cases of the same kernels: x [M,n_in] is an
// [M,1,1,n_in] image and w [n_in,n_out] a [1,1,n_in,n_out] filter).
#include "gather_dispatch.h"

using namespace aeth;

// Scratch of aeth_conv_fprop_f32_noalloc: the packed filter and, for few-tile products,
// the split-K partial tiles.  One copy per GPU, held until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels get g_scratch_ptr.
constexpr int64_t kNoallocScratchBytes = AETH_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kNoallocScratchBytes];
constexpr int kMaxDevices = 64;
static char* g_scratch_ptr[kMaxDevices] = {};          // device address of `scratch` on GPU i

namespace aeth {
int conv_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return fail(AETH_E_INVALID, "aeth_init: device %d out of range", device);
    if (g_scratch_ptr[device] != nullptr) return AETH_OK;
    void* p = nullptr;
    AETH_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr) return fail(AETH_E_HIP, "aeth_init: the scratch array has no device address");
    g_scratch_ptr[device] = static_cast<char*>(p);
    return AETH_OK;
}
}  // namespace aeth

extern "C" {

int aeth_conv_fprop_f32(const float* x, const float* w, const float* bias, float* y,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && w != nullptr && y != nullptr);
    return conv_fprop_impl<float>(__func__, x, w, bias, y, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

int aeth_conv_fprop_f32_noalloc(const float* x, const float* w, const float* bias, float* y,
                                int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && w != nullptr && y != nullptr);
    char* sp = g_scratch_ptr[ctx().device];
    if (sp == nullptr) return fail(AETH_E_STATE, "%s: the scratch array was not resolved by aeth_init", __func__);
    return conv_fprop_impl<float>(__func__, x, w, bias, y, S, H, W, C, D, fH, fW, sH, sW, pH, pW, sp, kNoallocScratchBytes);
}

int aeth_conv_dgrad_f32(const float* dy, const float* w, float* dx,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy != nullptr && w != nullptr && dx != nullptr);
    return conv_dgrad_impl<float>(__func__, dy, w, dx, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

int aeth_dense_fprop_f32(const float* x, const float* w, const float* bias, float* y, int M, int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && w != nullptr && y != nullptr);
    return conv_fprop_impl<float>(__func__, x, w, bias, y, M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0);
}

int aeth_dense_fprop_act_f32(const float* x, const float* w, const float* bias, float* y, float* act_y, float alpha, int M,
                             int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && w != nullptr && y != nullptr && act_y != nullptr);
    ActOut act{act_y, alpha, false};
    int rc = conv_fprop_impl<float>(__func__, x, w, bias, y, M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0, nullptr, 0, &act);
    if (rc) return rc;
    if (act.done) return AETH_OK;                       // the reduction of the split K wrote it
    return aeth_relu_fwd_f32(y, act_y, alpha, (int64_t)M * n_out);
}

int aeth_dense_dgrad_f32(const float* dy, const float* w, float* dx, int M, int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy != nullptr && w != nullptr && dx != nullptr);
    return conv_dgrad_impl<float>(__func__, dy, w, dx, M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0);
}

}  // extern "C"
