// Plain products with at most 16 output channels (a classifier head: Layer_Dense(256, 10)), fp32.
// The slab kernels give such a layer a 32- or 64-wide n tile, a packing launch and, for wgrad, a
// split and its reduction: 4 launches of 4 to 13 us for 0.65 MFLOP.  Here one thread owns one
// output and adds its products in order of k (fprop), n (dgrad) or m (wgrad): one launch each,
// no scratch memory.  Rows are few (the host limits M): a thread's loop is the latency of the launch.
#pragma once

#include "conv_common.h"
#include "tuning.h"

namespace aeth {

constexpr int kNarrowMaxN = 16;

struct NarrowParams {
    const float* a;      // fprop: x [M,K]; dgrad: dy [M,N]; wgrad: x [M,K]
    const float* b;      // fprop, dgrad: w [K,N]; wgrad: dy [M,N]
    const float* bias;   // fprop: [N] or nullptr
    float* out;          // fprop: y [M,N]; dgrad: dx [M,K]; wgrad: dw [K,N]
    float* out2;         // wgrad: dbias [N] or nullptr
    int M, K, N;
};

// y[m][n] = bias[n] + sum_k x[m][k] w[k][n]; a wave per row: lane = (quarter of k: k % 4, n), the four quarters added in order
static __global__ __launch_bounds__(kThreads) void narrow_fprop(const NarrowParams p) {
    const int t = (int)(blockIdx.x * kThreads + threadIdx.x);
    const int m = min(t >> 6, p.M - 1);                  // (rows past M repeat the last one: every lane takes part in the exchange)
    const int lane = t & 63, n = lane & 15, kq = lane >> 4;
    const float* x = p.a + (size_t)m * p.K;
    const float* w = p.b + min(n, p.N - 1);
    float acc = 0.0f;
#pragma unroll 8
    for (int k = kq; k < p.K; k += 4) acc = fmaf(x[k], w[(size_t)k * p.N], acc);
    float sum = (p.bias != nullptr && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
    for (int q = 0; q < 4; ++q) sum += __shfl(acc, n + 16 * q, 64);
    if (kq == 0 && n < p.N && (t >> 6) < p.M) p.out[(size_t)m * p.N + n] = sum;
}

// dx[m][k] = sum_n dy[m][n] w[k][n]; thread t = (m, k).  act_in != nullptr: the backward pass of the ReLU / leaky ReLU in
// front of the layer on the way, act_dx[t] = act_in[t] < 0 ? alpha dx : dx (what relu_bwd_kernel would write from dx).
__device__ __forceinline__ void narrow_dgrad_one(const NarrowParams& p, const unsigned t, const float* __restrict__ act_in,
                                                 float* __restrict__ act_dx, const float alpha) {
    const unsigned m = t / (unsigned)p.K, k = t - m * (unsigned)p.K;
    const float* dy = p.a + (size_t)m * p.N;
    const float* w = p.b + (size_t)k * p.N;
    float acc = 0.0f;
#pragma unroll 4
    for (int n = 0; n < p.N; ++n) acc = fmaf(dy[n], w[n], acc);
    p.out[t] = acc;
    if (act_in != nullptr) act_dx[t] = act_in[t] < 0.f ? alpha * acc : acc;
}

static __global__ __launch_bounds__(kThreads) void narrow_dgrad(const NarrowParams p, const unsigned total) {
    const unsigned t = blockIdx.x * kThreads + threadIdx.x;
    if (t >= total) return;
    narrow_dgrad_one(p, t, nullptr, nullptr, 0.f);
}

// dw[k][n] = sum_m x[m][k] dy[m][n], dbias[n] = sum_m dy[m][n] (row k == K of the thread grid); thread t = (k, n)
__device__ __forceinline__ void narrow_wgrad_one(const NarrowParams& p, const int t) {
    const int k = t >> 4, n = t & 15;
    if (k > p.K || n >= p.N || (k == p.K && p.out2 == nullptr)) return;
    const float* dy = p.b + n;
    float acc = 0.0f;
    if (k == p.K) {
#pragma unroll 16
        for (int m = 0; m < p.M; ++m) acc += dy[(size_t)m * p.N];
        p.out2[n] = acc;
        return;
    }
    const float* x = p.a + k;
#pragma unroll 16
    for (int m = 0; m < p.M; ++m) acc = fmaf(x[(size_t)m * p.K], dy[(size_t)m * p.N], acc);
    p.out[(size_t)k * p.N + n] = acc;
}

static __global__ __launch_bounds__(kThreads) void narrow_wgrad(const NarrowParams p) {
    narrow_wgrad_one(p, (int)(blockIdx.x * kThreads + threadIdx.x));
}

// A narrow dense layer's whole backward pass as one launch: the first `wgrad_blocks` workgroups are narrow_wgrad's, the
// others narrow_dgrad's (neither reads what the other writes), with the activation's backward pass as above.
static __global__ __launch_bounds__(kThreads) void narrow_bwd(const NarrowParams pw, const NarrowParams pd, const unsigned wgrad_blocks,
                                                              const unsigned dgrad_total, const float* __restrict__ act_in,
                                                              float* __restrict__ act_dx, const float alpha) {
    if (blockIdx.x < wgrad_blocks) {
        narrow_wgrad_one(pw, (int)(blockIdx.x * kThreads + threadIdx.x));
        return;
    }
    const unsigned t = (blockIdx.x - wgrad_blocks) * kThreads + threadIdx.x;
    if (t < dgrad_total) narrow_dgrad_one(pd, t, act_in, act_dx, alpha);
}

// 1x1 filter, unit stride, no padding, at most 16 output channels, few enough rows for one thread per output
// (tuning: narrow = 0 turns these kernels off)
static inline bool narrow_shape(int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    return D >= 1 && D <= kNarrowMaxN && fH == 1 && fW == 1 && sH == 1 && sW == 1 && pH == 0 && pW == 0 && tuning().narrow != 0;
}

}  // namespace aeth
