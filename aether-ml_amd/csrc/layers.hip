// Coalesced helper kernels for the layers either side of the convolution path:
// batch norm, ReLU / leaky ReLU, pooling, dropout masks, softmax + cross entropy,
// Adam, regulariser terms.  All tensors are row-major with the channel (or
// class) axis last, so consecutive lanes touch consecutive addresses.
#include "common.h"

namespace aeth {

constexpr int kEwThreads = 256;

static inline int ew_blocks(int64_t n, int per_thread = 1) {
    int64_t b = (n + (int64_t)kEwThreads * per_thread - 1) / ((int64_t)kEwThreads * per_thread);
    if (b > 8192) b = 8192;
    if (b < 1) b = 1;
    return (int)b;
}

// ------------------------------------------------------------------------------
// column reductions over a [rows, C] matrix
// Lane layout: when C < 64 divides 64 a wave covers 64/C rows per step, otherwise
// columns are tiled by 64 (blockIdx.y).  Each block reduces `rows_per_block` rows
// and writes NV partial values per column to part[(v*nblk + blockIdx.x)*C + c];
// a second kernel finishes in block order, so results do not depend on timing.
// ------------------------------------------------------------------------------
__device__ __forceinline__ void col_layout(int C, int& lanes_c, int& sub_rows) {
    lanes_c = (C < 64 && (64 % C) == 0) ? C : 64;
    sub_rows = 64 / lanes_c;
}

template <int NV, typename F>
__device__ __forceinline__ void column_partials(int rows, int C, int rows_per_block, float* __restrict__ part, F f) {
    __shared__ float red[NV][kEwThreads];
    int lanes_c, sub_rows;
    col_layout(C, lanes_c, sub_rows);
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int c = blockIdx.y * 64 + (lane % lanes_c);
    const int rl = wave * sub_rows + lane / lanes_c;   // row lane inside the block
    const int nrl = 4 * sub_rows;
    const int rbeg = blockIdx.x * rows_per_block;
    int rend = rbeg + rows_per_block;
    if (rend > rows) rend = rows;
    float acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = 0.f;
    if (c < C) {
        for (int r = rbeg + rl; r < rend; r += nrl) f((size_t)r * C + c, c, acc);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) red[v][tid] = acc[v];
    __syncthreads();
    // thread with rl == 0 owns column c: sum the nrl row lanes in fixed order
    if (rl == 0 && c < C) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            float s = 0.f;
            for (int w = 0; w < 4; ++w)
                for (int sr = 0; sr < sub_rows; ++sr) s += red[v][w * 64 + sr * lanes_c + (lane % lanes_c)];
            part[((size_t)v * gridDim.x + blockIdx.x) * C + c] = s;
        }
    }
}

static void col_grid(int rows, int C, int* nblk, int* rows_per_block, dim3* grid) {
    int nb = cdiv(rows, 256);
    if (nb > 256) nb = 256;
    if (nb < 1) nb = 1;
    int rpb = cdiv(rows, nb);
    nb = cdiv(rows, rpb);
    *nblk = nb;
    *rows_per_block = rpb;
    *grid = dim3(nb, cdiv(C, 64));
}

// Same reduction for C % 4 == 0 and 16-byte aligned rows: a lane owns 4 consecutive
// columns and reads them with one 16-byte load per row, four rows in flight.  The
// partials land in the same part[v][block][c] layout.
typedef float ew_f4 __attribute__((ext_vector_type(4)));

template <int NV, typename F>
__device__ __forceinline__ void column_partials4(int rows, int C, int rows_per_block, float* __restrict__ part, F f) {
    __shared__ ew_f4 red4[NV][kEwThreads];
    const int C4 = C >> 2;
    const int lanes_c = (C4 < 64 && (64 % C4) == 0) ? C4 : 64;
    const int sub_rows = 64 / lanes_c;
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int c4 = blockIdx.y * 64 + (lane % lanes_c);
    const int rl = wave * sub_rows + lane / lanes_c;
    const int nrl = 4 * sub_rows;
    const int rbeg = blockIdx.x * rows_per_block;
    int rend = rbeg + rows_per_block;
    if (rend > rows) rend = rows;
    ew_f4 acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = ew_f4{0.f, 0.f, 0.f, 0.f};
    if (c4 < C4) {
        int r = rbeg + rl;
        for (; r + 3 * nrl < rend; r += 4 * nrl) {
#pragma unroll
            for (int u = 0; u < 4; ++u) f((size_t)(r + u * nrl) * C4 + c4, c4, acc);
        }
        for (; r < rend; r += nrl) f((size_t)r * C4 + c4, c4, acc);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) red4[v][tid] = acc[v];
    __syncthreads();
    if (rl == 0 && c4 < C4) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            ew_f4 s = {0.f, 0.f, 0.f, 0.f};
            for (int w = 0; w < 4; ++w)
                for (int sr = 0; sr < sub_rows; ++sr) s += red4[v][w * 64 + sr * lanes_c + (lane % lanes_c)];
            *reinterpret_cast<ew_f4*>(part + ((size_t)v * gridDim.x + blockIdx.x) * C + 4 * c4) = s;
        }
    }
}

static bool col_vec4(int C, const void* a, const void* b) {
    return C % 4 == 0 && ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0;
}

// ---- batch norm ------------------------------------------------------------------
// Sums part[v][b][c] over the blocks b for v = 0, 1.  Launched with 256 threads =
// 64 channels x 4 block lanes; lane j adds blocks j, j+4, ... with four independent
// accumulators, then the lanes are added in order.  Returns true for the thread
// that holds the result (lane 0 of a valid channel).
__device__ __forceinline__ bool sum_partials2(const float* __restrict__ part, int nblk, int C, int c, float& s1,
                                              float& s2) {
    __shared__ float red[2][4][64];
    const int col = threadIdx.x & 63, bl = threadIdx.x >> 6;
    float a[4] = {0.f, 0.f, 0.f, 0.f}, q[4] = {0.f, 0.f, 0.f, 0.f};
    if (c < C) {
        int b = bl;
        for (; b + 12 < nblk; b += 16) {
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                a[u] += part[(size_t)(b + 4 * u) * C + c];
                q[u] += part[((size_t)nblk + b + 4 * u) * C + c];
            }
        }
        for (; b < nblk; b += 4) {
            a[0] += part[(size_t)b * C + c];
            q[0] += part[((size_t)nblk + b) * C + c];
        }
    }
    red[0][bl][col] = (a[0] + a[1]) + (a[2] + a[3]);
    red[1][bl][col] = (q[0] + q[1]) + (q[2] + q[3]);
    __syncthreads();
    s1 = (red[0][0][col] + red[0][1][col]) + (red[0][2][col] + red[0][3][col]);
    s2 = (red[1][0][col] + red[1][1][col]) + (red[1][2][col] + red[1][3][col]);
    return bl == 0 && c < C;
}

// Statistics use sums of (x - shift) and (x - shift)^2 with shift = x[0][c]: the
// variance then comes from numbers of the size of the spread, not of the mean.
__global__ __launch_bounds__(kEwThreads) void bn_stats_partial(const float* __restrict__ x, int rows, int C,
                                                              int rpb, float* __restrict__ part) {
    column_partials<2>(rows, C, rpb, part, [&](size_t i, int c, float* acc) {
        float d = x[i] - x[c];
        acc[0] += d;
        acc[1] += d * d;
    });
}

__global__ __launch_bounds__(kEwThreads) void bn_stats_partial4(const float* __restrict__ x, int rows, int C,
                                                               int rpb, float* __restrict__ part) {
    const ew_f4* __restrict__ x4 = reinterpret_cast<const ew_f4*>(x);
    column_partials4<2>(rows, C, rpb, part, [&](size_t i, int c4, ew_f4* acc) {
        const ew_f4 d = x4[i] - x4[c4];
        acc[0] += d;
        acc[1] += d * d;
    });
}

__global__ void bn_stats_final(const float* __restrict__ x, const float* __restrict__ part, int nblk, int rows, int C,
                               float eps, float momentum, float* __restrict__ running_mean,
                               float* __restrict__ running_var, float* __restrict__ save_mean,
                               float* __restrict__ save_invstd) {
    const int c = blockIdx.x * 64 + (threadIdx.x & 63);
    float s1, s2;
    if (!sum_partials2(part, nblk, C, c, s1, s2)) return;
    const float inv_n = 1.0f / (float)rows;
    const float dm = s1 * inv_n;
    const float mean = x[c] + dm;
    float var = s2 * inv_n - dm * dm;
    if (var < 0.f) var = 0.f;
    save_mean[c] = mean;
    save_invstd[c] = 1.0f / sqrtf(var + eps);
    running_mean[c] = momentum * running_mean[c] + (1.0f - momentum) * mean;
    running_var[c] = momentum * running_var[c] + (1.0f - momentum) * var;
}

// y = gamma * (x - mean) * invstd + beta
__global__ void bn_apply(const float* __restrict__ x, const float* __restrict__ gamma, const float* __restrict__ beta,
                         const float* __restrict__ mean, const float* __restrict__ invstd, float* __restrict__ y,
                         int64_t n, int C) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        int c = (int)(i % C);
        y[i] = gamma[c] * ((x[i] - mean[c]) * invstd[c]) + beta[c];
    }
}

// the same on groups of 4 channels (C % 4 == 0, 16-byte aligned tensors)
__global__ __launch_bounds__(kEwThreads) void bn_apply4(const ew_f4* __restrict__ x, const ew_f4* __restrict__ gamma,
                                                       const ew_f4* __restrict__ beta, const ew_f4* __restrict__ mean,
                                                       const ew_f4* __restrict__ invstd, ew_f4* __restrict__ y,
                                                       unsigned n4, int C4) {
    const unsigned stride = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const unsigned c4 = i % (unsigned)C4;
        y[i] = gamma[c4] * ((x[i] - mean[c4]) * invstd[c4]) + beta[c4];
    }
}

__global__ __launch_bounds__(kEwThreads) void bn_apply_infer4(const ew_f4* __restrict__ x, const ew_f4* __restrict__ gamma,
                                                             const ew_f4* __restrict__ beta, const ew_f4* __restrict__ rm,
                                                             const ew_f4* __restrict__ rv, ew_f4* __restrict__ y,
                                                             unsigned n4, int C4, float eps) {
    const unsigned stride = gridDim.x * blockDim.x;
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const unsigned c4 = i % (unsigned)C4;
        const ew_f4 v = rv[c4], d = x[i] - rm[c4];
        ew_f4 q;
#pragma unroll
        for (int e = 0; e < 4; ++e) q[e] = d[e] / sqrtf(v[e] + eps);
        y[i] = gamma[c4] * q + beta[c4];
    }
}

__global__ void bn_apply_infer(const float* __restrict__ x, const float* __restrict__ gamma,
                               const float* __restrict__ beta, const float* __restrict__ rm,
                               const float* __restrict__ rv, float* __restrict__ y, int64_t n, int C, float eps) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        int c = (int)(i % C);
        y[i] = gamma[c] * ((x[i] - rm[c]) / sqrtf(rv[c] + eps)) + beta[c];
    }
}

__global__ __launch_bounds__(kEwThreads) void bn_bwd_partial(const float* __restrict__ x, const float* __restrict__ dy,
                                                            const float* __restrict__ mean, int rows, int C, int rpb,
                                                            float* __restrict__ part) {
    column_partials<2>(rows, C, rpb, part, [&](size_t i, int c, float* acc) {
        float g = dy[i];
        acc[0] += g;
        acc[1] += g * (x[i] - mean[c]);
    });
}

__global__ __launch_bounds__(kEwThreads) void bn_bwd_partial4(const float* __restrict__ x, const float* __restrict__ dy,
                                                             const float* __restrict__ mean, int rows, int C, int rpb,
                                                             float* __restrict__ part) {
    const ew_f4* __restrict__ x4 = reinterpret_cast<const ew_f4*>(x);
    const ew_f4* __restrict__ dy4 = reinterpret_cast<const ew_f4*>(dy);
    const ew_f4* __restrict__ mean4 = reinterpret_cast<const ew_f4*>(mean);
    column_partials4<2>(rows, C, rpb, part, [&](size_t i, int c4, ew_f4* acc) {
        const ew_f4 g = dy4[i];
        acc[0] += g;
        acc[1] += g * (x4[i] - mean4[c4]);
    });
}

// coef[0*C+c] = gamma*invstd ; coef[1*C+c] = A ; coef[2*C+c] = B  with
// dx = coef0*dy + A*(x-mean) + B,  A = -gamma*s2*invstd^3/N,  B = -gamma*invstd*s1/N
__global__ void bn_bwd_final(const float* __restrict__ part, int nblk, int rows, int C,
                             const float* __restrict__ gamma, const float* __restrict__ invstd,
                             float* __restrict__ dgamma, float* __restrict__ dbeta, float* __restrict__ coef) {
    const int c = blockIdx.x * 64 + (threadIdx.x & 63);
    float s1, s2;
    if (!sum_partials2(part, nblk, C, c, s1, s2)) return;
    const float is = invstd[c], g = gamma[c];
    const float inv_n = 1.0f / (float)rows;
    dgamma[c] = s2 * is;
    dbeta[c] = s1;
    coef[c] = g * is;
    coef[C + c] = -g * s2 * is * is * is * inv_n;
    coef[2 * C + c] = -g * is * s1 * inv_n;
}

// dx16 (may be null): a bfloat16 copy of dx for a bf16 convolution that takes it as its upstream gradient
__global__ void bn_bwd_apply(const float* __restrict__ x, const float* __restrict__ dy, const float* __restrict__ mean,
                             const float* __restrict__ coef, float* __restrict__ dx, uint16_t* __restrict__ dx16,
                             int64_t n, int C) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        int c = (int)(i % C);
        const float v = coef[c] * dy[i] + coef[C + c] * (x[i] - mean[c]) + coef[2 * C + c];
        dx[i] = v;
        if (dx16 != nullptr) {
            const unsigned u = __float_as_uint(v);
            dx16[i] = (uint16_t)(((u & 0x7fffffffu) > 0x7f800000u) ? ((u >> 16) | 0x40u)
                                                                   : ((u + 0x7fffu + ((u >> 16) & 1u)) >> 16));
        }
    }
}

// ---- elementwise ---------------------------------------------------------------------
// (16-byte loads and stores over the aligned part when both pointers allow it, single floats for the rest)
__global__ void relu_fwd_kernel(const float* __restrict__ x, float* __restrict__ y, float alpha, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t done = 0;
    if (((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0) {
        const int64_t n4 = n >> 2;
        const ew_f4* __restrict__ x4 = reinterpret_cast<const ew_f4*>(x);
        ew_f4* __restrict__ y4 = reinterpret_cast<ew_f4*>(y);
        for (int64_t j = i; j < n4; j += stride) {
            const ew_f4 v = x4[j];
            ew_f4 r;
#pragma unroll
            for (int e = 0; e < 4; ++e) r[e] = v[e] > 0.f ? v[e] : alpha * v[e];
            y4[j] = r;
        }
        done = n4 << 2;
    }
    for (i += done; i < n; i += stride) {
        float v = x[i];
        y[i] = v > 0.f ? v : alpha * v;
    }
}

__global__ void relu_bwd_kernel(const float* __restrict__ x, const float* __restrict__ dy, float* __restrict__ dx,
                                float alpha, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dx[i] = x[i] < 0.f ? alpha * dy[i] : dy[i];
}

__global__ void mul_mask_kernel(const float* __restrict__ x, const float* __restrict__ mask, float* __restrict__ y,
                                int64_t n, int64_t mask_n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) y[i] = x[i] * mask[i % mask_n];
}

__global__ void axpy_kernel(float alpha, const float* __restrict__ x, float* __restrict__ y, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) y[i] += alpha * x[i];
}

__global__ void l1_grad_kernel(float lambda, const float* __restrict__ w, float* __restrict__ dw, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dw[i] += w[i] < 0.f ? -lambda : lambda;
}

// float32 -> bfloat16 bits, round to nearest even; NaN stays NaN
__device__ __forceinline__ unsigned bf16_bits(float f) {
    const unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
typedef unsigned ew_u2 __attribute__((ext_vector_type(2)));
typedef unsigned ew_u4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ ew_u2 pack_bf16x4(const ew_f4& v) {
    return ew_u2{bf16_bits(v[0]) | (bf16_bits(v[1]) << 16), bf16_bits(v[2]) | (bf16_bits(v[3]) << 16)};
}

__global__ void cast_bf16_kernel(const float* __restrict__ src, uint16_t* __restrict__ dst, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = (uint16_t)bf16_bits(src[i]);
}

// 8 elements per thread: two 16-byte loads, one 16-byte store (n8 = n / 8 groups)
__global__ __launch_bounds__(kEwThreads) void cast_bf16_kernel8(const ew_f4* __restrict__ src, ew_u4* __restrict__ dst,
                                                               int64_t n8) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n8; i += stride) {
        const ew_f4 a = src[2 * i], b = src[2 * i + 1];
        const ew_u2 lo = pack_bf16x4(a), hi = pack_bf16x4(b);
        dst[i] = ew_u4{lo[0], lo[1], hi[0], hi[1]};
    }
}

// ReLU / leaky ReLU on groups of 4 that also leaves a bfloat16 copy of its output (for a
// bf16 convolution that reads it next: the copy costs 2 bytes per element here instead of a
// cast pass of 6)
__global__ __launch_bounds__(kEwThreads) void relu_fwd_twin_kernel4(const ew_f4* __restrict__ x, ew_f4* __restrict__ y,
                                                                   ew_u2* __restrict__ y16, float alpha, int64_t n4) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += stride) {
        const ew_f4 v = x[i];
        ew_f4 r;
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = v[e] > 0.f ? v[e] : alpha * v[e];
        y[i] = r;
        y16[i] = pack_bf16x4(r);
    }
}

__global__ void relu_fwd_twin_kernel(const float* __restrict__ x, float* __restrict__ y, uint16_t* __restrict__ y16,
                                     float alpha, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        const float v = x[i];
        const float r = v > 0.f ? v : alpha * v;
        y[i] = r;
        y16[i] = (uint16_t)bf16_bits(r);
    }
}

__global__ void adam_kernel(float* __restrict__ theta, const float* __restrict__ g, float* __restrict__ m,
                            float* __restrict__ v, int64_t n, float lr, float b1, float b2, float eps, float c1,
                            float c2) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        float gi = g[i];
        float mi = b1 * m[i] + (1.0f - b1) * gi;
        float vi = b2 * v[i] + (1.0f - b2) * (gi * gi);
        m[i] = mi;
        v[i] = vi;
        float mh = mi / c1;
        float vh = vi / c2;
        theta[i] += -lr * mh / (sqrtf(vh) + eps);
    }
}

constexpr int kAdamMax = 32;
struct AdamTable {
    float* theta[kAdamMax];
    const float* grad[kAdamMax];
    float* m[kAdamMax];
    float* v[kAdamMax];
    int64_t n[kAdamMax];
};

// blockIdx.y selects the tensor, blockIdx.x strides over its elements
__global__ void adam_multi_kernel(const AdamTable tb, float lr, float b1, float b2, float eps, float c1, float c2) {
    const int t = blockIdx.y;
    float* __restrict__ theta = tb.theta[t];
    const float* __restrict__ g = tb.grad[t];
    float* __restrict__ m = tb.m[t];
    float* __restrict__ v = tb.v[t];
    const int64_t n = tb.n[t];
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        float gi = g[i];
        float mi = b1 * m[i] + (1.0f - b1) * gi;
        float vi = b2 * v[i] + (1.0f - b2) * (gi * gi);
        m[i] = mi;
        v[i] = vi;
        float mh = mi / c1;
        float vh = vi / c2;
        theta[i] += -lr * mh / (sqrtf(vh) + eps);
    }
}

// Adam with its step state on the device, for callers that replay a recorded step and
// cannot pass a new step number from the host.  state = {t, beta1^t, beta2^t, lr_t} as
// doubles.  adam_state_step advances it by one step; adam_multi_dev_kernel reads it.
__global__ void adam_state_step_kernel(double* __restrict__ state, double lr, double decay, double b1, double b2) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        const double t = state[0];
        state[3] = decay != 0.0 ? lr * (1.0 / (1.0 + decay * t)) : lr;   // learning rate of this step
        state[0] = t + 1.0;
        state[1] *= b1;
        state[2] *= b2;
    }
}

__global__ void adam_multi_dev_kernel(const AdamTable tb, float b1, float b2, float eps,
                                      const double* __restrict__ state) {
    const float lr = (float)state[3];
    const float c1 = (float)(1.0 - state[1]);
    const float c2 = (float)(1.0 - state[2]);
    const int t = blockIdx.y;
    float* __restrict__ theta = tb.theta[t];
    const float* __restrict__ g = tb.grad[t];
    float* __restrict__ m = tb.m[t];
    float* __restrict__ v = tb.v[t];
    const int64_t n = tb.n[t];
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        float gi = g[i];
        float mi = b1 * m[i] + (1.0f - b1) * gi;
        float vi = b2 * v[i] + (1.0f - b2) * (gi * gi);
        m[i] = mi;
        v[i] = vi;
        float mh = mi / c1;
        float vh = vi / c2;
        theta[i] += -lr * mh / (sqrtf(vh) + eps);
    }
}

// single block: out[0] = sum |x| (mode 0), sum x^2 (1) or sum x (2), summed in a fixed tree
__global__ __launch_bounds__(1024) void reduce_kernel(const float* __restrict__ x, int64_t n, int mode,
                                                      float* __restrict__ out) {
    __shared__ float red[1024];
    float s = 0.f;
    for (int64_t i = threadIdx.x; i < n; i += 1024) {
        float v = x[i];
        s += mode == 0 ? fabsf(v) : (mode == 1 ? v * v : v);
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (int w = 512; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) out[0] = red[0];
}

// the same sums over `chunk` consecutive elements per block, one partial each: the first stage for long inputs
// (the chunk size follows from n alone, so the order of the additions does too)
__global__ __launch_bounds__(256) void reduce_chunks_kernel(const float* __restrict__ x, int64_t n, int64_t chunk, int mode,
                                                            float* __restrict__ part) {
    __shared__ float red[256];
    const int64_t lo = (int64_t)blockIdx.x * chunk;
    const int64_t hi = lo + chunk < n ? lo + chunk : n;
    float s = 0.f;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) {
        float v = x[i];
        s += mode == 0 ? fabsf(v) : v * v;
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) part[blockIdx.x] = red[0];
}

// ---- pooling ---------------------------------------------------------------------------
struct PoolParams {
    int S, H, W, C, Ho, Wo, fH, fW, sH, sW;
    FastDiv div_c, div_w, div_h, div_sh, div_sw;   // tensors are below 2^31 elements: 32-bit index arithmetic
};

__global__ void maxpool_fwd_kernel(const float* __restrict__ x, float* __restrict__ y, uint8_t* __restrict__ idx,
                                   PoolParams p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        int c = (int)(i % p.C);
        int64_t t = i / p.C;
        int wo = (int)(t % p.Wo);
        t /= p.Wo;
        int ho = (int)(t % p.Ho);
        int s = (int)(t / p.Ho);
        const float* base = x + (((size_t)s * p.H + (size_t)ho * p.sH) * p.W + (size_t)wo * p.sW) * p.C + c;
        float best = base[0];
        int bi = 0;
        for (int fh = 0; fh < p.fH; ++fh)
            for (int fw = 0; fw < p.fW; ++fw) {
                float v = base[((size_t)fh * p.W + fw) * p.C];
                if (v > best) {          // strict: the first maximum keeps its place
                    best = v;
                    bi = fh * p.fW + fw;
                }
            }
        y[i] = best;
        idx[i] = (uint8_t)bi;
    }
}

// 4 neighbouring channels per thread (C % 4 == 0, 16-byte aligned tensors, 4-byte aligned idx): 16-byte loads, the same
// comparisons in the same order per channel.  p.div_c divides by C / 4, p.div_w by Wo, p.div_h by Ho here.
__global__ void maxpool_fwd_kernel4(const ew_f4* __restrict__ x, ew_f4* __restrict__ y, uint32_t* __restrict__ idx,
                                    PoolParams p, unsigned n4) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const unsigned C4 = (unsigned)p.C >> 2;
    unsigned t, u, c, wo, ho, s;
    p.div_c.divmod(i, t, c);
    p.div_w.divmod(t, u, wo);
    p.div_h.divmod(u, s, ho);
    const ew_f4* base = x + ((s * p.H + ho * p.sH) * p.W + wo * p.sW) * C4 + c;
    ew_f4 best = base[0];
    uint32_t bi = 0;
    for (int fh = 0; fh < p.fH; ++fh)
        for (int fw = 0; fw < p.fW; ++fw) {
            const ew_f4 v = base[(fh * p.W + fw) * C4];
            const uint32_t k = (uint32_t)(fh * p.fW + fw);
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (v[e] > best[e]) {    // strict: the first maximum keeps its place
                    best[e] = v[e];
                    bi = (bi & ~(0xffu << (8 * e))) | (k << (8 * e));
                }
        }
    y[i] = best;
    idx[i] = bi;
}

__global__ void avgpool_fwd_kernel4(const ew_f4* __restrict__ x, ew_f4* __restrict__ y, PoolParams p, unsigned n4) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const unsigned C4 = (unsigned)p.C >> 2;
    const float inv = 1.0f / (float)(p.fH * p.fW);
    unsigned t, u, c, wo, ho, s;
    p.div_c.divmod(i, t, c);
    p.div_w.divmod(t, u, wo);
    p.div_h.divmod(u, s, ho);
    const ew_f4* base = x + ((s * p.H + ho * p.sH) * p.W + wo * p.sW) * C4 + c;
    ew_f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int fh = 0; fh < p.fH; ++fh)
        for (int fw = 0; fw < p.fW; ++fw) acc += base[(fh * p.W + fw) * C4];
    y[i] = acc * inv;
}

// gather form of the scatter-add: every input element sums, in (h,w) order, the
// windows that contain it and whose argmax points at it
__global__ void maxpool_bwd_kernel(const float* __restrict__ dy, const uint8_t* __restrict__ idx,
                                   float* __restrict__ dx, PoolParams p, int64_t n) {
    unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    const unsigned stride = gridDim.x * blockDim.x;
    for (; i < (unsigned)n; i += stride) {
        unsigned t, u, c, col, row, s;
        p.div_c.divmod(i, t, c);
        p.div_w.divmod(t, u, col);
        p.div_h.divmod(u, s, row);
        int h_lo = (int)row - p.fH + 1;
        h_lo = h_lo <= 0 ? 0 : (int)p.div_sh.div((unsigned)(h_lo + p.sH - 1));
        int h_hi = (int)p.div_sh.div(row);
        if (h_hi > p.Ho - 1) h_hi = p.Ho - 1;
        int w_lo = (int)col - p.fW + 1;
        w_lo = w_lo <= 0 ? 0 : (int)p.div_sw.div((unsigned)(w_lo + p.sW - 1));
        int w_hi = (int)p.div_sw.div(col);
        if (w_hi > p.Wo - 1) w_hi = p.Wo - 1;
        float acc = 0.f;
        for (int h = h_lo; h <= h_hi; ++h)
            for (int w = w_lo; w <= w_hi; ++w) {
                const unsigned o = ((s * p.Ho + h) * p.Wo + w) * p.C + c;
                const int want = ((int)row - h * p.sH) * p.fW + ((int)col - w * p.sW);
                if ((int)idx[o] == want) acc += dy[o];
            }
        dx[i] = acc;
    }
}

// The same for 4 neighbouring channels per thread (C % 4 == 0, 16-byte aligned tensors): 16-byte loads and stores,
// 4-byte index loads; every element takes the sums of the scalar form in the same order.  p.div_c divides by C / 4.
__global__ void maxpool_bwd_kernel4(const ew_f4* __restrict__ dy, const uint32_t* __restrict__ idx,
                                    ew_f4* __restrict__ dx, PoolParams p, unsigned n4) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const unsigned C4 = (unsigned)p.C >> 2;
    unsigned t, u, c, col, row, s;
    p.div_c.divmod(i, t, c);
    p.div_w.divmod(t, u, col);
    p.div_h.divmod(u, s, row);
    int h_lo = (int)row - p.fH + 1;
    h_lo = h_lo <= 0 ? 0 : (int)p.div_sh.div((unsigned)(h_lo + p.sH - 1));
    int h_hi = (int)p.div_sh.div(row);
    if (h_hi > p.Ho - 1) h_hi = p.Ho - 1;
    int w_lo = (int)col - p.fW + 1;
    w_lo = w_lo <= 0 ? 0 : (int)p.div_sw.div((unsigned)(w_lo + p.sW - 1));
    int w_hi = (int)p.div_sw.div(col);
    if (w_hi > p.Wo - 1) w_hi = p.Wo - 1;
    ew_f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int h = h_lo; h <= h_hi; ++h)
        for (int w = w_lo; w <= w_hi; ++w) {
            const unsigned o = ((s * p.Ho + h) * p.Wo + w) * C4 + c;
            const unsigned want = (unsigned)(((int)row - h * p.sH) * p.fW + ((int)col - w * p.sW));
            const uint32_t k = idx[o];
            const ew_f4 g = dy[o];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (((k >> (8 * e)) & 0xffu) == want) acc[e] += g[e];
        }
    dx[i] = acc;
}

__global__ void avgpool_bwd_kernel4(const ew_f4* __restrict__ dy, ew_f4* __restrict__ dx, PoolParams p, unsigned n4) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n4) return;
    const unsigned C4 = (unsigned)p.C >> 2;
    const float div = (float)(p.fH * p.fW);
    unsigned t, u, c, col, row, s;
    p.div_c.divmod(i, t, c);
    p.div_w.divmod(t, u, col);
    p.div_h.divmod(u, s, row);
    int h_lo = (int)row - p.fH + 1;
    h_lo = h_lo <= 0 ? 0 : (int)p.div_sh.div((unsigned)(h_lo + p.sH - 1));
    int h_hi = (int)p.div_sh.div(row);
    if (h_hi > p.Ho - 1) h_hi = p.Ho - 1;
    int w_lo = (int)col - p.fW + 1;
    w_lo = w_lo <= 0 ? 0 : (int)p.div_sw.div((unsigned)(w_lo + p.sW - 1));
    int w_hi = (int)p.div_sw.div(col);
    if (w_hi > p.Wo - 1) w_hi = p.Wo - 1;
    ew_f4 acc = {0.f, 0.f, 0.f, 0.f};
    for (int h = h_lo; h <= h_hi; ++h)
        for (int w = w_lo; w <= w_hi; ++w) {
            const ew_f4 g = dy[((s * p.Ho + h) * p.Wo + w) * C4 + c];
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[e] += g[e] / div;
        }
    dx[i] = acc;
}

__global__ void avgpool_fwd_kernel(const float* __restrict__ x, float* __restrict__ y, PoolParams p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const float inv = 1.0f / (float)(p.fH * p.fW);
    for (; i < n; i += stride) {
        int c = (int)(i % p.C);
        int64_t t = i / p.C;
        int wo = (int)(t % p.Wo);
        t /= p.Wo;
        int ho = (int)(t % p.Ho);
        int s = (int)(t / p.Ho);
        const float* base = x + (((size_t)s * p.H + (size_t)ho * p.sH) * p.W + (size_t)wo * p.sW) * p.C + c;
        float acc = 0.f;
        for (int fh = 0; fh < p.fH; ++fh)
            for (int fw = 0; fw < p.fW; ++fw) acc += base[((size_t)fh * p.W + fw) * p.C];
        y[i] = acc * inv;
    }
}

__global__ void avgpool_bwd_kernel(const float* __restrict__ dy, float* __restrict__ dx, PoolParams p, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const float div = (float)(p.fH * p.fW);
    for (; i < n; i += stride) {
        int c = (int)(i % p.C);
        int64_t t = i / p.C;
        int col = (int)(t % p.W);
        t /= p.W;
        int row = (int)(t % p.H);
        int s = (int)(t / p.H);
        int h_lo = row - p.fH + 1;
        h_lo = h_lo <= 0 ? 0 : (h_lo + p.sH - 1) / p.sH;
        int h_hi = row / p.sH;
        if (h_hi > p.Ho - 1) h_hi = p.Ho - 1;
        int w_lo = col - p.fW + 1;
        w_lo = w_lo <= 0 ? 0 : (w_lo + p.sW - 1) / p.sW;
        int w_hi = col / p.sW;
        if (w_hi > p.Wo - 1) w_hi = p.Wo - 1;
        float acc = 0.f;
        for (int h = h_lo; h <= h_hi; ++h)
            for (int w = w_lo; w <= w_hi; ++w) acc += dy[(((size_t)s * p.Ho + h) * p.Wo + w) * p.C + c] / div;
        dx[i] = acc;
    }
}

// ---- softmax / cross entropy (one thread per row; K is the class count) -----------------
__global__ void softmax_kernel(const float* __restrict__ logits, float* __restrict__ probs, int rows, int K) {
    int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const float* in = logits + (size_t)r * K;
    float* out = probs + (size_t)r * K;
    float mx = in[0];
    for (int k = 1; k < K; ++k) mx = fmaxf(mx, in[k]);
    float sum = 0.f;
    for (int k = 0; k < K; ++k) {
        float e = expf(in[k] - mx);
        out[k] = e;
        sum += e;
    }
    for (int k = 0; k < K; ++k) out[k] = out[k] / sum;
}

__global__ void softmax_bwd_kernel(const float* __restrict__ probs, const float* __restrict__ dy,
                                   float* __restrict__ dx, int rows, int K) {
    int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const float* p = probs + (size_t)r * K;
    const float* g = dy + (size_t)r * K;
    float dot = 0.f;
    for (int k = 0; k < K; ++k) dot += p[k] * g[k];
    for (int k = 0; k < K; ++k) dx[(size_t)r * K + k] = p[k] * (g[k] - dot);
}

// The target row of a sample: class indices (the one-hot row of labels[r]) or a dense row of K floats given by
// the caller (soft or already smoothed targets, CNN_classes_cupy.py:622-626 uses a 2-D y_true as it is).  Label
// smoothing is the reference's t (1 - ls) + ls / K (:626-628) in both forms; for a one-hot row the dense form
// gives the very floats of the index form.
struct IndexTargets {
    const int32_t* __restrict__ labels;
    __device__ __forceinline__ float at(int r, int k, float ls, float t_off) const {
        return (k == labels[r]) ? (1.0f - ls) + t_off : t_off;
    }
};
struct DenseTargets {
    const float* __restrict__ t;
    int K;
    __device__ __forceinline__ float at(int r, int k, float ls, float t_off) const {
        return t[(size_t)r * K + k] * (1.0f - ls) + t_off;
    }
};

template <typename Targets>
__global__ void cce_fwd_kernel(const float* __restrict__ probs, const Targets tg, float ls,
                               float* __restrict__ loss, int32_t* __restrict__ pred, int rows, int K) {
    int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const float* p = probs + (size_t)r * K;
    const float t_off = ls / (float)K;
    float acc = 0.f;
    float best = p[0];
    int bi = 0;
    for (int k = 0; k < K; ++k) {
        float v = p[k];
        if (v > best) {
            best = v;
            bi = k;
        }
        float pc = fminf(fmaxf(v, 1e-7f), 1.0f - 1e-7f);
        acc += tg.at(r, k, ls, t_off) * logf(pc);
    }
    loss[r] = -acc;
    pred[r] = bi;
}

template <typename Targets>
__global__ void softmax_cce_bwd_kernel(const float* __restrict__ probs, const Targets tg, float ls,
                                       float* __restrict__ dlogits, int rows, int K) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= rows * K) return;
    int r = i / K, k = i - r * K;
    const float t_off = ls / (float)K;
    dlogits[i] = (probs[i] - tg.at(r, k, ls, t_off)) / (float)rows;
}

// softmax, the loss with the row argmax and the gradient of the logits in one pass over a row: the three kernels above
// one after the other, with the same operations in the same order (a training step's classifier head)
template <typename Targets>
__global__ void softmax_cce_train_kernel(const float* __restrict__ logits, const Targets tg, float ls,
                                         float* __restrict__ probs, float* __restrict__ loss, int32_t* __restrict__ pred,
                                         float* __restrict__ dlogits, int rows, int K) {
    int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= rows) return;
    const float* in = logits + (size_t)r * K;
    float* out = probs + (size_t)r * K;
    float* dl = dlogits + (size_t)r * K;
    float mx = in[0];
    for (int k = 1; k < K; ++k) mx = fmaxf(mx, in[k]);
    float sum = 0.f;
    for (int k = 0; k < K; ++k) {
        float e = expf(in[k] - mx);
        out[k] = e;
        sum += e;
    }
    const float t_off = ls / (float)K;
    float acc = 0.f;
    float best = 0.f;
    int bi = 0;
    for (int k = 0; k < K; ++k) {
        const float v = out[k] / sum;
        out[k] = v;
        if (k == 0 || v > best) {
            best = v;
            bi = k;
        }
        const float pc = fminf(fmaxf(v, 1e-7f), 1.0f - 1e-7f);
        const float t = tg.at(r, k, ls, t_off);
        acc += t * logf(pc);
        dl[k] = (v - t) / (float)rows;
    }
    loss[r] = -acc;
    pred[r] = bi;
}

// The same for at most 16 classes with 16 lanes per row: the exponentials and logarithms of a row are worked out side by
// side, the sums are added by the row's first lane in the order of the one-thread form (same bits).
template <typename Targets>
__global__ void softmax_cce_train16_kernel(const float* __restrict__ logits, const Targets tg, float ls,
                                           float* __restrict__ probs, float* __restrict__ loss, int32_t* __restrict__ pred,
                                           float* __restrict__ dlogits, int rows, int K) {
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    const int r = min(t >> 4, rows - 1), k = t & 15;     // (rows past the end repeat the last one: every lane takes part in the exchanges)
    const bool mine = k < K;
    const int base = (threadIdx.x & 63) & ~15;           // first lane of the row inside the wave
    const float in = mine ? logits[(size_t)r * K + k] : 0.0f;
    float mx = __shfl(in, base, 64);
    for (int j = 1; j < K; ++j) mx = fmaxf(mx, __shfl(in, base + j, 64));
    const float e = expf(in - mx);
    float sum = 0.f;
    for (int j = 0; j < K; ++j) sum += __shfl(e, base + j, 64);
    const float v = e / sum;
    const float t_off = ls / (float)K;
    const float tk = mine ? tg.at(r, k, ls, t_off) : t_off;
    const float term = tk * logf(fminf(fmaxf(v, 1e-7f), 1.0f - 1e-7f));
    float acc = 0.f, best = 0.f;
    int bi = 0;
    for (int j = 0; j < K; ++j) {
        const float vj = __shfl(v, base + j, 64);
        if (j == 0 || vj > best) {
            best = vj;
            bi = j;
        }
        acc += __shfl(term, base + j, 64);
    }
    if ((t >> 4) >= rows) return;
    if (mine) {
        probs[(size_t)r * K + k] = v;
        dlogits[(size_t)r * K + k] = (v - tk) / (float)rows;
    }
    if (k == 0) {
        loss[r] = -acc;
        pred[r] = bi;
    }
}

static int pool_dims(const char* fn, int S, int H, int W, int C, int fH, int fW, int sH, int sW, PoolParams* p) {
    if (S <= 0 || H <= 0 || W <= 0 || C <= 0 || fH <= 0 || fW <= 0 || sH <= 0 || sW <= 0)
        return fail(AETH_E_INVALID, "%s: non-positive dimension", fn);
    if (fH > H || fW > W) return fail(AETH_E_INVALID, "%s: window larger than input", fn);
    if (fH * fW > 256) return fail(AETH_E_INVALID, "%s: window larger than 256 elements", fn);
    p->S = S; p->H = H; p->W = W; p->C = C; p->fH = fH; p->fW = fW; p->sH = sH; p->sW = sW;
    p->Ho = (H - fH) / sH + 1;
    p->Wo = (W - fW) / sW + 1;
    if ((int64_t)S * H * W * C >= ((int64_t)1 << 31)) return fail(AETH_E_INVALID, "%s: tensor too large", fn);
    p->div_c = FastDiv(C); p->div_w = FastDiv(W); p->div_h = FastDiv(H); p->div_sh = FastDiv(sH); p->div_sw = FastDiv(sW);
    return AETH_OK;
}

static void adam_corrections(float beta1, float beta2, int t, float* c1, float* c2) {
    // 1 - beta^(t+1) by repeated squaring in double
    double p1 = 1.0, p2 = 1.0, b1 = beta1, b2 = beta2;
    for (unsigned e = (unsigned)t + 1; e; e >>= 1) {
        if (e & 1) { p1 *= b1; p2 *= b2; }
        b1 *= b1; b2 *= b2;
    }
    *c1 = (float)(1.0 - p1);
    *c2 = (float)(1.0 - p2);
}

}  // namespace aeth

using namespace aeth;

// ---- batch norm + (leaky) ReLU + 2x2 stride-2 max pooling in one pass ----------------
// The three layers of a convolution block read and write the same tensor three times
// over.  One thread takes a pooling window and 4 channels: it reads the 4 pixels once
// and writes what each layer would have written (the layers keep their outputs for
// the backward pass and for callers that look at them).  H and W even, C % 4 == 0.
struct Pool2Params {
    int S, H, W, C4, Ho, Wo;
    FastDiv div_c4, div_wo, div_ho;
};

__global__ __launch_bounds__(kEwThreads) void bn_relu_maxpool2_fwd_kernel(
    const ew_f4* __restrict__ x, const ew_f4* __restrict__ gamma, const ew_f4* __restrict__ beta,
    const ew_f4* __restrict__ mean, const ew_f4* __restrict__ invstd, ew_f4* __restrict__ bn_out,
    ew_f4* __restrict__ relu_out, ew_f4* __restrict__ pool_out, ew_u2* __restrict__ pool_out16,
    uint32_t* __restrict__ idx, float alpha, Pool2Params p, unsigned n) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    unsigned t, c4, u, wo, s, ho;
    p.div_c4.divmod(i, t, c4);
    p.div_wo.divmod(t, u, wo);
    p.div_ho.divmod(u, s, ho);
    const unsigned base = ((s * p.H + 2u * ho) * p.W + 2u * wo) * p.C4 + c4;
    const ew_f4 g = gamma[c4], b = beta[c4], m = mean[c4], is = invstd[c4];
    ew_f4 best;
    unsigned bi = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const unsigned off = base + ((unsigned)(k >> 1) * p.W + (unsigned)(k & 1)) * p.C4;
        const ew_f4 v = x[off];
        ew_f4 y, r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            y[e] = g[e] * ((v[e] - m[e]) * is[e]) + b[e];
            r[e] = y[e] > 0.f ? y[e] : alpha * y[e];
        }
        bn_out[off] = y;
        relu_out[off] = r;
        if (k == 0) {
            best = r;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (r[e] > best[e]) {        // strict: the first maximum keeps its place
                    best[e] = r[e];
                    bi = (bi & ~(0xffu << (8 * e))) | ((unsigned)k << (8 * e));
                }
        }
    }
    pool_out[i] = best;
    if (pool_out16 != nullptr) pool_out16[i] = pack_bf16x4(best);
    idx[i] = bi;
}

// backward of the pooling and the ReLU of such a block: every pixel belongs to one window
__global__ __launch_bounds__(kEwThreads) void maxpool2_relu_bwd_kernel(
    const ew_f4* __restrict__ dy, const uint32_t* __restrict__ idx, const ew_f4* __restrict__ relu_in,
    ew_f4* __restrict__ pool_dx, ew_f4* __restrict__ relu_dx, float alpha, Pool2Params p, unsigned n) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    unsigned t, c4, u, wo, s, ho;
    p.div_c4.divmod(i, t, c4);
    p.div_wo.divmod(t, u, wo);
    p.div_ho.divmod(u, s, ho);
    const unsigned base = ((s * p.H + 2u * ho) * p.W + 2u * wo) * p.C4 + c4;
    const ew_f4 g = dy[i];
    const unsigned bi = idx[i];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const unsigned off = base + ((unsigned)(k >> 1) * p.W + (unsigned)(k & 1)) * p.C4;
        const ew_f4 xin = relu_in[off];
        ew_f4 d, r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            d[e] = ((bi >> (8 * e)) & 0xffu) == (unsigned)k ? g[e] : 0.f;
            r[e] = xin[e] < 0.f ? alpha * d[e] : d[e];
        }
        pool_dx[off] = d;
        relu_dx[off] = r;
    }
}

// The same backward pass with the batch norm's column sums taken on the way: s1 = sum dz,
// s2 = sum dz * (x - mean) over the rows, dz = the activation's input gradient.  A thread
// keeps its channel group over the windows it walks (the stride is a multiple of C4) and
// the threads of a block that share a group are added through LDS in a fixed order: the
// partials land in the part[v][block][c] layout of bn_bwd_final.  256 % C4 == 0.
__global__ __launch_bounds__(kEwThreads) void maxpool2_relu_bnpart_bwd_kernel(
    const ew_f4* __restrict__ dy, const uint32_t* __restrict__ idx, const ew_f4* __restrict__ relu_in,
    const ew_f4* __restrict__ x, const ew_f4* __restrict__ mean, ew_f4* __restrict__ pool_dx,
    ew_f4* __restrict__ relu_dx, float* __restrict__ part, float alpha, Pool2Params p, unsigned n) {
    __shared__ ew_f4 red[2][kEwThreads];
    const unsigned tid = threadIdx.x;
    const unsigned stride = gridDim.x * blockDim.x;
    const unsigned c4 = tid % (unsigned)p.C4;            // the same for every window of this thread
    const ew_f4 mu = mean[c4];
    ew_f4 s1 = {0.f, 0.f, 0.f, 0.f}, s2 = {0.f, 0.f, 0.f, 0.f};
    for (unsigned i = blockIdx.x * blockDim.x + tid; i < n; i += stride) {
        unsigned t, u, wo, s, ho;
        t = p.div_c4.div(i);
        p.div_wo.divmod(t, u, wo);
        p.div_ho.divmod(u, s, ho);
        const unsigned base = ((s * p.H + 2u * ho) * p.W + 2u * wo) * p.C4 + c4;
        const ew_f4 g = dy[i];
        const unsigned bi = idx[i];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const unsigned off = base + ((unsigned)(k >> 1) * p.W + (unsigned)(k & 1)) * p.C4;
            const ew_f4 xin = relu_in[off];
            const ew_f4 xv = x[off];
            ew_f4 d, r;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                d[e] = ((bi >> (8 * e)) & 0xffu) == (unsigned)k ? g[e] : 0.f;
                r[e] = xin[e] < 0.f ? alpha * d[e] : d[e];
            }
            pool_dx[off] = d;
            relu_dx[off] = r;
            s1 += r;
            s2 += r * (xv - mu);
        }
    }
    red[0][tid] = s1;
    red[1][tid] = s2;
    __syncthreads();
    if (tid < (unsigned)p.C4) {
        ew_f4 a = {0.f, 0.f, 0.f, 0.f}, b = {0.f, 0.f, 0.f, 0.f};
        for (unsigned r = tid; r < kEwThreads; r += (unsigned)p.C4) {
            a += red[0][r];
            b += red[1][r];
        }
        const int C = 4 * p.C4;
        *reinterpret_cast<ew_f4*>(part + (size_t)blockIdx.x * C + 4 * tid) = a;
        *reinterpret_cast<ew_f4*>(part + ((size_t)gridDim.x + blockIdx.x) * C + 4 * tid) = b;
    }
}

// dx = coef0 * dy + A * (x - mean) + B on groups of 4 channels
__global__ __launch_bounds__(kEwThreads) void bn_bwd_apply4(const ew_f4* __restrict__ x, const ew_f4* __restrict__ dy,
                                                           const ew_f4* __restrict__ mean, const float* __restrict__ coef,
                                                           ew_f4* __restrict__ dx, ew_u2* __restrict__ dx16,
                                                           unsigned n4, int C4) {
    const unsigned stride = gridDim.x * blockDim.x;
    const ew_f4* c0 = reinterpret_cast<const ew_f4*>(coef);
    for (unsigned i = blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) {
        const unsigned c4 = i % (unsigned)C4;
        const ew_f4 v = c0[c4] * dy[i] + c0[C4 + c4] * (x[i] - mean[c4]) + c0[2 * C4 + c4];
        dx[i] = v;
        if (dx16 != nullptr) dx16[i] = pack_bf16x4(v);
    }
}

#define EW_LAUNCH(kernel, n, ...)                                                          \
    do {                                                                                   \
        hipLaunchKernelGGL(kernel, dim3(ew_blocks(n)), dim3(kEwThreads), 0, ctx().stream, __VA_ARGS__); \
        AETH_LAUNCH_CHECK();                                                               \
    } while (0)

extern "C" {

int aeth_bn_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* running_mean,
                          float* running_var, float* save_mean, float* save_invstd, float* y, int rows, int C,
                          float eps, float momentum) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x && gamma && beta && running_mean && running_var && save_mean && save_invstd && y);
    AETH_CHECK_ARG(rows > 0 && C > 0 && (int64_t)rows * C < ((int64_t)1 << 31));
    int nblk, rpb;
    dim3 grid;
    col_grid(rows, C, &nblk, &rpb, &grid);
    void* ws;
    int rc = workspace((int64_t)2 * nblk * C * sizeof(float), &ws);
    if (rc) return rc;
    float* part = (float*)ws;
    hipStream_t st = ctx().stream;
    if (col_vec4(C, x, part)) {
        hipLaunchKernelGGL(bn_stats_partial4, dim3(grid.x, cdiv(C / 4, 64)), dim3(kEwThreads), 0, st, x, rows, C, rpb, part);
    } else {
        hipLaunchKernelGGL(bn_stats_partial, grid, dim3(kEwThreads), 0, st, x, rows, C, rpb, part);
    }
    AETH_LAUNCH_CHECK();
    hipLaunchKernelGGL(bn_stats_final, dim3(cdiv(C, 64)), dim3(256), 0, st, x, part, nblk, rows, C, eps, momentum,
                       running_mean, running_var, save_mean, save_invstd);
    AETH_LAUNCH_CHECK();
    int64_t n = (int64_t)rows * C;
    if (col_vec4(C, x, y) && col_vec4(C, gamma, beta) && col_vec4(C, save_mean, save_invstd)) {
        const unsigned n4 = (unsigned)(n / 4);
        hipLaunchKernelGGL(bn_apply4, dim3(ew_blocks(n4)), dim3(kEwThreads), 0, st, (const ew_f4*)x, (const ew_f4*)gamma,
                           (const ew_f4*)beta, (const ew_f4*)save_mean, (const ew_f4*)save_invstd, (ew_f4*)y, n4, C / 4);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    EW_LAUNCH(bn_apply, n, x, gamma, beta, save_mean, save_invstd, y, n, C);
    return AETH_OK;
}

static int pool2_params(int S, int H, int W, int C, Pool2Params* p, unsigned* n) {
    if (S <= 0 || H <= 0 || W <= 0 || C <= 0 || H % 2 != 0 || W % 2 != 0 || C % 4 != 0) return AETH_E_INVALID;
    if ((int64_t)S * H * W * C >= ((int64_t)1 << 31)) return AETH_E_INVALID;
    p->S = S; p->H = H; p->W = W; p->C4 = C / 4; p->Ho = H / 2; p->Wo = W / 2;
    p->div_c4 = FastDiv(p->C4);
    p->div_wo = FastDiv(p->Wo);
    p->div_ho = FastDiv(p->Ho);
    *n = (unsigned)((int64_t)S * p->Ho * p->Wo * p->C4);
    return AETH_OK;
}

static inline bool aligned16(const void* q) { return (reinterpret_cast<uintptr_t>(q) & 15) == 0; }

static int bn_relu_maxpool2_fwd_impl(const float* x, const float* gamma, const float* beta,
                                     float* running_mean, float* running_var, float* save_mean, float* save_invstd,
                                     float* bn_out, float* relu_out, float* pool_out, uint8_t* idx, int S, int H, int W,
                                     int C, float eps, float momentum, float alpha, uint16_t* pool_out_bf16) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x && gamma && beta && running_mean && running_var && save_mean && save_invstd);
    AETH_CHECK_ARG(bn_out && relu_out && pool_out && idx);
    Pool2Params p;
    unsigned n;
    if (pool2_params(S, H, W, C, &p, &n) != AETH_OK)
        return fail(AETH_E_INVALID, "%s: needs even H and W, C %% 4 == 0 and fewer than 2^31 elements", __func__);
    AETH_CHECK_ARG(aligned16(x) && aligned16(gamma) && aligned16(beta) && aligned16(save_mean) &&
                   aligned16(save_invstd) && aligned16(bn_out) && aligned16(relu_out) && aligned16(pool_out) &&
                   aligned16(idx) && aligned16(pool_out_bf16));
    const int rows = S * H * W;
    int nblk, rpb;
    dim3 grid;
    col_grid(rows, C, &nblk, &rpb, &grid);
    void* ws;
    int rc = workspace((int64_t)2 * nblk * C * sizeof(float), &ws);
    if (rc) return rc;
    float* part = (float*)ws;
    hipStream_t st = ctx().stream;
    if (col_vec4(C, x, part)) {
        hipLaunchKernelGGL(bn_stats_partial4, dim3(grid.x, cdiv(C / 4, 64)), dim3(kEwThreads), 0, st, x, rows, C, rpb, part);
    } else {
        hipLaunchKernelGGL(bn_stats_partial, grid, dim3(kEwThreads), 0, st, x, rows, C, rpb, part);
    }
    AETH_LAUNCH_CHECK();
    hipLaunchKernelGGL(bn_stats_final, dim3(cdiv(C, 64)), dim3(256), 0, st, x, part, nblk, rows, C, eps, momentum,
                       running_mean, running_var, save_mean, save_invstd);
    AETH_LAUNCH_CHECK();
    hipLaunchKernelGGL(bn_relu_maxpool2_fwd_kernel, dim3(cdiv(n, kEwThreads)), dim3(kEwThreads), 0, st,
                       (const ew_f4*)x, (const ew_f4*)gamma, (const ew_f4*)beta, (const ew_f4*)save_mean,
                       (const ew_f4*)save_invstd, (ew_f4*)bn_out, (ew_f4*)relu_out, (ew_f4*)pool_out, (ew_u2*)pool_out_bf16,
                       (uint32_t*)idx, alpha, p, n);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

int aeth_bn_relu_maxpool2_fwd_f32(const float* x, const float* gamma, const float* beta, float* running_mean,
                                  float* running_var, float* save_mean, float* save_invstd, float* bn_out,
                                  float* relu_out, float* pool_out, uint8_t* idx, int S, int H, int W, int C,
                                  float eps, float momentum, float alpha) {
    return bn_relu_maxpool2_fwd_impl(x, gamma, beta, running_mean, running_var, save_mean, save_invstd, bn_out, relu_out,
                                     pool_out, idx, S, H, W, C, eps, momentum, alpha, nullptr);
}

int aeth_bn_relu_maxpool2_fwd_twin_f32(const float* x, const float* gamma, const float* beta, float* running_mean,
                                       float* running_var, float* save_mean, float* save_invstd, float* bn_out,
                                       float* relu_out, float* pool_out, uint16_t* pool_out_bf16, uint8_t* idx, int S,
                                       int H, int W, int C, float eps, float momentum, float alpha) {
    AETH_CHECK_ARG(pool_out_bf16 != nullptr);
    return bn_relu_maxpool2_fwd_impl(x, gamma, beta, running_mean, running_var, save_mean, save_invstd, bn_out, relu_out,
                                     pool_out, idx, S, H, W, C, eps, momentum, alpha, pool_out_bf16);
}

int aeth_maxpool2_relu_bwd_f32(const float* dy, const uint8_t* idx, const float* relu_in, float* pool_dx,
                               float* relu_dx, int S, int H, int W, int C, float alpha) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy && idx && relu_in && pool_dx && relu_dx);
    Pool2Params p;
    unsigned n;
    if (pool2_params(S, H, W, C, &p, &n) != AETH_OK)
        return fail(AETH_E_INVALID, "%s: needs even H and W, C %% 4 == 0 and fewer than 2^31 elements", __func__);
    AETH_CHECK_ARG(aligned16(dy) && aligned16(idx) && aligned16(relu_in) && aligned16(pool_dx) && aligned16(relu_dx));
    hipLaunchKernelGGL(maxpool2_relu_bwd_kernel, dim3(cdiv(n, kEwThreads)), dim3(kEwThreads), 0, ctx().stream,
                       (const ew_f4*)dy, (const uint32_t*)idx, (const ew_f4*)relu_in, (ew_f4*)pool_dx, (ew_f4*)relu_dx,
                       alpha, p, n);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

static int maxpool2_relu_bn_bwd_impl(const float* dy, const uint8_t* idx, const float* relu_in, const float* x,
                                     const float* gamma, const float* save_mean, const float* save_invstd,
                                     float* pool_dx, float* relu_dx, float* bn_dx, float* dgamma, float* dbeta,
                                     int S, int H, int W, int C, float alpha, uint16_t* bn_dx_bf16) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy && idx && relu_in && x && gamma && save_mean && save_invstd);
    AETH_CHECK_ARG(pool_dx && relu_dx && bn_dx && dgamma && dbeta);
    Pool2Params p;
    unsigned n;
    if (pool2_params(S, H, W, C, &p, &n) != AETH_OK || kEwThreads % p.C4 != 0)
        return fail(AETH_E_INVALID, "%s: needs even H and W, C / 4 a divisor of %d and fewer than 2^31 elements",
                    __func__, kEwThreads);
    AETH_CHECK_ARG(aligned16(dy) && aligned16(idx) && aligned16(relu_in) && aligned16(x) && aligned16(save_mean) &&
                   aligned16(pool_dx) && aligned16(relu_dx) && aligned16(bn_dx) && aligned16(bn_dx_bf16));
    const int rows = S * H * W;
    int nblk = cdiv(n, kEwThreads);
    if (nblk > 256) nblk = 256;
    void* ws;
    int rc = workspace(((int64_t)2 * nblk * C + 3 * C) * sizeof(float), &ws);
    if (rc) return rc;
    float* part = (float*)ws;
    float* coef = part + (int64_t)2 * nblk * C;
    hipStream_t st = ctx().stream;
    hipLaunchKernelGGL(maxpool2_relu_bnpart_bwd_kernel, dim3(nblk), dim3(kEwThreads), 0, st, (const ew_f4*)dy,
                       (const uint32_t*)idx, (const ew_f4*)relu_in, (const ew_f4*)x, (const ew_f4*)save_mean,
                       (ew_f4*)pool_dx, (ew_f4*)relu_dx, part, alpha, p, n);
    AETH_LAUNCH_CHECK();
    hipLaunchKernelGGL(bn_bwd_final, dim3(cdiv(C, 64)), dim3(256), 0, st, part, nblk, rows, C, gamma, save_invstd,
                       dgamma, dbeta, coef);
    AETH_LAUNCH_CHECK();
    const unsigned n4 = (unsigned)((int64_t)rows * C / 4);
    hipLaunchKernelGGL(bn_bwd_apply4, dim3(ew_blocks(n4)), dim3(kEwThreads), 0, st, (const ew_f4*)x,
                       (const ew_f4*)relu_dx, (const ew_f4*)save_mean, coef, (ew_f4*)bn_dx, (ew_u2*)bn_dx_bf16, n4, C / 4);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

int aeth_maxpool2_relu_bn_bwd_f32(const float* dy, const uint8_t* idx, const float* relu_in, const float* x,
                                  const float* gamma, const float* save_mean, const float* save_invstd,
                                  float* pool_dx, float* relu_dx, float* bn_dx, float* dgamma, float* dbeta,
                                  int S, int H, int W, int C, float alpha) {
    return maxpool2_relu_bn_bwd_impl(dy, idx, relu_in, x, gamma, save_mean, save_invstd, pool_dx, relu_dx, bn_dx, dgamma,
                                     dbeta, S, H, W, C, alpha, nullptr);
}

int aeth_maxpool2_relu_bn_bwd_twin_f32(const float* dy, const uint8_t* idx, const float* relu_in, const float* x,
                                       const float* gamma, const float* save_mean, const float* save_invstd,
                                       float* pool_dx, float* relu_dx, float* bn_dx, uint16_t* bn_dx_bf16,
                                       float* dgamma, float* dbeta, int S, int H, int W, int C, float alpha) {
    AETH_CHECK_ARG(bn_dx_bf16 != nullptr);
    return maxpool2_relu_bn_bwd_impl(dy, idx, relu_in, x, gamma, save_mean, save_invstd, pool_dx, relu_dx, bn_dx, dgamma,
                                     dbeta, S, H, W, C, alpha, bn_dx_bf16);
}

int aeth_bn_fwd_infer_f32(const float* x, const float* gamma, const float* beta, const float* running_mean,
                          const float* running_var, float* y, int rows, int C, float eps) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x && gamma && beta && running_mean && running_var && y);
    AETH_CHECK_ARG(rows > 0 && C > 0 && (int64_t)rows * C < ((int64_t)1 << 31));
    int64_t n = (int64_t)rows * C;
    if (col_vec4(C, x, y) && col_vec4(C, gamma, beta) && col_vec4(C, running_mean, running_var)) {
        const unsigned n4 = (unsigned)(n / 4);
        hipLaunchKernelGGL(bn_apply_infer4, dim3(ew_blocks(n4)), dim3(kEwThreads), 0, ctx().stream, (const ew_f4*)x,
                           (const ew_f4*)gamma, (const ew_f4*)beta, (const ew_f4*)running_mean, (const ew_f4*)running_var,
                           (ew_f4*)y, n4, C / 4, eps);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    EW_LAUNCH(bn_apply_infer, n, x, gamma, beta, running_mean, running_var, y, n, C, eps);
    return AETH_OK;
}

static int bn_bwd_impl(const float* x, const float* dy, const float* gamma, const float* save_mean,
                       const float* save_invstd, float* dx, uint16_t* dx_bf16, float* dgamma, float* dbeta, int rows,
                       int C) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x && dy && gamma && save_mean && save_invstd && dx && dgamma && dbeta);
    AETH_CHECK_ARG(rows > 0 && C > 0 && (int64_t)rows * C < ((int64_t)1 << 31));
    int nblk, rpb;
    dim3 grid;
    col_grid(rows, C, &nblk, &rpb, &grid);
    void* ws;
    int rc = workspace(((int64_t)2 * nblk * C + 3 * C) * sizeof(float), &ws);
    if (rc) return rc;
    float* part = (float*)ws;
    float* coef = part + (int64_t)2 * nblk * C;
    hipStream_t st = ctx().stream;
    if (col_vec4(C, x, dy) && col_vec4(C, save_mean, part)) {
        hipLaunchKernelGGL(bn_bwd_partial4, dim3(grid.x, cdiv(C / 4, 64)), dim3(kEwThreads), 0, st, x, dy, save_mean, rows, C,
                           rpb, part);
    } else {
        hipLaunchKernelGGL(bn_bwd_partial, grid, dim3(kEwThreads), 0, st, x, dy, save_mean, rows, C, rpb, part);
    }
    AETH_LAUNCH_CHECK();
    hipLaunchKernelGGL(bn_bwd_final, dim3(cdiv(C, 64)), dim3(256), 0, st, part, nblk, rows, C, gamma, save_invstd,
                       dgamma, dbeta, coef);
    AETH_LAUNCH_CHECK();
    int64_t n = (int64_t)rows * C;
    if (col_vec4(C, x, dy) && col_vec4(C, save_mean, dx) && aligned16(dx_bf16) && aligned16(coef)) {
        const unsigned n4 = (unsigned)(n / 4);
        hipLaunchKernelGGL(bn_bwd_apply4, dim3(ew_blocks(n4)), dim3(kEwThreads), 0, st, (const ew_f4*)x, (const ew_f4*)dy,
                           (const ew_f4*)save_mean, coef, (ew_f4*)dx, (ew_u2*)dx_bf16, n4, C / 4);
        AETH_LAUNCH_CHECK();
    } else {
        EW_LAUNCH(bn_bwd_apply, n, x, dy, save_mean, coef, dx, dx_bf16, n, C);
    }
    return AETH_OK;
}

int aeth_bn_bwd_f32(const float* x, const float* dy, const float* gamma, const float* save_mean,
                    const float* save_invstd, float* dx, float* dgamma, float* dbeta, int rows, int C) {
    return bn_bwd_impl(x, dy, gamma, save_mean, save_invstd, dx, nullptr, dgamma, dbeta, rows, C);
}

int aeth_bn_bwd_twin_f32(const float* x, const float* dy, const float* gamma, const float* save_mean,
                         const float* save_invstd, float* dx, uint16_t* dx_bf16, float* dgamma, float* dbeta,
                         int rows, int C) {
    AETH_CHECK_ARG(dx_bf16 != nullptr);
    return bn_bwd_impl(x, dy, gamma, save_mean, save_invstd, dx, dx_bf16, dgamma, dbeta, rows, C);
}

int aeth_relu_fwd_f32(const float* x, float* y, float alpha, int64_t n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(x && y);
    EW_LAUNCH(relu_fwd_kernel, n, x, y, alpha, n);
    return AETH_OK;
}

int aeth_relu_fwd_twin_f32(const float* x, float* y, uint16_t* y_bf16, float alpha, int64_t n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(x && y && y_bf16);
    if (n % 4 == 0 && aligned16(x) && aligned16(y) && (reinterpret_cast<uintptr_t>(y_bf16) & 7) == 0) {
        const int64_t n4 = n / 4;
        EW_LAUNCH(relu_fwd_twin_kernel4, n4, (const ew_f4*)x, (ew_f4*)y, (ew_u2*)y_bf16, alpha, n4);
    } else {
        EW_LAUNCH(relu_fwd_twin_kernel, n, x, y, y_bf16, alpha, n);
    }
    return AETH_OK;
}

int aeth_relu_bwd_f32(const float* x, const float* dy, float* dx, float alpha, int64_t n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(x && dy && dx);
    EW_LAUNCH(relu_bwd_kernel, n, x, dy, dx, alpha, n);
    return AETH_OK;
}

int aeth_maxpool_fwd_f32(const float* x, float* y, uint8_t* idx, int S, int H, int W, int C, int fH, int fW, int sH,
                         int sW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x && y && idx);
    PoolParams p;
    int rc = pool_dims(__func__, S, H, W, C, fH, fW, sH, sW, &p);
    if (rc) return rc;
    int64_t n = (int64_t)S * p.Ho * p.Wo * C;
    if (C % 4 == 0 && n > 0 && aligned16(x) && aligned16(y) && (reinterpret_cast<uintptr_t>(idx) & 3) == 0) {
        p.div_c = FastDiv(C / 4); p.div_w = FastDiv(p.Wo); p.div_h = FastDiv(p.Ho);
        const unsigned n4 = (unsigned)(n / 4);
        hipLaunchKernelGGL(maxpool_fwd_kernel4, dim3(cdiv(n4, kEwThreads)), dim3(kEwThreads), 0, ctx().stream,
                           (const ew_f4*)x, (ew_f4*)y, (uint32_t*)idx, p, n4);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    EW_LAUNCH(maxpool_fwd_kernel, n, x, y, idx, p, n);
    return AETH_OK;
}

int aeth_maxpool_bwd_f32(const float* dy, const uint8_t* idx, float* dx, int S, int H, int W, int C, int fH, int fW,
                         int sH, int sW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy && idx && dx);
    PoolParams p;
    int rc = pool_dims(__func__, S, H, W, C, fH, fW, sH, sW, &p);
    if (rc) return rc;
    int64_t n = (int64_t)S * H * W * C;
    if (C % 4 == 0 && aligned16(dy) && aligned16(dx) && (reinterpret_cast<uintptr_t>(idx) & 3) == 0) {
        p.div_c = FastDiv(C / 4);
        const unsigned n4 = (unsigned)(n / 4);
        hipLaunchKernelGGL(maxpool_bwd_kernel4, dim3(cdiv(n4, kEwThreads)), dim3(kEwThreads), 0, ctx().stream,
                           (const ew_f4*)dy, (const uint32_t*)idx, (ew_f4*)dx, p, n4);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    EW_LAUNCH(maxpool_bwd_kernel, n, dy, idx, dx, p, n);
    return AETH_OK;
}

int aeth_avgpool_fwd_f32(const float* x, float* y, int S, int H, int W, int C, int fH, int fW, int sH, int sW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x && y);
    PoolParams p;
    int rc = pool_dims(__func__, S, H, W, C, fH, fW, sH, sW, &p);
    if (rc) return rc;
    int64_t n = (int64_t)S * p.Ho * p.Wo * C;
    if (C % 4 == 0 && n > 0 && aligned16(x) && aligned16(y)) {
        p.div_c = FastDiv(C / 4); p.div_w = FastDiv(p.Wo); p.div_h = FastDiv(p.Ho);
        const unsigned n4 = (unsigned)(n / 4);
        hipLaunchKernelGGL(avgpool_fwd_kernel4, dim3(cdiv(n4, kEwThreads)), dim3(kEwThreads), 0, ctx().stream,
                           (const ew_f4*)x, (ew_f4*)y, p, n4);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    EW_LAUNCH(avgpool_fwd_kernel, n, x, y, p, n);
    return AETH_OK;
}

int aeth_avgpool_bwd_f32(const float* dy, float* dx, int S, int H, int W, int C, int fH, int fW, int sH, int sW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy && dx);
    PoolParams p;
    int rc = pool_dims(__func__, S, H, W, C, fH, fW, sH, sW, &p);
    if (rc) return rc;
    int64_t n = (int64_t)S * H * W * C;
    if (C % 4 == 0 && aligned16(dy) && aligned16(dx)) {
        p.div_c = FastDiv(C / 4);
        const unsigned n4 = (unsigned)(n / 4);
        hipLaunchKernelGGL(avgpool_bwd_kernel4, dim3(cdiv(n4, kEwThreads)), dim3(kEwThreads), 0, ctx().stream,
                           (const ew_f4*)dy, (ew_f4*)dx, p, n4);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    EW_LAUNCH(avgpool_bwd_kernel, n, dy, dx, p, n);
    return AETH_OK;
}

int aeth_mul_mask_f32(const float* x, const float* mask, float* y, int64_t n, int64_t mask_n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0 && mask_n > 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(x && mask && y);
    EW_LAUNCH(mul_mask_kernel, n, x, mask, y, n, mask_n);
    return AETH_OK;
}

int aeth_softmax_f32(const float* logits, float* probs, int rows, int K) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(logits && probs && rows > 0 && K > 0);
    hipLaunchKernelGGL(softmax_kernel, dim3(cdiv(rows, 64)), dim3(64), 0, ctx().stream, logits, probs, rows, K);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

int aeth_softmax_bwd_f32(const float* probs, const float* dy, float* dx, int rows, int K) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(probs && dy && dx && rows > 0 && K > 0);
    hipLaunchKernelGGL(softmax_bwd_kernel, dim3(cdiv(rows, 64)), dim3(64), 0, ctx().stream, probs, dy, dx, rows, K);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

extern "C++" {
template <typename Targets>
static int cce_fwd_impl(const char* fn, const float* probs, const Targets tg, const void* targets, float label_smoothing,
                        float* sample_loss, int32_t* pred, int rows, int K) {
    AETH_REQUIRE_INIT();
    if (!(probs && targets && sample_loss && pred && rows > 0 && K > 0)) return fail(AETH_E_INVALID, "%s: argument check failed", fn);
    hipLaunchKernelGGL(cce_fwd_kernel<Targets>, dim3(cdiv(rows, 64)), dim3(64), 0, ctx().stream, probs, tg,
                       label_smoothing, sample_loss, pred, rows, K);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

template <typename Targets>
static int softmax_cce_bwd_impl(const char* fn, const float* probs, const Targets tg, const void* targets,
                                float label_smoothing, float* dlogits, int rows, int K) {
    AETH_REQUIRE_INIT();
    if (!(probs && targets && dlogits && rows > 0 && K > 0 && (int64_t)rows * K < ((int64_t)1 << 31)))
        return fail(AETH_E_INVALID, "%s: argument check failed", fn);
    hipLaunchKernelGGL(softmax_cce_bwd_kernel<Targets>, dim3(cdiv((int64_t)rows * K, 256)), dim3(256), 0, ctx().stream,
                       probs, tg, label_smoothing, dlogits, rows, K);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

template <typename Targets>
static int softmax_cce_train_impl(const char* fn, const float* logits, const Targets tg, const void* targets,
                                  float label_smoothing, float* probs, float* sample_loss, int32_t* pred, float* dlogits,
                                  int rows, int K) {
    AETH_REQUIRE_INIT();
    if (!(logits && targets && probs && sample_loss && pred && dlogits && rows > 0 && K > 0 &&
          (int64_t)rows * K < ((int64_t)1 << 31)))
        return fail(AETH_E_INVALID, "%s: argument check failed", fn);
    if (K <= 16 && (int64_t)rows * 16 < ((int64_t)1 << 31))
        hipLaunchKernelGGL(softmax_cce_train16_kernel<Targets>, dim3(cdiv((int64_t)rows * 16, 256)), dim3(256), 0,
                           ctx().stream, logits, tg, label_smoothing, probs, sample_loss, pred, dlogits, rows, K);
    else
        hipLaunchKernelGGL(softmax_cce_train_kernel<Targets>, dim3(cdiv(rows, 64)), dim3(64), 0, ctx().stream, logits, tg,
                           label_smoothing, probs, sample_loss, pred, dlogits, rows, K);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

}  // extern "C++"

int aeth_cce_fwd_f32(const float* probs, const int32_t* labels, float label_smoothing, float* sample_loss,
                     int32_t* pred, int rows, int K) {
    return cce_fwd_impl(__func__, probs, IndexTargets{labels}, labels, label_smoothing, sample_loss, pred, rows, K);
}

int aeth_cce_fwd_dense_f32(const float* probs, const float* targets, float label_smoothing, float* sample_loss,
                           int32_t* pred, int rows, int K) {
    return cce_fwd_impl(__func__, probs, DenseTargets{targets, K}, targets, label_smoothing, sample_loss, pred, rows, K);
}

int aeth_softmax_cce_bwd_f32(const float* probs, const int32_t* labels, float label_smoothing, float* dlogits,
                             int rows, int K) {
    return softmax_cce_bwd_impl(__func__, probs, IndexTargets{labels}, labels, label_smoothing, dlogits, rows, K);
}

int aeth_softmax_cce_bwd_dense_f32(const float* probs, const float* targets, float label_smoothing, float* dlogits,
                                   int rows, int K) {
    return softmax_cce_bwd_impl(__func__, probs, DenseTargets{targets, K}, targets, label_smoothing, dlogits, rows, K);
}

int aeth_softmax_cce_train_f32(const float* logits, const int32_t* labels, float label_smoothing, float* probs,
                               float* sample_loss, int32_t* pred, float* dlogits, int rows, int K) {
    return softmax_cce_train_impl(__func__, logits, IndexTargets{labels}, labels, label_smoothing, probs, sample_loss, pred,
                                  dlogits, rows, K);
}

int aeth_softmax_cce_train_dense_f32(const float* logits, const float* targets, float label_smoothing, float* probs,
                                     float* sample_loss, int32_t* pred, float* dlogits, int rows, int K) {
    return softmax_cce_train_impl(__func__, logits, DenseTargets{targets, K}, targets, label_smoothing, probs, sample_loss,
                                  pred, dlogits, rows, K);
}

int aeth_adam_f32(float* theta, const float* grad, float* m, float* v, int64_t n, float lr, float beta1, float beta2,
                  float eps, int t) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0 && t >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(theta && grad && m && v);
    float c1, c2;
    adam_corrections(beta1, beta2, t, &c1, &c2);
    EW_LAUNCH(adam_kernel, n, theta, grad, m, v, n, lr, beta1, beta2, eps, c1, c2);
    return AETH_OK;
}

int aeth_adam_multi_f32(int count, float* const* host_theta, const float* const* host_grad, float* const* host_m,
                        float* const* host_v, const int64_t* host_n, float lr, float beta1, float beta2, float eps,
                        int t) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(count >= 1 && count <= kAdamMax && t >= 0);
    AETH_CHECK_ARG(host_theta && host_grad && host_m && host_v && host_n);
    AdamTable tb;
    int64_t nmax = 0;
    for (int i = 0; i < kAdamMax; ++i) {
        const int j = i < count ? i : 0;
        AETH_CHECK_ARG(host_n[j] >= 0);
        AETH_CHECK_ARG(host_n[j] == 0 || (host_theta[j] && host_grad[j] && host_m[j] && host_v[j]));
        tb.theta[i] = host_theta[j]; tb.grad[i] = host_grad[j]; tb.m[i] = host_m[j]; tb.v[i] = host_v[j];
        tb.n[i] = i < count ? host_n[j] : 0;
        if (tb.n[i] > nmax) nmax = tb.n[i];
    }
    if (nmax == 0) return AETH_OK;
    float c1, c2;
    adam_corrections(beta1, beta2, t, &c1, &c2);
    int bx = (int)((nmax + 4 * kEwThreads - 1) / (4 * kEwThreads));
    if (bx > 256) bx = 256;
    hipLaunchKernelGGL(adam_multi_kernel, dim3(bx, count), dim3(kEwThreads), 0, ctx().stream, tb, lr, beta1, beta2,
                       eps, c1, c2);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

int aeth_adam_state_step(double* state, double lr, double decay, double beta1, double beta2) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(state != nullptr);
    hipLaunchKernelGGL(adam_state_step_kernel, dim3(1), dim3(64), 0, ctx().stream, state, lr, decay, beta1, beta2);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

int aeth_adam_multi_dev_f32(int count, float* const* host_theta, const float* const* host_grad, float* const* host_m,
                            float* const* host_v, const int64_t* host_n, float beta1, float beta2, float eps,
                            const double* state) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(count >= 1 && count <= kAdamMax && state != nullptr);
    AETH_CHECK_ARG(host_theta && host_grad && host_m && host_v && host_n);
    AdamTable tb;
    int64_t nmax = 0;
    for (int i = 0; i < kAdamMax; ++i) {
        const int j = i < count ? i : 0;
        AETH_CHECK_ARG(host_n[j] >= 0);
        AETH_CHECK_ARG(host_n[j] == 0 || (host_theta[j] && host_grad[j] && host_m[j] && host_v[j]));
        tb.theta[i] = host_theta[j]; tb.grad[i] = host_grad[j]; tb.m[i] = host_m[j]; tb.v[i] = host_v[j];
        tb.n[i] = i < count ? host_n[j] : 0;
        if (tb.n[i] > nmax) nmax = tb.n[i];
    }
    if (nmax == 0) return AETH_OK;
    int bx = (int)((nmax + 4 * kEwThreads - 1) / (4 * kEwThreads));
    if (bx > 256) bx = 256;
    hipLaunchKernelGGL(adam_multi_dev_kernel, dim3(bx, count), dim3(kEwThreads), 0, ctx().stream, tb, beta1, beta2, eps,
                       state);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

int aeth_axpy_f32(float alpha, const float* x, float* y, int64_t n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(x && y);
    EW_LAUNCH(axpy_kernel, n, alpha, x, y, n);
    return AETH_OK;
}

int aeth_l1_grad_f32(float lambda, const float* w, float* dw, int64_t n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(w && dw);
    EW_LAUNCH(l1_grad_kernel, n, lambda, w, dw, n);
    return AETH_OK;
}

int aeth_reduce_f32(const float* x, int64_t n, int mode, float* out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0 && (mode == 0 || mode == 1) && out);
    AETH_CHECK_ARG(n == 0 || x);
    // one block up to 16 Ki elements; beyond that chunks of at least 4096 on at most 1024 blocks, then their partials
    // (a single block over the 786 432 weights of a 3072 x 256 layer: 81 us)
    if (n > 16384) {
        int64_t chunk = 4096;
        while (cdiv(n, chunk) > 1024) chunk *= 2;
        const int blocks = (int)cdiv(n, chunk);
        void* ws;
        int rc = workspace((int64_t)blocks * sizeof(float), &ws);
        if (rc) return rc;
        hipLaunchKernelGGL(reduce_chunks_kernel, dim3(blocks), dim3(256), 0, ctx().stream, x, n, chunk, mode, (float*)ws);
        AETH_LAUNCH_CHECK();
        hipLaunchKernelGGL(reduce_kernel, dim3(1), dim3(1024), 0, ctx().stream, (const float*)ws, (int64_t)blocks, 2, out);
        AETH_LAUNCH_CHECK();
        return AETH_OK;
    }
    hipLaunchKernelGGL(reduce_kernel, dim3(1), dim3(1024), 0, ctx().stream, x, n, mode, out);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

int aeth_cast_f32_to_bf16(const float* src, uint16_t* dst, int64_t n) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(n >= 0);
    if (n == 0) return AETH_OK;
    AETH_CHECK_ARG(src && dst);
    int64_t done = 0;
    if (n >= 8 && aligned16(src) && aligned16(dst)) {
        const int64_t n8 = n / 8;
        EW_LAUNCH(cast_bf16_kernel8, n8, (const ew_f4*)src, (ew_u4*)dst, n8);
        done = 8 * n8;
    }
    if (done < n) EW_LAUNCH(cast_bf16_kernel, n - done, src + done, dst + done, n - done);
    return AETH_OK;
}

}  // extern "C"
