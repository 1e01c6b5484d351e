// fp32 implicit-GEMM convolution for gfx950: fprop, dgrad, wgrad on
// v_mfma_f32_32x32x2_f32, plus the dense-layer products expressed as 1x1 cases.
//
// GEMM view (M = S*Ho*Wo, N = D, K = fH*fW*C):
//   fprop : Y[M,N]  = A[M,K] . W[K,N] + bias      A gathered from x on the fly
//   dgrad : dX[M',C] = A'[M',K'] . W'[K',C]        A' gathered from dy; one launch
//           per stride-parity class so that no tap multiplies a structural zero
//   wgrad : dW[K,N] = A[M,K]^T . dY[M,N]           reduction over M split across
//           workgroups, partial sums reduced in a fixed order
//
// "gather" kernel (fprop, dgrad, dense fprop/dgrad)
//   workgroup = 256 threads = 4 waves, tile BM x BN, K consumed in slabs of 32.
//   A slab (BM x 32) is read from HBM/L2 with one 128-bit load per thread per 4
//   channels (NHWC: channels are contiguous), zero where the tap falls in the
//   padding, and stored to LDS row-major with a row pitch of 36 floats; the B slab
//   comes from a pre-packed [N][K] copy of the filter and uses the same pitch.
//   With that pitch both the 128-bit stores and the 128-bit operand reads touch
//   32 distinct banks per 8 lanes.  Each lane reads 4 consecutive k of one row and
//   feeds them to 4 successive MFMAs: the k order inside a slab is permuted the
//   same way for A and B, which leaves the sum unchanged.
#include "common.h"

#include <limits.h>
#include <vector>

namespace aeth {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kBK = 32;      // K slab
constexpr int kLD = 36;      // LDS row pitch of a slab, in floats

// ------------------------------------------------------------------------------
// gather-GEMM
// ------------------------------------------------------------------------------
struct GatherParams {
    const float* src;    // [S, Hs, Ws, Cs]
    const float* bt;     // packed filter [Npad][Kpad], zero filled
    const float* bias;   // [N] or nullptr
    float* out;
    int S, Hs, Ws, Cs;
    int Hg, Wg;          // output pixel grid of this launch
    int M, N, K, Kpad;   // M = S*Hg*Wg, K = Th*Tw*Cs
    int Tw;              // taps per filter row
    int sh, sw;          // source step per output pixel
    int rh0, rw0;        // source offset of tap (0,0)
    // output element (s,i,j,n) lives at ((s*Hof + oh0 + i*ohs)*Wof + ow0 + j*ows)*N + n
    int Hof, Wof, oh0, ow0, ohs, ows;
    int dense_out;       // 1: row m is stored at out + m*N
    FastDiv div_hw, div_w, div_c, div_tw;
};

constexpr int kInvalidRow = -16384;

template <int BM, int BN, int WM, int WN, int VEC>
__global__ __launch_bounds__(kThreads) void gather_gemm_f32(const GatherParams p) {
    static_assert((BM / WM) * (BN / WN) == 4, "4 waves per workgroup");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "32x32 MFMA tiles");
    constexpr int AL = BM / 32;          // 128-bit A loads per thread per slab
    constexpr int BL = BN / 32;
    constexpr int TM = WM / 32;
    constexpr int TN = WN / 32;

    __shared__ float lds_a[BM * kLD];
    __shared__ float lds_b[BN * kLD];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int wm0 = (wave % (BM / WM)) * WM;
    const int wn0 = (wave / (BM / WM)) * WN;

    const int m0 = blockIdx.x * BM;
    const int n0 = blockIdx.y * BN;

    // ---- per-thread row bookkeeping for the A gather --------------------------
    const int k4 = tid & 7;              // which 4-float chunk of the slab row
    const int r0 = tid >> 3;             // first row handled (then +32 each)
    int base_off[AL];
    int base_rc[AL];                     // (row << 16) | (col & 0xffff) of tap (0,0)
#pragma unroll
    for (int i = 0; i < AL; ++i) {
        int m = m0 + r0 + 32 * i;
        if (m < p.M) {
            unsigned s, rem, ii, jj;
            p.div_hw.divmod((unsigned)m, s, rem);
            p.div_w.divmod(rem, ii, jj);
            int br = (int)ii * p.sh + p.rh0;
            int bc = (int)jj * p.sw + p.rw0;
            base_off[i] = (((int)s * p.Hs + br) * p.Ws + bc) * p.Cs;
            base_rc[i] = (int)(((unsigned)br << 16) | ((unsigned)bc & 0xffffu));
        } else {
            base_off[i] = 0;
            base_rc[i] = (int)((unsigned)kInvalidRow << 16);
        }
    }
    const float* bt_row = p.bt + (size_t)(n0 + r0) * p.Kpad + 4 * k4;

    f4 areg[AL];
    f4 breg[BL];

    auto load_slab = [&](int k0) {
        if (VEC == 4) {
            int kk = k0 + 4 * k4;
            unsigned tap, c, th, tw;
            p.div_c.divmod((unsigned)kk, tap, c);
            p.div_tw.divmod(tap, th, tw);
            bool kvalid = kk < p.K;
            int tap_off = ((int)th * p.Ws + (int)tw) * p.Cs + (int)c;
#pragma unroll
            for (int i = 0; i < AL; ++i) {
                int r = (base_rc[i] >> 16) + (int)th;
                int cc = ((int)((unsigned)base_rc[i] << 16) >> 16) + (int)tw;
                bool ok = kvalid && (unsigned)r < (unsigned)p.Hs && (unsigned)cc < (unsigned)p.Ws;
                f4 v = {0.f, 0.f, 0.f, 0.f};
                if (ok) v = *reinterpret_cast<const f4*>(p.src + (base_off[i] + tap_off));
                areg[i] = v;
            }
        } else {
#pragma unroll
            for (int i = 0; i < AL; ++i) areg[i] = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int kk = k0 + 4 * k4 + e;
                unsigned tap, c, th, tw;
                p.div_c.divmod((unsigned)kk, tap, c);
                p.div_tw.divmod(tap, th, tw);
                bool kvalid = kk < p.K;
                int tap_off = ((int)th * p.Ws + (int)tw) * p.Cs + (int)c;
#pragma unroll
                for (int i = 0; i < AL; ++i) {
                    int r = (base_rc[i] >> 16) + (int)th;
                    int cc = ((int)((unsigned)base_rc[i] << 16) >> 16) + (int)tw;
                    bool ok = kvalid && (unsigned)r < (unsigned)p.Hs && (unsigned)cc < (unsigned)p.Ws;
                    float v = 0.f;
                    if (ok) v = p.src[base_off[i] + tap_off];
                    areg[i][e] = v;
                }
            }
        }
#pragma unroll
        for (int i = 0; i < BL; ++i)
            breg[i] = *reinterpret_cast<const f4*>(bt_row + (size_t)(32 * i) * p.Kpad + k0);
    };

    auto store_slab = [&]() {
#pragma unroll
        for (int i = 0; i < AL; ++i)
            *reinterpret_cast<f4*>(&lds_a[(r0 + 32 * i) * kLD + 4 * k4]) = areg[i];
#pragma unroll
        for (int i = 0; i < BL; ++i)
            *reinterpret_cast<f4*>(&lds_b[(r0 + 32 * i) * kLD + 4 * k4]) = breg[i];
    };

    f16v acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    if (p.Kpad > 0) {
        load_slab(0);
        store_slab();
        __syncthreads();
    }

    for (int k0 = 0; k0 < p.Kpad; k0 += kBK) {
        const bool more = k0 + kBK < p.Kpad;
        if (more) load_slab(k0 + kBK);

#pragma unroll
        for (int g = 0; g < kBK / 8; ++g) {
            f4 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i)
                a[i] = *reinterpret_cast<const f4*>(&lds_a[(wm0 + 32 * i + l32) * kLD + 8 * g + 4 * lh]);
#pragma unroll
            for (int j = 0; j < TN; ++j)
                b[j] = *reinterpret_cast<const f4*>(&lds_b[(wn0 + 32 * j + l32) * kLD + 8 * g + 4 * lh]);
#pragma unroll
            for (int t = 0; t < 4; ++t)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][t], b[j][t], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
        if (more) {
            store_slab();
            __syncthreads();
        }
    }

    // ---- epilogue: bias add and store -------------------------------------------
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int n = n0 + wn0 + 32 * j + l32;
        const bool nok = n < p.N;
        const float bv = (p.bias != nullptr && nok) ? p.bias[n] : 0.f;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int m = m0 + wm0 + 32 * i + 8 * (v >> 2) + 4 * lh + (v & 3);
                if (nok && m < p.M) {
                    size_t row;
                    if (p.dense_out) {
                        row = (size_t)m;
                    } else {
                        unsigned s, rem, ii, jj;
                        p.div_hw.divmod((unsigned)m, s, rem);
                        p.div_w.divmod(rem, ii, jj);
                        row = ((size_t)s * p.Hof + p.oh0 + (size_t)ii * p.ohs) * p.Wof + p.ow0 + (size_t)jj * p.ows;
                    }
                    p.out[row * p.N + n] = acc[i][j][v] + bv;
                }
            }
        }
    }
}

// Packs the filter w[fH][fW][C][D] into bt[Npad][Kpad] (k contiguous) for one
// gather-GEMM launch.  k = (th*Tw + tw)*Ck + kc ; filter tap x = xa + xs*th,
// y = ya + ys*tw.  transposed == 0: n is the output channel d and kc the input
// channel c (fprop).  transposed == 1: n is c and kc is d (dgrad).
struct PackParams {
    const float* w;
    float* bt;
    int fW, C, D;
    int Tw, Ck;
    int xa, xs, ya, ys;
    int transposed;
    int N, K, Npad, Kpad;
};

__global__ void pack_filter_f32(const PackParams p) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    int total = p.Npad * p.Kpad;
    if (idx >= total) return;
    int n = idx / p.Kpad;
    int k = idx - n * p.Kpad;
    float v = 0.f;
    if (n < p.N && k < p.K) {
        int tap = k / p.Ck;
        int kc = k - tap * p.Ck;
        int th = tap / p.Tw;
        int tw = tap - th * p.Tw;
        int x = p.xa + p.xs * th;
        int y = p.ya + p.ys * tw;
        int c = p.transposed ? n : kc;
        int d = p.transposed ? kc : n;
        v = p.w[((size_t)(x * p.fW + y) * p.C + c) * p.D + d];
    }
    p.bt[idx] = v;
}

template <int BM, int BN, int WM, int WN>
static void launch_gather_cfg(const GatherParams& gp, bool vec4, hipStream_t st) {
    dim3 grid(cdiv(gp.M, BM), cdiv(gp.N, BN));
    if (vec4)
        hipLaunchKernelGGL((gather_gemm_f32<BM, BN, WM, WN, 4>), grid, dim3(kThreads), 0, st, gp);
    else
        hipLaunchKernelGGL((gather_gemm_f32<BM, BN, WM, WN, 1>), grid, dim3(kThreads), 0, st, gp);
}

static int gather_bn(int N) { return N <= 32 ? 32 : 64; }

static int gather_bm(int M, int N, int cus) {
    const int bn = gather_bn(N);
    const int ntiles = cdiv(N, bn);
    const int want = 2 * cus;
    const int cands[3] = {256, 128, 64};
    for (int i = 0; i < 3; ++i) {
        int bm = cands[i];
        if (bn == 32 && bm == 64) break;
        if ((int64_t)cdiv(M, bm) * ntiles >= want) return bm;
    }
    return bn == 32 ? 128 : 64;
}

static void launch_gather(const GatherParams& gp, bool vec4, int cus, hipStream_t st) {
    const int bn = gather_bn(gp.N);
    const int bm = gather_bm(gp.M, gp.N, cus);
    if (bn == 32) {
        if (bm == 256) launch_gather_cfg<256, 32, 64, 32>(gp, vec4, st);
        else launch_gather_cfg<128, 32, 32, 32>(gp, vec4, st);
    } else {
        if (bm == 256) launch_gather_cfg<256, 64, 64, 64>(gp, vec4, st);
        else if (bm == 128) launch_gather_cfg<128, 64, 32, 64>(gp, vec4, st);
        else launch_gather_cfg<64, 64, 32, 32>(gp, vec4, st);
    }
}

// One gather-GEMM problem: pack the filter into the workspace at `ws_off`, launch.
struct GatherSetup {
    GatherParams gp;
    PackParams pp;
    int64_t bt_bytes;
};

static int run_gather(GatherSetup& gs, char* ws, int64_t ws_off, bool vec4) {
    Context& c = ctx();
    float* bt = reinterpret_cast<float*>(ws + ws_off);
    gs.gp.bt = bt;
    gs.pp.bt = bt;
    int total = gs.pp.Npad * gs.pp.Kpad;
    if (total > 0) {
        hipLaunchKernelGGL(pack_filter_f32, dim3(cdiv(total, 256)), dim3(256), 0, c.stream, gs.pp);
        AETH_LAUNCH_CHECK();
    }
    if (gs.gp.M > 0 && gs.gp.N > 0) {
        launch_gather(gs.gp, vec4, c.prop.multiProcessorCount, c.stream);
        AETH_LAUNCH_CHECK();
    }
    return AETH_OK;
}

static int check_conv_dims(const char* fn, int S, int H, int W, int C, int D, int fH, int fW,
                           int sH, int sW, int pH, int pW, int* Ho, int* Wo) {
    if (S <= 0 || H <= 0 || W <= 0 || C <= 0 || D <= 0 || fH <= 0 || fW <= 0 || sH <= 0 || sW <= 0 ||
        pH < 0 || pW < 0)
        return fail(AETH_E_INVALID, "%s: non-positive dimension", fn);
    if (H + 2 * pH < fH || W + 2 * pW < fW) return fail(AETH_E_INVALID, "%s: filter larger than padded input", fn);
    if (H >= 8192 || W >= 8192 || fH > 64 || fW > 64 || pH >= 64 || pW >= 64)
        return fail(AETH_E_INVALID, "%s: spatial extent out of supported range", fn);
    *Ho = (H + 2 * pH - fH) / sH + 1;
    *Wo = (W + 2 * pW - fW) / sW + 1;
    const int64_t lim = (int64_t)INT_MAX - (1 << 24);
    if ((int64_t)S * (H + 2 * pH + fH) * (W + 2 * pW + fW) * C >= lim || (int64_t)S * *Ho * *Wo * D >= lim ||
        (int64_t)fH * fW * C * D >= lim)
        return fail(AETH_E_INVALID, "%s: tensor has 2^31 elements or more", fn);
    return AETH_OK;
}

static void set_out_divs(GatherParams& g) {
    g.div_hw = FastDiv(g.Hg * g.Wg > 0 ? g.Hg * g.Wg : 1);
    g.div_w = FastDiv(g.Wg > 0 ? g.Wg : 1);
    g.div_c = FastDiv(g.Cs);
    g.div_tw = FastDiv(g.Tw > 0 ? g.Tw : 1);
}

int conv_fprop_f32_impl(const float* x, const float* w, const float* bias, float* y,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    int Ho, Wo;
    int rc = check_conv_dims("aeth_conv_fprop_f32", S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    GatherSetup gs;
    GatherParams& g = gs.gp;
    g.src = x; g.bias = bias; g.out = y;
    g.S = S; g.Hs = H; g.Ws = W; g.Cs = C;
    g.Hg = Ho; g.Wg = Wo; g.M = S * Ho * Wo; g.N = D; g.K = fH * fW * C;
    g.Kpad = (int)round_up(g.K, kBK);
    g.Tw = fW; g.sh = sH; g.sw = sW; g.rh0 = -pH; g.rw0 = -pW;
    g.Hof = Ho; g.Wof = Wo; g.oh0 = 0; g.ow0 = 0; g.ohs = 1; g.ows = 1; g.dense_out = 1;
    set_out_divs(g);
    PackParams& pk = gs.pp;
    pk.w = w; pk.fW = fW; pk.C = C; pk.D = D; pk.Tw = fW; pk.Ck = C;
    pk.xa = 0; pk.xs = 1; pk.ya = 0; pk.ys = 1; pk.transposed = 0;
    pk.N = D; pk.K = g.K; pk.Npad = (int)round_up(D, 64); pk.Kpad = g.Kpad;
    gs.bt_bytes = (int64_t)pk.Npad * pk.Kpad * sizeof(float);
    void* ws;
    rc = workspace(gs.bt_bytes, &ws);
    if (rc) return rc;
    return run_gather(gs, (char*)ws, 0, C % 4 == 0);
}

// dgrad: for input row i the contributing taps are x with (i + pH - x) % sH == 0 and
// 0 <= (i + pH - x)/sH < Ho.  Rows are split by a = i % sH; inside a class the taps
// are x_t = xmax - sH*t (xmax = largest x < fH with x == (a+pH) mod sH), and the
// source row for class-row i' (i = a + sH*i') and tap t is i' + (a + pH - xmax)/sH + t:
// a unit-stride gather over dy with Th = number of such taps.
int conv_dgrad_f32_impl(const float* dy, const float* w, float* dx,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    int Ho, Wo;
    int rc = check_conv_dims("aeth_conv_dgrad_f32", S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    const int nclass = sH * sW;
    if (nclass > 64) return fail(AETH_E_INVALID, "aeth_conv_dgrad_f32: stride too large");
    std::vector<GatherSetup> sets;
    int64_t total_bytes = 0;
    for (int a = 0; a < sH; ++a) {
        if (a >= H) continue;
        int ra = (a + pH) % sH;
        int Th = ra < fH ? (fH - 1 - ra) / sH + 1 : 0;
        int xmax = ra + (Th - 1) * sH;
        int offh = Th > 0 ? (a + pH - xmax) / sH : 0;   // exact: (a+pH-xmax) is a multiple of sH
        int Hg = (H - a + sH - 1) / sH;
        for (int b = 0; b < sW; ++b) {
            if (b >= W) continue;
            int rb = (b + pW) % sW;
            int Tw = rb < fW ? (fW - 1 - rb) / sW + 1 : 0;
            int ymax = rb + (Tw - 1) * sW;
            int offw = Tw > 0 ? (b + pW - ymax) / sW : 0;
            int Wg = (W - b + sW - 1) / sW;
            GatherSetup gs;
            GatherParams& g = gs.gp;
            g.src = dy; g.bias = nullptr; g.out = dx;
            g.S = S; g.Hs = Ho; g.Ws = Wo; g.Cs = D;
            g.Hg = Hg; g.Wg = Wg; g.M = S * Hg * Wg; g.N = C;
            g.K = Th * Tw * D;
            g.Kpad = (int)round_up(g.K, kBK);
            g.Tw = Tw; g.sh = 1; g.sw = 1; g.rh0 = offh; g.rw0 = offw;
            g.Hof = H; g.Wof = W; g.oh0 = a; g.ow0 = b; g.ohs = sH; g.ows = sW;
            g.dense_out = (nclass == 1);
            set_out_divs(g);
            PackParams& pk = gs.pp;
            pk.w = w; pk.fW = fW; pk.C = C; pk.D = D; pk.Tw = Tw > 0 ? Tw : 1; pk.Ck = D;
            pk.xa = xmax; pk.xs = -sH; pk.ya = ymax; pk.ys = -sW; pk.transposed = 1;
            pk.N = C; pk.K = g.K; pk.Npad = (int)round_up(C, 64); pk.Kpad = g.Kpad;
            gs.bt_bytes = round_up((int64_t)pk.Npad * pk.Kpad * sizeof(float), 256);
            total_bytes += gs.bt_bytes;
            sets.push_back(gs);
        }
    }
    void* ws;
    rc = workspace(total_bytes > 0 ? total_bytes : 256, &ws);
    if (rc) return rc;
    int64_t off = 0;
    for (auto& gs : sets) {
        rc = run_gather(gs, (char*)ws, off, D % 4 == 0);
        if (rc) return rc;
        off += gs.bt_bytes;
    }
    return AETH_OK;
}

// ------------------------------------------------------------------------------
// wgrad: out[k][n] = sum_m A[m][k] * dy[m][n], k = (fx*fW + fy)*C + c
// Workgroup tile 128 (k) x 64 (n); each of the 4 waves owns 32 k-rows x 64 n.
// The M range of a workgroup (blockIdx.z) is walked in slabs of 32 rows; the
// partial tile goes to out + blockIdx.z * K * D.
// ------------------------------------------------------------------------------
struct WgradParams {
    const float* x;      // [S,H,W,C]
    const float* dy;     // [S,Ho,Wo,D] = [M,D]
    float* out;          // [splits][K][D]
    float* dbias_part;   // [splits][D] or nullptr
    int S, H, W, C, Ho, Wo, D;
    int M, K;
    int fW, sH, sW, pH, pW;
    int m_per_split;     // multiple of 32
    FastDiv div_howo, div_wo, div_c, div_fw;
};

constexpr int kWgBK = 128;   // k rows per workgroup
constexpr int kWgBN = 64;
constexpr int kWgBR = 32;    // m rows per slab
constexpr int kWgLDA = kWgBK + 32;
constexpr int kWgLDY = kWgBN + 32;

template <int VECA, int VECY>
__global__ __launch_bounds__(kThreads) void wgrad_gemm_f32(const WgradParams p) {
    __shared__ float lds_a[kWgBR * kWgLDA];
    __shared__ float lds_y[kWgBR * kWgLDY];
    __shared__ float lds_db[16 * 64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;

    const int kt0 = blockIdx.x * kWgBK;
    const int n0 = blockIdx.y * kWgBN;
    const int m_begin = blockIdx.z * p.m_per_split;
    int m_end = m_begin + p.m_per_split;
    if (m_end > p.M) m_end = p.M;

    // A chunk owned by this thread: 4 consecutive k starting at kt0 + 4*ka, rows ra0 + 8*i
    const int ka = tid & 31;
    const int ra0 = tid >> 5;
    int a_tap_off[VECA == 4 ? 1 : 4];
    int a_fx[VECA == 4 ? 1 : 4];
    int a_fy[VECA == 4 ? 1 : 4];
    bool a_kok[VECA == 4 ? 1 : 4];
#pragma unroll
    for (int e = 0; e < (VECA == 4 ? 1 : 4); ++e) {
        int kk = kt0 + 4 * ka + e;
        unsigned tap, c, fx, fy;
        p.div_c.divmod((unsigned)kk, tap, c);
        p.div_fw.divmod(tap, fx, fy);
        a_kok[e] = kk < p.K;
        a_fx[e] = (int)fx - p.pH;
        a_fy[e] = (int)fy - p.pW;
        a_tap_off[e] = (a_fx[e] * p.W + a_fy[e]) * p.C + (int)c;
    }
    // dy chunk: 4 consecutive n starting at n0 + 4*ky, rows ry0 + 16*i
    const int ky = tid & 15;
    const int ry0 = tid >> 4;
    const bool do_db = (p.dbias_part != nullptr) && (blockIdx.x == 0);

    f4 areg[4];
    f4 yreg[2];
    f4 dbsum = {0.f, 0.f, 0.f, 0.f};

    auto load_slab = [&](int mb) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int m = mb + ra0 + 8 * i;
            f4 v = {0.f, 0.f, 0.f, 0.f};
            if (m < m_end) {
                unsigned s, rem, ho, wo;
                p.div_howo.divmod((unsigned)m, s, rem);
                p.div_wo.divmod(rem, ho, wo);
                int r0 = (int)ho * p.sH;
                int c0 = (int)wo * p.sW;
                int pix = (((int)s * p.H + r0) * p.W + c0) * p.C;
                if (VECA == 4) {
                    bool ok = a_kok[0] && (unsigned)(r0 + a_fx[0]) < (unsigned)p.H &&
                              (unsigned)(c0 + a_fy[0]) < (unsigned)p.W;
                    if (ok) v = *reinterpret_cast<const f4*>(p.x + (pix + a_tap_off[0]));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int ee = VECA == 4 ? 0 : e;
                        bool ok = a_kok[ee] && (unsigned)(r0 + a_fx[ee]) < (unsigned)p.H &&
                                  (unsigned)(c0 + a_fy[ee]) < (unsigned)p.W;
                        if (ok) v[e] = p.x[pix + a_tap_off[ee]];
                    }
                }
            }
            areg[i] = v;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            int m = mb + ry0 + 16 * i;
            f4 v = {0.f, 0.f, 0.f, 0.f};
            int n = n0 + 4 * ky;
            if (m < m_end) {
                if (VECY == 4) {
                    if (n < p.D) v = *reinterpret_cast<const f4*>(p.dy + ((size_t)m * p.D + n));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (n + e < p.D) v[e] = p.dy[(size_t)m * p.D + n + e];
                }
            }
            yreg[i] = v;
        }
    };

    auto store_slab = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i)
            *reinterpret_cast<f4*>(&lds_a[(ra0 + 8 * i) * kWgLDA + 4 * ka]) = areg[i];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            *reinterpret_cast<f4*>(&lds_y[(ry0 + 16 * i) * kWgLDY + 4 * ky]) = yreg[i];
            if (do_db) dbsum += yreg[i];
        }
    };

    f16v acc[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

    if (m_begin < m_end) {
        load_slab(m_begin);
        store_slab();
        __syncthreads();
    }
    for (int mb = m_begin; mb < m_end; mb += kWgBR) {
        const bool more = mb + kWgBR < m_end;
        if (more) load_slab(mb + kWgBR);
        const int wk0 = wave * 32;
#pragma unroll
        for (int t2 = 0; t2 < kWgBR / 2; ++t2) {
            float a = lds_a[(2 * t2 + lh) * kWgLDA + wk0 + l32];
            float b0 = lds_y[(2 * t2 + lh) * kWgLDY + l32];
            float b1 = lds_y[(2 * t2 + lh) * kWgLDY + 32 + l32];
            acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b0, acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b1, acc[1], 0, 0, 0);
        }
        __syncthreads();
        if (more) {
            store_slab();
            __syncthreads();
        }
    }

    float* outp = p.out + (size_t)blockIdx.z * p.K * p.D;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = n0 + 32 * j + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int k = kt0 + wave * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (k < p.K && n < p.D) outp[(size_t)k * p.D + n] = acc[j][v];
        }
    }

    if (do_db) {
        // 16 row-lanes each hold a partial of the same 4 columns: fixed-order sum
#pragma unroll
        for (int e = 0; e < 4; ++e) lds_db[ry0 * 64 + 4 * ky + e] = dbsum[e];
        __syncthreads();
        if (tid < 64) {
            float s = 0.f;
#pragma unroll
            for (int r = 0; r < 16; ++r) s += lds_db[r * 64 + tid];
            if (n0 + tid < p.D) p.dbias_part[(size_t)blockIdx.z * p.D + n0 + tid] = s;
        }
    }
}

// out[i] = sum_s part[s*n + i] in split order
__global__ void reduce_splits_f32(const float* __restrict__ part, float* __restrict__ out, int n, int splits) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = 0.f;
    for (int k = 0; k < splits; ++k) s += part[(size_t)k * n + i];
    out[i] = s;
}

int conv_wgrad_f32_impl(const float* x, const float* dy, float* dw, float* dbias,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    int Ho, Wo;
    int rc = check_conv_dims("aeth_conv_wgrad_f32", S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    Context& c = ctx();
    WgradParams p;
    p.x = x; p.dy = dy;
    p.S = S; p.H = H; p.W = W; p.C = C; p.Ho = Ho; p.Wo = Wo; p.D = D;
    p.M = S * Ho * Wo; p.K = fH * fW * C;
    p.fW = fW; p.sH = sH; p.sW = sW; p.pH = pH; p.pW = pW;
    p.div_howo = FastDiv(Ho * Wo); p.div_wo = FastDiv(Wo); p.div_c = FastDiv(C); p.div_fw = FastDiv(fW);
    const int kt = cdiv(p.K, kWgBK), nt = cdiv(D, kWgBN);
    const int slabs = cdiv(p.M, kWgBR);
    int splits = cdiv(4 * c.prop.multiProcessorCount, kt * nt);
    if (splits > slabs) splits = slabs;
    if (splits < 1) splits = 1;
    int slabs_per = cdiv(slabs, splits);
    splits = cdiv(slabs, slabs_per);
    p.m_per_split = slabs_per * kWgBR;
    const int64_t kd = (int64_t)p.K * D;
    float* part = dw;
    float* db_part = dbias;
    if (splits > 1) {
        void* ws;
        rc = workspace((int64_t)splits * (kd + D) * sizeof(float), &ws);
        if (rc) return rc;
        part = (float*)ws;
        db_part = dbias ? part + (int64_t)splits * kd : nullptr;
    }
    p.out = part;
    p.dbias_part = db_part;
    dim3 grid(kt, nt, splits);
    const bool va = (C % 4 == 0), vy = (D % 4 == 0);
    if (va && vy) hipLaunchKernelGGL((wgrad_gemm_f32<4, 4>), grid, dim3(kThreads), 0, c.stream, p);
    else if (va) hipLaunchKernelGGL((wgrad_gemm_f32<4, 1>), grid, dim3(kThreads), 0, c.stream, p);
    else if (vy) hipLaunchKernelGGL((wgrad_gemm_f32<1, 4>), grid, dim3(kThreads), 0, c.stream, p);
    else hipLaunchKernelGGL((wgrad_gemm_f32<1, 1>), grid, dim3(kThreads), 0, c.stream, p);
    AETH_LAUNCH_CHECK();
    if (splits > 1) {
        hipLaunchKernelGGL(reduce_splits_f32, dim3(cdiv(kd, 256)), dim3(256), 0, c.stream, part, dw, (int)kd, splits);
        AETH_LAUNCH_CHECK();
        if (dbias) {
            hipLaunchKernelGGL(reduce_splits_f32, dim3(cdiv(D, 256)), dim3(256), 0, c.stream, db_part, dbias, D, splits);
            AETH_LAUNCH_CHECK();
        }
    }
    return AETH_OK;
}

}  // namespace aeth

using namespace aeth;

extern "C" {

int aeth_conv_fprop_f32(const float* x, const float* w, const float* bias, float* y,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && w != nullptr && y != nullptr);
    return conv_fprop_f32_impl(x, w, bias, y, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

int aeth_conv_dgrad_f32(const float* dy, const float* w, float* dx,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy != nullptr && w != nullptr && dx != nullptr);
    return conv_dgrad_f32_impl(dy, w, dx, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

int aeth_conv_wgrad_f32(const float* x, const float* dy, float* dw, float* dbias,
                        int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && dy != nullptr && dw != nullptr);
    return conv_wgrad_f32_impl(x, dy, dw, dbias, S, H, W, C, D, fH, fW, sH, sW, pH, pW);
}

// Dense products are the 1x1 cases of the same kernels: x [M,n_in] is an
// [M,1,1,n_in] image and w [n_in,n_out] a [1,1,n_in,n_out] filter.
int aeth_dense_fprop_f32(const float* x, const float* w, const float* bias, float* y, int M, int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && w != nullptr && y != nullptr);
    return conv_fprop_f32_impl(x, w, bias, y, M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0);
}

int aeth_dense_dgrad_f32(const float* dy, const float* w, float* dx, int M, int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(dy != nullptr && w != nullptr && dx != nullptr);
    return conv_dgrad_f32_impl(dy, w, dx, M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0);
}

int aeth_dense_wgrad_f32(const float* x, const float* dy, float* dw, float* dbias, int M, int n_in, int n_out) {
    AETH_REQUIRE_INIT();
    AETH_CHECK_ARG(x != nullptr && dy != nullptr && dw != nullptr);
    return conv_wgrad_f32_impl(x, dy, dw, dbias, M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0);
}

}  // extern "C"
