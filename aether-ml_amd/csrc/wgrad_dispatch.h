// Host side of wgrad: kernel choice, number of splits, the fixed-order reduction of the partials.
#pragma once
#include "wgrad_kernels.h"
#include "narrow_kernels.h"
#include "pair_launch.h"
#include "sample_runs.h"
#include "tuning.h"

namespace aeth {

// Fills the plan of wgrad_halo_bf16 and returns the number of workgroups (= splits), or 0 when the
// kernel does not apply: unit stride, 64 input channels, D a multiple of 8 up to 64, at most 9 taps,
// slabs of whole output rows (R rows with R * Wo a multiple of 16 up to 128, R dividing Ho) whose
// padded source rows fit the halo buffer, and at least 4 slabs per CU (tuning: wgrad_halo = 1 drops
// the last condition, 0 turns the kernel off).
static int plan_wgrad_halo(WgradHaloParams& p, int C, int sH, int sW, int cus) {
    if (sH != 1 || sW != 1 || C != 64 || p.D % 8 != 0 || p.D > 64 || p.fH * p.fW > kWhMaxTaps) return 0;
    if (tuning().wgrad_halo == 0) return 0;
    const bool force = tuning().wgrad_halo > 0;
    int R = 0;
    for (int r = 1; r * p.Wo <= kWhRows; ++r)
        if ((r * p.Wo) % 16 == 0 && p.Ho % r == 0) R = r;                  // the tallest slab that fits
    if (R == 0) return 0;
    p.R = R;
    p.slab_m = R * p.Wo;
    p.Wp = p.Wo + p.fW - 1;
    p.hslots = (R + p.fH - 1) * p.Wp;
    if (p.hslots > kWhSlots) return 0;
    const int64_t nslabs = (int64_t)p.S * (p.Ho / R);
    if (nslabs > (1 << 24) || (!force && nslabs < 4 * (int64_t)cus)) return 0;
    // byte offsets are formed in 32 bits from the pixel above and left of the image
    if (((int64_t)p.S * p.H + p.fH) * p.W * 128 >= ((int64_t)1 << 31)) return 0;
    p.nslabs = (int)nslabs;
    const int wgs = (int)std::min<int64_t>(nslabs, cus);
    p.per = cdiv(p.nslabs, wgs);
    p.div_wp = FastDiv(p.Wp);
    p.div_wo = FastDiv(p.Wo);
    p.div_fw = FastDiv(p.fW);
    p.div_spi = FastDiv(p.Ho / R);
    return cdiv(p.nslabs, p.per);
}

// Fills the plan of wgrad_halo_f32 and returns the number of workgroups (= splits), or 0 when the
// kernel does not apply: unit stride, 64 input channels, D a multiple of 4 up to 64, at most 9 taps,
// an even Wo of 28, 32, 56 or 64 (the built pair counts), at most 3 filter rows of at most 68 padded
// columns, and at least 4 output rows per CU (tuning: wgrad_halo = 1 drops the last condition, =0 turns
// the kernel off).
static int plan_wgrad_halo_f32(WgradHaloParams& p, int C, int sH, int sW, int cus) {
    if (sH != 1 || sW != 1 || C != 64 || p.D % 4 != 0 || p.D > 64 || p.fH * p.fW > 9) return 0;
    if (tuning().wgrad_halo == 0) return 0;
    const bool force = tuning().wgrad_halo > 0;
    if (p.Wo != 28 && p.Wo != 32 && p.Wo != 56 && p.Wo != 64) return 0;
    p.R = 1;
    p.slab_m = p.Wo;
    p.Wp = (int)round_up(p.Wo + p.fW - 1, 4);            // row pitch of the halo in LDS: whole loads of 4 slots
    p.hslots = p.fH * p.Wp;
    if (p.fH > 3 || p.Wp > kFhRowSlots) return 0;
    const int64_t nslabs = (int64_t)p.S * p.Ho;
    if (nslabs > (1 << 24) || (!force && nslabs < 4 * (int64_t)cus)) return 0;
    // byte offsets are formed in 32 bits from the pixel above and left of the image
    if (((int64_t)p.S * p.H + p.fH) * p.W * 256 >= ((int64_t)1 << 31)) return 0;
    p.nslabs = (int)nslabs;
    const int wgs = (int)std::min<int64_t>(nslabs, cus);
    p.per = cdiv(p.nslabs, wgs);
    p.div_wp = FastDiv(p.Wp);
    p.div_wo = FastDiv(p.Wo);
    p.div_fw = FastDiv(p.fW);
    p.div_spi = FastDiv(p.Ho);
    return cdiv(p.nslabs, p.per);
}

template <typename T>
int conv_wgrad_impl(const char* fn, const T* x, const T* dy, float* dw, float* dbias,
                    int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW,
                    bool swapped = false) {      // swapped: x and dy (C and D) arrive exchanged, see below
    int Ho, Wo;
    int rc = check_conv_dims(fn, S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    if (!swapped) {
        // An x or dy of 2^31 bytes and more: the samples go in runs (sample_runs.h), every run's dw and dbias into a
        // row of a temporary [runs][K D + D], and the rows are added in run order like the partial sums of one launch.
        const int64_t xs = (int64_t)H * W * C, ys = (int64_t)Ho * Wo * D;
        const SampleRuns runs = plan_sample_runs(S, xs * (int64_t)sizeof(T), ys * (int64_t)sizeof(T));
        if (runs.runs > 1) {
            const int64_t kd = (int64_t)fH * fW * C * D;
            const int64_t stride = round_up(kd, 4) + round_up(D, 4);            // rows and their dbias parts 16-byte aligned
            void* tmp = nullptr;
            rc = aeth_malloc(&tmp, runs.runs * stride * (int64_t)sizeof(float));
            if (rc) return rc;
            float* rows = static_cast<float*>(tmp);
            int r = 0;
            for (int s0 = 0; s0 < S && rc == AETH_OK; s0 += runs.per, ++r)
                rc = conv_wgrad_impl<T>(fn, x + s0 * xs, dy + s0 * ys, rows + r * stride,
                                        dbias ? rows + r * stride + round_up(kd, 4) : nullptr, std::min(runs.per, S - s0), H, W,
                                        C, D, fH, fW, sH, sW, pH, pW);
            if (rc == AETH_OK) {
                // two reductions over the rows: dw, then dbias (the plain kernel: any alignment of dw and dbias)
                hipLaunchKernelGGL(reduce_splits, dim3(cdiv(kd, 64)), dim3(kThreads), 0, ctx().stream, (const float*)rows, dw,
                                   (float*)nullptr, (int)kd, (int)kd, (int)stride, r);
                if (dbias)
                    hipLaunchKernelGGL(reduce_splits, dim3(cdiv(D, 64)), dim3(kThreads), 0, ctx().stream,
                                       (const float*)(rows + round_up(kd, 4)), dbias, (float*)nullptr, D, D, (int)stride, r);
                if (hipGetLastError() != hipSuccess) rc = fail(AETH_E_HIP, "%s: kernel launch failed", fn);
            }
            const int rc_free = aeth_free(tmp);             // (stream order: the block is reused only by later launches)
            return rc ? rc : rc_free;
        }
    }
    if constexpr (sizeof(T) == 4) {
        // at most 16 output channels and few rows: one thread per element of dw walks the rows
        const int64_t M = (int64_t)S * H * W;
        if (narrow_shape(D, fH, fW, sH, sW, pH, pW) && M > 0 && M <= 1024 && (int64_t)(C + 1) * 16 < ((int64_t)1 << 31)) {
            NarrowParams np;
            np.a = x; np.b = dy; np.bias = nullptr; np.out = dw; np.out2 = dbias;
            np.M = (int)M; np.K = C; np.N = D;
            hipLaunchKernelGGL(narrow_wgrad, dim3((unsigned)cdiv((int64_t)(C + 1) * 16, kThreads)), dim3(kThreads), 0, ctx().stream, np);
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    Context& c = ctx();
    if constexpr (sizeof(T) == 4) {
        // A 1x1 filter on at most 64 input channels, many more output channels and many rows (64 -> 256 on 56x56
        // images): as dw[64][D] the product has one half-width k tile, D / 64 n tiles that all re-read x, and two
        // MFMAs per pair of operand reads.  Its transpose dy^T . x has D / 128 full-width k tiles over one n tile:
        // the same kernel with the operands swapped, four MFMAs per pair of reads, dy read once and x twice
        // (0.256 ms against 0.290 on that shape); the reduction writes the transpose back.
        const int64_t M = (int64_t)S * H * W;
        const bool shape = fH == 1 && fW == 1 && sH == 1 && sW == 1 && pH == 0 && pW == 0 && C > 32 && C <= 64 &&
                           C % 4 == 0 && D >= 128 && D % 4 == 0 && (int64_t)C * D < ((int64_t)1 << 27) &&
                           M * D * 4 < ((int64_t)1 << 31);
        const bool swap = shape && (tuning().wgrad_swap > 0 ||
                                    (tuning().wgrad_swap < 0 && M >= (int64_t)256 * 3 * c.prop.multiProcessorCount));
        if (swap && !swapped) return conv_wgrad_impl<T>(fn, dy, x, dw, dbias, S, H, W, D, C, 1, 1, 1, 1, 0, 0, true);
    }
    WgradParams p;
    p.x = x; p.dy = dy;
    p.swap = swapped ? 1 : 0;
    p.db_len = swapped ? C : D;
    p.S = S; p.H = H; p.W = W; p.C = C; p.Ho = Ho; p.Wo = Wo; p.D = D;
    p.M = S * Ho * Wo; p.K = fH * fW * C;
    p.fW = fW; p.sH = sH; p.sW = sW; p.pH = pH; p.pW = pW;
    p.want_dbias = dbias != nullptr;
    p.div_howo = FastDiv(Ho * Wo); p.div_wo = FastDiv(Wo); p.div_c = FastDiv(C); p.div_fw = FastDiv(fW);
    constexpr int CE = Elem<T>::CE;
    const bool va = (C % CE == 0), vy = (D % CE == 0);
    const int64_t xb = (int64_t)S * H * W * C * (int64_t)sizeof(T), yb = (int64_t)p.M * D * (int64_t)sizeof(T);
    const bool fits = xb < ((int64_t)1 << 31) && yb < ((int64_t)1 << 31);
    // fp32: the LDS-direct kernel takes any C (one float per lane and load when C % 4 != 0)
    const bool dma = sizeof(T) == 4 && vy && fits;
    const bool dma16 = sizeof(T) == 2 && va && vy && fits;      // bf16 MFMA kernel, 64-row slabs
    p.x_bytes = (dma || dma16) ? (unsigned)xb : 0u;
    p.dy_bytes = (dma || dma16) ? (unsigned)yb : 0u;
    {
        WgradHaloParams hp;
        hp.x = x; hp.dy = dy;
        hp.x_bytes = p.x_bytes; hp.dy_bytes = p.dy_bytes;
        hp.S = S; hp.H = H; hp.W = W; hp.Ho = Ho; hp.Wo = Wo; hp.D = D; hp.fH = fH; hp.fW = fW; hp.pH = pH; hp.pW = pW;
        hp.want_dbias = dbias != nullptr;
        int splits = 0;
        if constexpr (sizeof(T) == 2) splits = dma16 ? plan_wgrad_halo(hp, C, sH, sW, c.prop.multiProcessorCount) : 0;
        else splits = (dma && va && !swapped) ? plan_wgrad_halo_f32(hp, C, sH, sW, c.prop.multiProcessorCount) : 0;
        if (splits > 0) {
            const int64_t kd = (int64_t)p.K * D;
            void* ws;
            rc = workspace((int64_t)splits * (kd + D) * sizeof(float), &ws);
            if (rc) return rc;
            hp.out = (float*)ws;
            if constexpr (sizeof(T) == 2) {
                hipLaunchKernelGGL(wgrad_halo_bf16, dim3(splits), dim3(64 * (fH * fW + 1)), 0, c.stream, hp);
            } else {
                const dim3 grid(splits), block(64 * kFhWaves);
                if (Wo == 56) hipLaunchKernelGGL(wgrad_halo_f32<28>, grid, block, 0, c.stream, hp);
                else if (Wo == 64) hipLaunchKernelGGL(wgrad_halo_f32<32>, grid, block, 0, c.stream, hp);
                else if (Wo == 32) hipLaunchKernelGGL(wgrad_halo_f32<16>, grid, block, 0, c.stream, hp);
                else hipLaunchKernelGGL(wgrad_halo_f32<14>, grid, block, 0, c.stream, hp);
            }
            AETH_LAUNCH_CHECK();
            const int n = (int)(kd + (dbias ? D : 0));
            const bool r4 = (reinterpret_cast<uintptr_t>(dw) & 15) == 0 &&
                            (dbias == nullptr || (reinterpret_cast<uintptr_t>(dbias) & 15) == 0);
            if (r4)
                hipLaunchKernelGGL(reduce_splits4, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream, (const float*)ws, dw,
                                   dbias, (int)kd, n, (int)(kd + D), splits);
            else
                hipLaunchKernelGGL(reduce_splits, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream, (const float*)ws, dw,
                                   dbias, (int)kd, n, (int)(kd + D), splits);
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    // operand width of the fp32 LDS-direct kernel: 192-wide k tiles where they pad fewer rows than 128-wide ones
    p.cw = !va ? 1 : (p.K <= 64 ? 2 : 4);
    if (dma && p.cw == 4) {
        // (equal padding and a last 128-wide tile at most a quarter full, K = 288: 27.5 us on 192-wide tiles against 29.2;
        // equal padding with whole 128-wide tiles, K = 384, 768, 1152: 128-wide is 3 to 6 % faster)
        const int pad192 = cdiv(p.K, 192) * 192, pad128 = cdiv(p.K, kWgBK) * kWgBK, last128 = p.K % kWgBK;
        if (pad192 < pad128 || (pad192 == pad128 && last128 != 0 && last128 <= kWgBK / 4)) p.cw = 6;
    }
    if (dma && va && p.K > 64 && (tuning().wgrad_cw == 4 || tuning().wgrad_cw == 6)) p.cw = tuning().wgrad_cw;
    if (swapped) p.cw = 4;                             // (the form that adds up the columns of its x slabs)
    // slab height of the 192-wide kernel: 16 rows (three workgroups per CU) where a workgroup walks at
    // least 64 of them (56x56x64: 0.481 ms against 0.487 with 32 rows; 8x8x64 -> 128, batch 128, 8 slabs of
    // 32 per workgroup: 27.2 us with 32 rows, 28.3 with 16); tuning: wgrad_br overrides
    int br = kWgBR;
    if (dma && p.cw == 6) {
        const int kt6 = cdiv(p.K, 192), nt6 = cdiv(D, kWgBN);
        const int64_t wgs = (int64_t)3 * c.prop.multiProcessorCount;
        if ((int64_t)cdiv(p.M, 32) * kt6 * nt6 >= 32 * wgs) br = 16;
        if (tuning().wgrad_br == 32 || tuning().wgrad_br == 16) br = tuning().wgrad_br;
    }
    {
        const int qs = br / (Ho * Wo), rem = br % (Ho * Wo), qh = rem / Wo, qw = rem % Wo;
        p.step_c = qw * sW;
        p.step_r = qh * sH;
        p.inc0 = 4 * C * (qw * sW + qh * sH * W + qs * H * W);
        p.inc1 = 4 * C * (-Wo * sW + sH * W);
        p.inc2 = 4 * C * (-Ho * sH * W + H * W);
    }
    // bf16: wide wave tiles (128 k x 256 n or 128 k x 128 n per workgroup) where they pad the output
    // channels by at most a third more than 64-wide tiles do (tuning: wgrad_wide = 0 never, >= 1 wherever D > 64)
    int wide_nb = 0;
    if (dma16 && D > 64 && tuning().wgrad_wide != 0) {
        const int64_t pad64 = round_up(D, 64), pad128 = round_up(D, 128), pad256 = round_up(D, 256);
        const bool force = tuning().wgrad_wide > 0;
        if (pad256 * 3 <= pad64 * 4) wide_nb = 4;
        else if (pad128 * 3 <= pad64 * 4 || force) wide_nb = 2;
    }
    // 256 k rows per workgroup (8 waves, one workgroup per CU) where K has more than two 128-row tiles and
    // the slabs are long enough to give every CU a share of m (tuning: wgrad_wide = 2 never, 3 always)
    const int tile_n = wide_nb ? 64 * wide_nb : kWgBN;
    bool wide_k = wide_nb == 4 && p.K > 256 && (int64_t)cdiv(p.M, kWwBR) * cdiv(p.K, 256) >= 8 * (int64_t)c.prop.multiProcessorCount;
    if (tuning().wgrad_wide == 2) wide_k = false;
    if (tuning().wgrad_wide == 3 && wide_nb == 4) wide_k = true;
    const int tkw = wide_k ? 256 : (!dma ? kWgBK : (p.cw == 1 ? 32 : (p.cw == 6 ? 192 : kWgBK)));
    const int kt = cdiv(p.K, tkw), nt = cdiv(D, tile_n);
    const int slab_rows = wide_nb ? kWwBR : (dma16 ? 64 : kWgBR);
    const int slabs = cdiv(p.M, slab_rows);           // fp32: counted in 32-row units for both tile shapes
    // one round of resident workgroups (3 per CU for the LDS-direct kernels, 2 for the 192-wide
    // one and the register-staged one), rounded down so that no second, nearly empty round follows.
    // Every further round costs a set-up, an epilogue and a share of the reduction per workgroup
    // (56x56x64: 0.485 ms with one round, 0.493 with two, 0.509 with four).
    int rounds = 1;
    if (tuning().wgrad_rounds >= 1 && tuning().wgrad_rounds <= 4) rounds = tuning().wgrad_rounds;
    const int per_cu2 = (wide_k ? 1 : wide_nb == 4 ? 2 : (((dma && (p.cw != 6 || br == 16)) || dma16) ? 3 : 2)) * rounds;
    int splits = (per_cu2 * c.prop.multiProcessorCount) / (kt * nt);
    // a workgroup's set-up, epilogue and its share of the reduction are worth several slabs
    // (training step of the 3-block CNN: 0.672 ms with 1, 0.642 with 4, 0.611 with 8, 0.658 with 16)
    const int min_slabs = 8;
    if (splits > cdiv(slabs, min_slabs)) splits = cdiv(slabs, min_slabs);
    if (splits < 1) splits = 1;
    int slabs_per = cdiv(slabs, splits);
    splits = cdiv(slabs, slabs_per);
    p.m_per_split = slabs_per * slab_rows;
    const int64_t kd = (int64_t)p.K * D;
    // one split (few rows: a dense layer on a small batch): the kernel writes dw and dbias themselves, no reduction launch
    // (dw aligned for the 16-byte stores of the fp32 kernel, as the workspace is)
    const bool single = splits == 1 && (reinterpret_cast<uintptr_t>(dw) & 15) == 0 && !swapped;   // (the reduction writes the transpose back)
    void* ws = nullptr;
    if (!single) {
        rc = workspace((int64_t)splits * (kd + p.db_len) * sizeof(float), &ws);
        if (rc) return rc;
    }
    p.out = single ? dw : (float*)ws;
    p.db_out = single ? dbias : nullptr;
    p.kt = kt; p.nt = nt;
    dim3 grid(kt * nt * splits);
    const int n = (int)(kd + (dbias ? p.db_len : 0));
    const bool r4 = kd % 4 == 0 && D % 4 == 0 && p.db_len % 4 == 0 && (reinterpret_cast<uintptr_t>(dw) & 15) == 0 &&
                    (dbias == nullptr || (reinterpret_cast<uintptr_t>(dbias) & 15) == 0);
    if constexpr (sizeof(T) == 4) {
        // An entry point that also computes this layer's input gradient is collecting the launches (pair_launch.h): the
        // two fp32 LDS-direct forms with 32-row slabs wait for the dgrad launch to share a grid with.
        PairCtl& pc = pair_ctl();
        if (pc.armed && pc.wgrad_kind == kHeldNone && dma && !swapped && (p.cw != 6 || br == 32) && (single || r4)) {
            pc.wgrad_kind = p.cw == 6 ? kHeldWgrad192 : kHeldWgrad128;
            pc.wgrad_blocks = grid.x;
            pc.wgrad_in_ws = !single;
            held_wgrad_params() = p;
            pc.wgrad_sum = HeldSum();
            if (!single) {
                pc.wgrad_sum.on = 1;
                pc.wgrad_sum.out = dw; pc.wgrad_sum.dbias = dbias;
                pc.wgrad_sum.n_out = (int)kd; pc.wgrad_sum.n = n; pc.wgrad_sum.stride = (int)(kd + p.db_len); pc.wgrad_sum.splits = splits;
                workspace_prefix((int64_t)splits * (kd + p.db_len) * (int64_t)sizeof(float));
            }
            return AETH_OK;
        }
    }
    if (wide_k) hipLaunchKernelGGL((wgrad_gemm_dma_bf16w<4, 4>), grid, dim3(512), 0, c.stream, p);
    else if (wide_nb == 4) hipLaunchKernelGGL((wgrad_gemm_dma_bf16w<2, 4>), grid, dim3(kThreads), 0, c.stream, p);
    else if (wide_nb == 2) hipLaunchKernelGGL((wgrad_gemm_dma_bf16w<2, 2>), grid, dim3(kThreads), 0, c.stream, p);
    else if (dma16) hipLaunchKernelGGL(wgrad_gemm_dma_bf16, grid, dim3(kThreads), 0, c.stream, p);
    else if (dma && p.cw == 6 && br == 16) hipLaunchKernelGGL(wgrad_gemm_dma192h, grid, dim3(kThreads), 0, c.stream, p);
    else if (dma && p.cw == 6) hipLaunchKernelGGL(wgrad_gemm_dma192, grid, dim3(kThreads), 0, c.stream, p);
    else if (dma) hipLaunchKernelGGL(wgrad_gemm_dma, grid, dim3(kThreads), 0, c.stream, p);
    else if (va && vy) hipLaunchKernelGGL((wgrad_gemm<T, CE, CE>), grid, dim3(kThreads), 0, c.stream, p);
    else if (va) hipLaunchKernelGGL((wgrad_gemm<T, CE, 1>), grid, dim3(kThreads), 0, c.stream, p);
    else if (vy) hipLaunchKernelGGL((wgrad_gemm<T, 1, CE>), grid, dim3(kThreads), 0, c.stream, p);
    else hipLaunchKernelGGL((wgrad_gemm<T, 1, 1>), grid, dim3(kThreads), 0, c.stream, p);
    AETH_LAUNCH_CHECK();
    if (single) return AETH_OK;
    const int tr = swapped ? D : 0;                      // the partials hold dw^T in rows of D (the caller's C) floats
    if (r4)
        hipLaunchKernelGGL(reduce_splits4, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream, (const float*)ws, dw, dbias,
                           (int)kd, n, (int)(kd + p.db_len), splits, tr);
    else
        hipLaunchKernelGGL(reduce_splits, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream, (const float*)ws, dw, dbias,
                           (int)kd, n, (int)(kd + p.db_len), splits, tr);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}


}  // namespace aeth
