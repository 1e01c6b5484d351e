// Host side of the gather-GEMM path: which kernel a problem gets, split K, and the fprop / dgrad
// entry points' shared implementation.
#pragma once
#include "gather_kernels.h"
#include "dgrad_parts.h"
#include "narrow_kernels.h"
#include "pair_launch.h"
#include "sample_runs.h"
#include "tuning.h"

namespace aeth {

// dense_res_f32 applies to fp32 gathers that are plain matrix products (one tap, unit stride, no
// padding), K = 32 or 64 whole, N a multiple of 4 up to 256 with more than one 64-wide tile, a dense
// output with 16-byte stores, and at least 4 tiles of 128 rows per CU (tuning: dense_res = 1 drops the
// last condition, =0 turns the kernel off).
static bool plan_dense_res(const GatherParams& gp, bool dma, int cus, int* mtiles) {
    if (!dma || gp.sh != 1 || gp.sw != 1 || gp.rh0 != 0 || gp.rw0 != 0 || gp.Hs != gp.Hg || gp.Ws != gp.Wg) return false;
    if (gp.K != gp.Cs || gp.K != gp.Kpad || (gp.K != 32 && gp.K != 64) || gp.split_slabs != 0) return false;
    if (gp.N <= 64 || gp.N > kD1MaxN || !gp.dense_out || gp.out_bytes == 0) return false;
    if (tuning().dense_res == 0) return false;
    const bool force = tuning().dense_res > 0;
    const int n = cdiv(gp.M, kD1BM);
    if (!force && n < 4 * cus) return false;
    *mtiles = n;
    return true;
}

// Tiles stored as runs of contiguous channels carry the non-temporal hint: right for an output that streams to memory,
// wrong for one that the next kernel would have found in L2 (the layers of a small network: training step of the three-block
// CNN 0.389 ms with them, 0.384 with the 16-byte pieces).  From 64 MB of output on; tuning: gather_runs = 1 always, 0 never.
static inline bool run_stores(const GatherParams& gp) {
    const int v = tuning().gather_runs;
    if (v == 0 || gp.out_bytes == 0) return false;
    return v > 0 || gp.out_bytes >= (64u << 20);
}

// The problems of a strided fp32 dgrad: while armed, a problem whose launch is the 128 x 64 slab kernel with scalar addressing
// and an unsplit K is collected here instead of going out, and conv_dgrad_impl launches what it has collected in grids of up to
// kMaxClassesF32 problems.
constexpr int kMaxHeldClasses = 16;
struct ClassHold {
    bool armed = false;
    int count = 0;
    bool runs[kMaxHeldClasses];
    bool bkn[kMaxHeldClasses];             // the problem reads the filter as the [K][N] operand (fprop)
    unsigned blocks[kMaxHeldClasses];
    GatherParams gp[kMaxHeldClasses];
};
static inline ClassHold& class_hold() {
    static ClassHold h;
    return h;
}
static inline bool hold_class(const GatherParams& gp, const dim3& grid, bool runs, bool bkn = false) {
    ClassHold& h = class_hold();
    if (!h.armed || h.count >= kMaxHeldClasses || grid.y != 1 || gp.split_slabs != 0) return false;
    h.runs[h.count] = runs;
    h.bkn[h.count] = bkn;
    h.blocks[h.count] = grid.x;
    h.gp[h.count] = gp;
    ++h.count;
    return true;
}
// Launches what was collected: shared grids, the problems with the most taps first, when all problems of the dgrad were collected
// with the same store form; else the collected ones one by one (the others have gone out already; the problems write
// disjoint pixels of dx).
static inline void flush_classes(int nsets, hipStream_t st) {
    ClassHold& h = class_hold();
    h.armed = false;
    bool same = h.count == nsets && h.count > 1;
    for (int i = 1; i < h.count; ++i) same = same && h.runs[i] == h.runs[0] && h.bkn[i] == h.bkn[0];
    if (!same) {
        for (int i = 0; i < h.count; ++i) {
            const dim3 g(h.blocks[i]), b(kThreads);
            if (h.bkn[i] && h.runs[i]) hipLaunchKernelGGL((gather_gemm_dma<float, 128, 64, 32, 64, true, 8, false, true, true, true>), g, b, 0, st, h.gp[i]);
            else if (h.bkn[i]) hipLaunchKernelGGL((gather_gemm_dma<float, 128, 64, 32, 64, true, 8, false, true, false, true>), g, b, 0, st, h.gp[i]);
            else if (h.runs[i]) hipLaunchKernelGGL((gather_gemm_dma<float, 128, 64, 32, 64, true, 8, false, true, true>), g, b, 0, st, h.gp[i]);
            else hipLaunchKernelGGL((gather_gemm_dma<float, 128, 64, 32, 64, true, 8, false, true>), g, b, 0, st, h.gp[i]);
        }
        h.count = 0;
        return;
    }
    int order[kMaxHeldClasses];                              // most taps first
    for (int i = 0; i < h.count; ++i) {
        int j = i;
        for (; j > 0 && h.gp[order[j - 1]].K < h.gp[i].K; --j) order[j] = order[j - 1];
        order[j] = i;
    }
    for (int first = 0; first < h.count; first += kMaxClassesF32) {
        GatherClassesF32 gc;
        ClassGrid cg;
        unsigned total = 0;
        gc.ncls = std::min(kMaxClassesF32, h.count - first);
        for (int i = 0; i < kMaxClassesF32; ++i) {
            cg.start[i] = total;
            cg.blocks[i] = 0;
            if (i >= gc.ncls) continue;
            gc.cls[i] = h.gp[order[first + i]];
            cg.blocks[i] = h.blocks[order[first + i]];
            total += (unsigned)round_up(cg.blocks[i], kXcds);
        }
        if (h.bkn[0] && h.runs[0]) hipLaunchKernelGGL((gather_classes_f32<true, true>), dim3(total), dim3(kThreads), 0, st, gc, cg);
        else if (h.bkn[0]) hipLaunchKernelGGL((gather_classes_f32<false, true>), dim3(total), dim3(kThreads), 0, st, gc, cg);
        else if (h.runs[0]) hipLaunchKernelGGL((gather_classes_f32<true, false>), dim3(total), dim3(kThreads), 0, st, gc, cg);
        else hipLaunchKernelGGL((gather_classes_f32<false, false>), dim3(total), dim3(kThreads), 0, st, gc, cg);
    }
    h.count = 0;
}

// A dgrad launch of one of the two slab-kernel forms that small layers get joins the wgrad launch that is being held
// for it (pair_launch.h) instead of going out on its own.
// Launches of at most 4 workgroups per CU: a pair has room for 2 per CU (the LDS of the larger body), which a launch that
// fills the GPU many times over would feel.  (tuning: pair_bwd > 0 is a mask of the dgrad kinds that may join, bit kind - 1)
static inline bool pair_accepts(int kind) {
    const PairCtl& pc = pair_ctl();
    if (!pc.armed || !pc.dgrad_ok || pc.wgrad_kind == kHeldNone || pc.dgrad_kind != kHeldNone) return false;
    const int v = tuning().pair_bwd;
    return v < 0 || ((v >> (kind - 1)) & 1) != 0;
}

static inline bool hold_gather_for_pair(const GatherParams& gp, const dim3& grid, int kind) {
    PairCtl& pc = pair_ctl();
    if (!pair_accepts(kind) || (int64_t)grid.x * grid.y > 4 * (int64_t)ctx().prop.multiProcessorCount) return false;
    pc.dgrad_kind = kind;
    pc.dgrad_gx = grid.x;
    pc.dgrad_gy = grid.y;
    pc.gather = gp;
    return true;
}

template <typename T, int BM, int BN, int WM, int WN, int KC>
static void launch_gather_dma(const GatherParams& gp, hipStream_t st) {
    constexpr int kThreads = 64 * (BM / WM) * (BN / WN);     // of this tile shape (shadows the 256 of the others)
    dim3 grid(cdiv(gp.M, BM) * cdiv(gp.N, BN));
    if (gp.split_slabs > 0) grid.y = (unsigned)cdiv(gp.Kpad / (KC * Elem<T>::CE), gp.split_slabs);
    const bool ut = gp.Cs % (KC * Elem<T>::CE) == 0 && gp.K == gp.Kpad && gp.K / gp.Cs <= 32;
    // short K, several n tiles: one workgroup per m tile walks the n tiles (128 x 64 tiles only)
    if constexpr (BM == 128 && BN == 64 && KC == 8) {
        if (gp.split_slabs == 0 && gp.Kpad / (KC * Elem<T>::CE) <= 2 && gp.N > BN && gp.N <= kNloopMaxN && gp.out_bytes != 0 &&
            tuning().gather_nloop != 0) {
            grid.x = (unsigned)cdiv(gp.M, BM);
            if (ut) hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, true>), grid, dim3(kThreads), 0, st, gp);
            else hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, false, KC, true>), grid, dim3(kThreads), 0, st, gp);
            return;
        }
    }
    if constexpr ((BM == 128 || BM == 64) && sizeof(T) == 4) {
        // scalar addressing (tuning: gather_sa = 0 turns it off); the moved base must stay a 32-bit extent
        const int taps = gp.Cs > 0 ? gp.K / gp.Cs : 0;
        const int64_t bias = ((int64_t)std::max(-gp.rh0, 0) * gp.Ws + std::max(-gp.rw0, 0)) * gp.Cs * (int64_t)sizeof(T);
        if (ut && taps <= 32 && (int64_t)gp.src_bytes + bias < ((int64_t)1 << 31) && tuning().gather_sa != 0) {
            // 64-column wave tiles store runs of 256 contiguous bytes per pixel (tuning: gather_runs = 0 keeps the 16-byte pieces)
            bool runs = false;
            if constexpr (WN == 64 || WN == 32) runs = gp.split_slabs == 0 && run_stores(gp);
            if constexpr (KC == 8) {
                if (gp.bt_kn) {
                    if constexpr (BM == 128 && BN == 64 && WM == 32 && WN == 64) {
                        if (hold_class(gp, grid, runs, true)) return;
                    }
                    if constexpr (WN == 64 || WN == 32) {
                        if (runs) {
                            hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false, true, true, true>), grid, dim3(kThreads), 0, st, gp);
                            return;
                        }
                    }
                    hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false, true, false, true>), grid, dim3(kThreads), 0, st, gp);
                    return;
                }
            }
            if constexpr (BM == 128 && BN == 64 && WM == 32 && WN == 64 && KC == 8) {
                if (hold_class(gp, grid, runs)) return;
            }
            if constexpr (WN == 64 || WN == 32) {
                if (runs) {
                    hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false, true, true>), grid, dim3(kThreads), 0, st, gp);
                    return;
                }
            }
            if constexpr (KC == 8 && WM == 32 && WN == 32 && ((BM == 128 && BN == 32) || (BM == 64 && BN == 64))) {
                if (hold_gather_for_pair(gp, grid, BM == 128 ? kHeldGather128x32 : kHeldGather64x64)) return;
            }
            hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false, true>), grid, dim3(kThreads), 0, st, gp);
            return;
        }
    }
    if constexpr (sizeof(T) == 4 && KC == 8 && kThreads == 256) {
        if (gp.bt_kn) {                                      // fprop reading the filter in place
            if (ut) hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false, false, false, true>), grid, dim3(kThreads), 0, st, gp);
            else hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, false, KC, false, false, false, true>), grid, dim3(kThreads), 0, st, gp);
            return;
        }
    }
    if constexpr (sizeof(T) == 2) {
        // the bf16 tiles store runs of contiguous channels (tuning: gather_runs = 0 keeps the 16-byte pieces per pixel)
        if (gp.split_slabs == 0 && run_stores(gp)) {
            if (ut) hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false, false, true>), grid, dim3(kThreads), 0, st, gp);
            else hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, false, KC, false, false, true>), grid, dim3(kThreads), 0, st, gp);
            return;
        }
    }
    if (ut) hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false>), grid, dim3(kThreads), 0, st, gp);
    else hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, false, KC, false>), grid, dim3(kThreads), 0, st, gp);
}

// kc4: shallow slabs (4 chunks of k per row) for the LDS-direct kernel where the tile allows it
template <typename T, int BM, int BN, int WM, int WN>
static void launch_gather_cfg(const GatherParams& gp, bool vec, bool kc4, hipStream_t st) {
    dim3 grid(cdiv(gp.M, BM) * cdiv(gp.N, BN));
    if (vec && gp.src_bytes != 0 && gp.bt_bytes != 0) {
        if constexpr (BM >= 64 && BN >= 64) {
            if (kc4) {
                launch_gather_dma<T, BM, BN, WM, WN, 4>(gp, st);
                return;
            }
        }
        launch_gather_dma<T, BM, BN, WM, WN, 8>(gp, st);
    }
    else if (vec)
        hipLaunchKernelGGL((gather_gemm<T, BM, BN, WM, WN, Elem<T>::CE>), grid, dim3(kThreads), 0, st, gp);
    else
        hipLaunchKernelGGL((gather_gemm<T, BM, BN, WM, WN, 1>), grid, dim3(kThreads), 0, st, gp);
}

static inline int gather_bn(int N) { return N <= 32 ? 32 : 64; }

// Set while the problems of one strided fp32 dgrad are planned and launched so that all of them, the border strips
// included, take the 128-row slab kernel with an unsplit K and can share one grid (conv_dgrad_impl).
static inline bool& uniform_class_tiles() {
    static bool on = false;
    return on;
}

// Tile height.  The LDS-direct kernel keeps two slabs per operand in LDS, so a
// 128-row tile (48 KB) lets three workgroups share a CU where a 256-row tile
// (80 KB) allows one or two; measured on the 56x56x64 shape, 128 rows is 11 %
// faster.  64-row tiles (32 KB, five per CU) leave a smaller last round and
// win on few tiles, 128-row tiles (wave tiles of 32 x 64: three operand reads per
// two MFMAs instead of two per one) on many: fp32 takes 128 rows from 10 tiles per
// CU on (128 against 64 rows on 56x56x64 -> 64 and 28x28x128 -> 128, 3x3: +10 % at
// 784 tiles, +4 % at 1568, +1 % at 2352, -1 % at 3136, -2 % at 4704, -3 % at 5488;
// 28x28x128 -> 256 stride 2, 2704 tiles: -3.8 %).  The register-staged kernel
// prefers 256 rows.
static inline int gather_bm(int M, int N, int cus, bool dma, int elem_bytes = 4) {
    const int bn = gather_bn(N);
    {                                                       // tuning override: 256, 128 or 64
        const int v = tuning().gather_bm;
        if (v == 256 || v == 128 || (v == 64 && bn == 64)) return v;
    }
    if (uniform_class_tiles() && elem_bytes == 4) return 128;
    const int ntiles = cdiv(N, bn);
    const int want = elem_bytes == 2 ? cus : 2 * cus;   // bf16: the taller tile pays off from one tile per CU on
    const int cands[3] = {256, 128, 64};
    // bf16 MFMAs are 8x shorter per slab: there the larger wave tile of the 256-row shape wins
    for (int i = (dma && elem_bytes == 4) ? 1 : 0; i < 3; ++i) {
        int bm = cands[i];
        if (bn == 32 && bm == 64) break;
        const int64_t tiles = (int64_t)cdiv(M, bm) * ntiles;
        if (dma && elem_bytes == 4 && bm == 128 && bn == 64 && tiles < 10 * (int64_t)cus) continue;
        if (tiles >= want) return bm;
    }
    return bn == 32 ? 128 : 64;
}

// gather_halo_bf16 applies to unit-stride gathers of 2 to 32 taps over whole 64-channel blocks
// when the span of every tile fits its buffer: with tiles cut per image (at most 10 % of empty
// rows) or, failing that, running over image boundaries.  Fills the halo fields of gp and the
// number of 256-row tiles when it does.
static bool plan_halo(GatherParams& gp, bool dma, int* mtiles, int* stages, int min_taps = 2, int max_slots = kHaloSlotsMax) {
    if (!dma || gp.sh != 1 || gp.sw != 1 || gp.Cs % 64 != 0 || gp.K != gp.Kpad || gp.split_slabs != 0) return false;
    const int taps = gp.Th * gp.Tw;
    if (taps < min_taps || taps > 32 || gp.N <= 32 || gp.Cs <= 0 || gp.K != taps * gp.Cs) return false;
    if (tuning().gather_halo == 0) return false;
    const int hw = gp.Hg * gp.Wg;
    // row pitch and image pitch of the padded tensor keep the parity of the pixel grid's (one idle slot per row or
    // image for even filter sizes): the kernel places a slot's chunks by the number of the pixel it serves
    int wp = gp.Wg + gp.Tw - 1, hp = gp.Hg + gp.Th - 1;
    if ((wp - gp.Wg) & 1) ++wp;
    if ((gp.Wg & 1) && ((hp - gp.Hg) & 1)) ++hp;
    if ((int64_t)gp.S * hp * wp >= ((int64_t)1 << 30)) return false;
    auto slot0 = [&](int64_t m) {
        const int64_t s = m / hw, rem = m % hw;
        return (s * hp + rem / gp.Wg) * wp + rem % gp.Wg;
    };
    int64_t longest = 0;
    auto fits = [&](int64_t first, int64_t last) {
        const int64_t span = slot0(last) + (int64_t)(gp.Th - 1) * wp + gp.Tw - slot0(first);
        longest = std::max(longest, span);
        return span <= max_slots;
    };
    // tiles cut per image: every image has the same tiles
    const int per_img = cdiv(hw, kHaloBM);
    bool ok = (int64_t)per_img * kHaloBM * 10 <= (int64_t)hw * 11;
    for (int t = 0; ok && t < per_img; ++t) ok = fits((int64_t)t * kHaloBM, std::min((t + 1) * kHaloBM, hw) - 1);
    if (!ok) longest = 0;
    if (ok) {
        gp.halo_tiles = per_img;
        *mtiles = gp.S * per_img;
    } else {
        const int n = cdiv(gp.M, kHaloBM);
        if (n > (1 << 20)) return false;
        ok = true;
        for (int t = 0; ok && t < n; ++t)
            ok = fits((int64_t)t * kHaloBM, std::min<int64_t>((int64_t)(t + 1) * kHaloBM, gp.M) - 1);
        if (!ok) return false;
        gp.halo_tiles = 0;
        *mtiles = n;
    }
    *stages = longest <= halo_slots(4) ? 4 : 3;
    gp.halo_wp = wp;
    gp.halo_hp = hp;
    gp.div_halo_wp = FastDiv(wp);
    gp.div_halo_hp = FastDiv(hp);
    gp.div_halo_tiles = FastDiv(gp.halo_tiles > 0 ? gp.halo_tiles : 1);
    return true;
}

// gather_halo_res_bf16 applies to unit-stride gathers of 2 to 9 taps over one 64-channel block
// with N in one tile, when 224-row tiles are whole rows of one image (Wg divides 224, at most
// 15 % of empty rows in an image's last tile), a tile's rows and its halo fit a halo buffer and
// there are at least 4 tiles per CU to walk (tuning: gather_res = 1 or 2 drops the last condition,
// 0 turns the kernel off).
static bool plan_halo_res(GatherParams& gp, bool dma, int cus, int* mtiles) {
    if (!dma || gp.sh != 1 || gp.sw != 1 || gp.Cs != 64 || gp.K != gp.Kpad || gp.split_slabs != 0) return false;
    const int taps = gp.Th * gp.Tw;
    if (taps < 2 || taps > kResMaxTaps || gp.N <= 32 || gp.N > 64 || gp.K != taps * gp.Cs) return false;
    if (tuning().gather_res == 0 || tuning().gather_halo == 0) return false;
    const bool force = tuning().gather_res > 0;
    if (gp.Wg <= 0 || kResBM % gp.Wg != 0) return false;
    const int hw = gp.Hg * gp.Wg;
    int wp = gp.Wg + gp.Tw - 1;                                          // row pitch of the halo: the parity of the pixel rows'
    if ((wp - gp.Wg) & 1) ++wp;                                          // (chunks are placed by pixel number, see the kernel)
    const int hp = gp.Hg + gp.Th - 1;
    const int rows = kResBM / gp.Wg;                                     // image rows per tile
    if ((int64_t)(rows + gp.Th - 1) * wp > kResSlots) return false;      // the tile's rows and the halo below them
    const int per_img = cdiv(hw, kResBM);
    if ((int64_t)per_img * kResBM * 100 > (int64_t)hw * 115) return false;
    const int64_t n = (int64_t)gp.S * per_img;
    if (n > (1 << 24) || (!force && n < 4 * (int64_t)cus)) return false;
    // byte offsets are formed in 32 bits from the pixel above and left of the image
    if (((int64_t)gp.S * gp.Hs + hp) * gp.Ws * 128 >= ((int64_t)1 << 31)) return false;
    *mtiles = (int)n;
    gp.halo_tiles = per_img;
    gp.halo_wp = wp;
    gp.halo_hp = hp;
    gp.div_halo_wp = FastDiv(wp);
    gp.div_halo_hp = FastDiv(hp);
    gp.div_halo_tiles = FastDiv(per_img);
    return true;
}

template <typename T>
static void launch_gather(const GatherParams& gp, bool vec, int cus, hipStream_t st) {
    const int bn = gather_bn(gp.N);
    const bool dma = vec && gp.src_bytes != 0 && gp.bt_bytes != 0;
    if constexpr (sizeof(T) == 2) {
        GatherParams hp = gp;
        int mtiles = 0, stages = 0;
        if (plan_halo(hp, dma, &mtiles, &stages)) {
            dim3 grid((unsigned)(mtiles * cdiv(gp.N, 64)));
            // a dense or strided output that the descriptor covers: tiles go out as runs of 256 contiguous bytes per pixel
            // (tuning: gather_runs = 0 keeps the 16-byte pieces; same bits)
            const bool lines = run_stores(hp);
            if (stages == 4 && lines) hipLaunchKernelGGL((gather_halo_bf16<4, true>), grid, dim3(kThreads), 0, st, hp);
            else if (stages == 4) hipLaunchKernelGGL((gather_halo_bf16<4, false>), grid, dim3(kThreads), 0, st, hp);
            else if (lines) hipLaunchKernelGGL((gather_halo_bf16<3, true>), grid, dim3(kThreads), 0, st, hp);
            else hipLaunchKernelGGL((gather_halo_bf16<3, false>), grid, dim3(kThreads), 0, st, hp);
            return;
        }
    }
    if constexpr (sizeof(T) == 2) {
        // Wide tiles for bf16 launches that the halo kernels do not take (strides, 1x1, long filters): the
        // slab kernel with 256 x 64 tiles fetches (256 + 64) rows of k per 256 x 64 outputs, 11.5 TB/s from
        // L2 on the 28x28x128 -> 256 stride-2 layer, and that rate is what bounds it; 256 x 256 tiles on 8 waves
        // (one workgroup per CU, 128 KB of slabs) fetch 2.5 times less per output, 256 x 128 tiles 1.7 times.
        // From 2 (256 wide) or 4 (128 wide) tiles per CU on (tuning: gather_wide = 1 always, 0 never).
        const bool force = tuning().gather_wide > 0;
        if (dma && gp.split_slabs == 0 && tuning().gather_wide != 0) {
            const int64_t mt = cdiv(gp.M, 256);
            if (gp.N > 192 && (force || mt * cdiv(gp.N, 256) >= 2 * (int64_t)cus)) {
                launch_gather_dma<T, 256, 256, 64, 128, 8>(gp, st);
                return;
            }
            // (the stride-2 layer's dgrad classes, 784 tiles of 1 to 4 taps each, are 4 % slower on them)
            if (gp.N > 64 && (force || mt * cdiv(gp.N, 128) >= 4 * (int64_t)cus)) {
                launch_gather_dma<T, 256, 128, 64, 64, 8>(gp, st);
                return;
            }
        }
    }
    if constexpr (sizeof(T) == 4) {
        int mtiles = 0;
        if (plan_dense_res(gp, dma, cus, &mtiles)) {
            const dim3 grid((unsigned)std::min(mtiles, cus));
            const bool runs = run_stores(gp) && gp.N % 2 == 0;
            if (gp.Kpad == 64 && runs) hipLaunchKernelGGL((dense_res_f32<2, true>), grid, dim3(kD1Threads), 0, st, gp, mtiles);
            else if (gp.Kpad == 64) hipLaunchKernelGGL((dense_res_f32<2, false>), grid, dim3(kD1Threads), 0, st, gp, mtiles);
            else if (runs) hipLaunchKernelGGL((dense_res_f32<1, true>), grid, dim3(kD1Threads), 0, st, gp, mtiles);
            else hipLaunchKernelGGL((dense_res_f32<1, false>), grid, dim3(kD1Threads), 0, st, gp, mtiles);
            return;
        }
    }
    const int bm = gather_bm(gp.M, gp.N, cus, dma, (int)sizeof(T));
    // shallow slabs measure the same as deep ones on the 56x56 layers (within 2 % either
    // way), so they stay a tuning switch: gather_kc = 4
    const bool kc4 = tuning().gather_kc == 4;
    if (bn == 32) {
        if (bm == 256) launch_gather_cfg<T, 256, 32, 64, 32>(gp, vec, false, st);
        else launch_gather_cfg<T, 128, 32, 32, 32>(gp, vec, false, st);
    } else {
        if (bm == 256) launch_gather_cfg<T, 256, 64, 64, 64>(gp, vec, kc4, st);
        else if (bm == 128) launch_gather_cfg<T, 128, 64, 32, 64>(gp, vec, kc4, st);
        else launch_gather_cfg<T, 64, 64, 32, 32>(gp, vec, kc4, st);
    }
}

// One gather-GEMM problem: pack the filter into the workspace at `ws_off`, launch.
struct GatherSetup {
    GatherParams gp;
    PackParams pp;
    int64_t bt_bytes;
    int nsplit = 1;          // > 1: split K, partial products behind the packed filter in the workspace
    int64_t part_bytes = 0;
    struct ActOut* act = nullptr;   // fprop: the activation behind the layer, written by the split reduction where there is one
    bool kn_part = false;    // a part of an fprop: its taps are the filter's taps (pp.xa + th, pp.ya + tw)
};

// The output of the ReLU / leaky ReLU that follows a dense layer, for the split reduction to write on the way
// (`done` says whether it did: a product that is not split leaves it to the caller's own launch).
struct ActOut {
    float* out;
    float alpha;
    bool done;
};

// The kernels that multiply two classes of one dgrad from one halo take 2 or 4 classes that gather_halo_bf16 would take
// (`sets`, already filled in by plan_halo) when every tile of `bm` pixels has a span of the common padded source tensor that
// fits `max_slots`.  The classes are paired (most taps with fewest) and given the common geometry.
static bool plan_class_pairs(const std::vector<GatherSetup>& sets, GatherClasses& gc, int bm, int max_slots, int64_t* mtiles, int64_t* longest) {
    const int n = (int)sets.size();
    if (n != 2 && n != 4) return false;
    const GatherParams& g0 = sets[0].gp;
    if (g0.Cs % 64 != 0 || g0.M <= 0 || g0.out_bytes == 0 || g0.bias != nullptr) return false;
    int rh_min = g0.rh0, rw_min = g0.rw0;
    for (const GatherSetup& gs : sets) {
        const GatherParams& g = gs.gp;
        if (g.Hg != g0.Hg || g.Wg != g0.Wg || g.M != g0.M || g.N != g0.N || g.Cs != g0.Cs || g.src != g0.src || g.S != g0.S ||
            g.Hs != g0.Hs || g.Ws != g0.Ws || g.Th < 1 || g.Tw < 1 || g.sh != 1 || g.sw != 1)
            return false;
        rh_min = std::min(rh_min, g.rh0);
        rw_min = std::min(rw_min, g.rw0);
    }
    int hth = 1, htw = 1;
    for (const GatherSetup& gs : sets) {
        hth = std::max(hth, gs.gp.rh0 - rh_min + gs.gp.Th);
        htw = std::max(htw, gs.gp.rw0 - rw_min + gs.gp.Tw);
    }
    const int hw = g0.Hg * g0.Wg;
    // The padded tensor's row pitch and image pitch keep the parity of the pixel grid's (one idle slot per row or
    // image where needed): a slot's number and the number of the pixel it serves under a tap then differ by an
    // even amount, which is what lets the kernel place chunks by pixel number (no bank conflicts at row ends).
    int wp = g0.Wg + htw - 1, hp = g0.Hg + hth - 1;
    if ((wp - g0.Wg) & 1) ++wp;
    if ((g0.Wg & 1) && ((hp - g0.Hg) & 1)) ++hp;
    if ((int64_t)g0.S * hp * wp >= ((int64_t)1 << 30)) return false;
    auto slot0 = [&](int64_t m) {
        const int64_t s = m / hw, rem = m % hw;
        return (s * hp + rem / g0.Wg) * wp + rem % g0.Wg;
    };
    const int64_t mt = cdiv(g0.M, bm);
    if (mt > (1 << 20)) return false;
    *longest = 0;
    for (int64_t t = 0; t < mt; ++t) {
        const int64_t first = t * bm, last = std::min<int64_t>((t + 1) * bm, g0.M) - 1;
        const int64_t span = slot0(last) + (int64_t)(hth - 1) * wp + htw - slot0(first);
        if (span > max_slots) return false;
        *longest = std::max(*longest, span);
    }
    // most taps first; pairs (0, n - 1), (1, n - 2)
    int order[kMaxClasses];
    for (int i = 0; i < n; ++i) {
        int j = i;
        const int taps = sets[i].gp.Th * sets[i].gp.Tw;
        for (; j > 0 && sets[order[j - 1]].gp.Th * sets[order[j - 1]].gp.Tw < taps; --j) order[j] = order[j - 1];
        order[j] = i;
    }
    for (int i = 0; i < n; ++i) {
        const int src = (i % 2 == 0) ? order[i / 2] : order[n - 1 - i / 2];
        GatherParams g = sets[src].gp;
        g.tap_dh = g.rh0 - rh_min;
        g.tap_dw = g.rw0 - rw_min;
        g.rh0 = rh_min;
        g.rw0 = rw_min;
        g.halo_th = hth;
        g.halo_tw = htw;
        g.halo_wp = wp;
        g.halo_hp = hp;
        g.halo_tiles = 0;
        g.div_halo_wp = FastDiv(wp);
        g.div_halo_hp = FastDiv(hp);
        gc.cls[i] = g;
    }
    gc.ncls = n;
    *mtiles = mt;
    return mt * cdiv(g0.N, 64) * n < ((int64_t)1 << 30);
}

// Split K when the tiles alone would leave most of the chip idle: at most one tile per
// two CUs and at least 8 slabs of K.  Only for the LDS-direct kernel with 16-byte stores
// to a dense [M, N] output.  Aim: about two workgroups per CU, at least 4 slabs each.
template <typename T>
static void plan_split(GatherSetup& gs, bool vec, int cus) {
    const GatherParams& g = gs.gp;
    gs.nsplit = 1;
    gs.part_bytes = 0;
    const int64_t lim = (int64_t)1 << 31;
    const int64_t sb = (int64_t)g.S * g.Hs * g.Ws * g.Cs * (int64_t)sizeof(T);
    const int64_t ob = (int64_t)g.M * g.N * (int64_t)sizeof(float);
    const bool dma = vec && sb < lim && gs.bt_bytes < lim;
    if (!dma || !g.dense_out || g.N % 4 != 0 || ob >= lim || (reinterpret_cast<uintptr_t>(g.out) & 15) != 0) return;
    if (tuning().gather_kc != -1) return;                    // the tuning switch changes the slab depth
    if (tuning().gather_split == 0) return;                  // lets small inputs reach the kernels of large ones
    if (uniform_class_tiles()) return;
    const int bn = gather_bn(g.N), bm = gather_bm(g.M, g.N, cus, true, (int)sizeof(T));
    const int64_t tiles = (int64_t)cdiv(g.M, bm) * cdiv(g.N, bn);
    const int nslabs = g.Kpad / Elem<T>::BK;
    if (tiles * 2 > cus || nslabs < 8) return;
    int n = (int)((2 * (int64_t)cus) / tiles);
    if (n > nslabs / 4) n = nslabs / 4;
    if (n > 64) n = 64;
    if (n < 2) return;
    const int per = cdiv(nslabs, n);
    gs.gp.split_slabs = per;
    gs.nsplit = cdiv(nslabs, per);
    gs.part_bytes = round_up((int64_t)gs.nsplit * ob, 256);
}

// Where the B operand of a problem comes from and how far its tensors reach: the workspace slot at
// `ws_off` for the packed filter, the byte extents for the buffer descriptors, the filter rows.
template <typename T>
static void fill_gather(GatherSetup& gs, char* ws, int64_t ws_off) {
    void* bt = ws + ws_off;
    gs.gp.bt = bt;
    gs.pp.bt = bt;
    const GatherParams& g = gs.gp;
    const int64_t total = (int64_t)gs.pp.Npad * gs.pp.Kpad;
    int64_t sb = (int64_t)g.S * g.Hs * g.Ws * g.Cs * (int64_t)sizeof(T);
    int64_t bb = total * (int64_t)sizeof(T);
    const int64_t lim = (int64_t)1 << 31;
    gs.gp.Th = (g.Tw > 0 && g.Cs > 0) ? (g.K / g.Cs) / g.Tw : 0;
    gs.gp.src_bytes = (sb < lim && bb < lim) ? (unsigned)sb : 0u;
    gs.gp.bt_bytes = (sb < lim && bb < lim) ? (unsigned)bb : 0u;
    const int64_t ob = (g.dense_out ? (int64_t)g.M : (int64_t)g.S * g.Hof * g.Wof) * g.N * (int64_t)sizeof(float);
    const bool ovec = ob < lim && g.N % 4 == 0 && (reinterpret_cast<uintptr_t>(g.out) & 15) == 0;
    gs.gp.out_bytes = ovec ? (unsigned)ob : 0u;
    gs.gp.bt_ld = gs.gp.Kpad;
    gs.gp.bt_direct = 0;
    gs.gp.bt_kn = 0;
}

// dgrad whose slabs lie inside one tap reads its B operand from w itself: row (tap, c) of w is
// contiguous in d, which is dgrad's k.  fp32 slab kernel with at least `min_slabs` = 3 slabs (shorter K
// goes to the n-loop and resident kernels, which keep the packed layout); tuning: gather_direct_b = 0 packs.
// Returns the number of elements pack_filter has to write (0: the filter is read in place).
template <typename T>
static int choose_b_operand(GatherSetup& gs, bool vec, int min_slabs = 3) {
    const GatherParams& g = gs.gp;
    const PackParams& pk = gs.pp;
    constexpr int BK = Elem<T>::BK;
    const int taps = g.Cs > 0 ? g.K / g.Cs : 0;
    // fp32: no B rows past C, such rows of the last tap would lie behind w and the fp32 kernel's loads carry the
    // tap in a scalar offset, which the range check does not see; the bf16 kernels' loads are checked in full,
    // their rows past C read zeros or other taps and feed only columns that are not stored
    const bool rows_ok = sizeof(T) == 4 ? g.N % gather_bn(g.N) == 0 : g.N % 8 == 0;
    if (pk.transposed && vec && g.src_bytes != 0 && g.Cs % BK == 0 && g.K == g.Kpad && taps >= 1 && taps <= 32 &&
        g.Kpad / BK >= min_slabs && g.Th * g.Tw == taps && pk.w_elems * (int64_t)sizeof(T) < ((int64_t)1 << 31) && rows_ok &&
        (reinterpret_cast<uintptr_t>(pk.w) & 15) == 0 && tuning().gather_direct_b != 0 && tuning().gather_kc == -1) {
        gs.gp.bt = pk.w;
        gs.gp.bt_bytes = (unsigned)(pk.w_elems * (int64_t)sizeof(T));
        gs.gp.bt_ld = pk.D;
        gs.gp.bt_direct = 1;
        gs.gp.bd_xa = pk.xa; gs.gp.bd_xs = pk.xs; gs.gp.bd_ya = pk.ya; gs.gp.bd_ys = pk.ys;
        gs.gp.bd_fw = pk.fW; gs.gp.bd_tap_elems = pk.C * pk.D;
        return 0;                                    // nothing to pack
    }
    // fp32 fprop with at least three slabs (the slab kernel): w[fH][fW][C][D] is the [K][N] matrix itself, rows of D floats.
    // Whole n tiles only: with the slab's row in the scalar offset the range check does not see columns past the last row.
    // (tuning: gather_direct_b = 0 packs)
    if constexpr (sizeof(T) == 4) {
        if (!pk.transposed && vec && g.src_bytes != 0 && g.Kpad / BK >= min_slabs && pk.D % 4 == 0 && g.N % gather_bn(g.N) == 0 &&
            g.K == pk.K && pk.w_elems * 4 < ((int64_t)1 << 31) && (reinterpret_cast<uintptr_t>(pk.w) & 15) == 0 &&
            tuning().gather_direct_b != 0 && tuning().gather_kc == -1 && tuning().gather_bkn != 0) {
            gs.gp.bt = pk.w;
            gs.gp.bt_bytes = (unsigned)(pk.w_elems * 4);
            gs.gp.bt_ld = pk.D;
            gs.gp.bt_kn = gs.kn_part ? 2 : 1;
            gs.gp.bd_xa = pk.xa; gs.gp.bd_ya = pk.ya; gs.gp.bd_fw = pk.fW;
            return 0;
        }
    }
    return pk.Npad * pk.Kpad;
}

// (gather_res9_bf16.hip)
void launch_halo_res9_bf16(const GatherParams& p, const PackParams& pk, int mtiles, unsigned grid, hipStream_t stream);

template <typename T>
static int run_gather(GatherSetup& gs, char* ws, int64_t ws_off, bool vec) {
    Context& c = ctx();
    fill_gather<T>(gs, ws, ws_off);
    if constexpr (sizeof(T) == 2) {
        // the kernel that keeps the whole filter in LDS reads it from w itself
        GatherParams hp = gs.gp;
        int mtiles = 0;
        const bool dma = vec && hp.src_bytes != 0 && gs.pp.w_elems * 2 < ((int64_t)1 << 31) && gs.pp.N % 2 == 0;
        if (gs.nsplit == 1 && hp.M > 0 && plan_halo_res(hp, dma, c.prop.multiProcessorCount, &mtiles)) {
            const dim3 rgrid((unsigned)std::min(mtiles, c.prop.multiProcessorCount));
            // 3 x 3 taps onto rows stored one after the other: the filter lives in registers (tuning: gather_res = 2 keeps
            // it in LDS)
            if (hp.Th == 3 && hp.Tw == 3 && hp.dense_out && run_stores(hp) && tuning().gather_res != 2) {
                launch_halo_res9_bf16(hp, gs.pp, mtiles, rgrid.x, c.stream);
                AETH_LAUNCH_CHECK();
                return AETH_OK;
            }
            // tiles stored as runs of 256 contiguous bytes per pixel (tuning: gather_runs = 0 keeps the 16-byte pieces)
            if (run_stores(hp))
                hipLaunchKernelGGL(gather_halo_res_bf16<true>, rgrid, dim3(kResThreads), 0, c.stream, hp, gs.pp, mtiles);
            else
                hipLaunchKernelGGL(gather_halo_res_bf16<false>, rgrid, dim3(kResThreads), 0, c.stream, hp, gs.pp, mtiles);
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    const int total = choose_b_operand<T>(gs, vec);
    if (total > 0) {
        hipLaunchKernelGGL(pack_filter<T>, dim3(cdiv(total, 256)), dim3(256), 0, c.stream, gs.pp);
        AETH_LAUNCH_CHECK();
    }
    if (gs.gp.M > 0 && gs.gp.N > 0) {
        float* real_out = gs.gp.out;
        if (gs.nsplit > 1) gs.gp.out = reinterpret_cast<float*>(ws + ws_off + round_up(gs.bt_bytes, 256));
        const int held_before = pair_ctl().dgrad_kind;
        launch_gather<T>(gs.gp, vec, c.prop.multiProcessorCount, c.stream);
        AETH_LAUNCH_CHECK();
        if (pair_ctl().dgrad_kind != held_before) {            // the launch is held for a pair: so is the sum of its splits
            HeldSum& hs = pair_ctl().dgrad_sum;
            hs = HeldSum();
            if (gs.nsplit > 1) {
                hs.on = 1;
                hs.part = gs.gp.out; hs.out = real_out;
                hs.n_out = hs.n = hs.stride = gs.gp.M * gs.gp.N; hs.splits = gs.nsplit;
            }
            return AETH_OK;
        }
        if (gs.nsplit > 1) {
            const int n = gs.gp.M * gs.gp.N;
            const bool act = gs.act != nullptr && gs.act->out != nullptr && (reinterpret_cast<uintptr_t>(gs.act->out) & 15) == 0;
            hipLaunchKernelGGL(reduce_splits4, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream,
                               (const float*)gs.gp.out, real_out, (float*)nullptr, n, n, n, gs.nsplit, 0,
                               act ? gs.act->out : (float*)nullptr, act ? gs.act->alpha : 0.f);
            AETH_LAUNCH_CHECK();
            if (act) gs.act->done = true;
        }
    }
    return AETH_OK;
}

static inline void set_out_divs(GatherParams& g) {
    g.div_hw = FastDiv(g.Hg * g.Wg > 0 ? g.Hg * g.Wg : 1);
    g.div_w = FastDiv(g.Wg > 0 ? g.Wg : 1);
    g.div_c = FastDiv(g.Cs);
    g.div_tw = FastDiv(g.Tw > 0 ? g.Tw : 1);
}

// The direct dgrad of a 3x3 filter on 3 input channels (a network's first layer) joins a held wgrad launch the same way.
template <typename T, int FH, int FW, int C>
static inline bool hold_direct_for_pair(const DirectParams& dp, const dim3& grid) {
    if constexpr (sizeof(T) == 4 && FH == 3 && FW == 3 && C == 3) {
        PairCtl& pc = pair_ctl();
        if (!pair_accepts(kHeldDirect333)) return false;
        pc.dgrad_kind = kHeldDirect333;
        pc.dgrad_gx = grid.x;
        pc.dgrad_gy = 1;
        pc.dgrad_sum = HeldSum();
        held_direct_params() = dp;
        return true;
    }
    return false;
}

template <typename T>
static bool launch_direct(DirectParams& dp, bool dgrad, hipStream_t st) {
    if (tuning().direct == 0) return false;
    const int chunks = dp.D / 4;
    if (dp.C > 3 || dp.D % 4 != 0 || chunks < 4 || chunks > 64 || (chunks & (chunks - 1)) != 0) return false;
    if ((int64_t)dp.fH * dp.fW * dp.C * dp.D > kDirectMaxW || (int64_t)dp.M * chunks >= ((int64_t)1 << 31)) return false;
    if ((reinterpret_cast<uintptr_t>(dp.a) & 15) != 0 || (reinterpret_cast<uintptr_t>(dp.out) & 15) != 0 ||
        (dp.bias != nullptr && (reinterpret_cast<uintptr_t>(dp.bias) & 15) != 0))
        return false;
    // fprop: 8 output channels per lane where D allows, 16 for filters of 48 values and more per channel (128x32x32x3 ->
    // 32, 3x3: 10.0 us with 4 per lane, 8.7 with 8, 11.5 with 16; 64x64x64x3 -> 64, 5x5: 89, 66 and 63 us; tuning: direct = 2 keeps 4)
    const bool few = dgrad || tuning().direct == 2;
    const bool wide = !few && dp.D % 16 == 0 && dp.fH * dp.fW * dp.C >= 48;
    const bool wide8 = !few && !wide && dp.D % 8 == 0;
    // dgrad: two groups of 4 output channels per lane where that leaves a lane per input channel (tuning: direct = 2 keeps one)
    const bool dgrad2 = dgrad && chunks >= 8 && tuning().direct != 2;
    const int lanes = wide ? chunks / 4 : (wide8 || dgrad2) ? chunks / 2 : chunks;   // per pixel: a power of two
    dp.q_shift = 0;
    while ((1 << dp.q_shift) < lanes) ++dp.q_shift;
    const dim3 grid((unsigned)cdiv((int64_t)dp.M * lanes, kThreads));
    const size_t lds = (size_t)dp.fH * dp.fW * dp.C * dp.D * sizeof(float);
#define AETH_DIRECT_CASE(FH_, FW_, C_)                                                                              \
    if (dp.fH == FH_ && dp.fW == FW_ && dp.C == C_) {                                                               \
        if (dgrad2 && hold_direct_for_pair<T, FH_, FW_, C_>(dp, grid)) return true;                                   \
        if (dgrad2) hipLaunchKernelGGL((direct_dgrad_smallc<T, FH_, FW_, C_, 2>), grid, dim3(kThreads), lds, st, dp); \
        else if (dgrad) hipLaunchKernelGGL((direct_dgrad_smallc<T, FH_, FW_, C_>), grid, dim3(kThreads), lds, st, dp); \
        else if (wide) hipLaunchKernelGGL((direct_fprop_smallc<T, FH_, FW_, C_, 16>), grid, dim3(kThreads), lds, st, dp); \
        else if (wide8) hipLaunchKernelGGL((direct_fprop_smallc<T, FH_, FW_, C_, 8>), grid, dim3(kThreads), lds, st, dp); \
        else hipLaunchKernelGGL((direct_fprop_smallc<T, FH_, FW_, C_>), grid, dim3(kThreads), lds, st, dp);         \
        return true;                                                                                                \
    }
    AETH_DIRECT_CASE(3, 3, 1)
    AETH_DIRECT_CASE(3, 3, 2)
    AETH_DIRECT_CASE(3, 3, 3)
    AETH_DIRECT_CASE(5, 5, 1)
    AETH_DIRECT_CASE(5, 5, 3)
#undef AETH_DIRECT_CASE
    return false;
}

// `fixed_scratch` (with its capacity) replaces the library's growing workspace: the call then
// allocates nothing and fails with AETH_E_INVALID when the packed filter and the split
// partials do not fit.
template <typename T>
int conv_fprop_impl(const char* fn, const T* x, const T* w, const float* bias, float* y,
                    int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW,
                    char* fixed_scratch = nullptr, int64_t fixed_capacity = 0, ActOut* act = nullptr) {
    int Ho, Wo;
    int rc = check_conv_dims(fn, S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    {   // a batch whose input or output reaches 2^31 bytes goes out in runs of whole samples (sample_runs.h)
        const int64_t xs = (int64_t)H * W * C, ys = (int64_t)Ho * Wo * D;
        const SampleRuns runs = plan_sample_runs(S, xs * (int64_t)sizeof(T), ys * 4);
        if (runs.runs > 1) {
            for (int s0 = 0; s0 < S; s0 += runs.per) {
                rc = conv_fprop_impl<T>(fn, x + s0 * xs, w, bias, y + s0 * ys, std::min(runs.per, S - s0), H, W, C, D, fH, fW,
                                        sH, sW, pH, pW, fixed_scratch, fixed_capacity);
                if (rc) return rc;
            }
            return AETH_OK;
        }
    }
    if constexpr (sizeof(T) == 4) {
        const int64_t M = (int64_t)S * H * W;
        if (narrow_shape(D, fH, fW, sH, sW, pH, pW) && M > 0 && M * 64 < ((int64_t)1 << 31) && C <= 16384) {
            NarrowParams np;
            np.a = x; np.b = w; np.bias = bias; np.out = y; np.out2 = nullptr;
            np.M = (int)M; np.K = C; np.N = D;
            hipLaunchKernelGGL(narrow_fprop, dim3((unsigned)cdiv(M * 64, kThreads)), dim3(kThreads), 0, ctx().stream, np);
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    if (C <= 3) {
        DirectParams dp;
        dp.a = x; dp.w = w; dp.bias = bias; dp.out = y;
        dp.S = S; dp.H = H; dp.W = W; dp.C = C; dp.Ho = Ho; dp.Wo = Wo; dp.D = D;
        dp.fH = fH; dp.fW = fW; dp.sH = sH; dp.sW = sW; dp.pH = pH; dp.pW = pW;
        dp.M = S * Ho * Wo;
        dp.div_hw = FastDiv(Ho * Wo);
        dp.div_w = FastDiv(Wo);
        if (launch_direct<T>(dp, false, ctx().stream)) {
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    constexpr int BK = Elem<T>::BK;
    GatherSetup gs;
    GatherParams& g = gs.gp;
    g.src = x; g.bias = bias; g.out = y;
    g.S = S; g.Hs = H; g.Ws = W; g.Cs = C;
    g.Hg = Ho; g.Wg = Wo; g.M = S * Ho * Wo; g.N = D; g.K = fH * fW * C;
    g.Kpad = (int)round_up(g.K, BK);
    g.Tw = fW; g.sh = sH; g.sw = sW; g.rh0 = -pH; g.rw0 = -pW;
    g.Hof = Ho; g.Wof = Wo; g.oh0 = 0; g.ow0 = 0; g.ohs = 1; g.ows = 1; g.dense_out = 1;
    set_out_divs(g);
    PackParams& pk = gs.pp;
    pk.w = w; pk.fW = fW; pk.C = C; pk.D = D; pk.Tw = fW; pk.Ck = C; pk.w_elems = (int64_t)fH * fW * C * D;
    pk.xa = 0; pk.xs = 1; pk.ya = 0; pk.ys = 1; pk.transposed = 0;
    pk.N = D; pk.K = g.K; pk.Npad = (int)round_up(D, 64); pk.Kpad = g.Kpad;
    gs.bt_bytes = (int64_t)pk.Npad * pk.Kpad * sizeof(T);
    g.split_slabs = 0;
    gs.act = act;
    plan_split<T>(gs, C % Elem<T>::CE == 0, ctx().prop.multiProcessorCount);
    if constexpr (sizeof(T) == 4) {
        // A padded fprop at unit stride that is large enough for the 128 x 64 slab kernel (or tuning: gather_border = 1) is cut
        // into the runs of output rows and columns that see the same taps inside x (interior, edges, corners: nine parts for
        // 3x3 "same"), each a problem with only those taps, all in one grid: no tile multiplies a tap that lies in the padding.
        // Taken from 2 % of the taps on (56x56 images: 2.4 %); the filter is read in place by every part.
        const int v = tuning().gather_border;
        const int cus = ctx().prop.multiProcessorCount;
        const bool large = gs.nsplit == 1 && gather_bn(D) == 64 && g.M > 0 && gather_bm(g.M, D, cus, true) == 128;
        if (sH == 1 && sW == 1 && (pH > 0 || pW > 0) && fixed_scratch == nullptr && act == nullptr && v != 0 &&
            tuning().gather_merge != 0 && C % BK == 0 && (large || v > 0)) {
            const FpropPlan plan = plan_fprop_parts(H, W, Ho, Wo, fH, fW, pH, pW);
            const size_t nparts = plan.parts.size();
            if (nparts >= 2 && nparts <= (size_t)kMaxHeldClasses && (v > 0 || plan.taps_parts * 100 <= plan.taps_whole * 98)) {
                std::vector<GatherSetup> parts;
                int64_t total = 0;
                uniform_class_tiles() = true;
                for (const FpropPart& part : plan.parts) {
                    GatherSetup ps = gs;
                    GatherParams& q = ps.gp;
                    q.Hg = part.Hg; q.Wg = part.Wg; q.M = S * q.Hg * q.Wg;
                    q.K = part.Th * part.Tw * C;
                    q.Kpad = (int)round_up(q.K, BK);
                    q.Tw = part.Tw; q.rh0 = part.rh0; q.rw0 = part.rw0;
                    q.oh0 = part.oh0; q.ow0 = part.ow0; q.dense_out = 0;
                    set_out_divs(q);
                    PackParams& pq = ps.pp;
                    pq.Tw = part.Tw > 0 ? part.Tw : 1; pq.xa = part.xa; pq.ya = part.ya; pq.K = q.K; pq.Kpad = q.Kpad;
                    ps.bt_bytes = (int64_t)pq.Npad * pq.Kpad * sizeof(T);
                    ps.kn_part = true;
                    ps.nsplit = 1; ps.part_bytes = 0; q.split_slabs = 0;
                    total += round_up(ps.bt_bytes, 256);
                    parts.push_back(ps);
                }
                void* ws;
                rc = workspace(total > 0 ? total : 256, &ws);
                if (rc) {
                    uniform_class_tiles() = false;
                    return rc;
                }
                class_hold().count = 0;
                class_hold().armed = true;
                int64_t off = 0;
                for (GatherSetup& ps : parts) {
                    rc = run_gather<T>(ps, (char*)ws, off, true);
                    if (rc) break;
                    off += round_up(ps.bt_bytes, 256);
                }
                uniform_class_tiles() = false;
                flush_classes((int)parts.size(), ctx().stream);
                if (rc == AETH_OK) AETH_LAUNCH_CHECK();
                return rc;
            }
        }
    }
    void* ws;
    const int64_t need = round_up(gs.bt_bytes, 256) + gs.part_bytes;
    if (fixed_scratch != nullptr) {
        if (need > fixed_capacity)
            return fail(AETH_E_INVALID, "%s: needs %lld bytes of scratch, this entry point holds %lld", fn,
                        (long long)need, (long long)fixed_capacity);
        ws = fixed_scratch;
    } else {
        rc = workspace(need, &ws);
        if (rc) return rc;
    }
    return run_gather<T>(gs, (char*)ws, 0, C % Elem<T>::CE == 0);
}

// dgrad: for input row i the contributing taps are x with (i + pH - x) % sH == 0 and
// 0 <= (i + pH - x)/sH < Ho.  Rows are split by a = i % sH; inside a class the taps
// are x_t = xmax - sH*t (xmax = largest x < fH with x == (a+pH) mod sH), and the
// source row for class-row i' (i = a + sH*i') and tap t is i' + (a + pH - xmax)/sH + t:
// a unit-stride gather over dy with Th = number of such taps.
template <typename T>
int conv_dgrad_impl(const char* fn, const T* dy, const T* w, float* dx,
                    int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    int Ho, Wo;
    int rc = check_conv_dims(fn, S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    {   // runs of whole samples for a dy or dx of 2^31 bytes and more (sample_runs.h)
        const int64_t xs = (int64_t)H * W * C, ys = (int64_t)Ho * Wo * D;
        const SampleRuns runs = plan_sample_runs(S, ys * (int64_t)sizeof(T), xs * 4);
        if (runs.runs > 1) {
            for (int s0 = 0; s0 < S; s0 += runs.per) {
                rc = conv_dgrad_impl<T>(fn, dy + s0 * ys, w, dx + s0 * xs, std::min(runs.per, S - s0), H, W, C, D, fH, fW, sH,
                                        sW, pH, pW);
                if (rc) return rc;
            }
            return AETH_OK;
        }
    }
    constexpr int BK = Elem<T>::BK;
    const int nclass = sH * sW;
    if (nclass > 64) return fail(AETH_E_INVALID, "%s: stride too large", fn);
    pair_ctl().dgrad_ok = nclass == 1;       // unit stride: one class, one launch, no strips of zeros
    if constexpr (sizeof(T) == 4) {
        const int64_t M = (int64_t)S * H * W;
        if (narrow_shape(D, fH, fW, sH, sW, pH, pW) && M > 0 && M * C < ((int64_t)1 << 31)) {
            NarrowParams np;
            np.a = dy; np.b = w; np.bias = nullptr; np.out = dx; np.out2 = nullptr;
            np.M = (int)M; np.K = C; np.N = D;
            hipLaunchKernelGGL(narrow_dgrad, dim3((unsigned)cdiv(M * C, kThreads)), dim3(kThreads), 0, ctx().stream, np, (unsigned)(M * C));
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    if (C <= 3) {
        DirectParams dp;
        dp.a = dy; dp.w = w; dp.bias = nullptr; dp.out = dx;
        dp.S = S; dp.H = H; dp.W = W; dp.C = C; dp.Ho = Ho; dp.Wo = Wo; dp.D = D;
        dp.fH = fH; dp.fW = fW; dp.sH = sH; dp.sW = sW; dp.pH = pH; dp.pW = pW;
        dp.M = S * H * W;
        dp.div_hw = FastDiv(H * W);
        dp.div_w = FastDiv(W);
        if (launch_direct<T>(dp, true, ctx().stream)) {
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    // Rows of dx beyond h_last and columns beyond w_last are reached by no output pixel (the largest
    // index a tap touches is (Ho - 1) sH + fH - 1 - pH): the classes' pixel grids stop there and one small
    // launch zeroes the strips, instead of multiplying rows of padding (tuning: gather_clip = 0 keeps the full grids).
    int h_lim = H, w_lim = W;
    if (tuning().gather_clip != 0) {
        h_lim = std::min(H, (Ho - 1) * sH + fH - pH);
        w_lim = std::min(W, (Wo - 1) * sW + fW - pW);
        if (h_lim < 1 || w_lim < 1) { h_lim = H; w_lim = W; }
    }
    std::vector<GatherSetup> sets;
    int64_t total_bytes = 0;
    // The problems of the dgrad (dgrad_parts.h); `borders`: the classes cut along their borders.
    int64_t taps_whole = 0, taps_inside = 0;                 // tap-pixels multiplied per sample without and with the cut
    auto build_sets = [&](int hl, int wl, bool borders = false) {
        sets.clear();
        total_bytes = 0;
        const DgradPlan plan = plan_dgrad_parts(H, W, Ho, Wo, fH, fW, sH, sW, pH, pW, hl, wl, borders);
        taps_whole = plan.taps_whole;
        taps_inside = plan.taps_parts;
        for (const DgradPart& part : plan.parts) {
            GatherSetup gs;
            GatherParams& g = gs.gp;
            g.src = dy; g.bias = nullptr; g.out = dx;
            g.S = S; g.Hs = Ho; g.Ws = Wo; g.Cs = D;
            g.Hg = part.Hg; g.Wg = part.Wg; g.M = S * part.Hg * part.Wg; g.N = C;
            g.K = part.Th * part.Tw * D;
            g.Kpad = (int)round_up(g.K, BK);
            g.Tw = part.Tw; g.sh = 1; g.sw = 1; g.rh0 = part.rh0; g.rw0 = part.rw0;
            g.Hof = H; g.Wof = W; g.oh0 = part.oh0; g.ow0 = part.ow0; g.ohs = sH; g.ows = sW;
            g.dense_out = (nclass == 1 && !part.cut);
            set_out_divs(g);
            PackParams& pk = gs.pp;
            pk.w = w; pk.fW = fW; pk.C = C; pk.D = D; pk.Tw = part.Tw > 0 ? part.Tw : 1; pk.Ck = D; pk.w_elems = (int64_t)fH * fW * C * D;
            pk.xa = part.xa; pk.xs = -sH; pk.ya = part.ya; pk.ys = -sW; pk.transposed = 1;
            pk.N = C; pk.K = g.K; pk.Npad = (int)round_up(C, 64); pk.Kpad = g.Kpad;
            gs.bt_bytes = round_up((int64_t)pk.Npad * pk.Kpad * sizeof(T), 256);
            g.split_slabs = 0;
            plan_split<T>(gs, D % Elem<T>::CE == 0, ctx().prop.multiProcessorCount);
            total_bytes += gs.bt_bytes + gs.part_bytes;
            sets.push_back(gs);
        }
    };
    // bf16, 2 or 4 classes with the same pixel grid, each of them a problem for gather_halo_bf16 with the same
    // tiles: one launch for all classes (tuning: gather_merge = 0 keeps one launch per class).  The full grids
    // are used, so that they are equal; the classes then write the zeros of the unreachable rows themselves.
    if constexpr (sizeof(T) == 2) {
        if (nclass > 1 && nclass <= kMaxClasses && H % sH == 0 && W % sW == 0 && tuning().gather_merge != 0) {
            build_sets(H, W);
            void* ws = nullptr;
            bool ok = (int)sets.size() == nclass;
            if (ok) {
                rc = workspace(total_bytes > 0 ? total_bytes : 256, &ws);
                if (rc) return rc;
            }
            const bool vec = D % Elem<T>::CE == 0;
            const int cus = ctx().prop.multiProcessorCount;
            GatherClasses gc;
            gc.ncls = nclass;
            int mtiles = 0, stages = 4;
            std::vector<int> pack(sets.size(), 0);
            int64_t off = 0;
            for (size_t i = 0; ok && i < sets.size(); ++i) {
                GatherSetup& gs = sets[i];
                ok = gs.nsplit == 1 && gs.gp.M > 0 && gs.gp.N > 0 && gs.gp.K > 0;
                if (!ok) break;
                fill_gather<T>(gs, (char*)ws, off);
                off += gs.bt_bytes + gs.part_bytes;
                GatherParams probe = gs.gp;
                int mt_res = 0;
                const bool dma_res = vec && probe.src_bytes != 0 && gs.pp.w_elems * 2 < ((int64_t)1 << 31) && gs.pp.N % 2 == 0;
                if (plan_halo_res(probe, dma_res, cus, &mt_res)) { ok = false; break; }   // that class has a faster kernel of its own
                pack[i] = choose_b_operand<T>(gs, vec, 1);
                const bool dma = vec && gs.gp.src_bytes != 0 && gs.gp.bt_bytes != 0;
                int mt = 0, st = 0;
                ok = plan_halo(gs.gp, dma, &mt, &st, 1) && (i == 0 || (mt == mtiles && gs.gp.halo_tiles == sets[0].gp.halo_tiles));
                mtiles = mt;
                stages = std::min(stages, st);
                gc.cls[i] = gs.gp;
            }
            if (ok) {
                for (size_t i = 0; i < sets.size(); ++i)
                    if (pack[i] > 0) {
                        hipLaunchKernelGGL(pack_filter<T>, dim3(cdiv(pack[i], 256)), dim3(256), 0, ctx().stream, sets[i].pp);
                        AETH_LAUNCH_CHECK();
                    }
                // two classes per workgroup from one halo, where all classes read the filter in place (tuning: gather_pairs = 0 never)
                if (tuning().gather_pairs != 0) {
                    bool direct = true;
                    for (const GatherSetup& gs : sets) direct = direct && gs.gp.bt_direct != 0;
                    GatherClasses pc;
                    int64_t pmt = 0, longest = 0;
                    if (direct && plan_class_pairs(sets, pc, kHaloBM, kHaloSlotsMax, &pmt, &longest)) {
                        const dim3 pgrid((unsigned)(pmt * (nclass / 2) * cdiv(C, 64)));
                        const bool nt = run_stores(pc.cls[0]);   // (the kernel stores whole lines either way; the hint only for outputs that stream)
                        if (longest <= halo_slots(4) && nt) hipLaunchKernelGGL((gather_halo_pairs_bf16<4, true>), pgrid, dim3(kThreads), 0, ctx().stream, pc);
                        else if (longest <= halo_slots(4)) hipLaunchKernelGGL((gather_halo_pairs_bf16<4, false>), pgrid, dim3(kThreads), 0, ctx().stream, pc);
                        else if (nt) hipLaunchKernelGGL((gather_halo_pairs_bf16<3, true>), pgrid, dim3(kThreads), 0, ctx().stream, pc);
                        else hipLaunchKernelGGL((gather_halo_pairs_bf16<3, false>), pgrid, dim3(kThreads), 0, ctx().stream, pc);
                        AETH_LAUNCH_CHECK();
                        return AETH_OK;
                    }
                }
                const dim3 grid((unsigned)((int64_t)mtiles * nclass * cdiv(C, 64)));
                // a dx that the descriptor covers: tiles go out as whole lines (0.197 against 0.213 ms on the stride-2 layer)
                const bool lines = run_stores(sets[0].gp);
                if (stages == 4 && lines) hipLaunchKernelGGL((gather_halo_classes_bf16<4, true>), grid, dim3(kThreads), 0, ctx().stream, gc);
                else if (stages == 4) hipLaunchKernelGGL((gather_halo_classes_bf16<4, false>), grid, dim3(kThreads), 0, ctx().stream, gc);
                else if (lines) hipLaunchKernelGGL((gather_halo_classes_bf16<3, true>), grid, dim3(kThreads), 0, ctx().stream, gc);
                else hipLaunchKernelGGL((gather_halo_classes_bf16<3, false>), grid, dim3(kThreads), 0, ctx().stream, gc);
                AETH_LAUNCH_CHECK();
                return AETH_OK;
            }
        }
    }
    build_sets(h_lim, w_lim);
    // fp32: where every class is large enough for the 128 x 64 slab kernel (or tuning: gather_border = 1), the classes are cut
    // along their borders into parts that see the same taps inside dy, all of them on 128-row tiles, if that takes at least 3 %
    // off the taps multiplied (3x3 "same" at unit stride: 4.7 % on 28x28 images, 2.4 % on 56x56, where the cut measured 0.432 ms
    // against 0.438; the stride-2 28x28 layer: 10.5 %) and leaves at most kMaxHeldClasses problems (tuning: gather_border = 0 never).  The problems of a
    // strided or cut dgrad that the 128 x 64 slab kernel takes are collected and go out in shared grids (tuning: gather_merge = 0
    // keeps a launch each).
    bool collect = false;
    if constexpr (sizeof(T) == 4) {
        const int v = tuning().gather_border;
        const bool merge = tuning().gather_merge != 0 && (int)sets.size() <= kMaxHeldClasses;
        bool borders = false;
        if (merge && v != 0 && D % Elem<T>::BK == 0) {
            bool large = gather_bn(C) == 64;
            for (const GatherSetup& gs : sets)
                large = large && gs.nsplit == 1 && gs.gp.M > 0 && gather_bm(gs.gp.M, C, ctx().prop.multiProcessorCount, true) == 128;
            if (large || v > 0) {
                uniform_class_tiles() = true;
                build_sets(h_lim, w_lim, true);
                borders = sets.size() >= 2 && (int)sets.size() <= kMaxHeldClasses && (v > 0 || taps_inside * 100 <= taps_whole * 98);
                if (!borders) {
                    uniform_class_tiles() = false;
                    build_sets(h_lim, w_lim);
                }
            }
        }
        collect = merge && sets.size() >= 2 && (nclass >= 2 || borders);
    }
    void* ws;
    rc = workspace(total_bytes > 0 ? total_bytes : 256, &ws);
    if (rc) {
        uniform_class_tiles() = false;
        return rc;
    }
    int64_t off = 0;
    if (collect) {
        class_hold().count = 0;
        class_hold().armed = true;
    }
    for (auto& gs : sets) {
        rc = run_gather<T>(gs, (char*)ws, off, D % Elem<T>::CE == 0);
        if (rc) break;
        off += gs.bt_bytes + gs.part_bytes;
    }
    uniform_class_tiles() = false;
    if (collect) {
        flush_classes((int)sets.size(), ctx().stream);
        if (rc == AETH_OK) AETH_LAUNCH_CHECK();
    }
    if (rc) return rc;
    if (h_lim < H || w_lim < W) {
        ZeroStripParams zp;
        zp.dx = dx; zp.S = S; zp.H = H; zp.W = W; zp.C = C; zp.h0 = h_lim; zp.w0 = w_lim;
        zp.per_image = (H - h_lim) * W + h_lim * (W - w_lim);
        zp.vec = (C % 4 == 0 && (reinterpret_cast<uintptr_t>(dx) & 15) == 0) ? 1 : 0;
        zp.cgroups = zp.vec ? C / 4 : C;
        zp.div_cg = FastDiv(zp.cgroups);
        zp.div_pi = FastDiv(zp.per_image);
        zp.div_w = FastDiv(W);
        zp.div_wt = FastDiv(W - w_lim > 0 ? W - w_lim : 1);
        const int64_t n = (int64_t)S * zp.per_image * zp.cgroups;     // below 2^31: it is a part of dx
        hipLaunchKernelGGL(zero_strips, dim3((unsigned)cdiv(n, kThreads)), dim3(kThreads), 0, ctx().stream, zp, (unsigned)n);
        AETH_LAUNCH_CHECK();
    }
    return AETH_OK;
}


}  // namespace aeth
