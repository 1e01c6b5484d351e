// Host-only check of the dgrad geometry (aether-ml_amd/csrc/dgrad_parts.h) against the definition of the input gradient
// (Conv_Layer.backward, CNN_classes_cupy.py:136-153): dx[i][j] receives filter tap (x, y) from dy[h][w] exactly when
// h * sH + x == i + pH and w * sW + y == j + pW with (h, w) inside dy.  For every geometry the parts of the plan, whole
// classes and classes cut along their borders, must list every such (i, j, x, y) exactly once, read the dy pixel the
// definition names, and cover every dx pixel below (hl, wl) exactly once; a cut plan must list no tap outside dy at all.
// Prints one "ok <name>" line per geometry.
#include <stdio.h>
#include <map>
#include <set>
#include <tuple>

#include "dgrad_parts.h"

using namespace aeth;

static int check(const char* name, int H, int W, int fH, int fW, int sH, int sW, int pH, int pW, bool clip) {
    const int Ho = (H + 2 * pH - fH) / sH + 1, Wo = (W + 2 * pW - fW) / sW + 1;
    int hl = H, wl = W;
    if (clip) {
        hl = std::min(H, (Ho - 1) * sH + fH - pH);
        wl = std::min(W, (Wo - 1) * sW + fW - pW);
        if (hl < 1 || wl < 1) { hl = H; wl = W; }
    }
    // the definition: every (i, j, x, y) with its dy pixel
    std::map<std::tuple<int, int, int, int>, std::pair<int, int>> want;
    for (int h = 0; h < Ho; ++h)
        for (int w = 0; w < Wo; ++w)
            for (int x = 0; x < fH; ++x)
                for (int y = 0; y < fW; ++y) {
                    const int i = h * sH + x - pH, j = w * sW + y - pW;
                    if (i < 0 || i >= H || j < 0 || j >= W) continue;
                    want[std::make_tuple(i, j, x, y)] = std::make_pair(h, w);
                }
    for (int borders = 0; borders < 2; ++borders) {
        const DgradPlan plan = plan_dgrad_parts(H, W, Ho, Wo, fH, fW, sH, sW, pH, pW, hl, wl, borders != 0);
        std::set<std::tuple<int, int, int, int>> got;
        std::map<std::pair<int, int>, int> pixels;
        int64_t multiplied = 0;
        for (const DgradPart& p : plan.parts) {
            if (p.Hg < 1 || p.Wg < 1 || p.Th < 0 || p.Tw < 0) { printf("FAIL %s: empty part\n", name); return 1; }
            for (int r = 0; r < p.Hg; ++r)
                for (int c = 0; c < p.Wg; ++c) {
                    const int i = p.oh0 + sH * r, j = p.ow0 + sW * c;
                    if (i < 0 || i >= H || j < 0 || j >= W) { printf("FAIL %s: pixel (%d, %d) outside dx\n", name, i, j); return 1; }
                    ++pixels[std::make_pair(i, j)];
                    for (int t = 0; t < p.Th; ++t)
                        for (int u = 0; u < p.Tw; ++u) {
                            ++multiplied;
                            const int x = p.xa - sH * t, y = p.ya - sW * u;
                            const int h = r + p.rh0 + t, w = c + p.rw0 + u;
                            if (x < 0 || x >= fH || y < 0 || y >= fW) { printf("FAIL %s: tap (%d, %d) outside the filter\n", name, x, y); return 1; }
                            const bool inside = h >= 0 && h < Ho && w >= 0 && w < Wo;
                            if (!inside) {
                                if (p.cut) { printf("FAIL %s: a cut part multiplies a tap outside dy\n", name); return 1; }
                                continue;                    // a whole class multiplies it as zero
                            }
                            const auto key = std::make_tuple(i, j, x, y);
                            const auto it = want.find(key);
                            if (it == want.end() || it->second != std::make_pair(h, w)) {
                                printf("FAIL %s: (%d, %d) tap (%d, %d) reads dy (%d, %d)\n", name, i, j, x, y, h, w);
                                return 1;
                            }
                            if (!got.insert(key).second) { printf("FAIL %s: (%d, %d) tap (%d, %d) listed twice\n", name, i, j, x, y); return 1; }
                        }
                }
        }
        if (got.size() != want.size()) { printf("FAIL %s: %zu of %zu contributions listed (borders %d)\n", name, got.size(), want.size(), borders); return 1; }
        for (int i = 0; i < H; ++i)
            for (int j = 0; j < W; ++j) {
                const bool reached = i < hl && j < wl;
                const auto it = pixels.find(std::make_pair(i, j));
                const int n = it == pixels.end() ? 0 : it->second;
                // every class keeps at least one row and column, so a clipped pixel may still belong to a problem (it then gets zero)
                if ((reached && n != 1) || n > 1) { printf("FAIL %s: dx (%d, %d) written %d times (borders %d)\n", name, i, j, n, borders); return 1; }
            }
        if (multiplied != (borders ? plan.taps_parts : plan.taps_whole) || plan.taps_parts > plan.taps_whole) {
            printf("FAIL %s: tap counts %lld / %lld / %lld\n", name, (long long)multiplied, (long long)plan.taps_parts, (long long)plan.taps_whole);
            return 1;
        }
        if (borders && (int64_t)got.size() != plan.taps_parts) {
            // a class all of whose taps fall outside for some rows keeps those rows as parts without taps: nothing is multiplied there
            printf("FAIL %s: the cut plan multiplies %lld tap-pixels for %zu contributions\n", name, (long long)plan.taps_parts, got.size());
            return 1;
        }
    }
    printf("ok %s\n", name);
    return 0;
}

// The parts of a padded fprop at unit stride (Conv_Layer.forward, CNN_classes_cupy.py:92-116): y[r][c] takes filter tap (x, y) from
// the image pixel (r + x - pH, c + y - pW) when that lies inside the image.  The parts must list every such (r, c, x, y) exactly
// once with that pixel, no tap outside the image, and every output pixel exactly once.
static int check_fprop(const char* name, int H, int W, int fH, int fW, int pH, int pW) {
    const int Ho = H + 2 * pH - fH + 1, Wo = W + 2 * pW - fW + 1;
    const FpropPlan plan = plan_fprop_parts(H, W, Ho, Wo, fH, fW, pH, pW);
    std::set<std::tuple<int, int, int, int>> got;
    std::map<std::pair<int, int>, int> pixels;
    for (const FpropPart& p : plan.parts) {
        if (p.Hg < 1 || p.Wg < 1 || p.Th < 0 || p.Tw < 0) { printf("FAIL %s: empty part\n", name); return 1; }
        for (int r = 0; r < p.Hg; ++r)
            for (int c = 0; c < p.Wg; ++c) {
                const int orow = p.oh0 + r, ocol = p.ow0 + c;
                if (orow < 0 || orow >= Ho || ocol < 0 || ocol >= Wo) { printf("FAIL %s: pixel outside y\n", name); return 1; }
                ++pixels[std::make_pair(orow, ocol)];
                for (int t = 0; t < p.Th; ++t)
                    for (int u = 0; u < p.Tw; ++u) {
                        const int x = p.xa + t, y = p.ya + u;
                        const int i = r + p.rh0 + t, j = c + p.rw0 + u;
                        if (x < 0 || x >= fH || y < 0 || y >= fW) { printf("FAIL %s: tap outside the filter\n", name); return 1; }
                        if (i < 0 || i >= H || j < 0 || j >= W) { printf("FAIL %s: a part multiplies a tap in the padding\n", name); return 1; }
                        if (i != orow + x - pH || j != ocol + y - pW) { printf("FAIL %s: (%d, %d) tap (%d, %d) reads x (%d, %d)\n", name, orow, ocol, x, y, i, j); return 1; }
                        if (!got.insert(std::make_tuple(orow, ocol, x, y)).second) { printf("FAIL %s: listed twice\n", name); return 1; }
                    }
            }
    }
    int64_t want = 0;
    for (int r = 0; r < Ho; ++r)
        for (int c = 0; c < Wo; ++c) {
            if (pixels[std::make_pair(r, c)] != 1) { printf("FAIL %s: y (%d, %d) written %d times\n", name, r, c, pixels[std::make_pair(r, c)]); return 1; }
            for (int x = 0; x < fH; ++x)
                for (int y = 0; y < fW; ++y) {
                    const int i = r + x - pH, j = c + y - pW;
                    if (i >= 0 && i < H && j >= 0 && j < W) ++want;
                }
        }
    if ((int64_t)got.size() != want || plan.taps_parts != want || plan.taps_whole != (int64_t)Ho * Wo * fH * fW) {
        printf("FAIL %s: %zu contributions listed, %lld exist\n", name, got.size(), (long long)want);
        return 1;
    }
    printf("ok %s\n", name);
    return 0;
}

int main() {
    int bad = 0;
    bad += check_fprop("fprop_same_56x56_3x3", 56, 56, 3, 3, 1, 1);                   // the headline layer: nine parts
    bad += check_fprop("fprop_same_12x10_5x3", 12, 10, 5, 3, 2, 1);
    bad += check_fprop("fprop_same_9x9_7x7", 9, 9, 7, 7, 3, 3);
    bad += check_fprop("fprop_valid_12x12_3x3", 12, 12, 3, 3, 0, 0);                  // one part
    bad += check_fprop("fprop_pad3_6x6_3x3", 6, 6, 3, 3, 3, 3);                       // more padding than the filter needs: rows without taps
    bad += check_fprop("fprop_rows_only_8x20_3x1", 8, 20, 3, 1, 1, 0);
    bad += check("stride2_valid_28x28_3x3", 28, 28, 3, 3, 2, 2, 0, 0, true);        // the benchmark layer: 16 parts, a clipped row and column
    bad += check("stride2_same_28x28_3x3", 28, 28, 3, 3, 2, 2, 1, 1, true);
    bad += check("unit_stride_same_56x56_3x3", 56, 56, 3, 3, 1, 1, 1, 1, true);     // 9 parts
    bad += check("unit_stride_valid_12x12_3x3", 12, 12, 3, 3, 1, 1, 0, 0, true);
    bad += check("stride2_same_17x15_5x5", 17, 15, 5, 5, 2, 2, 2, 2, true);
    bad += check("stride_1x2_same_12x16_3x3", 12, 16, 3, 3, 1, 2, 1, 1, true);
    bad += check("stride3_valid_14x13_2x2", 14, 13, 2, 2, 3, 3, 0, 0, true);        // filter smaller than the stride: classes without taps
    bad += check("stride3_valid_14x13_2x2_full_grids", 14, 13, 2, 2, 3, 3, 0, 0, false);
    bad += check("stride2_same_9x9_7x7", 9, 9, 7, 7, 2, 2, 3, 3, true);
    bad += check("stride_1x4_valid_9x16_3x3", 9, 16, 3, 3, 1, 4, 0, 0, true);
    bad += check("stride3_valid_11x9_5x5", 11, 9, 5, 5, 3, 3, 0, 0, true);
    bad += check("stride2_pad3_10x10_3x3", 10, 10, 3, 3, 2, 2, 3, 3, true);         // more padding than the filter needs
    bad += check("one_pixel_1x1", 1, 1, 1, 1, 1, 1, 0, 0, true);
    bad += check("stride4_valid_5x5_5x5", 5, 5, 5, 5, 4, 4, 0, 0, true);            // one output pixel
    return bad ? 1 : 0;
}
