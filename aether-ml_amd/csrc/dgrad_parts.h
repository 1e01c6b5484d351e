// The problems a dgrad is made of, and the parts of a padded fprop.
//
// dx[i][j] gets a contribution of filter tap (x, y) from dy[(i + pH - x) / sH][(j + pW - y) / sW] where the divisions are
// exact and the result lies inside dy.  Input rows are taken in classes a = i % sH (i = a + sH i'): a class sees only the
// taps x = xmax - sH t, t = 0 .. Th - 1, and tap t of class row i' reads dy row i' + off + t: a unit-stride gather.  Columns
// alike.  A class can further be cut into the runs of rows and columns that see the same taps INSIDE dy (first rows, interior,
// last rows), each part a problem with only those taps, so that no tile multiplies a tap that lies outside.
//
// Plain arithmetic without HIP calls, so that it can be checked on the host.
#pragma once

#include <stdint.h>
#include <algorithm>
#include <vector>

namespace aeth {

// Rows (or columns) [r0, r1) of a class and the taps [t0, t1) of the class that fall inside dy for all of them.
struct TapSpan {
    int r0, r1, t0, t1;
};

// Class row r reads dy row r + off + t under tap t (0 <= t < taps), which exists for 0 <= r + off + t < len.  Returns the
// maximal runs of rows with the same range of existing taps (`split`), or one span with all taps.
static inline std::vector<TapSpan> tap_spans(int rows, int off, int taps, int len, bool split) {
    std::vector<TapSpan> out;
    if (!split || taps <= 0) {
        out.push_back(TapSpan{0, rows, 0, taps > 0 ? taps : 0});
        return out;
    }
    for (int r = 0; r < rows; ++r) {
        const int lo = std::min(taps, std::max(0, -(r + off)));
        const int hi = std::max(lo, std::min(taps, len - (r + off)));
        if (!out.empty() && out.back().t0 == lo && out.back().t1 == hi) out.back().r1 = r + 1;
        else out.push_back(TapSpan{r, r + 1, lo, hi});
    }
    return out;
}

// One problem: part pixel (r, c), 0 <= r < Hg, 0 <= c < Wg, is dx pixel (oh0 + sH r, ow0 + sW c); its tap (t, u),
// 0 <= t < Th, 0 <= u < Tw, is filter tap (xa - sH t, ya - sW u) and reads dy pixel (r + rh0 + t, c + rw0 + u).
struct DgradPart {
    int Hg, Wg, Th, Tw;
    int rh0, rw0;
    int oh0, ow0;
    int xa, ya;
    bool cut;            // a part of a class (its pixels are not all pixels of the class)
};

struct DgradPlan {
    std::vector<DgradPart> parts;
    int64_t taps_whole = 0;     // tap-pixels per sample that the whole classes multiply
    int64_t taps_parts = 0;     // ... that the parts of this plan multiply
};

// hl, wl: rows / columns of dx from here on are reached by no output pixel and are not part of any problem
// (the caller fills them with zeros); H, W for "all".  borders: cut the classes.
static inline DgradPlan plan_dgrad_parts(int H, int W, int Ho, int Wo, int fH, int fW, int sH, int sW, int pH, int pW,
                                         int hl, int wl, bool borders) {
    DgradPlan plan;
    for (int a = 0; a < sH; ++a) {
        if (a >= H) continue;
        const int ra = (a + pH) % sH;
        const int Th = ra < fH ? (fH - 1 - ra) / sH + 1 : 0;
        const int xmax = ra + (Th - 1) * sH;
        const int offh = Th > 0 ? (a + pH - xmax) / sH : 0;   // exact: (a + pH - xmax) is a multiple of sH
        const int Hg = (std::min(H, std::max(hl, a + 1)) - a + sH - 1) / sH;      // class rows below hl (at least one)
        for (int b = 0; b < sW; ++b) {
            if (b >= W) continue;
            const int rb = (b + pW) % sW;
            const int Tw = rb < fW ? (fW - 1 - rb) / sW + 1 : 0;
            const int ymax = rb + (Tw - 1) * sW;
            const int offw = Tw > 0 ? (b + pW - ymax) / sW : 0;
            const int Wg = (std::min(W, std::max(wl, b + 1)) - b + sW - 1) / sW;
            plan.taps_whole += (int64_t)Hg * Wg * Th * Tw;
            const bool cut = borders && Th > 0 && Tw > 0;
            for (const TapSpan& rs : tap_spans(Hg, offh, Th, Ho, cut))
                for (const TapSpan& cs : tap_spans(Wg, offw, Tw, Wo, cut)) {
                    DgradPart p;
                    p.Hg = rs.r1 - rs.r0; p.Wg = cs.r1 - cs.r0;
                    p.Th = rs.t1 - rs.t0; p.Tw = cs.t1 - cs.t0;
                    // part row r is class row r + r0 and its tap t is class tap t + t0: dy row r + (off + r0 + t0) + t
                    p.rh0 = offh + rs.r0 + rs.t0; p.rw0 = offw + cs.r0 + cs.t0;
                    p.oh0 = a + sH * rs.r0; p.ow0 = b + sW * cs.r0;
                    p.xa = xmax - sH * rs.t0; p.ya = ymax - sW * cs.t0;
                    p.cut = cut;
                    plan.taps_parts += (int64_t)p.Hg * p.Wg * p.Th * p.Tw;
                    plan.parts.push_back(p);
                }
        }
    }
    return plan;
}

// A padded fprop at unit stride cut the same way: part pixel (r, c), 0 <= r < Hg, 0 <= c < Wg, is output pixel (oh0 + r,
// ow0 + c); its tap (t, u), 0 <= t < Th, 0 <= u < Tw, is filter tap (xa + t, ya + u) and reads x pixel (r + rh0 + t, c + rw0 + u),
// which lies inside x for every pixel and tap of the part.
struct FpropPart {
    int Hg, Wg, Th, Tw;
    int rh0, rw0;
    int oh0, ow0;
    int xa, ya;
};

struct FpropPlan {
    std::vector<FpropPart> parts;
    int64_t taps_whole = 0;     // tap-pixels per sample of the whole problem: Ho * Wo * fH * fW
    int64_t taps_parts = 0;     // ... that the parts multiply
};

static inline FpropPlan plan_fprop_parts(int H, int W, int Ho, int Wo, int fH, int fW, int pH, int pW) {
    FpropPlan plan;
    plan.taps_whole = (int64_t)Ho * Wo * fH * fW;
    // output row r reads x row r - pH + t under filter row t
    for (const TapSpan& rs : tap_spans(Ho, -pH, fH, H, true))
        for (const TapSpan& cs : tap_spans(Wo, -pW, fW, W, true)) {
            FpropPart p;
            p.Hg = rs.r1 - rs.r0; p.Wg = cs.r1 - cs.r0;
            p.Th = rs.t1 - rs.t0; p.Tw = cs.t1 - cs.t0;
            p.rh0 = -pH + rs.r0 + rs.t0; p.rw0 = -pW + cs.r0 + cs.t0;
            p.oh0 = rs.r0; p.ow0 = cs.r0;
            p.xa = rs.t0; p.ya = cs.t0;
            plan.taps_parts += (int64_t)p.Hg * p.Wg * p.Th * p.Tw;
            plan.parts.push_back(p);
        }
    return plan;
}

}  // namespace aeth
