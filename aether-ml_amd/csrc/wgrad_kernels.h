// Device side of wgrad: the register-staged and LDS-direct split-M kernels and the two persistent
// kernels that keep the whole filter gradient in registers.
#pragma once
#include "conv_common.h"

namespace aeth {

// ------------------------------------------------------------------------------
// wgrad: out[k][n] = sum_m A[m][k] * dy[m][n], k = (fx*fW + fy)*C + c
// Workgroup tile 128 (k) x 64 (n); each of the 4 waves owns 32 k-rows x 64 n.
// The M range of a workgroup (blockIdx.z) is walked in slabs of 32 rows which are
// kept in LDS as fp32 (bf16 inputs are widened on the way in: products of bf16
// values are exact in fp32, so this is bf16-in / fp32-accumulate arithmetic on
// v_mfma_f32_32x32x2_f32).  The partial tile of split z goes to
// out + z*(K*D + D); the trailing D floats of each split hold the dbias partial.
// ------------------------------------------------------------------------------
struct WgradParams {
    const void* x;       // [S,H,W,C] of T
    const void* dy;      // [S,Ho,Wo,D] = [M,D] of T
    float* out;          // [splits][K*D + D]
    float* db_out;       // one split only: dbias itself (out is then dw itself and no reduction follows); else null
    int want_dbias;
    int S, H, W, C, Ho, Wo, D;
    int M, K;
    int fW, sH, sW, pH, pW;
    int m_per_split;     // multiple of 32
    int kt, nt;          // output tiles along k and n
    int cw;              // fp32 LDS-direct kernel: floats of k per lane of an operand read (4, 2 or 1)
    // swap (fp32 LDS-direct kernel, 1x1 filters): the caller handed over dy as `x` and x as `dy`, the result is the
    // transpose of dw, and dbias is the column sums of the `x` operand: every k tile adds up its own columns.
    int swap;
    int db_len;          // floats of dbias behind the K*D floats of a split's partial block (D, or K when swapped)
    unsigned x_bytes, dy_bytes;   // extents for the buffer descriptors (LDS-direct kernel)
    // moving 32 rows of m ahead: 32 = qs*Ho*Wo + qh*Wo + qw.  step_c = qw*sW, step_r = qh*sH;
    // byte offset += inc0 (+ inc1 when the column wraps) (+ inc2 when the row wraps)
    int step_c, step_r, inc0, inc1, inc2;
    FastDiv div_howo, div_wo, div_c, div_fw;
};

constexpr int kWgBK = 128;   // k rows per workgroup
constexpr int kWgBN = 64;
constexpr int kWgBR = 32;    // m rows per slab
constexpr int kWgLDA = kWgBK + 32;
constexpr int kWgLDY = kWgBN + 32;

template <typename T, int VECA, int VECY>
__global__ __launch_bounds__(kThreads) void wgrad_gemm(const WgradParams p) {
    constexpr int CE = Elem<T>::CE;
    constexpr int A_CPR = kWgBK / CE;              // A chunks per slab row
    constexpr int A_RPP = kThreads / A_CPR;        // rows covered per pass
    constexpr int A_PASSES = kWgBR / A_RPP;
    constexpr int Y_CPR = kWgBN / CE;
    constexpr int Y_RPP = kThreads / Y_CPR;
    constexpr int Y_PASSES = kWgBR / Y_RPP;
    constexpr int NE = VECA == CE ? 1 : CE;        // tap decodes per thread

    __shared__ float lds_a[kWgBR * kWgLDA];
    __shared__ float lds_y[kWgBR * kWgLDY];
    __shared__ float lds_db[Y_RPP * 64];

    const T* __restrict__ xs = static_cast<const T*>(p.x);
    const T* __restrict__ dys = static_cast<const T*>(p.dy);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;

    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int tiles = p.kt * p.nt;
    const int split = lid / tiles;
    const int tile = lid - split * tiles;
    const int ktile = tile % p.kt;
    const int kt0 = ktile * kWgBK;
    const int n0 = (tile / p.kt) * kWgBN;
    const int m_begin = split * p.m_per_split;
    int m_end = m_begin + p.m_per_split;
    if (m_end > p.M) m_end = p.M;

    // A chunk owned by this thread: CE consecutive k starting at kt0 + CE*ka
    const int ka = tid % A_CPR;
    const int ra0 = tid / A_CPR;
    int a_tap_off[NE];
    int a_fx[NE];
    int a_fy[NE];
    bool a_kok[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e) {
        int kk = kt0 + CE * ka + e;
        unsigned tap, c, fx, fy;
        p.div_c.divmod((unsigned)kk, tap, c);
        p.div_fw.divmod(tap, fx, fy);
        a_kok[e] = kk < p.K;
        a_fx[e] = (int)fx - p.pH;
        a_fy[e] = (int)fy - p.pW;
        a_tap_off[e] = (a_fx[e] * p.W + a_fy[e]) * p.C + (int)c;
    }
    // dy chunk: CE consecutive n starting at n0 + CE*ky
    const int ky = tid % Y_CPR;
    const int ry0 = tid / Y_CPR;
    const bool do_db = p.want_dbias && (ktile == 0);

    float areg[A_PASSES][CE];
    float yreg[Y_PASSES][CE];
    float dbsum[CE];
#pragma unroll
    for (int e = 0; e < CE; ++e) dbsum[e] = 0.f;

    auto load_slab = [&](int mb) {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i) {
            int m = mb + ra0 + A_RPP * i;
            T raw[CE];
#pragma unroll
            for (int e = 0; e < CE; ++e) raw[e] = (T)0;
            if (m < m_end) {
                unsigned s, rem, ho, wo;
                p.div_howo.divmod((unsigned)m, s, rem);
                p.div_wo.divmod(rem, ho, wo);
                int r0 = (int)ho * p.sH;
                int c0 = (int)wo * p.sW;
                int pix = (((int)s * p.H + r0) * p.W + c0) * p.C;
                if (VECA == CE) {
                    bool ok = a_kok[0] && (unsigned)(r0 + a_fx[0]) < (unsigned)p.H &&
                              (unsigned)(c0 + a_fy[0]) < (unsigned)p.W;
                    if (ok) {
                        f4 v = *reinterpret_cast<const f4*>(xs + (pix + a_tap_off[0]));
                        __builtin_memcpy(raw, &v, 16);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < CE; ++e) {
                        const int ee = NE == 1 ? 0 : e;
                        bool ok = a_kok[ee] && (unsigned)(r0 + a_fx[ee]) < (unsigned)p.H &&
                                  (unsigned)(c0 + a_fy[ee]) < (unsigned)p.W;
                        if (ok) raw[e] = xs[pix + a_tap_off[ee]];
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < CE; ++e) areg[i][e] = Elem<T>::to_f32(raw[e]);
        }
#pragma unroll
        for (int i = 0; i < Y_PASSES; ++i) {
            int m = mb + ry0 + Y_RPP * i;
            T raw[CE];
#pragma unroll
            for (int e = 0; e < CE; ++e) raw[e] = (T)0;
            int n = n0 + CE * ky;
            if (m < m_end) {
                if (VECY == CE) {
                    if (n < p.D) {
                        f4 v = *reinterpret_cast<const f4*>(dys + ((size_t)m * p.D + n));
                        __builtin_memcpy(raw, &v, 16);
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < CE; ++e)
                        if (n + e < p.D) raw[e] = dys[(size_t)m * p.D + n + e];
                }
            }
#pragma unroll
            for (int e = 0; e < CE; ++e) yreg[i][e] = Elem<T>::to_f32(raw[e]);
        }
    };

    auto store_slab = [&]() {
#pragma unroll
        for (int i = 0; i < A_PASSES; ++i)
#pragma unroll
            for (int q = 0; q < CE / 4; ++q)
                *reinterpret_cast<f4*>(&lds_a[(ra0 + A_RPP * i) * kWgLDA + CE * ka + 4 * q]) =
                    f4{areg[i][4 * q], areg[i][4 * q + 1], areg[i][4 * q + 2], areg[i][4 * q + 3]};
#pragma unroll
        for (int i = 0; i < Y_PASSES; ++i) {
#pragma unroll
            for (int q = 0; q < CE / 4; ++q)
                *reinterpret_cast<f4*>(&lds_y[(ry0 + Y_RPP * i) * kWgLDY + CE * ky + 4 * q]) =
                    f4{yreg[i][4 * q], yreg[i][4 * q + 1], yreg[i][4 * q + 2], yreg[i][4 * q + 3]};
            if (do_db) {
#pragma unroll
                for (int e = 0; e < CE; ++e) dbsum[e] += yreg[i][e];
            }
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

    const size_t split_stride = (size_t)p.K * p.D + p.D;
    float* outp = p.out + (size_t)split * split_stride;
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
        // Y_RPP row lanes each hold a partial of the same CE columns: fixed-order sum
#pragma unroll
        for (int e = 0; e < CE; ++e) lds_db[ry0 * 64 + CE * ky + e] = dbsum[e];
        __syncthreads();
        if (tid < 64) {
            float s = 0.f;
#pragma unroll
            for (int r = 0; r < Y_RPP; ++r) s += lds_db[r * 64 + tid];
            if (n0 + tid < p.D) (p.db_out ? p.db_out : outp + (size_t)p.K * p.D)[n0 + tid] = s;
        }
    }
}

// ------------------------------------------------------------------------------
// wgrad, LDS-direct (fp32, C and D multiples of 4).  Output tile 128 k x 64 n per
// workgroup; the M range of a split is walked in slabs of 32 rows:
//   * x and dy slabs go straight into LDS (`buffer_load_dwordx4 ... lds`), two buffers,
//     one barrier per slab, operand reads of step t+1 issued before the MFMAs of step t;
//   * the x operand is read with ONE `ds_read_b128` per 4 MFMAs: lane i takes the 4
//     consecutive k values 4i..4i+3 of slab row m and MFMA q (q = 0..3) multiplies the
//     column k = 4i + q, i.e. accumulator q holds the output rows k == q (mod 4).  Which
//     rows an MFMA produces is free to choose, and this choice needs 2 LDS reads per
//     4 MFMAs where k-contiguous accumulator rows need 3 `ds_read_b32` per 2 (a
//     stand-alone loop: 132 against 118 TFLOP/s);
//   * the 4 waves are (n half) x (parity of the m pair): a wave owns all 128 k rows
//     of one 32-wide n half and every other pair of slab rows; the two parities
//     are added through LDS once, after the last slab;
//   * when all of K is at most 64 rows the kernel switches to `ds_read_b64` and two
//     accumulators (k = 2i + q);
//   * x rows are stored plainly (a 16-lane group reads 256 contiguous bytes); odd rows
//     of dy store their 32-float halves swapped, so the two half-waves of a
//     `ds_read_b32` (rows m and m+1) fall into different halves of the 64 banks;
//   * dbias fused: the workgroups of k tile 0 also add up the columns of every dy
//     slab they hold in LDS.
// ------------------------------------------------------------------------------
template <int CW, int BR = kWgBR>                        // BR rows of m per slab: 32, or 16 (CW == 6 only)
static __device__ __forceinline__ void wgrad_dma_body(const WgradParams& p, float* lds_a0, float* lds_a1, float* lds_y0,
                                                       float* lds_y1, const BlockId blk) {
    static_assert(BR == 32 || (BR == 16 && CW == 6), "slab heights");
    constexpr int RW = BR / 4;                           // slab rows a wave loads
    constexpr int YL = BR / 16;                          // dy loads per wave per slab (4 rows x 16 chunks each)
    // CW = 1: any channel count.  A lane loads ONE float per slab row (`buffer_load_dword ... lds`),
    // slab rows are 32 floats, the k tile is 32 wide and there is one accumulator.
    // CW = 6: a 192-wide k tile (K = 576 is 3 of them: no padded rows where 128-wide tiles
    // pad 10 %).  Accumulators 0..3 hold k = 4i + q of the first 128 columns, 4 and 5 hold
    // k = 128 + 2i + (q - 4) of the last 64 (one `ds_read_b128` and one `ds_read_b64`, both
    // aligned).  64 KB of LDS and 96 accumulator registers: 2 workgroups per CU, which a
    // stand-alone loop measured at 135 TFLOP/s against 132 for the 128-wide form at 3.
    constexpr int RS = CW == 1 ? 32 : (CW == 6 ? 192 : kWgBK);   // floats per x slab row in LDS
    constexpr int KSTEP = CW == 1 ? 1 : 4;               // k per lane of an x load
    constexpr int CPR = RS / KSTEP;                      // load lanes per slab row (32 or 48)
    constexpr int TKW = RS;                              // k tile width
    constexpr int XL = CPR * RW / 64;                    // x loads per wave per slab: RW rows x CPR lanes / 64
    constexpr int NA = CW == 6 ? 4 : CW;                 // accumulators fed by the first (wide) operand read
    typedef float fcw __attribute__((ext_vector_type(CW)));
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int nt = wave & 1;                             // n half of this wave
    const int mh = wave >> 1;                            // parity of the m pairs it multiplies

    const int lid = xcd_contiguous_id(blk.x, blk.gx);
    const int tiles = p.kt * p.nt;
    const int split = lid / tiles;
    const int tile = lid - split * tiles;
    const int ktile = tile % p.kt;
    const int kt0 = ktile * TKW;
    const int n0 = (tile / p.kt) * kWgBN;
    const int m_begin = split * p.m_per_split;
    int m_end = m_begin + p.m_per_split;
    if (m_end > p.M) m_end = p.M;
    const bool do_db = p.want_dbias && (ktile == 0) && !p.swap;
    const bool do_dba = CW == 4 && p.want_dbias && p.swap;     // (the 128-wide form is the one the host swaps operands for)

    // ---- x: a wave loads 8 slab rows with XL loads; lane l of load j is load lane 64 j + l ----
    //      of those rows: row (64 j + l) / CPR, chunk (64 j + l) % CPR
    // fp32 MFMA and ordinary vector (and scalar) instructions of a wave share its issue
    // slots, so the address work per load is kept to a handful of instructions:
    //  * lane l keeps the image position of slab row 8*wave + (l & 7) -- the 8 rows this
    //    wave loads -- and moves it by 32 rows per slab with adds and two carries
    //    (no division in the loop);
    //  * load i takes the rows 2i and 2i+1 of those 8 from their lanes with `ds_bpermute`;
    //  * the lane's own filter tap is tested against the row's position with the fields
    //    (row, column) packed in one register and guard bits catching both bounds.
    // Row state: rpos/cpos = position of tap (0,0) in the image + 64 (never negative),
    // off = byte offset of that pixel (wraps for padding positions; only used when valid).
    int st_r, st_c, st_off;
    {
        const int m = m_begin + RW * wave + (lane & (RW - 1));
        unsigned s_, rem, ho, wo;
        p.div_howo.divmod((unsigned)m, s_, rem);
        p.div_wo.divmod(rem, ho, wo);
        st_r = (int)ho * p.sH - p.pH;
        st_c = (int)wo * p.sW - p.pW;
        st_off = ((((int)s_ * p.H + st_r) * p.W + st_c) * p.C) * 4;
        st_r += 64;
        st_c += 64;
    }
    const int thr_c = p.Wo * p.sW - p.pW + 64, thr_r = p.Ho * p.sH - p.pH + 64;
    auto advance = [&]() {                               // m += BR
        st_c += p.step_c;
        const bool c1 = st_c >= thr_c;
        st_c -= c1 ? p.Wo * p.sW : 0;
        st_r += c1 ? p.step_r + p.sH : p.step_r;
        const bool c2 = st_r >= thr_r;
        st_r -= c2 ? p.Ho * p.sH : 0;
        st_off += c1 ? p.inc0 + p.inc1 : p.inc0;
        st_off += c2 ? p.inc2 : 0;
    };
    // per-lane tap constants, one set per load (with 32 lanes per row they coincide)
    unsigned tap_lo[XL], tap_hi[XL];                     // guard-bit constants, see test below
    int a_tap4[XL];
    int perm_idx[XL];                                    // byte index of the lane that tracks this load's row
#pragma unroll
    for (int j = 0; j < XL; ++j) {
        const int flat = 64 * j + lane;
        const int row = flat / CPR, chunk = flat % CPR;
        perm_idx[j] = row * 4;
        const int kk = kt0 + KSTEP * chunk;
        unsigned tap, c, fx, fy;
        p.div_c.divmod((unsigned)kk, tap, c);
        p.div_fw.divmod(tap, fx, fy);
        a_tap4[j] = (((int)fx * p.W + (int)fy) * p.C + (int)c) * 4;
        const unsigned tapc = (fx << 16) | fy;
        // t = rc + tapc has the fields (row + 64, column + 64) of the lane's tap.
        // lo = 0x803f803f - t : bit 15 of a field is set iff that coordinate is < 0
        // hi = t + (0x8000 - (H + 64), 0x8000 - (W + 64)) : set iff it is >= H (or W)
        tap_lo[j] = 0x803f803fu - tapc;
        tap_hi[j] = tapc + (((unsigned)(0x8000 - (p.H + 64)) << 16) | (unsigned)(0x8000 - (p.W + 64)));
        if (kk >= p.K) tap_lo[j] = 0xffffffffu;          // k past K: always out of range
    }

    // ---- dy: one wave-level load = 4 slab rows x 16 chunks; 2 loads per wave ------------
    // Rows past M lie beyond the descriptors' extents (and m_per_split is a multiple of
    // the slab height), so neither operand needs a test against m_end.
    const int y_row = lane >> 4;
    const int y_lc = (lane & 15) ^ ((y_row & 1) << 3);
    const int y_n = n0 + 4 * y_lc;
    const unsigned y_lane = ((unsigned)(y_row * p.D + y_n) * 4u) | ((unsigned)!(y_n < p.D) << 31);

    const __amdgpu_buffer_rsrc_t rsrc_x =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.x), 0, (int)p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_y =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.dy), 0, (int)p.dy_bytes, 0x00020000);

    // loads of the slab whose first row is mb; the row state must stand at mb.  The work
    // is cut in three so that a slab can spread it between its MFMA groups: a burst of
    // address arithmetic after the barrier keeps the wave off the matrix pipe, while the
    // same instructions issued behind an MFMA run in its shadow.
    unsigned perm_rc[XL];
    int perm_off[XL];
    // live == 0 (no next slab): rows read as (0, 0), which every tap sees as "above the image"
    auto fetch_rows = [&](int live) {                    // 8 LDS-crossbar permutes, no LDS memory
        const int rc = ((st_r << 16) | st_c) & live;
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            perm_rc[i] = (unsigned)__builtin_amdgcn_ds_bpermute(perm_idx[i], rc);
            perm_off[i] = __builtin_amdgcn_ds_bpermute(perm_idx[i], st_off);
        }
    };
    auto load_x = [&](int i, float* la) {
        const unsigned z = (tap_lo[i] - perm_rc[i]) | (perm_rc[i] + tap_hi[i]);
        const unsigned w = z | (z << 16);                // bit 31: row or column out of the image
        const unsigned voff = (w & 0x80000000u) | (unsigned)(perm_off[i] + a_tap4[i]);
        // the wave's RW rows are contiguous in LDS; load i fills the next 64 lanes' worth of them
        if constexpr (CW == 1)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr_t)(la + wave * RW * RS + i * 64), 4, (int)voff, 0, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr_t)(la + wave * RW * RS + i * 256), 16, (int)voff, 0, 0, 0);
    };
    auto load_y = [&](int i, int mb, float* ly, int live) {
        const int m = mb + (wave_u * YL + i) * 4;        // scalar
        const unsigned voff = y_lane + (live ? (unsigned)(m * p.D) * 4u : 0x80000000u);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_y, (lds_ptr_t)(ly + (wave * YL + i) * 256), 16, (int)voff, 0, 0, 0);
    };

    float dbsum = 0.f;
    const int db_col = tid & 63, db_rg = tid >> 6;
    auto add_columns = [&](const float* ly) {
#pragma unroll
        for (int j = 0; j < RW; ++j) dbsum += ly[(db_rg * RW + j) * kWgBN + (db_col ^ ((j & 1) << 5))];
    };
    // swapped operands: the column sums of the x slab (rows stored plainly, RS floats each); a thread owns 4
    // neighbouring columns of 4 rows
    f4 dbsum_a = {0.f, 0.f, 0.f, 0.f};
    auto add_columns_a = [&](const float* la) {
        if constexpr (CW == 4) {
#pragma unroll
            for (int j = 0; j < BR / 8; ++j) dbsum_a += *reinterpret_cast<const f4*>(la + ((tid >> 5) * (BR / 8) + j) * RS + 4 * (tid & 31));
        }
    };

    f16v acc[CW];
#pragma unroll
    for (int q = 0; q < CW; ++q)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[q][v] = 0.f;

    // operand addresses of m pair t' (slab rows 2*(2t'+mh) + lh); odd rows of dy have halves swapped
    const int row0 = 2 * mh + lh;                        // first slab row read; then +4 per step
    const int y_rd = nt * 32 + l32;                      // logical n; physical = y_rd ^ (lh << 5)
    // The MFMA takes dy as its A operand and x as B: accumulator q then holds
    // dW[k = kt0 + CW * (lane % 32) + q][n = 32 nt + 8 (v/4) + 4 (lane/32) + v%4], four
    // consecutive n per lane and v/4, which leave in 16-byte stores.
    typedef float fna __attribute__((ext_vector_type(NA)));
    typedef float f2v __attribute__((ext_vector_type(2)));
    auto slab = [&](int mb, const float* la, const float* ly, float* na, float* ny, bool has_next) {
        __builtin_amdgcn_s_waitcnt(0);                   // this wave's loads of the slab have landed
        __syncthreads();
        fna fa[2];
        f2v fa2[2];                                      // CW == 6: columns 128 + 2i, 128 + 2i + 1
        float fb[2];
        auto read_operands = [&](int row, int slot) {
            fa[slot] = *reinterpret_cast<const fna*>(la + row * RS + NA * l32);
            if constexpr (CW == 6) fa2[slot] = *reinterpret_cast<const f2v*>(la + row * RS + 128 + 2 * l32);
            fb[slot] = ly[row * kWgBN + (y_rd ^ (lh << 5))];
        };
        read_operands(row0, 0);
        // no branch in here: without a next slab the loads are issued with offsets past
        // the descriptors and fetch nothing
        const int live = has_next ? -1 : 0;
        advance();
        fetch_rows(live);
#pragma unroll
        for (int t = 0; t < BR / 4; ++t) {
            if (t + 1 < BR / 4) read_operands(row0 + 4 * t + 4, (t + 1) & 1);
            // one load per MFMA step: dy from step 0 (wide tiles) or 5 on, x from step 1 on
            constexpr int Y0 = (XL == 6 || BR == 16) ? 0 : 5;
            static_assert(XL <= BR / 4 - 1 && Y0 + YL <= BR / 4, "a slab's loads fit its steps");
            if (t >= 1 && t <= XL) load_x(t - 1, na);
            if (t >= Y0 && t < Y0 + YL) load_y(t - Y0, mb + BR, ny, live);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < NA; ++q)
                acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[t & 1], fa[t & 1][q], acc[q], 0, 0, 0);
            if constexpr (CW == 6) {
                acc[4] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[t & 1], fa2[t & 1][0], acc[4], 0, 0, 0);
                acc[5] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[t & 1], fa2[t & 1][1], acc[5], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (do_db) add_columns(ly);
        if (do_dba) add_columns_a(la);
    };

    if (m_begin < m_end) {
        fetch_rows(-1);
#pragma unroll
        for (int i = 0; i < XL; ++i) load_x(i, lds_a0);
#pragma unroll
        for (int i = 0; i < YL; ++i) load_y(i, m_begin, lds_y0, -1);
    }
    for (int mb = m_begin; mb < m_end; mb += 2 * BR) {
        slab(mb, lds_a0, lds_y0, lds_a1, lds_y1, mb + BR < m_end);
        if (mb + BR < m_end) slab(mb + BR, lds_a1, lds_y1, lds_a0, lds_y0, mb + 2 * BR < m_end);
    }

    // ---- add the two m parities: waves 2,3 hand their accumulators to waves 0,1 --------
    // through one x buffer per wave pair, QP accumulators (4 x 16 B x 64 lanes each) at a time
    constexpr int QP = (BR * RS * 4 >= CW * 4096) ? CW : CW / 2;
    static_assert(BR * RS * 4 >= QP * 4096 && CW % QP == 0, "accumulator exchange buffer");
    f4* xch = reinterpret_cast<f4*>(nt == 0 ? lds_a0 : lds_a1);
    const size_t split_stride = (size_t)p.K * p.D + p.db_len;
    float* outp = p.out + (size_t)split * split_stride;
    // one split's partial block is far below 2^31 bytes (K * D < 2^29 is checked by the host)
    const __amdgpu_buffer_rsrc_t rsrc_o =
        __builtin_amdgcn_make_buffer_rsrc(outp, 0, (int)((unsigned)p.K * (unsigned)p.D * 4u), 0x00020000);
    const int nb = n0 + nt * 32 + 4 * lh;
#pragma unroll
    for (int q0 = 0; q0 < CW; q0 += QP) {
        __syncthreads();                                 // slab buffers (or the pass before) are free now
        if (mh == 1) {
#pragma unroll
            for (int q = q0; q < q0 + QP; ++q)
#pragma unroll
                for (int g = 0; g < 4; ++g)
                    xch[((q - q0) * 4 + g) * 64 + lane] =
                        f4{acc[q][4 * g], acc[q][4 * g + 1], acc[q][4 * g + 2], acc[q][4 * g + 3]};
        }
        __syncthreads();
        if (mh == 0) {
#pragma unroll
            for (int q = q0; q < q0 + QP; ++q) {
                const int k = q < NA ? kt0 + NA * l32 + q : kt0 + 128 + 2 * l32 + (q - NA);   // rows past K fall outside the descriptor
                const unsigned base = (unsigned)(k * p.D + nb) * 4u;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    f4 v = xch[((q - q0) * 4 + g) * 64 + lane];
                    v[0] += acc[q][4 * g];
                    v[1] += acc[q][4 * g + 1];
                    v[2] += acc[q][4 * g + 2];
                    v[3] += acc[q][4 * g + 3];
                    const unsigned off = base | ((unsigned)!(nb + 8 * g < p.D) << 31);
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), rsrc_o, (int)off, 8 * g * 4, 0);
                }
            }
        }
    }
    if (do_db) {
        __syncthreads();
        lds_y0[db_rg * 64 + db_col] = dbsum;
        __syncthreads();
        if (tid < 64 && n0 + tid < p.D)
            (p.db_out ? p.db_out : outp + (size_t)p.K * p.D)[n0 + tid] = (lds_y0[tid] + lds_y0[64 + tid]) + (lds_y0[128 + tid] + lds_y0[192 + tid]);
    }
    if constexpr (CW == 4) {
        if (do_dba) {                                    // 8 row groups x 128 columns, added in order
            __syncthreads();
            *reinterpret_cast<f4*>(lds_a0 + (tid >> 5) * 128 + 4 * (tid & 31)) = dbsum_a;
            __syncthreads();
            if (tid < 128 && kt0 + tid < p.K) {
                float s = lds_a0[tid];
#pragma unroll
                for (int g = 1; g < 8; ++g) s += lds_a0[g * 128 + tid];
                (p.db_out ? p.db_out : outp + (size_t)p.K * p.D)[kt0 + tid] = s;
            }
        }
    }
}

static __global__ __launch_bounds__(kThreads, 3) void wgrad_gemm_dma(const WgradParams p) {
    __shared__ float lds_a0[kWgBR * kWgBK];
    __shared__ float lds_a1[kWgBR * kWgBK];
    __shared__ float lds_y0[kWgBR * kWgBN];
    __shared__ float lds_y1[kWgBR * kWgBN];
    static_assert(sizeof(lds_a0) >= 64 * 64 * sizeof(float), "accumulator exchange buffer");
    // The half-width form only when the whole of K fits in it.  As the LAST of several k
    // tiles it would run at up to twice the pace of its neighbours; the k tiles of a split
    // share their x and dy rows through L2 only while they move through m together
    // (measured on K = 576: 722 MB fetched with a fast last tile, 445 MB with an even pace
    // at 1.5 % more time for its padded MFMAs).
    // p.cw (workgroup-uniform): 1 for channel counts that are not multiples of 4
    if (p.cw == 1) wgrad_dma_body<1>(p, lds_a0, lds_a1, lds_y0, lds_y1, launch_block());
    else if (p.cw == 2) wgrad_dma_body<2>(p, lds_a0, lds_a1, lds_y0, lds_y1, launch_block());
    else wgrad_dma_body<4>(p, lds_a0, lds_a1, lds_y0, lds_y1, launch_block());
}

// The 192-wide k tile: 64 KB of LDS, two workgroups per CU.
static __global__ __launch_bounds__(kThreads, 2) void wgrad_gemm_dma192(const WgradParams p) {
    __shared__ float lds_a0[kWgBR * 192];
    __shared__ float lds_a1[kWgBR * 192];
    __shared__ float lds_y0[kWgBR * kWgBN];
    __shared__ float lds_y1[kWgBR * kWgBN];
    wgrad_dma_body<6>(p, lds_a0, lds_a1, lds_y0, lds_y1, launch_block());
}

// The same with 16-row slabs: 32 KB of LDS and half the per-load state, so that three
// workgroups fit a CU (a stand-alone loop: 140 TFLOP/s against 134 with 32-row slabs).
static __global__ __launch_bounds__(kThreads, 3) void wgrad_gemm_dma192h(const WgradParams p) {
    __shared__ float lds_a0[16 * 192];
    __shared__ float lds_a1[16 * 192];
    __shared__ float lds_y0[16 * kWgBN];
    __shared__ float lds_y1[16 * kWgBN];
    wgrad_dma_body<6, 16>(p, lds_a0, lds_a1, lds_y0, lds_y1, launch_block());
}

// ------------------------------------------------------------------------------
// wgrad for bf16 inputs on v_mfma_f32_32x32x16_bf16 (C and D multiples of 8).
// The MFMA reduces over m, so each lane needs 8 consecutive m of ONE k (or n)
// column, while the slabs arrive m-major ([m][k], k contiguous) straight from
// memory.  `ds_read_b64_tr_b16` does the transposition inside LDS reads: in every
// group of 16 lanes, lane j supplies the address of 4 consecutive elements of row
// j/4 and lane i receives element i%4 of the rows 4r + i/4, r = 0..3 -- i.e. four
// consecutive m of column i.  Two such reads give one MFMA operand.
//   tile 128 k x 64 n per workgroup, wave = 32 k x 64 n, slab = 64 rows of m,
//   two LDS buffers filled by `buffer_load_dwordx4 ... lds`, one barrier per slab.
//   Rows are unpadded (x: 256 B, dy: 128 B); 16-byte chunk c of row m is stored at
//   c ^ ((m & 3) << 1) for x and c ^ (((m >> 1) & 1) << 2) for dy, which spreads the
//   4 rows x 32 B touched by a 16-lane group (and its neighbour group) over all banks.
// ------------------------------------------------------------------------------
typedef short s4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) s4v* lds_s4_ptr_t;

static __global__ __launch_bounds__(kThreads) void wgrad_gemm_dma_bf16(const WgradParams p) {
    constexpr int BR = 64;                               // m rows per slab
    __shared__ uint16_t lds_a0[BR * kWgBK];
    __shared__ uint16_t lds_a1[BR * kWgBK];
    __shared__ uint16_t lds_y0[BR * kWgBN];
    __shared__ uint16_t lds_y1[BR * kWgBN];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;

    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int tiles = p.kt * p.nt;
    const int split = lid / tiles;
    const int tile = lid - split * tiles;
    const int ktile = tile % p.kt;
    const int kt0 = ktile * kWgBK;
    const int n0 = (tile / p.kt) * kWgBN;
    const int m_begin = split * p.m_per_split;
    int m_end = m_begin + p.m_per_split;
    if (m_end > p.M) m_end = p.M;
    const bool do_db = p.want_dbias && (ktile == 0);

    // ---- x: one wave-level load = 4 slab rows x 16 chunks (8 bf16 each); 4 per wave ---
    const int a_row = lane >> 4;
    const int a_lc = (lane & 15) ^ ((a_row & 3) << 1);   // logical chunk fetched
    int a_tap_off, a_fx, a_fy;
    bool a_kok;
    {
        int kk = kt0 + 8 * a_lc;
        unsigned tap, c, fx, fy;
        p.div_c.divmod((unsigned)kk, tap, c);
        p.div_fw.divmod(tap, fx, fy);
        a_kok = kk < p.K;
        a_fx = (int)fx - p.pH;
        a_fy = (int)fy - p.pW;
        a_tap_off = (a_fx * p.W + a_fy) * p.C + (int)c;
    }
    // ---- dy: one wave-level load = 8 slab rows x 8 chunks; 2 per wave -----------------
    const int y_row = lane >> 3;
    const int y_lc = (lane & 7) ^ (((y_row >> 1) & 1) << 2);
    const int y_n = n0 + 8 * y_lc;
    const bool y_nok = y_n < p.D;

    const __amdgpu_buffer_rsrc_t rsrc_x =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.x), 0, (int)p.x_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_y =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.dy), 0, (int)p.dy_bytes, 0x00020000);

    auto issue = [&](int mb, uint16_t* la, uint16_t* ly) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = mb + (wave * 4 + i) * 4 + a_row;
            unsigned s, rem, ho, wo;
            p.div_howo.divmod((unsigned)m, s, rem);
            p.div_wo.divmod(rem, ho, wo);
            const int r0 = (int)ho * p.sH, c0 = (int)wo * p.sW;
            const int pix = (((int)s * p.H + r0) * p.W + c0) * p.C;
            const unsigned bad = (unsigned)!((m < m_end) & a_kok & ((unsigned)(r0 + a_fx) < (unsigned)p.H) &
                                             ((unsigned)(c0 + a_fy) < (unsigned)p.W));
            const unsigned voff = ((unsigned)(pix + a_tap_off) * 2u) | (bad << 31);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_x, (lds_ptr_t)(la + (wave * 4 + i) * 512), 16, (int)voff, 0,
                                                     0, 0);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int m = mb + (wave * 2 + i) * 8 + y_row;
            const unsigned bad = (unsigned)!((m < m_end) & y_nok);
            const unsigned voff = ((unsigned)(m * p.D + y_n) * 2u) | (bad << 31);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_y, (lds_ptr_t)(ly + (wave * 2 + i) * 512), 16, (int)voff, 0,
                                                     0, 0);
        }
    };

    // ---- transposing operand reads -------------------------------------------------------
    // 16-lane group G: columns 16*(G&1).., rows 8*(G>>1)..; lane j of the group points at
    // row j>>2, elements 4*(j&3)..+3.
    const int G = lane >> 4, j16 = lane & 15;
    const int t_row = 8 * (G >> 1) + (j16 >> 2);         // row inside a 16-row step, first read (+4: second)
    const int a_col = wave * 32 + 16 * (G & 1) + 4 * (j16 & 3);      // first k element addressed
    const int y_col = 16 * (G & 1) + 4 * (j16 & 3);                  // first n element (n tile 0; +32: tile 1)
    // element offsets (in bf16) inside a slab row, swizzle applied; row & 3 == j16 >> 2, (row >> 1) & 1 == j16 >> 3
    const int a_eo = (((a_col >> 3) ^ ((j16 >> 2) << 1)) << 3) + (a_col & 4);
    // (odd waves number the two n blocks the other way round: the block a wave sums for dbias is then its block 0)
    const int nflip = wave & 1;
    const int y_eo0 = ((((y_col + 32 * nflip) >> 3) ^ ((j16 >> 3) << 2)) << 3) + (y_col & 4);
    const int y_eo1 = ((((y_col + 32 - 32 * nflip) >> 3) ^ ((j16 >> 3) << 2)) << 3) + (y_col & 4);
    auto tr = [&](const uint16_t* base) {
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr_t)base);
    };

    f16v acc[2];
#pragma unroll
    for (int jn = 0; jn < 2; ++jn)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[jn][v] = 0.f;
    const bool active = kt0 + wave * 32 < p.K;           // wave-uniform

    // dbias: the column sums of dy are one more product, ones times the dy operand the wave holds anyway (every
    // row of the result is the sum); waves 0 and 1 of the k tile 0 take one n block each.  (Adding the columns
    // with 16 two-byte LDS reads per thread and slab made the workgroups of that tile end last.)
    const bool wave_db = do_db && wave < 2;
    f16v acc_db;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_db[v] = 0.f;
    typedef short s8v __attribute__((ext_vector_type(8)));
    const s8v ones = (s8v)(short)0x3F80;

    auto slab = [&](int mb, const uint16_t* la, const uint16_t* ly, uint16_t* na, uint16_t* ny, bool has_next) {
        __builtin_amdgcn_s_waitcnt(0);                   // this wave's loads of the slab have landed
        __syncthreads();
        if (has_next) issue(mb + BR, na, ny);
        if (active || wave_db) {                         // (a wave past K that sums columns multiplies zeros)
#pragma unroll
            for (int st = 0; st < BR / 16; ++st) {
                const int r0 = st * 16 + t_row;
                s4v a0 = tr(la + r0 * kWgBK + a_eo);
                s4v a1 = tr(la + (r0 + 4) * kWgBK + a_eo);
                s4v b00 = tr(ly + r0 * kWgBN + y_eo0);
                s4v b01 = tr(ly + (r0 + 4) * kWgBN + y_eo0);
                s4v b10 = tr(ly + r0 * kWgBN + y_eo1);
                s4v b11 = tr(ly + (r0 + 4) * kWgBN + y_eo1);
                const s8v av = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
                const s8v bv0 = __builtin_shufflevector(b00, b01, 0, 1, 2, 3, 4, 5, 6, 7);
                const s8v bv1 = __builtin_shufflevector(b10, b11, 0, 1, 2, 3, 4, 5, 6, 7);
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av),
                                                                 __builtin_bit_cast(bf16x8, bv0), acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av),
                                                                 __builtin_bit_cast(bf16x8, bv1), acc[1], 0, 0, 0);
                if (wave_db)
                    acc_db = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ones),
                                                                     __builtin_bit_cast(bf16x8, bv0), acc_db, 0, 0, 0);
            }
        }
    };

    if (m_begin < m_end) issue(m_begin, lds_a0, lds_y0);
    for (int mb = m_begin; mb < m_end; mb += 2 * BR) {
        slab(mb, lds_a0, lds_y0, lds_a1, lds_y1, mb + BR < m_end);
        if (mb + BR < m_end) slab(mb + BR, lds_a1, lds_y1, lds_a0, lds_y0, mb + 2 * BR < m_end);
    }

    const size_t split_stride = (size_t)p.K * p.D + p.D;
    float* outp = p.out + (size_t)split * split_stride;
#pragma unroll
    for (int jn = 0; jn < 2; ++jn) {
        const int n = n0 + 32 * (jn ^ nflip) + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int k = kt0 + wave * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (k < p.K && n < p.D) outp[(size_t)k * p.D + n] = acc[jn][v];
        }
    }
    if (wave_db && lane < 32) {                          // row 0 of the sums: element 0 of the lanes 0..31
        const int n = n0 + 32 * nflip + lane;
        if (n < p.D) (p.db_out ? p.db_out : outp + (size_t)p.K * p.D)[n] = acc_db[0];
    }
}

// ------------------------------------------------------------------------------
// wgrad_gemm_dma_bf16w: the same product on wide wave tiles, for outputs of more than 64
// channels.  With a wave tile of 32 k x 64 n an MFMA step needs three transposing 8-byte
// reads per MFMA, 1536 B of LDS traffic for 32 MFMA cycles on each of the four SIMDs: the
// LDS (128 B per clock and CU) is asked for 48 clocks of work per 32 of MFMA and bounds the
// loop.  Here the four waves form a 2 x 2 grid of tiles of 64 k x (32 NB) n (NB = 4: 128 n,
// workgroup tile 128 k x 256 n; NB = 2: 64 n, 128 k x 128 n): 2 + NB operand blocks feed
// 2 NB MFMAs, 1.5 reads per MFMA for NB = 4 (24 clocks of LDS per 32 of MFMA).  One n tile
// also means that x, the larger operand, is gathered once per k tile instead of once per
// (k tile, n tile).
//   slab = 32 rows of m in a ring of three LDS buffers of (8 + 4 NB) KB filled by LDS-direct
//   loads two slabs ahead (one slab of 16 MFMAs per wave is 0.2 us, a fraction of the memory
//   latency), one barrier per slab; 16-byte chunk c of slab row m sits at c ^ ((m & 3) << 2) in
//   both operands: the 4 rows x 64 B that 32 lanes of a transposing read touch then fall into
//   the four 64-byte quarters of the banks.  The loads are inline assembly so that the compiler
//   does not order the LDS reads of a slab behind the loads of later slabs; the wave waits for
//   its own loads of the slab with a partial vmcnt, the barrier covers the other waves'.
//   dbias (column sums of dy) is one more MFMA on the dy operand, ones as the other operand,
//   in the waves of the k tile 0: adding the columns with ordinary LDS reads made those
//   workgroups end last (stride-2 layer 28x28x128 -> 256: 0.166 ms, 0.146 without dbias; the
//   same with it now).
// ------------------------------------------------------------------------------
constexpr int kWwBR = 32;

// KW x 2 waves of 64 k x (32 NB) n each: KW = 2 -> 128 k rows per workgroup, KW = 4 -> 256 (8 waves,
// one workgroup per CU: every dy slab is read by half as many workgroups, and the slabs that the
// workgroups pull out of L2 are what bounds this kernel: 1.17 GB per launch on the stride-2 layer with
// 128 k rows, 8.4 TB/s).
template <int KW, int NB>
static __global__ __launch_bounds__(128 * KW, KW == 4 ? 1 : (NB == 4 ? 2 : 3)) void wgrad_gemm_dma_bf16w(const WgradParams p) {
    constexpr int BR = kWwBR;
    constexpr int NWAVES = 2 * KW;
    constexpr int BK = 64 * KW;                          // k columns of the x slab
    constexpr int BN = 64 * NB;                          // n columns of the dy slab
    constexpr int XCH = BK / 8, YCH = BN / 8;            // 16-byte chunks per slab row
    constexpr int XROWS = 64 / XCH, YROWS = 64 / YCH;    // slab rows per wave-level load
    constexpr int XLOADS = BR / XROWS / NWAVES;          // loads per wave and slab
    constexpr int YLOADS = BR / YROWS / NWAVES;
    static_assert(XLOADS >= 1 && YLOADS >= 1 && XLOADS * XROWS * NWAVES == BR && YLOADS * YROWS * NWAVES == BR, "slab split");
    constexpr int RING = KW == 4 ? 4 : 3;
    __shared__ uint16_t lds_a[RING][BR * BK];
    __shared__ uint16_t lds_y[RING][BR * BN];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kw = wave % KW, nw = wave / KW;            // the wave's place in the KW x 2 grid
    const int l32 = lane & 31;
    const int lh = lane >> 5;

    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int tiles = p.kt * p.nt;
    const int split = lid / tiles;
    const int tile = lid - split * tiles;
    const int ktile = tile % p.kt;
    const int kt0 = ktile * BK;
    const int n0 = (tile / p.kt) * BN;
    const int m_begin = split * p.m_per_split;
    int m_end = m_begin + p.m_per_split;
    if (m_end > p.M) m_end = p.M;
    const bool do_db = p.want_dbias && (ktile == 0);

    // ---- x: one wave-level load = XROWS slab rows x XCH chunks -----------------------------
    // position pc of slab row r holds logical chunk pc ^ ((r & 3) << 2); XROWS divides 4, so the
    // rows a lane loads all have r & 3 == (lane / XCH) + XROWS * (i & (4 / XROWS - 1)): the tap decode
    // is done once per such row class
    const int x_row = lane / XCH;
    const int x_pc = lane % XCH;
    constexpr int XCLS = 4 / XROWS;                      // row classes per lane: 1 or 2
    int a_tap_off[XCLS], a_fx[XCLS], a_fy[XCLS];
    bool a_kok[XCLS];
#pragma unroll
    for (int q = 0; q < XCLS; ++q) {
        const int r3 = (x_row + XROWS * q) & 3;
        const int kk = kt0 + 8 * (x_pc ^ (r3 << 2));
        unsigned tap, c, fx, fy;
        p.div_c.divmod((unsigned)kk, tap, c);
        p.div_fw.divmod(tap, fx, fy);
        a_kok[q] = kk < p.K;
        a_fx[q] = (int)fx - p.pH;
        a_fy[q] = (int)fy - p.pW;
        a_tap_off[q] = (a_fx[q] * p.W + a_fy[q]) * p.C + (int)c;
    }
    // ---- dy: one wave-level load = YROWS slab rows x YCH chunks ------------------------------
    const int y_row = lane / YCH;
    const int y_pc = lane % YCH;

    const u32x4 rsrc_x = raw_rsrc(p.x, p.x_bytes);
    const u32x4 rsrc_y = raw_rsrc(p.dy, p.dy_bytes);

    // The slabs are issued in order, so the image position of the pixel a load fetches moves by 32 rows of m from
    // one call to the next: adds and two carries instead of two divisions per load (integer multiplies run at a
    // quarter of the rate; with the waves of a SIMD taking turns this is worth about 1 %).
    int xs_r[XLOADS], xs_c[XLOADS], xs_off[XLOADS];      // row, column (tap (0,0), no padding) and element offset of that pixel
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
        const int m = m_begin + (wave * XLOADS + i) * XROWS + x_row;
        unsigned s, rem, ho, wo;
        p.div_howo.divmod((unsigned)m, s, rem);
        p.div_wo.divmod(rem, ho, wo);
        xs_r[i] = (int)ho * p.sH;
        xs_c[i] = (int)wo * p.sW;
        xs_off[i] = (((int)s * p.H + xs_r[i]) * p.W + xs_c[i]) * p.C;
    }
    const int wrap_c = p.Wo * p.sW, wrap_r = p.Ho * p.sH;
    const int inc0 = p.inc0 >> 2, inc1 = p.inc1 >> 2, inc2 = p.inc2 >> 2;   // the host counts them in bytes of float32

    auto issue = [&](int mb, uint16_t* la, uint16_t* ly) {
        const unsigned la_base = lds_address(la), ly_base = lds_address(ly);
#pragma unroll
        for (int i = 0; i < XLOADS; ++i) {
            const int ld = wave * XLOADS + i;            // wave-level load number inside the slab
            const int q = XCLS == 1 ? 0 : (i & (XCLS - 1));          // (ld * XROWS) & 3 == XROWS * (i & (XCLS - 1)): XLOADS is even
            const int m = mb + ld * XROWS + x_row;
            const unsigned bad = (unsigned)!((m < m_end) & a_kok[q] & ((unsigned)(xs_r[i] + a_fx[q]) < (unsigned)p.H) &
                                             ((unsigned)(xs_c[i] + a_fy[q]) < (unsigned)p.W));
            const unsigned voff = ((unsigned)(xs_off[i] + a_tap_off[q]) * 2u) | (bad << 31);
            lds_direct_load16(rsrc_x, la_base + (unsigned)ld * 1024u, voff);
            xs_c[i] += p.step_c;                         // m += BR
            const bool c1 = xs_c[i] >= wrap_c;
            xs_c[i] -= c1 ? wrap_c : 0;
            xs_r[i] += c1 ? p.step_r + p.sH : p.step_r;
            const bool c2 = xs_r[i] >= wrap_r;
            xs_r[i] -= c2 ? wrap_r : 0;
            xs_off[i] += (c1 ? inc0 + inc1 : inc0) + (c2 ? inc2 : 0);
        }
#pragma unroll
        for (int i = 0; i < YLOADS; ++i) {
            const int ld = wave * YLOADS + i;
            const int row = ld * YROWS + y_row;          // slab row; the slab starts at a multiple of 32
            const int m = mb + row;
            const int y_n = n0 + 8 * (y_pc ^ ((row & 3) << 2));
            const unsigned bad = (unsigned)!((m < m_end) & (y_n < p.D));
            const unsigned voff = ((unsigned)(m * p.D + y_n) * 2u) | (bad << 31);
            lds_direct_load16(rsrc_y, ly_base + (unsigned)ld * 1024u, voff);
        }
    };
    constexpr int LOADS = XLOADS + YLOADS;               // per wave and slab
    static_assert(XCLS == 1 || XLOADS % XCLS == 0, "row classes repeat with the loads of a wave");

    // ---- transposing operand reads: 16-lane group G covers columns 16 (G & 1).., rows 8 (G >> 1)..;
    // lane j of the group points at row j >> 2, elements 4 (j & 3)..+3
    const int G = lane >> 4, j16 = lane & 15;
    const int t_row = 8 * (G >> 1) + (j16 >> 2);         // row inside a 16-row step, first read (+4: second); & 3 == j16 >> 2
    const int sw = (j16 >> 2) << 2;                      // chunk swizzle of that row (the same for row + 4)
    int a_eo[2], y_eo[NB];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
        const int col = kw * 64 + kb * 32 + 16 * (G & 1) + 4 * (j16 & 3);
        a_eo[kb] = (((col >> 3) ^ sw) << 3) + (col & 4);
    }
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {                    // the wave's block nb is n block (nb + kw) % NB of its half: see dbias
        const int col = nw * 32 * NB + ((nb + kw) % NB) * 32 + 16 * (G & 1) + 4 * (j16 & 3);
        y_eo[nb] = (((col >> 3) ^ sw) << 3) + (col & 4);
    }
    auto tr = [&](const uint16_t* base) {
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr_t)base);
    };
    typedef short s8v __attribute__((ext_vector_type(8)));

    f16v acc[2][NB];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[kb][nb][v] = 0.f;
    const bool active = kt0 + kw * 64 < p.K;             // wave-uniform

    // dbias: the column sums of dy are one more product, a block of ones times the dy operand that the wave
    // holds anyway (every row of the result is the sum; exact products, float32 sums).  Wave kw of the k tile 0
    // takes the n blocks kw, kw + KW, ...: one MFMA more per eight, no reads of its own.  Those are the wave's
    // blocks 0, KW, ... (its blocks are numbered from kw on), so no register is chosen at run time.
    constexpr int DBN = (NB + KW - 1) / KW;
    f16v acc_db[DBN];
#pragma unroll
    for (int j = 0; j < DBN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc_db[j][v] = 0.f;
    const bool wave_db = do_db && kw < NB;
    auto multiply_db = [&](const s8v* bv) {
        const s8v ones = (s8v)(short)0x3F80;
#pragma unroll
        for (int j = 0; j < DBN; ++j) {
            acc_db[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ones),
                                                                __builtin_bit_cast(bf16x8, bv[j * KW]), acc_db[j], 0, 0, 0);
        }
    };

    // operands of one 16-row step of a slab: 2 blocks of 32 k columns, NB blocks of 32 n columns
    auto load_ops = [&](const uint16_t* la, const uint16_t* ly, int st, s8v* av, s8v* bv) {
        const int r0 = st * 16 + t_row;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            const s4v lo = tr(la + r0 * BK + a_eo[kb]);
            const s4v hi = tr(la + (r0 + 4) * BK + a_eo[kb]);
            av[kb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const s4v lo = tr(ly + r0 * BN + y_eo[nb]);
            const s4v hi = tr(ly + (r0 + 4) * BN + y_eo[nb]);
            bv[nb] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
    };
    auto multiply = [&](const s8v* av, const s8v* bv) {
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            acc[0][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av[0]),
                                                                 __builtin_bit_cast(bf16x8, bv[nb]), acc[0][nb], 0, 0, 0);
            // (k rows past K were loaded as zeros: their products vanish without a branch between the MFMAs)
            acc[1][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av[1]),
                                                                 __builtin_bit_cast(bf16x8, bv[nb]), acc[1][nb], 0, 0, 0);
        }
    };
    auto wait_behind = [&](int slabs_behind) {           // this wave's loads have landed, all but those of the newest slabs
        if (RING >= 4 && slabs_behind >= 2) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * LOADS) : "memory");
        else if (slabs_behind >= 1) asm volatile("s_waitcnt vmcnt(%0)" :: "n"(LOADS) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };

    // slab k of the split lives in buffer k % RING; its loads go out RING - 1 slabs earlier
    const int nslab = m_begin < m_end ? (m_end - m_begin + BR - 1) / BR : 0;
#pragma unroll
    for (int k = 0; k < RING - 1; ++k)
        if (k < nslab) issue(m_begin + k * BR, lds_a[k], lds_y[k]);
    int cur = 0;
    for (int k = 0; k < nslab; ++k) {
        wait_behind(min(nslab - 1 - k, RING - 2));       // slab k has landed
        __syncthreads();                                 // ... and so have the other waves' loads; slab k - 1 has been read by all
        int nxt = cur + RING - 1;
        if (nxt >= RING) nxt -= RING;
        // the two waves of a SIMD (nw = 0 and 1) take turns: one works out the addresses of its loads while
        // the other multiplies
        const bool more = k + RING - 1 < nslab;
        if (more && nw == 0) issue(m_begin + (k + RING - 1) * BR, lds_a[nxt], lds_y[nxt]);
        if (active || wave_db) {                         // (a wave past K that sums columns multiplies zeros)
#pragma unroll
            for (int st = 0; st < BR / 16; ++st) {
                s8v av[2], bv[NB];
                load_ops(lds_a[cur], lds_y[cur], st, av, bv);
                multiply(av, bv);
                if (wave_db) multiply_db(bv);
            }
        }
        if (more && nw != 0) issue(m_begin + (k + RING - 1) * BR, lds_a[nxt], lds_y[nxt]);
        cur = cur + 1 == RING ? 0 : cur + 1;
    }

    const size_t split_stride = (size_t)p.K * p.D + p.D;
    float* outp = p.out + (size_t)split * split_stride;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int nb = 0; nb < NB; ++nb) {
            const int n = n0 + nw * 32 * NB + ((nb + kw) % NB) * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int k = kt0 + kw * 64 + kb * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                if (k < p.K && n < p.D) outp[(size_t)k * p.D + n] = acc[kb][nb][v];
            }
        }
    if (wave_db && lane < 32) {                          // row 0 of the sums: element 0 of the lanes 0..31
#pragma unroll
        for (int j = 0; j < DBN; ++j) {
            const int n = n0 + nw * 32 * NB + (j * KW + kw) * 32 + lane;
            if (n < p.D) (p.db_out ? p.db_out : outp + (size_t)p.K * p.D)[n] = acc_db[j][0];
        }
    }
}

// ------------------------------------------------------------------------------
// wgrad_halo_bf16: bf16 wgrad of a unit-stride filter of at most 9 taps on 64 input channels and
// at most 64 output channels, as one persistent workgroup per CU that holds the WHOLE K x N
// result in registers: wave t owns filter tap t (64 k rows x 64 n columns, four 32 x 32
// accumulators), one more wave does nothing but load.
// wgrad_gemm_dma_bf16 gives a workgroup 128 k rows: 4.5 workgroups read every dy row again, each
// x pixel is fetched once per tap, and a 64-row slab is 24 KB of loads for 1 MFLOP, which
// bounds the kernel by what L2 delivers (1.55 times the operands fetched from memory at 1.9 TB/s,
// matrix pipe 22 % busy).  Here a slab is some whole output rows (R rows, R * Wo a multiple of
// 16 and at most 128: two rows of 56) and the loading wave fetches, once, the padded image rows
// under them ("halo", (R + fH - 1) x (Wo + fW - 1) pixel slots of 128 B, padding as zeros from
// offsets outside the buffer descriptor) and the slab's dy rows, two buffers each, a slab ahead;
// tap (fx, fy) reads the halo at slots shifted by fx * Wp + fy.  The MFMA reduces over m, 8
// consecutive m of one k (or n) column per lane, while both tiles lie m-major in LDS:
// `ds_read_b64_tr_b16` transposes on the way (see wgrad_gemm_dma_bf16); chunk q of a 128-byte row
// is stored at q ^ (((row >> 1) & 1) << 2), row = slot number or dy row.
// dbias is one more MFMA (ones times the dy operand) in two of the waves.  Partial results go to
// out + z * (K * D + D) like those of the other wgrad kernels.
// ------------------------------------------------------------------------------
struct WgradHaloParams {
    const void* x;       // [S,H,W,64] bf16
    const void* dy;      // [S,Ho,Wo,D] bf16
    float* out;          // [splits][K*D + D]
    unsigned x_bytes, dy_bytes;
    int S, H, W, Ho, Wo, D, fH, fW, pH, pW;
    int R;               // output rows per slab
    int slab_m;          // R * Wo: multiple of 16, at most kWhRows
    int Wp;              // Wo + fW - 1
    int hslots;          // (R + fH - 1) * Wp, at most kWhSlots
    int nslabs;          // S * Ho / R
    int per;             // slabs per workgroup
    int want_dbias;
    FastDiv div_wp, div_wo, div_fw, div_spi;   // spi: slabs per image = Ho / R
};
constexpr int kWhSlots = 256;       // halo buffer: 256 pixel slots of 128 B
constexpr int kWhRows = 128;        // dy buffer: 128 rows of 128 B
constexpr int kWhMaxTaps = 9;

static __global__ __launch_bounds__(64 * (kWhMaxTaps + 1), 1) void wgrad_halo_bf16(const WgradHaloParams p) {
    constexpr int NLH = kWhSlots / 8, NLD = kWhRows / 8, STEPS = kWhRows / 16;
    __shared__ uint16_t halo[2][kWhSlots * 64];
    __shared__ uint16_t dyb[2][kWhRows * 64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int T = p.fH * p.fW;
    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int sl0 = lid * p.per;
    const int nsl = max(0, min(p.per, p.nslabs - sl0));
    const int K = T * 64;
    float* const outp = p.out + (size_t)lid * ((size_t)K * p.D + p.D);
    const int steps = p.slab_m >> 4;

    if (wave == T) {
        // ---- the loading wave ----
        // Halo load i brings the slots 8 i .. 8 i + 7, dy load j the rows 8 j .. 8 j + 7 (lane / 8 picks
        // the slot or row, lane % 8 the chunk position).  relx / rely: byte offset of the lane's chunk
        // from the slab's first padded pixel / first dy element; a slot is a padding column for all
        // slabs or not (colbad), and lies in a padded row inside the image or not per slab: slot in
        // [lo, hi).  Invalid pieces get bit 31, outside the buffer descriptor: zeros.
        const u32x4 rsrc_x = raw_rsrc(p.x, p.x_bytes);
        const u32x4 rsrc_y = raw_rsrc(p.dy, p.dy_bytes);
        const int lrow = lane >> 3;
        int relx[NLH], rely[NLD];
        unsigned colbad = 0;
#pragma unroll
        for (int i = 0; i < NLH; ++i) {
            const int slot = 8 * i + lrow;
            unsigned r, c;
            p.div_wp.divmod((unsigned)slot, r, c);
            relx[i] = ((int)r * p.W + (int)c) * 128 + (((lane & 7) ^ (((slot >> 1) & 1) << 2)) * 16);
            colbad |= ((unsigned)((int)c - p.pW) >= (unsigned)p.W || 8 * i >= p.hslots ? 1u : 0u) << i;
        }
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const int row = 8 * j + lrow;
            const int n8 = 8 * ((lane & 7) ^ (((row >> 1) & 1) << 2));
            rely[j] = (row * p.D + n8) * 2;
            if (n8 >= p.D || row >= p.slab_m) rely[j] = (int)0x80000000;
        }
        unsigned offx[NLH], offy[NLD];
        auto addresses = [&](int slab) __attribute__((always_inline)) {
            unsigned s_img, r_img;
            p.div_spi.divmod((unsigned)slab, s_img, r_img);
            const int R0 = (int)r_img * p.R - p.pH;                         // image row of padded row 0 of the slab
            const int base = (((int)s_img * p.H + R0) * p.W - p.pW) * 128;
            const int a0 = lrow + R0 * p.Wp;                                // slot - lo
            const int b0 = (p.H - R0) * p.Wp - 1 - lrow;                    // hi - 1 - slot
#pragma unroll
            for (int i = 0; i < NLH; ++i) {
                const unsigned rowbad = (unsigned)((a0 + 8 * i) | (b0 - 8 * i)) & 0x80000000u;
                offx[i] = (unsigned)(base + relx[i]) | rowbad | ((colbad << (31 - i)) & 0x80000000u);
            }
            const int ybase = (((int)s_img * p.Ho + (int)r_img * p.R) * p.Wo) * p.D * 2;
#pragma unroll
            for (int j = 0; j < NLD; ++j) offy[j] = (unsigned)(ybase + rely[j]) | ((unsigned)rely[j] & 0x80000000u);
        };
        auto issue = [&](int buf) __attribute__((always_inline)) {
            const unsigned hb = lds_address(&halo[buf][0]), yb = lds_address(&dyb[buf][0]);
            // every load is issued, without a branch; those past the slab have offsets outside the
            // descriptors (no memory access, zeros into buffer space nobody reads)
#pragma unroll
            for (int i = 0; i < NLH; ++i) lds_direct_load16(rsrc_x, hb + (unsigned)i * 1024u, offx[i]);
#pragma unroll
            for (int j = 0; j < NLD; ++j) lds_direct_load16(rsrc_y, yb + (unsigned)j * 1024u, offy[j]);
        };
        if (nsl > 0) {
            addresses(sl0);
            issue(0);
        }
        if (nsl > 1) addresses(sl0 + 1);
        __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
        asm volatile("s_barrier" ::: "memory");
        for (int t = 0; t < nsl; ++t) {
            // the multiplying waves are done with slab t - 1, whose buffers take slab t + 1
            if (t + 1 < nsl) issue((t + 1) & 1);
            if (t + 2 < nsl) addresses(sl0 + t + 2);
            __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
            asm volatile("s_barrier" ::: "memory");
        }
        return;
    }
    if (wave > T) return;                                                  // waves beyond the taps and the loader

    // ---- the multiplying waves: wave t owns tap t ----
    unsigned fx, fy;
    p.div_fw.divmod((unsigned)wave, fx, fy);
    const int shift = (int)fx * p.Wp + (int)fy;
    // transposing reads: 16-lane group G covers columns 16 (G & 1).. and rows 8 (G >> 1)..; lane j of the
    // group points at row j >> 2 (second read: + 4), elements 4 (j & 3)..+3
    const int tr_row = 8 * (lane >> 5) + ((lane & 15) >> 2);
    const int col0 = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    int offa[STEPS][2];                                                    // element offsets into a halo buffer (k block 0; ^ 32: block 1)
#pragma unroll
    for (int st = 0; st < STEPS; ++st)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int row = min(16 * st + tr_row + 4 * h, p.slab_m - 1);
            unsigned r, wo;
            p.div_wo.divmod((unsigned)row, r, wo);
            const int slot = (int)r * p.Wp + (int)wo + shift;
            offa[st][h] = slot * 64 + ((((col0 >> 3) ^ (((slot >> 1) & 1) << 2)) << 3) + (col0 & 4));
        }
    // into a dy buffer, step 0: the wave's n block 0 (^ 32: its block 1).  Odd waves number the two blocks the other
    // way round, so that the block a wave sums for dbias (below) is its block 0 whatever the wave.
    const int nflip = wave & 1;
    int offb[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row = tr_row + 4 * h;
        offb[h] = (row * 64 + ((((col0 >> 3) ^ (((row >> 1) & 1) << 2)) << 3) + (col0 & 4))) ^ (32 * nflip);
    }
    f16v acc[2][2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[kb][nb][v] = 0.f;
    typedef short s8v __attribute__((ext_vector_type(8)));
    auto tr = [&](const uint16_t* q) __attribute__((always_inline)) {
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr_t)q);
    };
    // dbias: the column sums of dy are one more product, ones times the dy operand a wave holds anyway (every row
    // of the result is the sum).  Two waves take one n block each, on SIMDs that carry two multiplying waves where
    // another carries three (waves 2 and 3 of a 3x3 filter's nine); a lone wave takes both blocks.
    const int db_first = T >= 4 ? 2 : 0;
    const bool db_one = p.want_dbias && (wave == db_first || (T >= 2 && wave == db_first + 1));
    const bool db_two = p.want_dbias && T == 1;
    f16v acc_db;
#pragma unroll
    for (int v = 0; v < 16; ++v) acc_db[v] = 0.f;
    // (the lone wave: ones in the rows 0..15 for block 0 and in the rows 16..31 for block 1, one set of accumulators)
    const s8v ones0 = (s8v)(short)(db_two && l32 >= 16 ? 0 : 0x3F80);
    const s8v ones1 = (s8v)(short)(l32 >= 16 ? 0x3F80 : 0);
    asm volatile("s_barrier" ::: "memory");
    for (int t = 0; t < nsl; ++t) {
        const uint16_t* hb = halo[t & 1];
        const uint16_t* yb = dyb[t & 1];
        // the operands of step st + 1 are read while the four MFMAs of step st run
        s8v a[2][2], b[2][2];
        auto read_step = [&](int st, s8v (&ra)[2], s8v (&rb)[2]) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < 2; ++q) {
                ra[q] = __builtin_shufflevector(tr(hb + (offa[st][0] ^ (32 * q))), tr(hb + (offa[st][1] ^ (32 * q))), 0, 1, 2,
                                                3, 4, 5, 6, 7);
                rb[q] = __builtin_shufflevector(tr(yb + st * 1024 + (offb[0] ^ (32 * q))),
                                                tr(yb + st * 1024 + (offb[1] ^ (32 * q))), 0, 1, 2, 3, 4, 5, 6, 7);
            }
        };
        read_step(0, a[0], b[0]);
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            if (st < steps) {
                if (st + 1 < STEPS && st + 1 < steps) read_step(st + 1, a[(st + 1) & 1], b[(st + 1) & 1]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int nb = 0; nb < 2; ++nb)
                        acc[kb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a[st & 1][kb]),
                                                                              __builtin_bit_cast(bf16x8, b[st & 1][nb]),
                                                                              acc[kb][nb], 0, 0, 0);
                if (db_one || db_two)
                    acc_db = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ones0),
                                                                     __builtin_bit_cast(bf16x8, b[st & 1][0]), acc_db, 0, 0, 0);
                if (db_two)
                    acc_db = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, ones1),
                                                                     __builtin_bit_cast(bf16x8, b[st & 1][1]), acc_db, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        asm volatile("s_barrier" ::: "memory");
    }
    if ((db_one || db_two) && lane < 32) {               // row 0 of the sums: element 0 of the lanes 0..31
        const int n = 32 * nflip + lane;                 // the wave's block 0
        if (n < p.D) outp[(size_t)K * p.D + n] = acc_db[0];
        if (db_two && 32 + lane < p.D) outp[(size_t)K * p.D + 32 + lane] = acc_db[8];       // row 16
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int n = 32 * (nb ^ nflip) + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int k = wave * 64 + 32 * kb + 8 * (v >> 2) + 4 * lh + (v & 3);
                if (n < p.D) outp[(size_t)k * p.D + n] = acc[kb][nb][v];
            }
        }
}

// ------------------------------------------------------------------------------
// wgrad_halo_f32: the fp32 twin of wgrad_halo_bf16 for 64 input channels, at most 64 output
// channels and at most 9 unit-stride taps.  One persistent workgroup per CU holds the whole
// K x N result in registers, 12 multiplying waves of three 32 x 32 accumulators each (wave w: n block
// w & 1, k blocks 3 (w >> 1) .. + 2, a k block being half a tap: 32 channels), three per SIMD, and a
// thirteenth wave that only loads.  A slab is ONE output row (Wo pixels = NPAIRS pairs: an MFMA
// 32x32x2 reduces over two pixels) and the three padded source rows under it (fH x Wp pixel slots
// of 256 B), two buffers each, loaded a slab ahead.  A lane's operand of pixel pair p is one float
// at a constant offset plus 512 p bytes from a per-lane base (ds_read_b32 with an immediate offset):
// the loop is four LDS reads and three MFMAs per pair, no address arithmetic, no wait on memory.
// A pixel's 64 floats are stored with their 128-byte halves swapped in odd slots (dy: odd rows), so
// that the two pixels of a pair, read by the two halves of a wave, fall into different banks.
// dbias: the waves of k blocks 0..2 add up the dy values they multiply.
// ------------------------------------------------------------------------------
constexpr int kFhRowSlots = 68;     // slots per padded row in LDS: Wo + fW - 1 rounded up to a multiple of 4
constexpr int kFhSlots = 3 * kFhRowSlots;   // halo buffer: at most 3 padded rows of 256-byte pixel slots
constexpr int kFhRows = 64;         // dy buffer: 64 rows of 256 B
constexpr int kFhWaves = 13;

template <int NPAIRS>
static __global__ __launch_bounds__(64 * kFhWaves, 1) void wgrad_halo_f32(const WgradHaloParams p) {
    constexpr int NLD = kFhRows / 4;
    __shared__ float halo[2][kFhSlots * 64];
    __shared__ float dyb[2][kFhRows * 64];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int T = p.fH * p.fW;
    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int sl0 = lid * p.per;
    const int nsl = max(0, min(p.per, p.nslabs - sl0));
    const int K = T * 64;
    float* const outp = p.out + (size_t)lid * ((size_t)K * p.D + p.D);

    if (wave == kFhWaves - 1) {
        // ---- the loading wave ----
        // It shares a SIMD with three waves that issue 64-cycle MFMAs back to back, and a vector
        // instruction of its own waits for a gap between them: with five vector instructions of
        // address arithmetic per load it needed 18 500 cycles for the 58 loads of a slab, more than the
        // slab's MFMAs take.  So a load is scalar work only: padded row r of the halo takes Wpl / 4
        // loads of 4 slots (lane / 16 picks the slot, lane % 16 the 16-byte chunk position; odd slots
        // hold chunk c at c ^ 8) whose per-lane byte offset inside an image row is a constant of the
        // workgroup (padding columns: bit 31, outside the descriptor: zeros); the row's start comes
        // in as the scalar offset, and a padded row above or below the image is read through an
        // empty descriptor.  dy rows likewise.
        __builtin_amdgcn_s_setprio(3);
        const u32x4 rsrc_x = raw_rsrc(p.x, p.x_bytes);
        const u32x4 rsrc_y = raw_rsrc(p.dy, p.dy_bytes);
        const u32x4 rsrc_none = raw_rsrc(p.x, 0u);
        const int lrow = lane >> 4;
        constexpr int NLR = kFhRowSlots / 4;
        unsigned voffx[NLR], voffy[NLD];
#pragma unroll
        for (int g = 0; g < NLR; ++g) {
            const int c = 4 * g + lrow;
            const int lc = (lane & 15) ^ ((c & 1) << 3);                    // Wpl is a multiple of 4: slot parity = column parity
            voffx[g] = (unsigned)(c - p.pW) < (unsigned)p.W ? (unsigned)(((c - p.pW) * 64 + 4 * lc) * 4) : 0x80000000u;
        }
#pragma unroll
        for (int j = 0; j < NLD; ++j) {
            const int row = 4 * j + lrow;
            const int n4 = 4 * ((lane & 15) ^ ((row & 1) << 3));
            voffy[j] = (n4 < p.D && row < p.slab_m) ? (unsigned)((row * p.D + n4) * 4) : 0x80000000u;
        }
        auto load = [&](const u32x4& rsrc, unsigned lds_base, unsigned voff, unsigned soff) __attribute__((always_inline)) {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                         :: "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
        };
        const int nlr = p.Wp >> 2;                                         // p.Wp is the padded row pitch Wpl here
        auto fetch = [&](int slab, int buf) __attribute__((always_inline)) {
            unsigned s_img, r_img;
            p.div_spi.divmod((unsigned)slab, s_img, r_img);
            const int s_u = __builtin_amdgcn_readfirstlane((int)s_img), r_u = __builtin_amdgcn_readfirstlane((int)r_img);
            const unsigned hb = lds_address(&halo[buf][0]), yb = lds_address(&dyb[buf][0]);
#pragma unroll
            for (int r = 0; r < 3; ++r) {
                if (r < p.fH) {
                    const int row = r_u - p.pH + r;                         // image row of padded row r
                    const bool ok = (unsigned)row < (unsigned)p.H;
                    const unsigned soff = ok ? (unsigned)((s_u * p.H + row) * p.W) * 256u : 0u;
                    const u32x4 rs = ok ? rsrc_x : rsrc_none;
#pragma unroll
                    for (int g = 0; g < NLR; ++g)
                        if (g < nlr) load(rs, hb + (unsigned)((r * p.Wp + 4 * g) * 256), voffx[g], soff);
                }
            }
            const unsigned ybase = (unsigned)((s_u * p.Ho + r_u) * p.Wo) * (unsigned)(p.D * 4);
#pragma unroll
            for (int j = 0; j < NLD; ++j) load(rsrc_y, yb + (unsigned)j * 1024u, voffy[j], ybase);
        };
        if (nsl > 0) fetch(sl0, 0);
        __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
        asm volatile("s_barrier" ::: "memory");
        for (int t = 0; t < nsl; ++t) {
            // the multiplying waves are done with slab t - 1, whose buffers take slab t + 1
            if (t + 1 < nsl) fetch(sl0 + t + 1, (t + 1) & 1);
            __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
            asm volatile("s_barrier" ::: "memory");
        }
        return;
    }

    // ---- the multiplying waves ----
    const int nb = wave & 1, kb0 = 3 * (wave >> 1);
    // byte offsets of the lane's operand of pair 0: x[pixel lh][k block q, channel l32] and dy[row lh][32 nb + l32]
    int offa[3];
    bool live[3];
#pragma unroll
    for (int q = 0; q < 3; ++q) {
        const int kb = kb0 + q;
        live[q] = kb < 2 * T;                                              // wave-uniform
        unsigned fx, fy;
        p.div_fw.divmod((unsigned)min(kb >> 1, T - 1), fx, fy);
        const int slot = lh + (int)fx * p.Wp + (int)fy;
        offa[q] = (slot * 64 + ((32 * (kb & 1) + l32) ^ ((slot & 1) << 5))) * 4;
    }
    const int offb = (lh * 64 + ((32 * nb + l32) ^ (lh << 5))) * 4;
    f16v acc[3];
#pragma unroll
    for (int q = 0; q < 3; ++q)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[q][v] = 0.f;
    float db = 0.f;
    const bool do_db = p.want_dbias && kb0 == 0;
    asm volatile("s_barrier" ::: "memory");
    for (int t = 0; t < nsl; ++t) {
        const char* hb = reinterpret_cast<const char*>(halo[t & 1]);
        const char* yb = reinterpret_cast<const char*>(dyb[t & 1]);
        const char* pa[3] = {hb + offa[0], hb + offa[1], hb + offa[2]};
        const char* pb = yb + offb;
        float a[2][3], b[2];
        auto read_pair = [&](int pr, int s) __attribute__((always_inline)) {
#pragma unroll
            for (int q = 0; q < 3; ++q) a[s][q] = *reinterpret_cast<const float*>(pa[q] + 512 * pr);
            b[s] = *reinterpret_cast<const float*>(pb + 512 * pr);
        };
        read_pair(0, 0);
#pragma unroll
        for (int pr = 0; pr < NPAIRS; ++pr) {
            if (pr + 1 < NPAIRS) read_pair(pr + 1, (pr + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < 3; ++q)                                      // blocks past the last tap too: no branch in here
                acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[pr & 1][q], b[pr & 1], acc[q], 0, 0, 0);
            db += b[pr & 1];
            __builtin_amdgcn_sched_barrier(0);
        }
        asm volatile("s_barrier" ::: "memory");
    }
    if (do_db) {
        // everyone is past the last barrier of the loop: the first dy buffer is free
        float* red = dyb[0];
        red[nb * 64 + lane] = db;
        __builtin_amdgcn_s_waitcnt(0);
        if (lh == 0 && 32 * nb + l32 < p.D) outp[(size_t)K * p.D + 32 * nb + l32] = red[nb * 64 + l32] + red[nb * 64 + 32 + l32];
    }
#pragma unroll
    for (int q = 0; q < 3; ++q) {
        if (live[q]) {
            const int n = 32 * nb + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int k = (kb0 + q) * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
                if (n < p.D) outp[(size_t)k * p.D + n] = acc[q][v];
            }
        }
    }
}


}  // namespace aeth
