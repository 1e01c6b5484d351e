// Device side of the gather-GEMM path (fprop, dgrad, dense fprop / dgrad): the register-staged
// and LDS-direct slab kernels, the halo kernels for bf16, the resident kernel for short-K fp32
// products, the filter packer and the direct kernels for 1 to 3 input channels.
#pragma once
#include "conv_common.h"

namespace aeth {

template <typename T, int BM, int BN, int WM, int WN, int VEC>
__global__ __launch_bounds__(kThreads, 3) void gather_gemm(const GatherParams p) {
    static_assert((BM / WM) * (BN / WN) == 4, "4 waves per workgroup");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "32x32 MFMA tiles");
    constexpr int CE = Elem<T>::CE;
    constexpr int BK = Elem<T>::BK;
    constexpr int AL = BM / 32;          // 128-bit A loads per thread per slab
    constexpr int BL = BN / 32;
    constexpr int TM = WM / 32;
    constexpr int TN = WN / 32;

    __shared__ f4 lds_a[BM * kLDC];
    __shared__ f4 lds_b[BN * kLDC];

    const T* __restrict__ src = static_cast<const T*>(p.src);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int wm0 = (wave % (BM / WM)) * WM;
    const int wn0 = (wave / (BM / WM)) * WN;

    const int ntile = (p.N + BN - 1) / BN;
    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int m0 = (lid / ntile) * BM;
    const int n0 = (lid % ntile) * BN;

    // ---- per-thread row bookkeeping for the A gather --------------------------
    const int k4 = tid & 7;              // which chunk of the slab row
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
    const T* bt_row = static_cast<const T*>(p.bt) + (size_t)(n0 + r0) * p.Kpad + CE * k4;

    f4 areg[AL];
    f4 breg[BL];

    auto load_slab = [&](int k0) {
        if (VEC == CE) {
            int kk = k0 + CE * k4;
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
                if (ok) v = *reinterpret_cast<const f4*>(src + (base_off[i] + tap_off));
                areg[i] = v;
            }
        } else {
            struct Chunk { T e[CE]; } tmp[AL];
#pragma unroll
            for (int e = 0; e < CE; ++e) {
                int kk = k0 + CE * k4 + e;
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
                    T v = (T)0;
                    if (ok) v = src[base_off[i] + tap_off];
                    tmp[i].e[e] = v;
                }
            }
#pragma unroll
            for (int i = 0; i < AL; ++i) areg[i] = __builtin_bit_cast(f4, tmp[i]);
        }
#pragma unroll
        for (int i = 0; i < BL; ++i)
            breg[i] = *reinterpret_cast<const f4*>(bt_row + (size_t)(32 * i) * p.Kpad + k0);
    };

    auto store_slab = [&]() {
#pragma unroll
        for (int i = 0; i < AL; ++i) lds_a[(r0 + 32 * i) * kLDC + k4] = areg[i];
#pragma unroll
        for (int i = 0; i < BL; ++i) lds_b[(r0 + 32 * i) * kLDC + k4] = breg[i];
    };

    f16v acc[TM][TN];
    init_acc<TM, TN>(p, p.bias, acc, n0 + wn0, lh);

    if (p.Kpad > 0) {
        load_slab(0);
        store_slab();
        __syncthreads();
    }

    for (int k0 = 0; k0 < p.Kpad; k0 += BK) {
        const bool more = k0 + BK < p.Kpad;
        if (more) load_slab(k0 + BK);

#pragma unroll
        for (int g = 0; g < kChunksPerRow / 2; ++g) {
            f4 a[TM], b[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) a[i] = lds_a[(wm0 + 32 * i + l32) * kLDC + 2 * g + lh];
#pragma unroll
            for (int j = 0; j < TN; ++j) b[j] = lds_b[(wn0 + 32 * j + l32) * kLDC + 2 * g + lh];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) mma_chunk<T>(b[j], a[i], acc[i][j]);
        }
        __syncthreads();
        if (more) {
            store_slab();
            __syncthreads();
        }
    }

    store_tile<TM, TN>(p, p.out, acc, m0 + wm0, n0 + wn0, l32, lh);
}

// ------------------------------------------------------------------------------
// gather-GEMM, LDS-direct variant (the fast path whenever channels come in whole
// 16-byte chunks).  Same tiling and MFMA schedule as gather_gemm, but the slabs go
// from memory straight into LDS with `buffer_load_dwordx4 ... lds`: no staging
// registers, no ds_write, and two LDS buffers so the loads of slab k+1 are in
// flight while slab k is multiplied (one barrier per slab).
//   * One wave-level load writes 64 consecutive 16-byte chunks = 8 slab rows, so
//     rows are unpadded (128 B) and bank conflicts are avoided by an XOR swizzle:
//     logical chunk c of row r lives at chunk position c ^ ((r >> 1) & 7).  A
//     128-bit operand read is served 16 lanes (= 16 consecutive rows) at a time
//     from 64 banks; rows r and r+1 differ in address bit 7 and the 8 row pairs get
//     8 different chunk positions, so the 16 lanes cover the 64 banks exactly once.
//     The swizzle is applied on the global side (each lane of a load fetches the
//     logical chunk that belongs at its LDS position) and undone by the operand reads.
//   * Padding taps and rows past M use a byte offset of 2^31, which is outside the
//     buffer descriptor's extent: the load returns zeros.
// ------------------------------------------------------------------------------


//   * UT ("uniform tap"): when the channel count is a multiple of the slab width and
//     the filter has at most 32 taps, a slab lies inside one tap.  fp32 MFMA shares
//     the FP32 lanes with ordinary vector instructions, so every address instruction
//     costs MFMA time; in this mode the tap decode runs on the scalar unit and each
//     row's per-tap validity is a precomputed bit mask: 3 vector instructions per load.
//   * KC = 16-byte chunks per slab row: 8 (slab = 32 floats of k, 48 KB of LDS for a
//     128 x 64 tile, 3 workgroups per CU) or 4 (16 floats, 24 KB, 5 per CU).  The
//     shallow slab pays a barrier twice as often but keeps more workgroups resident, and
//     those hide each other's set-up, first loads and epilogue.  With KC = 4 a wave-level
//     load covers 16 rows, chunk c of row r lives at c ^ ((r >> 2) & 3), and a 16-lane
//     read group (16 rows x 64 B) again covers the 64 banks exactly once.
//   * NLOOP: for a K of at most two slabs and several n tiles (1x1 convolutions onto many
//     channels: the HBM-bound case, where a one-tile workgroup is mostly set-up).  The
//     workgroup keeps its A tile, both slabs, in the two A buffers and walks over all n
//     tiles: one set-up and one fetch of A per m tile instead of one per output tile.
//   * SA ("scalar addressing", uniform-tap fp32 tiles of 64 or 128 rows): the loads of the slab
//     loop use no vector instruction at all.  A lane's offset is a constant of the tile (its row's tap (0,0)
//     plus its chunk, from a base moved down by the padding so that it is never negative: the range check
//     looks at the vector offset alone), the tap and the channel block go into the scalar offset, and what
//     lies outside the image at the slab's tap is one ballot per slab over the wave's 16 or 32 rows: a load whose
//     8 rows are all inside, nearly all of them, is issued as it is; else the 8 bits are spread over the
//     lanes on the scalar unit and one v_cndmask sends the outside lanes beyond the descriptor.

// RUNS (the 8-wave bf16 tiles, whose launches wait for their stores rather than for instruction issue): the pixels are the
// MFMAs' first operand and the filter rows of a wave's columns are fetched interleaved (column l of block j is channel
// TN l + j), so that the tile goes out in runs of 32 TN contiguous floats per pixel (store_tile_runs).
// BKN (fp32 fprop): the B operand is the filter w[fH][fW][C][D] itself, a [K][N] matrix with n contiguous: a slab is 32 rows of k
// x BN floats (1 KB loads of 4 or 8 rows; with 64 columns the odd rows are stored with their halves swapped, so that the two
// lane halves of a 4-byte operand read, which sit one row apart, use different banks), and an operand read is four 4-byte reads
// from four rows instead of one 16-byte read.  No packing launch.
// The body takes the workgroup's place in the launch and its four slab buffers as arguments, so that it can also be one
// part of a launch that holds two kernels (pair_f32.hip).
template <typename T, int BM, int BN, int WM, int WN, bool UT, int KC, bool NLOOP, bool SA = false, bool RUNS = false, bool BKN = false>
__device__ __forceinline__ void gather_gemm_dma_body(const GatherParams& p, const BlockId blk, f4* lds_a0, f4* lds_a1, f4* lds_b0,
                                                     f4* lds_b1) {
    static_assert(!BKN || (sizeof(T) == 4 && KC == 8 && !NLOOP && (BN == 64 || BN == 32)), "filter in place: fp32 slab tiles");
    // 4 waves, or 8 for the widest bf16 tiles (256 x 128 and 256 x 256: one workgroup per CU)
    constexpr int NW = (BM / WM) * (BN / WN);
    static_assert(NW == 4 || (NW == 8 && !NLOOP && !SA), "4 or 8 waves per workgroup");
    static_assert(!RUNS || !NLOOP, "runs: not in the n-loop mode");
    static_assert(!RUNS || ((sizeof(T) == 2 && (WN == 32 || WN == 64 || WN == 128)) || (SA && sizeof(T) == 4 && (WN == 64 || WN == 32))),
                  "runs: the bf16 tiles and the fp32 tiles with scalar addressing");
    static_assert(!SA || (UT && !NLOOP && (BM == 128 || BM == 64) && sizeof(T) == 4), "scalar addressing: fp32 uniform-tap tiles of 64 or 128 rows");
    static_assert(KC == 8 || KC == 4, "slab rows of 8 or 4 chunks");
    constexpr int CE = Elem<T>::CE;
    constexpr int BK = KC * CE;          // elements of k per slab
    constexpr int RPL = 64 / KC;         // slab rows per wave-level load
    constexpr int SH = KC == 8 ? 1 : 2;  // swizzle: chunk position = chunk ^ ((row >> SH) & (KC - 1))
    constexpr int G = KC / 2;            // MFMA groups per slab (one 16-byte chunk per lane half each)
    constexpr int AL = BM / (NW * RPL);  // wave-level A loads per wave per slab
    constexpr int BL = BN / (NW * RPL);
    static_assert(AL >= 1 && BL >= 1 && BM % (NW * RPL) == 0 && BN % (NW * RPL) == 0, "tile too small for KC");
    static_assert(KC == 4 || AL % 2 == 0, "8-row load blocks of a wave alternate even/odd");
    constexpr int TM = WM / 32;
    constexpr int TN = WN / 32;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int wm0 = (wave % (BM / WM)) * WM;
    const int wn0 = (wave / (BM / WM)) * WN;
    const int ntile = (p.N + BN - 1) / BN;
    const int lid = xcd_contiguous_id(blk.x, blk.gx);
    // (one n tile: no division; the compiler divides scalars by way of the vector unit's reciprocal, some 20
    // vector instructions that a workgroup starting next to busy ones waits for one by one)
    const int mt = (NLOOP || ntile == 1) ? lid : lid / ntile;
    const int m0 = mt * BM;
    int n0 = (NLOOP || ntile == 1) ? 0 : (lid - mt * ntile) * BN;

    // The bias is fetched first: its latency passes behind the row decode.
    const int split = blk.y;
    f4 bv[TN][4];
    load_bias<TN>(p, split == 0 ? p.bias : nullptr, bv, n0 + wn0, lh);

    const int lr = lane / KC;                  // row inside a load block
    // logical chunk this lane fetches: (lane % KC) ^ swizzle(row).  KC == 8: the 8-row
    // blocks alternate between row bits (0,lane>>4) and (4 | lane>>4), so odd blocks use
    // k4e ^ 4; KC == 4: 16-row blocks, the same for every block
    const int k4e = KC == 8 ? (lane & 7) ^ (lane >> 4) : (lane & 3) ^ (lane >> 4);
    constexpr int ODD = KC == 8 ? 4 : 0;       // what an odd load block xors into the chunk
    // Row decode: thread t works out the image position of row m0 + t once, and the
    // KC lanes that fetch a row take it from a table in LDS (decoding AL rows in every
    // lane made the set-up a quarter of the life of a 9-slab workgroup).  An entry is
    // (element offset of tap (0,0), aux); aux is, in uniform-tap mode, one bit per tap
    // that says "outside the image" (all ones for rows past M), else (row << 16 | column).
    // The table sits in the second B buffer, which is first written after the first
    // barrier of the K loop.
    static_assert(BM <= 64 * NW && BM * sizeof(int2) <= BN * KC * sizeof(f4), "row table fits the B buffer");
    int2* rowtab = reinterpret_cast<int2*>(lds_b1);
    if (tid < BM) {
        const int m = m0 + tid;
        int off = 0, br = kInvalidRow, bc = 0;
        if (m < p.M) {
            unsigned s, rem, ii, jj;
            p.div_hw.divmod((unsigned)m, s, rem);
            p.div_w.divmod(rem, ii, jj);
            br = (int)ii * p.sh + p.rh0;
            bc = (int)jj * p.sw + p.rw0;
            off = (((int)s * p.Hs + br) * p.Ws + bc) * p.Cs;
        }
        int aux = (int)(((unsigned)br << 16) | ((unsigned)bc & 0xffffu));
        if (UT) {
            // taps (th, tw) inside the image: th in [max(0,-br), min(Th, Hs-br)), same for tw;
            // a row past M has br = kInvalidRow and an empty range
            auto span = [](int lo, int hi) -> unsigned {     // bits [lo, hi) of a mask, 0 <= lo, hi <= 32
                const unsigned upto_hi = hi > 0 ? ~0u >> (32 - hi) : 0u;
                const unsigned upto_lo = lo > 0 ? ~0u >> (32 - lo) : 0u;
                return hi > lo ? upto_hi & ~upto_lo : 0u;
            };
            const int lo_r = min(max(-br, 0), 32), hi_r = min(max(p.Hs - br, 0), p.Th);
            const int lo_c = min(max(-bc, 0), 32), hi_c = min(max(p.Ws - bc, 0), p.Tw);
            const unsigned rmask = span(lo_r, hi_r), cmask = span(lo_c, hi_c);
            unsigned valid = 0;
            for (int th = 0; th < p.Th; ++th) valid |= (((rmask >> th) & 1u) ? cmask : 0u) << (th * p.Tw);
            aux = (int)~valid;
        }
        rowtab[tid] = int2{off, aux};
    }
    __syncthreads();
    int base_off[AL];
    int base_rc[AL];
    unsigned a_byte[AL], a_inv[AL];
#pragma unroll
    for (int i = 0; i < AL; ++i) {
        const int2 e = rowtab[(wave * AL + i) * RPL + lr];
        base_off[i] = e.x;
        base_rc[i] = e.y;
        a_inv[i] = (unsigned)e.y;
        a_byte[i] = (unsigned)(e.x + CE * (k4e ^ ((i & 1) ? ODD : 0))) * (unsigned)sizeof(T);
    }
    // SA: lane l keeps the outside-the-image bits, one per tap, of the wave's row l (modulo its 32 or 16 rows);
    // a ballot over the slab's tap bit gives the rows' mask in a scalar register (three vector instructions per
    // slab; nine masks held in scalar registers and selected by the tap made the compiler keep the
    // kernel's whole state in memory)
    unsigned aux_row = 0, cur_mask = 0;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const unsigned sa_bias = SA ? (unsigned)((max(-p.rh0, 0) * p.Ws + max(-p.rw0, 0)) * p.Cs) * (unsigned)sizeof(T) : 0u;
    if constexpr (SA) {
        aux_row = (unsigned)rowtab[wave * (AL * RPL) + (lane & (AL * RPL - 1))].y;
#pragma unroll
        for (int i = 0; i < AL; ++i) a_byte[i] += sa_bias;
    }
    const u32x4 sa_rsrc_a = raw_rsrc(static_cast<const char*>(p.src) - sa_bias, (unsigned)p.src_bytes + sa_bias);
    const u32x4 sa_rsrc_b = raw_rsrc(p.bt, (unsigned)p.bt_bytes);
    unsigned b_off[BL];
    auto set_b_off = [&]() {
#pragma unroll
        for (int i = 0; i < BL; ++i) {
            if constexpr (BKN) {
                // load ld = wave BL + i brings rows RB ld .. of the slab, 16-byte chunks of BN floats each
                constexpr int CPRB = BN / 4, RB = 64 / CPRB;
                const int row = (wave * BL + i) * RB + lane / CPRB;
                const int c = (lane % CPRB) ^ ((BN == 64 && (row & 1)) ? 8 : 0);
                b_off[i] = (unsigned)((row * p.bt_ld + n0 + 4 * c) * 4);
                continue;
            }
            const int k4 = k4e ^ (((wave * BL + i) & 1) ? ODD : 0);
            int r = (wave * BL + i) * RPL + lr;          // slab row; RUNS: it holds channel (r / WN) WN + TN (r % 32) + (r % WN) / 32
            if constexpr (RUNS) r = (r / WN) * WN + (WN / 32) * (r & 31) + (r % WN) / 32;
            b_off[i] = (unsigned)(((n0 + r) * p.bt_ld + CE * k4) * (int)sizeof(T));
        }
    };
    set_b_off();

    const __amdgpu_buffer_rsrc_t rsrc_a =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.src), 0, (int)p.src_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p.bt), 0, (int)p.bt_bytes, 0x00020000);

    // The loads of a slab are issued in parts between the MFMA groups of the slab
    // before it: a burst of AL + BL loads right after the barrier keeps the wave away
    // from the matrix pipe for the time the memory pipeline takes to accept them.
    // `prep` decodes the slab's tap(s) once, `issue_part(j)` issues load j of the
    // wave (j < AL: 8 rows of A, else 8 rows of B).
    unsigned ut_tap = 0, ut_tap_bytes = 0;              // UT: wave-uniform, scalar registers
    unsigned b_k_bytes = 0;                              // byte offset of the slab inside a B row (wave-uniform)
    int tap_off[2] = {0, 0}, tap_h[2] = {0, 0}, tap_w[2] = {0, 0};
    bool kvalid[2] = {false, false};
    auto prep = [&](int k0) {
        b_k_bytes = BKN ? (unsigned)k0 * (unsigned)p.bt_ld * 4u : (unsigned)k0 * (unsigned)sizeof(T);
        if (UT) {
            unsigned c0, th, tw;
            p.div_c.divmod((unsigned)k0, ut_tap, c0);
            p.div_tw.divmod(ut_tap, th, tw);
            ut_tap_bytes = (unsigned)(((int)th * p.Ws + (int)tw) * p.Cs + (int)c0) * (unsigned)sizeof(T);
            if (!BKN && p.bt_direct)                     // the filter itself: tap (th, tw) of this class, channels c0..
                b_k_bytes = (unsigned)(((p.bd_xa + p.bd_xs * (int)th) * p.bd_fw + p.bd_ya + p.bd_ys * (int)tw) * p.bd_tap_elems +
                                       (int)c0) * (unsigned)sizeof(T);
            if (BKN && p.bt_kn == 2)                     // a part of an fprop: its tap (th, tw) is the filter's tap (bd_xa + th, bd_ya + tw)
                b_k_bytes = (unsigned)(((p.bd_xa + (int)th) * p.bd_fw + p.bd_ya + (int)tw) * p.Cs + (int)c0) * (unsigned)p.bt_ld * 4u;
            if constexpr (SA) cur_mask = (unsigned)__builtin_amdgcn_ballot_w64(((aux_row >> ut_tap) & 1u) != 0u);
            return;
        }
        // tap decode for the two chunk columns a lane serves (even / odd 8-row blocks)
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            int kk = k0 + CE * (k4e ^ (q ? ODD : 0));
            unsigned tap, c, th, tw;
            p.div_c.divmod((unsigned)kk, tap, c);
            p.div_tw.divmod(tap, th, tw);
            kvalid[q] = kk < p.K;
            tap_h[q] = (int)th;
            tap_w[q] = (int)tw;
            tap_off[q] = ((int)th * p.Ws + (int)tw) * p.Cs + (int)c;
        }
    };
    auto issue_load = [&](int j, int k0, f4* la, f4* lb) {
        if constexpr (SA) {
            if (j >= AL) {
                const int i = j - AL;
                lds_direct_load16_s(sa_rsrc_b, lds_address(lb) + (unsigned)(wave_u * BL + i) * 1024u, b_off[i], b_k_bytes);
                return;
            }
            // the load's 8 (16 with half-depth slabs) rows of the mask, a bit per row
            const unsigned m8 = (cur_mask >> (RPL * j)) & ((1u << RPL) - 1u);
            const unsigned dst = lds_address(la) + (unsigned)(wave_u * AL + j) * 1024u;
            if (m8 != 0u) lds_direct_load16_s(sa_rsrc_a, dst, select_by_mask(a_byte[j], 0x80000000u, spread_rows<KC>(m8)), ut_tap_bytes);
            else lds_direct_load16_s(sa_rsrc_a, dst, a_byte[j], ut_tap_bytes);
            return;
        }
        if (j >= AL) {
            const int i = j - AL;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (lds_ptr_t)(lb + (wave * BL + i) * 64), 16,
                                                     (int)(b_off[i] + b_k_bytes), 0, 0, 0);
            return;
        }
        const int i = j;
        unsigned voff;
        if (UT) {
            const unsigned bad = (a_inv[i] >> ut_tap) & 1u;
            voff = (a_byte[i] + ut_tap_bytes) | (bad << 31);
        } else {
            const int q = i & 1;                        // AL is even: block parity = i & 1
            int r = (base_rc[i] >> 16) + tap_h[q];
            int cc = ((int)((unsigned)base_rc[i] << 16) >> 16) + tap_w[q];
            // bitwise, not short-circuit: keeps the slab issue free of branches
            const unsigned bad =
                (unsigned)!(kvalid[q] & ((unsigned)r < (unsigned)p.Hs) & ((unsigned)cc < (unsigned)p.Ws));
            voff = ((unsigned)(base_off[i] + tap_off[q]) * (unsigned)sizeof(T)) | (bad << 31);
        }
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (lds_ptr_t)(la + (wave * AL + i) * 64), 16, (int)voff, 0, 0, 0);
    };
    constexpr int NL = AL + BL;                          // loads per wave per slab
    constexpr int LPG = (NL + G - 2) / (G - 1);          // spread over all MFMA groups but the last
    auto issue_part = [&](int g, int k0, f4* la, f4* lb) {
#pragma unroll
        for (int j = g * LPG; j < (g + 1) * LPG && j < NL; ++j) issue_load(j, k0, la, lb);
    };
    auto issue = [&](int k0, f4* la, f4* lb) {
        prep(k0);
#pragma unroll
        for (int j = 0; j < NL; ++j) issue_load(j, k0, la, lb);
    };

    // split K (launches with few tiles and a long K, e.g. a dense layer on a small batch):
    // blockIdx.y walks its own range of slabs and writes a partial product; the bias goes
    // into split 0 and `reduce_splits` adds the partials in order
    f16v acc[TM][TN];

    const int sw7 = (l32 >> SH) & (KC - 1);    // swizzle of every operand row this lane reads
    f4 fa[2][TM], fb[2][TN];                   // operand fragments, double buffered across k groups
    auto read_frags = [&](const f4* la, const f4* lb, int g, int slot) {
        const int pc = (2 * g + lh) ^ sw7;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[slot][i] = la[(wm0 + 32 * i + l32) * KC + pc];
        if constexpr (BKN) {
            // k = 8 g + 4 lh + t for t = 0..3: rows of BN floats; odd rows of a 64-wide slab have their halves swapped
            const float* lbf = reinterpret_cast<const float*>(lb) + (8 * g + 4 * lh) * BN;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = RUNS ? wn0 + TN * l32 + j : wn0 + 32 * j + l32;   // (runs: a lane's blocks hold neighbouring channels)
#pragma unroll
                for (int t = 0; t < 4; ++t) fb[slot][j][t] = lbf[t * BN + (n ^ ((BN == 64 && (t & 1)) ? 32 : 0))];
            }
            return;
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[slot][j] = lb[(wn0 + 32 * j + l32) * KC + pc];
    };
    auto mma_group = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (RUNS) mma_chunk<T>(fa[slot][i], fb[slot][j], acc[i][j]);
                else mma_chunk<T>(fb[slot][j], fa[slot][i], acc[i][j]);
            }
    };
    // One slab: the first operand reads go out right after the barrier, then the
    // loads of the next slab are issued (their address arithmetic overlaps the LDS
    // latency), then each k group's MFMAs run while the next group's operands load.
    auto slab = [&](const f4* la, const f4* lb, f4* na, f4* nb, int next_k0, bool has_next) {
        __builtin_amdgcn_s_waitcnt(0);         // this wave's loads of the slab have landed
        __syncthreads();                       // everyone's have; everyone is done reading the other buffer
        read_frags(la, lb, 0, 0);
        if (has_next) prep(next_k0);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (g < G - 1) read_frags(la, lb, g + 1, (g + 1) & 1);
            if constexpr (SA && TM * TN * (G - 1) >= NL) {
                // one load in front of each run of 4 MFMAs; consecutive MFMAs go to different accumulator blocks
                __builtin_amdgcn_sched_barrier(0);
                static_assert(TM * TN == 2 || TM * TN == 1 || TM * TN == 4, "blocks per wave");
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int c = g * TM * TN + (t * TM * TN) / 4;
                    if (has_next && c < NL && (t * TM * TN) % 4 == 0) issue_load(c, next_k0, na, nb);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j) {
                            if constexpr (RUNS) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[g & 1][i][t], fb[g & 1][j][t], acc[i][j], 0, 0, 0);
                            else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[g & 1][j][t], fa[g & 1][i][t], acc[i][j], 0, 0, 0);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                if (has_next && g < G - 1) issue_part(g, next_k0, na, nb);
                // keep the prefetch ahead of the MFMAs (the scheduler would otherwise sink
                // the reads next to their first use and expose the LDS latency)
                __builtin_amdgcn_sched_barrier(0);
                mma_group(g & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    if constexpr (NLOOP) {
        // A (at most two slabs) stays in the two A buffers; the B slabs of all n tiles pass
        // through the two B buffers as one double-buffered sequence f = (n tile, slab):
        // the loads of step f+1 fly while step f is multiplied.
        const int nslabs = p.Kpad / BK;                // 1 or 2
        const int total = ntile * nslabs;
        // the bias of every n tile, kept in LDS: a tile's accumulators start from it without a
        // global load between the steps (tile 0 takes the registers fetched above)
        __shared__ __attribute__((aligned(16))) float lds_bias[kNloopMaxN];
        float bias_mine[kNloopMaxN / kThreads];
#pragma unroll
        for (int i = 0; i < kNloopMaxN / kThreads; ++i) {
            const int n = i * kThreads + tid;
            bias_mine[i] = (p.bias != nullptr && n < p.N) ? p.bias[n] : 0.f;
        }
        prep(0);
#pragma unroll
        for (int j = 0; j < AL; ++j) issue_load(j, 0, lds_a0, lds_b0);
        if (nslabs > 1) {
            prep(BK);
#pragma unroll
            for (int j = 0; j < AL; ++j) issue_load(j, BK, lds_a1, lds_b1);
        }
        b_k_bytes = 0;
#pragma unroll
        for (int j = AL; j < NL; ++j) issue_load(j, 0, lds_a0, lds_b0);         // B of step 0
        fill_acc<TM, TN>(bv, acc);
#pragma unroll
        for (int i = 0; i < kNloopMaxN / kThreads; ++i) lds_bias[i * kThreads + tid] = bias_mine[i];
        // One step.  `first_slab` / `last_slab`: this slab begins / completes an n tile.
        // A finished tile is copied to `done` and stored at the beginning of the next step,
        // after that step's loads are issued: the stores then have a whole step to drain
        // before the next wait.  (Waiting for "all but the stores" is not possible: loads
        // and stores of a wave may complete out of order with respect to each other, and
        // stores issued at the end of a step are waited for in full by the next one.)
        f16v done[TM][TN];
        auto step = [&](int f, const f4* la, const f4* lb, f4* nb, bool first_slab, bool last_slab) __attribute__((always_inline)) {
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            read_frags(la, lb, 0, 0);
            const int tile_now = n0;
            const bool more = f + 1 < total;
            const bool pending = first_slab && f > 0;     // the tile before this one waits in `done`
            if (pending) {
                // before this step's loads are issued: with an LDS-direct load in flight the
                // compiler makes every other LDS read wait for it
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f4 v = *reinterpret_cast<const f4*>(lds_bias + tile_now + wn0 + 32 * j + 8 * q + 4 * lh);
#pragma unroll
                        for (int i = 0; i < TM; ++i)
#pragma unroll
                            for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = v[e];
                    }
            }
            if (more) {
                const int fn = f + 1;
                const int nt_next = nslabs == 2 ? fn >> 1 : fn;
                const int k0_next = nslabs == 2 ? (fn & 1) * BK : 0;
                n0 = nt_next * BN;
                set_b_off();
                b_k_bytes = (unsigned)k0_next * (unsigned)sizeof(T);     // (the packed filter: this mode never reads w itself)
#pragma unroll
                for (int j = AL; j < NL; ++j) issue_load(j, k0_next, lds_a0, nb);
            }
            if (pending) store_tile<TM, TN, true>(p, p.out, done, m0 + wm0, tile_now - BN + wn0, l32, lh);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (g < G - 1) read_frags(la, lb, g + 1, (g + 1) & 1);
                __builtin_amdgcn_sched_barrier(0);
                mma_group(g & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (last_slab) {
                if (more) {
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j) done[i][j] = acc[i][j];
                } else {
                    store_tile<TM, TN, true>(p, p.out, acc, m0 + wm0, tile_now + wn0, l32, lh);
                }
            }
        };
        if (nslabs == 2) {
            for (int f = 0; f < total; f += 2) {
                step(f, lds_a0, lds_b0, lds_b1, true, false);
                step(f + 1, lds_a1, lds_b1, lds_b0, false, true);
            }
        } else {
            for (int f = 0; f < total; f += 2) {
                step(f, lds_a0, lds_b0, lds_b1, true, true);
                if (f + 1 < total) step(f + 1, lds_a0, lds_b1, lds_b0, true, true);
            }
        }
        return;
    }

    int s_begin = 0, nslabs = p.Kpad / BK;
    if (p.split_slabs > 0) {
        s_begin = split * p.split_slabs;
        if (s_begin + p.split_slabs < nslabs) nslabs = s_begin + p.split_slabs;
    }
    if (s_begin < nslabs) issue(s_begin * BK, lds_a0, lds_b0);
    if constexpr (RUNS) {
        // a lane's accumulators of block j all belong to channel n0 + wn0 + TN l32 + j
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + wn0 + TN * l32 + j;
            const float bj = (split == 0 && p.bias != nullptr && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = bj;
        }
    } else {
        fill_acc<TM, TN>(bv, acc);
    }
    for (int s = s_begin; s < nslabs; s += 2) {
        slab(lds_a0, lds_b0, lds_a1, lds_b1, (s + 1) * BK, s + 1 < nslabs);
        if (s + 1 < nslabs) slab(lds_a1, lds_b1, lds_a0, lds_b0, (s + 2) * BK, s + 2 < nslabs);
    }

    if constexpr (RUNS && TN == 1) store_tile_lines<TM, TN>(p, p.out + (size_t)split * p.M * p.N, acc, m0 + wm0, n0 + wn0, l32, lh, p.M);
    else if constexpr (RUNS) store_tile_runs<TM, TN>(p, p.out + (size_t)split * p.M * p.N, acc, m0 + wm0, n0 + wn0, l32, lh, p.M);
    else store_tile<TM, TN>(p, p.out + (size_t)split * p.M * p.N, acc, m0 + wm0, n0 + wn0, l32, lh);
}

template <typename T, int BM, int BN, int WM, int WN, bool UT, int KC, bool NLOOP, bool SA = false, bool RUNS = false, bool BKN = false>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN)) void gather_gemm_dma(const GatherParams p) {
    __shared__ f4 lds_a0[BM * KC];
    __shared__ f4 lds_a1[BM * KC];
    __shared__ f4 lds_b0[BN * KC];
    __shared__ f4 lds_b1[BN * KC];
    gather_gemm_dma_body<T, BM, BN, WM, WN, UT, KC, NLOOP, SA, RUNS, BKN>(p, launch_block(), lds_a0, lds_a1, lds_b0, lds_b1);
}

// ------------------------------------------------------------------------------
// gather_halo_bf16: unit-stride gathers with several filter taps on bf16 inputs
// (3x3 stride-1 fprop, every dgrad class with 2 taps or more).
// The bf16 MFMAs of a slab take a fifth of the time its LDS-direct loads need to
// arrive, and with the taps of a filter walked one slab at a time every source
// pixel is fetched once per tap (9 times for 3x3): gather_gemm_dma on these shapes
// waits for its loads (without the A loads of slabs 1..8 it runs 1.5x faster).
// Here a workgroup fetches the source pixels of its 256 output pixels ONCE, as a
// span of the zero-padded source tensor [S][Hp][Wp] in row-major order ("halo", 64
// channels = 128 B per pixel slot, at most kHaloSlots slots), and every tap reads it
// at a shifted slot:
//     slot(pixel (s, i, j), tap (th, tw)) = (s * Hp + i + th) * Wp + (j + tw) - first,
//     Hp = Hg + Th - 1, Wp = Wg + Tw - 1
// Padding pixels are slots the loads fill with zeros (offsets outside the buffer
// descriptor), so no tap needs a validity test.  Only the filter slabs stream, 8 KB
// per tap through a ring of three buffers, two taps ahead.
//   * A tile that runs over the end of an image needs (Th - 1) * Wp more slots.  Where
//     that does not fit (56x56: 500), tiles are cut per image and an image's last tile
//     is partly empty: taken when that costs at most 10 % of the rows; else tiles run
//     over all of M if every span fits; else gather_gemm_dma runs.
//   * a slot keeps logical 16-byte chunk c at position c ^ key, key from the number of the pixel it serves
//     (see the slot table below): 16 consecutive pixels cover the 64 banks once under every tap, row ends included;
//   * channel blocks beyond the first reload the halo (Cs = 64 j: j passes over the taps).
// ------------------------------------------------------------------------------
// STAGES ring buffers of 8 KB and the rest of 80 KB (two workgroups per CU) for the halo:
// 4 stages (three taps ahead) and 384 slots where every span fits that, else 3 and 448
// (56x56x64: 0.098 ms with 4 stages, 0.102 with 3).
constexpr int halo_slots(int stages) { return stages == 4 ? 384 : 448; }
// an LDS array of N 16-byte elements that takes no space for N == 0
template <int N> struct LdsBlock {
    static __device__ __forceinline__ f4* get() {
        __shared__ f4 block[N];
        return block;
    }
};
template <> struct LdsBlock<0> {
    static __device__ __forceinline__ f4* get() { return nullptr; }
};
constexpr int kHaloSlotsMax = 448;
constexpr int kHaloBM = 256;

// one tile of the kernel: `lid` numbers the (m tile, n tile) pairs of the problem p, n tiles first
template <int STAGES, bool LINES = false>
static __device__ __forceinline__ void halo_tile_bf16(const GatherParams& p, const int lid) {
    constexpr int BM = kHaloBM, BN = 64, TM = 2, TN = 2, KC = 8, BK = 64;
    constexpr int kHaloSlots = halo_slots(STAGES);
    constexpr int HL = kHaloSlots / 8 / 4;               // halo loads per wave (8 slots each)
    static_assert(STAGES == 3 || STAGES == 4, "ring of 3 or 4 filter slabs");
    __shared__ f4 halo[kHaloSlots * KC];
    __shared__ f4 ring0[BN * KC];
    __shared__ f4 ring1[BN * KC];
    __shared__ f4 ring2[BN * KC];
    f4* const ring3 = LdsBlock<STAGES == 4 ? BN * KC : 0>::get();    // no bytes when unused: 80 KB exactly either way
    f4* const ring_last = STAGES == 4 ? ring3 : ring2;
    static_assert(kHaloSlots * sizeof(int) <= sizeof(ring2), "slot table fits a ring buffer");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int wm0 = wave * 64;
    const int ntile = (p.N + BN - 1) / BN;
    const int mt = lid / ntile;
    const int n0 = (lid - mt * ntile) * BN;
    const int hw = p.Hg * p.Wg;
    int m0, m_end;                                       // the tile's rows and where its image (or M) ends
    if (p.halo_tiles > 0) {
        unsigned s_img, t_img;
        p.div_halo_tiles.divmod((unsigned)mt, s_img, t_img);
        m0 = (int)s_img * hw + (int)t_img * BM;
        m_end = ((int)s_img + 1) * hw;
    } else {
        m0 = mt * BM;
        m_end = p.M;
    }
    const int Wp = p.halo_wp, Hp = p.halo_hp;
    // slot of tap (0,0) of output pixel m in the padded source tensor
    auto slot0 = [&](int m) __attribute__((always_inline)) {
        unsigned s_, rem, ii, jj;
        p.div_hw.divmod((unsigned)m, s_, rem);
        p.div_w.divmod(rem, ii, jj);
        return ((int)s_ * Hp + (int)ii) * Wp + (int)jj;
    };
    const int T = p.Th * p.Tw;
    const int nsteps = (p.Cs / BK) * T;

    f4 bv[TN][4];
    load_bias<TN>(p, p.bias, bv, n0, lh);

    // the span: from the slot of tap (0,0) of the tile's first pixel to that of the last tap of its last pixel
    const int lfirst = slot0(m0);
    const int span = slot0(min(m0 + BM, m_end) - 1) + (p.Th - 1) * Wp + p.Tw - lfirst;   // <= kHaloSlots, checked by the host
    // slot -> byte offset of the pixel's channel 0 (bit 31: padding or past the span), one slot per
    // thread, through LDS to the lanes that fetch it.  The table sits in the last ring buffer, which
    // the filter loads reach after the first barrier of the loop.
    // Where a slot keeps its 16-byte chunks: chunk c at position c ^ key, key = bits 1..3 of the NUMBER OF THE PIXEL
    // the slot would be under tap (0, 0), v = (s Hg + row) Wg + column.  The 16 lanes of an operand read serve 16
    // consecutive pixels, and under any tap their slots have consecutive v, also across a row end, where the slot
    // numbers jump: parity (the slot's half of the banks; v and the slot number differ by an even amount, see the
    // host's choice of the pitches) and key are those of 16 consecutive numbers, all different.  (Keyed by the slot
    // number, rows of 14 pixels gave every read a pair of lanes 16 slots apart: 29 % of the LDS cycles were conflicts.)
    int* tab = reinterpret_cast<int*>(ring_last);
    int* tabkey = tab + kHaloSlots;
    static_assert(2 * kHaloSlots * sizeof(int) <= sizeof(ring2), "slot tables fit a ring buffer");
    for (int sl = tid; sl < kHaloSlots; sl += kThreads) {
        unsigned rg, cc, s_, rr;
        p.div_halo_wp.divmod((unsigned)(lfirst + sl), rg, cc);
        p.div_halo_hp.divmod(rg, s_, rr);
        const int srow = (int)rr + p.rh0, scol = (int)cc + p.rw0;
        const bool ok = sl < span && (unsigned)srow < (unsigned)p.Hs && (unsigned)scol < (unsigned)p.Ws && (int)s_ < p.S &&
                        (int)rr < p.Hg + p.Th - 1 && (int)cc < p.Wg + p.Tw - 1;                  // (not the idle slots of the pitch)
        const unsigned off = (unsigned)((((int)s_ * p.Hs + srow) * p.Ws + scol) * p.Cs) * 2u;
        tab[sl] = (int)(ok ? off : 0x80000000u);
        tabkey[sl] = ((((int)s_ * p.Hg + (int)rr) * p.Wg + (int)cc) >> 1) & 7;
    }
    __syncthreads();
    unsigned hoff[HL];
#pragma unroll
    for (int k = 0; k < HL; ++k) {
        const int sl = (wave * HL + k) * 8 + (lane >> 3);
        hoff[k] = (unsigned)tab[sl] + (unsigned)((((lane & 7) ^ tabkey[sl]) & 7) * 16);
    }
    // slot of tap (0,0) for the pixels this lane multiplies (rows past the end: slot 0, never stored), and their numbers
    int pslot[TM], pnum[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm0 + 32 * i + l32;
        pslot[i] = m < m_end ? slot0(m) - lfirst : 0;
        pnum[i] = m < m_end ? m : m0;
    }
    // filter slab loads: as in gather_gemm_dma (rows of 8 chunks, chunk c of row r at c ^ ((r >> 1) & 7))
    const int k4e = (lane & 7) ^ (lane >> 4);
    unsigned b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int k4 = k4e ^ (((wave * 2 + i) & 1) ? 4 : 0);
        // LINES: slab row r holds channel n0 + 2 (r % 32) + r / 32: a lane of the multiplying waves then owns two
        // neighbouring channels, one in each of its 32-column blocks (store_tile_runs)
        const int r = (wave * 2 + i) * 8 + (lane >> 3);
        const int n = LINES ? n0 + 2 * (r & 31) + (r >> 5) : n0 + r;
        b_off[i] = (unsigned)((n * p.bt_ld + 8 * k4) * 2);
    }
    const u32x4 rsrc_a = raw_rsrc(p.src, p.src_bytes);
    const u32x4 rsrc_b = raw_rsrc(p.bt, p.bt_bytes);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto load_halo = [&](int cb) __attribute__((always_inline)) {
        const unsigned base = lds_address(halo) + (unsigned)(wave_u * HL) * 1024u;
#pragma unroll
        for (int k = 0; k < HL; ++k) lds_direct_load16(rsrc_a, base + k * 1024u, hoff[k] + (unsigned)(cb * BK * 2));
    };
    // filter slab of step u = (channel block, tap): k0 = tap * Cs + 64 * block, as a byte offset
    auto load_filter = [&](unsigned k0_bytes, f4* lb) __attribute__((always_inline)) {
        const unsigned base = lds_address(lb) + (unsigned)(wave_u * 2) * 1024u;
#pragma unroll
        for (int i = 0; i < 2; ++i) lds_direct_load16(rsrc_b, base + i * 1024u, b_off[i] + k0_bytes);
    };
    // prefetch position: STAGES - 1 steps ahead of the one being multiplied.  Every step issues
    // exactly one slab, past the last step with an offset outside the descriptor (no memory
    // access): the wait of a step is then the same count in every step, without a branch
    // (with conditional loads the compiler cannot tell which loads a count leaves in
    // flight and waits for all of them before the first LDS read).
    int pf_tap = 0, pf_cb = 0;
    int pf_th = 0, pf_tw = 0;                            // the prefetched tap as (row, column) of the class
    auto pf_next = [&]() __attribute__((always_inline)) {
        // start of the slab inside a B row: packed filter k = tap * Cs + 64 * block; the filter itself (bt_direct):
        // tap (th, tw) of this class is w's tap (bd_xa + bd_xs th, bd_ya + bd_ys tw), whose rows hold the Cs channels
        const int k_elems = p.bt_direct
            ? ((p.bd_xa + p.bd_xs * pf_th) * p.bd_fw + p.bd_ya + p.bd_ys * pf_tw) * p.bd_tap_elems + pf_cb * BK
            : pf_tap * p.Cs + pf_cb * BK;
        const unsigned k0_bytes = pf_cb < p.Cs / BK ? (unsigned)k_elems * 2u : 0x80000000u;
        if (++pf_tw == p.Tw) { pf_tw = 0; ++pf_th; }
        if (++pf_tap == T) { pf_tap = 0; pf_th = 0; pf_tw = 0; ++pf_cb; }
        return k0_bytes;
    };
    load_halo(0);
    load_filter(pf_next(), ring0);
    load_filter(pf_next(), ring1);
    if constexpr (STAGES == 4) load_filter(pf_next(), ring2);

    f16v acc[TM][TN];
    if constexpr (LINES) {
        // a lane's accumulators of block j all belong to channel n0 + 2 l32 + j
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + 2 * l32 + j;
            const float bj = (p.bias != nullptr && n < p.N) ? p.bias[n] : 0.0f;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = bj;
        }
    } else {
        fill_acc<TM, TN>(bv, acc);
    }

    const int sw7 = (l32 >> 1) & 7;
    int th = 0, tw = 0, cb = 0;                          // the step being multiplied
    auto step = [&](int u, const f4* lb, f4* nb) __attribute__((always_inline)) {
        // loads complete in the order of issue (no stores are pending here): all but the
        // younger filter slabs (two loads each)
        __builtin_amdgcn_s_waitcnt((2 * (STAGES - 2)) | (7 << 4) | (15 << 8));
        // a bare barrier: the fence of __syncthreads() would wait for every load in flight
        asm volatile("s_barrier" ::: "memory");
        if (th == 0 && tw == 0 && cb > 0) {              // next channel block: everyone is done with the halo
            load_halo(cb);
            __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
            asm volatile("s_barrier" ::: "memory");
        }
        load_filter(pf_next(), nb);
        const int shift = th * Wp + tw, tapv = th * p.Wg + tw;
        int x0[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int sl = pslot[i] + shift;
            x0[i] = sl * 8 + ((lh ^ ((pnum[i] + tapv) >> 1)) & 7);
        }
        // all operand reads of the step go out at once (64 registers): with a read-ahead of one
        // k group the MFMAs of every group waited for LDS, whose queue under 8 waves of 16-byte
        // reads is longer than the four MFMAs that were meant to cover it
        f4 fa[4][TM], fb[4][TN];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[g][i] = halo[x0[i] ^ (g << 1)];
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[g][j] = lb[(32 * j + l32) * KC + ((2 * g + lh) ^ sw7)];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if (LINES) mma_chunk<uint16_t>(fa[g][i], fb[g][j], acc[i][j]);
                    else mma_chunk<uint16_t>(fb[g][j], fa[g][i], acc[i][j]);
                }
        __builtin_amdgcn_sched_barrier(0);
        if (++tw == p.Tw) { tw = 0; if (++th == p.Th) { th = 0; ++cb; } }
    };
    if constexpr (STAGES == 4) {
        for (int u = 0; u < nsteps; u += 4) {
            step(u, ring0, ring3);
            if (u + 1 < nsteps) step(u + 1, ring1, ring0);
            if (u + 2 < nsteps) step(u + 2, ring2, ring1);
            if (u + 3 < nsteps) step(u + 3, ring3, ring2);
        }
    } else {
        for (int u = 0; u < nsteps; u += 3) {
            step(u, ring0, ring2);
            if (u + 1 < nsteps) step(u + 1, ring1, ring0);
            if (u + 2 < nsteps) step(u + 2, ring2, ring1);
        }
    }
    if (LINES) store_tile_runs<TM, TN>(p, p.out, acc, m0 + wm0, n0, l32, lh, m_end);
    else store_tile<TM, TN>(p, p.out, acc, m0 + wm0, n0, l32, lh, m_end);
}

template <int STAGES, bool LINES = false>
static __global__ __launch_bounds__(kThreads, 2) void gather_halo_bf16(const GatherParams p) {
    halo_tile_bf16<STAGES, LINES>(p, xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x));
}

// The stride classes of one dgrad (2 or 4 problems over the same dy, each writing its own pixels of dx) as one
// launch.  All classes have the same pixel grid and therefore the same tiles; the workgroups of one m tile, all
// classes and n tiles, have consecutive logical ids: they run on one XCD at about the same time and the tile's
// span of dy comes from memory once instead of once per class launch.
constexpr int kMaxClasses = 4;
struct GatherClasses {
    GatherParams cls[kMaxClasses];
    int ncls;
};
// fp32: the problems of a dgrad or an fprop (stride classes, or the parts that classes and fprops are cut into along their
// borders) whose launches would all be the 128 x 64 slab kernel, in ONE launch.  Problem c owns the workgroups [start[c], start[c] +
// blocks[c]); every start is a multiple of the XCD count, so that a workgroup sits on the XCD it would sit on in a launch of
// its problem alone, and the workgroups that pad a problem do nothing.  The host puts the problems with the most taps first:
// the short ones fill the tail of the long ones, where a launch each leaves the GPU part empty every time.
constexpr int kMaxClassesF32 = 9;            // (the nine parts of a 3x3 "same" convolution at unit stride: one launch)
struct GatherClassesF32 {
    GatherParams cls[kMaxClassesF32];     // (the first kernel argument: the kernel reads it from the argument segment)
    int ncls;
};
struct ClassGrid {
    unsigned start[kMaxClassesF32];
    unsigned blocks[kMaxClassesF32];
};
template <bool RUNS, bool BKN = false>
static __global__ __launch_bounds__(kThreads) void gather_classes_f32(const GatherClassesF32 q, const ClassGrid cg) {
    __shared__ f4 lds_a0[128 * 8];
    __shared__ f4 lds_a1[128 * 8];
    __shared__ f4 lds_b0[64 * 8];
    __shared__ f4 lds_b1[64 * 8];
    const unsigned b = blockIdx.x;
    int c = 0;
    unsigned start = cg.start[0], blocks = cg.blocks[0];
#pragma unroll
    for (int i = 1; i < kMaxClassesF32; ++i)
        if (i < q.ncls && b >= cg.start[i]) {
            c = i;
            start = cg.start[i];
            blocks = cg.blocks[i];
        }
    const unsigned idx = b - start;
    if (idx >= blocks) return;
    // The problem's parameters are read where the launch put them, in the kernel argument segment (`q` is the first argument):
    // scalar loads at a wave-uniform address.  Indexing the by-value copy with a run-time index would go through per-lane memory.
    typedef __attribute__((address_space(4))) const GatherParams* const_params_t;
    const_params_t args = (const_params_t)__builtin_amdgcn_kernarg_segment_ptr();
    GatherParams p = q.cls[0];
    __builtin_memcpy(&p, (const void*)(args + c), sizeof(p));
    gather_gemm_dma_body<float, 128, 64, 32, 64, true, 8, false, true, RUNS, BKN>(p, BlockId{(int)idx, 0, (int)blocks}, lds_a0, lds_a1, lds_b0,
                                                                                  lds_b1);
}

template <int STAGES, bool LINES = false>
static __global__ __launch_bounds__(kThreads, 2) void gather_halo_classes_bf16(const GatherClasses q) {
    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int ntile = (q.cls[0].N + 63) / 64;
    const int grp = lid / ntile, nt = lid - grp * ntile;
    const int mt = grp / q.ncls, c = grp - mt * q.ncls;
    halo_tile_bf16<STAGES, LINES>(q.cls[c], mt * ntile + nt);
}

// ------------------------------------------------------------------------------
// gather_halo_pairs_bf16: gather_halo_bf16 for the stride classes of one dgrad, two classes per workgroup.
// The classes' taps are windows of one padded source tensor (class c's tap (th, tw) is the window at
// (th + tap_dh, tw + tap_dw)), so one halo per channel block serves both classes of a pair: 4 or 5 steps per halo
// instead of 1 to 4, half the halo loads, and the wait for a halo (nothing else to do in that workgroup; the other
// workgroup of the CU fills the gap) comes half as often.  The pixels are the MFMAs' first operand and the tiles go
// out in 4-byte stores of whole lines (store_tile_lines).  All classes read the filter in place (one descriptor).
// ------------------------------------------------------------------------------
template <int STAGES, bool NT>
static __global__ __launch_bounds__(kThreads, 2) void gather_halo_pairs_bf16(const GatherClasses q) {
    constexpr int BM = kHaloBM, BN = 64, TM = 2, TN = 2, KC = 8, BK = 64, CPP = 2;
    constexpr int kHaloSlots = halo_slots(STAGES);
    constexpr int HL = kHaloSlots / 8 / 4;               // halo loads per wave (8 slots each)
    __shared__ f4 halo[kHaloSlots * KC];
    __shared__ f4 ring[STAGES][BN * KC];
    static_assert(kHaloSlots * sizeof(int) <= sizeof(ring[0]), "slot table fits a ring buffer");

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int wm0 = wave * 64;
    const GatherParams& p0 = q.cls[0];                   // what all classes have in common: source, pixel grid, halo geometry, N
    const int npass = q.ncls / CPP;
    const int ntile = (p0.N + BN - 1) / BN;
    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int grp = lid / ntile;
    const int n0 = (lid - grp * ntile) * BN;
    const int mt = grp / npass, pass = grp - mt * npass;
    const GatherParams& pa = q.cls[pass * CPP];
    const GatherParams& pb = q.cls[pass * CPP + 1];
    const int m0 = mt * BM, m_end = p0.M;
    const int Wp = p0.halo_wp, Hp = p0.halo_hp;
    auto slot0 = [&](int m) __attribute__((always_inline)) {
        unsigned s_, rem, ii, jj;
        p0.div_hw.divmod((unsigned)m, s_, rem);
        p0.div_w.divmod(rem, ii, jj);
        return ((int)s_ * Hp + (int)ii) * Wp + (int)jj;
    };
    const int ncb = p0.Cs / BK;
    const int Ta = pa.Th * pa.Tw, Tb = pb.Th * pb.Tw;
    const int nsteps = ncb * (Ta + Tb);

    const int lfirst = slot0(m0);
    const int span = slot0(min(m0 + BM, m_end) - 1) + (p0.halo_th - 1) * Wp + p0.halo_tw - lfirst;   // <= kHaloSlots, checked by the host
    // Where a slot keeps its 16-byte chunks: chunk c at position c ^ key, key = bits 1..3 of the NUMBER OF THE PIXEL
    // the slot would be under tap (0, 0), v = (s Hg + row) Wg + column.  The 16 lanes of an operand read serve 16
    // consecutive pixels, and under any tap their slots have consecutive v, also across a row end, where the slot
    // numbers jump: parity (the slot's half of the banks; v and the slot number differ by an even amount, see the
    // host) and key are those of 16 consecutive numbers, all different.  (Keyed by the slot number, rows of 14
    // pixels gave every read a pair of lanes 16 slots apart: 29 % of the LDS cycles were conflicts.)
    int* tab = reinterpret_cast<int*>(&ring[STAGES - 1][0]);             // the filter loads reach it after the first barrier of the loop
    int* tabkey = tab + kHaloSlots;
    static_assert(2 * kHaloSlots * sizeof(int) <= sizeof(ring[0]), "slot tables fit a ring buffer");
    for (int sl = tid; sl < kHaloSlots; sl += kThreads) {
        unsigned rg, cc, s_, rr;
        p0.div_halo_wp.divmod((unsigned)(lfirst + sl), rg, cc);
        p0.div_halo_hp.divmod(rg, s_, rr);
        const int srow = (int)rr + p0.rh0, scol = (int)cc + p0.rw0;
        const bool ok = sl < span && (unsigned)srow < (unsigned)p0.Hs && (unsigned)scol < (unsigned)p0.Ws && (int)s_ < p0.S &&
                        (int)rr < p0.Hg + p0.halo_th - 1 && (int)cc < p0.Wg + p0.halo_tw - 1;    // (not the idle slots of the pitch)
        const unsigned off = (unsigned)((((int)s_ * p0.Hs + srow) * p0.Ws + scol) * p0.Cs) * 2u;
        tab[sl] = (int)(ok ? off : 0x80000000u);
        tabkey[sl] = ((((int)s_ * p0.Hg + (int)rr) * p0.Wg + (int)cc) >> 1) & 7;
    }
    __syncthreads();
    unsigned hoff[HL];
#pragma unroll
    for (int k = 0; k < HL; ++k) {
        const int sl = (wave * HL + k) * 8 + (lane >> 3);
        hoff[k] = (unsigned)tab[sl] + (unsigned)((((lane & 7) ^ tabkey[sl]) & 7) * 16);
    }
    int pslot[TM], pnum[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm0 + 32 * i + l32;
        pslot[i] = m < m_end ? slot0(m) - lfirst : 0;
        pnum[i] = m < m_end ? m : m0;                    // (a row past the end reads slot 0, whose key is that of pixel m0)
    }
    // filter slab loads: rows of 8 chunks, chunk c of row r at c ^ ((r >> 1) & 7); the filter itself, rows n of bt_ld elements
    const int k4e = (lane & 7) ^ (lane >> 4);
    unsigned b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int k4 = k4e ^ (((wave * 2 + i) & 1) ? 4 : 0);
        // slab row r holds channel n0 + 2 (r % 32) + r / 32: a lane of the multiplying waves then owns two neighbouring
        // channels, one in each of its 32-column blocks (store_tile_lines2)
        const int r = (wave * 2 + i) * 8 + (lane >> 3);
        b_off[i] = (unsigned)(((n0 + 2 * (r & 31) + (r >> 5)) * p0.bt_ld + 8 * k4) * 2);
    }
    const u32x4 rsrc_a = raw_rsrc(p0.src, p0.src_bytes);
    const u32x4 rsrc_b = raw_rsrc(p0.bt, p0.bt_bytes);
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    auto load_halo = [&](int cb) __attribute__((always_inline)) {
        const unsigned base = lds_address(halo) + (unsigned)(wave_u * HL) * 1024u;
#pragma unroll
        for (int k = 0; k < HL; ++k) lds_direct_load16(rsrc_a, base + k * 1024u, hoff[k] + (unsigned)(cb * BK * 2));
    };
    auto load_filter = [&](unsigned k0_bytes, int slot) __attribute__((always_inline)) {
        const unsigned base = lds_address(&ring[slot][0]) + (unsigned)(wave_u * 2) * 1024u;
#pragma unroll
        for (int i = 0; i < 2; ++i) lds_direct_load16(rsrc_b, base + i * 1024u, b_off[i] + k0_bytes);
    };
    // the slab fetched next, STAGES - 1 steps ahead of the one being multiplied: channel block, class of the pair, tap.
    // Every step issues exactly one slab, past the last step with an offset outside the descriptor.
    int pf_cb = 0, pf_ci = 0, pf_th = 0, pf_tw = 0;
    auto pf_next = [&]() __attribute__((always_inline)) {
        const GatherParams& pc = pf_ci ? pb : pa;
        const int k_elems = ((pc.bd_xa + pc.bd_xs * pf_th) * pc.bd_fw + pc.bd_ya + pc.bd_ys * pf_tw) * pc.bd_tap_elems + pf_cb * BK;
        const unsigned k0_bytes = pf_cb < ncb ? (unsigned)k_elems * 2u : 0x80000000u;
        if (++pf_tw == pc.Tw) {
            pf_tw = 0;
            if (++pf_th == pc.Th) {
                pf_th = 0;
                if (++pf_ci == CPP) { pf_ci = 0; ++pf_cb; }
            }
        }
        return k0_bytes;
    };
    load_halo(0);
#pragma unroll
    for (int sgi = 0; sgi < STAGES - 1; ++sgi) load_filter(pf_next(), sgi);

    f16v acc[CPP][TM][TN];
#pragma unroll
    for (int ci = 0; ci < CPP; ++ci)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[ci][i][j][v] = 0.0f;

    const int sw7 = (l32 >> 1) & 7;
    int u = 0;
    auto step = [&](int shift, int tapv, f16v (&a)[TM][TN], bool new_block, int cb) __attribute__((always_inline)) {
        // loads complete in the order of issue (no stores are pending here): all but the younger filter slabs (two loads each)
        __builtin_amdgcn_s_waitcnt((2 * (STAGES - 2)) | (7 << 4) | (15 << 8));
        asm volatile("s_barrier" ::: "memory");
        if (new_block) {                                 // next channel block: everyone is done with the halo
            load_halo(cb);
            __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
            asm volatile("s_barrier" ::: "memory");
        }
        const int rb = u % STAGES;
        load_filter(pf_next(), rb == 0 ? STAGES - 1 : rb - 1);
        const f4* lb = ring[rb];
        ++u;
        int x0[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int sl = pslot[i] + shift;
            x0[i] = sl * 8 + ((lh ^ ((pnum[i] + tapv) >> 1)) & 7);
        }
        f4 fa[4][TM], fb[4][TN];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[g][i] = halo[x0[i] ^ (g << 1)];
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[g][j] = lb[(32 * j + l32) * KC + ((2 * g + lh) ^ sw7)];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) mma_chunk<uint16_t>(fa[g][i], fb[g][j], a[i][j]);
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int cb = 0; cb < ncb; ++cb) {
        bool first = cb > 0;
        {
            const int shift0 = pa.tap_dh * Wp + pa.tap_dw, v0 = pa.tap_dh * p0.Wg + pa.tap_dw;
            for (int th = 0; th < pa.Th; ++th)
                for (int tw = 0; tw < pa.Tw; ++tw) {
                    step(shift0 + th * Wp + tw, v0 + th * p0.Wg + tw, acc[0], first, cb);
                    first = false;
                }
        }
        {
            const int shift0 = pb.tap_dh * Wp + pb.tap_dw, v0 = pb.tap_dh * p0.Wg + pb.tap_dw;
            for (int th = 0; th < pb.Th; ++th)
                for (int tw = 0; tw < pb.Tw; ++tw) step(shift0 + th * Wp + tw, v0 + th * p0.Wg + tw, acc[1], false, cb);
        }
    }
    (void)nsteps;
    store_tile_lines2<TM, NT>(pa, pa.out, acc[0], m0 + wm0, n0, l32, lh, m_end);
    store_tile_lines2<TM, NT>(pb, pb.out, acc[1], m0 + wm0, n0, l32, lh, m_end);
}

struct PackParams {
    const void* w;
    void* bt;
    int fW, C, D;
    int Tw, Ck;
    int xa, xs, ya, ys;
    int transposed;
    int N, K, Npad, Kpad;
    int64_t w_elems;     // fH * fW * C * D
};

// ------------------------------------------------------------------------------
// gather_halo_res_bf16: the halo gather for filters that fit LDS whole (at most 9 taps of 64 x 64
// bf16 = 72 KB: 3x3 on 64 channels), as one persistent workgroup of 8 waves per CU.
// gather_halo_bf16 pays per tile for a set-up, the latency of its halo and a store phase, each with
// the matrix pipe idle in that workgroup, and its filter slabs queue behind the other workgroup's
// stores in the CU's memory pipeline.  Here the filter is fetched once per workgroup, wave 7 does
// nothing but fetch the halo of the NEXT tile (two halo buffers) and waves 0..6 multiply the current
// one, 32 rows x 64 columns each, straight out of LDS: no wait on memory inside a tile, one barrier
// per tile, and since the multiplying waves issue no loads, nothing they wait for sits behind their
// stores.
// Tiles are 224 rows = whole image rows (Wg divides 224: 4 rows of 56) of one image (its last tile
// may be short), so every tile starts in column 0: where a slot lies relative to the tile's first
// pixel, and whether it is a padding column, is the same for all tiles and worked out once per
// lane; per tile only the rows above and below the image change.
// ------------------------------------------------------------------------------
constexpr int kResBM = 224;
constexpr int kResThreads = 512;
constexpr int kResSlots = 352;        // 2 x 352 x 128 B of halo + 72 KB of filter = 160 KB
constexpr int kResMaxTaps = 9;

// RUNS: the pixels are the MFMAs' first operand and slab row r of the filter holds channel 2 (r % 32) + r / 32, so that a lane
// owns two neighbouring channels of 16 pixels and 32 lanes write the 256 contiguous bytes of a pixel with one 8-byte store
// each (store_tile_runs, whole lines, non-temporal) instead of 64 pieces of 16 bytes in 32 lines per instruction; same bits.
template <bool RUNS>
static __global__ __launch_bounds__(kResThreads, 1) void gather_halo_res_bf16(const GatherParams p, const PackParams pk,
                                                                               const int mtiles) {
    constexpr int BM = kResBM, BN = 64, TN = 2, KC = 8, NL = kResSlots / 8;
    __shared__ f4 filt[kResMaxTaps * BN * KC];
    __shared__ f4 halo[2][kResSlots * KC];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int G = (int)gridDim.x;
    const int lid = xcd_contiguous_id((int)blockIdx.x, G);
    // tiles of this workgroup: a contiguous run of them, so that a tile's upper halo rows are the
    // lower rows of the tile the same CU has just had in its L2
    const int per = (mtiles + G - 1) / G;
    const int tile0 = lid * per;
    const int ntl = max(0, min(per, mtiles - tile0));
    const int hw = p.Hg * p.Wg;
    const int Wp = p.halo_wp;
    const int T = p.Th * p.Tw;
    const int tile_rows = BM / p.Wg;                       // image rows per tile (the host checks BM % Wg == 0)

    // The filter, straight from w[fH][fW][C][D] (no packing launch): T slabs of 64 rows (n) x 128 B
    // (the 64 k of one tap), laid out like the slabs of gather_gemm_dma (chunk c of row r at
    // c ^ ((r >> 1) & 7)).  Slab t holds tap x = xa + xs * (t / Tw), y = ya + ys * (t % Tw).
    {
        const unsigned w_bytes = (unsigned)(pk.w_elems * 2);
        if (pk.transposed) {
            // dgrad: n is the input channel c and k the output channel d, which is contiguous in w:
            // rows are copied as they are; wave w fetches the 1 KB pieces w, w + 8, ...
            const u32x4 rsrc_w = raw_rsrc(pk.w, w_bytes);
            const int k4e = (lane & 7) ^ (lane >> 4);
            for (int q = wave; q < T * 8; q += 8) {
                const int tap = q >> 3, part = q & 7;
                unsigned t_h, t_w;
                p.div_tw.divmod((unsigned)tap, t_h, t_w);
                const int x = pk.xa + pk.xs * (int)t_h, y = pk.ya + pk.ys * (int)t_w;
                const int row = part * 8 + (lane >> 3);
                const int n = RUNS ? 2 * (row & 31) + (row >> 5) : row;           // the channel this slab row holds
                const int k4 = k4e ^ ((part & 1) ? 4 : 0);
                const unsigned off = (unsigned)((((x * pk.fW + y) * pk.C + n) * pk.D + 8 * k4) * 2) |
                                     ((unsigned)(n >= p.N) << 31);
                lds_direct_load16(rsrc_w, lds_address(filt) + (unsigned)q * 1024u, off);
            }
        } else {
            // fprop: n is the output channel d, contiguous in w, and k the input channel c: a
            // transposition.  Half a wave reads two adjacent n of two adjacent c (4 bytes each) and
            // writes the two (n, c pair) words; row pairs 2 (8 i + wave) + half of the T * 32 pairs.
            const __amdgpu_buffer_rsrc_t rsrc_w =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(pk.w), 0, (int)w_bytes, 0x00020000);
            const int n2 = 2 * (lane & 31);
            const unsigned nbad = (unsigned)(n2 >= p.N) << 31;             // N is even here (checked by the host)
            char* const fbytes = reinterpret_cast<char*>(filt);
#pragma unroll
            for (int i = 0; i < 2 * kResMaxTaps; ++i) {
                if (i < 2 * T) {
                    const int r = 2 * ((i * 8 + wave) * 2 + lh);                // row = tap * 64 + c, c even
                    const int tap = r >> 6, c = r & 63;
                    unsigned t_h, t_w;
                    p.div_tw.divmod((unsigned)tap, t_h, t_w);
                    const int x = pk.xa + pk.xs * (int)t_h, y = pk.ya + pk.ys * (int)t_w;
                    const unsigned off = (unsigned)((((x * pk.fW + y) * pk.C + c) * pk.D + n2) * 2) | nbad;
                    const unsigned a = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, (int)off, 0, 0);
                    const unsigned b = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, (int)off, pk.D * 2, 0);
                    // the slab rows of channels n2 and n2 + 1: neighbours, or (RUNS) rows n2 / 2 and n2 / 2 + 32; the same key either way
                    const int r0 = RUNS ? (n2 >> 1) : n2, r1 = RUNS ? (n2 >> 1) + 32 : n2 + 1;
                    const int pos = ((c >> 3) ^ ((r0 >> 1) & 7)) * 16 + (c & 7) * 2;
                    *reinterpret_cast<unsigned*>(fbytes + tap * 8192 + r0 * 128 + pos) = (a & 0xffffu) | (b << 16);
                    *reinterpret_cast<unsigned*>(fbytes + tap * 8192 + r1 * 128 + pos) = (a >> 16) | (b & 0xffff0000u);
                }
            }
        }
    }

    if (wave == 7) {
        // ---- the loading wave ----
        // Load i of a tile brings the 8 slots 8 i .. 8 i + 7 (lane / 8 picks the slot, lane % 8 the
        // chunk).  rel[i]: byte offset of the lane's chunk from the pixel of slot 0 (row -pad, column
        // -pad of the tile); colbad: bit i set where the slot is a padding column.  Per tile a slot is
        // valid if its padded row lies inside the image: slot in [lo, hi).  Offsets of invalid slots
        // get bit 31, outside the buffer descriptor: the load writes zeros.  The offsets of a tile are
        // worked out while the loads of the tile before it are in flight.
        const u32x4 rsrc_a = raw_rsrc(p.src, p.src_bytes);
        const int lslot = lane >> 3;
        int rel[NL];
        unsigned colbad_lo = 0, colbad_hi = 0;
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int sl = i * 8 + lslot;
            unsigned r, c;
            p.div_halo_wp.divmod((unsigned)sl, r, c);
            // chunk q of the slot sits at q ^ key, key from the number of the pixel the slot is under tap (0, 0), counted
            // from the tile's first pixel: the 16 lanes of an operand read serve 16 consecutive pixels, whose slots under
            // any tap have consecutive such numbers also where the slot numbers jump at a row end (see halo_tile_bf16)
            const int key = (((int)r * p.Wg + (int)c) >> 1) & 7;
            rel[i] = ((int)r * p.Ws + (int)c) * 128 + (((lane & 7) ^ key) & 7) * 16;
            const unsigned bad = ((unsigned)((int)c + p.rw0) >= (unsigned)p.Ws || (int)c >= p.Wg + p.Tw - 1) ? 1u : 0u;
            if (i < 32) colbad_lo |= bad << i;
            else colbad_hi |= bad << (i - 32);
        }
        unsigned offs[NL];
        auto addresses = [&](int tile) __attribute__((always_inline)) {
            unsigned s_img, t_img;
            p.div_halo_tiles.divmod((unsigned)tile, s_img, t_img);
            const int R0 = (int)t_img * tile_rows + p.rh0;                 // image row of padded row 0 of the tile
            const int base = (((int)s_img * p.Hs + R0) * p.Ws + p.rw0) * 128;
            const int a0 = lslot + R0 * Wp;                                // slot - lo, lo = -R0 * Wp
            const int b0 = (p.Hs - R0) * Wp - 1 - lslot;                   // hi - 1 - slot, hi = (Hs - R0) * Wp
#pragma unroll
            for (int i = 0; i < NL; ++i) {
                const unsigned rowbad = (unsigned)((a0 + 8 * i) | (b0 - 8 * i)) & 0x80000000u;
                const unsigned colbad = i < 32 ? (colbad_lo << (31 - i)) : (colbad_hi << (63 - i));
                offs[i] = (unsigned)(base + rel[i]) | rowbad | (colbad & 0x80000000u);
            }
        };
        auto issue = [&](int buf) __attribute__((always_inline)) {
            const unsigned lbase = lds_address(&halo[buf][0]);
#pragma unroll
            for (int i = 0; i < NL; ++i) lds_direct_load16(rsrc_a, lbase + (unsigned)i * 1024u, offs[i]);
        };
        if (ntl > 0) {
            addresses(tile0);
            issue(0);
        }
        if (ntl > 1) addresses(tile0 + 1);
        __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8));                // its loads and its part of the filter
        asm volatile("s_barrier" ::: "memory");
        for (int t = 0; t < ntl; ++t) {
            // the multiplying waves are done with tile t - 1, whose buffer takes tile t + 1
            if (t + 1 < ntl) issue((t + 1) & 1);
            if (t + 2 < ntl) addresses(tile0 + t + 2);
            __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));
            asm volatile("s_barrier" ::: "memory");
        }
        return;
    }

    // ---- the multiplying waves ----
    f4 bv[TN][4];
    load_bias<TN>(p, p.bias, bv, 0, lh);
    float bias_run[TN];                                                    // RUNS: the lane's channels 2 l32 + j
#pragma unroll
    for (int j = 0; j < TN; ++j) bias_run[j] = (RUNS && p.bias != nullptr && 2 * l32 + j < p.N) ? p.bias[2 * l32 + j] : 0.f;
    const int sw7 = (l32 >> 1) & 7;
    int pslot;                                                             // slot of tap (0,0) of this lane's row
    {
        unsigned r, c;
        p.div_w.divmod((unsigned)(wave * 32 + l32), r, c);
        pslot = (int)r * Wp + (int)c;
    }
    f16v done[1][TN];                                                      // the tile before the current one
    int done_m0 = 0, done_end = 0;
    bool have_done = false;
    const int store_after = min(wave + 1, T - 1);
    auto store_done = [&]() __attribute__((always_inline)) {
        if constexpr (RUNS) store_tile_runs<1, TN>(p, p.out, done, done_m0, 0, l32, lh, done_end);
        else store_tile<1, TN>(p, p.out, done, done_m0, 0, l32, lh, done_end);
    };
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8));                   // this wave's part of the filter
    asm volatile("s_barrier" ::: "memory");
    for (int t = 0; t < ntl; ++t) {
        unsigned s_img, t_img;
        p.div_halo_tiles.divmod((unsigned)(tile0 + t), s_img, t_img);
        const int m0 = (int)s_img * hw + (int)t_img * BM;
        const int m_end = ((int)s_img + 1) * hw;                           // rows past the image: multiplied, never stored
        const f4* h = halo[t & 1];
        f16v acc[1][TN];
        if constexpr (RUNS) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[0][j][v] = bias_run[j];
        } else {
            fill_acc<1, TN>(bv, acc);
        }
        // the operands of tap u + 1 are read while the MFMAs of tap u run (two sets of 48 registers)
        int th = 0, tw = 0;
        f4 fa[2][4], fb[2][4][TN];
        auto read_tap = [&](int tap, f4 (&ra)[4], f4 (&rb)[4][TN]) __attribute__((always_inline)) {
            const int sl = pslot + th * Wp + tw;
            const int x0 = sl * 8 + ((lh ^ ((wave * 32 + l32 + th * p.Wg + tw) >> 1)) & 7);
            const f4* lb = filt + tap * (BN * KC);
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                ra[g] = h[x0 ^ (g << 1)];
#pragma unroll
                for (int j = 0; j < TN; ++j) rb[g][j] = lb[(32 * j + l32) * KC + ((2 * g + lh) ^ sw7)];
            }
            if (++tw == p.Tw) { tw = 0; ++th; }
        };
        auto multiply = [&](const f4 (&ra)[4], const f4 (&rb)[4][TN]) __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if constexpr (RUNS) mma_chunk<uint16_t>(ra[g], rb[g][j], acc[0][j]);
                    else mma_chunk<uint16_t>(rb[g][j], ra[g], acc[0][j]);
                }
            __builtin_amdgcn_sched_barrier(0);
        };
        // All seven waves finish a tile together; if they also stored together, each would wait
        // for room in the CU's memory pipeline with nobody left to use the matrix pipe.  A wave
        // keeps its finished tile in registers and stores it during the next tile, wave w after
        // tap w + 1, so that the stores of a CU are spread over the tile.
        read_tap(0, fa[0], fb[0]);
        for (int tap = 0; tap < T; tap += 2) {
            if (tap + 1 < T) read_tap(tap + 1, fa[1], fb[1]);
            multiply(fa[0], fb[0]);
            if (tap == store_after && have_done) store_done();
            if (tap + 1 < T) {
                if (tap + 2 < T) read_tap(tap + 2, fa[0], fb[0]);
                multiply(fa[1], fb[1]);
                if (tap + 1 == store_after && have_done) store_done();
            }
        }
        have_done = true;
#pragma unroll
        for (int j = 0; j < TN; ++j) done[0][j] = acc[0][j];
        done_m0 = m0 + wave * 32;
        done_end = m_end;
        asm volatile("s_barrier" ::: "memory");
    }
    if (have_done) store_done();
}

// Packs the filter w[fH][fW][C][D] into bt[Npad][Kpad] (k contiguous) for one
// gather-GEMM launch.  k = (th*Tw + tw)*Ck + kc ; filter tap x = xa + xs*th,
// y = ya + ys*tw.  transposed == 0: n is the output channel d and kc the input
// channel c (fprop).  transposed == 1: n is c and kc is d (dgrad).
// ------------------------------------------------------------------------------
// dense_res_f32: y[M, N] = x[M, K] . w + bias in fp32 for a short K (one or two slabs: K = 32 or 64)
// and N up to 256 -- a 1x1 convolution that widens the channels (64 -> 256 on 56x56 images: 205 MB in,
// 822 MB out, 26 GFLOP: the fp32 matrix pipe and the memory system need about the same time).  The
// n-loop mode of gather_gemm_dma reaches 63 % of what a plain copy moves there: its waves wait for
// the loads of the next filter slab together with the stores of the tile before.  Here one
// persistent workgroup of 8 waves per CU keeps the whole packed filter in LDS (64 KB), walks tiles
// of 128 rows x N (wave = 64 x 64, two A buffers of 32 KB) and never waits for a store: wave 0
// fetches the A rows of the next tile at the start of a tile; a wave keeps its finished tile in
// registers and stores it during the next one, wave w after k group w of the 8, so that the stores
// of a CU are spread over the tile and those of wave 0 have long left when it waits for its loads.
// ------------------------------------------------------------------------------
constexpr int kD1BM = 128;
constexpr int kD1Threads = 512;
constexpr int kD1MaxN = 256;

// RUNS: the pixels are the MFMAs' first operand and slab row r of the filter holds channel (r / 64) 64 + 2 (r % 32) + (r % 64) / 32,
// so that a lane owns two neighbouring channels and a tile goes out in runs of 256 contiguous bytes per pixel (store_tile_runs).
template <int NSLAB, bool RUNS>                        // K = 32 * NSLAB
static __global__ __launch_bounds__(kD1Threads, 1) void dense_res_f32(const GatherParams p, const int mtiles) {
    constexpr int BM = kD1BM, KC = 8, TM = 2, TN = 2, nslab = NSLAB;
    __shared__ f4 filt[2][kD1MaxN * KC];                 // slab s: rows n of 128 B, chunk c at c ^ ((n >> 1) & 7)
    __shared__ f4 abuf[2][2][BM * KC];                   // [buffer][slab]
    __shared__ f4 bias_lds[kD1MaxN / 4];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int G = (int)gridDim.x;
    const int lid = xcd_contiguous_id((int)blockIdx.x, G);
    const int per = (mtiles + G - 1) / G;
    const int tile0 = lid * per;
    const int ntl = max(0, min(per, mtiles - tile0));
    const int wm0 = 64 * (wave & 1), wn0 = 64 * (wave >> 1);
    const bool active = wn0 < p.N;                       // wave-uniform

    // 1 KB pieces: 8 rows x 8 chunks, lane / 8 picks the row, lane % 8 the chunk position
    const int prow = lane >> 3;
    const int k4e = (lane & 7) ^ (lane >> 4);            // logical chunk at this position for even pieces (odd: ^ 4)
    {
        const u32x4 rsrc_b = raw_rsrc(p.bt, p.bt_bytes);
        const int pieces = kD1MaxN / 8;                  // per slab; rows past the packed filter read as zeros
        for (int q = wave; q < nslab * pieces; q += 8) {
            const int sl = q / pieces, part = q - sl * pieces;
            const int k4 = k4e ^ ((part & 1) ? 4 : 0);
            int r = part * 8 + prow;
            if constexpr (RUNS) r = (r & ~63) + 2 * (r & 31) + ((r >> 5) & 1);
            const unsigned off = (unsigned)((r * p.Kpad + 32 * sl + 4 * k4) * 4);
            lds_direct_load16(rsrc_b, lds_address(&filt[sl][0]) + (unsigned)part * 1024u, off);
        }
        if (tid < kD1MaxN / 4) {
            f4 b = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (p.bias != nullptr && 4 * tid + e < p.N) b[e] = p.bias[4 * tid + e];
            bias_lds[tid] = b;
        }
    }
    // A rows of a tile: 16 pieces per slab; rows past M lie outside the descriptor and read as zeros
    const u32x4 rsrc_a = raw_rsrc(p.src, p.src_bytes);
    unsigned rela[2][2];                                 // [slab][piece parity]: the lane's part of a piece's offset
#pragma unroll
    for (int sl = 0; sl < 2; ++sl)
#pragma unroll
        for (int o = 0; o < 2; ++o) rela[sl][o] = (unsigned)((prow * p.Cs + 32 * sl + 4 * (k4e ^ (o ? 4 : 0))) * 4);
    const unsigned piece_bytes = (unsigned)(8 * p.Cs * 4);
    auto fetch = [&](int tile, int buf) __attribute__((always_inline)) {
        const unsigned base = (unsigned)tile * (unsigned)(BM * p.Cs * 4);
#pragma unroll
        for (int i = 0; i < 2 * (BM / 8); ++i) {
            if (i < nslab * (BM / 8)) {
                const int sl = i / (BM / 8), part = i % (BM / 8);
                lds_direct_load16(rsrc_a, lds_address(&abuf[buf][sl][0]) + (unsigned)part * 1024u,
                                  base + (unsigned)part * piece_bytes + rela[sl][part & 1]);
            }
        }
    };
    if (wave == 0 && ntl > 0) fetch(tile0, 0);
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("s_barrier" ::: "memory");

    // the bias as the C operand of a tile's first MFMAs: no copies into the accumulators at the start of a tile,
    // where the 8 waves have just met
    f16v bvec[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int n = RUNS ? wn0 + 2 * l32 + j : wn0 + 32 * j + 8 * (v >> 2) + 4 * lh + (v & 3);
            bvec[j][v] = reinterpret_cast<const float*>(bias_lds)[n];
        }

    const int sw7 = (l32 >> 1) & 7;
    f16v acc[TM][TN], done[TM][TN];
    for (int t = 0; t < ntl; ++t) {
        if (wave == 0 && t + 1 < ntl) fetch(tile0 + t + 1, (t + 1) & 1);
        if (active) {
            // k groups u = 4 slab + g of 8 k each; the operands of group u + 1 are read during the MFMAs of group u
            f4 fa[2][TM], fb[2][TN];
            auto read_frags = [&](int u, int slot) __attribute__((always_inline)) {
                const int sl = u >> 2, g = u & 3;
                const f4* la = abuf[t & 1][sl];
                const f4* lb = filt[sl];
                const int pc = (2 * g + lh) ^ sw7;
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[slot][i] = la[(wm0 + 32 * i + l32) * KC + pc];
#pragma unroll
                for (int j = 0; j < TN; ++j) fb[slot][j] = lb[(wn0 + 32 * j + l32) * KC + pc];
            };
            read_frags(0, 0);
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (u < 4 * nslab) {
                    if (u + 1 < 4 * nslab) read_frags(u + 1, (u + 1) & 1);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int j = 0; j < TN; ++j) {
                            const f4& a = RUNS ? fa[u & 1][i] : fb[u & 1][j];
                            const f4& b = RUNS ? fb[u & 1][j] : fa[u & 1][i];
                            if (u == 0) {
                                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[0], b[0], bvec[j], 0, 0, 0);
#pragma unroll
                                for (int e = 1; e < 4; ++e)
                                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], acc[i][j], 0, 0, 0);
                            } else {
                                mma_chunk<float>(a, b, acc[i][j]);
                            }
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
                // the finished tile leaves after k group `wave` (a few 16-byte pieces after every group
                // were slower: 0.298 ms against 0.266 on 56x56, 64 -> 256)
                if (t > 0 && u == min(wave, 4 * nslab - 1)) {
                    const int m0 = (tile0 + t - 1) * BM + wm0;       // (not the workgroup's last tile: it lies inside M)
                    if constexpr (RUNS) store_tile_runs<TM, TN, true>(p, p.out, done, m0, wn0, l32, lh, p.M);
                    else store_tile<TM, TN, true>(p, p.out, done, m0, wn0, l32, lh);
                }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) done[i][j] = acc[i][j];
        }
        if (wave == 0) __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));   // the next tile's rows (and its own old stores)
        asm volatile("s_barrier" ::: "memory");
    }
    if (active && ntl > 0) {
        const int m0 = (tile0 + ntl - 1) * BM + wm0;
        if constexpr (RUNS) store_tile_runs<TM, TN>(p, p.out, done, m0, wn0, l32, lh, p.M);
        else store_tile<TM, TN, true>(p, p.out, done, m0, wn0, l32, lh);
    }
}

// dx[s][i][j][:] = 0 for i >= h0 or j >= w0: the trailing rows and columns of a strided dgrad that
// no output pixel reaches (a 28 x 28 input under a 3 x 3 stride-2 "valid" filter: row and column 27).
// One thread per strip pixel and group of 4 channels (C % 4 == 0) or per channel.
struct ZeroStripParams {
    float* dx;
    int S, H, W, C, h0, w0;
    int per_image;       // strip pixels per image: (H - h0) * W + h0 * (W - w0)
    int cgroups, vec;    // channel groups per pixel; 1: groups of 4 with 16-byte stores
    FastDiv div_cg, div_pi, div_w, div_wt;
};

static __global__ __launch_bounds__(kThreads) void zero_strips(const ZeroStripParams p, const unsigned n) {
    const unsigned i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    unsigned t, cg, s, b;
    p.div_cg.divmod(i, t, cg);
    p.div_pi.divmod(t, s, b);
    unsigned row, col;
    const unsigned bottom = (unsigned)((p.H - p.h0) * p.W);
    if (b < bottom) {                                    // the rows from h0 on, whole width
        p.div_w.divmod(b, row, col);
        row += (unsigned)p.h0;
    } else {                                             // the columns from w0 on of the rows above
        p.div_wt.divmod(b - bottom, row, col);
        col += (unsigned)p.w0;
    }
    const size_t pix = ((size_t)s * p.H + row) * p.W + col;
    if (p.vec) *reinterpret_cast<f4*>(p.dx + pix * p.C + 4 * cg) = f4{0.f, 0.f, 0.f, 0.f};
    else p.dx[pix * p.C + cg] = 0.f;
}

template <typename T>
__global__ void pack_filter(const PackParams p) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    int total = p.Npad * p.Kpad;
    if (idx >= total) return;
    int n = idx / p.Kpad;
    int k = idx - n * p.Kpad;
    T v = (T)0;
    if (n < p.N && k < p.K) {
        int tap = k / p.Ck;
        int kc = k - tap * p.Ck;
        int th = tap / p.Tw;
        int tw = tap - th * p.Tw;
        int x = p.xa + p.xs * th;
        int y = p.ya + p.ys * tw;
        int c = p.transposed ? n : kc;
        int d = p.transposed ? kc : n;
        v = static_cast<const T*>(p.w)[((size_t)(x * p.fW + y) * p.C + c) * p.D + d];
    }
    static_cast<T*>(p.bt)[idx] = v;
}

// ------------------------------------------------------------------------------
// Direct kernels for convolutions on 1 to 3 input channels (the first layer of an
// image network: K = fH*fW*C is 9 to 27).  An implicit GEMM pads such a K to a slab
// and, for dgrad, N = C to a 32-wide tile: up to 10 times the useful MFMA work, and
// the gather moves single floats.  Here the filter sits in LDS as fp32 and a lane
// owns 4 output channels d of one pixel, so that the lanes of a pixel read (dgrad)
// or write (fprop) one contiguous row:
//   fprop: y[m][4q..4q+3] = b + sum_{tap,c} x[pixel(m,tap)][c] * w[tap][c][4q..4q+3]
//   dgrad: dx[p][c] = sum over the lanes q of the pixel of
//                     sum_{tap: p = stride*o + tap - pad} dy[o][4q..4q+3] . w[tap][c][4q..4q+3]
// D is a multiple of 4 and at most 256 (D/4 a power of two up to 64 for dgrad, whose
// lanes add up with xor-shuffles), fH*fW*C*D floats fit 32 KB of LDS.
// ------------------------------------------------------------------------------
struct DirectParams {
    const void* a;       // fprop: x [S,H,W,C];  dgrad: dy [S,Ho,Wo,D]
    const void* w;       // [fH,fW,C,D]
    const float* bias;   // fprop only, may be null
    float* out;          // fprop: y [S,Ho,Wo,D];  dgrad: dx [S,H,W,C]
    int S, H, W, C, Ho, Wo, D;
    int fH, fW, sH, sW, pH, pW;
    int M;               // pixels: S*Ho*Wo (fprop) or S*H*W (dgrad)
    int q_shift;         // log2(D / 4): lanes per pixel
    FastDiv div_hw, div_w;
};

constexpr int kDirectMaxW = 8192;    // floats of filter a direct kernel keeps in LDS

template <typename T>
__device__ __forceinline__ void direct_load_filter(const DirectParams& p, float* wl) {
    const T* __restrict__ w = static_cast<const T*>(p.w);
    const int n = p.fH * p.fW * p.C * p.D;
    for (int i = (int)threadIdx.x; i < n; i += kThreads) wl[i] = Elem<T>::to_f32(w[i]);
    __syncthreads();
}

// FH, FW, C are compile-time so that the taps unroll and their loads go out together; the
// filter takes as much LDS as it has floats (dynamic), so that a CU holds 8 workgroups.
// CPT = output channels per lane, 4, 8 or 16: the pixel's position, its FH*FW*C source values and their bounds tests are
// worked out per lane, so with 4 channels a lane spends more instructions on them than on its 4 FH FW C multiply-adds;
// the host picks CPT from the filter size.  The sums run over k in the same order whatever CPT: same bits.
template <typename T, int FH, int FW, int C, int CPT = 4>
static __global__ __launch_bounds__(kThreads) void direct_fprop_smallc(const DirectParams p) {
    extern __shared__ __attribute__((aligned(16))) float wl[];
    direct_load_filter<T>(p, wl);
    const T* __restrict__ x = static_cast<const T*>(p.a);
    const int g = (int)(blockIdx.x * kThreads + threadIdx.x);
    const int m = g >> p.q_shift;
    const int q = g & ((1 << p.q_shift) - 1);
    if (m >= p.M) return;
    unsigned s_, rem, ho, wo;
    p.div_hw.divmod((unsigned)m, s_, rem);
    p.div_w.divmod(rem, ho, wo);
    constexpr int NV = CPT / 4;
    f4 acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v)
        acc[v] = p.bias != nullptr ? *reinterpret_cast<const f4*>(p.bias + CPT * q + 4 * v) : f4{0.f, 0.f, 0.f, 0.f};
    const float* wq = wl + CPT * q;
    float xv[FH * FW * C];
#pragma unroll
    for (int fx = 0; fx < FH; ++fx)
#pragma unroll
        for (int fy = 0; fy < FW; ++fy) {
            const int r = (int)ho * p.sH + fx - p.pH;
            const int cc = (int)wo * p.sW + fy - p.pW;
            const bool ok = (unsigned)r < (unsigned)p.H && (unsigned)cc < (unsigned)p.W;
            const T* px = x + (size_t)((((int)s_ * p.H + (ok ? r : 0)) * p.W + (ok ? cc : 0)) * C);
#pragma unroll
            for (int c = 0; c < C; ++c) xv[(fx * FW + fy) * C + c] = ok ? Elem<T>::to_f32(px[c]) : 0.f;
        }
#pragma unroll
    for (int k = 0; k < FH * FW * C; ++k) {
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const f4 wv = *reinterpret_cast<const f4*>(wq + k * p.D + 4 * v);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[v][e] = fmaf(xv[k], wv[e], acc[v][e]);
        }
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) *reinterpret_cast<f4*>(p.out + (size_t)m * p.D + CPT * q + 4 * v) = acc[v];
}

// NG = groups of 4 output channels per lane, 1 or 2.  With 2 a lane does the work of two neighbouring lanes of the
// one-group form and adds their sums as the first xor-shuffle of that form would: same bits, half the address work.
// (the body takes the workgroup's number and the filter's place in LDS as arguments: see BlockId)
template <typename T, int FH, int FW, int C, int NG = 1>
static __device__ __forceinline__ void direct_dgrad_body(const DirectParams& p, const unsigned block, float* wl) {
    direct_load_filter<T>(p, wl);
    const T* __restrict__ dy = static_cast<const T*>(p.a);
    const int g = (int)(block * kThreads + threadIdx.x);
    const int m = g >> p.q_shift;                            // a pixel's lanes sit in one wave: q_shift <= 6
    const int q = g & ((1 << p.q_shift) - 1);
    unsigned s_, rem, i, j;
    p.div_hw.divmod((unsigned)min(m, p.M - 1), s_, rem);
    p.div_w.divmod(rem, i, j);
    float acc[NG][C];
#pragma unroll
    for (int h = 0; h < NG; ++h)
#pragma unroll
        for (int c = 0; c < C; ++c) acc[h][c] = 0.f;
    const float* wq = wl + 4 * NG * q;
    f4 gv[FH * FW][NG];
    bool oks[FH * FW];
#pragma unroll
    for (int fx = 0; fx < FH; ++fx)
#pragma unroll
        for (int fy = 0; fy < FW; ++fy) {
            const int t = (int)i + p.pH - fx, u = (int)j + p.pW - fy;        // = ho * sH, wo * sW
            const int ho = t / p.sH, wo = u / p.sW;
            const bool ok = t >= 0 && u >= 0 && ho * p.sH == t && wo * p.sW == u && ho < p.Ho && wo < p.Wo;
            const T* pd = dy + (size_t)(((int)s_ * p.Ho + (ok ? ho : 0)) * p.Wo + (ok ? wo : 0)) * p.D + 4 * NG * q;
            oks[fx * FW + fy] = ok;
#pragma unroll
            for (int h = 0; h < NG; ++h) {
                if constexpr (sizeof(T) == 4) {
                    gv[fx * FW + fy][h] = *reinterpret_cast<const f4*>(pd + 4 * h);
                } else {
                    const uint2 v = *reinterpret_cast<const uint2*>(pd + 4 * h);
                    gv[fx * FW + fy][h] = f4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                                             __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u)};
                }
            }
        }
#pragma unroll
    for (int tap = 0; tap < FH * FW; ++tap) {
#pragma unroll
        for (int c = 0; c < C; ++c) {
#pragma unroll
            for (int h = 0; h < NG; ++h) {
                const f4 wv = *reinterpret_cast<const f4*>(wq + (tap * C + c) * p.D + 4 * h);
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < 4; ++e) d = fmaf(gv[tap][h][e], wv[e], d);
                acc[h][c] += oks[tap] ? d : 0.f;
            }
        }
    }
    float sum[C];
#pragma unroll
    for (int c = 0; c < C; ++c) sum[c] = NG == 2 ? acc[0][c] + acc[NG - 1][c] : acc[0][c];
    // add up the lanes of the pixel; every lane ends with the full sums and lane q < C stores channel q
    for (int sh = 1; sh < (1 << p.q_shift); sh <<= 1) {
#pragma unroll
        for (int c = 0; c < C; ++c) sum[c] += __shfl_xor(sum[c], sh);
    }
    if (m < p.M) {
#pragma unroll
        for (int c = 0; c < C; ++c)
            if (q == c) p.out[(size_t)m * C + c] = sum[c];
    }
}

template <typename T, int FH, int FW, int C, int NG = 1>
static __global__ __launch_bounds__(kThreads) void direct_dgrad_smallc(const DirectParams p) {
    extern __shared__ __attribute__((aligned(16))) float wl[];
    direct_dgrad_body<T, FH, FW, C, NG>(p, blockIdx.x, wl);
}

// The shapes the direct kernels take; everything else goes to the gather kernels.

}  // namespace aeth
