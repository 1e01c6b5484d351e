// gather_halo_res9_bf16 and its launcher, in a translation unit of its own: the kernel wants its accumulators and most of
// the filter in the accumulation registers (all 512 registers of a lane are in use), which the other kernels' build flag,
// MFMA results in the ordinary registers, would forbid.
#include "gather_kernels.h"

namespace aeth {

// ------------------------------------------------------------------------------
// gather_halo_res9_bf16: gather_halo_res_bf16 for 3 x 3 taps with the FILTER IN REGISTERS.
// A tap's MFMAs need the pixels' 64 channels and the tap's 64 x 64 filter; read from LDS per tap, as
// gather_halo_res_bf16 does, that is (rows + 64) x 128 bytes per wave and tap, and what a wave gets
// out of LDS (one 16-byte read per lane every 40 clocks or so, measured) is then what bounds the
// tile: 1150 clocks per tap where the MFMAs of the busiest SIMD take 512.  Here a workgroup is 4
// waves, one per SIMD, so a wave may use all 512 registers of a lane, and keeps the whole filter in
// 288 of them for the life of the workgroup: per tap it reads its pixels only, 4 reads for 8 MFMAs.
// A wave takes 56 of the tile's 224 pixels as two halves (32 and 24 rows of a 32-row block) with an
// accumulator set each: while one half is accumulated the other, finished, is stored, one store
// behind every other chunk's MFMAs of eight taps, and the 11 loads a wave contributes to the next
// tile's halo follow the first 11 taps the same way: nothing is issued in a burst, and the reads of
// a tap are issued during the tap before it, across the halves too.
// Output rows are stored at out + m N (the host checks dense_out) as runs of 256 contiguous bytes per
// pixel, as in the RUNS form of gather_halo_res_bf16; the filter takes the same way into LDS first.
// What is left of a launch's time is the memory taking the fp32 output: on [256,56,56,64] -> 64 the
// launch moves 309 MB in 68 us where a copy of that size takes 59, and a build without the stores 55.
// ------------------------------------------------------------------------------
static __global__ __launch_bounds__(256, 1) void gather_halo_res9_bf16(const GatherParams p, const PackParams pk, const int mtiles) {
    constexpr int BM = kResBM, BN = 64, TN = 2, KC = 8, NW = 4, NL = kResSlots / 8 / NW, WR = BM / NW, NT = 9, FW = 3;
    static_assert(WR > 32 && WR <= 64 && WR % 8 == 0, "a wave's pixels are two halves; a store's two pixels are both in or both out");
    static_assert(NL * NW * 8 == kResSlots && NL <= 2 * NT, "the halo's loads divide among the waves and follow a tile's taps");
    __shared__ f4 filt[NT * BN * KC];
    __shared__ f4 halo[2][kResSlots * KC];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int G = (int)gridDim.x;
    const int lid = xcd_contiguous_id((int)blockIdx.x, G);
    const int per = (mtiles + G - 1) / G;                  // a contiguous run of tiles, see gather_halo_res_bf16
    const int tile0 = lid * per;
    const int ntl = max(0, min(per, mtiles - tile0));
    const int hw = p.Hg * p.Wg;
    const int Wp = p.halo_wp;
    const int tile_rows = BM / p.Wg;

    // ---- the halo's loads: load i brings the slots 8 i .. 8 i + 7, this wave issues the loads NW k + wave ----
    // (rel, colbad, the rows outside the image: see the loading wave of gather_halo_res_bf16)
    const u32x4 rsrc_a = raw_rsrc(p.src, p.src_bytes);
    const int lslot = lane >> 3;
    int h_base = 0, h_a0 = 0, h_b0 = 0;                    // of the tile being fetched
    unsigned h_lds = 0, h_none = 0;
    auto aim_halo = [&](int tile, int buf, bool any) __attribute__((always_inline)) {
        unsigned s_img, t_img;
        p.div_halo_tiles.divmod((unsigned)tile, s_img, t_img);
        const int R0 = (int)t_img * tile_rows + p.rh0;                     // image row of padded row 0 of the tile
        h_base = (((int)s_img * p.Hs + R0) * p.Ws + p.rw0) * 128;
        h_a0 = 8 * wave + lslot + R0 * Wp;                                 // slot - lo, lo = -R0 * Wp
        h_b0 = (p.Hs - R0) * Wp - 1 - lslot - 8 * wave;                    // hi - 1 - slot, hi = (Hs - R0) * Wp
        h_lds = lds_address(&halo[buf][0]) + (unsigned)wave * 1024u;
        h_none = any ? 0u : 0x80000000u;                                   // no tile to fetch: every load outside the descriptor
    };
    auto load_halo = [&](int k) __attribute__((always_inline)) {
        // (where the slot lies in the tile is worked out per load: eleven values kept per lane are registers the filter needs)
        const int sl = (NW * k + wave) * 8 + lslot;
        unsigned r, c;
        p.div_halo_wp.divmod((unsigned)sl, r, c);
        const int key = (((int)r * p.Wg + (int)c) >> 1) & 7;
        const int rel = ((int)r * p.Ws + (int)c) * 128 + (((lane & 7) ^ key) & 7) * 16;
        const unsigned colbad = ((unsigned)((int)c + p.rw0) >= (unsigned)p.Ws || (int)c >= p.Wg + FW - 1) ? 0x80000000u : 0u;
        const unsigned rowbad = (unsigned)((h_a0 + 8 * NW * k) | (h_b0 - 8 * NW * k)) & 0x80000000u;
        const unsigned off = (unsigned)(h_base + rel) | rowbad | colbad | h_none;
        lds_direct_load16(rsrc_a, (unsigned)__builtin_amdgcn_readfirstlane((int)(h_lds + (unsigned)(NW * k) * 1024u)), off);
    };
    aim_halo(tile0, 0, ntl > 0);
#pragma unroll
    for (int k = 0; k < NL; ++k) load_halo(k);             // under way while the filter is fetched

    // ---- the filter into LDS: slab t (tap x = xa + xs (t / 3), y = ya + ys (t % 3)) of 64 rows (n) x 128 B, chunk c of
    // row r at c ^ ((r >> 1) & 7), slab row r holding channel 2 (r % 32) + r / 32 ----
    {
        const unsigned w_bytes = (unsigned)(pk.w_elems * 2);
        if (pk.transposed) {
            // dgrad: n is the input channel c and k the output channel d, which is contiguous in w: rows are copied as
            // they are; wave w fetches the 1 KB pieces w, w + 4, ...
            const u32x4 rsrc_w = raw_rsrc(pk.w, w_bytes);
            const int k4e = (lane & 7) ^ (lane >> 4);
#pragma unroll
            for (int i = 0; i < NT * 8 / NW; ++i) {
                const int q = i * NW + wave;
                const int tap = q >> 3, part = q & 7;
                const int x = pk.xa + pk.xs * (tap / FW), y = pk.ya + pk.ys * (tap % FW);
                const int row = part * 8 + (lane >> 3);
                const int n = 2 * (row & 31) + (row >> 5);
                const int k4 = k4e ^ ((part & 1) ? 4 : 0);
                const unsigned off = (unsigned)((((x * pk.fW + y) * pk.C + n) * pk.D + 8 * k4) * 2) | ((unsigned)(n >= p.N) << 31);
                lds_direct_load16(rsrc_w, lds_address(filt) + (unsigned)q * 1024u, off);
            }
        } else {
            // fprop: n is the output channel d, contiguous in w, and k the input channel c: a transposition.  Half a wave
            // reads two adjacent n of two adjacent c (4 bytes each) and writes the two (n, c pair) words; the loads of a
            // batch are all issued before the first word is written: one latency per batch, not per pair.
            const __amdgpu_buffer_rsrc_t rsrc_w =
                __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(pk.w), 0, (int)w_bytes, 0x00020000);
            const int n2 = 2 * (lane & 31);
            const unsigned nbad = (unsigned)(n2 >= p.N) << 31;             // N is even here (checked by the host)
            char* const fbytes = reinterpret_cast<char*>(filt);
            constexpr int FB = 36;                                         // pairs of loads per batch: all of them
            static_assert(4 * NT % FB == 0, "whole batches");
            const int r0 = n2 >> 1, r1 = (n2 >> 1) + 32;                   // the slab rows of channels n2 and n2 + 1
            for (int i0 = 0; i0 < 4 * NT; i0 += FB) {
                unsigned a[FB], b[FB];
#pragma unroll
                for (int u = 0; u < FB; ++u) {
                    const int r = 2 * (((i0 + u) * NW + wave) * 2 + lh);       // row = tap * 64 + c, c even
                    const int tap = r >> 6, c = r & 63;
                    unsigned t_h, t_w;
                    p.div_tw.divmod((unsigned)tap, t_h, t_w);
                    const int x = pk.xa + pk.xs * (int)t_h, y = pk.ya + pk.ys * (int)t_w;
                    const unsigned off = (unsigned)((((x * pk.fW + y) * pk.C + c) * pk.D + n2) * 2) | nbad;
                    a[u] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, (int)off, 0, 0);
                    b[u] = __builtin_amdgcn_raw_buffer_load_b32(rsrc_w, (int)off, pk.D * 2, 0);
                }
#pragma unroll
                for (int u = 0; u < FB; ++u) {
                    const int r = 2 * (((i0 + u) * NW + wave) * 2 + lh);
                    const int tap = r >> 6, c = r & 63;
                    const int pos = ((c >> 3) ^ ((r0 >> 1) & 7)) * 16 + (c & 7) * 2;
                    *reinterpret_cast<unsigned*>(fbytes + tap * 8192 + r0 * 128 + pos) = (a[u] & 0xffffu) | (b[u] << 16);
                    *reinterpret_cast<unsigned*>(fbytes + tap * 8192 + r1 * 128 + pos) = (a[u] >> 16) | (b[u] & 0xffff0000u);
                }
            }
        }
    }
    float bias_run[TN];                                                    // the lane's channels 2 l32 + j
#pragma unroll
    for (int j = 0; j < TN; ++j) bias_run[j] = (p.bias != nullptr && 2 * l32 + j < p.N) ? p.bias[2 * l32 + j] : 0.f;
    // The wave's pixels: half hf has the pixels 32 hf + l32 of its WR, the lanes past the last one repeat it (multiplied,
    // never stored).  pslot: slot of tap (0, 0); pnum: the pixel's number in the tile.
    int pslot[2], pnum[2];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
        pnum[hf] = wave * WR + min(32 * hf + l32, WR - 1);
        unsigned r, c;
        p.div_w.divmod((unsigned)pnum[hf], r, c);
        pslot[hf] = (int)r * Wp + (int)c;
    }
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8));                   // the first halo and this wave's part of the filter
    asm volatile("s_barrier" ::: "memory");

    // ---- the filter into registers: wf[tap][g][j], the operand of the MFMA of chunk g (16 of the 64 k) and column block j ----
    f4 wf[NT][4][TN];
    {
        const int sw7 = (l32 >> 1) & 7;
#pragma unroll
        for (int tap = 0; tap < NT; ++tap) {
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int j = 0; j < TN; ++j) wf[tap][g][j] = filt[tap * (BN * KC) + (32 * j + l32) * KC + ((2 * g + lh) ^ sw7)];
            __builtin_amdgcn_sched_barrier(0);           // a tap at a time: all 72 reads in flight at once would need their 288 registers twice
        }
    }

    // ---- the products ----
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const __amdgpu_buffer_rsrc_t rsrc_o = __builtin_amdgcn_make_buffer_rsrc(p.out, 0, (int)p.out_bytes, 0x00020000);
    const unsigned rowb = (unsigned)p.N * 4u;
    const unsigned colb = ((unsigned)(TN * l32) * 4u) | ((unsigned)!(TN * l32 < p.N) << 31);
    f16v acc[2][TN];                                                       // of the two halves
#pragma unroll
    for (int hf = 0; hf < 2; ++hf)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[hf][j][v] = bias_run[j];
    // where a finished half goes: the lane's byte offset of pixel 0 of the half, and how many of the half's pixels from the
    // lane's first one (4 lh) on are stored (none before the first half is finished, fewer in an image's last tile)
    unsigned st_off[2] = {0, 0};
    int st_rows[2] = {0, 0};
    auto store_one = [&](int hf, int v) __attribute__((always_inline)) {
        const int r = 8 * (v >> 2) + (v & 3);                              // the pixel of the lanes 0..31 within the half; the others: + 4
        if (32 * hf + r + 4 < WR) {
            const unsigned off = (st_off[hf] + colb) | (r < st_rows[hf] ? 0u : 0x80000000u);
            const u2 value = {__float_as_uint(acc[hf][0][v]), __float_as_uint(acc[hf][1][v])};
            __builtin_amdgcn_raw_buffer_store_b64(value, rsrc_o, (int)off, (int)((unsigned)r * rowb), 2);
        }
    };
    f4 fa[2][4];                                                           // the pixels' operands of two taps
    auto read_pixels = [&](int hf, int tap, const f4* h, f4 (&ra)[4]) __attribute__((always_inline)) {
        const int th = tap / FW, tw = tap % FW;
        const int x0 = (pslot[hf] + th * Wp + tw) * 8 + ((lh ^ ((pnum[hf] + th * p.Wg + tw) >> 1)) & 7);
#pragma unroll
        for (int g = 0; g < 4; ++g) ra[g] = h[x0 ^ (g << 1)];
    };
    for (int t = 0; t < ntl; ++t) {
        // everyone is done with tile t - 1, whose buffer takes tile t + 1
        aim_halo(tile0 + t + 1, (t + 1) & 1, t + 1 < ntl);
        unsigned s_img, t_img;
        p.div_halo_tiles.divmod((unsigned)(tile0 + t), s_img, t_img);
        const int m0 = (int)s_img * hw + (int)t_img * BM + wave * WR;       // the wave's first pixel
        const int m_end = ((int)s_img + 1) * hw;                           // rows past the image: multiplied, never stored
        const f4* h = halo[t & 1];
#if defined(__HIP_DEVICE_COMPILE__)
        // (the taps' addresses are the same in every tile; worked out once and kept, 18 of them, they would push the
        // filter out of the registers: the compiler is told that the pixels' slots change per tile)
        asm volatile("" : "+v"(pslot[0]), "+v"(pslot[1]), "+v"(pnum[0]), "+v"(pnum[1]));
#endif
        read_pixels(0, 0, h, fa[0]);
#pragma unroll
        for (int q = 0; q < 2 * NT; ++q) {                                 // the taps of half 0, then those of half 1
            const int hf = q / NT, tap = q % NT;
            const f4 (&ca)[4] = fa[q & 1];
            f4 (&na)[4] = fa[(q + 1) & 1];
            int x0n = 0;
            if (q + 1 < 2 * NT) {
                const int th = ((q + 1) % NT) / FW, tw = ((q + 1) % NT) % FW, hn = (q + 1) / NT;
                x0n = (pslot[hn] + th * Wp + tw) * 8 + ((lh ^ ((pnum[hn] + th * p.Wg + tw) >> 1)) & 7);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                if (q + 1 < 2 * NT) na[g] = h[x0n ^ (g << 1)];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int j = 0; j < TN; ++j) mma_chunk<uint16_t>(ca[g], wf[tap][g][j], acc[hf][j]);
                // the other half, finished a half-tile ago: its 16 stores behind every other chunk of the taps 0 to 7 (in a
                // burst, one per chunk, they fill the CU's memory pipeline and the MFMAs behind them in the wave wait with
                // them: 12 us of the 67 a call took)
                if (tap < NT - 1 && g % 2 == 0) store_one(1 - hf, 2 * tap + g / 2);
                __builtin_amdgcn_sched_barrier(0);
            }
            if (tap == NT - 1) {                                           // the other half starts over
#pragma unroll
                for (int j = 0; j < TN; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[1 - hf][j][v] = bias_run[j];
            }
            if (q < NL) load_halo(q);
            if (tap == NT - 1) {                                           // this half is finished
                const int mh = m0 + 32 * hf + 4 * lh;
                st_off[hf] = (unsigned)mh * rowb;
                st_rows[hf] = m_end - mh;
            }
        }
        __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));             // the next tile's halo (and the stores before it)
        asm volatile("s_barrier" ::: "memory");
    }
    // Half 0 of the last tile went out during its half 1; half 1 is left.  (A workgroup without tiles stores nothing:
    // st_rows is 0.)
#pragma unroll
    for (int v = 0; v < 16; ++v) store_one(1, v);
}

void launch_halo_res9_bf16(const GatherParams& p, const PackParams& pk, int mtiles, unsigned grid, hipStream_t stream) {
    hipLaunchKernelGGL(gather_halo_res9_bf16, dim3(grid), dim3(256), 0, stream, p, pk, mtiles);
}

}  // namespace aeth
