// Implicit-GEMM convolution kernels for gfx950, shared by the fp32 and the
// bf16-input entry points (T = float or uint16_t holding bf16 bits).
//
// GEMM view (M = S*Ho*Wo, N = D, K = fH*fW*C):
//   fprop : Y[M,N]  = A[M,K] . W[K,N] + bias      A gathered from x on the fly
//   dgrad : dX[M',C] = A'[M',K'] . W'[K',C]        A' gathered from dy; one launch
//           per stride-parity class so that no tap multiplies a structural zero
//   wgrad : dW[K,N] = A[M,K]^T . dY[M,N]           reduction over M split across
//           workgroups, partial sums reduced in a fixed order
//
// "gather" kernel (fprop, dgrad, dense fprop/dgrad)
//   workgroup = 256 threads = 4 waves, tile BM x BN; K is consumed in slabs of
//   128 bytes per row (32 floats or 64 bf16).  An A slab is read with one 128-bit
//   load per thread per chunk (NHWC: channels are contiguous), zero where the tap
//   falls in the padding, and stored to LDS row-major with a row pitch of 144
//   bytes; the B slab comes from a pre-packed [N][K] copy of the filter and uses
//   the same pitch.  With that pitch the 128-bit stores and the 128-bit operand
//   reads both touch 32 distinct banks per 8 lanes.
//   fp32: each lane feeds the 4 floats of its chunk to 4 successive
//   v_mfma_f32_32x32x2_f32; the k order inside a slab is permuted identically for
//   A and B, which leaves the sum unchanged.
//   bf16: a chunk is exactly the 8 k-values one lane supplies to
//   v_mfma_f32_32x32x16_bf16.
#pragma once
#include <type_traits>

#include "common.h"

#include <limits.h>
#include <stdlib.h>
#include <vector>

namespace aeth {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kChunksPerRow = 8;   // 16-byte chunks per slab row
constexpr int kLDC = 9;            // LDS row pitch in chunks (8 data + 1 pad)

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int CE = 4;   // elements per 16-byte chunk
    static constexpr int BK = 32;  // elements per slab row
    static __device__ __forceinline__ float to_f32(float v) { return v; }
};
template <> struct Elem<uint16_t> {
    static constexpr int CE = 8;
    static constexpr int BK = 64;
    static __device__ __forceinline__ float to_f32(uint16_t v) { return __uint_as_float((unsigned)v << 16); }
};

template <typename T>
__device__ __forceinline__ void mma_chunk(const f4& a, const f4& b, f16v& acc);

template <>
__device__ __forceinline__ void mma_chunk<float>(const f4& a, const f4& b, f16v& acc) {
#pragma unroll
    for (int t = 0; t < 4; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b[t], acc, 0, 0, 0);
}

template <>
__device__ __forceinline__ void mma_chunk<uint16_t>(const f4& a, const f4& b, f16v& acc) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc,
                                                  0, 0, 0);
}

// ------------------------------------------------------------------------------
// gather-GEMM
// ------------------------------------------------------------------------------
struct GatherParams {
    const void* src;     // [S, Hs, Ws, Cs] of T
    const void* bt;      // packed filter [Npad][Kpad] of T, zero filled (or the filter itself: bt_direct)
    const float* bias;   // [N] or nullptr
    float* out;
    int S, Hs, Ws, Cs;
    int Hg, Wg;          // output pixel grid of this launch
    int M, N, K, Kpad;   // M = S*Hg*Wg, K = Th*Tw*Cs
    int Tw, Th;          // taps per filter row, filter rows (Th is filled in by run_gather)
    int sh, sw;          // source step per output pixel
    int rh0, rw0;        // source offset of tap (0,0)
    // output element (s,i,j,n) lives at ((s*Hof + oh0 + i*ohs)*Wof + ow0 + j*ows)*N + n
    int Hof, Wof, oh0, ow0, ohs, ows;
    int dense_out;       // 1: row m is stored at out + m*N
    unsigned src_bytes;  // extent of src / bt for the buffer descriptors (0: too large, not used)
    unsigned bt_bytes;
    unsigned out_bytes;  // extent of out; 0: no 16-byte stores (too large, N not a multiple of 4, or unaligned)
    int split_slabs;     // 0, or slabs of K per blockIdx.y: split y writes its partial product at out + y*M*N
    // B operand addressing of the slab kernels: row n of the B matrix starts bt_ld elements after row n - 1.
    // bt_direct (dgrad on uniform-tap slabs): bt is the filter w[fH][fW][C][D] itself, whose rows (tap, c) are
    // already contiguous in k = d; the slab of tap (th, tw), channel offset c0 starts at element
    // ((bd_xa + bd_xs th) bd_fw + bd_ya + bd_ys tw) * bd_tap_elems + c0 of row 0: no packing launch.
    int bt_ld, bt_direct;
    int bt_kn;           // fp32 fprop: bt is the filter itself as a [K][N] matrix (row k = (tap, c), bt_ld = D floats apart);
                         // 2: the problem is a part of an fprop with the taps (bd_xa + th, bd_ya + tw) of a filter bd_fw taps wide
    int bd_xa, bd_xs, bd_ya, bd_ys, bd_fw, bd_tap_elems;
    // gather_halo_bf16: columns and rows of the padded source image, 256-row tiles per image (0: tiles
    // run over image boundaries)
    int halo_wp, halo_hp, halo_tiles;
    // gather_halo_pairs_bf16: the classes of a dgrad share one padded source tensor of halo_th x halo_tw windows per
    // pixel; this class's tap (th, tw) is the window (th + tap_dh, tw + tap_dw)
    int halo_th, halo_tw, tap_dh, tap_dw;
    FastDiv div_hw, div_w, div_c, div_tw, div_halo_wp, div_halo_hp, div_halo_tiles;
};

constexpr int kInvalidRow = -16384;
constexpr int kNloopMaxN = 1024;   // widest output the n-loop mode of the gather kernel takes (its bias sits in LDS)
constexpr int kXcds = 8;

// A workgroup's place in its launch.  A kernel body that takes it as an argument can also run as one part of a launch
// that holds two kernels, where the hardware's numbers count the workgroups of both.
struct BlockId {
    int x, y;            // what blockIdx.x and blockIdx.y are in a launch of the kernel alone
    int gx;              // gridDim.x of that launch
};
__device__ __forceinline__ BlockId launch_block() { return BlockId{(int)blockIdx.x, (int)blockIdx.y, (int)gridDim.x}; }

// Workgroups are handed to the 8 XCDs round-robin by linear id, and each XCD has its
// own L2.  This maps the hardware id to a logical id such that every XCD works on
// one contiguous range of logical ids: tiles that share operands (the N tiles of
// one M tile, the k tiles of one wgrad split, neighbouring M tiles with their
// common halo rows) then hit the same L2 at about the same time.
__device__ __forceinline__ int xcd_contiguous_id(int wg, int total) {
    const int per = total / kXcds, rem = total % kXcds;
    const int xcd = wg % kXcds, idx = wg / kXcds;
    return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

// The MFMAs are issued with the operands swapped (filter rows as A, gathered pixels
// as B), so the accumulators hold the TRANSPOSED output tile:
//   acc[i][j][v] = out[m = mw0 + 32 i + lane%32][n = nw0 + 32 j + 8 (v/4) + 4 (lane/32) + v%4]
// A lane owns one output row per tile and 4 consecutive channels per v/4: the tile
// goes out in 16-byte stores whose addresses differ by compile-time constants, with
// one row decode per lane.  fp32 MFMA and ordinary vector instructions compete for
// the same issue cycles, so an epilogue of 32 scalar stores with per-element address
// arithmetic costs measurable matrix time (9 % on the 56x56x64 layer).
// The bias is added by starting the accumulators from it.
// Bias values for the accumulator layout above, through a buffer descriptor that ends
// after channel N (after nothing when there is no bias): channels past N read as zero
// without a branch.  Per-lane branches around ordinary loads made the compiler wait
// for each load in turn, several microseconds at the start of every workgroup.
template <int TN>
__device__ __forceinline__ void load_bias(const GatherParams& p, const float* bias, f4 (&bv)[TN][4], int nw0, int lh) {
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(bias), 0, bias != nullptr ? p.N * 4 : 0, 0x00020000);
    if (p.N % 4 == 0) {                                 // whole groups of 4 channels: inside or outside as one
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int n = nw0 + 32 * j + 8 * q + 4 * lh;
                bv[j][q] = __builtin_bit_cast(f4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, n * 4, 0, 0));
            }
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int n = nw0 + 32 * j + 8 * q + 4 * lh + e;
                    bv[j][q][e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, n * 4, 0, 0));
                }
    }
}

template <int TM, int TN>
__device__ __forceinline__ void fill_acc(const f4 (&bv)[TN][4], f16v (&acc)[TM][TN]) {
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = bv[j][q][e];
}

template <int TM, int TN>
__device__ __forceinline__ void init_acc(const GatherParams& p, const float* bias, f16v (&acc)[TM][TN], int nw0, int lh) {
    f4 bv[TN][4];
    load_bias<TN>(p, bias, bv, nw0, lh);
    fill_acc<TM, TN>(bv, acc);
}

// VEC_ONLY: the caller guarantees p.out_bytes != 0 (16-byte stores through the descriptor)
// m_end: rows from here on are not stored (default: p.M)
template <int TM, int TN, bool VEC_ONLY = false>
__device__ __forceinline__ void store_tile(const GatherParams& p, float* out, const f16v (&acc)[TM][TN], int mw0,
                                           int nw0, int l32, int lh, int m_end = -1) {
    if (m_end < 0) m_end = p.M;
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const bool full_n = nw0 + 32 * TN <= p.N;           // wave-uniform
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)p.out_bytes, 0x00020000);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = mw0 + 32 * i + l32;
        const bool mok = m < m_end;
        unsigned row = (unsigned)m;
        if (!p.dense_out) {
            unsigned s, rem, ii, jj;
            p.div_hw.divmod(mok ? (unsigned)m : 0u, s, rem);
            p.div_w.divmod(rem, ii, jj);
            row = ((unsigned)s * p.Hof + p.oh0 + ii * p.ohs) * p.Wof + p.ow0 + jj * p.ows;
        }
        const unsigned elem = row * (unsigned)p.N + (unsigned)(nw0 + 4 * lh);   // < 2^31: checked by the host
        if (VEC_ONLY || p.out_bytes != 0) {
            // rows past M (and, in edge tiles, channels past N) get a byte offset beyond
            // the descriptor's extent: the hardware drops the store
            const unsigned base = (elem * 4u) | ((unsigned)!mok << 31);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f4 v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    unsigned off = base;
                    if (!full_n) off |= (unsigned)!(nw0 + 32 * j + 8 * q + 4 * lh < p.N) << 31;
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u4, v), rsrc, (int)off,
                                                           (32 * j + 8 * q) * 4, 0);
                }
        } else if (mok) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int n = nw0 + 32 * j + 8 * (v >> 2) + 4 * lh + (v & 3);
                    if (n < p.N) out[(size_t)row * p.N + n] = acc[i][j][v];
                }
        }
    }
    // The stored registers stay untouched for a few cycles after the last store has been issued.
    // Where the instruction after a 16-byte store was free to reuse its data registers (a
    // persistent workgroup whose scheduler had moved the next tile's address arithmetic up), the
    // last lanes of each row of 16 now and then stored the new value instead.
#if defined(__HIP_DEVICE_COMPILE__)                      // the host pass does not know the register class
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) asm volatile("s_nop 3" :: "v"(acc[i][j]));
#endif
}

// The same tile from accumulators of MFMAs issued with the pixels as the first operand:
//   acc[i][j][v] = out[m = mw0 + 32 i + 8 (v/4) + 4 (lane/32) + v%4][n = nw0 + 32 j + lane%32]
// 32 lanes write the 128 contiguous bytes of one pixel's 32 channels, 4 bytes each: one store
// instruction is two whole lines, where the 16-byte stores of store_tile are 64 pieces of 16 bytes
// in 32 lines.  Four times the store instructions; for kernels that wait for their stores, not for
// instruction issue.  Every lane works out the row of one pixel of the block, the stores fetch the
// rows of their two pixels from those lanes.  Needs p.out_bytes != 0 (the descriptor drops rows
// past m_end and channels past N).
template <int TM, int TN>
__device__ __forceinline__ void store_tile_lines(const GatherParams& p, float* out, const f16v (&acc)[TM][TN], int mw0,
                                                 int nw0, int l32, int lh, int m_end) {
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)p.out_bytes, 0x00020000);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = mw0 + 32 * i + l32;
        const bool mok = m < m_end;
        unsigned row = (unsigned)m;
        if (!p.dense_out) {
            unsigned s, rem, ii, jj;
            p.div_hw.divmod(mok ? (unsigned)m : 0u, s, rem);
            p.div_w.divmod(rem, ii, jj);
            row = ((unsigned)s * p.Hof + p.oh0 + ii * p.ohs) * p.Wof + p.ow0 + jj * p.ows;
        }
        const int rowbytes = (int)((row * (unsigned)p.N * 4u) | ((unsigned)!mok << 31));   // < 2^31: checked by the host
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int pix = 8 * (v >> 2) + (v & 3);
            const unsigned base = (unsigned)__builtin_amdgcn_ds_bpermute(4 * pix + 16 * lh, rowbytes);
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = nw0 + 32 * j + l32;
                const unsigned off = (base + (unsigned)n * 4u) | ((unsigned)!(n < p.N) << 31);   // bit 31 from either part: outside the descriptor
                const float value = acc[i][j][v];        // (a bit cast of the vector element itself reads element 0)
                __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(value), rsrc, (int)off, 0, 2);
            }
        }
    }
}

// The same for a wave tile of two 32-column blocks whose columns are interleaved: column l of block j is channel
// nw0 + 2 l + j (the kernel fetches the filter rows in that order), so a lane holds two neighbouring channels of a pixel
// and 32 lanes write 256 contiguous bytes with 8-byte stores: half the store instructions of store_tile_lines.
template <int TM, bool NT>
__device__ __forceinline__ void store_tile_lines2(const GatherParams& p, float* out, const f16v (&acc)[TM][2], int mw0,
                                                  int nw0, int l32, int lh, int m_end) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)p.out_bytes, 0x00020000);
    const int n = nw0 + 2 * l32;
    const unsigned col = ((unsigned)n * 4u) | ((unsigned)!(n < p.N) << 31);      // N is even: both channels or neither
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = mw0 + 32 * i + l32;
        const bool mok = m < m_end;
        unsigned row = (unsigned)m;
        if (!p.dense_out) {
            unsigned s, rem, ii, jj;
            p.div_hw.divmod(mok ? (unsigned)m : 0u, s, rem);
            p.div_w.divmod(rem, ii, jj);
            row = ((unsigned)s * p.Hof + p.oh0 + ii * p.ohs) * p.Wof + p.ow0 + jj * p.ows;
        }
        const int rowbytes = (int)((row * (unsigned)p.N * 4u) | ((unsigned)!mok << 31));   // < 2^31: checked by the host
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int pix = 8 * (v >> 2) + (v & 3);
            const unsigned base = (unsigned)__builtin_amdgcn_ds_bpermute(4 * pix + 16 * lh, rowbytes);
            const float a = acc[i][0][v], b = acc[i][1][v];    // (a bit cast of the vector element itself reads element 0)
            const u2 value = {__float_as_uint(a), __float_as_uint(b)};
            // (2: the non-temporal hint, for whole lines that stream to memory)
            if constexpr (NT) __builtin_amdgcn_raw_buffer_store_b64(value, rsrc, (int)((base + (col & 0x7fffffffu)) | (col & 0x80000000u)), 0, 2);
            else __builtin_amdgcn_raw_buffer_store_b64(value, rsrc, (int)((base + (col & 0x7fffffffu)) | (col & 0x80000000u)), 0, 0);
        }
    }
}

// (These whole-line stores carry the non-temporal hint, cache policy 2: the output streams to memory.  Worth 5 to 15 % of a
// launch that writes hundreds of MB; on the 16-byte pieces of store_tile the hint costs 50 %, and an output that the next
// kernel reads out of L2 is better off without it: the host takes these forms for large outputs only.)
// The general form: a wave tile of TN 32-column blocks with interleaved columns (column l of block j is channel
// nw0 + TN l + j; TN = 2 or 4): a lane holds TN neighbouring channels of a pixel and 32 lanes write 32 TN contiguous
// floats per pixel with one 8- or 16-byte store each.  N is a multiple of 4 (p.out_bytes != 0).
// PLAIN: the caller guarantees p.dense_out and a tile that lies inside m_end.
template <int TM, int TN, bool PLAIN = false>
__device__ __forceinline__ void store_tile_runs(const GatherParams& p, float* out, const f16v (&acc)[TM][TN], int mw0,
                                                int nw0, int l32, int lh, int m_end) {
    static_assert(TN == 2 || TN == 4, "8- or 16-byte stores");
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(out, 0, (int)p.out_bytes, 0x00020000);
    const int n = nw0 + TN * l32;
    const unsigned col = (unsigned)n * 4u, colbad = (unsigned)!(n < p.N) << 31;   // N is a multiple of TN here: all channels or none
    // Rows stored at out + m N with the whole tile inside m_end (mw0 is wave-uniform): one vector offset per tile, the
    // pixel's row as the scalar offset of an 8-byte store (one addition per 16-byte store), no lane exchange.  (Measured
    // as a run-time choice in every kernel that stores runs: 4 % for dense_res_f32, whose stores sit between MFMA groups,
    // nothing or a loss of 0.3 % where the stores end a workgroup.)
    if constexpr (PLAIN) {
        const unsigned rowb = (unsigned)p.N * 4u;
        const int voff = (int)(((unsigned)(mw0 + 4 * lh) * rowb + col) | colbad);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int soff = (int)((unsigned)(32 * i + 8 * (v >> 2) + (v & 3)) * rowb);
                float e[TN];
#pragma unroll
                for (int j = 0; j < TN; ++j) e[j] = acc[i][j][v];
                if constexpr (TN == 2) {
                    const u2 value = {__float_as_uint(e[0]), __float_as_uint(e[1])};
                    __builtin_amdgcn_raw_buffer_store_b64(value, rsrc, voff, soff, 2);
                } else {
                    // (a 16-byte store with its scalar offset in a register is the form behind which the compiler leaves
                    // no wait state before the next write of the data registers, see store_tile, and here the next store's
                    // data is assembled in the same registers right behind it: the row goes into the vector offset)
                    const u4 value = {__float_as_uint(e[0]), __float_as_uint(e[1]), __float_as_uint(e[2]), __float_as_uint(e[3])};
                    __builtin_amdgcn_raw_buffer_store_b128(value, rsrc, voff + soff, 0, 2);
                }
            }
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = mw0 + 32 * i + l32;
            const bool mok = m < m_end;
            unsigned row = (unsigned)m;
            if (!p.dense_out) {
                unsigned s, rem, ii, jj;
                p.div_hw.divmod(mok ? (unsigned)m : 0u, s, rem);
                p.div_w.divmod(rem, ii, jj);
                row = ((unsigned)s * p.Hof + p.oh0 + ii * p.ohs) * p.Wof + p.ow0 + jj * p.ows;
            }
            const int rowbytes = (int)((row * (unsigned)p.N * 4u) | ((unsigned)!mok << 31));   // < 2^31: checked by the host
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int pix = 8 * (v >> 2) + (v & 3);
                const unsigned base = (unsigned)__builtin_amdgcn_ds_bpermute(4 * pix + 16 * lh, rowbytes);
                const int off = (int)((base + col) | colbad);
                float e[TN];                             // (a bit cast of the vector element itself reads element 0)
#pragma unroll
                for (int j = 0; j < TN; ++j) e[j] = acc[i][j][v];
                if constexpr (TN == 2) {
                    const u2 value = {__float_as_uint(e[0]), __float_as_uint(e[1])};
                    __builtin_amdgcn_raw_buffer_store_b64(value, rsrc, off, 0, 2);
                } else {
                    const u4 value = {__float_as_uint(e[0]), __float_as_uint(e[1]), __float_as_uint(e[2]), __float_as_uint(e[3])};
                    __builtin_amdgcn_raw_buffer_store_b128(value, rsrc, off, 0, 2);
                }
            }
        }
    }
#if defined(__HIP_DEVICE_COMPILE__)                      // see store_tile: the stored registers stay untouched for a few cycles
    if constexpr (TN == 4) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("s_nop 3" :: "v"(acc[i][j]));
    }
#endif
}

// ------------------------------------------------------------------------------
// LDS-direct loads and wave-uniform mask helpers shared by the gather and the wgrad kernels
// ------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// A 16-byte-per-lane LDS-direct load the compiler does not see as one.  It orders every LDS
// read behind the LDS-direct loads it knows to be in flight unless it can prove where they
// land, and with a ring of buffers in a loop it cannot: the reads of a step then wait for the
// slabs fetched for later steps.  The caller waits (vmcnt + barrier) before reading what a
// load brings.  lds_base: wave-uniform LDS byte address; the lanes land at lds_base + 16 * lane.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void lds_direct_load16(const u32x4& rsrc, unsigned lds_base, unsigned voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :: "s"(lds_base), "v"(voff), "s"(rsrc) : "memory", "m0");
}
// the same with a scalar byte offset added to every lane's (the range check looks at `voff` alone)
__device__ __forceinline__ void lds_direct_load16_s(const u32x4& rsrc, unsigned lds_base, unsigned voff, unsigned soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :: "s"(lds_base), "v"(voff), "s"(rsrc), "s"(soff) : "memory", "m0");
}
__device__ __forceinline__ u32x4 raw_rsrc(const void* base, unsigned bytes) {
    const unsigned long long a = reinterpret_cast<unsigned long long>(base);
    return u32x4{(unsigned)a, (unsigned)(a >> 32) & 0xffffu, bytes, 0x00020000u};
}
__device__ __forceinline__ unsigned lds_address(const void* q) {
    return (unsigned)reinterpret_cast<uintptr_t>((lds_ptr_t)const_cast<void*>(q));
}

// bit b of a wave-uniform mask of 64 / LANES bits to lanes LANES * b .. LANES * b + LANES - 1, on the scalar unit
template <int LANES>
__device__ __forceinline__ unsigned long long spread_rows(unsigned m) {
    static_assert(LANES == 8 || LANES == 4, "8 or 4 lanes per row");
    unsigned long long r;
    asm("s_bitreplicate_b64_b32 %0, %1" : "=s"(r) : "s"(m));
    asm("s_bitreplicate_b64_b32 %0, %1" : "=s"(r) : "s"((unsigned)r));
    if (LANES == 8) asm("s_bitreplicate_b64_b32 %0, %1" : "=s"(r) : "s"((unsigned)r));
    return r;
}
// lane l gets b where bit l of the wave-uniform mask is set, else a
__device__ __forceinline__ unsigned select_by_mask(unsigned a, unsigned b, unsigned long long mask) {
    unsigned v;
    asm("v_cndmask_b32 %0, %1, %2, %3" : "=v"(v) : "v"(a), "v"(b), "s"(mask));
    return v;
}

// out[i] = sum_s part[s*stride + i] for i < n, in a fixed order: 4 split lanes per
// output (splits s, s+4, ...), then the 4 lanes in order.  i < n_dw goes to dw,
// the rest to dbias.  tr > 0: the partials hold the transpose, rows of tr floats: element
// i = r tr + c of a partial is dw[c (n_dw / tr) + r].
static __global__ __launch_bounds__(kThreads) void reduce_splits(const float* __restrict__ part, float* __restrict__ dw,
                                                         float* __restrict__ dbias, int n_dw, int n, int stride,
                                                         int splits, int tr = 0) {
    __shared__ float red[4][64];
    const int col = threadIdx.x & 63;
    const int sl = threadIdx.x >> 6;
    const int i = blockIdx.x * 64 + col;
    float s = 0.f;
    if (i < n) {
        const float* q = part + i;
        int k = sl;
        float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
        for (; k + 12 < splits; k += 16) {
            s0 += q[(size_t)k * stride];
            s1 += q[(size_t)(k + 4) * stride];
            s2 += q[(size_t)(k + 8) * stride];
            s3 += q[(size_t)(k + 12) * stride];
        }
        for (; k < splits; k += 4) s0 += q[(size_t)k * stride];
        s = (s0 + s1) + (s2 + s3);
    }
    red[sl][col] = s;
    __syncthreads();
    if (sl == 0 && i < n) {
        float t = (red[0][col] + red[1][col]) + (red[2][col] + red[3][col]);
        if (i < n_dw) dw[tr > 0 ? (i % tr) * (n_dw / tr) + i / tr : i] = t;
        else if (dbias != nullptr) dbias[i - n_dw] = t;
    }
}

// The same sum for 16-byte aligned partials (stride and n_dw multiples of 4): a thread
// owns 4 consecutive outputs, 16 split lanes per output add splits j, j+16, ... with
// four loads in flight, and the lanes are added in lane order.
// (tr as above, a multiple of 4: the 4 outputs of a thread then go to 4 rows of dw)
// act_out != nullptr (tr == 0): the sums also go through a ReLU / leaky ReLU, act_out[i] = t > 0 ? t : alpha t, the
// layer behind a dense product whose K was split (what relu_fwd_kernel would write from dw in a launch of its own).
// (the body takes the workgroup's number as an argument: see BlockId)
static __device__ __forceinline__ void reduce_splits4_body(const unsigned block, const float* __restrict__ part, float* __restrict__ dw,
                                                           float* __restrict__ dbias, int n_dw, int n, int stride, int splits, int tr,
                                                           float* __restrict__ act_out, float alpha) {
    __shared__ f4 red[16][16];
    const int cg = threadIdx.x & 15;                     // group of 4 outputs
    const int sl = threadIdx.x >> 4;                     // split lane
    const int i = (block * 16 + cg) * 4;
    f4 s = {0.f, 0.f, 0.f, 0.f};
    if (i < n) {
        const float* q = part + i;
        int k = sl;
        f4 s0 = s, s1 = s, s2 = s, s3 = s;
        for (; k + 48 < splits; k += 64) {
            s0 += *reinterpret_cast<const f4*>(q + (size_t)k * stride);
            s1 += *reinterpret_cast<const f4*>(q + (size_t)(k + 16) * stride);
            s2 += *reinterpret_cast<const f4*>(q + (size_t)(k + 32) * stride);
            s3 += *reinterpret_cast<const f4*>(q + (size_t)(k + 48) * stride);
        }
        for (; k < splits; k += 16) s0 += *reinterpret_cast<const f4*>(q + (size_t)k * stride);
        s = (s0 + s1) + (s2 + s3);
    }
    red[sl][cg] = s;
    __syncthreads();
    if (sl == 0 && i < n) {
        f4 t = red[0][cg];
#pragma unroll
        for (int j = 1; j < 16; ++j) t += red[j][cg];
        if (i < n_dw && tr > 0) {
            const int r = i / tr, c = i - r * tr, ld = n_dw / tr;
#pragma unroll
            for (int e = 0; e < 4; ++e) dw[(c + e) * ld + r] = t[e];
        } else if (i < n_dw) {
            *reinterpret_cast<f4*>(dw + i) = t;
            if (act_out != nullptr) {
                f4 a;
#pragma unroll
                for (int e = 0; e < 4; ++e) a[e] = t[e] > 0.f ? t[e] : alpha * t[e];
                *reinterpret_cast<f4*>(act_out + i) = a;
            }
        } else if (dbias != nullptr) {
            *reinterpret_cast<f4*>(dbias + (i - n_dw)) = t;
        }
    }
}

static __global__ __launch_bounds__(kThreads) void reduce_splits4(const float* __restrict__ part, float* __restrict__ dw,
                                                          float* __restrict__ dbias, int n_dw, int n, int stride,
                                                          int splits, int tr = 0, float* __restrict__ act_out = nullptr,
                                                          float alpha = 0.f) {
    reduce_splits4_body(blockIdx.x, part, dw, dbias, n_dw, n, stride, splits, tr, act_out, alpha);
}

static inline int check_conv_dims(const char* fn, int S, int H, int W, int C, int D, int fH, int fW,
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

}  // namespace aeth
