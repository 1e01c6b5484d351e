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
    const void* bt;      // packed filter [Npad][Kpad] of T, zero filled
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
    // gather_halo_bf16: columns and rows of the padded source image, 256-row tiles per image (0: tiles
    // run over image boundaries)
    int halo_wp, halo_hp, halo_tiles;
    FastDiv div_hw, div_w, div_c, div_tw, div_halo_wp, div_halo_hp, div_halo_tiles;
};

constexpr int kInvalidRow = -16384;
constexpr int kNloopMaxN = 1024;   // widest output the n-loop mode of the gather kernel takes (its bias sits in LDS)
constexpr int kXcds = 8;

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

template <typename T, int BM, int BN, int WM, int WN, bool UT, int KC, bool NLOOP, bool SA = false>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN)) void gather_gemm_dma(const GatherParams p) {
    // 4 waves, or 8 for the widest bf16 tiles (256 x 128 and 256 x 256: one workgroup per CU)
    constexpr int NW = (BM / WM) * (BN / WN);
    static_assert(NW == 4 || (NW == 8 && !NLOOP && !SA), "4 or 8 waves per workgroup");
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

    __shared__ f4 lds_a0[BM * KC];
    __shared__ f4 lds_a1[BM * KC];
    __shared__ f4 lds_b0[BN * KC];
    __shared__ f4 lds_b1[BN * KC];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int wm0 = (wave % (BM / WM)) * WM;
    const int wn0 = (wave / (BM / WM)) * WN;
    const int ntile = (p.N + BN - 1) / BN;
    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    // (one n tile: no division; the compiler divides scalars by way of the vector unit's reciprocal, some 20
    // vector instructions that a workgroup starting next to busy ones waits for one by one)
    const int mt = (NLOOP || ntile == 1) ? lid : lid / ntile;
    const int m0 = mt * BM;
    int n0 = (NLOOP || ntile == 1) ? 0 : (lid - mt * ntile) * BN;

    // The bias is fetched first: its latency passes behind the row decode.
    const int split = (int)blockIdx.y;
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
            const int k4 = k4e ^ (((wave * BL + i) & 1) ? ODD : 0);
            b_off[i] = (unsigned)(((n0 + (wave * BL + i) * RPL + lr) * p.Kpad + CE * k4) * (int)sizeof(T));
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
    int tap_off[2] = {0, 0}, tap_h[2] = {0, 0}, tap_w[2] = {0, 0};
    bool kvalid[2] = {false, false};
    auto prep = [&](int k0) {
        if (UT) {
            unsigned c0, th, tw;
            p.div_c.divmod((unsigned)k0, ut_tap, c0);
            p.div_tw.divmod(ut_tap, th, tw);
            ut_tap_bytes = (unsigned)(((int)th * p.Ws + (int)tw) * p.Cs + (int)c0) * (unsigned)sizeof(T);
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
                lds_direct_load16_s(sa_rsrc_b, lds_address(lb) + (unsigned)(wave_u * BL + i) * 1024u, b_off[i],
                                    (unsigned)k0 * (unsigned)sizeof(T));
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
                                                     (int)(b_off[i] + (unsigned)k0 * (unsigned)sizeof(T)), 0, 0, 0);
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
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[slot][j] = lb[(wn0 + 32 * j + l32) * KC + pc];
    };
    auto mma_group = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) mma_chunk<T>(fb[slot][j], fa[slot][i], acc[i][j]);
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
                        for (int j = 0; j < TN; ++j)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[g & 1][j][t], fa[g & 1][i][t], acc[i][j], 0, 0, 0);
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
    fill_acc<TM, TN>(bv, acc);
    for (int s = s_begin; s < nslabs; s += 2) {
        slab(lds_a0, lds_b0, lds_a1, lds_b1, (s + 1) * BK, s + 1 < nslabs);
        if (s + 1 < nslabs) slab(lds_a1, lds_b1, lds_a0, lds_b0, (s + 2) * BK, s + 2 < nslabs);
    }

    store_tile<TM, TN>(p, p.out + (size_t)split * p.M * p.N, acc, m0 + wm0, n0 + wn0, l32, lh);
}

// ------------------------------------------------------------------------------
// gather_gemm_persist: the uniform-tap, 8-chunk-slab form of gather_gemm_dma for launches of many
// rounds of tiles.  A one-tile workgroup spends a sixth of its life outside the slab loop (row decode,
// the first slab's memory latency, the epilogue), and the workgroups that share a CU start together and
// stay in step, so those gaps reach the matrix pipe.  Here 3 workgroups per CU stay resident and walk
// tiles; the slab loop runs through the tile boundaries: the last slab of a tile issues the loads of the
// next tile's first slab, the next tile's row table is worked out by the threads of slab 1 and picked up
// at the last slab, and a finished tile stays in the accumulators until the next tile's first slab has
// begun: it is stored there, behind that slab's loads, and the accumulators start again from the bias.  Slab order, operand reads and MFMA order are those of gather_gemm_dma: the
// results are bit-identical.  Measured on the 56x56x64 layer the time is linear in the number of tiles
// with this kernel and with the one-tile kernel alike (57.4 us per 768 tiles from 4.6 to 8.2 rounds): what
// bounds both is the slab loop itself, not the start and the end of a workgroup or the last round, so this
// kernel is kept as a tuning switch only.
// Round i gives workgroup b the tile i * G + (b's place in an XCD-contiguous order), so that one XCD works
// on neighbouring image rows at the same time; the last, partial round goes to the first workgroups in
// launch order, which are spread over all XCDs.
// ------------------------------------------------------------------------------
constexpr int kPersistMaxN = 512;

template <typename T, int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(kThreads, 3) void gather_gemm_persist(const GatherParams p, const int tiles) {
    static_assert((BM / WM) * (BN / WN) == 4, "4 waves per workgroup");
    constexpr int KC = 8;
    constexpr int CE = Elem<T>::CE;
    constexpr int BK = KC * CE;
    constexpr int RPL = 64 / KC;
    constexpr int G = KC / 2;
    constexpr int AL = BM / (4 * RPL);
    constexpr int BL = BN / (4 * RPL);
    static_assert(AL >= 2 && AL % 2 == 0 && BL >= 1, "8-row load blocks of a wave alternate even/odd");
    static_assert(BM <= kThreads, "one thread per row of the table");
    constexpr int TM = WM / 32;
    constexpr int TN = WN / 32;

    __shared__ f4 lds_a0[BM * KC];
    __shared__ f4 lds_a1[BM * KC];
    __shared__ f4 lds_b0[BN * KC];
    __shared__ f4 lds_b1[BN * KC];
    __shared__ int2 rowtab[BM];
    __shared__ __attribute__((aligned(16))) float lds_bias[kPersistMaxN];   // zeros past N and without a bias

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int l32 = lane & 31;
    const int lh = lane >> 5;
    const int wm0 = (wave % (BM / WM)) * WM;
    const int wn0 = (wave / (BM / WM)) * WN;
    const int ntile = (p.N + BN - 1) / BN;
    const int nwg = (int)gridDim.x;
    const int rounds = tiles / nwg, rest = tiles - rounds * nwg;
    const int my_count = rounds + ((int)blockIdx.x < rest ? 1 : 0);
    if (my_count == 0) return;
    const int lid = xcd_contiguous_id((int)blockIdx.x, nwg);
    auto tile_of = [&](int i) { return i < rounds ? i * nwg + lid : rounds * nwg + (int)blockIdx.x; };

    const int lr = lane / KC;
    const int k4e = (lane & 7) ^ (lane >> 4);
    // (element offset of tap (0,0), one bit per tap that says "outside the image") of row m0 + tid
    auto decode_rows = [&](int m0) {
        if (tid < BM) {
            const int m = m0 + tid;
            int off = 0, br = kInvalidRow, bc = 0;
            if (m < p.M) {
                unsigned s_, rem, ii, jj;
                p.div_hw.divmod((unsigned)m, s_, rem);
                p.div_w.divmod(rem, ii, jj);
                br = (int)ii * p.sh + p.rh0;
                bc = (int)jj * p.sw + p.rw0;
                off = (((int)s_ * p.Hs + br) * p.Ws + bc) * p.Cs;
            }
            auto span = [](int lo, int hi) -> unsigned {
                const unsigned upto_hi = hi > 0 ? ~0u >> (32 - hi) : 0u;
                const unsigned upto_lo = lo > 0 ? ~0u >> (32 - lo) : 0u;
                return hi > lo ? upto_hi & ~upto_lo : 0u;
            };
            const int lo_r = min(max(-br, 0), 32), hi_r = min(max(p.Hs - br, 0), p.Th);
            const int lo_c = min(max(-bc, 0), 32), hi_c = min(max(p.Ws - bc, 0), p.Tw);
            const unsigned rmask = span(lo_r, hi_r), cmask = span(lo_c, hi_c);
            unsigned valid = 0;
            for (int th = 0; th < p.Th; ++th) valid |= (((rmask >> th) & 1u) ? cmask : 0u) << (th * p.Tw);
            rowtab[tid] = int2{off, (int)~valid};
        }
    };
    // Loads addressed on the scalar unit, as in the SA form of gather_gemm_dma: a lane's offset is a constant
    // of the tile, counted from a base the padding below the tensor; lane l keeps the outside-the-image bits,
    // one per tap, of the wave's row l % 32, and a ballot per slab makes the 32 rows' mask of the slab's tap.
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);
    const unsigned sa_bias = (unsigned)((max(-p.rh0, 0) * p.Ws + max(-p.rw0, 0)) * p.Cs) * (unsigned)sizeof(T);
    unsigned a_byte[AL], b_off[BL], aux_row = 0, cur_mask = 0;
    auto take_rows = [&]() {
#pragma unroll
        for (int i = 0; i < AL; ++i) {
            const int2 e = rowtab[(wave * AL + i) * RPL + lr];
            a_byte[i] = (unsigned)(e.x + CE * (k4e ^ ((i & 1) ? 4 : 0))) * (unsigned)sizeof(T) + sa_bias;
        }
        aux_row = (unsigned)rowtab[wave * (AL * RPL) + (lane & (AL * RPL - 1))].y;
    };
    auto set_b_off = [&](int n0) {
#pragma unroll
        for (int i = 0; i < BL; ++i) {
            const int k4 = k4e ^ (((wave * BL + i) & 1) ? 4 : 0);
            b_off[i] = (unsigned)(((n0 + (wave * BL + i) * RPL + lr) * p.Kpad + CE * k4) * (int)sizeof(T));
        }
    };
    const u32x4 rsrc_a = raw_rsrc(static_cast<const char*>(p.src) - sa_bias, (unsigned)p.src_bytes + sa_bias);
    const u32x4 rsrc_b = raw_rsrc(p.bt, (unsigned)p.bt_bytes);

    unsigned ut_tap = 0, ut_tap_bytes = 0;
    auto prep = [&](int k0) {
        unsigned c0, th, tw;
        p.div_c.divmod((unsigned)k0, ut_tap, c0);
        p.div_tw.divmod(ut_tap, th, tw);
        ut_tap_bytes = (unsigned)(((int)th * p.Ws + (int)tw) * p.Cs + (int)c0) * (unsigned)sizeof(T);
        cur_mask = (unsigned)__builtin_amdgcn_ballot_w64(((aux_row >> ut_tap) & 1u) != 0u);
    };
    auto issue_load = [&](int j, int k0, f4* la, f4* lb) {
        if (j >= AL) {
            const int i = j - AL;
            lds_direct_load16_s(rsrc_b, lds_address(lb) + (unsigned)(wave_u * BL + i) * 1024u, b_off[i],
                                (unsigned)k0 * (unsigned)sizeof(T));
            return;
        }
        const unsigned m8 = (cur_mask >> (RPL * j)) & ((1u << RPL) - 1u);
        const unsigned dst = lds_address(la) + (unsigned)(wave_u * AL + j) * 1024u;
        if (m8 != 0u) lds_direct_load16_s(rsrc_a, dst, select_by_mask(a_byte[j], 0x80000000u, spread_rows<KC>(m8)), ut_tap_bytes);
        else lds_direct_load16_s(rsrc_a, dst, a_byte[j], ut_tap_bytes);
    };
    constexpr int NL = AL + BL;
    static_assert(TM * TN == 2 && NL <= 2 * (G - 1), "one load in front of each run of 4 MFMAs");

    f16v acc[TM][TN];
    const int sw7 = (l32 >> 1) & (KC - 1);
    f4 fa[2][TM], fb[2][TN];
    auto read_frags = [&](const f4* la, const f4* lb, int g, int slot) {
        const int pc = (2 * g + lh) ^ sw7;
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[slot][i] = la[(wm0 + 32 * i + l32) * KC + pc];
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[slot][j] = lb[(wn0 + 32 * j + l32) * KC + pc];
    };

    // the first tile: as a one-tile workgroup starts
    const int nslabs = p.Kpad / BK;
    int ti = 0, s = 0;
    int m0, n0;
    {
        const int t = tile_of(0);
        m0 = (t / ntile) * BM;
        n0 = (t % ntile) * BN;
    }
    for (int n = tid; n < kPersistMaxN; n += kThreads) lds_bias[n] = (p.bias != nullptr && n < p.N) ? p.bias[n] : 0.f;
    decode_rows(m0);
    __syncthreads();
    take_rows();
    set_b_off(n0);
    prep(0);
#pragma unroll
    for (int j = 0; j < NL; ++j) issue_load(j, 0, lds_a0, lds_b0);
    // a tile's accumulators start from the bias of its channels
    auto start_acc = [&](int nw0) {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const f4 v = *reinterpret_cast<const f4*>(lds_bias + nw0 + 32 * j + 8 * q + 4 * lh);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = v[e];
            }
    };
    int done_m0 = 0, done_n0 = 0;
    bool have_done = false;

    auto step = [&](const f4* la, const f4* lb, f4* na, f4* nb) __attribute__((always_inline)) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        read_frags(la, lb, 0, 0);
        const bool last = s == nslabs - 1;
        const bool more_tiles = ti + 1 < my_count;
        bool has_next = true;
        int next_k0 = (s + 1) * BK;
        int nm0 = 0, nn0 = 0;
        if (last) {
            next_k0 = 0;
            has_next = more_tiles;
            if (more_tiles) {
                // from here on this wave's loads belong to the next tile
                const int t = tile_of(ti + 1);
                nm0 = (t / ntile) * BM;
                nn0 = (t % ntile) * BN;
                take_rows();
                set_b_off(nn0);
            }
        }
        if (has_next) prep(next_k0);
        if (s == 0) {
            // the finished tile is still in the accumulators: it is stored here, behind the loads of this
            // tile's first slab, and the accumulators then start again from the bias
            if (have_done) store_tile<TM, TN, true>(p, p.out, acc, done_m0 + wm0, done_n0 + wn0, l32, lh);
            start_acc(n0 + wn0);
        }
        if (s == 1 && more_tiles) decode_rows((tile_of(ti + 1) / ntile) * BM);
#pragma unroll
        for (int g = 0; g < G; ++g) {
            if (g < G - 1) read_frags(la, lb, g + 1, (g + 1) & 1);
            // one load in front of each run of 4 MFMAs; consecutive MFMAs go to different accumulator blocks
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int c = 2 * g + t / 2;
                if (has_next && c < NL && t % 2 == 0) issue_load(c, next_k0, na, nb);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[g & 1][j][t], fa[g & 1][i][t], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (last) {
            done_m0 = m0;
            done_n0 = n0;
            have_done = true;
            m0 = nm0;
            n0 = nn0;
            ++ti;
            s = 0;
        } else {
            ++s;
        }
    };
    // The workgroups of a CU start a third of a slab apart (launch order b / 8 modulo 3 differs between the
    // three that share a CU whether the dispatcher fills a CU first or deals them round): started together
    // they reach their barriers together, slab after slab, and the matrix pipe drains each time
    // (0.491 -> 0.470 ms on the 56x56x64 layer).
    {
        const int ph = ((int)blockIdx.x >> 3) % 3;
        if (ph >= 1) __builtin_amdgcn_s_sleep(36);
        if (ph >= 2) __builtin_amdgcn_s_sleep(36);
    }
    const int total = my_count * nslabs;
    for (int f = 0; f < total; f += 2) {
        step(lds_a0, lds_b0, lds_a1, lds_b1);
        if (f + 1 < total) step(lds_a1, lds_b1, lds_a0, lds_b0);
    }
    store_tile<TM, TN, true>(p, p.out, acc, done_m0 + wm0, done_n0 + wn0, l32, lh);
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
//   * slot s keeps logical 16-byte chunk c at position c ^ ((s >> 1) & 7), like the
//     slab rows of gather_gemm_dma: 16 consecutive pixels cover the 64 banks once;
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

template <int STAGES>
static __global__ __launch_bounds__(kThreads, 2) void gather_halo_bf16(const GatherParams p) {
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
    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
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
    int* tab = reinterpret_cast<int*>(ring_last);
    for (int sl = tid; sl < kHaloSlots; sl += kThreads) {
        unsigned rg, cc, s_, rr;
        p.div_halo_wp.divmod((unsigned)(lfirst + sl), rg, cc);
        p.div_halo_hp.divmod(rg, s_, rr);
        const int srow = (int)rr + p.rh0, scol = (int)cc + p.rw0;
        const bool ok = sl < span && (unsigned)srow < (unsigned)p.Hs && (unsigned)scol < (unsigned)p.Ws && (int)s_ < p.S;
        const unsigned off = (unsigned)((((int)s_ * p.Hs + srow) * p.Ws + scol) * p.Cs) * 2u;
        tab[sl] = (int)(ok ? off : 0x80000000u);
    }
    __syncthreads();
    unsigned hoff[HL];
#pragma unroll
    for (int k = 0; k < HL; ++k) {
        const int sl = (wave * HL + k) * 8 + (lane >> 3);
        hoff[k] = (unsigned)tab[sl] + (unsigned)((((lane & 7) ^ (sl >> 1)) & 7) * 16);
    }
    // slot of tap (0,0) for the pixels this lane multiplies (rows past the end: slot 0, never stored)
    int pslot[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm0 + 32 * i + l32;
        pslot[i] = m < m_end ? slot0(m) - lfirst : 0;
    }
    // filter slab loads: as in gather_gemm_dma (rows of 8 chunks, chunk c of row r at c ^ ((r >> 1) & 7))
    const int k4e = (lane & 7) ^ (lane >> 4);
    unsigned b_off[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int k4 = k4e ^ (((wave * 2 + i) & 1) ? 4 : 0);
        b_off[i] = (unsigned)(((n0 + (wave * 2 + i) * 8 + (lane >> 3)) * p.Kpad + 8 * k4) * 2);
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
    auto pf_next = [&]() __attribute__((always_inline)) {
        const unsigned k0_bytes = pf_cb < p.Cs / BK ? (unsigned)(pf_tap * p.Cs + pf_cb * BK) * 2u : 0x80000000u;
        if (++pf_tap == T) { pf_tap = 0; ++pf_cb; }
        return k0_bytes;
    };
    load_halo(0);
    load_filter(pf_next(), ring0);
    load_filter(pf_next(), ring1);
    if constexpr (STAGES == 4) load_filter(pf_next(), ring2);

    f16v acc[TM][TN];
    fill_acc<TM, TN>(bv, acc);

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
        const int shift = th * Wp + tw;
        int x0[TM];
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int sl = pslot[i] + shift;
            x0[i] = sl * 8 + ((lh ^ (sl >> 1)) & 7);
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
                for (int j = 0; j < TN; ++j) mma_chunk<uint16_t>(fb[g][j], fa[g][i], acc[i][j]);
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
    store_tile<TM, TN>(p, p.out, acc, m0 + wm0, n0, l32, lh, m_end);
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
                const int n = part * 8 + (lane >> 3);
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
                    const int pos = ((c >> 3) ^ ((n2 >> 1) & 7)) * 16 + (c & 7) * 2;   // n2 and n2 + 1 share the key
                    *reinterpret_cast<unsigned*>(fbytes + tap * 8192 + n2 * 128 + pos) = (a & 0xffffu) | (b << 16);
                    *reinterpret_cast<unsigned*>(fbytes + tap * 8192 + (n2 + 1) * 128 + pos) = (a >> 16) | (b & 0xffff0000u);
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
            rel[i] = ((int)r * p.Ws + (int)c) * 128 + (((lane & 7) ^ (sl >> 1)) & 7) * 16;
            const unsigned bad = (unsigned)((int)c + p.rw0) >= (unsigned)p.Ws ? 1u : 0u;
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
    __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (0 << 8));                   // this wave's part of the filter
    asm volatile("s_barrier" ::: "memory");
    for (int t = 0; t < ntl; ++t) {
        unsigned s_img, t_img;
        p.div_halo_tiles.divmod((unsigned)(tile0 + t), s_img, t_img);
        const int m0 = (int)s_img * hw + (int)t_img * BM;
        const int m_end = ((int)s_img + 1) * hw;                           // rows past the image: multiplied, never stored
        const f4* h = halo[t & 1];
        f16v acc[1][TN];
        fill_acc<1, TN>(bv, acc);
        // the operands of tap u + 1 are read while the MFMAs of tap u run (two sets of 48 registers)
        int th = 0, tw = 0;
        f4 fa[2][4], fb[2][4][TN];
        auto read_tap = [&](int tap, f4 (&ra)[4], f4 (&rb)[4][TN]) __attribute__((always_inline)) {
            const int sl = pslot + th * Wp + tw;
            const int x0 = sl * 8 + ((lh ^ (sl >> 1)) & 7);
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
                for (int j = 0; j < TN; ++j) mma_chunk<uint16_t>(rb[g][j], ra[g], acc[0][j]);
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
            if (tap == store_after && have_done) store_tile<1, TN>(p, p.out, done, done_m0, 0, l32, lh, done_end);
            if (tap + 1 < T) {
                if (tap + 2 < T) read_tap(tap + 2, fa[0], fb[0]);
                multiply(fa[1], fb[1]);
                if (tap + 1 == store_after && have_done) store_tile<1, TN>(p, p.out, done, done_m0, 0, l32, lh, done_end);
            }
        }
        have_done = true;
#pragma unroll
        for (int j = 0; j < TN; ++j) done[0][j] = acc[0][j];
        done_m0 = m0 + wave * 32;
        done_end = m_end;
        asm volatile("s_barrier" ::: "memory");
    }
    if (have_done) store_tile<1, TN>(p, p.out, done, done_m0, 0, l32, lh, done_end);
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

template <int NSLAB>                                   // K = 32 * NSLAB
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
            const unsigned off = (unsigned)(((part * 8 + prow) * p.Kpad + 32 * sl + 4 * k4) * 4);
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
    unsigned rela[2 * (BM / 8)];
#pragma unroll
    for (int i = 0; i < 2 * (BM / 8); ++i) {
        const int sl = i / (BM / 8), part = i % (BM / 8);
        const int k4 = k4e ^ ((part & 1) ? 4 : 0);
        rela[i] = (unsigned)(((part * 8 + prow) * p.Cs + 32 * sl + 4 * k4) * 4);
    }
    auto fetch = [&](int tile, int buf) __attribute__((always_inline)) {
        const unsigned base = (unsigned)tile * (unsigned)(BM * p.Cs * 4);
#pragma unroll
        for (int i = 0; i < 2 * (BM / 8); ++i) {
            if (i < nslab * (BM / 8)) {
                const int sl = i / (BM / 8), part = i % (BM / 8);
                lds_direct_load16(rsrc_a, lds_address(&abuf[buf][sl][0]) + (unsigned)part * 1024u, base + rela[i]);
            }
        }
    };
    if (wave == 0 && ntl > 0) fetch(tile0, 0);
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("s_barrier" ::: "memory");

    const int sw7 = (l32 >> 1) & 7;
    f16v acc[TM][TN], done[TM][TN];
    int done_m0 = 0;
    bool have_done = false;
    auto store_done = [&]() __attribute__((always_inline)) {
        store_tile<TM, TN, true>(p, p.out, done, done_m0 + wm0, wn0, l32, lh);
    };
    for (int t = 0; t < ntl; ++t) {
        if (wave == 0 && t + 1 < ntl) fetch(tile0 + t + 1, (t + 1) & 1);
        if (active) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f4 b = bias_lds[(wn0 + 32 * j + 8 * q + 4 * lh) >> 2];
#pragma unroll
                    for (int i = 0; i < TM; ++i)
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[i][j][4 * q + e] = b[e];
                }
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
                        for (int j = 0; j < TN; ++j) mma_chunk<float>(fb[u & 1][j], fa[u & 1][i], acc[i][j]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // the finished tile leaves after k group `wave` (a few 16-byte pieces after every group
                // were slower: 0.298 ms against 0.266 on 56x56, 64 -> 256)
                if (have_done && u == min(wave, 4 * nslab - 1)) store_done();
            }
            have_done = true;
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) done[i][j] = acc[i][j];
            done_m0 = (tile0 + t) * BM;
        }
        if (wave == 0) __builtin_amdgcn_s_waitcnt(0 | (7 << 4) | (15 << 8));   // the next tile's rows (and its own old stores)
        asm volatile("s_barrier" ::: "memory");
    }
    if (active && have_done) store_done();
}

// dense_res_f32 applies to fp32 gathers that are plain matrix products (one tap, unit stride, no
// padding), K = 32 or 64 whole, N a multiple of 4 up to 256 with more than one 64-wide tile, a dense
// output with 16-byte stores, and at least 4 tiles of 128 rows per CU (AETHER_DENSE_RES=1 drops the
// last condition, =0 turns the kernel off).
static bool plan_dense_res(const GatherParams& gp, bool dma, int cus, int* mtiles) {
    if (!dma || gp.sh != 1 || gp.sw != 1 || gp.rh0 != 0 || gp.rw0 != 0 || gp.Hs != gp.Hg || gp.Ws != gp.Wg) return false;
    if (gp.K != gp.Cs || gp.K != gp.Kpad || (gp.K != 32 && gp.K != 64) || gp.split_slabs != 0) return false;
    if (gp.N <= 64 || gp.N > kD1MaxN || !gp.dense_out || gp.out_bytes == 0) return false;
    bool force = false;
    if (const char* f = getenv("AETHER_DENSE_RES")) {
        if (atoi(f) == 0) return false;
        force = true;
    }
    const int n = cdiv(gp.M, kD1BM);
    if (!force && n < 4 * cus) return false;
    *mtiles = n;
    return true;
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

template <typename T, int BM, int BN, int WM, int WN, int KC>
static void launch_gather_dma(const GatherParams& gp, hipStream_t st) {
    constexpr int kThreads = 64 * (BM / WM) * (BN / WN);     // of this tile shape (shadows the 256 of the others)
    dim3 grid(cdiv(gp.M, BM) * cdiv(gp.N, BN));
    if (gp.split_slabs > 0) grid.y = (unsigned)cdiv(gp.Kpad / (KC * Elem<T>::CE), gp.split_slabs);
    const bool ut = gp.Cs % (KC * Elem<T>::CE) == 0 && gp.K == gp.Kpad && gp.K / gp.Cs <= 32;
    // short K, several n tiles: one workgroup per m tile walks the n tiles (128 x 64 tiles only)
    if constexpr (BM == 128 && BN == 64 && KC == 8) {
        if (gp.split_slabs == 0 && gp.Kpad / (KC * Elem<T>::CE) <= 2 && gp.N > BN && gp.N <= kNloopMaxN && gp.out_bytes != 0 &&
            getenv("AETHER_GATHER_NLOOP_OFF") == nullptr) {
            grid.x = (unsigned)cdiv(gp.M, BM);
            if (ut) hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, true>), grid, dim3(kThreads), 0, st, gp);
            else hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, false, KC, true>), grid, dim3(kThreads), 0, st, gp);
            return;
        }
    }
    if constexpr ((BM == 128 || BM == 64) && sizeof(T) == 4) {
        // scalar addressing (AETHER_GATHER_SA=0 turns it off); the moved base must stay a 32-bit extent
        const int taps = gp.Cs > 0 ? gp.K / gp.Cs : 0;
        const int64_t bias = ((int64_t)std::max(-gp.rh0, 0) * gp.Ws + std::max(-gp.rw0, 0)) * gp.Cs * (int64_t)sizeof(T);
        const char* f = getenv("AETHER_GATHER_SA");
        if (ut && taps <= 32 && (int64_t)gp.src_bytes + bias < ((int64_t)1 << 31) && (f == nullptr || atoi(f) != 0)) {
            hipLaunchKernelGGL((gather_gemm_dma<T, BM, BN, WM, WN, true, KC, false, true>), grid, dim3(kThreads), 0, st, gp);
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

// Tile height.  The LDS-direct kernel keeps two slabs per operand in LDS, so a
// 128-row tile (48 KB) lets three workgroups share a CU where a 256-row tile
// (80 KB) allows one or two; measured on the 56x56x64 shape, 128 rows is 11 %
// faster.  64-row tiles (32 KB, five per CU) run at the same rate and leave a
// smaller last round, so fp32 takes 128 rows only from about 8 rounds of tiles on
// (6272 tiles, 56x56x64: 0.483 ms either way; 1568 tiles, 56x56x256 batch 64: 0.503 ms
// with 128 rows, 0.488 with 64).  The register-staged kernel prefers 256 rows.
static inline int gather_bm(int M, int N, int cus, bool dma, int elem_bytes = 4) {
    const int bn = gather_bn(N);
    if (const char* f = getenv("AETHER_GATHER_BM")) {       // tuning override: 256, 128 or 64
        int v = atoi(f);
        if (v == 256 || v == 128 || (v == 64 && bn == 64)) return v;
    }
    const int ntiles = cdiv(N, bn);
    const int want = elem_bytes == 2 ? cus : 2 * cus;   // bf16: the taller tile pays off from one tile per CU on
    const int cands[3] = {256, 128, 64};
    // bf16 MFMAs are 8x shorter per slab: there the larger wave tile of the 256-row shape wins
    for (int i = (dma && elem_bytes == 4) ? 1 : 0; i < 3; ++i) {
        int bm = cands[i];
        if (bn == 32 && bm == 64) break;
        const int64_t tiles = (int64_t)cdiv(M, bm) * ntiles;
        if (dma && elem_bytes == 4 && bm == 128 && bn == 64 && tiles < 24 * (int64_t)cus) continue;
        if (tiles >= want) return bm;
    }
    return bn == 32 ? 128 : 64;
}

// gather_halo_bf16 applies to unit-stride gathers of 2 to 32 taps over whole 64-channel blocks
// when the span of every tile fits its buffer: with tiles cut per image (at most 10 % of empty
// rows) or, failing that, running over image boundaries.  Fills the halo fields of gp and the
// number of 256-row tiles when it does.
static bool plan_halo(GatherParams& gp, bool dma, int* mtiles, int* stages) {
    if (!dma || gp.sh != 1 || gp.sw != 1 || gp.Cs % 64 != 0 || gp.K != gp.Kpad || gp.split_slabs != 0) return false;
    const int taps = gp.Th * gp.Tw;
    if (taps < 2 || taps > 32 || gp.N <= 32 || gp.Cs <= 0 || gp.K != taps * gp.Cs) return false;
    if (getenv("AETHER_GATHER_HALO_OFF") != nullptr) return false;
    const int hw = gp.Hg * gp.Wg;
    const int wp = gp.Wg + gp.Tw - 1, hp = gp.Hg + gp.Th - 1;
    if ((int64_t)gp.S * hp * wp >= ((int64_t)1 << 30)) return false;
    auto slot0 = [&](int64_t m) {
        const int64_t s = m / hw, rem = m % hw;
        return (s * hp + rem / gp.Wg) * wp + rem % gp.Wg;
    };
    int64_t longest = 0;
    auto fits = [&](int64_t first, int64_t last) {
        const int64_t span = slot0(last) + (int64_t)(gp.Th - 1) * wp + gp.Tw - slot0(first);
        longest = std::max(longest, span);
        return span <= kHaloSlotsMax;
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
// there are at least 4 tiles per CU to walk (AETHER_GATHER_RES=1 drops the last condition,
// =0 turns the kernel off).
static bool plan_halo_res(GatherParams& gp, bool dma, int cus, int* mtiles) {
    if (!dma || gp.sh != 1 || gp.sw != 1 || gp.Cs != 64 || gp.K != gp.Kpad || gp.split_slabs != 0) return false;
    const int taps = gp.Th * gp.Tw;
    if (taps < 2 || taps > kResMaxTaps || gp.N <= 32 || gp.N > 64 || gp.K != taps * gp.Cs) return false;
    bool force = false;
    if (const char* f = getenv("AETHER_GATHER_RES")) {
        if (atoi(f) == 0) return false;
        force = true;
    }
    if (getenv("AETHER_GATHER_HALO_OFF") != nullptr) return false;
    if (gp.Wg <= 0 || kResBM % gp.Wg != 0) return false;
    const int hw = gp.Hg * gp.Wg;
    const int wp = gp.Wg + gp.Tw - 1, hp = gp.Hg + gp.Th - 1;
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

// gather_gemm_persist applies to fp32 launches of 128 x 64 tiles whose slabs lie inside one tap (channels
// in whole slabs of 32, at most 32 taps), with 3 slabs or more, no split of K, 16-byte stores and at most
// 512 output channels.  It runs only when AETHER_GATHER_PERSIST=1 asks for it: on the 56x56x64 layer it is
// 3 % faster than the one-tile kernel where launches of one direction follow each other, no faster in a
// training step or alone, and its workgroups, which all walk the taps at the same time, fetch 40 % more
// through L2 (295 MB against 216 MB per launch).
static bool plan_persist(const GatherParams& gp, bool dma, int* tiles) {
    if (!dma || gp.split_slabs != 0 || gp.Cs % 32 != 0 || gp.K != gp.Kpad || gp.K / gp.Cs > 32 || gp.Kpad / 32 < 3) return false;
    if (gp.N > kPersistMaxN || gp.out_bytes == 0) return false;
    // the descriptor of the source starts the padding below the tensor: its extent must stay a 32-bit offset
    const int64_t bias = ((int64_t)std::max(-gp.rh0, 0) * gp.Ws + std::max(-gp.rw0, 0)) * gp.Cs * 4;
    if ((int64_t)gp.src_bytes + bias >= ((int64_t)1 << 31)) return false;
    const char* f = getenv("AETHER_GATHER_PERSIST");
    if (f == nullptr || atoi(f) == 0) return false;
    const int64_t n = (int64_t)cdiv(gp.M, 128) * cdiv(gp.N, 64);
    if (n > (1 << 30)) return false;
    *tiles = (int)n;
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
            if (stages == 4) hipLaunchKernelGGL(gather_halo_bf16<4>, grid, dim3(kThreads), 0, st, hp);
            else hipLaunchKernelGGL(gather_halo_bf16<3>, grid, dim3(kThreads), 0, st, hp);
            return;
        }
    }
    if constexpr (sizeof(T) == 2) {
        // Wide tiles for bf16 launches that the halo kernels do not take (strides, 1x1, long filters): the
        // slab kernel with 256 x 64 tiles fetches (256 + 64) rows of k per 256 x 64 outputs, 11.5 TB/s from
        // L2 on the 28x28x128 -> 256 stride-2 layer, and that rate is what bounds it; 256 x 256 tiles on 8 waves
        // (one workgroup per CU, 128 KB of slabs) fetch 2.5 times less per output, 256 x 128 tiles 1.7 times.
        // From 2 (256 wide) or 4 (128 wide) tiles per CU on (AETHER_GATHER_WIDE=1: always, =0: never).
        const char* f = getenv("AETHER_GATHER_WIDE");
        const bool force = f != nullptr && atoi(f) != 0;
        if (dma && gp.split_slabs == 0 && !(f != nullptr && atoi(f) == 0)) {
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
            if (gp.Kpad == 64) hipLaunchKernelGGL(dense_res_f32<2>, grid, dim3(kD1Threads), 0, st, gp, mtiles);
            else hipLaunchKernelGGL(dense_res_f32<1>, grid, dim3(kD1Threads), 0, st, gp, mtiles);
            return;
        }
    }
    const int bm = gather_bm(gp.M, gp.N, cus, dma, (int)sizeof(T));
    if constexpr (sizeof(T) == 4) {
        int tiles = 0;
        if (bm == 128 && bn == 64 && plan_persist(gp, dma, &tiles)) {
            int wgs = std::min(tiles, 3 * cus);
            // AETHER_GATHER_PERSIST_WGS: fewer workgroups, so that small inputs give each of them several tiles
            if (const char* f = getenv("AETHER_GATHER_PERSIST_WGS")) wgs = std::max(1, std::min(wgs, atoi(f)));
            hipLaunchKernelGGL((gather_gemm_persist<T, 128, 64, 32, 64>), dim3((unsigned)wgs), dim3(kThreads), 0, st, gp, tiles);
            return;
        }
    }
    // shallow slabs measure the same as deep ones on the 56x56 layers (within 2 % either
    // way), so they stay a tuning switch: AETHER_GATHER_KC=4
    bool kc4 = false;
    if (const char* f = getenv("AETHER_GATHER_KC")) kc4 = atoi(f) == 4;
    if (bn == 32) {
        if (bm == 256) launch_gather_cfg<T, 256, 32, 64, 32>(gp, vec, false, st);
        else launch_gather_cfg<T, 128, 32, 32, 32>(gp, vec, false, st);
    } else {
        if (bm == 256) launch_gather_cfg<T, 256, 64, 64, 64>(gp, vec, kc4, st);
        else if (bm == 128) launch_gather_cfg<T, 128, 64, 32, 64>(gp, vec, kc4, st);
        else launch_gather_cfg<T, 64, 64, 32, 32>(gp, vec, kc4, st);
    }
}

// out[i] = sum_s part[s*stride + i] for i < n, in a fixed order: 4 split lanes per
// output (splits s, s+4, ...), then the 4 lanes in order.  i < n_dw goes to dw,
// the rest to dbias.
static __global__ __launch_bounds__(kThreads) void reduce_splits(const float* __restrict__ part, float* __restrict__ dw,
                                                         float* __restrict__ dbias, int n_dw, int n, int stride,
                                                         int splits) {
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
        if (i < n_dw) dw[i] = t;
        else if (dbias != nullptr) dbias[i - n_dw] = t;
    }
}

// The same sum for 16-byte aligned partials (stride and n_dw multiples of 4): a thread
// owns 4 consecutive outputs, 16 split lanes per output add splits j, j+16, ... with
// four loads in flight, and the lanes are added in lane order.
static __global__ __launch_bounds__(kThreads) void reduce_splits4(const float* __restrict__ part, float* __restrict__ dw,
                                                          float* __restrict__ dbias, int n_dw, int n, int stride,
                                                          int splits) {
    __shared__ f4 red[16][16];
    const int cg = threadIdx.x & 15;                     // group of 4 outputs
    const int sl = threadIdx.x >> 4;                     // split lane
    const int i = (blockIdx.x * 16 + cg) * 4;
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
        if (i < n_dw) *reinterpret_cast<f4*>(dw + i) = t;
        else if (dbias != nullptr) *reinterpret_cast<f4*>(dbias + (i - n_dw)) = t;
    }
}

// One gather-GEMM problem: pack the filter into the workspace at `ws_off`, launch.
struct GatherSetup {
    GatherParams gp;
    PackParams pp;
    int64_t bt_bytes;
    int nsplit = 1;          // > 1: split K, partial products behind the packed filter in the workspace
    int64_t part_bytes = 0;
};

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
    if (getenv("AETHER_GATHER_KC") != nullptr) return;       // the tuning switch changes the slab depth
    if (getenv("AETHER_GATHER_SPLIT_OFF") != nullptr) return; // lets small inputs reach the kernels of large ones
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

template <typename T>
static int run_gather(GatherSetup& gs, char* ws, int64_t ws_off, bool vec) {
    Context& c = ctx();
    void* bt = ws + ws_off;
    gs.gp.bt = bt;
    gs.pp.bt = bt;
    int total = gs.pp.Npad * gs.pp.Kpad;
    {
        const GatherParams& g = gs.gp;
        int64_t sb = (int64_t)g.S * g.Hs * g.Ws * g.Cs * (int64_t)sizeof(T);
        int64_t bb = (int64_t)total * (int64_t)sizeof(T);
        const int64_t lim = (int64_t)1 << 31;
        gs.gp.Th = (g.Tw > 0 && g.Cs > 0) ? (g.K / g.Cs) / g.Tw : 0;
        gs.gp.src_bytes = (sb < lim && bb < lim) ? (unsigned)sb : 0u;
        gs.gp.bt_bytes = (sb < lim && bb < lim) ? (unsigned)bb : 0u;
        const int64_t ob = (g.dense_out ? (int64_t)g.M : (int64_t)g.S * g.Hof * g.Wof) * g.N * (int64_t)sizeof(float);
        const bool ovec = ob < lim && g.N % 4 == 0 && (reinterpret_cast<uintptr_t>(g.out) & 15) == 0;
        gs.gp.out_bytes = ovec ? (unsigned)ob : 0u;
    }
    if constexpr (sizeof(T) == 2) {
        // the kernel that keeps the whole filter in LDS reads it from w itself
        GatherParams hp = gs.gp;
        int mtiles = 0;
        const bool dma = vec && hp.src_bytes != 0 && gs.pp.w_elems * 2 < ((int64_t)1 << 31) && gs.pp.N % 2 == 0;
        if (gs.nsplit == 1 && hp.M > 0 && plan_halo_res(hp, dma, c.prop.multiProcessorCount, &mtiles)) {
            hipLaunchKernelGGL(gather_halo_res_bf16, dim3((unsigned)std::min(mtiles, c.prop.multiProcessorCount)),
                               dim3(kResThreads), 0, c.stream, hp, gs.pp, mtiles);
            AETH_LAUNCH_CHECK();
            return AETH_OK;
        }
    }
    if (total > 0) {
        hipLaunchKernelGGL(pack_filter<T>, dim3(cdiv(total, 256)), dim3(256), 0, c.stream, gs.pp);
        AETH_LAUNCH_CHECK();
    }
    if (gs.gp.M > 0 && gs.gp.N > 0) {
        float* real_out = gs.gp.out;
        if (gs.nsplit > 1) gs.gp.out = reinterpret_cast<float*>(ws + ws_off + round_up(gs.bt_bytes, 256));
        launch_gather<T>(gs.gp, vec, c.prop.multiProcessorCount, c.stream);
        AETH_LAUNCH_CHECK();
        if (gs.nsplit > 1) {
            const int n = gs.gp.M * gs.gp.N;
            hipLaunchKernelGGL(reduce_splits4, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream,
                               (const float*)gs.gp.out, real_out, (float*)nullptr, n, n, n, gs.nsplit);
            AETH_LAUNCH_CHECK();
        }
    }
    return AETH_OK;
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

static inline void set_out_divs(GatherParams& g) {
    g.div_hw = FastDiv(g.Hg * g.Wg > 0 ? g.Hg * g.Wg : 1);
    g.div_w = FastDiv(g.Wg > 0 ? g.Wg : 1);
    g.div_c = FastDiv(g.Cs);
    g.div_tw = FastDiv(g.Tw > 0 ? g.Tw : 1);
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
template <typename T, int FH, int FW, int C>
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
    f4 acc = p.bias != nullptr ? *reinterpret_cast<const f4*>(p.bias + 4 * q) : f4{0.f, 0.f, 0.f, 0.f};
    const float* wq = wl + 4 * q;
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
        const f4 wv = *reinterpret_cast<const f4*>(wq + k * p.D);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(xv[k], wv[e], acc[e]);
    }
    *reinterpret_cast<f4*>(p.out + (size_t)m * p.D + 4 * q) = acc;
}

template <typename T, int FH, int FW, int C>
static __global__ __launch_bounds__(kThreads) void direct_dgrad_smallc(const DirectParams p) {
    extern __shared__ __attribute__((aligned(16))) float wl[];
    direct_load_filter<T>(p, wl);
    const T* __restrict__ dy = static_cast<const T*>(p.a);
    const int g = (int)(blockIdx.x * kThreads + threadIdx.x);
    const int m = g >> p.q_shift;                            // a pixel's lanes sit in one wave: q_shift <= 6
    const int q = g & ((1 << p.q_shift) - 1);
    unsigned s_, rem, i, j;
    p.div_hw.divmod((unsigned)min(m, p.M - 1), s_, rem);
    p.div_w.divmod(rem, i, j);
    float acc[C];
#pragma unroll
    for (int c = 0; c < C; ++c) acc[c] = 0.f;
    const float* wq = wl + 4 * q;
    f4 gv[FH * FW];
    bool oks[FH * FW];
#pragma unroll
    for (int fx = 0; fx < FH; ++fx)
#pragma unroll
        for (int fy = 0; fy < FW; ++fy) {
            const int t = (int)i + p.pH - fx, u = (int)j + p.pW - fy;        // = ho * sH, wo * sW
            const int ho = t / p.sH, wo = u / p.sW;
            const bool ok = t >= 0 && u >= 0 && ho * p.sH == t && wo * p.sW == u && ho < p.Ho && wo < p.Wo;
            const T* pd = dy + (size_t)(((int)s_ * p.Ho + (ok ? ho : 0)) * p.Wo + (ok ? wo : 0)) * p.D + 4 * q;
            oks[fx * FW + fy] = ok;
            if constexpr (sizeof(T) == 4) {
                gv[fx * FW + fy] = *reinterpret_cast<const f4*>(pd);
            } else {
                const uint2 v = *reinterpret_cast<const uint2*>(pd);
                gv[fx * FW + fy] = f4{__uint_as_float(v.x << 16), __uint_as_float(v.x & 0xffff0000u),
                                      __uint_as_float(v.y << 16), __uint_as_float(v.y & 0xffff0000u)};
            }
        }
#pragma unroll
    for (int tap = 0; tap < FH * FW; ++tap) {
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const f4 wv = *reinterpret_cast<const f4*>(wq + (tap * C + c) * p.D);
            float d = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) d = fmaf(gv[tap][e], wv[e], d);
            acc[c] += oks[tap] ? d : 0.f;
        }
    }
    // add up the lanes of the pixel; every lane ends with the full sums and lane q < C stores channel q
    for (int sh = 1; sh < (1 << p.q_shift); sh <<= 1) {
#pragma unroll
        for (int c = 0; c < C; ++c) acc[c] += __shfl_xor(acc[c], sh);
    }
    if (m < p.M) {
#pragma unroll
        for (int c = 0; c < C; ++c)
            if (q == c) p.out[(size_t)m * C + c] = acc[c];
    }
}

// The shapes the direct kernels take; everything else goes to the gather kernels.
template <typename T>
static bool launch_direct(DirectParams& dp, bool dgrad, hipStream_t st) {
    if (getenv("AETHER_DIRECT_OFF") != nullptr) return false;
    const int chunks = dp.D / 4;
    if (dp.C > 3 || dp.D % 4 != 0 || chunks < 4 || chunks > 64 || (chunks & (chunks - 1)) != 0) return false;
    if ((int64_t)dp.fH * dp.fW * dp.C * dp.D > kDirectMaxW || (int64_t)dp.M * chunks >= ((int64_t)1 << 31)) return false;
    if ((reinterpret_cast<uintptr_t>(dp.a) & 15) != 0 || (reinterpret_cast<uintptr_t>(dp.out) & 15) != 0 ||
        (dp.bias != nullptr && (reinterpret_cast<uintptr_t>(dp.bias) & 15) != 0))
        return false;
    dp.q_shift = 0;
    while ((1 << dp.q_shift) < chunks) ++dp.q_shift;
    const dim3 grid((unsigned)cdiv((int64_t)dp.M * chunks, kThreads));
    const size_t lds = (size_t)dp.fH * dp.fW * dp.C * dp.D * sizeof(float);
#define AETH_DIRECT_CASE(FH_, FW_, C_)                                                                              \
    if (dp.fH == FH_ && dp.fW == FW_ && dp.C == C_) {                                                               \
        if (dgrad) hipLaunchKernelGGL((direct_dgrad_smallc<T, FH_, FW_, C_>), grid, dim3(kThreads), lds, st, dp);   \
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

template <typename T>
int conv_fprop_impl(const char* fn, const T* x, const T* w, const float* bias, float* y,
                    int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    int Ho, Wo;
    int rc = check_conv_dims(fn, S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
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
    plan_split<T>(gs, C % Elem<T>::CE == 0, ctx().prop.multiProcessorCount);
    void* ws;
    rc = workspace(round_up(gs.bt_bytes, 256) + gs.part_bytes, &ws);
    if (rc) return rc;
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
    constexpr int BK = Elem<T>::BK;
    const int nclass = sH * sW;
    if (nclass > 64) return fail(AETH_E_INVALID, "%s: stride too large", fn);
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
            g.Kpad = (int)round_up(g.K, BK);
            g.Tw = Tw; g.sh = 1; g.sw = 1; g.rh0 = offh; g.rw0 = offw;
            g.Hof = H; g.Wof = W; g.oh0 = a; g.ow0 = b; g.ohs = sH; g.ows = sW;
            g.dense_out = (nclass == 1);
            set_out_divs(g);
            PackParams& pk = gs.pp;
            pk.w = w; pk.fW = fW; pk.C = C; pk.D = D; pk.Tw = Tw > 0 ? Tw : 1; pk.Ck = D; pk.w_elems = (int64_t)fH * fW * C * D;
            pk.xa = xmax; pk.xs = -sH; pk.ya = ymax; pk.ys = -sW; pk.transposed = 1;
            pk.N = C; pk.K = g.K; pk.Npad = (int)round_up(C, 64); pk.Kpad = g.Kpad;
            gs.bt_bytes = round_up((int64_t)pk.Npad * pk.Kpad * sizeof(T), 256);
            g.split_slabs = 0;
            plan_split<T>(gs, D % Elem<T>::CE == 0, ctx().prop.multiProcessorCount);
            total_bytes += gs.bt_bytes + gs.part_bytes;
            sets.push_back(gs);
        }
    }
    void* ws;
    rc = workspace(total_bytes > 0 ? total_bytes : 256, &ws);
    if (rc) return rc;
    int64_t off = 0;
    for (auto& gs : sets) {
        rc = run_gather<T>(gs, (char*)ws, off, D % Elem<T>::CE == 0);
        if (rc) return rc;
        off += gs.bt_bytes + gs.part_bytes;
    }
    return AETH_OK;
}

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
    int want_dbias;
    int S, H, W, C, Ho, Wo, D;
    int M, K;
    int fW, sH, sW, pH, pW;
    int m_per_split;     // multiple of 32
    int kt, nt;          // output tiles along k and n
    int cw;              // fp32 LDS-direct kernel: floats of k per lane of an operand read (4, 2 or 1)
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
            if (n0 + tid < p.D) outp[(size_t)p.K * p.D + n0 + tid] = s;
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
                                                       float* lds_y1) {
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

    const int lid = xcd_contiguous_id((int)blockIdx.x, (int)gridDim.x);
    const int tiles = p.kt * p.nt;
    const int split = lid / tiles;
    const int tile = lid - split * tiles;
    const int ktile = tile % p.kt;
    const int kt0 = ktile * TKW;
    const int n0 = (tile / p.kt) * kWgBN;
    const int m_begin = split * p.m_per_split;
    int m_end = m_begin + p.m_per_split;
    if (m_end > p.M) m_end = p.M;
    const bool do_db = p.want_dbias && (ktile == 0);

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
    const size_t split_stride = (size_t)p.K * p.D + p.D;
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
            outp[(size_t)p.K * p.D + n0 + tid] = (lds_y0[tid] + lds_y0[64 + tid]) + (lds_y0[128 + tid] + lds_y0[192 + tid]);
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
    if (p.cw == 1) wgrad_dma_body<1>(p, lds_a0, lds_a1, lds_y0, lds_y1);
    else if (p.cw == 2) wgrad_dma_body<2>(p, lds_a0, lds_a1, lds_y0, lds_y1);
    else wgrad_dma_body<4>(p, lds_a0, lds_a1, lds_y0, lds_y1);
}

// The 192-wide k tile: 64 KB of LDS, two workgroups per CU.
static __global__ __launch_bounds__(kThreads, 2) void wgrad_gemm_dma192(const WgradParams p) {
    __shared__ float lds_a0[kWgBR * 192];
    __shared__ float lds_a1[kWgBR * 192];
    __shared__ float lds_y0[kWgBR * kWgBN];
    __shared__ float lds_y1[kWgBR * kWgBN];
    wgrad_dma_body<6>(p, lds_a0, lds_a1, lds_y0, lds_y1);
}

// The same with 16-row slabs: 32 KB of LDS and half the per-load state, so that three
// workgroups fit a CU (a stand-alone loop: 140 TFLOP/s against 134 with 32-row slabs).
static __global__ __launch_bounds__(kThreads, 3) void wgrad_gemm_dma192h(const WgradParams p) {
    __shared__ float lds_a0[16 * 192];
    __shared__ float lds_a1[16 * 192];
    __shared__ float lds_y0[16 * kWgBN];
    __shared__ float lds_y1[16 * kWgBN];
    wgrad_dma_body<6, 16>(p, lds_a0, lds_a1, lds_y0, lds_y1);
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
    __shared__ float lds_db[4 * 64];

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
    const int y_eo0 = (((y_col >> 3) ^ ((j16 >> 3) << 2)) << 3) + (y_col & 4);
    const int y_eo1 = ((((y_col + 32) >> 3) ^ ((j16 >> 3) << 2)) << 3) + (y_col & 4);
    auto tr = [&](const uint16_t* base) {
        return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4_ptr_t)base);
    };

    f16v acc[2];
#pragma unroll
    for (int jn = 0; jn < 2; ++jn)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[jn][v] = 0.f;
    const bool active = kt0 + wave * 32 < p.K;           // wave-uniform

    float dbsum = 0.f;
    const int db_col = tid & 63, db_rg = tid >> 6;       // 4 row groups of 16 rows
    auto add_columns = [&](const uint16_t* ly) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int row = db_rg * 16 + r;
            const int e = (((db_col >> 3) ^ (((row >> 1) & 1) << 2)) << 3) + (db_col & 7);
            dbsum += __uint_as_float((unsigned)ly[row * kWgBN + e] << 16);
        }
    };

    auto slab = [&](int mb, const uint16_t* la, const uint16_t* ly, uint16_t* na, uint16_t* ny, bool has_next) {
        __builtin_amdgcn_s_waitcnt(0);                   // this wave's loads of the slab have landed
        __syncthreads();
        if (has_next) issue(mb + BR, na, ny);
        if (do_db) add_columns(ly);
        if (active) {
#pragma unroll
            for (int st = 0; st < BR / 16; ++st) {
                const int r0 = st * 16 + t_row;
                s4v a0 = tr(la + r0 * kWgBK + a_eo);
                s4v a1 = tr(la + (r0 + 4) * kWgBK + a_eo);
                s4v b00 = tr(ly + r0 * kWgBN + y_eo0);
                s4v b01 = tr(ly + (r0 + 4) * kWgBN + y_eo0);
                s4v b10 = tr(ly + r0 * kWgBN + y_eo1);
                s4v b11 = tr(ly + (r0 + 4) * kWgBN + y_eo1);
                typedef short s8v __attribute__((ext_vector_type(8)));
                const s8v av = __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7);
                const s8v bv0 = __builtin_shufflevector(b00, b01, 0, 1, 2, 3, 4, 5, 6, 7);
                const s8v bv1 = __builtin_shufflevector(b10, b11, 0, 1, 2, 3, 4, 5, 6, 7);
                acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av),
                                                                 __builtin_bit_cast(bf16x8, bv0), acc[0], 0, 0, 0);
                acc[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, av),
                                                                 __builtin_bit_cast(bf16x8, bv1), acc[1], 0, 0, 0);
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
        const int n = n0 + 32 * jn + l32;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int k = kt0 + wave * 32 + 8 * (v >> 2) + 4 * lh + (v & 3);
            if (k < p.K && n < p.D) outp[(size_t)k * p.D + n] = acc[jn][v];
        }
    }
    if (do_db) {
        lds_db[db_rg * 64 + db_col] = dbsum;
        __syncthreads();
        if (tid < 64 && n0 + tid < p.D)
            outp[(size_t)p.K * p.D + n0 + tid] = (lds_db[tid] + lds_db[64 + tid]) + (lds_db[128 + tid] + lds_db[192 + tid]);
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
// The loading wave also adds up the dy columns for dbias.  Partial results go to
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
    int offb[2];                                                           // into a dy buffer, step 0 (n block 0; ^ 32: block 1)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int row = tr_row + 4 * h;
        offb[h] = row * 64 + ((((col0 >> 3) ^ (((row >> 1) & 1) << 2)) << 3) + (col0 & 4));
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
    // dbias: wave t adds up the dy rows of the 8-row groups t, t + T, ... of every slab; a lane takes one
    // chunk position (8 columns) of row lrow of those groups
    const int lrow = lane >> 3;
    float db[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    asm volatile("s_barrier" ::: "memory");
    for (int t = 0; t < nsl; ++t) {
        const uint16_t* hb = halo[t & 1];
        const uint16_t* yb = dyb[t & 1];
        if (p.want_dbias) {
            for (int j = wave; 8 * j < p.slab_m; j += T) {
                const f4 v = reinterpret_cast<const f4*>(yb)[(8 * j + lrow) * 8 + (lane & 7)];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const unsigned u = __float_as_uint(v[e]);
                    db[2 * e] += __uint_as_float(u << 16);
                    db[2 * e + 1] += __uint_as_float(u & 0xffff0000u);
                }
            }
        }
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
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        asm volatile("s_barrier" ::: "memory");
    }
    if (p.want_dbias) {
        // everyone is past the last barrier of the loop: the first halo buffer is free.  Row lrow of wave
        // t holds its sums by logical chunk: the position with bit 2 flipped for rows whose bit 1 is set.
        float* red = reinterpret_cast<float*>(&halo[0][0]);
        const int lc = (lane & 7) ^ (((lrow >> 1) & 1) << 2);
#pragma unroll
        for (int e = 0; e < 8; ++e) red[(wave * 8 + lrow) * 64 + 8 * lc + e] = db[e];
        __syncthreads();
        if (wave == 0 && lane < p.D) {
            float sum = 0.f;
            for (int r = 0; r < 8 * T; ++r) sum += red[r * 64 + lane];
            outp[(size_t)K * p.D + lane] = sum;
        }
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const int n = 32 * nb + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int k = wave * 64 + 32 * kb + 8 * (v >> 2) + 4 * lh + (v & 3);
                if (n < p.D) outp[(size_t)k * p.D + n] = acc[kb][nb][v];
            }
        }
}

// Fills the plan of wgrad_halo_bf16 and returns the number of workgroups (= splits), or 0 when the
// kernel does not apply: unit stride, 64 input channels, D a multiple of 8 up to 64, at most 9 taps,
// slabs of whole output rows (R rows with R * Wo a multiple of 16 up to 128, R dividing Ho) whose
// padded source rows fit the halo buffer, and at least 4 slabs per CU (AETHER_WGRAD_HALO=1 drops
// the last condition, =0 turns the kernel off).
static int plan_wgrad_halo(WgradHaloParams& p, int C, int sH, int sW, int cus) {
    if (sH != 1 || sW != 1 || C != 64 || p.D % 8 != 0 || p.D > 64 || p.fH * p.fW > kWhMaxTaps) return 0;
    bool force = false;
    if (const char* f = getenv("AETHER_WGRAD_HALO")) {
        if (atoi(f) == 0) return 0;
        force = true;
    }
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

// Fills the plan of wgrad_halo_f32 and returns the number of workgroups (= splits), or 0 when the
// kernel does not apply: unit stride, 64 input channels, D a multiple of 4 up to 64, at most 9 taps,
// an even Wo of 28, 32, 56 or 64 (the built pair counts), at most 3 filter rows of at most 68 padded
// columns, and at least 4 output rows per CU (AETHER_WGRAD_HALO=1 drops the last condition, =0 turns
// the kernel off).
static int plan_wgrad_halo_f32(WgradHaloParams& p, int C, int sH, int sW, int cus) {
    if (sH != 1 || sW != 1 || C != 64 || p.D % 4 != 0 || p.D > 64 || p.fH * p.fW > 9) return 0;
    bool force = false;
    if (const char* f = getenv("AETHER_WGRAD_HALO")) {
        if (atoi(f) == 0) return 0;
        force = true;
    }
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
                    int S, int H, int W, int C, int D, int fH, int fW, int sH, int sW, int pH, int pW) {
    int Ho, Wo;
    int rc = check_conv_dims(fn, S, H, W, C, D, fH, fW, sH, sW, pH, pW, &Ho, &Wo);
    if (rc) return rc;
    Context& c = ctx();
    WgradParams p;
    p.x = x; p.dy = dy;
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
        else splits = (dma && va) ? plan_wgrad_halo_f32(hp, C, sH, sW, c.prop.multiProcessorCount) : 0;
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
    if (dma && p.cw == 4 && cdiv(p.K, 192) * 192 < cdiv(p.K, kWgBK) * kWgBK) p.cw = 6;
    if (const char* f = getenv("AETHER_WGRAD_CW")) {
        if (dma && va && p.K > 64 && (atoi(f) == 4 || atoi(f) == 6)) p.cw = atoi(f);
    }
    // slab height of the 192-wide kernel: 16 rows (three workgroups per CU) where a workgroup walks at
    // least 64 of them (56x56x64: 0.481 ms against 0.487 with 32 rows; 8x8x64 -> 128, batch 128, 8 slabs of
    // 32 per workgroup: 27.2 us with 32 rows, 28.3 with 16); AETHER_WGRAD_BR overrides
    int br = kWgBR;
    if (dma && p.cw == 6) {
        const int kt6 = cdiv(p.K, 192), nt6 = cdiv(D, kWgBN);
        const int64_t wgs = (int64_t)3 * c.prop.multiProcessorCount;
        if ((int64_t)cdiv(p.M, 32) * kt6 * nt6 >= 32 * wgs) br = 16;
        if (const char* f = getenv("AETHER_WGRAD_BR")) br = atoi(f) == 32 ? 32 : (atoi(f) == 16 ? 16 : br);
    }
    {
        const int qs = br / (Ho * Wo), rem = br % (Ho * Wo), qh = rem / Wo, qw = rem % Wo;
        p.step_c = qw * sW;
        p.step_r = qh * sH;
        p.inc0 = 4 * C * (qw * sW + qh * sH * W + qs * H * W);
        p.inc1 = 4 * C * (-Wo * sW + sH * W);
        p.inc2 = 4 * C * (-Ho * sH * W + H * W);
    }
    const int tkw = !dma ? kWgBK : (p.cw == 1 ? 32 : (p.cw == 6 ? 192 : kWgBK));
    const int kt = cdiv(p.K, tkw), nt = cdiv(D, kWgBN);
    const int slab_rows = dma16 ? 64 : kWgBR;
    const int slabs = cdiv(p.M, slab_rows);           // fp32: counted in 32-row units for both tile shapes
    // one round of resident workgroups (3 per CU for the LDS-direct kernels, 2 for the 192-wide
    // one and the register-staged one), rounded down so that no second, nearly empty round follows.
    // Every further round costs a set-up, an epilogue and a share of the reduction per workgroup
    // (56x56x64: 0.485 ms with one round, 0.493 with two, 0.509 with four).
    int rounds = 1;
    if (const char* f = getenv("AETHER_WGRAD_ROUNDS")) {      // tuning override: 1 to 4
        if (atoi(f) >= 1 && atoi(f) <= 4) rounds = atoi(f);
    }
    const int per_cu2 = (((dma && (p.cw != 6 || br == 16)) || dma16) ? 3 : 2) * rounds;
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
    void* ws;
    rc = workspace((int64_t)splits * (kd + D) * sizeof(float), &ws);
    if (rc) return rc;
    p.out = (float*)ws;
    p.kt = kt; p.nt = nt;
    dim3 grid(kt * nt * splits);
    if (dma16) hipLaunchKernelGGL(wgrad_gemm_dma_bf16, grid, dim3(kThreads), 0, c.stream, p);
    else if (dma && p.cw == 6 && br == 16) hipLaunchKernelGGL(wgrad_gemm_dma192h, grid, dim3(kThreads), 0, c.stream, p);
    else if (dma && p.cw == 6) hipLaunchKernelGGL(wgrad_gemm_dma192, grid, dim3(kThreads), 0, c.stream, p);
    else if (dma) hipLaunchKernelGGL(wgrad_gemm_dma, grid, dim3(kThreads), 0, c.stream, p);
    else if (va && vy) hipLaunchKernelGGL((wgrad_gemm<T, CE, CE>), grid, dim3(kThreads), 0, c.stream, p);
    else if (va) hipLaunchKernelGGL((wgrad_gemm<T, CE, 1>), grid, dim3(kThreads), 0, c.stream, p);
    else if (vy) hipLaunchKernelGGL((wgrad_gemm<T, 1, CE>), grid, dim3(kThreads), 0, c.stream, p);
    else hipLaunchKernelGGL((wgrad_gemm<T, 1, 1>), grid, dim3(kThreads), 0, c.stream, p);
    AETH_LAUNCH_CHECK();
    const int n = (int)(kd + (dbias ? D : 0));
    const bool r4 = kd % 4 == 0 && D % 4 == 0 && (reinterpret_cast<uintptr_t>(dw) & 15) == 0 &&
                    (dbias == nullptr || (reinterpret_cast<uintptr_t>(dbias) & 15) == 0);
    if (r4)
        hipLaunchKernelGGL(reduce_splits4, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream, (const float*)ws, dw, dbias,
                           (int)kd, n, (int)(kd + D), splits);
    else
        hipLaunchKernelGGL(reduce_splits, dim3(cdiv(n, 64)), dim3(kThreads), 0, c.stream, (const float*)ws, dw, dbias,
                           (int)kd, n, (int)(kd + D), splits);
    AETH_LAUNCH_CHECK();
    return AETH_OK;
}

}  // namespace aeth
