// Kernel-choice overrides for tests and measurements.
//
// Every dispatch decision of the library follows from the problem's shape.  The fields below
// let a test reach a kernel with an input smaller than the shapes it is chosen for, or run a
// problem on a second, independently scheduled kernel; -1 always means "decide from the shape".
// They are set through aeth_debug_set() or, once, at aeth_init from the single environment
// variable AETHER_TUNE ("name=value,name=value").  Nothing else in the library reads the
// environment.
#pragma once

namespace aeth {

struct Tuning {
    int gather_bm = -1;      // tile height of the slab kernels: 256, 128 or 64
    int gather_kc = -1;      // slab depth in 16-byte chunks: 8, or 4 (half-depth slabs; also turns split K off)
    int gather_nloop = -1;   // 0: no n-loop mode for short-K products
    int gather_halo = -1;    // 0: no halo kernels (bf16)
    int gather_split = -1;   // 0: no split K (lets small inputs reach the kernels of large ones)
    int gather_sa = -1;      // 0: vector-addressed loads instead of scalar-addressed ones (fp32)
    int gather_direct_b = -1; // 0: dgrad always packs its filter (no reads from w itself)
    int gather_clip = -1;    // 0: strided dgrad multiplies its classes' full pixel grids (no zeroed strips)
    int gather_merge = -1;   // 0: a strided dgrad launches its classes one by one
    int gather_border = -1;  // fp32 dgrad classes cut into border strips and interiors: 0 never, 1 also for small inputs
    int gather_pairs = -1;   // 0: the merged launch keeps one class per workgroup
    int gather_bkn = -1;     // 0: fp32 fprop always packs its filter
    int narrow = -1;         // 0: products with at most 16 output channels go to the slab kernels too
    int gather_runs = -1;    // tiles stored as runs of contiguous channels (non-temporal): 0 never, 1 always (default: from 64 MB of output on)
    int gather_wide = -1;    // bf16 8-wave tiles: 0 never, 1 also for few tiles
    int gather_res = -1;     // gather_halo_res_bf16 / gather_halo_res9_bf16: 0 off, 1 also for few tiles, 2 the same with the filter in LDS for 3 x 3 taps too
    int dense_res = -1;      // dense_res_f32: 0 off, 1 also for few tiles
    int direct = -1;         // 0: no direct kernels for 1 to 3 input channels; 2: 4 output channels per lane in them
    int wgrad_halo = -1;     // wgrad_halo_f32 / _bf16: 0 off, 1 also for few slabs
    int wgrad_wide = -1;     // bf16 wgrad on wide wave tiles: 0 never, 1 wherever D > 64 (2: but never 256 k rows, 3: always)
    int wgrad_cw = -1;       // fp32 wgrad tile form: 4 (128-wide) or 6 (192-wide)
    int wgrad_br = -1;       // slab height of the 192-wide form: 32 or 16
    int wgrad_swap = -1;     // fp32 1x1 wgrad on few input channels with the operands swapped: 0 never, 1 wherever it applies
    int wgrad_rounds = -1;   // rounds of resident workgroups the splits are sized for: 1 to 4
    int pair_bwd = -1;       // 0: the backward entry points launch a layer's wgrad and dgrad one after the other
};

Tuning& tuning();
// Sets one field by name; name == nullptr resets all of them.  False for an unknown name.
bool tuning_set(const char* name, int value);
// Parses "name=value,name=value"; unknown names are reported through `bad` (may be null).
void tuning_parse(const char* spec, const char** bad);

}  // namespace aeth
