"""bf16-input / fp32-accumulate convolution against the oracle.

Two comparisons per case:
  * exact-input: the oracle (float64) evaluated on the bf16-rounded x, w, dy.
    Products of bf16 values are exact in fp32 and accumulation is fp32, so the
    fp32 tolerance applies: 1e-5 + 1e-4*|oracle| (rms-scaled for wgrad/dbias).
  * the stated bf16 tolerance against the unrounded fp32 oracle: relative 2e-2,
    measured against the rms of the output tensor (elements near zero carry the
    rounding noise of the whole dot product)."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

CASES = [
    (2, 6, 7, 3, 4, 3, 3, 1, 1, "same"),          # scalar-gather path (C, D not multiples of 8)
    (2, 9, 7, 4, 12, 3, 3, 2, 2, "same"),
    (4, 12, 12, 8, 16, 3, 3, 1, 1, "same"),
    (3, 16, 16, 32, 64, 3, 3, 1, 1, "same"),
    (2, 8, 8, 64, 128, 3, 3, 1, 1, "same"),
    (2, 14, 14, 64, 64, 3, 3, 1, 1, "same"),
    (2, 14, 14, 64, 256, 1, 1, 1, 1, "valid"),
    (3, 13, 13, 128, 256, 3, 3, 2, 2, "valid"),
    (5, 9, 9, 24, 40, 3, 3, 1, 1, "same"),
    (40, 16, 16, 3, 32, 3, 3, 1, 1, "same"),
    (5, 28, 28, 1, 32, 3, 3, 1, 1, "same"),       # direct kernels on bf16 inputs
    (3, 12, 12, 2, 16, 5, 5, 2, 2, "same"),       # 5x5 on 2 channels: not built, gather kernels
    (2, 11, 13, 3, 64, 5, 5, 1, 1, "same"),
    (3, 10, 10, 16, 48, 1, 1, 1, 1, "valid"),     # K = 16: wgrad waves past K still sum their dbias columns
    (2, 9, 9, 32, 64, 1, 1, 1, 1, "valid"),       # K = 32
    (2, 9, 9, 8, 24, 1, 1, 1, 1, "valid"),
]


def _case(case, seed):
    from tests import abi
    S, H, W, C, D, fH, fW, sH, sW, pad = case
    r = np.random.RandomState(seed)
    x = r.randn(S, H, W, C).astype(np.float32)
    w = (r.randn(fH, fW, C, D) * np.sqrt(2.0 / (fH * fW * C))).astype(np.float32)
    b = r.randn(D).astype(np.float32)
    _, yshape = abi.conv_dims(x.shape, w.shape, (sH, sW), pad)
    dy = r.randn(*yshape).astype(np.float32)
    return x, w, b, dy


def _loose(got, want, rel=2e-2):
    want = np.asarray(want, np.float64)
    rms = max(float(np.sqrt(np.mean(want * want))), 1e-30)
    assert np.max(np.abs(got - want)) <= rel * (np.abs(want).max() + rms), np.max(np.abs(got - want)) / rms
    assert np.sqrt(np.mean((got - want) ** 2)) <= rel * rms


def test_cast_is_round_to_nearest_even_bit_exact():
    from tests import abi
    r = np.random.RandomState(0)
    a = (r.randn(100000) * 10.0 ** r.randint(-8, 8, 100000)).astype(np.float32)
    a[:6] = [0.0, -0.0, np.inf, -np.inf, 1.00390625, 1.01171875]     # the last two are ties
    got = abi.to_bf16_device(a).get()
    assert np.array_equal(got, O.bf16_bits(a))
    nan = abi.to_bf16_device(np.array([np.nan], np.float32)).get()
    assert (nan[0] & 0x7F80) == 0x7F80 and (nan[0] & 0x7F) != 0


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_fprop_dgrad_wgrad(case):
    from tests import abi
    x, w, b, dy = _case(case, 3)
    stride, pad = (case[7], case[8]), case[9]
    xr, wr, dyr = O.round_to_bf16(x), O.round_to_bf16(w), O.round_to_bf16(dy)

    y = abi.fprop_bf16(x, w, b, stride, pad)
    abi.close(y, O.conv_fprop(xr, wr, b, stride, pad, dtype=np.float64))
    _loose(y, O.conv_fprop(x, w, b, stride, pad, dtype=np.float64))

    dx = abi.dgrad_bf16(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dyr, wr, x.shape[1:3], stride, pad, dtype=np.float64))
    _loose(dx, O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64))

    dw, db = abi.wgrad_bf16(x, dy, w.shape, stride, pad)
    abi.close(dw, O.conv_wgrad(xr, dyr, w.shape[:2], stride, pad, dtype=np.float64), rms_scaled=True)
    abi.close(db, O.conv_dbias(dyr, dtype=np.float64), rms_scaled=True)
    _loose(dw, O.conv_wgrad(x, dy, w.shape[:2], stride, pad, dtype=np.float64))


def test_conv_layer_bf16_precision_switch():
    import aether
    np.random.seed(5)
    layer = aether.Conv_Layer((10, 10, 16), num_filters=32)
    layer.precision = "bf16"
    x = np.random.randn(3, 10, 10, 16).astype(np.float32)
    dy = np.random.randn(3, 10, 10, 32).astype(np.float32)
    w, b = layer.filter_weights.get(), layer.biases.get()
    layer.forward(x, True)
    layer.backward(dy)
    _loose(layer.output.get(), O.conv_fprop(x, w, b, (1, 1), "same", dtype=np.float64))
    _loose(layer.dinputs.get(), O.conv_dgrad(dy, w, (10, 10), (1, 1), "same", dtype=np.float64))
    _loose(layer.dweights.get(), O.conv_wgrad(x, dy, (3, 3), (1, 1), "same", dtype=np.float64))
    _loose(layer.dbiases.get(), O.conv_dbias(dy, dtype=np.float64))


def test_bf16_filter_follows_parameters_set_twice_in_a_row():
    """The layer keeps a bfloat16 copy of its filter.  Two set_parameters calls without a forward pass between
    them can put the second filter at the address the first one had (the allocator hands a freed block out
    again): the copy must follow the tensor, not the address."""
    import aether
    np.random.seed(6)
    layer = aether.Conv_Layer((10, 10, 16), num_filters=32)
    layer.precision = "bf16"
    x = np.random.randn(3, 10, 10, 16).astype(np.float32)
    layer.forward(x, False)
    b = np.zeros(32, np.float32)
    p1 = np.random.randn(3, 3, 16, 32).astype(np.float32)
    p2 = np.random.randn(3, 3, 16, 32).astype(np.float32)
    for rounds in range(3):                                  # the first filter's block is free from the second round on
        layer.set_parameters(p1, b)
        layer.set_parameters(p2, b)
        got = layer.forward(x, False).get()
        fresh = aether.Conv_Layer((10, 10, 16), num_filters=32)
        fresh.precision = "bf16"
        fresh.set_parameters(p2, b)
        assert np.array_equal(got, fresh.forward(x, False).get()), rounds
        layer.set_parameters(p1, b)
        assert not np.array_equal(got, layer.forward(x, False).get())


# Unit-stride gathers over whole 64-channel blocks on images of about a multiple of 256 pixels
# take the kernel that keeps the source pixels of a tile in LDS for all taps.  Small inputs
# would split K instead; the tuning switch turns that off so that they reach the same code.
HALO_CASES = [
    (3, 16, 16, 64, 64, 3, 3, 1, 1, "same"),      # one tile per image
    (2, 16, 32, 128, 96, 3, 3, 1, 1, "same"),     # two channel blocks, two n tiles (the second ragged)
    (1, 50, 50, 64, 64, 3, 3, 1, 1, "same"),      # ten tiles, the last one partly empty
    (2, 17, 17, 64, 64, 2, 2, 1, 1, "valid"),     # even filter
    (2, 31, 31, 64, 64, 3, 3, 2, 2, "valid"),     # stride 2: the dgrad class of 2x2 taps on a 16x16 grid
    (2, 16, 16, 64, 64, 3, 5, 1, 1, "same"),      # 3x5 filter, pad 1 on both axes: columns lose their border
    (1, 16, 16, 64, 64, 5, 5, 1, 1, "same"),      # 25 taps: span too long for the buffer, the slab kernel runs
    (2, 15, 15, 64, 64, 2, 2, 1, 1, "valid"),     # even filter on an odd grid (dgrad): the halo's row and image pitches get an idle slot
    (2, 13, 13, 64, 64, 4, 4, 1, 1, "same"),      # 4x4 on 13x13
    (3, 14, 14, 128, 64, 3, 3, 1, 1, "same"),     # rows of 14: every 16-lane read group crosses a row end
]


@pytest.mark.parametrize("case", HALO_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_fprop_dgrad_without_split_k(case, tune):
    from tests import abi
    tune(gather_split=0, gather_runs=1)           # (run stores are taken from 64 MB of output on)
    x, w, b, dy = _case(case, 5)
    stride, pad = (case[7], case[8]), case[9]
    xr, wr, dyr = O.round_to_bf16(x), O.round_to_bf16(w), O.round_to_bf16(dy)
    got = abi.fprop_bf16(x, w, b, stride, pad)
    abi.close(got, O.conv_fprop(xr, wr, b, stride, pad, dtype=np.float64))
    abi.close(abi.fprop_bf16(x, w, None, stride, pad), O.conv_fprop(xr, wr, None, stride, pad, dtype=np.float64))
    dx = abi.dgrad_bf16(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dyr, wr, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_runs=0)                           # tiles stored as 16-byte pieces instead of runs of contiguous channels: same bits
    assert np.array_equal(got, abi.fprop_bf16(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))


def _random_halo_cases(n, seed):
    """Seeded random geometries around the conditions of the kernel that keeps a tile's source
    pixels in LDS (whole 64-channel blocks on the gathered side, output images of about a multiple
    of 256 pixels, 4 taps or more, unit stride): two thirds are drawn inside them, the rest around."""
    r = np.random.RandomState(seed)
    grids = [(16, 16), (16, 32), (32, 16), (8, 32), (32, 24), (16, 48), (20, 38), (25, 31), (51, 5)]
    out = []
    while len(out) < n:
        S = int(r.choice([1, 2, 3]))
        if r.rand() < 0.67:
            Ho, Wo = grids[r.randint(len(grids))]
            kind = r.randint(4)
            if kind == 0:
                fH, fW, pad, H, W = 3, 3, "same", Ho, Wo
            elif kind == 1:
                fH, fW, pad, H, W = 2, 2, "valid", Ho + 1, Wo + 1
            elif kind == 2:
                fH, fW, pad, H, W = 3, 3, "valid", Ho + 2, Wo + 2
            else:
                fH, fW, pad, H, W = 3, 2, "same", Ho, Wo - 1          # pad 1 on both axes: Wo = W + 2 - 2 + 1
            st = 1
            C, D = int(r.choice([64, 128])), int(r.choice([64, 128, 40]))
        else:
            fH, fW = int(r.choice([2, 3, 3, 4, 5])), int(r.choice([1, 2, 3, 3, 5]))
            st = int(r.choice([1, 2]))
            H, W = int(r.randint(10, 34)), int(r.randint(10, 34))
            C, D = int(r.choice([64, 128, 8])), int(r.choice([64, 128, 40, 8]))
            pad = "same" if r.rand() < 0.6 else "valid"
        if H < fH or W < fW or S * H * W * C * D * fH * fW > 6e8:
            continue
        out.append((S, H, W, C, D, fH, fW, st, st, pad))
    return out


@pytest.mark.parametrize("case", _random_halo_cases(28, 777), ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_random_geometries_without_split_k(case, tune):
    from tests import abi
    tune(gather_split=0)
    x, w, b, dy = _case(case, 9)
    stride, pad = (case[7], case[8]), case[9]
    xr, wr, dyr = O.round_to_bf16(x), O.round_to_bf16(w), O.round_to_bf16(dy)
    abi.close(abi.fprop_bf16(x, w, b, stride, pad), O.conv_fprop(xr, wr, b, stride, pad, dtype=np.float64))
    abi.close(abi.dgrad_bf16(dy, w, x.shape, stride, pad),
              O.conv_dgrad(dyr, wr, x.shape[1:3], stride, pad, dtype=np.float64))



# A filter of at most 9 taps on 64 channels and at most 64 output channels stays in LDS whole: one
# persistent workgroup per CU, one wave fetching the source pixels of the next 224-row tile while
# seven multiply the current one.  Tiles are whole image rows (the width divides 224).  A 3 x 3 filter
# whose output rows lie one after the other goes into the registers of four waves instead.  The library
# takes these kernels from 4 tiles per CU on; the gather_res switch lets small inputs reach them.
RES_CASES = [
    (2, 56, 56, 64, 64, 3, 3, 1, 1, "same"),      # the 56x56x64 layer: 14 tiles of 4 image rows per image
    (3, 28, 28, 64, 64, 3, 3, 1, 1, "same"),      # 784 pixels per image: the fourth tile is half empty
    (9, 14, 14, 64, 64, 3, 3, 1, 1, "same"),      # 196 pixels per image: one short tile each
    (2, 30, 30, 64, 48, 3, 3, 1, 1, "valid"),     # ragged N (no bias beyond channel 48), no padding
    (2, 29, 17, 64, 64, 2, 2, 1, 1, "valid"),     # even filter, 16 columns
    (2, 28, 28, 64, 64, 3, 3, 2, 2, "valid"),     # stride 2: dgrad classes of 4, 2 and 2 taps on a 14x14 grid
    (2, 8, 56, 64, 36, 1, 3, 1, 1, "same"),       # one filter row
    (100, 28, 28, 64, 64, 3, 3, 1, 1, "same"),    # 400 tiles on 256 workgroups: two tiles, or none
    (1, 16, 112, 64, 64, 3, 3, 1, 1, "same"),     # two rows per tile, but four rows of 114 slots do not fit: other kernels
    (2, 20, 20, 64, 64, 3, 3, 1, 1, "same"),      # width does not divide 224: other kernels
]


@pytest.mark.parametrize("case", RES_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_fprop_dgrad_with_the_filter_resident_in_lds(case, tune):
    from tests import abi
    tune(gather_split=0, gather_runs=1)
    tune(gather_res=1)
    x, w, b, dy = _case(case, 11)
    stride, pad = (case[7], case[8]), case[9]
    xr, wr, dyr = O.round_to_bf16(x), O.round_to_bf16(w), O.round_to_bf16(dy)
    got = abi.fprop_bf16(x, w, b, stride, pad)
    abi.close(got, O.conv_fprop(xr, wr, b, stride, pad, dtype=np.float64))
    abi.close(abi.fprop_bf16(x, w, None, stride, pad), O.conv_fprop(xr, wr, None, stride, pad, dtype=np.float64))
    dx = abi.dgrad_bf16(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dyr, wr, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_res=2)                            # 3 x 3 taps too with the filter in LDS, not in registers: same bits
    assert np.array_equal(got, abi.fprop_bf16(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))
    tune(gather_runs=0)                           # tiles stored as 16-byte pieces (the filter as the MFMAs' first operand): same bits
    assert np.array_equal(got, abi.fprop_bf16(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))
    # the same sums of the same products in another order of taps and tiles
    tune(gather_res=0)
    abi.close(abi.fprop_bf16(x, w, b, stride, pad), got, rtol=1e-5, atol=1e-5)


def test_bf16_register_filter_kernel_replayed_from_a_graph(tune):
    """The 3 x 3 kernel that keeps its filter in registers, recorded between aeth_graph_begin and aeth_graph_end (fprop and
    dgrad of one layer: nothing runs) and replayed three times with new inputs and eager work in between: every replay
    gives the bits of the eager calls."""
    import ctypes as C
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    tune(gather_split=0, gather_runs=1, gather_res=1)
    lib = _lib.lib()
    rng = np.random.default_rng(23)
    xshape, wshape = (3, 28, 28, 64), (3, 3, 64, 64)
    dims, yshape = abi.conv_dims(xshape, wshape, (1, 1), "same")
    w = (rng.standard_normal(wshape) * 0.1).astype(np.float32)
    b = rng.standard_normal(64).astype(np.float32)
    wd, bd = abi.to_bf16_device(w), DeviceTensor.from_numpy(b, np.float32)
    x16, dy16 = DeviceTensor(xshape, np.uint16), DeviceTensor(yshape, np.uint16)
    y, dx = DeviceTensor.full(yshape, np.nan), DeviceTensor.full(xshape, np.nan)
    _lib.check(lib.aeth_graph_begin())
    rc1 = lib.aeth_conv_fprop_bf16(x16.ptr, wd.ptr, bd.ptr, y.ptr, *dims)
    rc2 = lib.aeth_conv_dgrad_bf16(dy16.ptr, wd.ptr, dx.ptr, *dims)
    handle = C.c_void_p()
    rc_end = lib.aeth_graph_end(C.byref(handle))
    _lib.check(rc1), _lib.check(rc2), _lib.check(rc_end)
    assert np.all(np.isnan(y.get())) and np.all(np.isnan(dx.get()))           # recorded, not run
    try:
        for rep in range(3):
            x = rng.standard_normal(xshape).astype(np.float32)
            dy = rng.standard_normal(yshape).astype(np.float32)
            for src, dst in ((x, x16), (dy, dy16)):
                f = DeviceTensor.from_numpy(src, np.float32)
                _lib.check(lib.aeth_cast_f32_to_bf16(f.ptr, dst.ptr, f.size))
            _lib.check(lib.aeth_graph_launch(handle))
            got_y, got_dx = y.get(), dx.get()
            assert np.array_equal(got_y, abi.fprop_bf16(x, w, b, (1, 1), "same")), rep      # eager work between the replays
            assert np.array_equal(got_dx, abi.dgrad_bf16(dy, w, xshape, (1, 1), "same")), rep
    finally:
        _lib.check(lib.aeth_graph_destroy(handle))


# bf16 launches outside the halo kernels (strides, 1x1, more than 64 channels in) with more than 64 output
# channels use tiles of 256 x 128 or 256 x 256 on 8 waves.  The library takes them from 2 tiles per CU on;
# the gather_wide switch lets small inputs reach them, at 0 it gives the 4-wave tiles: the same sums in the same order.
WIDE_CASES = [
    (4, 28, 28, 128, 256, 3, 3, 2, 2, "valid"),   # the stride-2 layer: 256 x 256 tiles; dgrad: 256 x 128 per class
    (3, 15, 15, 64, 200, 3, 3, 2, 2, "same"),     # ragged n tile of 256 (channels 200 .. 255 read as zero)
    (2, 20, 20, 96, 128, 1, 1, 1, 1, "valid"),    # 1x1, 96 channels: K is not a whole slab
    (5, 9, 11, 128, 100, 3, 3, 1, 1, "same"),     # unit stride on 128 channels: 256 x 128 tiles, rows past M
    (2, 12, 12, 48, 192, 5, 5, 1, 1, "same"),     # 25 taps of 48 channels: slabs run over tap boundaries
    (300, 1, 1, 512, 160, 1, 1, 1, 1, "valid"),   # a dense layer: two n tiles of 128, the second of 32
]


@pytest.mark.parametrize("case", WIDE_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_fprop_dgrad_with_wide_tiles_on_eight_waves(case, tune):
    from tests import abi
    tune(gather_split=0, gather_merge=0)          # (one launch per dgrad class: the merged launch has kernels of its own)
    tune(gather_wide=1, gather_runs=1)
    x, w, b, dy = _case(case, 13)
    stride, pad = (case[7], case[8]), case[9]
    xr, wr, dyr = O.round_to_bf16(x), O.round_to_bf16(w), O.round_to_bf16(dy)
    y = abi.fprop_bf16(x, w, b, stride, pad)
    abi.close(y, O.conv_fprop(xr, wr, b, stride, pad, dtype=np.float64))
    abi.close(abi.fprop_bf16(x, w, None, stride, pad), O.conv_fprop(xr, wr, None, stride, pad, dtype=np.float64))
    dx = abi.dgrad_bf16(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dyr, wr, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_runs=0)                           # 16-byte pieces per pixel instead of runs of contiguous channels
    assert np.array_equal(y, abi.fprop_bf16(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))
    tune(gather_wide=0)
    assert np.array_equal(y, abi.fprop_bf16(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))


# wgrad of a unit-stride filter of at most 9 taps on 64 input channels and at most 64 output channels:
# one persistent workgroup per CU keeps the whole K x N result in registers (a wave per tap) and a
# loading wave brings slabs of whole output rows with the padded source rows under them.  The library
# takes that kernel from 4 slabs per CU on; the wgrad_halo switch lets small inputs reach it.
WGRAD_HALO_CASES = [
    (2, 56, 56, 64, 64, 3, 3, 1, 1, "same"),      # slabs of 2 rows of 56
    (3, 28, 28, 64, 64, 3, 3, 1, 1, "same"),      # 4 rows of 28
    (2, 30, 30, 64, 48, 3, 3, 1, 1, "valid"),     # no padding, 48 output channels
    (2, 18, 34, 64, 64, 3, 3, 1, 1, "valid"),     # 4 rows of 32: full 128-row slabs
    (2, 17, 17, 64, 64, 2, 2, 1, 1, "valid"),     # even filter, 8 rows of 16
    (2, 8, 58, 64, 40, 1, 3, 1, 1, "valid"),      # one filter row
    (24, 56, 56, 64, 64, 3, 3, 1, 1, "same"),     # 672 slabs on 224 workgroups of 3
    (2, 14, 14, 64, 64, 3, 3, 1, 1, "same"),      # 8 rows of 14 would make a slab, but 8 does not divide 14: other kernel
    (2, 16, 16, 128, 64, 3, 3, 1, 1, "same"),     # 128 input channels: other kernel
    (2, 16, 16, 64, 64, 1, 1, 1, 1, "valid"),     # one tap: the lone multiplying wave sums both column blocks for dbias
    (2, 16, 16, 64, 40, 1, 1, 1, 1, "valid"),     # ... the second block partly filled
    (2, 8, 33, 64, 24, 1, 2, 1, 1, "valid"),      # two taps, 24 columns: the second block's sums are never stored
]


@pytest.mark.parametrize("case", WGRAD_HALO_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_wgrad_with_the_whole_result_in_registers(case, tune):
    from tests import abi
    tune(wgrad_halo=1)
    x, w, b, dy = _case(case, 13)
    stride, pad = (case[7], case[8]), case[9]
    xr, dyr = O.round_to_bf16(x), O.round_to_bf16(dy)
    dw, db = abi.wgrad_bf16(x, dy, w.shape, stride, pad)
    abi.close(dw, O.conv_wgrad(xr, dyr, w.shape[:2], stride, pad, dtype=np.float64), rms_scaled=True)
    abi.close(db, O.conv_dbias(dyr, dtype=np.float64), rms_scaled=True)
    dw2, db2 = abi.wgrad_bf16(x, dy, w.shape, stride, pad)
    assert np.array_equal(dw, dw2) and np.array_equal(db, db2)            # deterministic
    # the same sums of the same products in another order
    tune(wgrad_halo=0)
    dw3, db3 = abi.wgrad_bf16(x, dy, w.shape, stride, pad)
    abi.close(dw3, dw, rtol=1e-4, atol=1e-5, rms_scaled=True)
    abi.close(db3, db, rtol=1e-4, atol=1e-5, rms_scaled=True)


# bf16 dgrad reads its filter operand from w itself where slabs lie inside one tap (output channels in whole
# slabs of 64): the halo kernel, the slab kernel and its 8-wave tiles.  The gather_direct_b switch at 0 packs;
# same bits either way.
DIRECT_B_BF16_CASES = [
    (2, 16, 16, 64, 64, 3, 3, 1, 1, "same", {}),                    # gather_halo_res_bf16 reads w itself anyway
    (2, 16, 16, 64, 128, 3, 3, 1, 1, "same", {"gather_split": 0}),    # halo kernel, two slabs per tap
    (3, 13, 13, 128, 256, 3, 3, 2, 2, "valid", {"gather_split": 0}),  # the stride-2 layer: classes of 4, 2, 2, 1 taps
    (2, 14, 14, 64, 256, 1, 1, 1, 1, "valid", {"gather_split": 0}),   # 1x1: one tap of 4 slabs, slab kernel
    (2, 9, 9, 40, 128, 3, 3, 1, 1, "same", {"gather_split": 0}),      # 40 input channels: rows past C in the tile
    (2, 12, 12, 256, 192, 3, 3, 1, 1, "same", {"gather_split": 0, "gather_wide": 1}),   # 8-wave tiles
    (2, 10, 10, 64, 96, 3, 3, 1, 1, "same", {"gather_split": 0}),     # 96 output channels: slabs straddle taps, packed
]


@pytest.mark.parametrize("case", DIRECT_B_BF16_CASES, ids=lambda c: "x".join(str(v) for v in c[:10]))
def test_bf16_dgrad_reading_the_filter_in_place(case, tune):
    from tests import abi
    x, w, b, dy = _case(case[:10], 23)
    stride, pad = (case[7], case[8]), case[9]
    tune(**case[10])
    dyr, wr = O.round_to_bf16(dy), O.round_to_bf16(w)
    dx = abi.dgrad_bf16(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dyr, wr, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_direct_b=0)
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))


# bf16 dgrad of a strided layer whose stride classes all have the same pixel grid (H and W multiples of the
# strides) and all go to the halo kernel: one launch for the 2 or 4 classes, whose workgroups for one tile of
# pixels run next to each other.  The gather_merge switch at 0 launches class by class (clipped grids, a
# zeroed strip): same bits either way.
MERGE_CASES = [
    (3, 28, 28, 128, 256, 3, 3, 2, 2, "valid"),   # the stride-2 layer: classes of 4, 2, 2 and 1 taps, row and column 27 of dx unreachable
    (2, 16, 16, 64, 64, 3, 3, 2, 2, "same"),      # one channel block; 'same' padding shifts the classes
    (2, 20, 12, 40, 128, 4, 4, 2, 2, "valid"),    # 4 taps in every class, 40 channels of dx
    (2, 16, 16, 36, 64, 2, 2, 2, 2, "valid"),     # one tap per class; 36 channels: the filter is packed
    (2, 16, 16, 64, 128, 3, 3, 2, 1, "same"),     # two classes (rows only)
    (2, 12, 18, 64, 64, 5, 5, 2, 2, "same"),      # 9, 6, 6 and 4 taps
    (5, 8, 8, 128, 192, 3, 3, 2, 2, "same"),      # 16 pixels per class and image: tiles run over images
    (1, 18, 12, 48, 64, 3, 2, 1, 2, "valid"),     # two classes (columns only), 3 x 2 filter
    (40, 28, 28, 128, 128, 3, 3, 2, 2, "valid"),  # 31 tiles of 256 pixels per class
    (9, 16, 16, 200, 64, 3, 3, 2, 2, "same"),     # 200 channels of dx: four n tiles, the last ragged
    (4, 16, 16, 96, 128, 3, 3, 2, 1, "same"),     # two classes (one pair) and 96 channels of dx
    (3, 12, 18, 72, 64, 5, 5, 2, 2, "same"),      # 9, 6, 6 and 4 taps on 72 channels of dx: windows of 3 x 3 in the common halo
    (2, 24, 24, 128, 128, 4, 4, 2, 2, "valid"),   # 4 taps in every class
    (2, 18, 14, 64, 64, 3, 3, 2, 2, "valid"),     # class grids of 9 x 7 pixels, windows of 2 x 2: odd widths, both pitches padded
    (3, 10, 22, 128, 64, 4, 4, 2, 2, "valid"),    # class grids of 5 x 11
]


@pytest.mark.parametrize("case", MERGE_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_dgrad_with_all_stride_classes_in_one_launch(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 29)
    stride, pad = (case[7], case[8]), case[9]
    tune(gather_split=0, gather_pairs=0, gather_runs=1)   # one class per workgroup, tiles stored as runs of contiguous channels
    dyr, wr = O.round_to_bf16(dy), O.round_to_bf16(w)
    dx = abi.dgrad_bf16(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dyr, wr, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_runs=0)                           # ... as 16-byte pieces
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))
    tune(gather_merge=0)
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))
    # two classes per workgroup from one halo (what the library takes where all classes read the filter in place),
    # with and without the non-temporal hint on its stores
    tune(gather_merge=-1, gather_pairs=-1, gather_runs=1)
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))
    tune(gather_runs=-1)
    assert np.array_equal(dx, abi.dgrad_bf16(dy, w, x.shape, stride, pad))


# bf16 wgrad onto more than 64 output channels: wave tiles of 64 k x 128 n (workgroup 128 k x 256 n) or
# 64 k x 64 n (128 x 128), where the library takes them from the channel padding they cost; the
# wgrad_wide switch forces them (1: the narrower form wherever D > 64) or turns them off (0).
WGRAD_WIDE_CASES = [
    (3, 13, 13, 128, 256, 3, 3, 2, 2, "valid"),   # the stride-2 layer's shape: 9 k tiles, one n tile of 256
    (2, 14, 14, 64, 256, 1, 1, 1, 1, "valid"),    # 1x1: K = 64, the wave's second k block is empty
    (2, 9, 9, 72, 200, 3, 3, 1, 1, "same"),       # K = 648: ragged last k tile; 200 of 256 columns
    (2, 12, 12, 32, 128, 3, 3, 1, 1, "same"),     # 128 columns: the 128 x 128 form
    (2, 11, 11, 40, 96, 3, 3, 1, 1, "same"),      # 96 of 128 columns
    (2, 10, 10, 16, 320, 2, 2, 1, 1, "valid"),    # two n tiles, the second a quarter full
    (5, 7, 9, 24, 72, 3, 3, 1, 1, "same"),        # 72 columns: forced onto the 128-wide form
    (40, 8, 8, 64, 128, 3, 3, 1, 1, "same"),      # 2560 rows: several slabs per split
]


@pytest.mark.parametrize("mode", [1, 3], ids=["wide", "wide_256k"])   # 3: also 256 k rows per workgroup (8 waves)
@pytest.mark.parametrize("case", WGRAD_WIDE_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_bf16_wgrad_on_wide_wave_tiles(case, mode, tune):
    from tests import abi
    tune(wgrad_wide=mode, wgrad_halo=0)
    x, w, b, dy = _case(case, 17)
    stride, pad = (case[7], case[8]), case[9]
    xr, dyr = O.round_to_bf16(x), O.round_to_bf16(dy)
    dw, db = abi.wgrad_bf16(x, dy, w.shape, stride, pad)
    abi.close(dw, O.conv_wgrad(xr, dyr, w.shape[:2], stride, pad, dtype=np.float64), rms_scaled=True)
    abi.close(db, O.conv_dbias(dyr, dtype=np.float64), rms_scaled=True)
    dw2, db2 = abi.wgrad_bf16(x, dy, w.shape, stride, pad)
    assert np.array_equal(dw, dw2) and np.array_equal(db, db2)            # deterministic
    tune(wgrad_wide=0)                                                    # 64-wide tiles: another order of the same sums
    dw3, db3 = abi.wgrad_bf16(x, dy, w.shape, stride, pad)
    abi.close(dw3, dw, rtol=1e-4, atol=1e-5, rms_scaled=True)
    abi.close(db3, db, rtol=1e-4, atol=1e-5, rms_scaled=True)


# ---- bfloat16 copies left by the producing kernels ------------------------------------------
# A bf16 convolution reads bfloat16 x and dy.  The layers that produce them (ReLU / leaky ReLU,
# the fused batch-norm block, batch norm's backward pass) can leave the bfloat16 copy beside the
# float32 tensor they write anyway; the copy must be the round-to-nearest-even image of exactly
# the float32 values written, bit for bit, so that a convolution fed by it computes what it
# computes after a cast pass.
@pytest.mark.parametrize("n", [4096 * 7, 1001])            # 16-byte groups, and a length that is not a multiple of 4
def test_relu_twin_is_the_cast_of_what_relu_writes(n):
    from aether import _lib
    from aether.tensor import DeviceTensor
    r = np.random.RandomState(2)
    x = r.randn(n).astype(np.float32)
    xd = DeviceTensor.from_numpy(x)
    for alpha in (0.0, 0.01):
        y, y2 = DeviceTensor.full(n, np.nan), DeviceTensor.full(n, np.nan)
        y16 = DeviceTensor(n, np.uint16)
        _lib.check(_lib.lib().aeth_relu_fwd_f32(xd.ptr, y.ptr, alpha, n))
        _lib.check(_lib.lib().aeth_relu_fwd_twin_f32(xd.ptr, y2.ptr, y16.ptr, alpha, n))
        assert np.array_equal(y.get(), y2.get())
        assert np.array_equal(y.get(), np.where(x > 0, x, np.float32(alpha) * x))
        assert np.array_equal(y16.get(), O.bf16_bits(y.get()))


@pytest.mark.parametrize("shape", [(6, 10, 10, 32), (5, 7, 7, 6)])       # 16-byte path, scalar path
def test_bn_bwd_twin_is_the_cast_of_what_bn_bwd_writes(shape):
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    r = np.random.RandomState(3)
    C = shape[-1]
    rows = int(np.prod(shape[:-1]))
    x = r.randn(*shape).astype(np.float32) * 2 + 1
    dy = r.randn(*shape).astype(np.float32)
    g = (r.rand(C) + 0.5).astype(np.float32)
    mu = x.reshape(rows, C).mean(0).astype(np.float32)
    var = x.reshape(rows, C).var(0)
    invstd = (1.0 / np.sqrt(var + 1e-5)).astype(np.float32)
    d = {k: DeviceTensor.from_numpy(v) for k, v in dict(x=x, dy=dy, g=g, mu=mu, invstd=invstd).items()}
    dx, dx2 = DeviceTensor.full(shape, np.nan), DeviceTensor.full(shape, np.nan)
    dx16 = DeviceTensor(shape, np.uint16)
    dg, db, dg2, db2 = (DeviceTensor.full(C, np.nan) for _ in range(4))
    L = _lib.lib()
    _lib.check(L.aeth_bn_bwd_f32(d["x"].ptr, d["dy"].ptr, d["g"].ptr, d["mu"].ptr, d["invstd"].ptr, dx.ptr, dg.ptr,
                                 db.ptr, rows, C))
    _lib.check(L.aeth_bn_bwd_twin_f32(d["x"].ptr, d["dy"].ptr, d["g"].ptr, d["mu"].ptr, d["invstd"].ptr, dx2.ptr,
                                      dx16.ptr, dg2.ptr, db2.ptr, rows, C))
    assert np.array_equal(dg.get(), dg2.get()) and np.array_equal(db.get(), db2.get())
    want, _, _ = O.bn_backward(x.astype(np.float64), dy.astype(np.float64), g.astype(np.float64),
                               mu.astype(np.float64).reshape((1,) * (len(shape) - 1) + (C,)),
                               var.reshape((1,) * (len(shape) - 1) + (C,)), 1e-5)
    abi.close(dx2.get(), want, rtol=2e-4)
    abi.close(dx.get(), want, rtol=2e-4)
    assert np.array_equal(dx16.get(), O.bf16_bits(dx2.get()))


def test_bf16_convolution_between_producers_uses_their_copies():
    """ReLU -> Conv_Layer(bf16) -> Batch_Norm, linked as Model.finalize links them: the
    convolution finds bfloat16 copies of its input and of its upstream gradient and casts
    nothing but its filter; results equal, bit for bit, those of the same layers without
    the links (where the convolution casts x and dy itself)."""
    import aether

    def chain(linked):
        np.random.seed(8)
        relu, conv, bn = aether.ReLU(), aether.Conv_Layer((12, 12, 64), num_filters=64), aether.Batch_Norm()
        conv.precision = "bf16"
        if linked:
            relu.next, conv.prev, conv.next, bn.prev = conv, relu, bn, conv
        return relu, conv, bn

    r = np.random.RandomState(9)
    x = r.randn(4, 12, 12, 64).astype(np.float32)
    dy = r.randn(4, 12, 12, 64).astype(np.float32)
    outs = []
    for linked in (True, False):
        relu, conv, bn = chain(linked)
        relu.forward(x, True)
        conv.forward(relu.output, True)
        bn.forward(conv.output, True)
        bn.backward(dy)
        conv.backward(bn.dinputs)
        if linked:
            assert relu.output._bf16 is not None and conv._x_bf16 is relu.output._bf16
            assert bn.dinputs._bf16 is not None
            assert np.array_equal(relu.output._bf16.get(), O.bf16_bits(relu.output.get()))
            assert np.array_equal(bn.dinputs._bf16.get(), O.bf16_bits(bn.dinputs.get()))
        else:
            assert relu.output._bf16 is None and bn.dinputs._bf16 is None
        outs.append([t.get() for t in (conv.output, conv.dinputs, conv.dweights, conv.dbiases)])
    for a, b in zip(*outs):
        assert np.array_equal(a, b)
    # the filter is cast once per version of the weights: set_parameters and an in-place change make it stale
    relu, conv, bn = chain(True)
    relu.forward(x, True)
    conv.forward(relu.output, True)
    first = conv._w16
    conv.forward(relu.output, True)
    assert conv._w16 is first
    conv.filter_weights.set(conv.filter_weights.get() * 2)
    y1 = conv.forward(relu.output, True).get()
    assert conv._w16 is not first
    np.testing.assert_allclose(y1, 2 * outs[0][0], rtol=1e-6, atol=1e-6)


def test_bf16_training_steps_of_the_cnn_recorded_and_eager(monkeypatch):
    """The three-block CNN with every convolution on bf16 inputs (AETHER_PRECISION=bf16): the
    fused blocks hand their bfloat16 pooling output to the next convolution, the fused backward
    pass its bfloat16 batch-norm gradient.  Loss within the bf16 tolerance of the float32
    model's, and recorded steps equal eager ones bit for bit (the filter casts are part of the
    recording)."""
    import aether
    from tests.test_gpu_model import build_model
    rng = np.random.RandomState(4)
    X, y = rng.rand(32, 16, 16, 3).astype(np.float32), rng.randint(0, 10, 32)

    def make(precision):
        monkeypatch.setenv("AETHER_PRECISION", precision)
        np.random.seed(6)
        m = build_model(aether, hw=16)
        m.loss.new_pass()
        m.accuracy.new_pass()
        return m

    f32, eager, rec = make("fp32"), make("bf16"), make("bf16")
    rec.record_steps(True)
    for step in range(5):
        a, b, c = f32.train_step(X, y), eager.train_step(X, y), rec.train_step(X, y)
        assert b == c, "step %d: eager %r, recorded %r" % (step, b, c)
        assert abs(a[0] - b[0]) <= 2e-2 * abs(a[0]), (step, a, b)
        for la, lb in zip(eager.trainable_layers, rec.trainable_layers):
            assert np.array_equal(np.asarray(la.weights), np.asarray(lb.weights))
    convs = [l for l in eager.layers if isinstance(l, aether.Conv_Layer)]
    assert all(c.precision == "bf16" for c in convs)
    assert convs[1].inputs._bf16 is not None and convs[1]._x_bf16 is convs[1].inputs._bf16
    rec.record_steps(False)
