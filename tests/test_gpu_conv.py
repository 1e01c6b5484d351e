"""Parity of the fp32 HIP convolution (through the C ABI) with the CPU oracle.
Tolerance (fp32): |gpu - oracle| <= 1e-5 + 1e-4*|oracle| per element, oracle
evaluated in float64 on the float32 inputs."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

# S, H, W, C, D, fH, fW, sH, sW, padding
CASES = [
    (2, 5, 5, 1, 1, 3, 3, 1, 1, "valid"),
    (2, 6, 7, 3, 4, 3, 3, 1, 1, "same"),
    (3, 8, 8, 4, 5, 3, 3, 2, 2, "valid"),
    (2, 9, 7, 2, 3, 3, 3, 2, 2, "same"),
    (2, 7, 7, 4, 6, 1, 1, 1, 1, "valid"),
    (1, 8, 9, 3, 2, 5, 3, 1, 2, "same"),
    (2, 6, 6, 2, 2, 2, 2, 2, 2, "valid"),
    (1, 10, 10, 2, 3, 3, 3, 3, 3, "valid"),
    (4, 12, 12, 8, 16, 3, 3, 1, 1, "same"),
    (3, 16, 16, 32, 64, 3, 3, 1, 1, "same"),     # config-2a channel counts
    (2, 8, 8, 64, 128, 3, 3, 1, 1, "same"),      # config-2b channel counts
    (2, 14, 14, 64, 64, 3, 3, 1, 1, "same"),     # config-4 channel counts, ragged M
    (2, 14, 14, 64, 256, 1, 1, 1, 1, "valid"),   # config-4 1x1
    (3, 13, 13, 128, 256, 3, 3, 2, 2, "valid"),  # config-5 channel counts
    (5, 9, 9, 20, 36, 3, 3, 1, 1, "same"),       # C,D multiples of 4 but not of 32
    (2, 9, 9, 6, 10, 3, 3, 1, 1, "same"),        # C,D not multiples of 4
    (2, 9, 9, 5, 7, 1, 1, 2, 2, "same"),         # 1x1 stride 2: dgrad classes without taps
    (40, 16, 16, 3, 32, 3, 3, 1, 1, "same"),     # config-1 channel counts
    (2, 4, 4, 256, 64, 3, 3, 1, 1, "same"),      # one tile, K = 2304: fprop splits K
    (1, 8, 16, 512, 256, 1, 1, 1, 1, "valid"),   # dense-like, batch 128, K = 512: fprop and dgrad split K
    (3, 6, 6, 128, 96, 3, 3, 1, 1, "valid"),     # split K with a ragged last split (36 slabs)
    (8, 48, 48, 64, 256, 1, 1, 1, 1, "valid"),   # K of two slabs, 4 n tiles: one workgroup walks the n tiles
    (8, 48, 48, 32, 192, 1, 1, 1, 1, "valid"),   # same with one slab, 3 n tiles
    (8, 48, 48, 48, 136, 1, 1, 1, 1, "valid"),   # same, padded second slab, ragged last n tile
    # 1 to 3 input channels, 3x3 or 5x5, D/4 a power of two: the direct kernels (filter in LDS, a lane per 4 channels)
    (5, 28, 28, 1, 32, 3, 3, 1, 1, "same"),      # first layer of the 28x28x1 topology
    (3, 12, 12, 2, 16, 3, 3, 2, 2, "same"),      # stride 2: dgrad taps that do not divide
    (2, 11, 13, 3, 64, 5, 5, 1, 1, "same"),
    (2, 9, 9, 3, 256, 3, 3, 1, 1, "valid"),      # 64 lanes per pixel
    (2, 9, 9, 3, 48, 3, 3, 1, 1, "same"),        # D/4 = 12: not a power of two, gather kernels
    (3, 10, 10, 1, 32, 5, 5, 3, 2, "valid"),     # 5x5 on one channel, strides 3 and 2
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


def test_library_reports_gfx950():
    from aether import _lib
    info = _lib.device_info()
    assert str(info["arch"]).startswith("gfx950")
    assert info["cus"] > 0


def test_notebook_known_answers_on_gpu():
    from tests import abi
    # CNN/notebooks/CNN_Implementation.ipynb:421-472 -> :411-414
    img = np.array([[1, 2, 3, 0], [0, 1, 2, 3], [3, 0, 1, 2], [2, 3, 0, 1]], dtype=np.float32)
    k = np.array([[1, 0, -1]] * 3, dtype=np.float32)
    y = abi.fprop(img[None, :, :, None], k[:, :, None, None], None, (1, 1), "same")
    want = np.array([[-3, -4, 0, 5], [-3, -2, -2, 6], [-4, 2, -2, 3], [-3, 4, 0, 1]], dtype=np.float32)
    assert np.array_equal(y[0, :, :, 0], want)
    # :747-752, :774-779, :803-811
    y = abi.fprop(np.ones((1, 5, 5, 1), np.float32), np.ones((3, 3, 1, 1), np.float32), np.zeros(1, np.float32),
                  (1, 1), "valid")
    assert y.shape == (1, 3, 3, 1) and np.all(y == 9)
    y = abi.fprop(np.ones((1, 5, 5, 3), np.float32), np.ones((3, 3, 3, 1), np.float32), np.zeros(1, np.float32),
                  (1, 1), "valid")
    assert np.all(y == 27)
    w = np.ones((3, 3, 1, 2), np.float32)
    w[..., 1] = 2
    y = abi.fprop(np.ones((1, 5, 5, 1), np.float32), w, np.zeros(2, np.float32), (1, 1), "valid")
    assert np.all(y[..., 0] == 9) and np.all(y[..., 1] == 18)
    # CNN/notebooks/Backpropagation_Conv.ipynb:84-110: taps accumulate
    dy = np.zeros((1, 4, 4, 1), np.float32)
    dy[0, 0, :, 0] = [1, 2, 3, 0]
    dx = abi.dgrad(dy, np.ones((3, 3, 1, 1), np.float32), (1, 4, 4, 1), (1, 1), "same")
    assert np.array_equal(dx[0, 0, :, 0], [3, 6, 5, 3])


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_fprop_parity(case):
    from tests import abi
    x, w, b, dy = _case(case, 0)
    stride, pad = (case[7], case[8]), case[9]
    want = O.conv_fprop(x, w, b, stride, pad, dtype=np.float64)
    abi.close(abi.fprop(x, w, b, stride, pad), want)
    abi.close(abi.fprop(x, w, None, stride, pad), O.conv_fprop(x, w, None, stride, pad, dtype=np.float64))


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_dgrad_parity(case):
    from tests import abi
    x, w, b, dy = _case(case, 1)
    stride, pad = (case[7], case[8]), case[9]
    want = O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64)
    abi.close(abi.dgrad(dy, w, x.shape, stride, pad), want)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_wgrad_parity(case):
    from tests import abi
    x, w, b, dy = _case(case, 2)
    stride, pad = (case[7], case[8]), case[9]
    dw, db = abi.wgrad(x, dy, w.shape, stride, pad)
    want = O.conv_wgrad(x, dy, w.shape[:2], stride, pad, dtype=np.float64)
    abi.close(dw, want, rms_scaled=True)
    abi.close(db, O.conv_dbias(dy, dtype=np.float64), rms_scaled=True)
    # and no less accurate than the reference arithmetic run in float32
    ref32 = O.conv_wgrad(x, dy, w.shape[:2], stride, pad, dtype=np.float32)
    assert np.abs(dw - want).max() <= 2.0 * np.abs(ref32 - want).max() + 1e-6
    dw2, none = abi.wgrad(x, dy, w.shape, stride, pad, want_dbias=False)
    assert none is None and np.array_equal(dw, dw2)       # deterministic


# The benchmark's first configurations at their exact workload: shape, input distribution and draw order.
BASELINE_SMALL = [
    ("cfg1 [128,32,32,3] U[0,1) -> 32", "rand", (128, 32, 32, 3), 32),
    ("cfg2a [128,16,16,32] relu(N(0,1)) -> 64", "relu_randn", (128, 16, 16, 32), 64),
    ("cfg2b [128,8,8,64] relu(N(0,1)) -> 128", "relu_randn", (128, 8, 8, 64), 128),
]


@pytest.mark.parametrize("cfg", BASELINE_SMALL, ids=lambda c: c[0].split()[0])
def test_baseline_configs_at_their_exact_workload(cfg):
    """3x3, stride 1, "same": every output element of fprop and dgrad within 1e-5 + 1e-4*|oracle|; wgrad and dbias
    under the same bar with the absolute term scaled by max(1, rms) (tests/abi.py says why), and no further from
    the float64 value than twice the reference arithmetic run in float32."""
    from tests import abi
    name, kind, x_shape, D = cfg
    x, w, b, dy = abi.baseline_inputs(kind, x_shape, D)
    assert not b.any() and w.shape == (3, 3, x_shape[3], D)
    if kind != "randn":
        assert x.min() >= 0
    st, pad = (1, 1), "same"
    abi.report(name, "fprop", abi.close(abi.fprop(x, w, b, st, pad), O.conv_fprop(x, w, b, st, pad, dtype=np.float64)))
    abi.report(name, "dgrad", abi.close(abi.dgrad(dy, w, x.shape, st, pad),
                                        O.conv_dgrad(dy, w, x.shape[1:3], st, pad, dtype=np.float64)))
    dw, db = abi.wgrad(x, dy, w.shape, st, pad)
    want = O.conv_wgrad(x, dy, (3, 3), st, pad, dtype=np.float64)
    rms = float(np.sqrt(np.mean(want * want)))
    abi.report(name, "wgrad", abi.close(dw, want, rms_scaled=True), "atol * max(1, rms), rms = %.3g" % rms)
    abi.report(name, "dbias", abi.close(db, O.conv_dbias(dy, dtype=np.float64), rms_scaled=True))
    ref32 = O.conv_wgrad(x, dy, (3, 3), st, pad, dtype=np.float32)
    assert np.abs(dw - want).max() <= 2.0 * np.abs(ref32 - want).max() + 1e-6
    abi.report(name, "wgrad vs float32 reference arithmetic",
               float(np.abs(dw - want).max() / max(np.abs(ref32 - want).max(), 1e-30)),
               "max |gpu - f64| / max |f32 einsum - f64|")


def test_bad_arguments_are_errors_not_crashes():
    from aether import _lib
    from aether.tensor import DeviceTensor
    L = _lib.lib()
    t = DeviceTensor.zeros(16)
    assert L.aeth_conv_fprop_f32(None, t.ptr, None, t.ptr, 1, 2, 2, 1, 1, 1, 1, 1, 1, 0, 0) == _lib.AETH_E_INVALID
    assert L.aeth_conv_fprop_f32(t.ptr, t.ptr, None, t.ptr, 1, 2, 2, 1, 1, 3, 3, 1, 1, 0, 0) == _lib.AETH_E_INVALID
    assert L.aeth_conv_fprop_f32(t.ptr, t.ptr, None, t.ptr, 0, 2, 2, 1, 1, 1, 1, 1, 1, 0, 0) == _lib.AETH_E_INVALID
    assert b"aeth_conv_fprop_f32" in L.aeth_last_error()
    with pytest.raises(ValueError):
        _lib.check(L.aeth_conv_wgrad_f32(t.ptr, t.ptr, t.ptr, None, 1, 2, 2, 1, 1, 1, 1, 0, 1, 0, 0))
    with pytest.raises(ValueError):
        _lib.check(L.aeth_free(12345))


def _random_cases(n, seed):
    """Seeded random geometries: channel counts around the vector widths and tile edges,
    strides 1-3, filters 1-5, both paddings, batch sizes that leave ragged row tiles."""
    r = np.random.RandomState(seed)
    out = []
    chans = [1, 2, 3, 4, 5, 8, 12, 16, 20, 31, 32, 33, 48, 64, 72, 96, 128, 136]
    while len(out) < n:
        fH, fW = int(r.choice([1, 2, 3, 3, 3, 5])), int(r.choice([1, 2, 3, 3, 3, 4]))
        sH, sW = int(r.choice([1, 1, 1, 2, 3])), int(r.choice([1, 1, 1, 2, 3]))
        H, W = int(r.randint(fH, 20)), int(r.randint(fW, 20))
        C, D = int(r.choice(chans)), int(r.choice(chans))
        S = int(r.choice([1, 2, 3, 5, 9, 17]))
        pad = "same" if r.rand() < 0.5 else "valid"
        if S * H * W * C * D * fH * fW > 3e8:
            continue
        out.append((S, H, W, C, D, fH, fW, sH, sW, pad))
    return out


@pytest.mark.parametrize("case", _random_cases(48, 20240607), ids=lambda c: "x".join(str(v) for v in c))
def test_random_geometries(case):
    """All three directions on random geometries (the fixed list above names the paths;
    this one looks for the combinations nobody thought of)."""
    from tests import abi
    S, H, W, C, D, fH, fW, sH, sW, pad = case
    x, w, b, dy = _case(case, 11)
    abi.close(abi.fprop(x, w, b, (sH, sW), pad), O.conv_fprop(x, w, b, (sH, sW), pad, dtype=np.float64))
    abi.close(abi.dgrad(dy, w, x.shape, (sH, sW), pad), O.conv_dgrad(dy, w, (H, W), (sH, sW), pad, dtype=np.float64))
    dw, db = abi.wgrad(x, dy, w.shape, (sH, sW), pad)
    abi.close(dw, O.conv_wgrad(x, dy, (fH, fW), (sH, sW), pad, dtype=np.float64), rms_scaled=True)
    abi.close(db, O.conv_dbias(dy, dtype=np.float64), rms_scaled=True)


@pytest.mark.parametrize("case", _random_cases(40, 20250911), ids=lambda c: "x".join(str(v) for v in c))
def test_random_geometries_through_the_backward_call_and_with_cut_classes(case, tune):
    """aeth_conv_bwd_f32 gives the bits of the wgrad and the dgrad call whatever the geometry selects; a dgrad whose classes are
    cut along their borders (forced here: the library cuts large layers only) gives the values of the uncut one."""
    from tests import abi
    from tests.test_gpu_pair import conv_bwd
    S, H, W, C, D, fH, fW, sH, sW, pad = case
    x, w, b, dy = _case(case, 12)
    dw0, db0 = abi.wgrad(x, dy, w.shape, (sH, sW), pad)
    dx0 = abi.dgrad(dy, w, x.shape, (sH, sW), pad)
    dw1, db1, dx1 = conv_bwd(x, dy, w, (sH, sW), pad)
    assert np.array_equal(dw0, dw1) and np.array_equal(db0, db1) and np.array_equal(dx0, dx1)
    tune(gather_border=1)
    cut = abi.dgrad(dy, w, x.shape, (sH, sW), pad)
    abi.close(cut, O.conv_dgrad(dy, w, (H, W), (sH, sW), pad, dtype=np.float64))
    tune(gather_split=0)
    cut2 = abi.dgrad(dy, w, x.shape, (sH, sW), pad)
    tune(gather_border=0, gather_bm=128)
    assert np.array_equal(cut2, abi.dgrad(dy, w, x.shape, (sH, sW), pad))


# The mode in which one workgroup keeps its rows of x in LDS and walks all n tiles is chosen
# for 128-row tiles only, which the library takes from about 800 000 output pixels on; the
# tuning switch forces that tile height so that small inputs reach the same code.
NLOOP_CASES = [
    (8, 48, 48, 64, 256, 1, 1, 1, 1, "valid"),    # K of two slabs, 4 n tiles
    (8, 48, 48, 32, 192, 1, 1, 1, 1, "valid"),    # one slab, 3 n tiles
    (8, 48, 48, 48, 136, 1, 1, 1, 1, "valid"),    # padded second slab, ragged last n tile
    (3, 37, 41, 64, 1024, 1, 1, 1, 1, "valid"),   # the widest output it takes, rows past M in the last tile
    (3, 37, 41, 16, 1088, 1, 1, 1, 1, "valid"),   # wider: back to one workgroup per tile
    (2, 40, 40, 4, 128, 3, 3, 1, 1, "same"),      # K = 36: two slabs of a 3x3 filter, taps decoded per lane
]


@pytest.mark.parametrize("case", NLOOP_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_fprop_parity_with_128_row_tiles(case, tune):
    from tests import abi
    tune(gather_bm=128)
    x, w, b, dy = _case(case, 11)
    stride, pad = (case[7], case[8]), case[9]
    want = O.conv_fprop(x, w, b, stride, pad, dtype=np.float64)
    abi.close(abi.fprop(x, w, b, stride, pad), want)
    abi.close(abi.fprop(x, w, None, stride, pad), O.conv_fprop(x, w, None, stride, pad, dtype=np.float64))



# Plain matrix products with a short K (32 or 64) and a wide output (up to 256 columns, e.g. the 1x1
# convolution 64 -> 256): one persistent workgroup per CU with the whole filter in LDS.  The library
# takes that kernel from 4 tiles of 128 rows per CU on; the dense_res switch lets small inputs reach it.
DENSE_RES_CASES = [
    (8, 48, 48, 64, 256, 1, 1, 1, 1, "valid"),    # 144 tiles: one each
    (8, 48, 48, 32, 192, 1, 1, 1, 1, "valid"),    # one slab, 3 n tiles: two waves have nothing to multiply
    (3, 50, 50, 64, 136, 1, 1, 1, 1, "valid"),    # ragged last n tile, rows past M in the last tile
    (40, 56, 56, 64, 256, 1, 1, 1, 1, "valid"),   # 980 tiles on 256 workgroups: 4 each, the last ones fewer
    (1000, 1, 1, 64, 100, 1, 1, 1, 1, "valid"),   # a dense layer
    (8, 48, 48, 64, 256, 1, 1, 1, 1, "same"),     # "same" with a 1x1 filter pads nothing either
    (8, 24, 24, 48, 256, 1, 1, 1, 1, "valid"),    # K = 48 is not a whole slab: the other kernels
    (8, 24, 24, 64, 256, 1, 1, 2, 2, "valid"),    # stride 2: the other kernels
]


@pytest.mark.parametrize("case", DENSE_RES_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_fprop_with_the_filter_resident_in_lds(case, tune):
    from tests import abi
    tune(dense_res=1, gather_runs=1)              # (run stores are taken from 64 MB of output on)
    x, w, b, dy = _case(case, 12)
    stride, pad = (case[7], case[8]), case[9]
    got = abi.fprop(x, w, b, stride, pad)
    abi.close(got, O.conv_fprop(x, w, b, stride, pad, dtype=np.float64))
    abi.close(abi.fprop(x, w, None, stride, pad), O.conv_fprop(x, w, None, stride, pad, dtype=np.float64))
    tune(gather_runs=0)                           # tiles stored as 16-byte pieces per pixel instead of runs of contiguous channels
    assert np.array_equal(got, abi.fprop(x, w, b, stride, pad))
    # the other kernels add the same products in the same order of k
    tune(dense_res=0)
    assert np.array_equal(got, abi.fprop(x, w, b, stride, pad))


# The direct kernels' fprop gives a lane 8 output channels (16 for 5x5 filters on 2 or 3 channels) and their dgrad 8 from
# 32 output channels on; 4 with direct = 2: the same sums in the same order.
DIRECT_CASES = [
    (5, 28, 28, 1, 32, 3, 3, 1, 1, "same"),
    (3, 12, 12, 2, 16, 3, 3, 2, 2, "same"),      # 16 output channels: two lanes per pixel
    (2, 11, 13, 3, 64, 5, 5, 1, 1, "same"),      # 75 values per channel: 16 per lane
    (2, 9, 9, 3, 256, 3, 3, 1, 1, "valid"),
    (3, 10, 10, 1, 32, 5, 5, 3, 2, "valid"),
    (40, 16, 16, 3, 32, 3, 3, 1, 1, "same"),
]


@pytest.mark.parametrize("case", DIRECT_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_direct_kernels_with_more_channels_per_lane(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 31)
    stride, pad = (case[7], case[8]), case[9]
    got = abi.fprop(x, w, b, stride, pad)
    abi.close(got, O.conv_fprop(x, w, b, stride, pad, dtype=np.float64))
    dx = abi.dgrad(dy, w, x.shape, stride, pad)         # two groups of 4 output channels per lane from 32 channels on
    abi.close(dx, O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(direct=2)
    assert np.array_equal(got, abi.fprop(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))


# fp32 gathers whose slabs lie inside one tap load with addresses made on the scalar unit: lane offsets
# that are constants of the tile, counted from a base the padding below the tensor, the tap in the scalar
# offset, rows outside the image told by one ballot per slab.  the gather_sa switch at 0 is the form with vector
# address arithmetic; both must give the same bits.
SA_CASES = [
    (2, 12, 12, 32, 64, 5, 5, 1, 1, "same"),      # padding 2: the base lies 2 rows and 2 pixels below the tensor
    (1, 9, 9, 64, 64, 3, 3, 1, 1, "same"),        # one small image: most rows of a tile touch a border
    (3, 10, 14, 32, 40, 1, 3, 1, 1, "same"),      # fH = 1: no padding at all under the reference's rule, columns run out
    (3, 10, 14, 32, 40, 3, 1, 1, 1, "same"),      # padding 1 on both axes with a filter one pixel wide
    (2, 17, 17, 64, 64, 3, 3, 2, 2, "same"),      # stride 2
    (2, 16, 16, 96, 72, 3, 3, 1, 1, "valid"),     # 3 slabs per tap, ragged n tile, no padding
    (5, 7, 7, 128, 128, 3, 3, 1, 1, "same"),      # 245 rows: tiles run over image boundaries
    (2, 13, 11, 32, 64, 4, 4, 1, 1, "same"),      # even filter: padding 1, the last taps run out at the far side
]


@pytest.mark.parametrize("bm", ["64", "128"])
@pytest.mark.parametrize("case", SA_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_fprop_dgrad_with_scalar_addressed_loads(case, bm, tune):
    from tests import abi
    tune(gather_bm=int(bm))
    tune(gather_split=0)
    x, w, b, dy = _case(case, 16)
    stride, pad = (case[7], case[8]), case[9]
    y = abi.fprop(x, w, b, stride, pad)
    abi.close(y, O.conv_fprop(x, w, b, stride, pad, dtype=np.float64))
    dx = abi.dgrad(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_sa=0)
    assert np.array_equal(y, abi.fprop(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))
    # tiles stored as runs of contiguous channels (what outputs of 64 MB and more get): the pixels as the MFMAs' first
    # operand, the filter's columns read interleaved
    tune(gather_sa=-1, gather_runs=1)
    assert np.array_equal(y, abi.fprop(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))
    tune(gather_bkn=0, gather_direct_b=0)          # ... with the filter packed
    assert np.array_equal(y, abi.fprop(x, w, b, stride, pad))
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))


# dgrad whose slabs lie inside one filter tap (output channels in whole slabs of 32, input channels filling
# their tiles) reads its B operand from the filter itself instead of a packed copy: row (tap, c) of
# w[fH][fW][C][D] is contiguous in d, which is dgrad's k.  The gather_direct_b switch at 0 packs as before;
# both must give the same bits (same slabs, same order).
DIRECT_B_CASES = [
    (4, 16, 16, 32, 64, 3, 3, 1, 1, "same"),      # 32 input channels: 32-wide tiles
    (3, 8, 8, 64, 128, 3, 3, 1, 1, "same"),       # 4 slabs per tap
    (2, 20, 20, 64, 64, 3, 3, 2, 2, "same"),      # stride 2: classes of 4, 2, 2 and 1 taps (the 1- and 2-tap ones keep packing: K < 3 slabs)
    (2, 13, 11, 128, 96, 5, 5, 1, 1, "same"),     # 25 taps of 3 slabs, two n tiles
    (2, 12, 12, 64, 32, 4, 4, 3, 3, "valid"),     # stride 3, even filter: taps differ per class
    (128, 1, 1, 2048, 256, 1, 1, 1, 1, "valid"),  # a dense layer's input gradient: one tap, split K
    (2, 12, 12, 48, 64, 3, 3, 1, 1, "same"),      # 48 input channels do not fill a 64-wide tile: packed
    (2, 12, 12, 64, 40, 3, 3, 1, 1, "same"),      # 40 output channels: slabs straddle taps, packed
]


@pytest.mark.parametrize("case", DIRECT_B_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_dgrad_reading_the_filter_in_place(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 21)
    stride, pad = (case[7], case[8]), case[9]
    dx = abi.dgrad(dy, w, x.shape, stride, pad)
    abi.close(dx, O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_direct_b=0)
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))
    tune(gather_direct_b=-1, gather_sa=0)             # vector-addressed loads: the other form of the B loads
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))


# fp32 fprop with at least three slabs of K and whole n tiles reads its B operand from the filter itself too:
# w[fH][fW][C][D] is the [K][N] matrix with n contiguous, fetched as slabs of 32 rows of k and read with 4-byte
# operand reads.  The gather_bkn switch at 0 packs as before; same bits (same slabs, same order).
BKN_CASES = [
    (4, 16, 16, 32, 64, 3, 3, 1, 1, "same"),      # 9 slabs, 64-wide tiles: odd rows stored with their halves swapped
    (4, 16, 16, 32, 32, 3, 3, 1, 1, "same"),      # 32-wide tiles: 8 rows per load
    (3, 9, 9, 64, 128, 3, 3, 2, 2, "valid"),      # stride 2, two n tiles
    (2, 10, 10, 3, 64, 5, 5, 1, 1, "same"),       # K = 75: the last slab has rows past K, taps decoded per lane
    (2, 10, 10, 12, 32, 3, 3, 1, 1, "valid"),     # K = 108, 12 channels
    (128, 1, 1, 2048, 256, 1, 1, 1, 1, "valid"),  # a dense layer on a small batch: split K
    (40, 12, 12, 64, 64, 3, 3, 1, 1, "same"),     # 5760 rows: 128-row tiles
    (2, 12, 12, 64, 40, 3, 3, 1, 1, "same"),      # 40 output channels are not whole n tiles: packed
]


@pytest.mark.parametrize("case", BKN_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_fprop_reading_the_filter_in_place(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 22)
    stride, pad = (case[7], case[8]), case[9]
    y = abi.fprop(x, w, b, stride, pad)
    abi.close(y, O.conv_fprop(x, w, b, stride, pad, dtype=np.float64))
    tune(gather_bkn=0)
    assert np.array_equal(y, abi.fprop(x, w, b, stride, pad))
    tune(gather_bkn=-1, gather_sa=0)                  # vector-addressed loads
    assert np.array_equal(y, abi.fprop(x, w, b, stride, pad))


# Products with at most 16 output channels (a classifier head) and a 1x1 filter go to kernels with one thread
# per output, one launch per direction and no scratch memory; wgrad only where the rows are few (at most 1024).
# The narrow switch at 0 sends them to the slab kernels: other orders of the same sums.
NARROW_CASES = [
    (128, 1, 1, 256, 10, 1, 1, 1, 1, "valid"),    # Layer_Dense(256, 10) on a batch of 128
    (1000, 1, 1, 37, 16, 1, 1, 1, 1, "valid"),    # 16 channels, K not a multiple of 4
    (3, 9, 7, 24, 1, 1, 1, 1, 1, "same"),         # a 1x1 convolution onto one channel
    (1500, 1, 1, 64, 5, 1, 1, 1, 1, "valid"),     # 1500 rows: wgrad by the slab kernels
    (2, 6, 6, 8, 17, 1, 1, 1, 1, "valid"),        # 17 channels: the slab kernels
]


@pytest.mark.parametrize("case", NARROW_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_products_with_few_output_channels(case, tune):
    from tests import abi
    S, H, W, C, D, fH, fW, sH, sW, pad = case
    x, w, b, dy = _case(case, 31)
    got = {}
    for mode in (-1, 0):
        tune(narrow=mode)
        y = abi.fprop(x, w, b, (sH, sW), pad)
        abi.close(y, O.conv_fprop(x, w, b, (sH, sW), pad, dtype=np.float64))
        abi.close(abi.fprop(x, w, None, (sH, sW), pad), O.conv_fprop(x, w, None, (sH, sW), pad, dtype=np.float64))
        dx = abi.dgrad(dy, w, x.shape, (sH, sW), pad)
        abi.close(dx, O.conv_dgrad(dy, w, (H, W), (sH, sW), pad, dtype=np.float64))
        dw, db = abi.wgrad(x, dy, w.shape, (sH, sW), pad)
        abi.close(dw, O.conv_wgrad(x, dy, (fH, fW), (sH, sW), pad, dtype=np.float64), rms_scaled=True)
        abi.close(db, O.conv_dbias(dy, dtype=np.float64), rms_scaled=True)
        dw2, _ = abi.wgrad(x, dy, w.shape, (sH, sW), pad, want_dbias=False)
        assert np.array_equal(dw, dw2)
        got[mode] = (y, dx, dw, db)
    for a, c in zip(got[-1], got[0]):
        abi.close(a, c, rtol=1e-4, atol=1e-5, rms_scaled=True)


# Strided dgrad whose last rows / columns are reached by no output pixel: the classes' pixel grids stop
# at the last reachable index and one small launch zeroes the strips.  The gather_clip switch at 0
# multiplies the full grids (every tap of those pixels falls outside dy: zeros); same bits either way.
CLIP_CASES = [
    (3, 12, 12, 8, 16, 3, 3, 2, 2, "valid"),      # row and column 11 untouched
    (2, 28, 28, 32, 64, 3, 3, 2, 2, "valid"),     # the stride-2 benchmark layer's geometry, fewer channels
    (2, 14, 13, 6, 8, 2, 2, 3, 3, "valid"),       # filter smaller than the stride: gaps (classes without taps) and two untouched columns
    (2, 11, 9, 5, 8, 5, 5, 3, 3, "valid"),        # 5 channels: scalar stores in the strip; one untouched column
    (2, 10, 10, 4, 8, 3, 3, 2, 2, "same"),        # nothing to clip
    (2, 9, 16, 64, 32, 3, 3, 1, 4, "valid"),      # stride (1, 4): three untouched columns, none of the rows
]


@pytest.mark.parametrize("case", CLIP_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_strided_dgrad_with_clipped_class_grids(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 22)
    stride, pad = (case[7], case[8]), case[9]
    dx = abi.dgrad(dy, w, x.shape, stride, pad)          # the output buffer starts as NaN: every element must be written
    abi.close(dx, O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64))
    tune(gather_clip=0)
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))


# Strided fp32 dgrad whose classes all take the 128 x 64 slab kernel (64 input channels and more, many pixels; the
# gather_bm switch lets small inputs reach it): the classes go out as ONE grid, most taps first.  With gather_merge at 0
# every class is a launch of its own; same bits either way.  S, H, W, C, D, fH, fW, sH, sW, padding
MERGED_CLASS_CASES = [
    (6, 13, 13, 64, 64, 3, 3, 2, 2, "valid"),     # 4 classes of 4, 2, 2 and 1 taps, clipped to different pixel grids
    (4, 12, 14, 128, 96, 3, 3, 2, 2, "same"),     # two n tiles per class
    (5, 9, 16, 64, 32, 3, 3, 1, 2, "same"),       # stride (1, 2): 2 classes
    (3, 11, 11, 72, 64, 5, 5, 2, 2, "same"),      # 72 input channels: a ragged n tile; 9, 6, 6 and 4 taps
    (2, 12, 12, 64, 64, 3, 3, 3, 3, "valid"),     # 9 classes: more than one grid takes, one launch each
    (4, 10, 10, 64, 40, 2, 2, 2, 2, "valid"),     # one tap per class; 40 output channels: slabs that are not whole
]


@pytest.mark.parametrize("case", MERGED_CLASS_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_strided_dgrad_with_its_classes_in_one_launch(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 23)
    stride, pad = (case[7], case[8]), case[9]
    want = O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64)
    tune(gather_bm=128, gather_split=0)
    dx = abi.dgrad(dy, w, x.shape, stride, pad)
    abi.close(dx, want)
    tune(gather_runs=1)                                  # the tiles stored as runs of contiguous channels
    dx_runs = abi.dgrad(dy, w, x.shape, stride, pad)
    assert np.array_equal(dx, dx_runs)
    tune(gather_merge=0)
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))
    tune(gather_runs=0)
    assert np.array_equal(dx, abi.dgrad(dy, w, x.shape, stride, pad))


# The classes of an fp32 dgrad cut along their borders: the first and last rows and columns of a class see fewer of
# its taps inside dy than the interior does, and a tile that mixes them multiplies the missing taps as zeros.  Cut into the
# runs of rows and columns that see the same taps, every part is a problem with only those taps; all parts take 128-row tiles
# and go out in grids of up to 9 problems.  The library does this for layers whose classes are large; the gather_border switch
# lets small inputs reach it.  The sums run over the same taps in the same order: same values as the uncut classes.
BORDER_CASES = [
    (6, 28, 28, 64, 64, 3, 3, 2, 2, "valid"),     # the stride-2 benchmark layer's geometry: 16 parts (9 + 3 + 3 + 1)
    (4, 28, 28, 64, 96, 3, 3, 2, 2, "same"),      # padding 1: other classes lose their taps at the other end
    (3, 17, 15, 96, 64, 5, 5, 2, 2, "same"),      # 5x5: up to 3 taps per dimension and class, two border rows at each end
    (3, 12, 16, 64, 32, 3, 3, 1, 2, "same"),      # stride (1, 2): 2 classes, rows cut as well as columns
    (2, 14, 13, 64, 32, 2, 2, 3, 3, "valid"),     # filter smaller than the stride: classes without taps
    (2, 9, 9, 72, 64, 7, 7, 2, 2, "same"),        # more parts than one dgrad may hold: the classes stay whole
    (5, 10, 10, 24, 64, 3, 3, 2, 2, "same"),      # 24 input channels: 32-wide tiles, a launch per part
    (3, 11, 11, 64, 40, 3, 3, 2, 2, "same"),      # 40 output channels: not whole slabs, the classes stay whole
    (3, 14, 14, 64, 64, 3, 3, 1, 1, "same"),      # unit stride: one class, 9 parts (interior, 4 edges, 4 corners)
    (2, 12, 10, 128, 32, 5, 3, 1, 1, "same"),     # 5x3 at unit stride: 5 row parts x 3 column parts
    (2, 12, 12, 64, 64, 3, 3, 1, 1, "valid"),     # no padding: every tap inside, the class stays whole
]


@pytest.mark.parametrize("case", BORDER_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_dgrad_cut_along_the_borders_of_its_classes(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 24)
    stride, pad = (case[7], case[8]), case[9]
    want = O.conv_dgrad(dy, w, x.shape[1:3], stride, pad, dtype=np.float64)
    tune(gather_border=0, gather_bm=128, gather_split=0)  # the same tiles and an unsplit K for the classes left whole
    whole = abi.dgrad(dy, w, x.shape, stride, pad)
    abi.close(whole, want)
    tune(gather_border=1)
    cut = abi.dgrad(dy, w, x.shape, stride, pad)          # the output buffer starts as NaN: every element must be written
    abi.close(cut, want)
    assert np.array_equal(whole, cut)
    tune(gather_merge=0)                                  # a launch per part
    assert np.array_equal(cut, abi.dgrad(dy, w, x.shape, stride, pad))
    tune(gather_merge=-1, gather_runs=1)
    assert np.array_equal(cut, abi.dgrad(dy, w, x.shape, stride, pad))


# The same cut for a padded fp32 fprop at unit stride: the output's first and last rows and columns see fewer taps inside x.
# Every part reads the filter in place as the [K][N] operand, at the rows of its own taps.  S, H, W, C, D, fH, fW, sH, sW, padding
FPROP_BORDER_CASES = [
    (3, 14, 14, 64, 64, 3, 3, 1, 1, "same"),      # nine parts: interior, four edges, four corners
    (2, 56, 56, 64, 64, 3, 3, 1, 1, "same"),      # the headline layer's geometry
    (2, 12, 10, 32, 128, 5, 3, 1, 1, "same"),     # 5x3: five row parts x three column parts, two n tiles
    (2, 9, 9, 64, 64, 7, 7, 1, 1, "same"),        # more parts than one call may hold: the fprop stays whole
    (3, 11, 13, 96, 96, 3, 3, 1, 1, "same"),      # 96 output channels: not whole n tiles, every part packs its taps
    (2, 12, 12, 64, 64, 3, 3, 1, 1, "valid"),     # no padding: nothing to cut
    (2, 10, 10, 24, 64, 3, 3, 1, 1, "same"),      # 24 input channels: slabs that are not whole, the fprop stays whole
    (2, 16, 16, 64, 64, 2, 2, 1, 1, "same"),      # even filter: "same" pads nothing here (P = 0)
]


@pytest.mark.parametrize("case", FPROP_BORDER_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_fprop_cut_along_the_borders_of_the_output(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 25)
    stride, pad = (case[7], case[8]), case[9]
    want = O.conv_fprop(x, w, b, stride, pad, dtype=np.float64)
    tune(gather_border=0, gather_bm=128, gather_split=0)
    whole = abi.fprop(x, w, b, stride, pad)
    abi.close(whole, want)
    tune(gather_border=1)
    cut = abi.fprop(x, w, b, stride, pad)                 # the output buffer starts as NaN: every element must be written
    abi.close(cut, want)
    assert np.array_equal(whole, cut)
    tune(gather_merge=0)                                  # nothing is cut without the shared launch
    assert np.array_equal(cut, abi.fprop(x, w, b, stride, pad))
    tune(gather_merge=-1, gather_runs=1)
    assert np.array_equal(cut, abi.fprop(x, w, b, stride, pad))
    tune(gather_bkn=0)                                    # the parts pack their taps instead of reading the filter in place
    assert np.array_equal(cut, abi.fprop(x, w, b, stride, pad))
    nb = abi.fprop(x, w, None, stride, pad)               # no bias
    abi.close(nb, O.conv_fprop(x, w, np.zeros_like(b), stride, pad, dtype=np.float64))


# fp32 wgrad of a unit-stride filter of at most 9 taps on 64 input channels and at most 64 output
# channels, on rows of 28, 32, 56 or 64 output pixels: one persistent workgroup per CU keeps the whole
# K x N result in registers (12 multiplying waves of three 32 x 32 blocks) and a loading wave brings one
# output row and the padded source rows under it at a time.  The library takes that kernel from 4 rows
# per CU on; the wgrad_halo switch lets small inputs reach it.
WGRAD_HALO_F32_CASES = [
    (2, 56, 56, 64, 64, 3, 3, 1, 1, "same"),      # the 56x56x64 layer
    (3, 28, 28, 64, 64, 3, 3, 1, 1, "same"),
    (2, 30, 34, 64, 48, 3, 3, 1, 1, "valid"),     # 32 pixels per row, no padding, 48 output channels
    (2, 20, 65, 64, 64, 2, 2, 1, 1, "valid"),     # even filter: 8 k blocks of the 18 carry taps
    (2, 8, 58, 64, 40, 1, 3, 1, 1, "valid"),      # one filter row
    (7, 56, 56, 64, 64, 3, 3, 1, 1, "same"),      # 392 rows on 196 workgroups of 2
    (2, 14, 14, 64, 64, 3, 3, 1, 1, "same"),      # rows of 14 pixels: other kernels
    (2, 28, 28, 32, 64, 3, 3, 1, 1, "same"),      # 32 input channels: other kernels
]


@pytest.mark.parametrize("case", WGRAD_HALO_F32_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_wgrad_with_the_whole_result_in_registers(case, tune):
    from tests import abi
    tune(wgrad_halo=1)
    x, w, b, dy = _case(case, 14)
    stride, pad = (case[7], case[8]), case[9]
    dw, db = abi.wgrad(x, dy, w.shape, stride, pad)
    want = O.conv_wgrad(x, dy, w.shape[:2], stride, pad, dtype=np.float64)
    abi.close(dw, want, rms_scaled=True)
    abi.close(db, O.conv_dbias(dy, dtype=np.float64), rms_scaled=True)
    ref32 = O.conv_wgrad(x, dy, w.shape[:2], stride, pad, dtype=np.float32)
    assert np.abs(dw - want).max() <= 2.0 * np.abs(ref32 - want).max() + 1e-6
    dw2, none = abi.wgrad(x, dy, w.shape, stride, pad, want_dbias=False)
    assert none is None and np.array_equal(dw, dw2)       # deterministic


# 1x1 filters on 33 to 64 input channels and at least 128 output channels: the library multiplies dy^T . x (full-width
# k tiles over dy's columns, one n tile over x's) and the split reduction writes the transpose back.
WGRAD_SWAP_CASES = [
    (2, 56, 56, 64, 256, 1, 1, 1, 1, "valid"),    # the 64 -> 256 layer
    (3, 9, 11, 64, 128, 1, 1, 1, 1, "valid"),     # 297 rows: a last slab with 9 rows
    (2, 14, 14, 48, 192, 1, 1, 1, 1, "valid"),    # 48 input channels, a second k tile half full
    (1, 33, 31, 36, 132, 1, 1, 1, 1, "valid"),    # 36 and 132 channels: edge tiles in both directions
    (5, 1, 1, 64, 320, 1, 1, 1, 1, "valid"),      # 5 rows (a dense layer's shape), three k tiles
    (2, 28, 28, 64, 256, 1, 1, 1, 1, "same"),     # "same" on a 1x1 filter pads nothing
]


@pytest.mark.parametrize("case", WGRAD_SWAP_CASES, ids=lambda c: "x".join(str(v) for v in c))
def test_wgrad_of_1x1_filters_with_swapped_operands(case, tune):
    from tests import abi
    x, w, b, dy = _case(case, 15)
    stride, pad = (case[7], case[8]), case[9]
    want = O.conv_wgrad(x, dy, w.shape[:2], stride, pad, dtype=np.float64)
    want_db = O.conv_dbias(dy, dtype=np.float64)
    ref32 = O.conv_wgrad(x, dy, w.shape[:2], stride, pad, dtype=np.float32)
    results = {}
    for swap in (1, 0):
        tune(wgrad_swap=swap)
        dw, db = abi.wgrad(x, dy, w.shape, stride, pad)
        abi.close(dw, want, rms_scaled=True)
        abi.close(db, want_db, rms_scaled=True)
        assert np.abs(dw - want).max() <= 2.0 * np.abs(ref32 - want).max() + 1e-6
        dw2, none = abi.wgrad(x, dy, w.shape, stride, pad, want_dbias=False)
        assert none is None and np.array_equal(dw, dw2)   # deterministic, with and without dbias
        results[swap] = dw
    # two orders of summation over the same products
    assert np.allclose(results[0], results[1], rtol=1e-4, atol=1e-4 * max(1.0, float(np.abs(want).max())))
