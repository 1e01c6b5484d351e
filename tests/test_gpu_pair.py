"""aeth_conv_bwd_f32 / aeth_dense_bwd_f32: a layer's weight gradient and input gradient in one call, which on small layers
is one launch shared between the two kernels.  The call must give the bits of aeth_conv_wgrad_f32 followed by
aeth_conv_dgrad_f32 (Conv_Layer.backward, CNN_classes_cupy.py:122-153; Layer_Dense.backward :333-354), whichever kernels
the shape selects, and the values of the oracle."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu


def conv_bwd(x, dy, w, strides, padding):
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    dims, _ = abi.conv_dims(x.shape, w.shape, strides, padding)
    xd, dyd, wd = (DeviceTensor.from_numpy(a, np.float32) for a in (x, dy, w))
    dw, db, dx = DeviceTensor.full(w.shape, np.nan), DeviceTensor.full(w.shape[3], np.nan), DeviceTensor.full(x.shape, np.nan)
    _lib.check(_lib.lib().aeth_conv_bwd_f32(xd.ptr, dyd.ptr, wd.ptr, dw.ptr, db.ptr, dx.ptr, *dims))
    return dw.get(), db.get(), dx.get()


def inputs(rng, x_shape, D, f, strides, padding):
    from tests import abi
    x = rng.standard_normal(x_shape).astype(np.float32)
    w = (rng.standard_normal((f, f, x_shape[3], D)) * 0.1).astype(np.float32)
    _, yshape = abi.conv_dims(x.shape, w.shape, strides, padding)
    dy = rng.standard_normal(yshape).astype(np.float32)
    return x, w, dy


# (x shape, filters, filter size, strides, padding, what the shape selects)
CASES = [
    ((128, 32, 32, 3), 32, 3, (1, 1), "same", "direct dgrad + 128-wide wgrad (first layer of the three-block CNN)"),
    ((128, 16, 16, 32), 64, 3, (1, 1), "same", "128x32 dgrad tiles + 192-wide wgrad"),
    ((128, 8, 8, 64), 128, 3, (1, 1), "same", "64x64 dgrad tiles with split K + 192-wide wgrad"),
    ((64, 12, 12, 32), 32, 3, (1, 1), "valid", "no padding"),
    ((32, 9, 11, 24), 40, 3, (1, 1), "same", "ragged tiles, channel counts off the tile sizes"),
    ((16, 10, 10, 5), 8, 3, (1, 1), "same", "channels not a multiple of 4: one float per lane in wgrad"),
    ((8, 8, 8, 256), 128, 1, (1, 1), "valid", "1x1 filter"),
    ((16, 16, 16, 64), 64, 3, (1, 1), "same", "64 input channels"),
    ((32, 14, 14, 32), 48, 3, (2, 2), "same", "stride 2: the dgrad goes out in classes, the wgrad alone"),
    ((4, 20, 20, 3), 16, 5, (1, 1), "same", "5x5 on 3 channels: direct dgrad of another shape"),
    ((64, 56, 56, 32), 64, 3, (1, 1), "same", "many tiles: the launches stay apart"),
]


@pytest.mark.parametrize("x_shape,D,f,strides,padding,what", CASES, ids=[c[-1] for c in CASES])
def test_conv_bwd_is_wgrad_then_dgrad(x_shape, D, f, strides, padding, what, tune):
    from tests import abi
    rng = np.random.default_rng(sum(x_shape) * 131 + D * 7 + f)
    x, w, dy = inputs(rng, x_shape, D, f, strides, padding)
    dw0, db0 = abi.wgrad(x, dy, w.shape, strides, padding)
    dx0 = abi.dgrad(dy, w, x.shape, strides, padding)
    dw1, db1, dx1 = conv_bwd(x, dy, w, strides, padding)
    assert np.array_equal(dw0, dw1) and np.array_equal(db0, db1) and np.array_equal(dx0, dx1), what
    tune(pair_bwd=0)                                       # the same call with the launches kept apart
    dw2, db2, dx2 = conv_bwd(x, dy, w, strides, padding)
    assert np.array_equal(dw0, dw2) and np.array_equal(db0, db2) and np.array_equal(dx0, dx2)
    if x.size <= 2_000_000:
        abi.close(dw1, O.conv_wgrad(x, dy, w.shape[:2], strides, padding, dtype=np.float64), rms_scaled=True)
        abi.close(db1, O.conv_dbias(dy, dtype=np.float64), rms_scaled=True)
        abi.close(dx1, O.conv_dgrad(dy, w, x.shape[1:3], strides, padding, dtype=np.float64))


def test_conv_bwd_twice_and_after_a_larger_layer():
    """The held wgrad's partial sums sit at the start of the workspace and the dgrad's plan may grow the workspace before the
    pair is launched: a small layer first (small workspace), then one whose dgrad needs more, then the small one again."""
    from tests import abi
    rng = np.random.default_rng(7)
    small = inputs(rng, (16, 8, 8, 64), 64, 3, (1, 1), "same")
    large = inputs(rng, (128, 8, 8, 64), 128, 3, (1, 1), "same")
    for x, w, dy in (small, large, small):
        dw0, db0 = abi.wgrad(x, dy, w.shape, (1, 1), "same")
        dx0 = abi.dgrad(dy, w, x.shape, (1, 1), "same")
        for _ in range(2):
            dw1, db1, dx1 = conv_bwd(x, dy, w, (1, 1), "same")
            assert np.array_equal(dw0, dw1) and np.array_equal(db0, db1) and np.array_equal(dx0, dx1)


@pytest.mark.parametrize("M,n_in,n_out,act", [(128, 2048, 256, True), (128, 2048, 256, False), (64, 512, 128, True),
                                               (96, 300, 52, False), (256, 64, 1000, True)])
def test_dense_bwd_is_its_three_products(M, n_in, n_out, act):
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    rng = np.random.default_rng(M + n_in)
    x = rng.standard_normal((M, n_in)).astype(np.float32)
    w = (rng.standard_normal((n_in, n_out)) * 0.05).astype(np.float32)
    dy = rng.standard_normal((M, n_out)).astype(np.float32)
    pre = rng.standard_normal((M, n_in)).astype(np.float32)              # input of the activation in front of the layer
    L = _lib.lib()
    xd, wd, dyd, pred = (DeviceTensor.from_numpy(a, np.float32) for a in (x, w, dy, pre))
    dw0, db0, dx0 = DeviceTensor.full(w.shape, np.nan), DeviceTensor.full(n_out, np.nan), DeviceTensor.full(x.shape, np.nan)
    _lib.check(L.aeth_dense_wgrad_f32(xd.ptr, dyd.ptr, dw0.ptr, db0.ptr, M, n_in, n_out))
    _lib.check(L.aeth_dense_dgrad_f32(dyd.ptr, wd.ptr, dx0.ptr, M, n_in, n_out))
    adx0 = DeviceTensor.full(x.shape, np.nan)
    _lib.check(L.aeth_relu_bwd_f32(pred.ptr, dx0.ptr, adx0.ptr, 0.01, x.size))
    dw1, db1, dx1 = DeviceTensor.full(w.shape, np.nan), DeviceTensor.full(n_out, np.nan), DeviceTensor.full(x.shape, np.nan)
    adx1 = DeviceTensor.full(x.shape, np.nan)
    _lib.check(L.aeth_dense_bwd_f32(xd.ptr, dyd.ptr, wd.ptr, dw1.ptr, db1.ptr, dx1.ptr, pred.ptr if act else None,
                                    adx1.ptr if act else None, 0.01, M, n_in, n_out))
    assert np.array_equal(dw0.get(), dw1.get()) and np.array_equal(db0.get(), db1.get()) and np.array_equal(dx0.get(), dx1.get())
    if act:
        assert np.array_equal(adx0.get(), adx1.get())
    abi.close(dw1.get(), x.astype(np.float64).T @ dy.astype(np.float64), rms_scaled=True)
    abi.close(dx1.get(), dy.astype(np.float64) @ w.astype(np.float64).T)
