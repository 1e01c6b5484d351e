"""The benchmark's full-size shapes on the GPU.

Every output element of fprop and dgrad is compared with the float64 oracle (the
oracle runs over the batch in chunks on a few host threads: convolution is independent
per sample), and bit for bit with a second, independently scheduled kernel of the
library (other loads, other tiles, other store schedule, same order of k): a handful of
wrong elements among tens of millions cannot hide in a global sum.  wgrad is linear in
the upstream gradient, so a gradient that is zero outside one sample must reproduce the
oracle's wgrad of that sample; and the adjoint identities <y - b, dy> = <x, dx> = <W, dW>
tie the three full-size results together."""
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

# the second kernel each full-size result is compared with, bit for bit
OTHER_KERNELS = dict(gather_sa=0, gather_res=0, dense_res=0, gather_wide=0)


def whole_tensor_close(got, oracle_of_rows, S, chunk=8, threads=8):
    """abi.close(got[rows], oracle_of_rows(lo, hi)) for every chunk of the batch."""
    from tests import abi
    spans = [(lo, min(lo + chunk, S)) for lo in range(0, S, chunk)]

    def check(span):
        lo, hi = span
        return abi.close(got[lo:hi], oracle_of_rows(lo, hi))

    with ThreadPoolExecutor(max_workers=threads) as pool:
        return max(pool.map(check, spans))

def whole_batch_wgrad(x, dy, filter_size, stride, pad, chunk=8, threads=8):
    """The oracle's float64 wgrad of the whole batch: the sum of its wgrads of the chunks (wgrad is additive over
    samples; float64 addition of 32 to 128 partial results does not touch the digits compared)."""
    spans = [(lo, min(lo + chunk, x.shape[0])) for lo in range(0, x.shape[0], chunk)]
    with ThreadPoolExecutor(max_workers=threads) as pool:
        parts = pool.map(lambda s: O.conv_wgrad(x[s[0]:s[1]], dy[s[0]:s[1]], filter_size, stride, pad,
                                                dtype=np.float64), spans)
        return sum(parts)


FULL = [
    # name, S, H, W, C, D, fH, fW, stride, padding
    ("resnet3x3", 256, 56, 56, 64, 64, 3, 3, 1, "same"),
    ("resnet1x1", 256, 56, 56, 64, 256, 1, 1, 1, "valid"),
    ("wide_s2", 1024, 28, 28, 128, 256, 3, 3, 2, "valid"),
]
LABEL = {"resnet3x3": "cfg4 [256,56,56,64] N(0,1) -> 64, 3x3", "resnet1x1": "cfg4' [256,56,56,64] N(0,1) -> 256, 1x1 valid",
         "wide_s2": "cfg5 [1024,28,28,128] N(0,1) -> 256, 3x3 stride 2 valid"}


@pytest.mark.parametrize("cfg", FULL, ids=lambda c: c[0])
def test_full_size_conv(cfg, tune):
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    name, S, H, W, C, D, fH, fW, st, pad = cfg
    stride = (st, st)
    # the benchmark's draw: seed 0, input, layer constructor, upstream gradient; then a bias that is not zero
    x, w, _, dy = abi.baseline_inputs("randn", (S, H, W, C), D, (fH, fW), stride, pad)
    b = np.random.randn(D).astype(np.float32)
    dims, yshape = abi.conv_dims(x.shape, w.shape, stride, pad)
    L = _lib.lib()
    xd, wd, bd, dyd = (DeviceTensor.from_numpy(a) for a in (x, w, b, dy))
    y = DeviceTensor.full(yshape, np.nan)
    dx = DeviceTensor.full(x.shape, np.nan)
    dw = DeviceTensor.full(w.shape, np.nan)
    db = DeviceTensor.full(D, np.nan)
    _lib.check(L.aeth_conv_fprop_f32(xd.ptr, wd.ptr, bd.ptr, y.ptr, *dims))
    _lib.check(L.aeth_conv_dgrad_f32(dyd.ptr, wd.ptr, dx.ptr, *dims))
    _lib.check(L.aeth_conv_wgrad_f32(xd.ptr, dyd.ptr, dw.ptr, db.ptr, *dims))
    y_h, dx_h, dw_h, db_h = y.get(), dx.get(), dw.get(), db.get()
    assert np.all(np.isfinite(y_h)) and np.all(np.isfinite(dx_h))

    # every element against the oracle
    abi.report(LABEL[name], "fprop", whole_tensor_close(
        y_h, lambda lo, hi: O.conv_fprop(x[lo:hi], w, b, stride, pad, dtype=np.float64), S))
    abi.report(LABEL[name], "dgrad", whole_tensor_close(
        dx_h, lambda lo, hi: O.conv_dgrad(dy[lo:hi], w, (H, W), stride, pad, dtype=np.float64), S))
    # and bit for bit against the library's other kernels for these shapes
    tune(**OTHER_KERNELS)
    y2 = DeviceTensor.full(yshape, np.nan)
    _lib.check(L.aeth_conv_fprop_f32(xd.ptr, wd.ptr, bd.ptr, y2.ptr, *dims))
    assert np.array_equal(y_h, y2.get()), "fprop: the two kernels disagree"
    del y2
    dx2 = DeviceTensor.full(x.shape, np.nan)
    _lib.check(L.aeth_conv_dgrad_f32(dyd.ptr, wd.ptr, dx2.ptr, *dims))
    assert np.array_equal(dx_h, dx2.get()), "dgrad: the two kernels disagree"
    del dx2
    tune(**{k: -1 for k in OTHER_KERNELS})
    if name == "wide_s2":
        # 28x28, 3x3 stride 2 valid: row/column 27 is never read, so its gradient is exactly 0
        assert np.all(dx_h[:, 27] == 0) and np.all(dx_h[:, :, 27] == 0)

    # adjoint identities in float64 on the full tensors
    lhs = float(np.sum((y_h.astype(np.float64) - b.astype(np.float64)) * dy))
    rhs_x = float(np.sum(x.astype(np.float64) * dx_h))
    rhs_w = float(np.sum(w.astype(np.float64) * dw_h))
    scale = float(np.sqrt(np.sum(y_h.astype(np.float64) ** 2)) * np.sqrt(np.sum(dy.astype(np.float64) ** 2)))
    assert abs(lhs - rhs_x) <= 1e-6 * scale, (lhs, rhs_x)
    assert abs(lhs - rhs_w) <= 1e-6 * scale, (lhs, rhs_w)
    abi.report(LABEL[name], "dbias", abi.close(db_h, np.sum(dy.astype(np.float64), axis=(0, 1, 2)), rms_scaled=True))
    # every element of wgrad against the oracle's float64 sum over the whole batch
    want = whole_batch_wgrad(x, dy, (fH, fW), stride, pad)
    abi.report(LABEL[name], "wgrad", abi.close(dw_h, want, rms_scaled=True),
               "atol * max(1, rms), rms = %.3g" % float(np.sqrt(np.mean(want * want))))

    # wgrad of a gradient supported on one sample == the oracle's wgrad of that sample
    for s in (0, S - 1):
        dy1 = np.zeros_like(dy)
        dy1[s] = dy[s]
        dyd.set(dy1)
        _lib.check(L.aeth_conv_wgrad_f32(xd.ptr, dyd.ptr, dw.ptr, db.ptr, *dims))
        want = O.conv_wgrad(x[s:s + 1], dy[s:s + 1], (fH, fW), stride, pad, dtype=np.float64)
        abi.close(dw.get(), want, rms_scaled=True)
        abi.close(db.get(), np.sum(dy[s].astype(np.float64), axis=(0, 1)), rms_scaled=True)

    # wgrad is additive over the batch: halves sum to the whole
    half = S // 2
    dy1 = dy.copy()
    dy1[half:] = 0
    dyd.set(dy1)
    _lib.check(L.aeth_conv_wgrad_f32(xd.ptr, dyd.ptr, dw.ptr, None, *dims))
    first = dw.get().astype(np.float64)
    dy1 = dy.copy()
    dy1[:half] = 0
    dyd.set(dy1)
    _lib.check(L.aeth_conv_wgrad_f32(xd.ptr, dyd.ptr, dw.ptr, None, *dims))
    abi.close(dw_h, first + dw.get().astype(np.float64), rms_scaled=True)


@pytest.mark.parametrize("cfg", FULL, ids=lambda c: c[0] + "_bf16")
def test_full_size_conv_bf16(cfg, tune):
    """The bf16-input kernels at the same full-size shapes.  Inputs are rounded to bf16
    on the device; the oracle gets the same rounded values, so the fp32 tolerance
    applies (bf16 products are exact in fp32, accumulation is fp32).  The adjoint
    identities hold for the rounded operands: <y - b, r(dy)> = <r(x), dx> when dx is
    computed from r(dy) and r(w), and likewise for dW."""
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    name, S, H, W, C, D, fH, fW, st, pad = cfg
    stride = (st, st)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((S, H, W, C), dtype=np.float32)
    w = (rng.standard_normal((fH, fW, C, D), dtype=np.float32) * np.float32(np.sqrt(2.0 / (fH * fW * C))))
    b = rng.standard_normal(D, dtype=np.float32)
    dims, yshape = abi.conv_dims(x.shape, w.shape, stride, pad)
    dy = rng.standard_normal(yshape, dtype=np.float32)
    xr, wr, dyr = (O.round_to_bf16(a) for a in (x, w, dy))
    L = _lib.lib()
    xd, wd, dyd = (abi.to_bf16_device(a) for a in (x, w, dy))
    bd = DeviceTensor.from_numpy(b)
    y = DeviceTensor.full(yshape, np.nan)
    dx = DeviceTensor.full(x.shape, np.nan)
    dw = DeviceTensor.full(w.shape, np.nan)
    db = DeviceTensor.full(D, np.nan)
    _lib.check(L.aeth_conv_fprop_bf16(xd.ptr, wd.ptr, bd.ptr, y.ptr, *dims))
    _lib.check(L.aeth_conv_dgrad_bf16(dyd.ptr, wd.ptr, dx.ptr, *dims))
    _lib.check(L.aeth_conv_wgrad_bf16(xd.ptr, dyd.ptr, dw.ptr, db.ptr, *dims))
    y_h, dx_h, dw_h, db_h = y.get(), dx.get(), dw.get(), db.get()
    assert np.all(np.isfinite(y_h)) and np.all(np.isfinite(dx_h)) and np.all(np.isfinite(dw_h))

    label = LABEL[name] + ", bf16 inputs"
    abi.report(label, "fprop", whole_tensor_close(
        y_h, lambda lo, hi: O.conv_fprop(xr[lo:hi], wr, b, stride, pad, dtype=np.float64), S))
    abi.report(label, "dgrad", whole_tensor_close(
        dx_h, lambda lo, hi: O.conv_dgrad(dyr[lo:hi], wr, (H, W), stride, pad, dtype=np.float64), S))
    want = whole_batch_wgrad(xr, dyr, (fH, fW), stride, pad)
    abi.report(label, "wgrad", abi.close(dw_h, want, rms_scaled=True),
               "atol * max(1, rms), rms = %.3g" % float(np.sqrt(np.mean(want * want))))
    tune(**OTHER_KERNELS)
    y2 = DeviceTensor.full(yshape, np.nan)
    _lib.check(L.aeth_conv_fprop_bf16(xd.ptr, wd.ptr, bd.ptr, y2.ptr, *dims))
    assert np.array_equal(y_h, y2.get()), "fprop: the two kernels disagree"
    del y2
    dx2 = DeviceTensor.full(x.shape, np.nan)
    _lib.check(L.aeth_conv_dgrad_bf16(dyd.ptr, wd.ptr, dx2.ptr, *dims))
    assert np.array_equal(dx_h, dx2.get()), "dgrad: the two kernels disagree"
    del dx2
    tune(**{k: -1 for k in OTHER_KERNELS})

    lhs = float(np.sum((y_h.astype(np.float64) - b.astype(np.float64)) * dyr))
    rhs_x = float(np.sum(xr.astype(np.float64) * dx_h))
    rhs_w = float(np.sum(wr.astype(np.float64) * dw_h))
    scale = float(np.sqrt(np.sum(y_h.astype(np.float64) ** 2)) * np.sqrt(np.sum(dyr.astype(np.float64) ** 2)))
    assert abs(lhs - rhs_x) <= 1e-6 * scale, (lhs, rhs_x)
    assert abs(lhs - rhs_w) <= 1e-6 * scale, (lhs, rhs_w)
    abi.report(label, "dbias", abi.close(db_h, np.sum(dyr.astype(np.float64), axis=(0, 1, 2)), rms_scaled=True))

    # one-sample-supported gradient: wgrad of that sample alone
    s = S - 1
    dy1 = np.zeros_like(dy)
    dy1[s] = dy[s]
    dyd1 = abi.to_bf16_device(dy1)
    _lib.check(L.aeth_conv_wgrad_bf16(xd.ptr, dyd1.ptr, dw.ptr, db.ptr, *dims))
    want = O.conv_wgrad(xr[s:s + 1], dyr[s:s + 1], (fH, fW), stride, pad, dtype=np.float64)
    abi.close(dw.get(), want, rms_scaled=True)
