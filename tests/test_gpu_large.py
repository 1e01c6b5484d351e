"""Tensors of 2^31 bytes and more.  The fast kernels address their operands with 32-bit byte offsets, so the
library cuts such a batch into runs of whole samples (aether-ml_amd/csrc/sample_runs.h; the arithmetic is checked
on the host by tests/cpu/sample_runs_check.cpp).  Here: NHWC [1536,56,56,128] -> 64 filters 3x3 "same", an input of
2.47 GB, float32.  The first and last sample and the two either side of the cut against the float64 oracle; every
element bit for bit against the same data handed in as three calls of 512 samples; the float64 adjoint identities
<y - b, dy> = <x, dx> = <W, dW> on the whole tensors; dbias against the column sum."""
import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

S, H, W, C, D = 1536, 56, 56, 128, 64


def _dot64(a, b, chunk=32):
    """<a, b> in float64 without a float64 copy of the whole tensors."""
    total = 0.0
    for lo in range(0, a.shape[0], chunk):
        total += float(np.vdot(a[lo:lo + chunk].astype(np.float64), b[lo:lo + chunk].astype(np.float64)))
    return total


def test_batch_beyond_two_gib():
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    rng = np.random.default_rng(5)
    x = rng.standard_normal((S, H, W, C), dtype=np.float32)
    assert x.nbytes > 2.4e9
    w = rng.standard_normal((3, 3, C, D), dtype=np.float32) * np.float32(np.sqrt(2.0 / (9 * C)))
    b = rng.standard_normal(D, dtype=np.float32)
    dy = rng.standard_normal((S, H, W, D), dtype=np.float32)
    dims, yshape = abi.conv_dims(x.shape, w.shape, (1, 1), "same")
    L = _lib.lib()
    xd, wd, bd, dyd = (DeviceTensor.from_numpy(a) for a in (x, w, b, dy))
    y, dx = DeviceTensor.full(yshape, np.nan), DeviceTensor.full(x.shape, np.nan)
    dw, db = DeviceTensor.full(w.shape, np.nan), DeviceTensor.full(D, np.nan)
    _lib.check(L.aeth_conv_fprop_f32(xd.ptr, wd.ptr, bd.ptr, y.ptr, *dims))
    _lib.check(L.aeth_conv_dgrad_f32(dyd.ptr, wd.ptr, dx.ptr, *dims))
    _lib.check(L.aeth_conv_wgrad_f32(xd.ptr, dyd.ptr, dw.ptr, db.ptr, *dims))
    y_h, dx_h, dw_h, db_h = y.get(), dx.get(), dw.get(), db.get()
    assert np.all(np.isfinite(y_h)) and np.all(np.isfinite(dx_h)) and np.all(np.isfinite(dw_h))

    # samples at the ends and either side of the cut (two runs of 768) against the oracle
    for s in (0, 767, 768, S - 1):
        abi.close(y_h[s:s + 1], O.conv_fprop(x[s:s + 1], w, b, (1, 1), "same", dtype=np.float64))
        abi.close(dx_h[s:s + 1], O.conv_dgrad(dy[s:s + 1], w, (H, W), (1, 1), "same", dtype=np.float64))

    # the same data as three calls of 512 samples, each far below 2 GiB: the same bits everywhere
    part = 512
    dims3 = (part,) + dims[1:]
    y3, dx3 = DeviceTensor.full(yshape, np.nan), DeviceTensor.full(x.shape, np.nan)
    dw3 = np.zeros(w.shape, np.float64)
    db3 = np.zeros(D, np.float64)
    dwp, dbp = DeviceTensor.full(w.shape, np.nan), DeviceTensor.full(D, np.nan)
    xs, ys = H * W * C * 4, H * W * D * 4
    for k in range(S // part):
        _lib.check(L.aeth_conv_fprop_f32(xd.ptr + k * part * xs, wd.ptr, bd.ptr, y3.ptr + k * part * ys, *dims3))
        _lib.check(L.aeth_conv_dgrad_f32(dyd.ptr + k * part * ys, wd.ptr, dx3.ptr + k * part * xs, *dims3))
        _lib.check(L.aeth_conv_wgrad_f32(xd.ptr + k * part * xs, dyd.ptr + k * part * ys, dwp.ptr, dbp.ptr, *dims3))
        dw3 += dwp.get()
        db3 += dbp.get()
    assert np.array_equal(y_h, y3.get()), "fprop differs from the three smaller calls"
    del y3
    assert np.array_equal(dx_h, dx3.get()), "dgrad differs from the three smaller calls"
    del dx3
    abi.close(dw_h, dw3, rms_scaled=True)
    abi.close(db_h, db3, rms_scaled=True)

    # adjoint identities in float64 on the whole tensors
    lhs = _dot64(y_h, dy) - float(np.dot(b.astype(np.float64), db3))       # <y - b, dy>, with sum dy from the three calls' dbias
    rhs_x = _dot64(x, dx_h)
    rhs_w = float(np.vdot(w.astype(np.float64), dw_h.astype(np.float64)))
    scale = float(np.sqrt(_dot64(y_h, y_h)) * np.sqrt(_dot64(dy, dy)))
    assert abs(lhs - rhs_x) <= 1e-6 * scale, (lhs, rhs_x)
    assert abs(lhs - rhs_w) <= 1e-6 * scale, (lhs, rhs_w)

    # throughput above and below the cut (HIP events, 5 launches each)
    fl = 2.0 * H * W * 9 * C * D
    for batch in (1536, 1280):                               # 2.47 GB (two runs) and 2.06 GB (one launch)
        d = (batch,) + dims[1:]
        for name, call in (("fprop", lambda: L.aeth_conv_fprop_f32(xd.ptr, wd.ptr, bd.ptr, y.ptr, *d)),
                           ("dgrad", lambda: L.aeth_conv_dgrad_f32(dyd.ptr, wd.ptr, dx.ptr, *d)),
                           ("wgrad", lambda: L.aeth_conv_wgrad_f32(xd.ptr, dyd.ptr, dw.ptr, db.ptr, *d))):
            _lib.check(call())
            e0, e1 = _lib.Event(), _lib.Event()
            e0.record()
            for _ in range(5):
                _lib.check(call())
            e1.record()
            ms = e0.elapsed_ms(e1) / 5
            abi.report("[%d,56,56,128] -> 64, 3x3 (%.2f GB input)" % (batch, batch * xs / 1e9), name,
                       fl * batch / (ms * 1e-3) / 1e12, "TFLOP/s, %.3f ms" % ms)
