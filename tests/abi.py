"""Thin helpers the GPU parity tests use to call the C ABI directly (through
ctypes) on NumPy inputs and get NumPy outputs back."""
import json
import os

import numpy as np

from aether import _lib
from aether.tensor import DeviceTensor
from oracle import oracle as O


def conv_dims(x_shape, w_shape, strides, padding):
    S, H, W, C = x_shape
    fH, fW, _, D = w_shape
    sH, sW = strides
    P, Ho, Wo = O.conv_geometry(H, W, fH, fW, sH, sW, padding)
    return (S, H, W, C, D, fH, fW, sH, sW, P, P), (S, Ho, Wo, D)


def fprop(x, w, b, strides, padding):
    dims, yshape = conv_dims(x.shape, w.shape, strides, padding)
    xd, wd = DeviceTensor.from_numpy(x, np.float32), DeviceTensor.from_numpy(w, np.float32)
    bd = DeviceTensor.from_numpy(b, np.float32) if b is not None else None
    y = DeviceTensor.full(yshape, np.nan)
    _lib.check(_lib.lib().aeth_conv_fprop_f32(xd.ptr, wd.ptr, bd.ptr if bd else None, y.ptr, *dims))
    return y.get()


def dgrad(dy, w, x_shape, strides, padding):
    dims, yshape = conv_dims(x_shape, w.shape, strides, padding)
    assert tuple(dy.shape) == yshape
    dyd, wd = DeviceTensor.from_numpy(dy, np.float32), DeviceTensor.from_numpy(w, np.float32)
    dx = DeviceTensor.full(x_shape, np.nan)
    _lib.check(_lib.lib().aeth_conv_dgrad_f32(dyd.ptr, wd.ptr, dx.ptr, *dims))
    return dx.get()


def wgrad(x, dy, w_shape, strides, padding, want_dbias=True):
    dims, yshape = conv_dims(x.shape, w_shape, strides, padding)
    assert tuple(dy.shape) == yshape
    xd, dyd = DeviceTensor.from_numpy(x, np.float32), DeviceTensor.from_numpy(dy, np.float32)
    dw = DeviceTensor.full(w_shape, np.nan)
    db = DeviceTensor.full(w_shape[3], np.nan) if want_dbias else None
    _lib.check(_lib.lib().aeth_conv_wgrad_f32(xd.ptr, dyd.ptr, dw.ptr, db.ptr if db else None, *dims))
    return dw.get(), (db.get() if db else None)


def close(got, want, rtol=1e-4, atol=1e-5, rms_scaled=False):
    """|got - want| <= atol + rtol*|want| elementwise; returns the worst ratio.

    ``rms_scaled`` multiplies atol by max(1, rms(want)).  It is used for the
    reductions over the whole batch (wgrad, dbias, dense dW): their outputs are
    sums of 10^4..10^6 products whose magnitude grows like sqrt(length), and an
    element that happens to cancel to ~0 cannot be reproduced to 1e-5 absolute by
    any float32 summation order (the reference's own float32 einsum misses the
    float64 value by more than that)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    if rms_scaled and want.size:
        atol = atol * max(1.0, float(np.sqrt(np.mean(want * want))))
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.all(np.isfinite(got)), "non-finite values (unwritten output?)"
    err = np.abs(got - want)
    tol = atol + rtol * np.abs(want)
    worst = float(np.max(err / tol)) if err.size else 0.0
    assert worst <= 1.0, "max err/tol = %.3g (max abs err %.3g)" % (worst, float(err.max()))
    return worst


# ---- bf16-input variants: inputs are cast on the device by aeth_cast_f32_to_bf16 ----
def to_bf16_device(a):
    src = DeviceTensor.from_numpy(a, np.float32)
    dst = DeviceTensor(a.shape, np.uint16)
    _lib.check(_lib.lib().aeth_cast_f32_to_bf16(src.ptr, dst.ptr, src.size))
    return dst


def fprop_bf16(x, w, b, strides, padding):
    dims, yshape = conv_dims(x.shape, w.shape, strides, padding)
    xd, wd = to_bf16_device(x), to_bf16_device(w)
    bd = DeviceTensor.from_numpy(b, np.float32) if b is not None else None
    y = DeviceTensor.full(yshape, np.nan)
    _lib.check(_lib.lib().aeth_conv_fprop_bf16(xd.ptr, wd.ptr, bd.ptr if bd else None, y.ptr, *dims))
    return y.get()


def dgrad_bf16(dy, w, x_shape, strides, padding):
    dims, yshape = conv_dims(x_shape, w.shape, strides, padding)
    dyd, wd = to_bf16_device(dy), to_bf16_device(w)
    dx = DeviceTensor.full(x_shape, np.nan)
    _lib.check(_lib.lib().aeth_conv_dgrad_bf16(dyd.ptr, wd.ptr, dx.ptr, *dims))
    return dx.get()


def wgrad_bf16(x, dy, w_shape, strides, padding):
    dims, yshape = conv_dims(x.shape, w_shape, strides, padding)
    xd, dyd = to_bf16_device(x), to_bf16_device(dy)
    dw = DeviceTensor.full(w_shape, np.nan)
    db = DeviceTensor.full(w_shape[3], np.nan)
    _lib.check(_lib.lib().aeth_conv_wgrad_bf16(xd.ptr, dyd.ptr, dw.ptr, db.ptr, *dims))
    return dw.get(), db.get()


# ---- the benchmark's input recipe and the parity figures quoted beside its timings ----
def baseline_inputs(kind, x_shape, num_filters, filter_size=(3, 3), strides=(1, 1), padding="same"):
    """Inputs of one benchmark configuration, drawn the way the benchmark draws them: the legacy global RNG
    seeded with 0, then in this order the input (`kind`: "rand" = U[0,1), "randn" = N(0,1), "relu_randn" =
    N(0,1) clipped at 0), the layer (its constructor draws the He-normal filter, CNN_classes_cupy.py:61-66; zero
    bias) and the upstream gradient N(0,1).  Returns x, w, b, dy as float32 host arrays."""
    import aether
    np.random.seed(0)
    if kind == "rand":
        x = np.random.rand(*x_shape).astype(np.float32)
    else:
        x = np.random.randn(*x_shape).astype(np.float32)
        if kind == "relu_randn":
            x = np.maximum(x, 0)
    layer = aether.Conv_Layer(x_shape[1:], num_filters=num_filters, filter_size=filter_size, strides=strides,
                              padding=padding)
    w, b = layer.filter_weights.get(), layer.biases.get()
    _, yshape = conv_dims(x.shape, w.shape, strides, padding)
    dy = np.random.randn(*yshape).astype(np.float32)
    return x, w, b, dy


def report(config, direction, worst, note=""):
    """Appends one measured max err/tol to the file $AETHER_PARITY_REPORT names (JSON lines), if it names one:
    the source of the parity table that stands beside the benchmark's timings."""
    path = os.environ.get("AETHER_PARITY_REPORT")
    if path:
        with open(path, "a") as f:
            f.write(json.dumps({"config": config, "direction": direction, "max_err_over_tol": worst,
                                "note": note}) + "\n")
