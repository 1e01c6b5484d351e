"""The binding a maintainer of the reference would write, run end to end: classes shaped like the reference's
`Conv_Layer` (CNN_classes_cupy.py:37-161) and `Layer_Dense` (:315-362) that keep their own arrays and call
libaether_hip.so through nothing but ctypes.  No `aether` class is involved: buffers come from aeth_malloc,
results are read with aeth_memcpy_d2h, and forward / backward make one library call per product in place of
the reference's pad + as_strided + einsum lines.  Checked against the CPU oracle at the float32 bar."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

_p, _i, _i64 = C.c_void_p, C.c_int, C.c_int64


def _bind():
    from aether._lib import LIB_PATH                        # only the path of the built library
    lib = C.CDLL(LIB_PATH)
    lib.aeth_last_error.restype = C.c_char_p
    lib.aeth_malloc.argtypes = [C.POINTER(_p), _i64]
    lib.aeth_free.argtypes = [_p]
    lib.aeth_memcpy_h2d.argtypes = [_p, _p, _i64]
    lib.aeth_memcpy_d2h.argtypes = [_p, _p, _i64]
    lib.aeth_conv_fprop_f32.argtypes = [_p, _p, _p, _p] + [_i] * 11
    lib.aeth_conv_dgrad_f32.argtypes = [_p, _p, _p] + [_i] * 11
    lib.aeth_conv_wgrad_f32.argtypes = [_p, _p, _p, _p] + [_i] * 11
    lib.aeth_dense_fprop_f32.argtypes = [_p, _p, _p, _p, _i, _i, _i]
    lib.aeth_dense_dgrad_f32.argtypes = [_p, _p, _p, _i, _i, _i]
    lib.aeth_dense_wgrad_f32.argtypes = [_p, _p, _p, _p, _i, _i, _i]
    lib.aeth_axpy_f32.argtypes = [C.c_float, _p, _p, _i64]

    def ck(rc):
        if rc:
            raise (ValueError if rc == -1 else RuntimeError)(lib.aeth_last_error().decode())

    ck(lib.aeth_init(0))
    return lib, ck


class _Array:
    """What a CuPy array is to the reference: a shape and a device pointer (here from aeth_malloc)."""

    def __init__(self, lib, ck, shape, host=None):
        self.lib, self.ck, self.shape = lib, ck, tuple(shape)
        self.nbytes = 4 * int(np.prod(self.shape))
        p = _p()
        ck(lib.aeth_malloc(C.byref(p), self.nbytes))
        self.ptr = p.value
        if host is not None:
            host = np.ascontiguousarray(host, dtype=np.float32)
            ck(lib.aeth_memcpy_h2d(self.ptr, host.ctypes.data, self.nbytes))

    def get(self):
        out = np.empty(self.shape, np.float32)
        self.ck(self.lib.aeth_memcpy_d2h(out.ctypes.data, self.ptr, self.nbytes))    # synchronises
        return out

    def __del__(self):
        try:
            self.lib.aeth_free(self.ptr)
        except Exception:
            pass


def _classes(lib, ck):
    def empty(shape):
        return _Array(lib, ck, shape)

    class Conv_Layer:
        def __init__(self, input_shape, num_filters=1, filter_size=(3, 3), strides=(1, 1), padding="same"):
            self.num_filters, self.filter_size, self.strides, self.padding = num_filters, filter_size, strides, padding
            n = filter_size[0] * filter_size[1] * input_shape[-1]
            w = np.random.randn(filter_size[0], filter_size[1], input_shape[-1], num_filters).astype(np.float32)
            self.filter_weights = _Array(lib, ck, w.shape, w * np.sqrt(np.float32(2.0 / n)))
            self.weights = self.filter_weights
            self.biases = _Array(lib, ck, (num_filters,), np.zeros(num_filters))

        def forward(self, inputs, training):
            S, H, W, Cin = inputs.shape
            fH, fW = self.filter_size
            sH, sW = self.strides
            P = (fH - 1) // 2 if self.padding == "same" else 0
            Ho, Wo = (H + 2 * P - fH) // sH + 1, (W + 2 * P - fW) // sW + 1
            self.output = empty((S, Ho, Wo, self.num_filters))
            self._dims = (S, H, W, Cin, self.num_filters, fH, fW, sH, sW, P, P)
            ck(lib.aeth_conv_fprop_f32(inputs.ptr, self.filter_weights.ptr, self.biases.ptr, self.output.ptr, *self._dims))
            self.inputs = inputs
            return self.output

        def backward(self, dvalues):
            self.dweights, self.dbiases = empty(self.filter_weights.shape), empty(self.biases.shape)
            self.dinputs = empty(self.inputs.shape)
            ck(lib.aeth_conv_wgrad_f32(self.inputs.ptr, dvalues.ptr, self.dweights.ptr, self.dbiases.ptr, *self._dims))
            ck(lib.aeth_conv_dgrad_f32(dvalues.ptr, self.filter_weights.ptr, self.dinputs.ptr, *self._dims))
            return self.dinputs

    class Layer_Dense:
        def __init__(self, n_inputs, n_neurons, weight_regularizer_l2=0):
            w = .01 * np.random.randn(n_inputs, n_neurons) * np.sqrt(2.0 / n_inputs)
            self.weights = _Array(lib, ck, w.shape, w)
            self.biases = _Array(lib, ck, (1, n_neurons), np.zeros((1, n_neurons)))
            self.weight_regularizer_l2 = weight_regularizer_l2

        def forward(self, inputs, training):
            self.inputs = inputs
            M, (n_in, n_out) = inputs.shape[0], self.weights.shape
            self.output = empty((M, n_out))
            ck(lib.aeth_dense_fprop_f32(inputs.ptr, self.weights.ptr, self.biases.ptr, self.output.ptr, M, n_in, n_out))

        def backward(self, dvalues):
            M, (n_in, n_out) = self.inputs.shape[0], self.weights.shape
            self.dweights, self.dbiases, self.dinputs = empty(self.weights.shape), empty((1, n_out)), empty(self.inputs.shape)
            ck(lib.aeth_dense_wgrad_f32(self.inputs.ptr, dvalues.ptr, self.dweights.ptr, self.dbiases.ptr, M, n_in, n_out))
            if self.weight_regularizer_l2 > 0:
                ck(lib.aeth_axpy_f32(2 * self.weight_regularizer_l2, self.weights.ptr, self.dweights.ptr, n_in * n_out))
            ck(lib.aeth_dense_dgrad_f32(dvalues.ptr, self.weights.ptr, self.dinputs.ptr, M, n_in, n_out))

    return Conv_Layer, Layer_Dense


def test_reference_shaped_classes_over_raw_ctypes():
    from tests import abi
    lib, ck = _bind()
    Conv_Layer, Layer_Dense = _classes(lib, ck)
    np.random.seed(0)
    # conv (stride 2, "same") -> flatten (a reshape of the same buffer) -> dense with an L2 term
    x = np.random.randn(6, 12, 12, 8).astype(np.float32)
    conv = Conv_Layer((12, 12, 8), num_filters=16, filter_size=(3, 3), strides=(2, 2), padding="same")
    dense = Layer_Dense(6 * 6 * 16, 10, weight_regularizer_l2=1e-3)
    dlogits = np.random.randn(6, 10).astype(np.float32)
    w, b = conv.filter_weights.get(), conv.biases.get()
    wd, bd = dense.weights.get(), dense.biases.get()

    conv.forward(_Array(lib, ck, x.shape, x), True)
    assert conv.output.shape == (6, 6, 6, 16)
    flat = conv.output
    flat.shape = (6, 6 * 6 * 16)                              # Flatten: the same memory, another shape
    dense.forward(flat, True)
    dense.backward(_Array(lib, ck, dlogits.shape, dlogits))
    back = dense.dinputs
    back.shape = (6, 6, 6, 16)
    conv.backward(back)

    y64 = O.conv_fprop(x, w, b, (2, 2), "same", dtype=np.float64)
    flat.shape = (6, 6, 6, 16)
    abi.close(flat.get(), y64)
    abi.close(dense.output.get(), O.dense_forward(y64.reshape(6, -1), wd, bd, dtype=np.float64))
    dw, db, dx = O.dense_backward(y64.reshape(6, -1), wd, bd, dlogits, wl2=1e-3, dtype=np.float64)
    abi.close(dense.dweights.get(), dw, rms_scaled=True)
    abi.close(dense.dbiases.get(), db, rms_scaled=True)
    abi.close(dense.dinputs.get().reshape(6, -1), dx)
    dy64 = dx.reshape(6, 6, 6, 16)
    abi.close(conv.dinputs.get(), O.conv_dgrad(dy64, w, (12, 12), (2, 2), "same", dtype=np.float64))
    abi.close(conv.dweights.get(), O.conv_wgrad(x, dy64, (3, 3), (2, 2), "same", dtype=np.float64), rms_scaled=True)
    abi.close(conv.dbiases.get(), O.conv_dbias(dy64, dtype=np.float64), rms_scaled=True)
    with pytest.raises(ValueError):                           # error behaviour of the boundary: a code and a message
        ck(lib.aeth_conv_fprop_f32(None, conv.filter_weights.ptr, None, conv.output.ptr, *conv._dims))
