"""ctypes binding of libaether_hip.so (the C ABI declared in include/aether_hip.h).

The library is looked up in ``aether/lib/`` (or at ``$AETHER_HIP_LIB``).  There is
no fallback of any kind: if the library is missing, or the GPU is not a gfx950,
every entry point raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("AETHER_HIP_LIB", os.path.join(_HERE, "lib", "libaether_hip.so"))

_i, _f, _p, _i64, _d = C.c_int, C.c_float, C.c_void_p, C.c_int64, C.c_double
_conv_dims = [_i] * 11

# name -> argument types (all return int)
SIGNATURES = {
    "aeth_init": [_i],
    "aeth_shutdown": [],
    "aeth_device_info": [C.c_char_p, _i],
    "aeth_debug_set": [C.c_char_p, _i],
    "aeth_malloc": [C.POINTER(_p), _i64],
    "aeth_free": [_p],
    "aeth_memcpy_h2d": [_p, _p, _i64],
    "aeth_memcpy_d2h": [_p, _p, _i64],
    "aeth_memcpy_d2d": [_p, _p, _i64],
    "aeth_d2h_begin": [_p, _i64, C.POINTER(_i)],
    "aeth_d2h_end": [_i, _p, _i64],
    "aeth_fill_f32": [_p, _f, _i64],
    "aeth_sync": [],
    "aeth_event_create": [C.POINTER(_p)],
    "aeth_event_destroy": [_p],
    "aeth_event_record": [_p],
    "aeth_event_elapsed_ms": [_p, _p, C.POINTER(_f)],
    "aeth_conv_fprop_f32": [_p, _p, _p, _p] + _conv_dims,
    "aeth_conv_fprop_f32_noalloc": [_p, _p, _p, _p] + _conv_dims,
    "aeth_conv_dgrad_f32": [_p, _p, _p] + _conv_dims,
    "aeth_conv_bwd_f32": [_p, _p, _p, _p, _p, _p] + _conv_dims,
    "aeth_conv_wgrad_f32": [_p, _p, _p, _p] + _conv_dims,
    "aeth_cast_f32_to_bf16": [_p, _p, _i64],
    "aeth_conv_fprop_bf16": [_p, _p, _p, _p] + _conv_dims,
    "aeth_conv_dgrad_bf16": [_p, _p, _p] + _conv_dims,
    "aeth_conv_wgrad_bf16": [_p, _p, _p, _p] + _conv_dims,
    "aeth_dense_fprop_f32": [_p, _p, _p, _p, _i, _i, _i],
    "aeth_dense_dgrad_f32": [_p, _p, _p, _i, _i, _i],
    "aeth_dense_wgrad_f32": [_p, _p, _p, _p, _i, _i, _i],
    "aeth_dense_fprop_act_f32": [_p, _p, _p, _p, _p, _f, _i, _i, _i],
    "aeth_dense_bwd_f32": [_p, _p, _p, _p, _p, _p, _p, _p, _f, _i, _i, _i],
    "aeth_axpy_f32": [_f, _p, _p, _i64],
    "aeth_l1_grad_f32": [_f, _p, _p, _i64],
    "aeth_reduce_f32": [_p, _i64, _i, _p],
    "aeth_bn_fwd_train_f32": [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i, _f, _f],
    "aeth_bn_fwd_infer_f32": [_p, _p, _p, _p, _p, _p, _i, _i, _f],
    "aeth_bn_bwd_f32": [_p, _p, _p, _p, _p, _p, _p, _p, _i, _i],
    "aeth_relu_fwd_f32": [_p, _p, _f, _i64],
    "aeth_relu_bwd_f32": [_p, _p, _p, _f, _i64],
    "aeth_relu_fwd_twin_f32": [_p, _p, _p, _f, _i64],
    "aeth_bn_bwd_twin_f32": [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i, _i],
    "aeth_maxpool_fwd_f32": [_p, _p, _p] + [_i] * 8,
    "aeth_bn_relu_maxpool2_fwd_f32": [_p] * 11 + [_i] * 4 + [_f, _f, _f],
    "aeth_bn_relu_maxpool2_fwd_twin_f32": [_p] * 12 + [_i] * 4 + [_f, _f, _f],
    "aeth_maxpool2_relu_bwd_f32": [_p] * 5 + [_i] * 4 + [_f],
    "aeth_maxpool2_relu_bn_bwd_f32": [_p] * 12 + [_i] * 4 + [_f],
    "aeth_maxpool2_relu_bn_bwd_twin_f32": [_p] * 13 + [_i] * 4 + [_f],
    "aeth_maxpool_bwd_f32": [_p, _p, _p] + [_i] * 8,
    "aeth_avgpool_fwd_f32": [_p, _p] + [_i] * 8,
    "aeth_avgpool_bwd_f32": [_p, _p] + [_i] * 8,
    "aeth_mul_mask_f32": [_p, _p, _p, _i64, _i64],
    "aeth_softmax_f32": [_p, _p, _i, _i],
    "aeth_softmax_bwd_f32": [_p, _p, _p, _i, _i],
    "aeth_cce_fwd_f32": [_p, _p, _f, _p, _p, _i, _i],
    "aeth_softmax_cce_bwd_f32": [_p, _p, _f, _p, _i, _i],
    "aeth_softmax_cce_train_f32": [_p, _p, _f, _p, _p, _p, _p, _i, _i],
    "aeth_cce_fwd_dense_f32": [_p, _p, _f, _p, _p, _i, _i],
    "aeth_softmax_cce_bwd_dense_f32": [_p, _p, _f, _p, _i, _i],
    "aeth_softmax_cce_train_dense_f32": [_p, _p, _f, _p, _p, _p, _p, _i, _i],
    "aeth_adam_f32": [_p, _p, _p, _p, _i64, _f, _f, _f, _f, _i],
    "aeth_adam_multi_f32": [_i, _p, _p, _p, _p, _p, _f, _f, _f, _f, _i],
    "aeth_adam_state_step": [_p, _d, _d, _d, _d],
    "aeth_adam_multi_dev_f32": [_i, _p, _p, _p, _p, _p, _f, _f, _f, _p],
    "aeth_graph_begin": [],
    "aeth_graph_end": [C.POINTER(_p)],
    "aeth_graph_launch": [_p],
    "aeth_graph_destroy": [_p],
}

AETH_E_INVALID = -1
AETH_E_HIP = -2
AETH_E_NOMEM = -3
AETH_E_STATE = -4

_lib = None
_initialised = False


def load():
    """dlopen the library and attach argument types; no GPU call is made."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libaether_hip.so not found at %s -- build it with `python aether-ml_amd/build.py`" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the symbol is missing
        fn.argtypes = args
        fn.restype = _i
    lib.aeth_last_error.argtypes = []
    lib.aeth_last_error.restype = C.c_char_p
    _lib = lib
    return lib


def check(rc):
    """Translate a status code into the exception the reference would raise:
    ValueError for bad shapes / arguments, RuntimeError (MemoryError) otherwise."""
    if rc == 0:
        return
    msg = load().aeth_last_error().decode("utf-8", "replace")
    if rc == AETH_E_INVALID:
        raise ValueError(msg)
    if rc == AETH_E_NOMEM:
        raise MemoryError(msg)
    raise RuntimeError("libaether_hip error %d: %s" % (rc, msg))


def lib():
    """The loaded library with the context bound to GPU ``$AETHER_DEVICE`` (default 0)."""
    global _initialised
    L = load()
    if not _initialised:
        check(L.aeth_init(int(os.environ.get("AETHER_DEVICE", "0"))))
        _initialised = True
    return L


def debug_set(name=None, value=-1):
    """Kernel-choice override for tests and measurements (aeth_debug_set); no name resets all."""
    check(load().aeth_debug_set(name.encode() if name is not None else None, int(value)))


def device_info():
    buf = C.create_string_buffer(512)
    check(lib().aeth_device_info(buf, 512))
    out = {}
    for kv in buf.value.decode().split(";"):
        k, _, v = kv.partition("=")
        out[k] = int(v) if v.lstrip("-").isdigit() else v
    return out


def sync():
    check(lib().aeth_sync())


class Event:
    """HIP event recorded on the library's stream."""

    def __init__(self):
        self._h = _p()
        check(lib().aeth_event_create(C.byref(self._h)))

    def record(self):
        check(lib().aeth_event_record(self._h))
        return self

    def elapsed_ms(self, stop):
        ms = _f()
        check(lib().aeth_event_elapsed_ms(self._h, stop._h, C.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            if self._h and _lib is not None:
                _lib.aeth_event_destroy(self._h)
        except Exception:
            pass
