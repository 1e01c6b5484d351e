"""aeth_conv_fprop_f32_noalloc: the forward convolution for callers that cannot
allocate.  Its scratch (packed filter, split-K partial tiles) is a fixed array on the
GPU instead of the library's growing workspace; kernels, their order and therefore
the results are those of aeth_conv_fprop_f32, so the comparison is bit for bit
(the integer/byte bar: both entry points run the same float32 instruction stream).

Two calls in a row, the second with a smaller input: the array keeps the first call's
contents, and whatever the second call reads must have been written by the second
call."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(entry, x, w, b, strides, padding):
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    dims, yshape = abi.conv_dims(x.shape, w.shape, strides, padding)
    xd, wd = DeviceTensor.from_numpy(x, np.float32), DeviceTensor.from_numpy(w, np.float32)
    bd = DeviceTensor.from_numpy(b, np.float32) if b is not None else None
    y = DeviceTensor.full(yshape, np.nan)
    _lib.check(getattr(_lib.lib(), entry)(xd.ptr, wd.ptr, bd.ptr if bd else None, y.ptr, *dims))
    return y.get()


CASES = [
    # (x shape, filter shape, strides, padding): large first, smaller second
    ((16, 28, 28, 64), (3, 3, 64, 128), (1, 1), "same"),
    ((4, 14, 14, 32), (3, 3, 32, 64), (2, 2), "valid"),
]


def test_noalloc_equals_the_allocating_entry_point_on_two_calls_in_a_row():
    from oracle import oracle as O
    from tests import abi
    rng = np.random.RandomState(11)
    for xs, ws, strides, padding in CASES:
        x = rng.randn(*xs).astype(np.float32)
        w = (rng.randn(*ws) * np.sqrt(2.0 / np.prod(ws[:3]))).astype(np.float32)
        b = rng.randn(ws[3]).astype(np.float32)
        got = _run("aeth_conv_fprop_f32_noalloc", x, w, b, strides, padding)
        want = _run("aeth_conv_fprop_f32", x, w, b, strides, padding)
        assert np.array_equal(got, want), "no-alloc result differs from aeth_conv_fprop_f32 for %r" % (xs,)
        abi.close(got, O.conv_fprop(x, w, b, strides, padding, dtype=np.float64))


def test_noalloc_split_k_partials_live_in_the_fixed_array():
    """A dense product with few tiles and long K is split over K: the partial tiles sit
    behind the packed filter in the scratch.  Large first, smaller second."""
    rng = np.random.RandomState(12)
    for M, n_in, n_out in ((128, 2048, 256), (64, 1024, 128)):
        x = rng.randn(M, 1, 1, n_in).astype(np.float32)
        w = (rng.randn(1, 1, n_in, n_out) * 0.02).astype(np.float32)
        b = rng.randn(n_out).astype(np.float32)
        got = _run("aeth_conv_fprop_f32_noalloc", x, w, b, (1, 1), "valid")
        want = _run("aeth_conv_fprop_f32", x, w, b, (1, 1), "valid")
        assert np.array_equal(got, want)
        ref = x.reshape(M, n_in).astype(np.float64) @ w.reshape(n_in, n_out).astype(np.float64) + b
        from tests import abi
        abi.close(got.reshape(M, n_out), ref)


def test_noalloc_rejects_filters_beyond_its_scratch():
    import ctypes as C
    from aether import _lib
    from aether.tensor import DeviceTensor
    lib = _lib.lib()
    # 3x3x512x1024 floats pack to 18 MiB: more than the 8 MiB array
    x = DeviceTensor.zeros((1, 4, 4, 512))
    w = DeviceTensor.zeros((3, 3, 512, 1024))
    y = DeviceTensor.zeros((1, 4, 4, 1024))
    rc = lib.aeth_conv_fprop_f32_noalloc(x.ptr, w.ptr, None, y.ptr, 1, 4, 4, 512, 1024, 3, 3, 1, 1, 1, 1)
    assert rc == _lib.AETH_E_INVALID
    assert b"scratch" in lib.aeth_last_error()
    # the allocating entry point takes the same shape
    _lib.check(lib.aeth_conv_fprop_f32(x.ptr, w.ptr, None, y.ptr, 1, 4, 4, 512, 1024, 3, 3, 1, 1, 1, 1))
    assert np.all(y.get() == 0)
