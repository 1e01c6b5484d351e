"""aeth_conv_fprop_f32_noalloc: the forward convolution for callers that cannot
allocate.  Its scratch (packed filter, split-K partial tiles) is a fixed array on the
GPU instead of the library's growing workspace; kernels, their order and therefore
the results are those of aeth_conv_fprop_f32, so the comparison is bit for bit
(the integer/byte bar: both entry points run the same float32 instruction stream).

Two calls in a row, the second with a smaller input: the array keeps the first call's
contents, and whatever the second call reads must have been written by the second
call.  Shapes that read the filter in place (only split-K partials in the array),
shapes that pack it, a packed filter with partials behind it, and the call recorded
into a HIP graph and replayed."""
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


PACKING = [
    # shapes whose filter is packed into the scratch (the default fprop reads w in place only for whole 64-wide n tiles
    # and at least three slabs of K): large first, smaller second
    [((8, 20, 20, 64), (3, 3, 64, 48), (1, 1), "same"), ((3, 9, 9, 64), (3, 3, 64, 40), (1, 1), "same")],     # D % 64 != 0
    [((16, 24, 24, 4), (3, 3, 4, 64), (1, 1), "same"), ((2, 10, 10, 4), (3, 3, 4, 64), (2, 2), "valid")],      # K = 36: two slabs
]


@pytest.mark.parametrize("pair", PACKING, ids=["ragged_n", "short_k"])
def test_noalloc_with_a_packed_filter_in_the_fixed_array(pair):
    from oracle import oracle as O
    from tests import abi
    rng = np.random.RandomState(13)
    for xs, ws, strides, padding in pair:
        x = rng.randn(*xs).astype(np.float32)
        w = (rng.randn(*ws) * np.sqrt(2.0 / np.prod(ws[:3]))).astype(np.float32)
        b = rng.randn(ws[3]).astype(np.float32)
        got = _run("aeth_conv_fprop_f32_noalloc", x, w, b, strides, padding)
        assert np.array_equal(got, _run("aeth_conv_fprop_f32", x, w, b, strides, padding)), xs
        abi.close(got, O.conv_fprop(x, w, b, strides, padding, dtype=np.float64))


def test_noalloc_with_a_packed_filter_and_split_k_partials_behind_it(tune):
    """`gather_bkn = 0` makes fprop pack every filter: the dense products below then hold the packed filter at the
    start of the array and their split-K partial tiles behind it (at the next multiple of 256 bytes).  Large first,
    smaller second; the capacity check sees the sum of the two."""
    from tests import abi
    tune(gather_bkn=0)
    rng = np.random.RandomState(14)
    for M, n_in, n_out in ((128, 2048, 256), (64, 1024, 120)):
        x = rng.randn(M, 1, 1, n_in).astype(np.float32)
        w = (rng.randn(1, 1, n_in, n_out) * 0.02).astype(np.float32)
        b = rng.randn(n_out).astype(np.float32)
        got = _run("aeth_conv_fprop_f32_noalloc", x, w, b, (1, 1), "valid")
        assert np.array_equal(got, _run("aeth_conv_fprop_f32", x, w, b, (1, 1), "valid"))
        ref = x.reshape(M, n_in).astype(np.float64) @ w.reshape(n_in, n_out).astype(np.float64) + b
        abi.close(got.reshape(M, n_out), ref)
    # a packing shape whose packed filter alone fits but not with its partials is refused, not truncated
    import ctypes as C
    from aether import _lib
    from aether.tensor import DeviceTensor
    lib = _lib.lib()
    xz, wz, yz = DeviceTensor.zeros((128, 1, 1, 8000)), DeviceTensor.zeros((1, 1, 8000, 256)), DeviceTensor.zeros((128, 1, 1, 256))
    rc = lib.aeth_conv_fprop_f32_noalloc(xz.ptr, wz.ptr, None, yz.ptr, 128, 1, 1, 8000, 256, 1, 1, 1, 1, 0, 0)
    assert rc == _lib.AETH_E_INVALID and b"scratch" in lib.aeth_last_error()   # 8000 x 256 floats pack to 7.8 MiB + partials


def test_noalloc_inside_a_recording():
    """The callers this entry point is for: code under HIP graph capture.  The call is recorded between
    aeth_graph_begin and aeth_graph_end (nothing runs, nothing is allocated), then replayed three times with new
    inputs copied into the buffers it reads and eager work in between; every replay equals the eager result."""
    import ctypes as C
    from aether import _lib
    from aether.tensor import DeviceTensor
    from tests import abi
    lib = _lib.lib()
    rng = np.random.RandomState(15)
    M, n_in, n_out = 128, 2048, 256                          # splits K: partial tiles in the fixed array
    w = (rng.randn(1, 1, n_in, n_out) * 0.02).astype(np.float32)
    b = rng.randn(n_out).astype(np.float32)
    dims = (M, 1, 1, n_in, n_out, 1, 1, 1, 1, 0, 0)
    xd, wd, bd = DeviceTensor.zeros((M, 1, 1, n_in)), DeviceTensor.from_numpy(w), DeviceTensor.from_numpy(b)
    y = DeviceTensor.full((M, 1, 1, n_out), np.nan)
    _lib.check(lib.aeth_graph_begin())
    rc = lib.aeth_conv_fprop_f32_noalloc(xd.ptr, wd.ptr, bd.ptr, y.ptr, *dims)
    handle = C.c_void_p()
    rc_end = lib.aeth_graph_end(C.byref(handle))
    _lib.check(rc)
    _lib.check(rc_end)
    assert np.all(np.isnan(y.get()))                         # recorded, not run
    try:
        for rep in range(3):
            x = rng.randn(M, 1, 1, n_in).astype(np.float32)
            xd.set(x)
            _lib.check(lib.aeth_graph_launch(handle))
            got = y.get()
            want = _run("aeth_conv_fprop_f32", x, w, b, (1, 1), "valid")   # eager work between the replays
            assert np.array_equal(got, want), rep
            other = rng.randn(4, 14, 14, 32).astype(np.float32)          # another user of the fixed array in between
            _run("aeth_conv_fprop_f32_noalloc", other, (rng.randn(3, 3, 32, 48) * 0.1).astype(np.float32), None, (1, 1), "same")
    finally:
        _lib.check(lib.aeth_graph_destroy(handle))


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
