"""DeviceTensor: a dense C-contiguous array living in MI355X HBM, owned through
aeth_malloc / aeth_free.  It plays the role the CuPy ndarray plays in the
reference (CNN/models/CNN_classes_cupy.py): layers keep activations and
parameters in it between forward and backward, and ``np.asarray(t)`` / ``t.get()``
bring a copy to the host."""
import ctypes as C

import numpy as np

from . import _lib


class DeviceTensor:
    __slots__ = ("ptr", "shape", "dtype", "_base", "_cache", "_bf16", "_version", "__weakref__")

    def __init__(self, shape, dtype=np.float32, _ptr=None, _base=None):
        if isinstance(shape, (int, np.integer)):
            shape = (int(shape),)
        self.shape = tuple(int(s) for s in shape)
        self.dtype = np.dtype(dtype)
        self._base = _base
        self._cache = None      # host-side values derived from this tensor by a kernel (e.g. row argmax)
        self._bf16 = None       # a bfloat16 copy of the contents left by the kernel that wrote them, if any
        self._version = 0       # bumped by everything that rewrites the contents in place
        if _ptr is None:
            p = C.c_void_p()
            _lib.check(_lib.lib().aeth_malloc(C.byref(p), self.nbytes))
            self.ptr = p.value
        else:
            self.ptr = _ptr

    # -- construction ---------------------------------------------------------------
    @classmethod
    def from_numpy(cls, a, dtype=None):
        a = np.ascontiguousarray(a, dtype=dtype if dtype is not None else None)
        t = cls(a.shape, a.dtype)
        if a.nbytes:
            _lib.check(_lib.lib().aeth_memcpy_h2d(t.ptr, a.ctypes.data, a.nbytes))
        return t

    @classmethod
    def zeros(cls, shape, dtype=np.float32):
        t = cls(shape, dtype)
        t.fill(0)
        return t

    @classmethod
    def full(cls, shape, value, dtype=np.float32):
        t = cls(shape, dtype)
        t.fill(value)
        return t

    # -- properties -------------------------------------------------------------------
    @property
    def size(self):
        n = 1
        for s in self.shape:
            n *= s
        return n

    @property
    def nbytes(self):
        return self.size * self.dtype.itemsize

    @property
    def ndim(self):
        return len(self.shape)

    def __len__(self):
        return self.shape[0]

    def __getitem__(self, rows):
        """A run of consecutive rows (a slice of the first axis with step 1) as a view of the same memory:
        what batching a data set that lives on the device needs (`X[start:start + batch_size]`)."""
        if not isinstance(rows, slice) or self.ndim == 0:
            raise TypeError("DeviceTensor supports slices of its first axis only")
        start, stop, step = rows.indices(self.shape[0])
        if step != 1:
            raise ValueError("DeviceTensor slices must have step 1")
        n = max(0, stop - start)
        row_bytes = (self.nbytes // self.shape[0]) if self.shape[0] else 0
        return DeviceTensor((n,) + self.shape[1:], self.dtype, _ptr=self.ptr + start * row_bytes,
                            _base=self._base if self._base is not None else self)

    # -- host transfer ------------------------------------------------------------------
    def get(self):
        out = np.empty(self.shape, dtype=self.dtype)
        if out.nbytes:
            _lib.check(_lib.lib().aeth_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes))
        return out

    numpy = get

    def get_later(self):
        """Queues the copy to the host behind what is queued so far and returns at once; calling the result
        waits for that copy alone and gives the array (at most 256 KB; for a loop that reads one step's
        scalars while the next step already runs).  Every result must be called once."""
        if self.nbytes == 0 or self.nbytes > 256 * 1024:
            value = self.get()
            return lambda: value
        ticket = C.c_int(-1)
        _lib.check(_lib.lib().aeth_d2h_begin(self.ptr, self.nbytes, C.byref(ticket)))
        shape, dtype, nbytes = self.shape, self.dtype, self.nbytes

        def result():
            out = np.empty(shape, dtype=dtype)
            _lib.check(_lib.lib().aeth_d2h_end(ticket.value, out.ctypes.data, nbytes))
            return out
        return result

    def __array__(self, dtype=None, copy=None):
        a = self.get()
        return a if dtype is None else a.astype(dtype, copy=False)

    def set(self, a):
        a = np.ascontiguousarray(a, dtype=self.dtype)
        if a.shape != self.shape:
            if a.size != self.size:
                raise ValueError("cannot set shape %s from %s" % (self.shape, a.shape))
            a = a.reshape(self.shape)
        if a.nbytes:
            _lib.check(_lib.lib().aeth_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes))
        self.touched()
        return self

    def touched(self):
        """The contents were rewritten in place: copies derived from them are stale."""
        self._version += 1
        self._bf16 = None
        self._cache = None

    # -- device ops -----------------------------------------------------------------------
    def fill(self, value):
        if self.size == 0:
            return self
        if self.dtype == np.float32:
            _lib.check(_lib.lib().aeth_fill_f32(self.ptr, float(value), self.size))
            self.touched()
        else:
            self.set(np.full(self.shape, value, dtype=self.dtype))
        return self

    def copy(self):
        t = DeviceTensor(self.shape, self.dtype)
        if self.nbytes:
            _lib.check(_lib.lib().aeth_memcpy_d2d(t.ptr, self.ptr, self.nbytes))
        return t

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        shape = list(int(s) for s in shape)
        if -1 in shape:
            known = 1
            for s in shape:
                if s != -1:
                    known *= s
            shape[shape.index(-1)] = self.size // known if known else 0
        n = 1
        for s in shape:
            n *= s
        if n != self.size:
            raise ValueError("cannot reshape %s into %s" % (self.shape, tuple(shape)))
        return DeviceTensor(shape, self.dtype, _ptr=self.ptr, _base=self._base if self._base is not None else self)

    def __repr__(self):
        return "DeviceTensor(shape=%s, dtype=%s)" % (self.shape, self.dtype)

    def __del__(self):
        try:
            if self._base is None and self.ptr and _lib._lib is not None and _lib._initialised:
                _lib._lib.aeth_free(self.ptr)
        except Exception:
            pass


def as_device(a, dtype=np.float32):
    """Pass a DeviceTensor through; upload anything array-like as ``dtype``."""
    if isinstance(a, DeviceTensor):
        if a.dtype != np.dtype(dtype):
            return DeviceTensor.from_numpy(a.get().astype(dtype))
        return a
    return DeviceTensor.from_numpy(np.asarray(a), dtype=dtype)
