"""Device array of the ``hip`` backend, seen from Python.

It plays the role of ``chainerx.ndarray`` for the harness and the tests: a (buffer, offset, shape,
byte-strides, dtype) tuple, with views made on the host and every arithmetic operation forwarded
to one C-ABI kernel call.  Device memory comes from the library's own pool (``hipcx_malloc`` /
``hipcx_free``) and crosses the host boundary through its copy entry points
(``hipcx_from_host_memory``, ``hipcx_memcpy_to_host``): the Device interface of the backend.
PyTorch is only asked for the current stream (and captures HIP graphs in the benchmarks).
"""
import ctypes

import numpy

from chainer_amd import _lib

# chainerx::Dtype codes (CX/dtype.h:19-29)
_DTYPE_CODES = {
    numpy.dtype('bool'): 1,
    numpy.dtype('int8'): 2,
    numpy.dtype('int16'): 3,
    numpy.dtype('int32'): 4,
    numpy.dtype('int64'): 5,
    numpy.dtype('uint8'): 6,
    numpy.dtype('float16'): 7,
    numpy.dtype('float32'): 8,
    numpy.dtype('float64'): 9,
}

_torch = None


def torch():
    global _torch
    if _torch is None:
        import torch as _t
        _torch = _t
    return _torch


def device_available():
    return torch().cuda.is_available()


def _require_device():
    if not torch().cuda.is_available():
        raise _lib.BackendError('no HIP device is visible: the hip backend has no CPU fallback')


def current_stream():
    return ctypes.c_void_p(torch().cuda.current_stream().cuda_stream)


def synchronize():
    """Device::Synchronize (CX/device.h:71).  Raises the IndexError of an earlier take / add_at (default bounds mode) whose indices
    were out of range."""
    torch().cuda.synchronize()
    _lib.call('hipcx_synchronize', DEVICE_INDEX)


def dtype_code(dtype):
    try:
        return _DTYPE_CODES[numpy.dtype(dtype)]
    except KeyError:
        raise _lib.DtypeError('unsupported dtype: %s' % (dtype,))


def contiguous_strides(shape, itemsize):
    """C-contiguous byte strides; zero-sized axes count as 1 (CX/strides.cc:17-26)."""
    st = []
    acc = itemsize
    for d in reversed(shape):
        st.append(acc)
        acc *= max(1, d)
    return tuple(reversed(st))


DEVICE_INDEX = 0


class DeviceBuffer(object):
    """One allocation of the backend's memory pool (Device::Allocate, CX/device.h:33); returned to the pool when the last
    array that refers to it goes away, like the deleter of the reference's ``shared_ptr<void>``."""

    __slots__ = ('ptr', 'nbytes', '__weakref__')

    def __init__(self, nbytes):
        self.ptr = 0
        _require_device()
        self.nbytes = int(nbytes)
        out = ctypes.c_void_p()
        _lib.call('hipcx_malloc_on_stream', DEVICE_INDEX, max(self.nbytes, 1), current_stream(), ctypes.byref(out))
        self.ptr = out.value or 0

    @classmethod
    def adopt(cls, ptr, nbytes):
        """Takes ownership of a pointer the pool has already handed out (hipcx_from_host_memory)."""
        self = cls.__new__(cls)
        self.ptr = int(ptr or 0)
        self.nbytes = int(nbytes)
        return self

    def data_ptr(self):
        return self.ptr

    def record_stream(self, stream=None):
        """Announces that work on this block is queued on ``stream`` (a raw stream handle; default: the current stream), which is
        not the stream it was allocated on: the pool then holds the block back after its release until that work has run
        (hipcx_record_stream)."""
        if self.ptr:
            _lib.call('hipcx_record_stream', DEVICE_INDEX, ctypes.c_void_p(self.ptr), current_stream() if stream is None else stream)

    def __del__(self):
        ptr, self.ptr = self.ptr, 0
        if ptr:
            try:
                _lib.load().hipcx_free(DEVICE_INDEX, ctypes.c_void_p(ptr))
            except Exception:  # interpreter shutdown: the library may be gone already
                pass


def alloc_bytes(nbytes):
    return DeviceBuffer(nbytes)


def pool_stats():
    """Counters of the device memory pool (hipcx_pool_stats)."""
    st = _lib.CPoolStats()
    _lib.call('hipcx_pool_stats', DEVICE_INDEX, ctypes.byref(st))
    return {name: int(getattr(st, name)) for name, _ in _lib.CPoolStats._fields_}


def free_unused_blocks():
    """MemoryPool::FreeUnusedBlocks (CX/cuda/memory_pool.cc:172-203)."""
    _lib.call('hipcx_pool_free_unused', DEVICE_INDEX)


_next_arena = [1]


class memory_arena(object):
    """Allocations made inside the ``with`` block come from, and return to, free lists of their own.  A HIP graph is
    captured inside one (after an eager pass in the same arena has filled its free lists, so that the capture itself never
    reaches the driver): the addresses baked into the graph are then not handed to anybody else until ``release()``."""

    def __init__(self):
        self.id = _next_arena[0]
        _next_arena[0] += 1

    def __enter__(self):
        _lib.call('hipcx_pool_set_arena', DEVICE_INDEX, self.id)
        return self

    def __exit__(self, *exc):
        _lib.call('hipcx_pool_set_arena', DEVICE_INDEX, 0)
        return False

    def release(self):
        _lib.call('hipcx_pool_release_arena', DEVICE_INDEX, self.id)


class ndarray(object):
    """Strided view of device memory."""

    __slots__ = ('_buf', '_offset', 'shape', 'strides', 'dtype', '_desc', '_ptr')

    def __init__(self, buf, offset, shape, strides, dtype):
        self._buf = buf
        self._offset = int(offset)
        self.shape = tuple(int(s) for s in shape)
        self.strides = tuple(int(s) for s in strides)
        self.dtype = numpy.dtype(dtype)
        if len(self.shape) > _lib.MAX_NDIM:
            raise _lib.DimensionError('ndim %d exceeds the maximum of %d' % (len(self.shape), _lib.MAX_NDIM))
        self._ptr = buf.data_ptr() + self._offset
        self._desc = None

    # ---- construction -------------------------------------------------------------------
    @staticmethod
    def empty(shape, dtype, strides=None):
        shape = _as_shape(shape)
        dtype = numpy.dtype(dtype)
        dtype_code(dtype)
        if strides is None:
            strides = contiguous_strides(shape, dtype.itemsize)
            nbytes = _prod(shape) * dtype.itemsize
        else:
            nbytes = 0 if 0 in shape else dtype.itemsize + sum((d - 1) * abs(s) for d, s in zip(shape, strides))
        return ndarray(alloc_bytes(nbytes), 0, shape, strides, dtype)

    # ---- properties ---------------------------------------------------------------------
    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        return _prod(self.shape)

    @property
    def itemsize(self):
        return self.dtype.itemsize

    @property
    def nbytes(self):
        return self.size * self.itemsize

    def record_stream(self, stream=None):
        """See DeviceBuffer.record_stream: call it when the array is used on a stream other than the one it was created on and may
        be dropped before that stream is waited for."""
        self._buf.record_stream(stream)

    @property
    def data_ptr(self):
        return self._ptr

    @property
    def is_contiguous(self):
        """C-contiguity ignoring unit axes (CX/shape.cc:15-32)."""
        expect = self.itemsize
        for d, s in zip(reversed(self.shape), reversed(self.strides)):
            if d == 0:
                return True
            if d != 1 and s != expect:
                return False
            expect *= d
        return True

    @property
    def T(self):
        return self.transpose()

    def desc(self):
        """The hipcx_array descriptor of this view (built once; views are immutable)."""
        d = self._desc
        if d is None:
            d = _lib.CArray()
            d.data = self._ptr
            d.dtype = dtype_code(self.dtype)
            d.ndim = len(self.shape)
            for i, (n, s) in enumerate(zip(self.shape, self.strides)):
                d.shape[i] = n
                d.strides[i] = s
            self._desc = d
        return ctypes.byref(d)

    def __repr__(self):
        return 'chainer_amd.ndarray(shape=%r, dtype=%s, strides=%r, device=hip:0)' % (self.shape, self.dtype, self.strides)

    def __len__(self):
        if not self.shape:
            raise TypeError('len() of unsized object')
        return self.shape[0]

    # ---- views (host-only, no kernel) ---------------------------------------------------
    def _view(self, offset, shape, strides, dtype=None):
        return ndarray(self._buf, offset, shape, strides, self.dtype if dtype is None else dtype)

    def transpose(self, *axes):
        if len(axes) == 1 and (axes[0] is None or isinstance(axes[0], (tuple, list))):
            axes = axes[0]
        if axes is None or len(axes) == 0:
            axes = tuple(reversed(range(self.ndim)))
        axes = tuple(_normalize_axis(a, self.ndim) for a in axes)
        if sorted(axes) != list(range(self.ndim)):
            raise _lib.DimensionError('axes do not match the array: %r' % (axes,))
        return self._view(self._offset, [self.shape[a] for a in axes], [self.strides[a] for a in axes])

    def broadcast_to(self, shape):
        """Stride-0 broadcast view (CX/routines/manipulation.cc:316-358)."""
        shape = _as_shape(shape)
        if len(shape) < self.ndim:
            raise _lib.DimensionError('cannot broadcast %r to %r' % (self.shape, shape))
        strides = [0] * len(shape)
        lead = len(shape) - self.ndim
        for i in range(self.ndim):
            d, s = self.shape[i], self.strides[i]
            if d == shape[lead + i]:
                strides[lead + i] = s if d != 1 else 0
            elif d == 1:
                strides[lead + i] = 0
            else:
                raise _lib.DimensionError('cannot broadcast %r to %r' % (self.shape, shape))
        return self._view(self._offset, shape, strides)

    def reshape(self, *shape):
        """View when the strides allow it, else a contiguous copy (CX/routines/manipulation.cc:153-258)."""
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = shape[0]
        shape = list(int(s) for s in shape)
        if shape.count(-1) > 1:
            raise _lib.DimensionError('can only specify one unknown dimension')
        if -1 in shape:
            rest = _prod([s for s in shape if s != -1])
            if rest == 0 or self.size % rest != 0:
                raise _lib.DimensionError('cannot reshape array of size %d into shape %r' % (self.size, tuple(shape)))
            shape[shape.index(-1)] = self.size // rest
        shape = tuple(shape)
        if _prod(shape) != self.size:
            raise _lib.DimensionError('cannot reshape array of size %d into shape %r' % (self.size, shape))
        if shape == self.shape:
            return self
        strides = _nocopy_reshape_strides(self.shape, self.strides, shape, self.itemsize)
        if strides is not None:
            return self._view(self._offset, shape, strides)
        c = self.copy()
        return c._view(c._offset, shape, contiguous_strides(shape, self.itemsize))

    def squeeze(self, axis=None):
        if axis is None:
            keep = [i for i in range(self.ndim) if self.shape[i] != 1]
        else:
            if not isinstance(axis, (tuple, list)):
                axis = (axis,)
            axis = set(_normalize_axis(a, self.ndim) for a in axis)
            for a in axis:
                if self.shape[a] != 1:
                    raise _lib.DimensionError('cannot squeeze an axis of extent %d' % self.shape[a])
            keep = [i for i in range(self.ndim) if i not in axis]
        return self._view(self._offset, [self.shape[i] for i in keep], [self.strides[i] for i in keep])

    def __getitem__(self, key):
        """Basic indexing only (ints, slices, None, Ellipsis): Array::At (CX/routines/indexing.cc)."""
        if not isinstance(key, tuple):
            key = (key,)
        n_real = sum(1 for k in key if k is not None and k is not Ellipsis)
        if n_real > self.ndim:
            raise _lib.DimensionError('too many indices for array')
        if key.count(Ellipsis) > 1:
            raise _lib.DimensionError('an index can only have a single ellipsis')
        if Ellipsis in key:
            i = key.index(Ellipsis)
            key = key[:i] + (slice(None),) * (self.ndim - n_real) + key[i + 1:]
        else:
            key = key + (slice(None),) * (self.ndim - n_real)
        offset = self._offset
        shape, strides = [], []
        axis = 0
        for k in key:
            if k is None:
                shape.append(1)
                strides.append(0)
                continue
            dim, st = self.shape[axis], self.strides[axis]
            if isinstance(k, slice):
                start, stop, step = k.indices(dim)
                n = len(range(start, stop, step))
                offset += start * st if n > 0 else 0
                shape.append(n)
                strides.append(st * step)
            else:
                k = int(k)
                if k < -dim or k >= dim:
                    raise _lib.ChainerxIndexError('index %d is out of bounds for axis %d with size %d' % (k, axis, dim))
                if k < 0:
                    k += dim
                offset += k * st
            axis += 1
        return self._view(offset, shape, strides)

    # ---- kernels ------------------------------------------------------------------------
    def copy(self):
        """C-contiguous copy (CopyKernel)."""
        out = ndarray.empty(self.shape, self.dtype)
        _lib.call('hipcx_copy', self.desc(), out.desc(), current_stream())
        return out

    def astype(self, dtype, copy=True):
        """Array::AsType (CX/array.cc): a new C-contiguous array unless copy=False and the dtype matches."""
        dtype = numpy.dtype(dtype)
        if not copy and dtype == self.dtype:
            return self
        out = ndarray.empty(self.shape, dtype)
        _lib.call('hipcx_copy', self.desc(), out.desc(), current_stream())
        return out

    def as_contiguous(self):
        return self if self.is_contiguous else self.copy()

    def fill(self, value):
        _lib.call('hipcx_fill', self.desc(), _lib.make_scalar(value), current_stream())

    def get(self):
        """Device -> host (numpy) copy; synchronises like Array::ToNative (CX/array.cc:399-444)."""
        a = self.as_contiguous()
        n = a.size * a.itemsize
        host = numpy.empty(a.shape, a.dtype)
        if n == 0:
            return host
        _lib.call('hipcx_memcpy_to_host', DEVICE_INDEX, ctypes.c_void_p(host.ctypes.data), ctypes.c_void_p(a._ptr), n, current_stream())
        return host

    def __array__(self, dtype=None, copy=None):
        a = self.get()
        return a if dtype is None else a.astype(dtype)

    def item(self):
        return self.get().item()

    def __float__(self):
        return float(self.item())

    def __int__(self):
        return int(self.item())

    # arithmetic operators are attached by chainer_amd.routines


def _prod(xs):
    n = 1
    for x in xs:
        n *= int(x)
    return n


def _as_shape(shape):
    if isinstance(shape, (int, numpy.integer)):
        return (int(shape),)
    return tuple(int(s) for s in shape)


def _normalize_axis(axis, ndim):
    axis = int(axis)
    if axis < -ndim or axis >= ndim:
        raise _lib.DimensionError('axis %d is out of bounds for array of dimension %d' % (axis, ndim))
    return axis + ndim if axis < 0 else axis


def _nocopy_reshape_strides(old_shape, old_strides, new_shape, itemsize):
    """Strides of `new_shape` over the same memory, or None if a copy is needed."""
    if _prod(old_shape) == 0:
        return contiguous_strides(new_shape, itemsize)
    # drop unit axes of the source
    od = [(d, s) for d, s in zip(old_shape, old_strides) if d != 1]
    new_strides = [0] * len(new_shape)
    oi = 0
    ni = 0
    nn = len(new_shape)
    while ni < nn:
        if new_shape[ni] == 1:
            new_strides[ni] = itemsize
            ni += 1
            continue
        if oi >= len(od):
            return None
        # grow a group of new axes and a group of old axes until their sizes match
        np_ = new_shape[ni]
        op = od[oi][0]
        nj, oj = ni + 1, oi + 1
        while np_ != op:
            if np_ < op:
                while nj < nn and new_shape[nj] == 1:
                    nj += 1
                if nj >= nn:
                    return None
                np_ *= new_shape[nj]
                nj += 1
            else:
                if oj >= len(od):
                    return None
                op *= od[oj][0]
                oj += 1
        # the old group must be internally contiguous
        for k in range(oi, oj - 1):
            if od[k][1] != od[k + 1][0] * od[k + 1][1]:
                return None
        # assign strides to the new group, innermost first
        st = od[oj - 1][1]
        for k in range(nj - 1, ni - 1, -1):
            new_strides[k] = st
            st *= new_shape[k]
        ni, oi = nj, oj
    if oi != len(od):
        return None
    return tuple(new_strides)


def array(obj, dtype=None):
    """Host -> device upload: chainerx.array(numpy_array, device='hip:0') (Device::FromHostMemory)."""
    if isinstance(obj, ndarray):
        return obj.astype(dtype if dtype is not None else obj.dtype)
    a = numpy.asarray(obj, dtype=dtype)
    dtype_code(a.dtype)
    a = numpy.ascontiguousarray(a)
    _require_device()
    if a.size == 0:
        return ndarray.empty(a.shape, a.dtype)
    out = ctypes.c_void_p()
    _lib.call('hipcx_from_host_memory', DEVICE_INDEX, ctypes.c_void_p(a.ctypes.data), a.nbytes, ctypes.byref(out), current_stream())
    buf = DeviceBuffer.adopt(out.value, a.nbytes)
    return ndarray(buf, 0, a.shape, contiguous_strides(a.shape, a.dtype.itemsize), a.dtype)


def to_numpy(a):
    return a.get()
