"""Array types held in ``Tensor.data``.

``nparray``  host array: ``numpy.ndarray`` subclass carrying the shared in-place version
             counter ``_version`` (a one-element list), as ``src/tortto/xparray.py:23-37``.
``hiparray`` device array: the counterpart of the reference's CuPy-backed ``cparray``
             (``src/tortto/xparray.py:65-78``).  It owns a buffer obtained from
             ``libtortto_hip.so`` through ctypes; data are always C-contiguous.  Only what
             the convolution / BatchNorm path and its callers touch is provided -- it is not
             an array library.
"""
import ctypes
import weakref
from math import prod

import numpy as np

from . import _hip


class nparray(np.ndarray):
    def __new__(cls, input_array, *args, **kwargs):
        if input_array.__class__ is cls:
            return input_array
        if kwargs.get('copy') is False:
            # NumPy >= 2 raises for copy=False when a cast forces a copy; the reference relies
            # on the older "copy only if needed" meaning
            kwargs['copy'] = None
        obj = np.array(input_array, *args, **kwargs).view(cls)
        obj._version = [0]
        return obj

    def __array_finalize__(self, obj):
        if obj is None:
            return
        base = self.base
        if base is not None and base.base is not None:   # a view of an nparray shares its counter
            self._version = getattr(obj, '_version', [0])
        else:
            self._version = [0]


class Device:
    """What ``Tensor.device`` returns for device tensors."""

    def __init__(self, index=0):
        self.id = index

    def __repr__(self):
        return f'hip:{self.id}'

    def __eq__(self, other):
        return isinstance(other, Device) and other.id == self.id

    def __hash__(self):
        return hash(('hip', self.id))


class _Buffer:
    """One ``tt_malloc`` allocation; freed (returned to the library's pool) with the last array
    that refers to it.  With ``lazy`` the block is taken on the first use of ``ptr``, and
    ``on_demand`` (a callable receiving the buffer) then fills it: the output of an operation that
    was absorbed into its successor exists only if somebody else asks for it."""
    __slots__ = ('_ptr', 'nbytes', 'on_demand', 'deps', '__weakref__')

    def __init__(self, nbytes, lazy=False):
        self.nbytes = nbytes
        self._ptr = 0
        self.on_demand = None
        self.deps = ()
        if not lazy:
            self._allocate()

    def _allocate(self):
        p = ctypes.c_void_p()
        _hip.call('tt_malloc', ctypes.byref(p), self.nbytes)
        self._ptr = p.value or 0

    def fill_on_demand(self, fill, operands):
        """Let ``fill(buffer)`` produce the contents when they are first asked for.  ``operands``
        are the arrays ``fill`` will read: the reference computed the values when the operation
        ran, so they must not see a later in-place change of an operand -- ``before_write`` fills
        this buffer just before any of them is written."""
        with _hip._lock:
            self.on_demand = fill
            self.deps = tuple(a._buf for a in operands if a is not None)
            _unfilled.add(self)

    @property
    def ptr(self):
        if (not self._ptr and self.nbytes) or self.on_demand is not None:
            with _hip._lock:            # two threads may ask for the same unfilled buffer
                if not self._ptr and self.nbytes:
                    # a parked operation may be the one that produces this very buffer: let it run
                    # (and allocate the buffer itself) before the block is taken here
                    _hip.flush()
                    if not self._ptr:
                        self._allocate()
                if self.on_demand is not None:
                    fill, self.on_demand = self.on_demand, None
                    _unfilled.discard(self)
                    fill(self)
                    self.deps = ()
        return self._ptr

    def __del__(self):
        try:
            if self._ptr:
                _hip.load_library().tt_free(ctypes.c_void_p(self._ptr))
                self._ptr = 0
        except Exception:   # interpreter shutdown
            pass


# buffers whose contents are still to be produced on demand (normally none or a handful: the
# array of an absorbed BatchNorm or Add output lives only as long as somebody holds its tensor)
_unfilled = weakref.WeakSet()


def before_write(buf):
    """Called before ``buf`` is overwritten in place: every on-demand buffer that would read it
    is filled now, from the values the reference's eager evaluation saw."""
    if not _unfilled:
        return
    with _hip._lock:
        for lazy in list(_unfilled):
            if any(d is buf for d in lazy.deps):
                lazy.ptr


def poison(arrays, exc):
    """Make every later use of ``arrays`` raise ``exc``: the operation that was to fill them failed."""
    def fail(buf):
        buf.on_demand = fail
        raise exc
    for a in arrays:
        if a is not None:
            a._buf.on_demand = fail


class hiparray:
    __slots__ = ('_buf', '_shape', '_dtype', '_version', '_shared', '__weakref__')

    def __new__(cls, input_array=None, dtype=None, copy=True, _buf=None, _shape=None, _version=None):
        if input_array.__class__ is cls:
            if dtype is None or np.dtype(dtype) == input_array._dtype:
                return input_array
            input_array = input_array.get()
        self = object.__new__(cls)
        self._shared = False
        if _buf is not None:            # internal: wrap an existing buffer
            self._buf, self._shape, self._dtype = _buf, tuple(_shape), np.dtype(dtype)
            self._version = _version if _version is not None else [0]
            return self
        given = np.asarray(input_array, dtype=dtype)
        host = np.ascontiguousarray(given).reshape(given.shape)     # ascontiguousarray turns 0-d into 1-d
        self._shape = host.shape
        self._dtype = host.dtype
        self._version = [0]
        self._buf = _Buffer(host.nbytes)
        if host.nbytes:
            _hip.call('tt_memcpy_h2d', self.ptr, host.ctypes.data, host.nbytes)
        return self

    # ---- construction helpers -------------------------------------------------------------
    @classmethod
    def empty(cls, shape, dtype=np.float32):
        shape = (shape,) if isinstance(shape, int) else tuple(shape)
        dtype = np.dtype(dtype)
        return cls(_buf=_Buffer(prod(shape) * dtype.itemsize), _shape=shape, dtype=dtype)

    @classmethod
    def lazy(cls, shape, dtype=np.float32):
        """An array whose block is allocated when its ``ptr`` is first used."""
        shape = (shape,) if isinstance(shape, int) else tuple(shape)
        dtype = np.dtype(dtype)
        return cls(_buf=_Buffer(prod(shape) * dtype.itemsize, lazy=True), _shape=shape, dtype=dtype)

    @classmethod
    def zeros(cls, shape, dtype=np.float32):
        out = cls.empty(shape, dtype)
        if out.nbytes:
            _hip.call('tt_memset', out.ptr, 0, out.nbytes)
        return out

    @classmethod
    def empty_like(cls, other):
        return cls.empty(other.shape, other.dtype)

    # ---- ndarray-like attributes ----------------------------------------------------------
    @property
    def ptr(self):
        return self._buf.ptr

    @property
    def shape(self):
        return self._shape

    @property
    def dtype(self):
        return self._dtype

    @property
    def ndim(self):
        return len(self._shape)

    @property
    def size(self):
        return prod(self._shape)

    @property
    def itemsize(self):
        return self._dtype.itemsize

    @property
    def nbytes(self):
        return self.size * self._dtype.itemsize

    @property
    def strides(self):
        st, acc = [], self._dtype.itemsize
        for d in reversed(self._shape):
            st.append(acc)
            acc *= d
        return tuple(reversed(st))

    @property
    def device(self):
        return Device(0)

    def __len__(self):
        return self._shape[0]

    def __repr__(self):
        return f'hiparray(shape={self._shape}, dtype={self._dtype}, ptr=0x{self._buf._ptr:x})'

    # ---- data movement --------------------------------------------------------------------
    def get(self):
        """Device -> host copy as a plain ``numpy.ndarray`` (waits for pending kernels)."""
        out = np.empty(self._shape, dtype=self._dtype)
        if out.nbytes:
            _hip.call('tt_memcpy_d2h', out.ctypes.data, self.ptr, out.nbytes)
        return out

    def item(self):
        return self.get().item()

    def alias(self):
        """A second array on the same block for a holder that only reads it.  Both arrays are marked
        shared: whoever is about to write one of them in place (``+=``, ``fill``, ``set``, a kernel
        with ``out=``) calls ``own()`` first, which moves that array to a copy.  Gradients handed to
        two operands travel this way: each holder has an array of its own, as the reference's
        copies give it, and the copy is made only for a holder that writes."""
        self._shared = True
        other = hiparray(_buf=self._buf, _shape=self._shape, dtype=self._dtype)
        other._shared = True
        return other

    def own(self):
        """Make sure this array is the only one on its block before it is written in place, and
        that nothing still to be computed on demand depends on the values about to be replaced."""
        if not self._shared:
            before_write(self._buf)
        else:
            fresh = _Buffer(self.nbytes)
            if self.nbytes:
                _hip.call('tt_memcpy_d2d', fresh.ptr, self._buf.ptr, self.nbytes)
            self._buf = fresh
            self._shared = False
        return self

    def copy(self):
        out = hiparray.empty(self._shape, self._dtype)
        if out.nbytes:
            _hip.call('tt_memcpy_d2d', out.ptr, self.ptr, out.nbytes)
        return out

    def set(self, host):
        """Overwrite the contents from a host array of the same shape (used by ``copy_``)."""
        host = np.asarray(host, dtype=self._dtype)
        if host.shape != self._shape:
            host = np.broadcast_to(host, self._shape)
        host = np.ascontiguousarray(host)               # (a 0-d array comes back 1-d: same bytes)
        self.own()
        if host.nbytes:
            _hip.call('tt_memcpy_h2d', self.ptr, host.ctypes.data, host.nbytes)
        return self

    def reshape(self, *shape):
        """A view with another shape on the same buffer (shares the version counter)."""
        if len(shape) == 1 and not isinstance(shape[0], int):
            shape = tuple(shape[0])
        shape = list(shape)
        if -1 in shape:
            i = shape.index(-1)
            rest = prod(s for j, s in enumerate(shape) if j != i)
            shape[i] = self.size // rest if rest else 0
        if prod(shape) != self.size:
            raise ValueError(f'cannot reshape array of size {self.size} into shape {tuple(shape)}')
        view = hiparray(_buf=self._buf, _shape=shape, dtype=self._dtype, _version=self._version)
        view._shared = self._shared
        return view

    def view(self, _cls=None):
        return self

    # ---- the few in-place operations autograd and the modules need ---------------------------
    def _require_f32(self, what):
        if self._dtype != np.float32:
            raise TypeError(f'{what} on a device array is implemented for float32 only, got {self._dtype}')

    def fill(self, value):
        self._require_f32('fill')
        self.own()
        if self.size:
            _hip.call('tt_fill_f32', self.ptr, float(value), self.size)

    def __iadd__(self, other):
        self._require_f32('+=')
        self.own()
        if isinstance(other, hiparray):
            if other.shape != self._shape or other.dtype != self._dtype:
                raise ValueError(f'device += needs equal shapes and dtypes, got {self._shape} and {other.shape}')
            if self.size:
                _hip.call('tt_axpy_f32', 1.0, other.ptr, self.ptr, self.size)
        elif isinstance(other, (int, float, np.floating, np.integer)):
            if self.size:
                _hip.call('tt_add_scalar_f32', self.ptr, float(other), self.size)
        else:
            raise TypeError(f'device += is not defined for {other.__class__.__name__}')
        return self


def ascontiguousarray(a):
    """Device arrays are always contiguous."""
    return a
