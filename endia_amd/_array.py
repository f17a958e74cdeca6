"""Device-resident Array: the host-side mirror of endia/_array/_array.mojo.

An Array is a handle on a node: a (possibly shared) device buffer, a shape / element-stride / offset
triple, and the autograd fields of the reference's Node (`requires_grad`, the stored gradient, the
argument list and the VJP rule: _array.mojo:55-179). Views (permute, expand, squeeze, reshape, real)
share the buffer of their base, as in the reference. Storage is fp32, row-major; complex arrays are
interleaved (re, im) pairs (_array.mojo:126,528-536) and `is_complex` arrays count COMPLEX elements in
their shape and strides.

All arithmetic happens in libendia_hip.so; numpy appears only where data crosses the host boundary.
"""
import ctypes

import numpy as np

from . import _lib as L


# Small buffers that die are kept here, by exact size, and handed out again without a call into the library: a
# small model's eager step creates a few dozen arrays, and two library calls per array were a third of its time.
# Only buffers of at most 8 MiB, at most 256 MiB in total; never while a step is being captured, and never a buffer
# that was allocated during a capture (the library keeps those for the captured step's replays).
_FREE = {}
_FREE_BYTES = [0]
_CACHE_MAX_BUFFER = 8 << 20
_CACHE_MAX_TOTAL = 256 << 20


class Buffer:
    """One allocation from the library's pool; returned to the pool when the last view dies."""

    __slots__ = ("address", "nbytes", "captured", "pending", "version")

    def __init__(self, nbytes):
        nbytes = int(nbytes)
        self.nbytes = nbytes
        self.captured = L.capturing
        self.pending = False  # a parked product (see _lib.park_product) has yet to write this buffer
        self.version = 0      # counts in-place writes by user-visible updates (optimizer steps, -=, copy_from_numpy, a[...] = v)
        if not L.capturing:
            held = _FREE.get(nbytes)
            if held:
                self.address = held.pop()
                _FREE_BYTES[0] -= nbytes
                return
        p = ctypes.c_void_p()
        L.call("endia_hip_malloc", nbytes, ctypes.byref(p))
        self.address = p.value or 0

    @property
    def ptr(self):
        """The device address, for a kernel argument or a copy: whatever is still to write this buffer is launched first."""
        if self.pending:
            L.flush(self)
        return self.address

    def __del__(self):
        ptr = getattr(self, "address", 0)
        if not ptr:
            return
        self.address = 0
        try:
            if (not self.captured and not L.capturing and self.nbytes <= _CACHE_MAX_BUFFER
                    and _FREE_BYTES[0] + self.nbytes <= _CACHE_MAX_TOTAL):
                _FREE.setdefault(self.nbytes, []).append(ptr)
                _FREE_BYTES[0] += self.nbytes
            else:
                L.lib().endia_hip_free(ctypes.c_void_p(ptr))
        except Exception:
            pass


def release_cached_buffers():
    """Give the buffers held above back to the library's pool."""
    for held in _FREE.values():
        for ptr in held:
            L.lib().endia_hip_free(ctypes.c_void_p(ptr))
    _FREE.clear()
    _FREE_BYTES[0] = 0


def contiguous_strides(shape):
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= s
    return tuple(reversed(st))


def _prod(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


class Array:
    """`Array(shape)` gives a zero-filled array like the reference's constructor (_array.mojo:198-214)."""

    # autograd fields that most arrays never change live on the class; an instance stores what differs
    _requires_grad = False
    _grad = None
    _args = ()
    _vjp = None
    _name = "arg"
    _meta = None
    _id = -1
    _consumers = 0
    _contributions_left = 0  # during a reverse walk: consumers whose VJP has not run yet
    _is_seed = False
    _act_applied = False  # a gradient that already carries the producer's activation derivative
    _grad_fused = None    # such a gradient on its way to this node's own VJP rule; never what grad() returns
    _true_grad = None     # on an _act_applied gradient: a function that computes the gradient without the derivative
    _on_final_grad = None  # set by an optimizer with fused_backward=True: called by backward() when this leaf's gradient is complete
    _lazy_mlp = None      # on the output of functional.mlp_forward while its launch is parked: what mse() needs to fuse with it
    _internal = False     # a node that a VJP rule created (the transposes and broadcasts inside a recorded backward pass)
    _absorbed = False     # a VJP result that already includes the gradient its primal held (functional._absorb)
    _offset = 0
    is_complex_ = False

    def __init__(self, shape=None, requires_grad=False, is_complex=False, _buffer=None, _strides=None, _offset=0,
                 _zero=True):
        if isinstance(shape, np.ndarray):
            raise TypeError("use endia_amd.array(ndarray) / Array.from_numpy to upload host data")
        if isinstance(shape, int):
            shape = [shape]
        shape = tuple(int(s) for s in (shape if shape is not None else (0,)))
        self._shape = shape
        self._strides = tuple(_strides) if _strides is not None else contiguous_strides(shape)
        if _offset:
            self._offset = int(_offset)
        if is_complex:
            self.is_complex_ = True
        if _buffer is None:
            n = _prod(shape) * (2 if is_complex else 1)
            _buffer = Buffer(4 * n)
            if _zero and n:
                L.call("endia_hip_fill", _buffer.ptr, n, 0.0)
        self._buf = _buffer
        if requires_grad:
            self._requires_grad = True

    # ---- construction / host transfer ---------------------------------------------------------
    @staticmethod
    def empty(shape, is_complex=False):
        """An array whose contents the caller is about to overwrite (no fill launch). `shape` holds ints."""
        self = object.__new__(Array)
        self._shape = shape = tuple(shape)
        self._strides = contiguous_strides(shape)
        n = 4
        for s in shape:
            n *= s
        if is_complex:
            self.is_complex_ = True
            n *= 2
        self._buf = Buffer(n)
        return self

    @staticmethod
    def from_numpy(a, requires_grad=False):
        a = np.asarray(a)
        cplx = np.iscomplexobj(a)
        a = np.ascontiguousarray(a, dtype=np.complex64 if cplx else np.float32)
        shape = a.shape if a.ndim else (1,)
        out = Array(shape, requires_grad=requires_grad, is_complex=cplx, _zero=False)
        if a.size:
            L.call("endia_hip_memcpy_h2d", out._buf.ptr, a.ctypes.data, a.nbytes)
        return out

    def copy_from_numpy(self, a):
        """Overwrite this (contiguous) array's buffer in place, e.g. to feed a captured step its next batch."""
        a = np.ascontiguousarray(a, dtype=np.complex64 if self.is_complex_ else np.float32)
        if a.size != self.size() or not self.is_contiguous():
            raise ValueError("copy_from_numpy: need a contiguous destination of the same element count")
        if a.size:
            L.call("endia_hip_memcpy_h2d", self.data_ptr(), a.ctypes.data, a.nbytes)
        self._buf.version += 1
        return self

    def to_numpy(self):
        c = self if self.is_contiguous() else _contiguous_copy(self)
        out = np.empty(self._shape, dtype=np.complex64 if self.is_complex_ else np.float32)
        if out.size:
            L.call("endia_hip_memcpy_d2h", out.ctypes.data, c.data_ptr(), out.nbytes)
        return out

    # ---- shape queries (names follow the reference) ---------------------------------------------
    def shape(self):
        return list(self._shape)

    def stride(self):
        return list(self._strides)

    def storage_offset(self):
        return self._offset

    def ndim(self):
        return len(self._shape)

    def size(self):
        return _prod(self._shape)

    def is_complex(self):
        return self.is_complex_

    def is_contiguous(self):
        expect = 1
        for s, st in zip(reversed(self._shape), reversed(self._strides)):
            if s != 1 and st != expect:
                return False
            expect *= s
        return True

    def data_ptr(self):
        """Device address of element 0 of this view."""
        return self._buf.ptr + 4 * self._offset * (2 if self.is_complex_ else 1)

    def load(self, i):
        return self.to_numpy().reshape(-1)[i]

    def item(self):
        return self.to_numpy().reshape(-1)[0]

    # ---- autograd fields ------------------------------------------------------------------------
    def requires_grad(self):
        return self._requires_grad

    def requires_grad_(self, flag=True):
        self._requires_grad = bool(flag)
        return self

    def has_grad(self):
        return self._grad is not None or self._grad_fused is not None

    def grad_(self, g):
        self._grad = g

    def grad(self):
        if self._grad is None:
            if self._grad_fused is not None:
                # A fused layer handed this node dL/dh * act'(h) for its own backward rule. The gradient a caller
                # reads is dL/dh itself, as the reference stores it on every node: computed here, on first use.
                self._grad = self._grad_fused._true_grad()
                self._grad_fused._true_grad = None  # evaluated once: let go of the cotangent it held
                return self._grad
            return Array(self._shape, is_complex=self.is_complex_)
        return self._grad

    def remove_grad(self):
        self._grad = None
        self._grad_fused = None

    def args(self):
        return list(self._args)

    def clear_args(self):
        self._args = []
        self._vjp = None

    def name(self):
        return self._name

    def backward(self, create_graph=False):
        from .autograd.functional import backward
        backward(self, create_graph)

    def zero_grad(self):
        from .autograd.functional import zero_grad_rec
        zero_grad_rec(self)

    # ---- operators (endia/_array/_array.mojo:791-1099) ---------------------------------------------
    def T(self):
        from . import functional as F
        if self.ndim() == 1:
            return self
        return F.permute(self, [-1, -2])

    def reshape(self, shape):
        from . import functional as F
        return F.reshape(self, shape)

    @staticmethod
    def _as_slices(index):
        index = list(index) if isinstance(index, tuple) else [index]
        return [i if isinstance(i, slice) else slice(i, i + 1 if i != -1 else None) for i in index]

    def __getitem__(self, index):
        """a[1:3, ::2] is array_slice (_array.mojo:805-809); an integer keeps its axis with length 1."""
        from . import functional as F
        return F.array_slice(self, self._as_slices(index))

    def __setitem__(self, index, value):
        """Write an array of the block's shape, or a scalar, through the slice view (_array.mojo:811-880)."""
        from . import functional as F
        sub = F.array_slice(F.detach(self), self._as_slices(index))
        if not isinstance(value, Array):
            value = F.full(sub.shape(), float(value))
        if value.shape() != sub.shape() or value.is_complex_ != self.is_complex_:
            raise ValueError("Error: Shapes do not match")
        src = value if value.is_contiguous() else _contiguous_copy(value)
        if src.size():
            L.call("endia_hip_strided_scatter", sub.ndim(), L.i64_array(sub._shape), L.i64_array(sub._strides),
                   sub._offset, src.data_ptr(), self._buf.ptr, 0, 1 if self.is_complex_ else 0)
            self._buf.version += 1

    def _bin(self, other, fn, reverse=False):
        from . import functional as F
        if not isinstance(other, Array):
            # scalars become a one-row `full` operand and broadcast (_array.mojo:1014-1016)
            last = self._shape[-1] if self._shape else 1
            other = F.full([last], float(other))
        return fn(other, self) if reverse else fn(self, other)

    def __add__(self, o):
        from . import functional as F
        return self._bin(o, F.add)

    __radd__ = __add__

    def __sub__(self, o):
        from . import functional as F
        return self._bin(o, F.sub)

    def __rsub__(self, o):
        from . import functional as F
        return self._bin(o, F.sub, reverse=True)

    def __mul__(self, o):
        from . import functional as F
        return self._bin(o, F.mul)

    __rmul__ = __mul__

    def __truediv__(self, o):
        from . import functional as F
        return self._bin(o, F.div)

    def __rtruediv__(self, o):
        from . import functional as F
        return self._bin(o, F.div, reverse=True)

    def __matmul__(self, o):
        from . import functional as F
        return F.matmul(self, o)

    def __neg__(self):
        from . import functional as F
        return F.neg(self)

    def __pow__(self, o):  # pow_to, with a scalar spread over the last axis (_array.mojo:1074-1079)
        from . import functional as F
        return self._bin(o, F.pow)

    def __rpow__(self, o):
        from . import functional as F
        return self._bin(o, F.pow, reverse=True)

    # in-place updates write through to the existing buffer (execute_copy_raw, _array.mojo:998-1006)
    def _assign_from(self, other):
        assert other.size() == self.size() and other.is_complex_ == self.is_complex_
        src = other if other.is_contiguous() else _contiguous_copy(other)
        assert self.is_contiguous()
        L.call("endia_hip_memcpy_d2d", self.data_ptr(), src.data_ptr(), 4 * self.size() * (2 if self.is_complex_ else 1))
        self._buf.version += 1

    def __isub__(self, o):
        self._assign_from(self - o)
        return self

    def __iadd__(self, o):
        self._assign_from(self + o)
        return self

    def __repr__(self):
        return "Array(shape=%s%s, requires_grad=%s)" % (list(self._shape), ", complex" if self.is_complex_ else "",
                                                        self._requires_grad)

    def __str__(self):
        return str(self.to_numpy())


def _contiguous_copy(x):
    out = Array.empty(x._shape, x.is_complex_)
    if x.size():
        L.call("endia_hip_strided_copy", x.ndim(), L.i64_array(x._shape), L.i64_array(x._strides), x._offset,
               x._buf.ptr, out._buf.ptr, 1 if x.is_complex_ else 0)
    return out


Tensor = Array
ndarray = Array
