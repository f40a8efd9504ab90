"""DeviceArray: the array type HipHandler works on.

A dense, C-contiguous float32 array in device memory, described by a raw device
address and a shape. brainstorm's buffer manager allocates one flat array per
network and carves every layer's inputs, outputs, parameters and internals out
of it by slicing and reshaping (brainstorm/structure/buffers.py:79-83,
buffer_structure.py:218-245), and the recurrent layers index time steps with
negative integers (lstm_layer.py:117), so this type supports exactly that:
integer / slice / tuple indexing (step 1 only), ``reshape``, zero-sized and
0-d arrays -- all returning views that alias the parent. The minimal array
contract is the one brainstorm's DebugArray states (debug_handler.py:12-35).

Views that stay dense are plain DeviceArrays. A slice that needs a row pitch
(e.g. ``a[:, 1:3]`` of a wider matrix) raises NotImplementedError unless the
handler was created with ``pitched_views=True``, in which case it becomes a
PitchedDeviceArray (see there).
"""
from __future__ import annotations

import numpy as np

ITEMSIZE = 4


class _Block:
    """Owner of one pool block; returns it to the pool when the last view dies."""

    __slots__ = ("ptr", "_free")

    def __init__(self, ptr, free_fn):
        self.ptr = ptr
        self._free = free_fn

    def __del__(self):
        if self.ptr and self._free is not None:
            try:
                self._free(self.ptr)
            except Exception:   # interpreter shutdown
                pass
            self.ptr = 0


def _prod(shape):
    n = 1
    for s in shape:
        n *= s
    return n


class DeviceArray:
    __slots__ = ("ptr", "shape", "size", "_owner", "_handler", "_steps")

    dtype = np.dtype(np.float32)

    def __init__(self, ptr, shape, owner, handler=None):
        self.ptr = ptr              # device address of element 0 (int; 0 for empty arrays)
        self.shape = shape          # tuple of ints
        self.size = _prod(shape)
        self._owner = owner         # keeps the pool block alive
        self._handler = handler     # for get()
        self._steps = None          # a[i] views handed out so far (see __getitem__)

    @classmethod
    def _view_of(cls, parent, ptr, shape, size):
        """A dense view into ``parent``'s memory whose size is known (the views of the recurrent
        layers' inner loops are made thousands of times per step: no product over the shape)."""
        v = cls.__new__(cls)
        v.ptr = ptr
        v.shape = shape
        v.size = size
        v._owner = parent._owner
        v._handler = parent._handler
        v._steps = None
        return v

    # ---------------------------------------------------------------- basics
    @property
    def ndim(self):
        return len(self.shape)

    @property
    def nbytes(self):
        return self.size * ITEMSIZE

    def __len__(self):
        if not self.shape:
            raise TypeError("len() of a 0-d array")
        return self.shape[0]

    def __repr__(self):
        return "DeviceArray(shape=%r, ptr=0x%x)" % (self.shape, self.ptr or 0)

    def get(self):
        """NumPy copy of the contents (blocks until the device has caught up)."""
        return self._handler.get_numpy_copy(self)

    # ------------------------------------------------------------ arithmetic
    # brainstorm's ConstrainL2Norm writes `mat * mat` and `sq_norm ** 0.5` on handler arrays
    # (value_modifiers.py:79-80). As with NumPy arrays each expression yields a NEW array;
    # NumPy evaluates `x ** 0.5` as sqrt and `x ** 2` as x * x, so do these.
    def _binary(self, other, tt, st):
        h = self._handler
        out = h._scratch(self.shape)         # every element is written by the operation below
        if isinstance(other, DeviceArray):
            if other.shape != self.shape:
                raise ValueError("operands have shapes %r and %r; broadcasting is not supported"
                                 % (self.shape, other.shape))
            getattr(h, tt)(self, other, out)
        elif st is not None and isinstance(other, (int, float, np.integer, np.floating)):
            getattr(h, st)(other, self, out)
        else:
            return NotImplemented
        return out

    def __mul__(self, other):
        return self._binary(other, "mult_tt", "mult_st")

    __rmul__ = __mul__

    def __add__(self, other):
        return self._binary(other, "add_tt", "add_st")

    __radd__ = __add__

    def __sub__(self, other):
        return self._binary(other, "subtract_tt", None)

    def __truediv__(self, other):
        return self._binary(other, "divide_tt", None)

    def __pow__(self, exponent):
        h = self._handler
        out = h._scratch(self.shape)         # every element is written by the operation below
        if exponent == 0.5:
            h.sqrt_t(self, out)
        elif exponent == 2:
            h.mult_tt(self, self, out)
        elif exponent == 1:
            h.copy_to(self, out)
        else:
            raise NotImplementedError("DeviceArray ** %r: only the exponents 0.5, 1 and 2 are supported" % (exponent,))
        return out

    # --------------------------------------------------------------- reshape
    def reshape(self, *new_shape):
        if len(new_shape) == 1 and type(new_shape[0]) is tuple:
            new_shape = new_shape[0]
        # fast path (the layers reshape their buffers on every call): plain non-negative ints
        n = 1
        for s in new_shape:
            if type(s) is not int or s < 0:
                break
            n *= s
        else:
            if n != self.size:
                raise ValueError("cannot reshape array of size %d into shape %r" % (self.size, new_shape))
            out = DeviceArray.__new__(DeviceArray)
            out.ptr, out.shape, out.size, out._owner, out._handler = self.ptr, new_shape, n, self._owner, self._handler
            out._steps = None
            return out
        if len(new_shape) == 1 and not isinstance(new_shape[0], (int, np.integer)):
            new_shape = tuple(new_shape[0])
        new_shape = tuple(int(s) for s in new_shape)
        if -1 in new_shape:
            if new_shape.count(-1) > 1:
                raise ValueError("can only specify one unknown dimension")
            known = _prod(s for s in new_shape if s != -1)
            if known == 0 or self.size % known:
                raise ValueError("cannot reshape array of size %d into shape %r"
                                 % (self.size, new_shape))
            new_shape = tuple(self.size // known if s == -1 else s for s in new_shape)
        if any(s < 0 for s in new_shape) or _prod(new_shape) != self.size:
            raise ValueError("cannot reshape array of size %d into shape %r"
                             % (self.size, new_shape))
        return DeviceArray(self.ptr, new_shape, self._owner, self._handler)

    # -------------------------------------------------------------- indexing
    def __getitem__(self, key):
        shape = self.shape
        # fast paths: a[i] and a[i:j] on the first axis (the recurrent layers' inner loop)
        if type(key) is int:
            # a[t]: the recurrent layers take the same time-step views of the same buffers in every call of
            # every step (lstm_layer.py:117-145 indexes Za[t] three times in a row); a view is an immutable
            # (address, shape) pair, so the ones handed out are kept and handed out again
            steps = self._steps
            if steps is not None:
                v = steps.get(key)
                if v is not None:
                    return v
            if not shape:
                raise IndexError("too many indices for a 0-d array")
            n = shape[0]
            index = key + n if key < 0 else key
            if not 0 <= index < n:
                raise IndexError("index out of bounds for axis 0 with size %d" % n)
            inner = self.size // n
            v = DeviceArray._view_of(self, self.ptr + index * inner * ITEMSIZE if self.ptr else 0, shape[1:], inner)
            if steps is None:
                steps = self._steps = {}
            steps[key] = v
            return v
        if type(key) is slice:
            if not shape:
                raise IndexError("too many indices for a 0-d array")
            if key.step not in (None, 1):
                raise NotImplementedError("DeviceArray slices must have step 1")
            n = shape[0]
            start, stop, _ = key.indices(n)
            length = max(0, stop - start)
            inner = self.size // n if n else _prod(shape[1:])
            return DeviceArray._view_of(self, self.ptr + start * inner * ITEMSIZE if self.ptr else 0,
                                        (length,) + shape[1:], length * inner)
        return self._getitem_general(key)

    def _getitem_general(self, key):
        if not isinstance(key, tuple):
            key = (key,)
        shape = self.shape
        if any(k is Ellipsis for k in key):
            if sum(1 for k in key if k is Ellipsis) > 1:
                raise IndexError("an index can only have a single ellipsis")
            pos = next(i for i, k in enumerate(key) if k is Ellipsis)
            fill = len(shape) - (len(key) - 1)
            if fill < 0:
                raise IndexError("too many indices for array")
            key = key[:pos] + (slice(None),) * fill + key[pos + 1:]
        if len(key) > len(shape):
            raise IndexError("too many indices for array: array is %d-dimensional, "
                             "but %d were indexed" % (len(shape), len(key)))
        key = key + (slice(None),) * (len(shape) - len(key))
        strides = self._strides()
        offset = 0
        new_shape, new_strides = [], []
        for ax, k in enumerate(key):
            n = shape[ax]
            if isinstance(k, (int, np.integer)):
                k = int(k)
                if k < 0:
                    k += n
                if not 0 <= k < n:
                    raise IndexError("index out of bounds for axis %d with size %d" % (ax, n))
                offset += k * strides[ax]
            elif isinstance(k, slice):
                if k.step not in (None, 1):
                    raise NotImplementedError("DeviceArray slices must have step 1")
                start, stop, _ = k.indices(n)
                length = max(0, stop - start)
                if length:
                    offset += start * strides[ax]
                new_shape.append(length)
                new_strides.append(strides[ax])
            else:
                raise IndexError("DeviceArray indices must be integers or slices, not %s"
                                 % type(k).__name__)
        return _view(self, offset, tuple(new_shape), new_strides, key)

    def _strides(self):
        """Element strides (dense, C order)."""
        strides = [0] * len(self.shape)
        acc = 1
        for ax in range(len(self.shape) - 1, -1, -1):
            strides[ax] = acc
            acc *= self.shape[ax]
        return strides

    def _address(self):
        return self.ptr

    pitch = None      # dense: rows follow each other without gaps


class PitchedViewError(TypeError):
    """A row-pitched view reached code that needs a dense array."""


class PitchedDeviceArray(DeviceArray):
    """A view made of contiguous runs of ``run`` elements that lie ``pitch`` elements apart.

    brainstorm lets several layers write side by side into one hub and hands each of
    them the feature slice ``hub[:, :, a:b]`` (buffer_structure.py:232-245), reshaped
    to the layer's own feature shape (an image layer gets ``(T, B, H, W, C)`` whose
    H*W*C elements are one run); NumPy addresses such a slice with strides. Here the
    trailing axes whose sizes multiply to ``run`` are dense, and the axes in front of
    them count the runs ("rows") in C order. A handler created with
    ``pitched_views=True`` passes such views to kernels that take the pitch, or moves
    them through a dense temporary where no such kernel exists.
    Reading ``ptr`` raises, so that no code path can mistake the view for a dense array.
    """

    __slots__ = ("_base", "pitch", "run")

    def __init__(self, base, shape, pitch, owner, handler, run=None):
        # DeviceArray.__init__ would assign self.ptr, which is read-only here
        self._base = base
        self.shape = shape
        self.size = _prod(shape)
        self.pitch = pitch
        self.run = shape[-1] if run is None else run
        self._owner = owner
        self._handler = handler
        self._steps = None

    @property
    def ptr(self):
        raise PitchedViewError(
            "row-pitched view of shape %r (runs of %d, pitch %d) used where a dense array is needed"
            % (self.shape, self.run, self.pitch))

    @property
    def rows(self):
        return self.size // self.run if self.run else 0

    def _address(self):
        return self._base

    def _strides(self):
        strides = [1] * len(self.shape)
        acc = 1
        ax = len(self.shape) - 1
        while ax >= 0 and acc < self.run:          # the axes of one run: dense
            strides[ax] = acc
            acc *= self.shape[ax]
            ax -= 1
        while ax >= 0 and self.shape[ax] == 1 and acc == self.run:
            strides[ax] = acc                      # size-1 axes next to the run: any stride serves
            ax -= 1
        acc = self.pitch
        for k in range(ax, -1, -1):
            strides[k] = acc
            acc *= self.shape[k]
        return strides

    def __repr__(self):
        return "PitchedDeviceArray(shape=%r, run=%d, pitch=%d, ptr=0x%x)" % (self.shape, self.run, self.pitch,
                                                                            self._base)

    def __getitem__(self, key):
        return self._getitem_general(key)

    def reshape(self, *new_shape):
        if len(new_shape) == 1 and not isinstance(new_shape[0], (int, np.integer)):
            new_shape = tuple(new_shape[0])
        new_shape = tuple(int(s) for s in new_shape)
        if -1 in new_shape:
            known = _prod(s for s in new_shape if s != -1)
            if new_shape.count(-1) > 1 or known == 0 or self.size % known:
                raise ValueError("cannot reshape array of size %d into shape %r" % (self.size, new_shape))
            new_shape = tuple(self.size // known if s == -1 else s for s in new_shape)
        if any(s < 0 for s in new_shape) or _prod(new_shape) != self.size:
            raise ValueError("cannot reshape array of size %d into shape %r" % (self.size, new_shape))
        # some trailing axes of the new shape must make up exactly one run
        acc = 1
        for s in reversed(new_shape):
            if acc >= self.run:
                break
            acc *= s
        if acc != self.run:
            raise NotImplementedError("a row-pitched view can only be reshaped within its runs of %d elements and "
                                      "over the axes that count them (%r -> %r)" % (self.run, self.shape, new_shape))
        return PitchedDeviceArray(self._base, new_shape, self.pitch, self._owner, self._handler, self.run)


def _view(parent, offset, shape, strides, key):
    """The view of `parent` at element `offset` with the given shape and element strides:
    dense if it is, row-pitched if the parent's handler allows that, else an error."""
    base = parent._address()
    ptr = base + offset * ITEMSIZE if base else 0
    owner, handler = parent._owner, parent._handler
    if _prod(shape) == 0 or not shape:
        return DeviceArray(ptr if _prod(shape) else 0, shape, owner, handler)
    # the longest dense suffix of axes is the contiguous run
    run, k = 1, len(shape)
    while k > 0 and (shape[k - 1] == 1 or strides[k - 1] == run):
        run *= shape[k - 1]
        k -= 1
    # the axes in front of it must advance like the rows of one matrix: stride = pitch * rows below
    pitch = None
    below = 1
    ok = True
    for n, st in zip(reversed(shape[:k]), reversed(strides[:k])):
        if n != 1:
            if pitch is None:
                if st % below:
                    ok = False
                pitch = st // below
            elif st != pitch * below:
                ok = False
        below *= n
    if not ok:
        raise NotImplementedError("slicing %r out of shape %r leaves more than a row pitch; "
                                  "such views are not supported" % (key, parent.shape))
    if pitch is None or pitch == run:
        return DeviceArray(ptr, shape, owner, handler)
    if not getattr(handler, "pitched_views", False):
        raise NotImplementedError(
            "slicing %r out of shape %r needs a row pitch; create the handler with "
            "pitched_views=True to work on such views" % (key, parent.shape))
    return PitchedDeviceArray(ptr, shape, pitch, owner, handler, run)
