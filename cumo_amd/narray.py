"""Host-side mirror of the Cumo::NArray classes for the array hot path.

This is the caller of the C-ABI: what the Ruby extension's generated method
bodies and ndloop do on the host, restated so that the parity tests read like
the reference's own tests. Per operation it

  * resolves broadcasting over the operands' views
    (reference: ext/cumo/narray/ndloop.c:493-595),
  * allocates the result from the device pool
    (reference: ext/cumo/narray/narray.c:710-771, gen/tmpl/allocate.c:14-39),
  * fills the launch descriptors the way the generated iterators do
    (reference: ext/cumo/include/cumo/indexer.h:114-220, gen/tmpl/binary.c:114-176,
    gen/tmpl/accum.c:41-45), and
  * calls the launcher of that name in libcumo_hip.so.

Nothing here computes on the CPU. Arrays live in device memory from the pool and
come back to the host only through explicit copies (`to_numpy`, `extract_cpu`).

Classes: SFloat, DFloat, Int32, Bit (and Int64/UInt64 as result holders, which is
what Int32#sum and Bit#count_true answer). `NMath` carries the module functions.
"""
import ctypes as C
import numbers

import numpy as np

from . import _lib
from ._lib import (MAX_DIM, BitIArray, BitIArrayStridx, IArray, IArrayStridx, Indexer, ReductionArg, ShapeError,
                   call, fn)

P = C.POINTER


class _Buffer:
    """One pool allocation; returned to the pool when the last view dies
    (reference: gen/tmpl/alloc_func.c:33-56)."""

    __slots__ = ("ptr", "nbytes")

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        self.ptr = call(_lib.lib.cumo_cuda_runtime_malloc, self.nbytes) if nbytes else None
        if nbytes and not self.ptr:
            raise _lib.OutOfMemoryError("allocation of %d bytes failed" % nbytes)

    def __del__(self):
        try:
            if self.ptr:
                _lib.lib.cumo_cuda_runtime_free_no_raise(self.ptr)
                self.ptr = None
        except Exception:
            pass


def _prod(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


def _contiguous_strides(shape, unit):
    st = [0] * len(shape)
    s = unit
    for d in range(len(shape) - 1, -1, -1):
        st[d] = s
        s *= int(shape[d])
    return tuple(st)


def _make_indexer(shape):
    ix = Indexer()
    if len(shape) > MAX_DIM:
        raise ValueError("too many dimensions")
    ix.ndim = len(shape)
    ix.total_size = _prod(shape)
    for d, s in enumerate(shape):
        ix.shape[d] = int(s)
    return ix


def _broadcast_shapes(*shapes):
    """reference: ndloop.c:493-516 (right-aligned, a size-1 dimension repeats)."""
    nd = max(len(s) for s in shapes)
    out = [1] * nd
    for s in shapes:
        off = nd - len(s)
        for k, n in enumerate(s):
            i = off + k
            if n != 1:
                if out[i] == 1:
                    out[i] = n
                elif out[i] != n:
                    raise ShapeError("shape1[%d](=%d) != shape2[%d](=%d)" % (i, out[i], k, n))
    return tuple(out)


class NArray:
    """Base of the typed arrays. shape/strides/offset describe a view into a
    pool buffer; strides and offset are bytes (bits for Bit)."""

    type_name = None   # 'sfloat', ... as it appears in launcher symbols
    np_dtype = None
    elmsz = 0          # bytes per element; Bit overrides addressing
    ctype = None
    is_float = False

    # ---- construction ----------------------------------------------------
    def __init__(self, *shape, _buffer=None, _offset=0, _strides=None):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        self.shape = tuple(int(s) for s in shape)
        if len(self.shape) > MAX_DIM:
            raise ValueError("too many dimensions")
        if _buffer is None:
            _buffer = _Buffer(self._storage_bytes(_prod(self.shape)))
        self._buf = _buffer
        self._offset = int(_offset)
        self._strides = tuple(_strides) if _strides is not None else _contiguous_strides(self.shape, self._unit())

    @classmethod
    def _unit(cls):
        return cls.elmsz

    @classmethod
    def _storage_bytes(cls, n):
        return n * cls.elmsz

    @classmethod
    def new(cls, *shape):
        return cls(*shape)

    @classmethod
    def zeros(cls, *shape):
        a = cls(*shape)
        if a._buf.nbytes:
            call(_lib.lib.cumo_hip_memset, a._buf.ptr, 0, a._buf.nbytes)
        return a

    @classmethod
    def cast(cls, data):
        """Host data in (the from_binary / cast(Array) route of the reference,
        ext/cumo/narray/narray.c:1391-1461): one synchronous copy to the device."""
        if isinstance(data, NArray):
            if type(data) is cls:
                return data
            return data._cast_to(cls)
        arr = np.ascontiguousarray(np.asarray(data, dtype=cls.np_dtype))
        a = cls(*arr.shape)
        if arr.nbytes:
            call(_lib.lib.cumo_hip_memcpy_h2d, a._buf.ptr, arr.ctypes.data, arr.nbytes)
        return a

    from_numpy = cast

    # ---- properties --------------------------------------------------------
    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        return _prod(self.shape)

    def __len__(self):
        return self.shape[0] if self.shape else 0

    def is_contiguous(self):
        return self._strides == _contiguous_strides(self.shape, self._unit()) or self.size <= 1

    contiguous_p = is_contiguous

    def _ptr(self):
        return (self._buf.ptr or 0) + self._offset

    def _view(self, shape, strides, offset):
        return type(self)(*shape, _buffer=self._buf, _offset=offset, _strides=strides)

    # ---- views (reference: narray/index.c:445-516,602-609, narray/data.c:272-297)
    def __getitem__(self, key):
        if not isinstance(key, tuple):
            key = (key,)
        if any(k is Ellipsis for k in key):
            i = next(j for j, k in enumerate(key) if k is Ellipsis)
            fill = self.ndim - (len(key) - 1)
            key = key[:i] + (slice(None),) * fill + key[i + 1:]
        if len(key) > self.ndim:
            raise IndexError("too many indices")
        key = key + (slice(None),) * (self.ndim - len(key))
        shape, strides, offset = [], [], self._offset
        for n, st, k in zip(self.shape, self._strides, key):
            if k is True:
                k = slice(None)
            if isinstance(k, numbers.Integral):
                k = int(k)
                if k < 0:
                    k += n
                if not 0 <= k < n:
                    raise IndexError("index out of range")
                offset += k * st
            elif isinstance(k, slice):
                start, stop, step = k.indices(n)
                cnt = len(range(start, stop, step))
                offset += start * st
                shape.append(cnt)
                strides.append(st * step)
            else:
                raise TypeError("index arrays are outside this path")
        return self._view(shape, strides, offset)

    def transpose(self, *axes):
        if len(axes) == 1 and isinstance(axes[0], (tuple, list)):
            axes = tuple(axes[0])
        if not axes:
            axes = tuple(range(self.ndim - 1, -1, -1))
        axes = tuple(a + self.ndim if a < 0 else a for a in axes)
        if sorted(axes) != list(range(self.ndim)):
            raise ValueError("invalid axes")
        return self._view([self.shape[a] for a in axes], [self._strides[a] for a in axes], self._offset)

    def swapaxes(self, a, b):
        ax = list(range(self.ndim))
        ax[a], ax[b] = ax[b], ax[a]
        return self.transpose(*ax)

    def reverse(self, *axes):
        axes = [a + self.ndim if a < 0 else a for a in (axes or range(self.ndim))]
        strides, offset = list(self._strides), self._offset
        for a in axes:
            offset += (self.shape[a] - 1) * strides[a]
            strides[a] = -strides[a]
        return self._view(self.shape, strides, offset)

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        src = self if self.is_contiguous() else self.copy()
        shape = list(shape)
        if -1 in shape:
            i = shape.index(-1)
            rest = _prod(s for s in shape if s != -1)
            shape[i] = src.size // rest if rest else 0
        if _prod(shape) != src.size:
            raise ShapeError("reshape size mismatch")
        return src._view(shape, _contiguous_strides(shape, self._unit()), src._offset)

    def expand_dims(self, axis):
        shape, strides = list(self.shape), list(self._strides)
        if axis < 0:
            axis += self.ndim + 1
        shape.insert(axis, 1)
        strides.insert(axis, 0)
        return self._view(shape, strides, self._offset)

    # ---- descriptors -------------------------------------------------------
    def _iarray(self, loop_shape):
        """cumo_na_make_iarray over the broadcast loop shape: ptr + view offset,
        byte step per loop dimension, 0 where this operand repeats."""
        ia = IArray()
        ia.ptr = self._ptr()
        off = len(loop_shape) - self.ndim
        for k, (n, st) in enumerate(zip(self.shape, self._strides)):
            ia.step[off + k] = st if n != 1 else 0
        return ia

    # ---- host read-back ------------------------------------------------------
    def copy(self):
        """Contiguous copy of any view (reference: narray/data.c:84-113)."""
        out = type(self)(*self.shape)
        if self.size:
            ix = _make_indexer(self.shape)
            a1, a2 = self._iarray(self.shape), out._iarray(self.shape)
            f = fn("cumo_iter_copy_bytes_indexer_kernel_launch", None, [P(IArray), P(IArray), P(Indexer), C.c_ssize_t])
            call(f, C.byref(a1), C.byref(a2), C.byref(ix), self.elmsz)
        return out

    dup = copy

    def to_numpy(self):
        src = self if (self.is_contiguous() and self._strides == _contiguous_strides(self.shape, self._unit())) else self.copy()
        out = np.empty(self.shape, dtype=self.np_dtype)
        if out.nbytes:
            call(_lib.lib.cumo_hip_memcpy_d2h, out.ctypes.data, src._ptr(), out.nbytes)
        return out

    def to_a(self):
        return self.to_numpy().tolist()

    def extract_cpu(self):
        """reference: gen/tmpl/extract_cpu.c:17-23 -- a 0-dim array answers its element."""
        if self.size != 1:
            raise ValueError("not a 0-dim / single-element array")
        return self.to_numpy().reshape(()).item()

    def __float__(self):
        return float(self.extract_cpu())

    def __int__(self):
        return int(self.extract_cpu())

    def __repr__(self):
        return "%s%r" % (type(self).__name__, self.shape)

    # ---- casts ----------------------------------------------------------------
    def _cast_to(self, cls):
        if isinstance(self, Bit) or cls is Bit:
            raise TypeError("Bit casts are outside this path")
        out = cls(*self.shape)
        if self.size:
            ix = _make_indexer(self.shape)
            a1, a2 = out._iarray(self.shape), self._iarray(self.shape)
            f = fn("cumo_iter_%s_store_%s_kernel_launch" % (cls.type_name, self.type_name), None,
                   [P(IArray), P(IArray), P(Indexer)])
            call(f, C.byref(a1), C.byref(a2), C.byref(ix))
        return out

    def store(self, src):
        """self[...] = src with broadcasting and cast (reference: gen/tmpl/store_from.c)."""
        if not isinstance(src, NArray):
            return self.fill(src)
        shape = _broadcast_shapes(self.shape, src.shape)
        if shape != self.shape:
            raise ShapeError("cannot broadcast to the destination")
        ix = _make_indexer(shape)
        a1, a2 = self._iarray(shape), src._iarray(shape)
        f = fn("cumo_iter_%s_store_%s_kernel_launch" % (self.type_name, src.type_name), None,
               [P(IArray), P(IArray), P(Indexer)])
        call(f, C.byref(a1), C.byref(a2), C.byref(ix))
        return self

    def fill(self, value):
        if self.size:
            ix = _make_indexer(self.shape)
            a1 = self._iarray(self.shape)
            f = fn("cumo_iter_%s_fill_kernel_launch" % self.type_name, None, [P(IArray), P(Indexer), self.ctype])
            call(f, C.byref(a1), C.byref(ix), self.ctype(value))
        return self


# ---------------------------------------------------------------------------
# numeric arrays
# ---------------------------------------------------------------------------
_UPCAST_RANK = {"int32": 0, "sfloat": 1, "dfloat": 2}


def _upcast(a, b):
    """reference: gen/def/{sfloat,dfloat,int32}.rb upcast tables."""
    return a if _UPCAST_RANK[a.type_name] >= _UPCAST_RANK[b.type_name] else b


class _Numeric(NArray):
    sum_type = None  # class of the result of sum/prod

    # -- binary ---------------------------------------------------------------
    def _binary(self, other, op, scalar_is_left=False):
        cls = type(self)
        if isinstance(other, numbers.Number):
            # reference: gen/tmpl/binary.c:184-209 -- the number rides in the launch
            if isinstance(other, float) and not cls.is_float:
                return self._cast_to(DFloat)._binary(other, op, scalar_is_left)
            out = cls(*self.shape)
            if self.size:
                ix = _make_indexer(self.shape)
                a1, a3 = self._iarray(self.shape), out._iarray(self.shape)
                f = fn("cumo_iter_%s_%s_s_kernel_launch" % (cls.type_name, op), None,
                       [P(IArray), cls.ctype, P(IArray), P(Indexer), P(C.c_int), C.c_int])
                flag = _lib.lib.cumo_cuda_runtime_error_flag_new() if not cls.is_float and op in ("div", "mod") else None
                call(f, C.byref(a1), cls.ctype(other), C.byref(a3), C.byref(ix), flag, 1 if scalar_is_left else 0)
                self._raise_if_flag(flag, ZeroDivisionError("error in NArray operation"))
            return out
        if not isinstance(other, _Numeric):
            return NotImplemented
        if scalar_is_left:
            return other._binary(self, op)
        up = _upcast(cls, type(other))
        a, b = (self if cls is up else self._cast_to(up)), (other if type(other) is up else other._cast_to(up))
        shape = _broadcast_shapes(a.shape, b.shape)
        out = up(*shape)
        if out.size:
            ix = _make_indexer(shape)
            a1, a2, a3 = a._iarray(shape), b._iarray(shape), out._iarray(shape)
            f = fn("cumo_iter_%s_%s_kernel_launch" % (up.type_name, op), None,
                   [P(IArray), P(IArray), P(IArray), P(Indexer), P(C.c_int)])
            flag = _lib.lib.cumo_cuda_runtime_error_flag_new() if not up.is_float and op in ("div", "mod") else None
            call(f, C.byref(a1), C.byref(a2), C.byref(a3), C.byref(ix), flag)
            self._raise_if_flag(flag, ZeroDivisionError("error in NArray operation"))
        return out

    @staticmethod
    def _raise_if_flag(flag, exc):
        # reference: gen/tmpl/binary.c:120-126 -- the caller reads the flag with a device sync
        if flag is not None and call(_lib.lib.cumo_cuda_runtime_error_flag_get, flag):
            raise exc

    def __add__(self, o): return self._binary(o, "add")
    def __radd__(self, o): return self._binary(o, "add", True)
    def __sub__(self, o): return self._binary(o, "sub")
    def __rsub__(self, o): return self._binary(o, "sub", True)
    def __mul__(self, o): return self._binary(o, "mul")
    def __rmul__(self, o): return self._binary(o, "mul", True)
    def __truediv__(self, o): return self._binary(o, "div")
    def __rtruediv__(self, o): return self._binary(o, "div", True)
    def __mod__(self, o): return self._binary(o, "mod")
    def __rmod__(self, o): return self._binary(o, "mod", True)

    # -- unary ----------------------------------------------------------------
    def _unary(self, op, flag_exc=None):
        out = type(self)(*self.shape)
        if self.size:
            ix = _make_indexer(self.shape)
            a1, a2 = self._iarray(self.shape), out._iarray(self.shape)
            f = fn("cumo_iter_%s_%s_kernel_launch" % (self.type_name, op), None, [P(IArray), P(IArray), P(Indexer), P(C.c_int)])
            flag = _lib.lib.cumo_cuda_runtime_error_flag_new() if flag_exc is not None else None
            call(f, C.byref(a1), C.byref(a2), C.byref(ix), flag)
            self._raise_if_flag(flag, flag_exc)
        return out

    def __neg__(self): return self._unary("minus")
    def minus(self): return self._unary("minus")
    def square(self): return self._unary("square")
    def sign(self): return self._unary("sign")

    def reciprocal(self):
        return self._unary("reciprocal", None if self.is_float else ZeroDivisionError("error in NArray operation"))

    def abs(self):
        return self._unary("abs", None if self.is_float else ValueError("cannot convert the minimum integer"))

    __abs__ = abs

    # -- comparisons into Bit ----------------------------------------------------
    def _compare(self, other, op, scalar_is_left=False):
        cls = type(self)
        if isinstance(other, numbers.Number):
            if isinstance(other, float) and not cls.is_float:
                return self._cast_to(DFloat)._compare(other, op, scalar_is_left)
            out = Bit(*self.shape)
            if self.size:
                ix = _make_indexer(self.shape)
                a1, a3 = self._iarray(self.shape), out._bit_iarray(self.shape)
                f = fn("cumo_iter_%s_%s_s_kernel_launch" % (cls.type_name, op), None,
                       [P(IArray), cls.ctype, P(BitIArray), P(Indexer), C.c_int])
                call(f, C.byref(a1), cls.ctype(other), C.byref(a3), C.byref(ix), 1 if scalar_is_left else 0)
            return out
        if not isinstance(other, _Numeric):
            return NotImplemented
        up = _upcast(cls, type(other))
        a, b = (self if cls is up else self._cast_to(up)), (other if type(other) is up else other._cast_to(up))
        shape = _broadcast_shapes(a.shape, b.shape)
        out = Bit(*shape)
        if out.size:
            ix = _make_indexer(shape)
            a1, a2, a3 = a._iarray(shape), b._iarray(shape), out._bit_iarray(shape)
            f = fn("cumo_iter_%s_%s_kernel_launch" % (up.type_name, op), None, [P(IArray), P(IArray), P(BitIArray), P(Indexer)])
            call(f, C.byref(a1), C.byref(a2), C.byref(a3), C.byref(ix))
        return out

    def eq(self, o): return self._compare(o, "eq")
    def ne(self, o): return self._compare(o, "ne")
    def gt(self, o): return self._compare(o, "gt")
    def ge(self, o): return self._compare(o, "ge")
    def lt(self, o): return self._compare(o, "lt")
    def le(self, o): return self._compare(o, "le")
    __gt__ = gt
    __ge__ = ge
    __lt__ = lt
    __le__ = le

    def nearly_eq(self, o):
        return self._compare(o, "nearly_eq" if self.is_float else "eq")

    # -- reductions ------------------------------------------------------------
    def _reduce_axes(self, axis):
        """reference: narray/narray.c:1733-1856 (axis: / negative axes wrap)."""
        if axis is None:
            return tuple(range(self.ndim))
        if isinstance(axis, numbers.Integral):
            axis = (axis,)
        out = []
        for a in axis:
            a = int(a)
            if a < 0:
                a += self.ndim
            if not 0 <= a < self.ndim:
                raise ValueError("dimension is out of range")
            if a not in out:
                out.append(a)
        return tuple(sorted(out))

    def _reduction_arg(self, axes, out, keepdims):
        """cumo_na_make_reduction_arg after ndloop has moved the reduce dims to
        the end (reference: indexer.h:189-220, ndloop.c:421-451)."""
        keep = [d for d in range(self.ndim) if d not in axes]
        order = keep + list(axes)
        arg = ReductionArg()
        arg.in_.ptr = self._ptr()
        arg.in_indexer.ndim = self.ndim
        arg.in_indexer.total_size = self.size
        for k, d in enumerate(order):
            arg.in_indexer.shape[k] = self.shape[d]
            arg.in_.step[k] = self._strides[d]
        arg.out_indexer.ndim = len(keep)
        arg.out_indexer.total_size = _prod(self.shape[d] for d in keep)
        for k, d in enumerate(keep):
            arg.out_indexer.shape[k] = self.shape[d]
        return arg, keep

    def _out_iarray(self, out, keep, keepdims):
        ia = IArray()
        ia.ptr = out._ptr()
        out_dims = keep if keepdims else list(range(len(keep)))
        for k, d in enumerate(out_dims):
            ia.step[k] = out._strides[d]
        return ia

    def _reduce(self, name, out_cls, axis=None, keepdims=False, nan=False, index_bits=None, pair=False):
        if self.size == 0 and name in ("min", "max", "ptp", "minmax", "argmin", "argmax", "min_index", "max_index"):
            raise ValueError("cannot get min/max of an empty array")
        axes = self._reduce_axes(axis)
        src = self
        if name in ("min_index", "max_index") and not self.is_contiguous():
            src = self.copy()  # reference: gen/tmpl/accum_index.c -- the answer indexes the view's own flattening
        keep = [d for d in range(src.ndim) if d not in axes]
        out_shape = [src.shape[d] if d in keep else 1 for d in range(src.ndim)] if keepdims else [src.shape[d] for d in keep]
        out = out_cls(*out_shape)
        out2 = out_cls(*out_shape) if pair else None
        arg, keep = src._reduction_arg(axes, out, keepdims)
        arg.out = src._out_iarray(out, keep, keepdims)
        sym = "cumo_%s_%s%s" % (src.type_name, name, "_nan" if (nan and src.is_float) else "")
        if index_bits:
            sym += "_int%d" % index_bits
        sym += "_kernel_launch"
        if pair:
            o2 = src._out_iarray(out2, keep, keepdims)
            f = fn(sym, None, [P(ReductionArg), P(IArray)])
            call(f, C.byref(arg), C.byref(o2))
            return out, out2
        f = fn(sym, None, [P(ReductionArg)])
        call(f, C.byref(arg))
        return out

    def sum(self, axis=None, keepdims=False, nan=False):
        return self._reduce("sum", self.sum_type or type(self), axis, keepdims, nan)

    def prod(self, axis=None, keepdims=False, nan=False):
        return self._reduce("prod", self.sum_type or type(self), axis, keepdims, nan)

    def min(self, axis=None, keepdims=False, nan=False):
        return self._reduce("min", type(self), axis, keepdims, nan)

    def max(self, axis=None, keepdims=False, nan=False):
        return self._reduce("max", type(self), axis, keepdims, nan)

    def ptp(self, axis=None, keepdims=False, nan=False):
        return self._reduce("ptp", type(self), axis, keepdims, nan)

    def minmax(self, axis=None, keepdims=False, nan=False):
        return self._reduce("minmax", type(self), axis, keepdims, nan, pair=True)

    def _index_cls(self):
        # reference: gen/tmpl/accum_arg.c:92-110
        return (Int64, 64) if self.size > 2 ** 31 - 1 else (Int32, 32)

    def argmin(self, axis=None, keepdims=False, nan=False):
        cls, bits = self._index_cls()
        return self._reduce("argmin", cls, axis, keepdims, nan, index_bits=bits)

    def argmax(self, axis=None, keepdims=False, nan=False):
        cls, bits = self._index_cls()
        return self._reduce("argmax", cls, axis, keepdims, nan, index_bits=bits)

    def min_index(self, axis=None, keepdims=False, nan=False):
        cls, bits = self._index_cls()
        return self._reduce("min_index", cls, axis, keepdims, nan, index_bits=bits)

    def max_index(self, axis=None, keepdims=False, nan=False):
        cls, bits = self._index_cls()
        return self._reduce("max_index", cls, axis, keepdims, nan, index_bits=bits)


class _Float(_Numeric):
    is_float = True

    def mean(self, axis=None, keepdims=False, nan=False):
        return self._reduce("mean", type(self), axis, keepdims, nan)

    def var(self, axis=None, keepdims=False, nan=False):
        return self._reduce("var", type(self), axis, keepdims, nan)

    def stddev(self, axis=None, keepdims=False, nan=False):
        return self._reduce("stddev", type(self), axis, keepdims, nan)

    def rms(self, axis=None, keepdims=False, nan=False):
        return self._reduce("rms", type(self), axis, keepdims, nan)

    def floor(self): return self._unary("floor")
    def round(self): return self._unary("round")
    def ceil(self): return self._unary("ceil")
    def trunc(self): return self._unary("trunc")
    def rint(self): return self._unary("rint")
    def copysign(self, o): return self._binary(o, "copysign")

    def _cond_unary(self, op):
        out = Bit(*self.shape)
        if self.size:
            ix = _make_indexer(self.shape)
            a1, a2 = self._iarray(self.shape), out._bit_iarray(self.shape)
            f = fn("cumo_iter_%s_%s_kernel_launch" % (self.type_name, op), None, [P(IArray), P(BitIArray), P(Indexer)])
            call(f, C.byref(a1), C.byref(a2), C.byref(ix))
        return out

    def isnan(self): return self._cond_unary("isnan")
    def isinf(self): return self._cond_unary("isinf")
    def isposinf(self): return self._cond_unary("isposinf")
    def isneginf(self): return self._cond_unary("isneginf")
    def isfinite(self): return self._cond_unary("isfinite")
    def signbit(self): return self._cond_unary("signbit")


class SFloat(_Float):
    type_name, np_dtype, elmsz, ctype = "sfloat", np.float32, 4, C.c_float


class DFloat(_Float):
    type_name, np_dtype, elmsz, ctype = "dfloat", np.float64, 8, C.c_double

    def kahan_sum(self, axis=None, keepdims=False, nan=False):
        return self._reduce("kahan_sum", DFloat, axis, keepdims, nan)


class Int64(NArray):
    """Result holder (Int32#sum, argmax over more than 2^31-1 elements)."""
    type_name, np_dtype, elmsz, ctype = "int64", np.int64, 8, C.c_int64


class UInt64(NArray):
    """Result holder (Bit#count_true)."""
    type_name, np_dtype, elmsz, ctype = "uint64", np.uint64, 8, C.c_uint64


class Int32(_Numeric):
    type_name, np_dtype, elmsz, ctype = "int32", np.int32, 4, C.c_int32
    sum_type = Int64

    def __and__(self, o): return self._binary(o, "bit_and")
    def __or__(self, o): return self._binary(o, "bit_or")
    def __xor__(self, o): return self._binary(o, "bit_xor")
    def __lshift__(self, o): return self._binary(o, "left_shift")
    def __rshift__(self, o): return self._binary(o, "right_shift")
    def __invert__(self): return self._unary("bit_not")
    def __floordiv__(self, o): return self._binary(o, "div")


# ---------------------------------------------------------------------------
# Bit
# ---------------------------------------------------------------------------
class Bit(NArray):
    """1 bit per element, LSB first in 32-bit words
    (reference: ext/cumo/include/cumo/narray.h:492-496, template.h:110-138).
    Strides and offset are in bits."""

    type_name, np_dtype, elmsz, ctype = "bit", np.uint8, 0, C.c_uint32

    @classmethod
    def _unit(cls):
        return 1

    @classmethod
    def _storage_bytes(cls, n):
        return ((n + 31) // 32) * 4  # reference: gen/tmpl/alloc_func.c:7-9

    @classmethod
    def cast(cls, data):
        arr = np.ascontiguousarray(np.asarray(data) != 0)
        a = cls(*arr.shape)
        n = arr.size
        if n:
            bits = np.packbits(arr.reshape(-1), bitorder="little")
            words = np.zeros(((n + 31) // 32) * 4, dtype=np.uint8)
            words[:bits.size] = bits
            call(_lib.lib.cumo_hip_memcpy_h2d, a._buf.ptr, words.ctypes.data, words.nbytes)
        return a

    from_numpy = cast

    def _bit_iarray(self, loop_shape):
        ia = BitIArray()
        ia.ptr = self._buf.ptr
        ia.pos = self._offset
        off = len(loop_shape) - self.ndim
        for k, (n, st) in enumerate(zip(self.shape, self._strides)):
            ia.step[off + k] = st if n != 1 else 0
        return ia

    def _bit_stridx(self, loop_shape):
        ia = BitIArrayStridx()
        ia.ptr = self._buf.ptr
        ia.pos = self._offset
        off = len(loop_shape) - self.ndim
        for k in range(len(loop_shape)):
            ia.stridx[k] = 1  # stride 0
        for k, (n, st) in enumerate(zip(self.shape, self._strides)):
            ia.stridx[off + k] = ((st if n != 1 else 0) << 1) | 1
        return ia

    def _iarray(self, loop_shape):
        raise TypeError("a Bit operand has no byte descriptor")

    def _raw_words(self):
        """All words of the underlying buffer, on the host."""
        nbytes = self._buf.nbytes
        words = np.zeros(nbytes // 4, dtype=np.uint32)
        if nbytes:
            call(_lib.lib.cumo_hip_memcpy_d2h, words.ctypes.data, self._buf.ptr, nbytes)
        return words

    def copy(self):
        out = Bit(*self.shape)
        if self.size:
            self._bit_op1("copy", out)
        return out

    def to_numpy(self):
        src = self if (self._offset == 0 and self._strides == _contiguous_strides(self.shape, 1)) else self.copy()
        words = src._raw_words()
        bits = np.unpackbits(words.view(np.uint8), bitorder="little")[:self.size]
        return bits.reshape(self.shape).astype(np.uint8)

    # reference: gen/tmpl_bit/binary.c:17-31 -- the word kernel when everything is flat
    def _flat(self):
        return self.ndim == 1 and self._strides[0] == 1

    def _bit_op1(self, op, out):
        ix = _make_indexer(self.shape)
        a1, a3 = self._bit_stridx(self.shape), out._bit_stridx(self.shape)
        f = fn("cumo_iter_bit_%s_kernel_launch" % op, None, [P(BitIArrayStridx), P(BitIArrayStridx), P(Indexer)])
        call(f, C.byref(a1), C.byref(a3), C.byref(ix))

    def _bit_op2(self, other, op):
        if not isinstance(other, Bit):
            return NotImplemented
        shape = _broadcast_shapes(self.shape, other.shape)
        out = Bit(*shape)
        if not out.size:
            return out
        if self._flat() and other._flat() and self.shape == other.shape:
            f = fn("cumo_iter_bit_%s_contiguous_kernel_launch" % op, None,
                   [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_uint64])
            call(f, self._buf.ptr + (self._offset // 32) * 4, self._offset % 32,
                 other._buf.ptr + (other._offset // 32) * 4, other._offset % 32, out._buf.ptr, 0, out.size)
            return out
        ix = _make_indexer(shape)
        a1, a2, a3 = self._bit_stridx(shape), other._bit_stridx(shape), out._bit_stridx(shape)
        f = fn("cumo_iter_bit_%s_kernel_launch" % op, None,
               [P(BitIArrayStridx), P(BitIArrayStridx), P(BitIArrayStridx), P(Indexer)])
        call(f, C.byref(a1), C.byref(a2), C.byref(a3), C.byref(ix))
        return out

    def __and__(self, o): return self._bit_op2(o, "and")
    def __or__(self, o): return self._bit_op2(o, "or")
    def __xor__(self, o): return self._bit_op2(o, "xor")
    def eq(self, o): return self._bit_op2(o, "eq")

    def __invert__(self):
        out = Bit(*self.shape)
        if self.size:
            self._bit_op1("not", out)
        return out

    def _count(self, name, axis, keepdims):
        """reference: gen/tmpl_bit/bit_count.c:9-68 and the host-walked loop of
        narray/ndloop.c:1569-1613: reduce dims go last, mergeable dims merge, the
        innermost run is one launch and the outer dims are walked on the host."""
        if self.size == 0:
            return 0
        nd = self.ndim
        if axis is None:
            axes = tuple(range(nd))
        else:
            axes = tuple(sorted({(a + nd if a < 0 else a) for a in ((axis,) if isinstance(axis, numbers.Integral) else axis)}))
        keep = [d for d in range(nd) if d not in axes]
        out_shape = [self.shape[d] if d in keep else 1 for d in range(nd)] if keepdims else [self.shape[d] for d in keep]
        out = UInt64.zeros(*out_shape)
        out_st = _contiguous_strides([self.shape[d] for d in keep], 8)
        # loop dims: kept dims (output step 8*...), then reduce dims (output step 0)
        dims = [(self.shape[d], self._strides[d], out_st[k]) for k, d in enumerate(keep)] + \
               [(self.shape[d], self._strides[d], 0) for d in axes]
        dims = [t for t in dims if t[0] != 1] or [(1, 0, 0)]
        merged = [dims[0]]
        for n, s1, s2 in dims[1:]:
            pn, ps1, ps2 = merged[-1]
            if ps1 == s1 * n and ps2 == s2 * n:
                merged[-1] = (pn * n, s1, s2)
            else:
                merged.append((n, s1, s2))
        inner_n, inner_s1, inner_s2 = merged[-1]
        outer = merged[:-1]
        f1 = fn("cumo_iter_bit_%s_stride_kernel_launch" % name, None,
                [C.c_size_t, C.c_void_p, C.c_void_p, C.c_ssize_t, C.c_uint64])
        f2 = fn("cumo_iter_bit_%s_stride_stride_kernel_launch" % name, None,
                [C.c_size_t, C.c_void_p, C.c_void_p, C.c_ssize_t, C.c_ssize_t, C.c_uint64])

        def walk(level, pos, optr):
            if level == len(outer):
                # CUMO_INIT_PTR_BIT_IDX: rebase the word pointer when the step is not negative
                a, p = self._buf.ptr, pos
                if inner_s1 >= 0:
                    a, p = a + (pos // 32) * 4, pos % 32
                if inner_s2 == 0:
                    call(f1, p, optr, a, inner_s1, inner_n)
                else:
                    call(f2, p, optr, a, inner_s1, inner_s2, inner_n)
                return
            n, s1, s2 = outer[level]
            for i in range(n):
                walk(level + 1, pos + i * s1, optr + i * s2)

        walk(0, self._offset, out._ptr())
        return out

    def count_true(self, axis=None, keepdims=False):
        return self._count("count_true", axis, keepdims)

    def count_false(self, axis=None, keepdims=False):
        return self._count("count_false", axis, keepdims)

    count = count_true
    count_1 = count_true
    count_0 = count_false

    def count_true_cpu(self):
        r = self.count_true()
        return int(r) if not isinstance(r, int) else r

    def _store_into(self, cls):
        """Bit -> 0/1 numbers (reference: gen/tmpl/store_bit.c)."""
        out = cls(*self.shape)
        if self.size:
            ix = _make_indexer(self.shape)
            a1 = IArrayStridx()
            a1.ptr = out._ptr()
            for k, st in enumerate(out._strides):
                a1.stridx[k] = (st << 1) | 1
            a2 = self._bit_stridx(self.shape)
            f = fn("cumo_iter_%s_store_bit_kernel_launch" % cls.type_name, None, [P(IArrayStridx), P(BitIArrayStridx), P(Indexer)])
            call(f, C.byref(a1), C.byref(a2), C.byref(ix))
        return out


# ---------------------------------------------------------------------------
# NMath
# ---------------------------------------------------------------------------
class _NMath:
    """Cumo::NMath (reference: narray/math.c:111-112 forwards to the dtype's
    Math module; function list gen/spec.rb:427-457)."""

    _ONE = ("sqrt cbrt log log2 log10 exp exp2 exp10 sin cos tan asin acos atan sinh cosh tanh "
            "asinh acosh atanh sinc erf erfc log1p expm1").split()
    _TWO = ("atan2", "hypot")

    def __getattr__(self, name):
        if name in self._ONE:
            return lambda x: self._call1(name, x)
        if name in self._TWO:
            return lambda x, y: self._call2(name, x, y)
        raise AttributeError(name)

    @staticmethod
    def _as_float(x):
        if isinstance(x, _Float):
            return x
        if isinstance(x, Int32):
            return x._cast_to(DFloat)
        raise TypeError("NMath needs a float array")

    def _call1(self, name, x):
        x = self._as_float(x)
        out = type(x)(*x.shape)
        if x.size:
            ix = _make_indexer(x.shape)
            a1, a2 = x._iarray(x.shape), out._iarray(x.shape)
            f = fn("cumo_iter_%s_math_s_%s_kernel_launch" % (x.type_name, name), None, [P(IArray), P(IArray), P(Indexer)])
            call(f, C.byref(a1), C.byref(a2), C.byref(ix))
        return out

    def _call2(self, name, x, y):
        if isinstance(x, numbers.Number) and isinstance(y, numbers.Number):
            raise TypeError("NMath needs an array operand")
        if isinstance(y, numbers.Number) or isinstance(x, numbers.Number):
            left = isinstance(x, numbers.Number)
            arr, sv = (y, x) if left else (x, y)
            arr = self._as_float(arr)
            out = type(arr)(*arr.shape)
            if arr.size:
                ix = _make_indexer(arr.shape)
                a1, a3 = arr._iarray(arr.shape), out._iarray(arr.shape)
                f = fn("cumo_iter_%s_math_s_%s_s_kernel_launch" % (arr.type_name, name), None,
                       [P(IArray), P(IArray), P(Indexer), arr.ctype, C.c_int])
                call(f, C.byref(a1), C.byref(a3), C.byref(ix), arr.ctype(sv), 1 if left else 0)
            return out
        x, y = self._as_float(x), self._as_float(y)
        up = _upcast(type(x), type(y))
        x, y = up.cast(x), up.cast(y)
        shape = _broadcast_shapes(x.shape, y.shape)
        out = up(*shape)
        if out.size:
            ix = _make_indexer(shape)
            a1, a2, a3 = x._iarray(shape), y._iarray(shape), out._iarray(shape)
            f = fn("cumo_iter_%s_math_s_%s_kernel_launch" % (up.type_name, name), None,
                   [P(IArray), P(IArray), P(IArray), P(Indexer)])
            call(f, C.byref(a1), C.byref(a2), C.byref(a3), C.byref(ix))
        return out


NMath = _NMath()
