"""Host-side mirror of the Cumo::NArray classes for the array hot path.

This is the object model only: a typed view (shape, strides, offset) of a
buffer from the device pool, the view-making methods, and one thin method per
operation that hands the views to the library's host launch layer
(include/cumo_hip_ndloop.h). Broadcasting, result allocation, the launch
descriptors and the choice of launcher all happen in the library
(cumo_amd/csrc/ndloop.cpp), as they happen in C in the reference
(ext/cumo/narray/ndloop.c, ext/cumo/narray/gen/tmpl/*.c); what stays here is what
Ruby itself does there: picking the method, coercing a Ruby number, parsing
`axis:`.

Nothing here computes on the CPU. Arrays live in device memory from the pool and
come back to the host only through explicit copies (`to_numpy`, `extract_cpu`).

Classes: SFloat, DFloat, Int32, Bit (and Int64/UInt64 as result holders, which is
what Int32#sum and Bit#count_true answer). `NMath` carries the module functions.
"""
import ctypes as C
import numbers

import numpy as np

from . import _lib
from ._lib import MAX_DIM, DimensionError, NArrayDesc, ShapeError, call

_L = _lib.lib


class _Buffer:
    """One pool allocation; returned to the pool when the last view dies
    (reference: gen/tmpl/alloc_func.c:33-56)."""

    __slots__ = ("ptr", "nbytes")

    def __init__(self, nbytes, ptr=None):
        self.nbytes = int(nbytes)
        if ptr is not None:
            self.ptr = ptr or None  # adopted from the library
            return
        self.ptr = call(_L.cumo_cuda_runtime_malloc, self.nbytes) if nbytes else None
        if nbytes and not self.ptr:
            raise _lib.OutOfMemoryError("allocation of %d bytes failed" % nbytes)

    def __del__(self):
        try:
            rec = _lib._recording
            if self.ptr and rec is not None:
                # released inside a recording: the recorded calls still name this memory
                rec.keep.append(_Buffer(self.nbytes, ptr=self.ptr))
                self.ptr = None
                return
            if self.ptr:
                _L.cumo_cuda_runtime_free_no_raise(self.ptr)
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


_CLASS_BY_CODE = {}


def _wrap(desc):
    """The array the library allocated for a result descriptor."""
    cls = _CLASS_BY_CODE[desc.type]
    shape = tuple(int(desc.shape[d]) for d in range(desc.ndim))
    buf = _Buffer(cls._storage_bytes(_prod(shape)), ptr=desc.ptr or 0)
    return cls(*shape, _buffer=buf)


def _run(f, *args, results=()):
    """Calls one host-layer function; `results` are the descriptors it may have
    allocated, released again if the call fails."""
    try:
        call(f, *args)
    except BaseException:
        for d in results:
            if d.ptr:
                _L.cumo_cuda_runtime_free_no_raise(d.ptr)
                d.ptr = None
        raise
    outs = [_wrap(d) for d in results]
    return outs[0] if len(outs) == 1 else outs


def _reduce_mask(ndim, axis):
    """`axis:` as the bit set ndloop takes (reference: narray/narray.c:1733-1856;
    negative axes wrap, out of range raises DimensionError)."""
    if axis is None:
        return 0
    if isinstance(axis, numbers.Integral):
        axis = (axis,)
    m = 0
    for a in axis:
        a = int(a)
        if a < 0:
            a += ndim
        if not 0 <= a < ndim:
            raise DimensionError("dimension is out of range")
        m |= 1 << a
    return m


def _is_index_array(k):
    # (a Bit array in a key of several entries selects the positions where it is set: narray/index.c:160-165)
    if isinstance(k, (list, np.ndarray, range)):
        return True
    return isinstance(k, NArray)


def _index_positions(k, n):
    """Positions one index array selects in a dimension of n elements, as the
    reference parses them on the host (narray/index.c:112-142,201-233): 1-D,
    negative values count from the end, out of range raises IndexError."""
    if isinstance(k, NArray) and type(k).__name__ == "Bit":
        # a Bit array stands for the positions where it is set (narray/index.c:156-166)
        if k.ndim != 1:
            raise IndexError("should be 1-d NArray")
        if k.size != n:
            raise IndexError("Bit-NArray size mismatch")
        k = k.where()
    arr = np.asarray(k.to_numpy() if isinstance(k, NArray) else (list(k) if isinstance(k, range) else k))
    if arr.size == 0:
        return np.zeros(0, dtype=np.uint64)
    if arr.ndim != 1:
        raise IndexError("index array should be 1-dimensional")
    if arr.dtype.kind not in "iu":
        if arr.dtype.kind == "f" and np.all(arr == np.floor(arr)):
            arr = arr.astype(np.int64)
        else:
            raise IndexError("index array must hold integers")
    arr = arr.astype(np.int64)
    arr = np.where(arr < 0, arr + n, arr)
    if np.any((arr < 0) | (arr >= n)):
        raise IndexError("index array value out of range (size %d)" % n)
    return arr.astype(np.uint64)


def _upload_index(pos):
    buf = _Buffer(8 * max(len(pos), 1))
    if len(pos):
        pos = np.ascontiguousarray(pos, dtype=np.uint64)
        call(_L.cumo_hip_copy_from_host, buf.ptr, pos.ctypes.data, pos.nbytes)
    return buf


def _index_launchers():
    v, sz, ss, u64 = C.c_void_p, C.c_size_t, C.c_ssize_t, C.c_uint64
    P = C.POINTER
    return {
        "aref_nadata_index_stride": _lib.fn("cumo_na_index_aref_nadata_index_stride_kernel_launch", None, [v, ss, u64]),
        "aref_naview_index_stride": _lib.fn("cumo_na_index_aref_naview_index_stride_kernel_launch", None, [v, ss, u64]),
        "aref_naview_index_stride_last": _lib.fn("cumo_na_index_aref_naview_index_stride_last_kernel_launch", None, [v, ss, sz, u64]),
        "at_nadata_index_stride_add": _lib.fn("cumo_na_index_at_nadata_index_stride_add_kernel_launch", None, [v, v, ss, u64]),
        "at_nadata_index_beg_step_stride": _lib.fn("cumo_na_index_at_nadata_index_beg_step_stride_kernel_launch", None, [v, sz, ss, ss, u64]),
        "at_nadata_index_beg_step_stride_add": _lib.fn("cumo_na_index_at_nadata_index_beg_step_stride_add_kernel_launch", None, [v, sz, ss, ss, u64]),
        "copy_bytes": _lib.fn("cumo_iter_copy_bytes_kernel_launch", None, [v, v, ss, ss, v, v, u64, ss]),
        "copy_to_buffer": _lib.fn("cumo_ndloop_copy_to_buffer_kernel_launch", None, [P(_lib.IArrayStridx), P(_lib.Indexer), v, sz]),
        "copy_from_buffer": _lib.fn("cumo_ndloop_copy_from_buffer_kernel_launch", None, [P(_lib.IArrayStridx), P(_lib.Indexer), v, sz]),
    }


_IX = _index_launchers()


class NArray:
    """Base of the typed arrays. shape/strides/offset describe a view into a
    pool buffer; strides and offset are bytes (bits for Bit)."""

    type_name = None   # 'sfloat', ... as it appears in launcher symbols
    type_code = None   # CUMO_HIP_SFLOAT, ...
    np_dtype = None
    elmsz = 0          # bytes per element; Bit overrides addressing
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
        return int(_L.cumo_hip_na_storage_bytes(cls.type_code, n))

    @classmethod
    def new(cls, *shape):
        return cls(*shape)

    @classmethod
    def zeros(cls, *shape):
        a = cls(*shape)
        if a._buf.nbytes:
            call(_L.cumo_hip_memset, a._buf.ptr, 0, a._buf.nbytes)
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
            call(_L.cumo_hip_copy_from_host, a._buf.ptr, arr.ctypes.data, arr.nbytes)
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

    def _desc(self):
        """This view as the library's cumo_hip_narray_t."""
        d = NArrayDesc()
        d.type = self.type_code
        d.ndim = len(self.shape)
        d.ptr = self._buf.ptr
        d.offset = self._offset
        for k, (n, st) in enumerate(zip(self.shape, self._strides)):
            d.shape[k] = n
            d.stride[k] = st
        return d

    # ---- views (reference: narray/index.c:445-516,602-609, narray/data.c:272-297)
    def _expand_key(self, key):
        if not isinstance(key, tuple):
            key = (key,)
        if any(k is Ellipsis for k in key):
            i = next(j for j, k in enumerate(key) if k is Ellipsis)
            fill = self.ndim - (len(key) - 1)
            key = key[:i] + (slice(None),) * fill + key[i + 1:]
        if len(key) > self.ndim:
            raise IndexError("too many indices")
        return key + (slice(None),) * (self.ndim - len(key))

    def __getitem__(self, key):
        if isinstance(key, NArray) and type(key).__name__ == "Bit":
            return key.mask(self)  # a[mask]: the elements where the mask is set
        key = self._expand_key(key)
        if any(_is_index_array(k) for k in key):
            return self._gather(key)
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
                raise TypeError("unsupported index %r" % (k,))
        return self._view(shape, strides, offset)

    def __setitem__(self, key, value):
        """a[key] = value: a store into the view, or a scatter when the key holds
        index arrays (reference: gen/tmpl/aset.c, narray/ndloop.c:1316)."""
        if isinstance(key, NArray) and type(key).__name__ == "Bit" and (key.ndim != 1 or self.ndim != 1):
            raise TypeError("a store through a mask of several dimensions is outside this path")
        key = self._expand_key(key)
        if any(_is_index_array(k) for k in key):
            return self._scatter(key, value)
        self[key].store(value)

    # ---- index arrays (reference: narray/index.c:460-614 builds the view,
    # narray/ndloop.c:1251-1330 stages it through a contiguous buffer)
    def _stridx_view(self, key):
        """The view a key with index arrays selects, as the launcher's descriptor:
        one device array of byte offsets per indexed dimension, a stride for the rest.
        Each indexed dimension selects independently (an outer product, not numpy's
        zipped fancy indexing). Returns (descriptor, indexer, shape, keep-alives)."""
        if type(self).__name__ == "Bit":
            raise TypeError("index arrays on Bit are outside this path")
        a = _lib.IArrayStridx()
        shape, keep, offset, d = [], [], self._offset, 0
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
                continue
            if isinstance(k, slice):
                start, stop, step = k.indices(n)
                shape.append(len(range(start, stop, step)))
                offset += start * st
                a.stridx[d] = ((st * step) << 1) | 1
            else:
                pos = _index_positions(k, n)
                buf = _upload_index(pos)
                keep.append(buf)
                if len(pos):
                    if st < 0:
                        # a reversed dimension counts from its far end (index.c:580-590)
                        offset += st * (n - 1)
                        call(_IX["aref_naview_index_stride_last"], buf.ptr, -st, n - 1, len(pos))
                    else:
                        call(_IX["aref_naview_index_stride"], buf.ptr, st, len(pos))
                shape.append(len(pos))
                a.stridx[d] = buf.ptr or 0
            d += 1
        a.ptr = (self._buf.ptr or 0) + offset
        ix = _lib.Indexer()
        ix.ndim = len(shape)
        ix.total_size = _prod(shape)
        for j, m in enumerate(shape):
            ix.shape[j] = m
        return a, ix, shape, keep

    def _gather(self, key):
        a, ix, shape, keep = self._stridx_view(key)
        out = type(self)(*shape)
        if out.size:
            call(_IX["copy_to_buffer"], C.byref(a), C.byref(ix), out._buf.ptr, self.elmsz)
        del keep
        return out

    def _scatter(self, key, value):
        a, ix, shape, keep = self._stridx_view(key)
        if (type(value) is type(self) and value.shape == tuple(shape)
                and value._strides == _contiguous_strides(value.shape, self._unit())):
            tmp = value  # already the contiguous buffer the scatter reads
        else:
            tmp = type(self)(*shape)
            tmp.store(value)
        if tmp.size:
            call(_IX["copy_from_buffer"], C.byref(a), C.byref(ix), tmp._ptr(), self.elmsz)
        del keep

    def at(self, *keys):
        """Elements at zipped positions: a.at([0, 1], [2, 3]) answers a[0, 2] and
        a[1, 3] as a 1-D array (reference: narray/index.c:622-682,842-870). A key is an
        index array or a range / slice; all must select the same number of positions."""
        if type(self).__name__ == "Bit":
            raise TypeError("index arrays on Bit are outside this path")
        if len(keys) != self.ndim:
            raise IndexError("the number of arguments must equal the number of dimensions")
        sel = []
        for k, n in zip(keys, self.shape):
            if isinstance(k, range):
                k = slice(k.start, k.stop, k.step)
            if isinstance(k, slice):
                start, stop, step = k.indices(n)
                sel.append((None, start, step, len(range(start, stop, step))))
            else:
                pos = _index_positions(k, n)
                sel.append((pos, 0, 0, len(pos)))
        size = sel[-1][3] if sel else 0
        if size == 0:
            raise ShapeError("cannot get element of empty array")
        if any(s[3] != size for s in sel):
            raise ShapeError("index array sizes mismatch")
        # the index array accumulates from the last dimension to the first
        last_pos = sel[-1][0]
        index = _upload_index(last_pos) if last_pos is not None else _Buffer(8 * size)
        offset = self._offset
        for i in range(self.ndim - 1, -1, -1):
            pos, beg, step, _ = sel[i]
            st, n = self._strides[i], self.shape[i]
            first = i == self.ndim - 1
            if pos is not None:
                if st < 0 and first:
                    # a reversed dimension counts from its far end (index.c:745-754)
                    offset += st * (n - 1)
                    call(_IX["aref_naview_index_stride_last"], index.ptr, -st, n - 1, size)
                elif first:
                    call(_IX["aref_nadata_index_stride"], index.ptr, st, size)
                else:
                    other = _upload_index(pos)
                    call(_IX["at_nadata_index_stride_add"], index.ptr, other.ptr, st, size)
            else:
                offset += beg * st
                name = "at_nadata_index_beg_step_stride" if first else "at_nadata_index_beg_step_stride_add"
                call(_IX[name], index.ptr, 0, step, st, size)
        out = type(self)(size)
        call(_IX["copy_bytes"], (self._buf.ptr or 0) + offset, out._buf.ptr, 0, self.elmsz, index.ptr, None, size, self.elmsz)
        return out

    def diagonal(self, offset=0, axes=(-2, -1)):
        """View of a diagonal as the last dimension (reference: narray/data.c:649-820;
        for views without index arrays it is stride arithmetic only)."""
        if self.ndim < 2:
            raise DimensionError("less than 2-d array")
        ax = [a + self.ndim if a < 0 else a for a in axes]
        if len(ax) != 2 or ax[0] == ax[1] or not all(0 <= a < self.ndim for a in ax):
            raise ValueError("invalid axes")
        k0, k1 = (0, offset) if offset >= 0 else (-offset, 0)
        n0, n1 = self.shape[ax[0]], self.shape[ax[1]]
        if k0 >= n0 or k1 >= n1:
            raise ShapeError("invalid diagonal offset(%d) for the shape" % offset)
        length = min(n0 - k0, n1 - k1)
        rest = [d for d in range(self.ndim) if d not in ax]
        shape = [self.shape[d] for d in rest] + [length]
        strides = [self._strides[d] for d in rest] + [self._strides[ax[0]] + self._strides[ax[1]]]
        return self._view(shape, strides, self._offset + k0 * self._strides[ax[0]] + k1 * self._strides[ax[1]])

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

    # ---- copies, casts, stores ------------------------------------------------
    def copy(self):
        """Contiguous copy of any view (reference: narray/data.c:84-113)."""
        x, z = self._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_copy, C.byref(x), C.byref(z), results=(z,))

    dup = copy

    def _cast_to(self, cls):
        out = cls(*self.shape)
        out.store(self)
        return out

    def store(self, src):
        """self[...] = src with broadcasting and cast (reference: gen/tmpl/store_from.c, store_bit.c)."""
        if not isinstance(src, NArray):
            return self.fill(src)
        d, s = self._desc(), src._desc()
        _run(_L.cumo_hip_na_store, C.byref(d), C.byref(s))
        return self

    def fill(self, value):
        d = self._desc()
        _run(_L.cumo_hip_na_fill, C.byref(d), float(value))
        return self

    def seq(self, beg=0, step=1):
        """self's elements in row-major order become beg + step * i (reference: gen/tmpl/seq.c:77-107)."""
        d = self._desc()
        _run(_L.cumo_hip_na_seq, C.byref(d), float(beg), float(step))
        return self

    indgen = seq

    def logseq(self, beg, step, base=10):
        """base ** (beg + step * i), float types only (reference: gen/tmpl/logseq.c)."""
        d = self._desc()
        _run(_L.cumo_hip_na_logseq, C.byref(d), float(beg), float(step), float(base))
        return self

    def eye(self, element=1, offset=0):
        """`element` on the diagonal `offset` away from the main one of every matrix of the last
        two dimensions, zero elsewhere (reference: gen/tmpl/eye.c:52-107)."""
        d = self._desc()
        _run(_L.cumo_hip_na_eye, C.byref(d), float(element), int(offset))
        return self

    # ---- host read-back and ingest ------------------------------------------------
    def to_numpy(self):
        out = np.empty(self.shape, dtype=self.np_dtype)
        if out.nbytes:
            d = self._desc()
            call(_L.cumo_hip_na_to_host, C.byref(d), out.ctypes.data, out.nbytes)
        return out

    def byte_size(self):
        return self.size * self.elmsz

    def to_binary(self):
        """The elements' bytes in row-major order (reference: narray/narray.c:1530-1560)."""
        out = bytearray(self.byte_size())
        if out:
            d = self._desc()
            call(_L.cumo_hip_na_to_host, C.byref(d), (C.c_char * len(out)).from_buffer(out), len(out))
        return bytes(out)

    to_string = to_binary

    @classmethod
    def from_binary(cls, data, shape=None):
        """reference: narray/narray.c:1391-1461 -- without a shape, as many whole
        elements as the string holds; with one, the string may be longer, never shorter."""
        data = bytes(data)
        unit = cls.elmsz if cls.elmsz else 0.125
        if shape is None:
            n = int(len(data) // unit)
            if n == 0:
                raise ValueError("string is empty or too short")
            shape = (n,)
        elif isinstance(shape, numbers.Integral):
            shape = (int(shape),)
        a = cls(*shape)
        if int(np.ceil(a.size * unit)) > len(data):
            raise ValueError("specified size is too large")
        a.store_binary(data)
        return a

    from_string = from_binary

    def store_binary(self, data, offset=0):
        """reference: narray/narray.c:1474-1521; answers the number of bytes stored."""
        data = bytes(data)
        if len(data) < offset:
            raise ValueError("offset is larger than string length")
        need = self.byte_size()
        if need > len(data) - offset:
            raise ValueError("string is too short to store")
        if need:
            buf = (C.c_char * need).from_buffer_copy(data, offset)
            d = self._desc()
            call(_L.cumo_hip_na_from_host, C.byref(d), buf, need)
        return need

    def aref_cpu(self, *index):
        """One element read back to the host (reference: gen/tmpl/aref_cpu.c)."""
        if len(index) != self.ndim:
            raise IndexError("the number of indices must equal the number of dimensions")
        idx = (C.c_size_t * max(self.ndim, 1))()
        for d, (k, n) in enumerate(zip(index, self.shape)):
            k = int(k)
            if k < 0:
                k += n
            if not 0 <= k < n:
                raise IndexError("index out of range")
            idx[d] = k
        out = np.zeros(1, dtype=self.np_dtype)
        d = self._desc()
        call(_L.cumo_hip_na_extract, C.byref(d), idx, out.ctypes.data)
        return out[0].item()

    def to_a(self):
        return self.to_numpy().tolist()

    def extract_cpu(self):
        """reference: gen/tmpl/extract_cpu.c:17-23 -- a 0-dim array answers its element."""
        if self.size != 1:
            raise ValueError("not a 0-dim / single-element array")
        out = np.zeros(1, dtype=self.np_dtype)
        d = self._desc()
        call(_L.cumo_hip_na_extract, C.byref(d), None, out.ctypes.data)
        return out[0].item()

    def __float__(self):
        return float(self.extract_cpu())

    def __int__(self):
        return int(self.extract_cpu())

    def __repr__(self):
        return "%s%r" % (type(self).__name__, self.shape)


# ---------------------------------------------------------------------------
# numeric arrays
# ---------------------------------------------------------------------------
class _Numeric(NArray):
    def _scalar_operand(self, other):
        """A Ruby Float meeting an integer array moves the array to DFloat first
        (reference: the upcast tables of gen/def/int32.rb)."""
        if isinstance(other, float) and not self.is_float:
            return self._cast_to(DFloat)
        return self

    # -- binary ---------------------------------------------------------------
    def _binary(self, other, op, scalar_is_left=False):
        z = NArrayDesc()
        if isinstance(other, numbers.Number):
            # reference: gen/tmpl/binary.c:184-209 -- the number rides in the launch
            if isinstance(other, float) and not self.is_float and op in ("add", "sub", "mul", "div"):
                # (the library moves the array to DFloat: in the same launch where it is one contiguous run)
                x = self._desc()
                return _run(_L.cumo_hip_na_binary_fs, op.encode(), C.byref(x), float(other), 1 if scalar_is_left else 0,
                            C.byref(z), results=(z,))
            x = self._scalar_operand(other)._desc()
            return _run(_L.cumo_hip_na_binary_s, op.encode(), C.byref(x), float(other), 1 if scalar_is_left else 0,
                        C.byref(z), results=(z,))
        if not isinstance(other, _Numeric):
            return NotImplemented
        a, b = (other, self) if scalar_is_left else (self, other)
        x, y = a._desc(), b._desc()
        return _run(_L.cumo_hip_na_binary, op.encode(), C.byref(x), C.byref(y), C.byref(z), results=(z,))

    def divmod(self, other):
        """[quotient, remainder] (reference: gen/tmpl/binary2.c; a number is cast to an array
        first, the template has no scalar form). Int32 by zero raises ZeroDivisionError."""
        if isinstance(other, numbers.Number):
            x = self._scalar_operand(other)
            other = type(x).cast(np.array([other], dtype=x.np_dtype))
        else:
            x = self
        if not isinstance(other, _Numeric):
            raise TypeError("divmod needs a numeric operand")
        dx, dy, q, r = x._desc(), other._desc(), NArrayDesc(), NArrayDesc()
        return _run(_L.cumo_hip_na_divmod, C.byref(dx), C.byref(dy), C.byref(q), C.byref(r), results=(q, r))

    def poly(self, *coef):
        """a0 + a1 x + ... + an x**n by Horner's rule in the array's type (reference: gen/tmpl/poly.c:38-78);
        numbers and arrays are cast to the array's type first."""
        cls = type(self)
        arrs = [c if isinstance(c, cls) else (cls.cast(c) if isinstance(c, NArray) else cls.cast(np.array([c], dtype=self.np_dtype)))
                for c in coef]
        descs = [a._desc() for a in arrs]
        ptrs = (C.POINTER(NArrayDesc) * max(1, len(descs)))(*[C.pointer(d) for d in descs])
        d, z = self._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_poly, C.byref(d), len(descs), ptrs, C.byref(z), results=(z,))

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

    # -- pow, clip, maximum / minimum -------------------------------------------
    def __pow__(self, other):
        """reference: gen/tmpl/pow.c:117-215. An Integer exponent takes the
        repeated-product form, a Float exponent pow(); a Float exponent over an
        Int32 array moves the array to DFloat first."""
        z = NArrayDesc()
        if isinstance(other, numbers.Number):
            is_int = isinstance(other, numbers.Integral)
            x = (self if is_int else self._scalar_operand(float(other)))._desc()
            return _run(_L.cumo_hip_na_pow_s, C.byref(x), float(other), 1 if is_int else 0, 0, C.byref(z), results=(z,))
        if not isinstance(other, _Numeric):
            return NotImplemented
        x, y = self._desc(), other._desc()
        return _run(_L.cumo_hip_na_pow, C.byref(x), C.byref(y), C.byref(z), results=(z,))

    def __rpow__(self, other):
        if not isinstance(other, numbers.Number):
            return NotImplemented
        z = NArrayDesc()
        x = self._desc()
        return _run(_L.cumo_hip_na_pow_s, C.byref(x), float(other), 1 if isinstance(other, numbers.Integral) else 0, 1,
                    C.byref(z), results=(z,))

    def pow(self, other): return self.__pow__(other)

    def clip(self, min=None, max=None):
        """reference: gen/tmpl/clip.c:199-254"""
        def bound(b):
            if b is None:
                return 0, 0.0, None
            if isinstance(b, numbers.Number):
                return 1, float(b), None
            if not isinstance(b, _Numeric):
                b = type(self).cast(b)
            return 2, 0.0, b._desc()
        lk, ls, la = bound(min)
        hk, hs, ha = bound(max)
        z = NArrayDesc()
        x = self._desc()
        return _run(_L.cumo_hip_na_clip, C.byref(x), lk, ls, C.byref(la) if la is not None else None, hk, hs,
                    C.byref(ha) if ha is not None else None, C.byref(z), results=(z,))

    @classmethod
    def _ewcomp(cls, op, a, b, nan):
        a = a if isinstance(a, _Numeric) else cls.cast(a)
        b = b if isinstance(b, _Numeric) else cls.cast(b)
        z = NArrayDesc()
        x, y = a._desc(), b._desc()
        return _run(_L.cumo_hip_na_ewcomp, op.encode(), C.byref(x), C.byref(y), 1 if nan else 0, C.byref(z), results=(z,))

    @classmethod
    def maximum(cls, a, b, nan=False):
        """reference: gen/tmpl/ewcomp.c:40-75"""
        return cls._ewcomp("maximum", a, b, nan)

    @classmethod
    def minimum(cls, a, b, nan=False):
        return cls._ewcomp("minimum", a, b, nan)

    # -- mulsum, cumsum / cumprod ---------------------------------------------------
    def mulsum(self, other, axis=None, keepdims=False, nan=False):
        """reference: gen/tmpl/accum_binary.c:62-110"""
        if not isinstance(other, _Numeric):
            other = type(self).cast(other)
        nd = max(self.ndim, other.ndim)
        z = NArrayDesc()
        x, y = self._desc(), other._desc()
        return _run(_L.cumo_hip_na_mulsum, C.byref(x), C.byref(y), _reduce_mask(nd, axis), 1 if keepdims else 0,
                    1 if nan else 0, C.byref(z), results=(z,))

    def _cum(self, op, axis, nan):
        z = NArrayDesc()
        x = self._desc()
        return _run(_L.cumo_hip_na_cum, op.encode(), C.byref(x), _reduce_mask(self.ndim, axis), 1 if nan else 0, C.byref(z),
                    results=(z,))

    def cumsum(self, axis=None, nan=False):
        """reference: gen/tmpl/cum.c:48-80"""
        return self._cum("cumsum", axis, nan)

    def cumprod(self, axis=None, nan=False): return self._cum("cumprod", axis, nan)

    # -- unary ----------------------------------------------------------------
    def _unary(self, op):
        x, z = self._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_unary, op.encode(), C.byref(x), C.byref(z), results=(z,))

    def __neg__(self): return self._unary("minus")
    def minus(self): return self._unary("minus")
    def square(self): return self._unary("square")
    def sign(self): return self._unary("sign")
    def reciprocal(self): return self._unary("reciprocal")
    def abs(self): return self._unary("abs")

    __abs__ = abs

    # -- comparisons into Bit ----------------------------------------------------
    def _compare(self, other, op, scalar_is_left=False):
        z = NArrayDesc()
        if isinstance(other, numbers.Number):
            x = self._scalar_operand(other)._desc()
            return _run(_L.cumo_hip_na_compare_s, op.encode(), C.byref(x), float(other), 1 if scalar_is_left else 0,
                        C.byref(z), results=(z,))
        if not isinstance(other, _Numeric):
            return NotImplemented
        x, y = self._desc(), other._desc()
        return _run(_L.cumo_hip_na_compare, op.encode(), C.byref(x), C.byref(y), C.byref(z), results=(z,))

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
    def _reduce(self, name, axis=None, keepdims=False, nan=False):
        x, z = self._desc(), NArrayDesc()
        mask = _reduce_mask(self.ndim, axis)
        if name == "minmax":
            z2 = NArrayDesc()
            return tuple(_run(_L.cumo_hip_na_reduce, name.encode(), C.byref(x), mask, int(bool(keepdims)), int(bool(nan)),
                              C.byref(z), C.byref(z2), results=(z, z2)))
        return _run(_L.cumo_hip_na_reduce, name.encode(), C.byref(x), mask, int(bool(keepdims)), int(bool(nan)),
                    C.byref(z), None, results=(z,))

    def sum(self, axis=None, keepdims=False, nan=False): return self._reduce("sum", axis, keepdims, nan)
    def prod(self, axis=None, keepdims=False, nan=False): return self._reduce("prod", axis, keepdims, nan)
    def min(self, axis=None, keepdims=False, nan=False): return self._reduce("min", axis, keepdims, nan)
    def max(self, axis=None, keepdims=False, nan=False): return self._reduce("max", axis, keepdims, nan)
    def ptp(self, axis=None, keepdims=False, nan=False): return self._reduce("ptp", axis, keepdims, nan)
    def minmax(self, axis=None, keepdims=False, nan=False): return self._reduce("minmax", axis, keepdims, nan)
    def argmin(self, axis=None, keepdims=False, nan=False): return self._reduce("argmin", axis, keepdims, nan)
    def argmax(self, axis=None, keepdims=False, nan=False): return self._reduce("argmax", axis, keepdims, nan)
    def min_index(self, axis=None, keepdims=False, nan=False): return self._reduce("min_index", axis, keepdims, nan)
    def max_index(self, axis=None, keepdims=False, nan=False): return self._reduce("max_index", axis, keepdims, nan)


class _Float(_Numeric):
    is_float = True

    def mean(self, axis=None, keepdims=False, nan=False): return self._reduce("mean", axis, keepdims, nan)
    def var(self, axis=None, keepdims=False, nan=False): return self._reduce("var", axis, keepdims, nan)
    def stddev(self, axis=None, keepdims=False, nan=False): return self._reduce("stddev", axis, keepdims, nan)
    def rms(self, axis=None, keepdims=False, nan=False): return self._reduce("rms", axis, keepdims, nan)

    def modf(self):
        """[fraction, integral part], each with the sign of the element (reference: gen/tmpl/unary_ret2.c)."""
        d, f, w = self._desc(), NArrayDesc(), NArrayDesc()
        return _run(_L.cumo_hip_na_modf, C.byref(d), C.byref(f), C.byref(w), results=(f, w))

    def floor(self): return self._unary("floor")
    def round(self): return self._unary("round")
    def ceil(self): return self._unary("ceil")
    def trunc(self): return self._unary("trunc")
    def rint(self): return self._unary("rint")
    def copysign(self, o): return self._binary(o, "copysign")

    def _cond_unary(self, op):
        x, z = self._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_cond_unary, op.encode(), C.byref(x), C.byref(z), results=(z,))

    def isnan(self): return self._cond_unary("isnan")
    def isinf(self): return self._cond_unary("isinf")
    def isposinf(self): return self._cond_unary("isposinf")
    def isneginf(self): return self._cond_unary("isneginf")
    def isfinite(self): return self._cond_unary("isfinite")
    def signbit(self): return self._cond_unary("signbit")


class SFloat(_Float):
    type_name, type_code, np_dtype, elmsz = "sfloat", 0, np.float32, 4


class DFloat(_Float):
    type_name, type_code, np_dtype, elmsz = "dfloat", 1, np.float64, 8

    def kahan_sum(self, axis=None, keepdims=False, nan=False): return self._reduce("kahan_sum", axis, keepdims, nan)


class Int64(NArray):
    """Result holder (Int32#sum, arg reductions over more than 2^32-1 elements)."""
    type_name, type_code, np_dtype, elmsz = "int64", 3, np.int64, 8


class UInt64(NArray):
    """Result holder (Bit#count_true)."""
    type_name, type_code, np_dtype, elmsz = "uint64", 4, np.uint64, 8


class Int32(_Numeric):
    type_name, type_code, np_dtype, elmsz = "int32", 2, np.int32, 4

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

    type_name, type_code, np_dtype, elmsz = "bit", 5, np.uint8, 0

    @classmethod
    def _unit(cls):
        return 1

    @classmethod
    def cast(cls, data):
        """Bit.cast(array): nonzero is 1. An array on the device is stored by the number -> Bit
        launcher (reference: gen/tmpl_bit/store_from.c); host data is packed into a staging
        buffer, bit 0 first, and placed by the store_array launcher, as the reference does for
        a Ruby Array (gen/tmpl_bit/store_array.c:60-113)."""
        if isinstance(data, NArray):
            a = cls(*data.shape)
            if data.size:
                a.store(data)
            return a
        arr = np.ascontiguousarray(np.asarray(data) != 0)
        a = cls(*arr.shape)
        n = arr.size
        if n:
            bits = np.packbits(arr.reshape(-1), bitorder="little")
            words = np.zeros(((n + 31) // 32) * 4, dtype=np.uint8)
            words[:bits.size] = bits
            stage = call(_L.cumo_cuda_runtime_malloc, words.nbytes)
            try:
                call(_L.cumo_hip_copy_from_host, stage, words.ctypes.data, words.nbytes)
                f = _lib.fn("cumo_iter_bit_store_array_contiguous_kernel_launch", None,
                            [C.c_void_p, C.c_size_t, C.c_void_p, C.c_uint64])
                call(f, a._buf.ptr, a._offset, stage, n)
            finally:
                _L.cumo_cuda_runtime_free(stage)   # stream ordered: the launch above is already queued
        return a

    from_numpy = cast

    def _raw_words(self):
        """All words of the underlying buffer, on the host."""
        nbytes = self._buf.nbytes
        words = np.zeros(nbytes // 4, dtype=np.uint32)
        if nbytes:
            call(_L.cumo_hip_copy_to_host, words.ctypes.data, self._buf.ptr, nbytes)
        return words

    def byte_size(self):
        return (self.size + 7) // 8

    def to_numpy(self):
        packed = np.frombuffer(self.to_binary(), dtype=np.uint8)
        bits = np.unpackbits(packed, bitorder="little")[:self.size]
        return bits.reshape(self.shape).astype(np.uint8)

    def aref_cpu(self, *index):
        return int(NArray.aref_cpu(self, *index))

    def fill(self, value):
        """reference: gen/tmpl_bit/fill.c:11-58 -- 0 / 1 / false / true, anything else is an ArgumentError."""
        if value is True or value is False:
            value = int(value)
        if not isinstance(value, numbers.Number) or value not in (0, 1):
            raise ValueError("invalid value for Bit")
        d = self._desc()
        _run(_L.cumo_hip_na_fill, C.byref(d), float(value))
        return self

    def _bit_op2(self, other, op):
        if not isinstance(other, Bit):
            return NotImplemented
        x, y, z = self._desc(), other._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_bit_binary, op.encode(), C.byref(x), C.byref(y), C.byref(z), results=(z,))

    def __and__(self, o): return self._bit_op2(o, "and")
    def __or__(self, o): return self._bit_op2(o, "or")
    def __xor__(self, o): return self._bit_op2(o, "xor")
    def eq(self, o): return self._bit_op2(o, "eq")

    def __invert__(self):
        x, z = self._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_bit_unary, b"not", C.byref(x), C.byref(z), results=(z,))

    def _count(self, count_false, axis, keepdims):
        """reference: gen/tmpl_bit/bit_count.c:49-68 -- an empty array answers 0."""
        if self.size == 0:
            return 0
        x, z = self._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_bit_count, C.byref(x), _reduce_mask(self.ndim, axis), int(bool(keepdims)),
                    1 if count_false else 0, C.byref(z), results=(z,))

    def where(self):
        """Positions of the set bits (reference: gen/tmpl_bit/where.c:98-127)."""
        d, z = self._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_where, C.byref(d), 0, C.byref(z), results=(z,))

    def where2(self):
        """[positions of the set bits, positions of the clear bits] (tmpl_bit/where2.c)"""
        d, z0, z1 = self._desc(), NArrayDesc(), NArrayDesc()
        return [_run(_L.cumo_hip_na_where, C.byref(d), 0, C.byref(z0), results=(z0,)),
                _run(_L.cumo_hip_na_where, C.byref(d), 1, C.byref(z1), results=(z1,))]

    def mask(self, array):
        """The elements of `array` where self is set (reference: gen/tmpl_bit/mask.c:96-167)."""
        if not isinstance(array, NArray):
            raise TypeError("mask needs an array")
        m, x, z = self._desc(), array._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_mask, C.byref(m), C.byref(x), C.byref(z), results=(z,))

    def count_true(self, axis=None, keepdims=False): return self._count(False, axis, keepdims)
    def count_false(self, axis=None, keepdims=False): return self._count(True, axis, keepdims)

    count = count_true
    count_1 = count_true
    count_0 = count_false

    def count_true_cpu(self):
        r = self.count_true()
        return int(r) if not isinstance(r, int) else r

    # all? / any? / none? (reference: gen/tmpl_bit/bit_reduce.c:106-146, none_p.c; spec.rb:185-186).
    # Without axis the answer is true / false, read back from a one-bit result; with axis it is
    # a Bit array. An empty array answers false (bit_reduce.c:132-134).
    def _bit_reduce(self, op, axis, keepdims):
        if self.size == 0:
            return False
        x, z = self._desc(), NArrayDesc()
        r = _run(_L.cumo_hip_na_bit_reduce, op, C.byref(x), _reduce_mask(self.ndim, axis), int(bool(keepdims)), C.byref(z), results=(z,))
        if axis is None and not keepdims:
            return bool(r.extract_cpu())
        return r

    def all_p(self, axis=None, keepdims=False):
        return self._bit_reduce(b"all_p", axis, keepdims)

    def any_p(self, axis=None, keepdims=False):
        return self._bit_reduce(b"any_p", axis, keepdims)

    def none_p(self, axis=None, keepdims=False):
        r = self.any_p(axis, keepdims)
        return (not r) if isinstance(r, bool) else ~r

    def _store_into(self, cls):
        """Bit -> 0/1 numbers (reference: gen/tmpl/store_bit.c)."""
        return self._cast_to(cls)


for _cls in (SFloat, DFloat, Int32, Int64, UInt64, Bit):
    _CLASS_BY_CODE[_cls.type_code] = _cls


# ---------------------------------------------------------------------------
# NMath
# ---------------------------------------------------------------------------
class _NMath:
    """Cumo::NMath (reference: narray/math.c:111-112 forwards to the dtype's
    Math module; function list gen/spec.rb:427-457)."""

    _ONE = ("sqrt cbrt log log2 log10 exp exp2 exp10 sin cos tan asin acos atan sinh cosh tanh "
            "asinh acosh atanh sinc erf erfc log1p expm1").split()
    _TWO = ("atan2", "hypot", "ldexp")

    def __getattr__(self, name):
        if name in self._ONE:
            return lambda x: self._call1(name, x)
        if name in self._TWO:
            return lambda x, y: self._call2(name, x, y)
        raise AttributeError(name)

    @staticmethod
    def _check(x):
        if not isinstance(x, _Numeric):
            raise TypeError("NMath needs a numeric array")
        return x

    def frexp(self, x):
        """[mantissa, exponent] with x = mantissa * 2**exponent; the exponent is Int32
        (reference: gen/tmpl/frexp.c:32-38)."""
        d, m, e = self._check(x)._desc(), NArrayDesc(), NArrayDesc()
        return _run(_L.cumo_hip_na_frexp, C.byref(d), C.byref(m), C.byref(e), results=(m, e))

    def _call1(self, name, x):
        d, z = self._check(x)._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_math, name.encode(), C.byref(d), C.byref(z), results=(z,))

    def _call2(self, name, x, y):
        xn, yn = isinstance(x, numbers.Number), isinstance(y, numbers.Number)
        if xn and yn:
            raise TypeError("NMath needs an array operand")
        z = NArrayDesc()
        if xn or yn:
            arr, sv = (y, x) if xn else (x, y)
            d = self._check(arr)._desc()
            return _run(_L.cumo_hip_na_math2_s, name.encode(), C.byref(d), float(sv), 1 if xn else 0, C.byref(z), results=(z,))
        dx, dy = self._check(x)._desc(), self._check(y)._desc()
        return _run(_L.cumo_hip_na_math2, name.encode(), C.byref(dx), C.byref(dy), C.byref(z), results=(z,))


NMath = _NMath()


class _Fused:
    """Row-wise composites along the last dimension in one launch (library additions;
    the reference writes them as chains of array operations,
    bench/transformer_bench.rb:110-124). Layouts the row kernels do not take fall
    back to that chain inside the library."""

    @staticmethod
    def softmax(x):
        d, z = _NMath._check(x)._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_softmax, C.byref(d), C.byref(z), results=(z,))

    @staticmethod
    def layernorm(x, eps=1e-5):
        d, z = _NMath._check(x)._desc(), NArrayDesc()
        return _run(_L.cumo_hip_na_layernorm, C.byref(d), float(eps), C.byref(z), results=(z,))


Fused = _Fused()
