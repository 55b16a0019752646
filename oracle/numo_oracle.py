"""ctypes front end of the CPU oracle (oracle/numo_oracle.c). TEST INFRASTRUCTURE:
only tests/, the smoke check and the cpu_baseline leg of bench.py import it.

Operands are numpy arrays (any strides, views welcome); broadcasting is resolved
here with numpy's own stride-0 views so that the C side sees exactly the
shape/steps descriptors the launch layer hands to the device.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libnumo_oracle.so")

T_SFLOAT, T_DFLOAT, T_INT32, T_INT64, T_UINT64 = 0, 1, 2, 3, 4
_TCODE = {np.dtype(np.float32): T_SFLOAT, np.dtype(np.float64): T_DFLOAT, np.dtype(np.int32): T_INT32,
          np.dtype(np.int64): T_INT64, np.dtype(np.uint64): T_UINT64}


def build():
    """Compiles the oracle."""
    subprocess.run(["make", "-C", HERE], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def _load():
    if not os.path.exists(LIB):
        build()
    return C.CDLL(LIB)


lib = _load()
SZ = C.c_size_t
SSZ = C.c_ssize_t
lib.numo_binary.restype = C.c_int
lib.numo_unary.restype = C.c_int
lib.numo_compare.restype = C.c_int
lib.numo_cond_unary.restype = C.c_int
lib.numo_store.restype = C.c_int
lib.numo_store_bit.restype = C.c_int
lib.numo_copy_bytes.restype = C.c_int
lib.numo_fill.restype = C.c_int
lib.numo_bit_binary.restype = C.c_int
lib.numo_bit_count.restype = C.c_uint64
lib.numo_cum_run.argtypes = [C.c_int, C.c_int, C.c_int, SZ, C.c_void_p, SSZ, C.c_void_p, SSZ]
lib.numo_cum_run.restype = C.c_int
lib.numo_mulsum_run.argtypes = [C.c_int, C.c_int, SZ, C.c_void_p, SSZ, C.c_void_p, SSZ, C.c_void_p]
lib.numo_mulsum_run.restype = C.c_int
lib.numo_pow_int.argtypes = [C.c_int, SZ, C.c_void_p, SSZ, C.c_void_p, SSZ, C.c_void_p]
lib.numo_pow_int.restype = C.c_int
lib.numo_bit_count.argtypes = [C.c_void_p, SZ, SSZ, C.c_uint64, C.c_int]
lib.numo_reduce.restype = C.c_int
lib.numo_sfloat_f.restype = C.c_float
lib.numo_sfloat_f.argtypes = [C.c_char_p, SZ, C.c_void_p]
lib.numo_dfloat_f.restype = C.c_double
lib.numo_dfloat_f.argtypes = [C.c_char_p, SZ, C.c_void_p]
lib.numo_sfloat_index_f.restype = C.c_int64
lib.numo_sfloat_index_f.argtypes = [C.c_char_p, SZ, C.c_void_p]
lib.numo_dfloat_index_f.restype = C.c_int64
lib.numo_dfloat_index_f.argtypes = [C.c_char_p, SZ, C.c_void_p]


def _desc(a, shape):
    """(pointer, steps) of `a` broadcast to `shape`."""
    b = np.broadcast_to(a, shape)
    steps = (SSZ * max(1, len(shape)))(*[int(s) for s in b.strides])
    return C.c_void_p(b.__array_interface__["data"][0]), steps


def _shape(shape):
    return (SZ * max(1, len(shape)))(*[int(s) for s in shape])


def _tcode(a):
    return _TCODE[np.dtype(a.dtype)]


class FlagError(Exception):
    """The operation rejected an element (division by zero, abs(INT_MIN))."""

    def __init__(self, result):
        super().__init__("flag raised")
        self.result = result


def binary(op, x, y, scalar_is_left=False, out=None):
    """x op y. Either side may be a Python number (the scalar form)."""
    if isinstance(x, np.ndarray) and isinstance(y, np.ndarray):
        shape = np.broadcast_shapes(x.shape, y.shape)
        res = np.zeros(shape, dtype=x.dtype) if out is None else out
        p1, s1 = _desc(x, shape)
        p2, s2 = _desc(y, shape)
        p3, s3 = _desc(res, shape)
        rc = lib.numo_binary(op.encode(), _tcode(x), len(shape), _shape(shape), p1, s1, p2, s2, p3, s3, C.c_double(0), 0)
    else:
        arr, sv = (y, x) if scalar_is_left else (x, y)
        shape = arr.shape
        res = np.zeros(shape, dtype=arr.dtype) if out is None else out
        p1, s1 = _desc(arr, shape)
        p3, s3 = _desc(res, shape)
        rc = lib.numo_binary(op.encode(), _tcode(arr), len(shape), _shape(shape), p1, s1, None, None, p3, s3,
                             C.c_double(float(sv)), 1 if scalar_is_left else 0)
    if rc < 0:
        raise ValueError("oracle: unknown op %s" % op)
    if rc == 1:
        raise FlagError(res)
    return res


def unary(op, x, out=None):
    res = np.zeros(x.shape, dtype=x.dtype) if out is None else out
    p1, s1 = _desc(x, x.shape)
    p2, s2 = _desc(res, x.shape)
    rc = lib.numo_unary(op.encode(), _tcode(x), x.ndim, _shape(x.shape), p1, s1, p2, s2)
    if rc < 0:
        raise ValueError("oracle: unknown op %s" % op)
    if rc == 1:
        raise FlagError(res)
    return res


def seq(shape, dtype, beg=0, step=1):
    """A new array whose row-major element i is beg + step * i: the float types take beg and
    step in their own type, compute in double and round once; Int32 computes in double and
    converts through a signed 64-bit integer (types/float_macro.h:145-148, xint_macro.h:153-156,
    gen/tmpl/seq_kernel.cu:14-37)."""
    dt = np.dtype(dtype)
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    i = np.arange(n, dtype=np.float64)
    if dt.kind == "f":
        v = (np.float64(dt.type(beg)) + np.float64(dt.type(step)) * i).astype(dt)
    else:
        v = (np.float64(beg) + np.float64(step) * i).astype(np.int64).astype(dt)
    return v.reshape(shape)


def logseq(shape, dtype, beg, step, base=10):
    """base ** x with x the seq value rounded to the element type first; the power is the C
    library's double pow, stored once (gen/tmpl/logseq_kernel.cu:5-15, types/float_macro.h:64)."""
    dt = np.dtype(dtype)
    x = seq(shape, dt, beg, step)
    return np.power(np.float64(dt.type(base)), x.astype(np.float64)).astype(dt)


def eye(shape, dtype, element=1, offset=0):
    """`element` where row + offset == column in every matrix of the last two dimensions
    (gen/tmpl/eye_kernel.cu:2-9)."""
    out = np.zeros(shape, dtype=dtype)
    r = np.arange(shape[-2])[:, None]
    c = np.arange(shape[-1])[None, :]
    out[..., (r + offset) == c] = np.dtype(dtype).type(element)
    return out


def modf(x):
    """(fraction, integral part), the C library's modf element by element on the promoted
    argument, each result stored once (types/float_macro.h:48, gen/tmpl/unary_ret2.c)."""
    f, w = np.modf(x.astype(np.float64))
    return f.astype(x.dtype), w.astype(x.dtype)


def divmod_(x, y):
    """(x / y, x mod y) by the two operators (types/float_macro.h:32, xint_macro.h:20)."""
    return binary("div", x, y), binary("mod", x, y)


def poly(x, *coef):
    """Horner's rule with the element type's own multiplication and addition, each rounded
    separately; Int32 wraps (gen/tmpl/poly_kernel.cu:9-17). Coefficients are cast to x's type
    and broadcast; none answers x."""
    dt = x.dtype
    cs = [np.asarray(c).astype(dt) for c in coef]
    if not cs:
        return x.copy()
    shape = np.broadcast_shapes(x.shape, *[c.shape for c in cs])
    xb = np.broadcast_to(x, shape)
    y = np.broadcast_to(cs[-1], shape).copy()
    with np.errstate(all="ignore"):
        for c in reversed(cs[:-1]):
            y = (xb * y).astype(dt)
            y = (y + np.broadcast_to(c, shape)).astype(dt)
    return y


def frexp(x):
    """(mantissa, Int32 exponent) with x = mantissa * 2**exponent, the C library's frexp
    element by element (types/float_macro.h:118, gen/tmpl/frexp.c:32-38); numpy calls the
    same C function."""
    m, e = np.frexp(x)
    return m.astype(x.dtype), e.astype(np.int32)


def pow_int(x, p):
    """Float array (or one float) ** Int32 array (or one integer): the repeated-product
    form of types/float_macro.h:125-144. Operands are broadcast; x fixes the type."""
    xa = np.asarray(x)
    pa = np.asarray(p, dtype=np.int32)
    shape = np.broadcast_shapes(xa.shape, pa.shape)
    xf = np.ascontiguousarray(np.broadcast_to(xa, shape)).reshape(-1)
    pf = np.ascontiguousarray(np.broadcast_to(pa, shape)).reshape(-1)
    out = np.zeros(xf.shape, dtype=xf.dtype)
    rc = lib.numo_pow_int(_tcode(xf), xf.size, C.c_void_p(xf.ctypes.data), 1, C.c_void_p(pf.ctypes.data), 1,
                          C.c_void_p(out.ctypes.data))
    if rc:
        raise ValueError("oracle: pow_int of a non-float type")
    return out.reshape(shape)


def clip(x, lo=None, hi=None):
    """x.clip(lo, hi) (narray/gen/tmpl/clip.c:23-33,199-254); bounds are numbers, arrays
    of x's type, or None. Raises FlagError when a lower bound exceeds its upper bound
    (the elements concerned keep the zeros of the fresh result)."""
    res = x.copy()
    if lo is not None and hi is not None:
        lo_a = np.broadcast_to(np.asarray(lo, dtype=x.dtype), x.shape)
        hi_a = np.broadcast_to(np.asarray(hi, dtype=x.dtype), x.shape)
        with np.errstate(invalid="ignore"):
            bad = lo_a > hi_a
        res = binary("clip_max", binary("clip_min", x, np.ascontiguousarray(lo_a)), np.ascontiguousarray(hi_a))
        if bad.any():
            res[bad] = 0
            raise FlagError(res)
        return res
    if lo is not None:
        return binary("clip_min", x, lo if not isinstance(lo, np.ndarray) else lo.astype(x.dtype))
    if hi is not None:
        return binary("clip_max", x, hi if not isinstance(hi, np.ndarray) else hi.astype(x.dtype))
    raise ValueError("min and max are not given")


def _axes(ndim, axis):
    if axis is None:
        return tuple(range(ndim))
    if isinstance(axis, (int, np.integer)):
        axis = (axis,)
    return tuple(sorted(a + ndim if a < 0 else a for a in axis))


def cum(op, x, axis=None, nan=False):
    """x.cumsum / x.cumprod (narray/gen/tmpl/cum.c:12-80): the running value along
    the given axes taken together in row-major order, all of them by default."""
    prod = {"cumsum": 0, "cumprod": 1}[op]
    ax = _axes(x.ndim, axis)
    keep = tuple(d for d in range(x.ndim) if d not in ax)
    xt = np.ascontiguousarray(np.transpose(x, keep + ax))
    n = int(np.prod([x.shape[d] for d in ax])) if ax else 1
    rows = xt.size // n if n else 0
    flat = xt.reshape(rows, n) if n else xt.reshape(0, 0)
    out = np.zeros_like(flat)
    es = flat.dtype.itemsize
    for r in range(rows):
        rc = lib.numo_cum_run(prod, _tcode(flat), 1 if nan else 0, n, C.c_void_p(flat[r].ctypes.data), es,
                              C.c_void_p(out[r].ctypes.data), es)
        if rc:
            raise ValueError("oracle: cum of an unsupported type")
    res = out.reshape(xt.shape)
    return np.ascontiguousarray(np.transpose(res, np.argsort(keep + ax)))


def mulsum(x, y, axis=None, keepdims=False, nan=False):
    """x.mulsum(y) (narray/gen/tmpl/accum_binary.c:27-38,62-110): the sum of the
    products over the given axes, sequentially in row-major order, started from 0.
    Operands are broadcast and must have one type."""
    assert x.dtype == y.dtype
    shape = np.broadcast_shapes(x.shape, y.shape)
    ax = _axes(len(shape), axis)
    keep = tuple(d for d in range(len(shape)) if d not in ax)
    perm = keep + ax
    xt = np.ascontiguousarray(np.transpose(np.broadcast_to(x, shape), perm))
    yt = np.ascontiguousarray(np.transpose(np.broadcast_to(y, shape), perm))
    n = int(np.prod([shape[d] for d in ax])) if ax else 1
    oshape = tuple(shape[d] for d in keep)
    rows = int(np.prod(oshape)) if oshape else 1
    out = np.zeros(rows, dtype=x.dtype)
    es = x.dtype.itemsize
    if xt.size:
        xf, yf = xt.reshape(rows, n), yt.reshape(rows, n)
        for r in range(rows):
            rc = lib.numo_mulsum_run(_tcode(xf), 1 if nan else 0, n, C.c_void_p(xf[r].ctypes.data), es,
                                     C.c_void_p(yf[r].ctypes.data), es, C.c_void_p(out[r:].ctypes.data))
            if rc:
                raise ValueError("oracle: mulsum of an unsupported type")
    res = out.reshape(oshape)
    if keepdims:
        res = res.reshape(tuple(1 if d in ax else shape[d] for d in range(len(shape))))
    return res


def _bit_words(nbits):
    return np.zeros((nbits + 31) // 32 + 1, dtype=np.uint32)


def unpack(words, pos, shape, steps=None):
    """Bits of a packed word array as a uint8 array of `shape`."""
    n = int(np.prod(shape)) if len(shape) else 1
    bits = np.unpackbits(words.view(np.uint8), bitorder="little")
    if steps is None:
        return bits[pos:pos + n].reshape(shape).astype(np.uint8)
    idx = np.full(shape, pos, dtype=np.int64)
    for d, (s, st) in enumerate(zip(shape, steps)):
        sh = [1] * len(shape)
        sh[d] = s
        idx = idx + (np.arange(s, dtype=np.int64) * st).reshape(sh)
    return bits[idx].astype(np.uint8)


def pack(bits):
    """uint8 0/1 array -> packed uint32 words (contiguous, position 0)."""
    flat = np.ascontiguousarray(bits).reshape(-1) != 0
    w = np.zeros(((flat.size + 31) // 32) * 4, dtype=np.uint8)
    p = np.packbits(flat, bitorder="little")
    w[:p.size] = p
    return w.view(np.uint32)


def compare(op, x, y, scalar_is_left=False):
    """Returns the result as an unpacked uint8 array (0/1)."""
    if isinstance(x, np.ndarray) and isinstance(y, np.ndarray):
        shape = np.broadcast_shapes(x.shape, y.shape)
        arr = x
    else:
        arr, sv = (y, x) if scalar_is_left else (x, y)
        shape = arr.shape
    n = int(np.prod(shape)) if len(shape) else 1
    words = _bit_words(n)
    bs = (SSZ * max(1, len(shape)))(*[int(s // 1) for s in (np.empty(shape, dtype=np.uint8).strides or (1,))])
    if isinstance(x, np.ndarray) and isinstance(y, np.ndarray):
        p1, s1 = _desc(x, shape)
        p2, s2 = _desc(y, shape)
        rc = lib.numo_compare(op.encode(), _tcode(x), len(shape), _shape(shape), p1, s1, p2, s2,
                              words.ctypes.data_as(C.c_void_p), SZ(0), bs, C.c_double(0), 0)
    else:
        p1, s1 = _desc(arr, shape)
        rc = lib.numo_compare(op.encode(), _tcode(arr), len(shape), _shape(shape), p1, s1, None, None,
                              words.ctypes.data_as(C.c_void_p), SZ(0), bs, C.c_double(float(sv)), 1 if scalar_is_left else 0)
    if rc < 0:
        raise ValueError("oracle: unknown op %s" % op)
    return unpack(words, 0, shape)


def cond_unary(op, x):
    shape = x.shape
    n = int(np.prod(shape)) if len(shape) else 1
    words = _bit_words(n)
    bs = (SSZ * max(1, len(shape)))(*[int(s) for s in (np.empty(shape, dtype=np.uint8).strides or (1,))])
    p1, s1 = _desc(x, shape)
    rc = lib.numo_cond_unary(op.encode(), _tcode(x), len(shape), _shape(shape), p1, s1,
                             words.ctypes.data_as(C.c_void_p), SZ(0), bs)
    if rc < 0:
        raise ValueError("oracle: unknown op %s" % op)
    return unpack(words, 0, shape)


def store(dst_dtype, src):
    res = np.zeros(src.shape, dtype=dst_dtype)
    pd, sd = _desc(res, src.shape)
    ps, ss = _desc(src, src.shape)
    rc = lib.numo_store(_TCODE[np.dtype(dst_dtype)], _tcode(src), src.ndim, _shape(src.shape), pd, sd, ps, ss)
    if rc < 0:
        raise ValueError("oracle: unsupported store")
    return res


def copy(src):
    res = np.zeros(src.shape, dtype=src.dtype)
    pd, sd = _desc(res, src.shape)
    ps, ss = _desc(src, src.shape)
    lib.numo_copy_bytes(SZ(src.dtype.itemsize), src.ndim, _shape(src.shape), ps, ss, pd, sd)
    return res


def fill(dtype, shape, value):
    res = np.zeros(shape, dtype=dtype)
    pd, sd = _desc(res, shape)
    lib.numo_fill(_TCODE[np.dtype(dtype)], len(shape), _shape(shape), pd, sd, C.c_double(float(value)))
    return res


def bit_binary(op, x, y=None):
    """x, y: uint8 0/1 arrays (broadcastable). Packs, runs the per-bit loop, unpacks."""
    shape = x.shape if y is None else np.broadcast_shapes(x.shape, y.shape)
    xb = pack(np.broadcast_to(x, shape))
    yb = pack(np.broadcast_to(y, shape)) if y is not None else None
    n = int(np.prod(shape)) if len(shape) else 1
    words = _bit_words(n)
    bs = (SSZ * max(1, len(shape)))(*[int(s) for s in (np.empty(shape, dtype=np.uint8).strides or (1,))])
    rc = lib.numo_bit_binary(op.encode(), len(shape), _shape(shape), xb.ctypes.data_as(C.c_void_p), SZ(0), bs,
                             yb.ctypes.data_as(C.c_void_p) if yb is not None else None, SZ(0), bs,
                             words.ctypes.data_as(C.c_void_p), SZ(0), bs)
    if rc < 0:
        raise ValueError("oracle: unknown bit op %s" % op)
    return unpack(words, 0, shape)


def bit_count(words, pos, step, n, count_false=False):
    return int(lib.numo_bit_count(words.ctypes.data_as(C.c_void_p), pos, step, n, 1 if count_false else 0))


def where(bits, invert=False):
    """Bit#where (narray/gen/tmpl_bit/where.c:34-52,98-127): the row-major positions of
    the set bits (of the clear ones with invert), ascending, as the index type the
    reference picks (Int32 unless the array has more than 2^32 - 1 elements)."""
    flat = np.asarray(bits).reshape(-1) != 0
    if invert:
        flat = ~flat
    pos = [i for i in range(flat.size) if flat[i]] if flat.size <= 4096 else np.flatnonzero(flat)
    return np.asarray(pos, dtype=np.int64 if flat.size > 4294967295 else np.int32)


def mask(bits, x):
    """Bit#mask (narray/gen/tmpl_bit/mask.c:96-167): the elements of x where the bit of
    the same position is set, in row-major order; shapes must be equal."""
    bits, x = np.asarray(bits), np.asarray(x)
    if bits.shape != x.shape:
        raise ValueError("mask and masked arrays must have the same shape")
    return np.ascontiguousarray(x).reshape(-1)[where(bits).astype(np.int64)]


def _positions(k, n):
    """One index of a[...]: an integer, a slice or an index array, as positions in a
    dimension of n elements (narray/index.c:112-233: negative values count from the end)."""
    if isinstance(k, (int, np.integer)):
        k = int(k) + (n if k < 0 else 0)
        if not 0 <= k < n:
            raise IndexError("index out of range")
        return [k], True
    if isinstance(k, slice):
        return list(range(*k.indices(n))), False
    out = []
    for v in np.asarray(k).reshape(-1).tolist():
        v = int(v) + (n if v < 0 else 0)
        if not 0 <= v < n:
            raise IndexError("index out of range")
        out.append(v)
    return out, False


def take(x, key):
    """a[key] with index arrays (narray/index.c:445-614): every dimension selects on its
    own (an outer product of the selections, not numpy's zipped indexing); an integer
    drops its dimension."""
    x = np.asarray(x)
    key = tuple(key) + (slice(None),) * (x.ndim - len(key))
    sel = [_positions(k, n) for k, n in zip(key, x.shape)]
    out = x[np.ix_(*[np.asarray(p, dtype=np.int64) for p, _ in sel])] if x.ndim else x
    return out.reshape([len(p) for p, drop in sel if not drop])


def put(x, key, value):
    """a[key] = value with index arrays (gen/tmpl/aset.c; the store goes through
    ndloop's scatter, narray/ndloop.c:1316): x is changed in place, value broadcasts
    over the selection."""
    key = tuple(key) + (slice(None),) * (x.ndim - len(key))
    sel = [_positions(k, n) for k, n in zip(key, x.shape)]
    shape = [len(p) for p, _ in sel]
    kept = [len(p) for p, drop in sel if not drop]
    v = np.broadcast_to(np.asarray(value, dtype=x.dtype), kept).reshape(shape)
    x[np.ix_(*[np.asarray(p, dtype=np.int64) for p, _ in sel])] = v
    return x


def at(x, *keys):
    """a.at(i0, i1, ...) (narray/index.c:622-682,842-870): the elements at the zipped
    positions, as a 1-D array; every key selects the same number of positions."""
    x = np.asarray(x)
    if len(keys) != x.ndim:
        raise IndexError("the number of arguments must equal the number of dimensions")
    sel = [_positions(slice(k.start, k.stop, k.step) if isinstance(k, range) else k, n)[0] for k, n in zip(keys, x.shape)]
    if not sel or len(sel[-1]) == 0:
        raise ValueError("cannot get element of empty array")
    if any(len(p) != len(sel[-1]) for p in sel):
        raise ValueError("index array sizes mismatch")
    return np.array([x[tuple(p[i] for p in sel)] for i in range(len(sel[-1]))], dtype=x.dtype)


def store_bit(dst_dtype, bits):
    w = pack(bits)
    shape = bits.shape
    res = np.zeros(shape, dtype=dst_dtype)
    pd, sd = _desc(res, shape)
    bs = (SSZ * max(1, len(shape)))(*[int(s) for s in (np.empty(shape, dtype=np.uint8).strides or (1,))])
    lib.numo_store_bit(_TCODE[np.dtype(dst_dtype)], len(shape), _shape(shape), pd, sd, w.ctypes.data_as(C.c_void_p), SZ(0), bs)
    return res


_OUT_DTYPE = {"sum": {T_INT32: np.int64}, "prod": {T_INT32: np.int64}}


def reduce(op, x, axis=None, keepdims=False, nan=False, index_dtype=np.int32):
    """The reduction `op` of x over `axis` (None = all) the way Numo answers it."""
    nd = x.ndim
    if axis is None:
        axes = tuple(range(nd))
    elif isinstance(axis, (int, np.integer)):
        axes = (int(axis) % nd,)
    else:
        axes = tuple(sorted(int(a) % nd for a in axis))
    keep = [d for d in range(nd) if d not in axes]
    order = keep + list(axes)
    xt = x.transpose(order) if nd else x
    shape = xt.shape
    steps = (SSZ * max(1, nd))(*[int(s) for s in xt.strides])
    out_shape = tuple(x.shape[d] for d in keep)
    name = op + ("_nan" if nan and x.dtype.kind == "f" else "")
    is_idx = op.startswith("arg") or op.endswith("_index")
    if is_idx:
        odt = np.dtype(index_dtype)
    else:
        odt = np.dtype(_OUT_DTYPE.get(op, {}).get(_tcode(x), x.dtype))
    res = np.zeros(out_shape, dtype=odt)
    so = (SSZ * max(1, len(out_shape)))(*[int(s) for s in res.strides])
    n_red = int(np.prod([x.shape[d] for d in axes])) if axes else 1
    scratch = np.zeros(max(1, n_red), dtype=x.dtype)
    rc = lib.numo_reduce(name.encode(), _tcode(x), nd, len(keep), _shape(shape),
                         C.c_void_p(xt.__array_interface__["data"][0]), steps,
                         res.ctypes.data_as(C.c_void_p), so, odt.itemsize, scratch.ctypes.data_as(C.c_void_p))
    if rc < 0:
        raise ValueError("oracle: unknown reduction %s" % name)
    if keepdims:
        res = res.reshape([x.shape[d] if d in keep else 1 for d in range(nd)])
    return res


def f1d(op, x):
    """The sequential 1-d loop f_<op> on a contiguous 1-d array."""
    x = np.ascontiguousarray(x)
    if op.endswith("_index") or op.endswith("_index_nan") or op.startswith("arg"):
        f = lib.numo_sfloat_index_f if x.dtype == np.float32 else lib.numo_dfloat_index_f
        return int(f(op.encode(), x.size, x.ctypes.data_as(C.c_void_p)))
    f = lib.numo_sfloat_f if x.dtype == np.float32 else lib.numo_dfloat_f
    return f(op.encode(), x.size, x.ctypes.data_as(C.c_void_p))
