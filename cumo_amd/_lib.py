"""ctypes binding of libcumo_hip.so (the C-ABI declared in include/cumo_hip.h).

There is no fallback: if the library has not been built, importing this module
raises. Every call goes through `call`, which turns an error latched by the
library into the exception the reference's Ruby extension would have raised.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libcumo_hip.so")

MAX_DIM = 12  # CUMO_NA_MAX_DIMENSION


class RuntimeError_(RuntimeError):
    """Cumo::CUDA::RuntimeError (reference: ext/cumo/cuda/runtime.c:16-20)."""


class OutOfMemoryError(MemoryError):
    """Cumo::CUDA::OutOfMemoryError (reference: ext/cumo/cuda/memory_pool.cpp:90-92)."""


class ShapeError(ValueError):
    """Cumo::NArray::ShapeError (reference: ext/cumo/narray/ndloop.c:508-512)."""


class DimensionError(ValueError):
    """Cumo::NArray::DimensionError (reference: ext/cumo/narray/narray.c:1757-1759)."""


class OperationError(ValueError):
    """Cumo::NArray::OperationError (reference: ext/cumo/narray/gen/tmpl/clip.c:48-51,222)."""


class Indexer(C.Structure):
    # reference: ext/cumo/include/cumo/indexer.h:16-22
    _fields_ = [("ndim", C.c_ubyte), ("total_size", C.c_size_t), ("shape", C.c_size_t * MAX_DIM),
                ("index", C.c_uint64 * MAX_DIM), ("raw_index", C.c_uint64)]


class IArray(C.Structure):
    # reference: indexer.h:28-31
    _fields_ = [("ptr", C.c_void_p), ("step", C.c_ssize_t * MAX_DIM)]


class BitIArray(C.Structure):
    # reference: indexer.h:40-44
    _fields_ = [("ptr", C.c_void_p), ("pos", C.c_size_t), ("step", C.c_ssize_t * MAX_DIM)]


class IArrayStridx(C.Structure):
    # reference: indexer.h:46-49; a stride s is stored as (s << 1) | 1
    _fields_ = [("ptr", C.c_void_p), ("stridx", C.c_ssize_t * MAX_DIM)]


class BitIArrayStridx(C.Structure):
    # reference: indexer.h:57-61
    _fields_ = [("ptr", C.c_void_p), ("pos", C.c_size_t), ("stridx", C.c_ssize_t * MAX_DIM)]


class ReductionArg(C.Structure):
    # reference: indexer.h:63-68
    _fields_ = [("in_", IArray), ("out", IArray), ("in_indexer", Indexer), ("out_indexer", Indexer)]


class NArrayDesc(C.Structure):
    """cumo_hip_narray_t (include/cumo_hip_ndloop.h): a view of device memory."""
    _fields_ = [("type", C.c_int), ("ndim", C.c_int), ("ptr", C.c_void_p), ("offset", C.c_ssize_t),
                ("shape", C.c_size_t * MAX_DIM), ("stride", C.c_ssize_t * MAX_DIM)]


class LoopArgs(C.Structure):
    """cumo_hip_loop_args_t"""
    _fields_ = [("type", C.c_int), ("elmsz", C.c_ssize_t), ("ptr", C.c_void_p), ("bitpos", C.c_size_t),
                ("step", C.c_ssize_t * MAX_DIM)]


class Loop(C.Structure):
    """cumo_hip_loop_t"""
    _fields_ = [("narg", C.c_int), ("ndim", C.c_int), ("n", C.c_size_t * MAX_DIM), ("args", LoopArgs * 4),
                ("reduce_dim", C.c_int), ("opt_ptr", C.c_void_p), ("status", C.c_int)]


ITER_FUNC = C.CFUNCTYPE(None, C.POINTER(Loop))


class NdFunc(C.Structure):
    """cumo_hip_ndfunc_t"""
    _fields_ = [("func", ITER_FUNC), ("flag", C.c_uint), ("nin", C.c_int), ("nout", C.c_int), ("out_type", C.c_int * 2)]


NDF_FLAT_REDUCE = 1 << 6
NDF_KEEP_DIM = 1 << 3
TYPE_CODE = {"sfloat": 0, "dfloat": 1, "int32": 2, "int64": 3, "uint64": 4, "bit": 5}


class EwPlan(C.Structure):
    _fields_ = [("kind", C.c_int), ("ndim", C.c_int), ("vec", C.c_int), ("fast_dim", C.c_int), ("tr_dim", C.c_int),
                ("shape", C.c_uint64 * MAX_DIM), ("step", (C.c_int64 * MAX_DIM) * 4)]


class ReducePlan(C.Structure):
    _fields_ = [("kind", C.c_int), ("vec", C.c_int), ("threads_per_row", C.c_int), ("n_split", C.c_int),
                ("out_ndim", C.c_int), ("red_ndim", C.c_int), ("out_total", C.c_uint64), ("red_total", C.c_uint64),
                ("out_shape", C.c_uint64 * MAX_DIM), ("red_shape", C.c_uint64 * MAX_DIM),
                ("in_out_step", C.c_int64 * MAX_DIM), ("in_red_step", C.c_int64 * MAX_DIM),
                ("out_step", C.c_int64 * MAX_DIM)]


if not os.path.exists(LIB_PATH):
    raise ImportError(
        "cumo_amd: %s is missing. Build it with `python cumo_amd/build.py` (needs hipcc); "
        "there is no CPU fallback." % LIB_PATH)

lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)

P = C.POINTER
_sig = {
    "cumo_cuda_runtime_malloc": (C.c_void_p, [C.c_size_t]),
    "cumo_cuda_runtime_free": (None, [C.c_void_p]),
    "cumo_cuda_runtime_free_no_raise": (None, [C.c_void_p]),
    "cumo_cuda_runtime_check_kernel_launch": (None, []),
    "cumo_cuda_runtime_error_flag_ptr": (P(C.c_int), []),
    "cumo_cuda_runtime_error_flag_new": (P(C.c_int), []),
    "cumo_cuda_runtime_error_flag_get": (C.c_bool, [P(C.c_int)]),
    "cumo_hip_last_error": (C.c_int, [P(C.c_char_p)]),
    "cumo_hip_set_stream": (None, [C.c_void_p]),
    "cumo_hip_get_stream": (C.c_void_p, []),
    "cumo_hip_stream_create": (C.c_void_p, []),
    "cumo_hip_stream_destroy": (None, [C.c_void_p]),
    "cumo_hip_device_count": (C.c_int, []),
    "cumo_hip_synchronize": (None, []),
    "cumo_hip_event_create": (C.c_void_p, []),
    "cumo_hip_event_record": (None, [C.c_void_p]),
    "cumo_hip_event_elapsed_ms": (C.c_float, [C.c_void_p, C.c_void_p]),
    "cumo_hip_event_destroy": (None, [C.c_void_p]),
    "cumo_hip_memcpy_h2d": (None, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "cumo_hip_memcpy_d2h": (None, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "cumo_hip_memset": (None, [C.c_void_p, C.c_int, C.c_size_t]),
    "cumo_hip_copy_to_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "cumo_hip_copy_from_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t]),
    "cumo_hip_pool_malloc": (C.c_int, [C.c_size_t, C.c_void_p, P(C.c_void_p)]),
    "cumo_hip_pool_free": (C.c_int, [C.c_void_p]),
    "cumo_hip_pool_free_all_blocks": (None, []),
    "cumo_hip_pool_free_all_blocks_stream": (None, [C.c_void_p]),
    "cumo_hip_pool_n_free_blocks": (C.c_size_t, []),
    "cumo_hip_pool_used_bytes": (C.c_size_t, []),
    "cumo_hip_pool_free_bytes": (C.c_size_t, []),
    "cumo_hip_pool_total_bytes": (C.c_size_t, []),
    "cumo_hip_pool_device_malloc_calls": (C.c_size_t, []),
    "cumo_hip_pool_enable": (C.c_int, [C.c_int]),
    "cumo_hip_pool_set_limit": (None, [C.c_size_t]),
    "cumo_hip_pool_use_host_backend": (C.c_int, [C.c_int]),
    "cumo_hip_plan_elementwise": (C.c_int, [P(Indexer), C.c_int, P(P(IArray)), P(C.c_int), P(C.c_size_t), P(EwPlan)]),
    "cumo_hip_plan_reduce": (C.c_int, [P(ReductionArg), C.c_int, C.c_int, P(ReducePlan)]),
    # host launch layer (include/cumo_hip_ndloop.h)
    "cumo_hip_na_storage_bytes": (C.c_size_t, [C.c_int, C.c_size_t]),
    "cumo_hip_na_alloc": (C.c_int, [P(NArrayDesc), C.c_int, C.c_int, P(C.c_size_t)]),
    "cumo_hip_na_ndloop": (C.c_int, [P(NdFunc), P(P(NArrayDesc)), P(P(NArrayDesc)), C.c_uint, C.c_void_p]),
    "cumo_hip_na_ndloop_prepare": (C.c_int, [P(NdFunc), P(P(NArrayDesc)), P(P(NArrayDesc)), C.c_uint, P(Loop)]),
    "cumo_hip_make_indexer": (None, [P(Loop), P(Indexer)]),
    "cumo_hip_make_iarray": (None, [P(Loop), C.c_int, P(IArray)]),
    "cumo_hip_make_bit_iarray": (None, [P(Loop), C.c_int, P(BitIArray)]),
    "cumo_hip_make_iarray_stridx": (None, [P(Loop), C.c_int, P(IArrayStridx)]),
    "cumo_hip_make_bit_iarray_stridx": (None, [P(Loop), C.c_int, P(BitIArrayStridx)]),
    "cumo_hip_make_reduction_arg": (None, [P(Loop), P(ReductionArg)]),
    "cumo_hip_na_binary": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_binary_s": (C.c_int, [C.c_char_p, P(NArrayDesc), C.c_double, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_binary_fs": (C.c_int, [C.c_char_p, P(NArrayDesc), C.c_double, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_unary": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_pow": (C.c_int, [P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_pow_s": (C.c_int, [P(NArrayDesc), C.c_double, C.c_int, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_mulsum": (C.c_int, [P(NArrayDesc), P(NArrayDesc), C.c_uint, C.c_int, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_cum": (C.c_int, [C.c_char_p, P(NArrayDesc), C.c_uint, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_where": (C.c_int, [P(NArrayDesc), C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_mask": (C.c_int, [P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_softmax": (C.c_int, [P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_layernorm": (C.c_int, [P(NArrayDesc), C.c_double, P(NArrayDesc)]),
    "cumo_hip_na_ewcomp": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc), C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_clip": (C.c_int, [P(NArrayDesc), C.c_int, C.c_double, P(NArrayDesc), C.c_int, C.c_double, P(NArrayDesc),
                                   P(NArrayDesc)]),
    "cumo_hip_na_math": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_math2": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_math2_s": (C.c_int, [C.c_char_p, P(NArrayDesc), C.c_double, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_frexp": (C.c_int, [P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_poly": (C.c_int, [P(NArrayDesc), C.c_int, C.POINTER(P(NArrayDesc)), P(NArrayDesc)]),
    "cumo_hip_na_modf": (C.c_int, [P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_divmod": (C.c_int, [P(NArrayDesc), P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_compare": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_compare_s": (C.c_int, [C.c_char_p, P(NArrayDesc), C.c_double, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_cond_unary": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_store": (C.c_int, [P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_copy": (C.c_int, [P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_fill": (C.c_int, [P(NArrayDesc), C.c_double]),
    "cumo_hip_na_seq": (C.c_int, [P(NArrayDesc), C.c_double, C.c_double]),
    "cumo_hip_na_logseq": (C.c_int, [P(NArrayDesc), C.c_double, C.c_double, C.c_double]),
    "cumo_hip_na_eye": (C.c_int, [P(NArrayDesc), C.c_double, C.c_ssize_t]),
    "cumo_hip_na_to_host": (C.c_int, [P(NArrayDesc), C.c_void_p, C.c_size_t]),
    "cumo_hip_na_from_host": (C.c_int, [P(NArrayDesc), C.c_void_p, C.c_size_t]),
    "cumo_hip_na_extract": (C.c_int, [P(NArrayDesc), P(C.c_size_t), C.c_void_p]),
    "cumo_hip_na_reduce": (C.c_int, [C.c_char_p, P(NArrayDesc), C.c_uint, C.c_int, C.c_int, P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_bit_binary": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_bit_unary": (C.c_int, [C.c_char_p, P(NArrayDesc), P(NArrayDesc)]),
    "cumo_hip_na_bit_count": (C.c_int, [P(NArrayDesc), C.c_uint, C.c_int, C.c_int, P(NArrayDesc)]),
    "cumo_hip_na_bit_reduce": (C.c_int, [C.c_char_p, P(NArrayDesc), C.c_uint, C.c_int, P(NArrayDesc)]),
}
for _name, (_res, _args) in _sig.items():
    _f = getattr(lib, _name)
    _f.restype = _res
    _f.argtypes = _args

CTYPE = {"sfloat": C.c_float, "dfloat": C.c_double, "int32": C.c_int32}


def fn(name, restype=None, argtypes=None):
    """Looks a launcher up by its C name; fails loudly when the symbol is missing."""
    try:
        f = getattr(lib, name)
    except AttributeError:
        raise NotImplementedError("libcumo_hip.so does not export %s" % name)
    if argtypes is not None:
        f.argtypes = argtypes
    f.restype = restype
    return f


def check():
    """Raises what the Ruby extension would have raised for a latched error."""
    msg = C.c_char_p()
    kind = lib.cumo_hip_last_error(C.byref(msg))
    if kind == 0:
        return
    text = msg.value.decode("utf-8", "replace") if msg.value else ""
    if kind == 2:
        raise OutOfMemoryError(text)
    if kind in (3, 7):
        raise ValueError(text)
    if kind == 4:
        raise ShapeError(text)
    if kind == 5:
        raise ZeroDivisionError(text)
    if kind == 6:
        raise TypeError(text)
    if kind == 8:
        raise DimensionError(text)
    if kind == 9:
        raise OperationError(text)
    raise RuntimeError_(text)


_recording = None


def call(f, *args):
    if _recording is not None and (f.__name__.endswith("_kernel_launch") or f.__name__.startswith("cumo_hip_na_")
                                   or f.__name__ == "cumo_hip_memset"):
        _recording.append((f, args))
    r = f(*args)
    check()
    return r


class _Calls(list):
    def __init__(self):
        super().__init__()
        self.keep = []


class record:
    """Collects the library calls (function, arguments) that launch work inside the
    block, so that a caller can issue exactly the same calls again without the
    Python-side work of building them: `with record() as calls: y = a + b`, then
    `replay(calls)`. A recorded host-layer call carries its result descriptor with
    the memory the first call allocated, so a replay writes into the same array;
    the arrays involved must be kept alive. Temporaries the recorded operations
    themselves release inside the block (index arrays, staging buffers) stay allocated
    for as long as the returned list lives (its `keep` attribute holds them)."""

    def __enter__(self):
        global _recording
        self._prev = _recording
        _recording = _Calls()
        self.calls = _recording
        return self.calls

    def __exit__(self, *exc):
        global _recording
        _recording = self._prev
        return False


def replay(calls, times=1):
    for _ in range(times):
        for f, args in calls:
            f(*args)
    check()
