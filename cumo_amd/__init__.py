"""cumo_amd: the MI355X (gfx950) array-compute hot path behind Cumo's C-extension API.

The product is libcumo_hip.so (hand-written HIP kernels behind the C-ABI of
include/cumo_hip.h). This package is the host-side mirror of the Cumo::NArray
classes that drives it: SFloat, DFloat, Int32, Bit, NMath and MemoryPool.
Importing it loads the library and fails if it has not been built; there is no
CPU fallback.
"""
from . import _lib
from ._lib import OutOfMemoryError, RuntimeError_ as RuntimeError, ShapeError
from .narray import Bit, DFloat, Fused, Int32, Int64, NArray, NMath, SFloat, UInt64


class MemoryPool:
    """Cumo::CUDA::MemoryPool (reference: ext/cumo/cuda/memory_pool.cpp:140-260)."""

    @staticmethod
    def enable():
        return bool(_lib.lib.cumo_hip_pool_enable(1))

    @staticmethod
    def disable():
        return bool(_lib.lib.cumo_hip_pool_enable(0))

    @staticmethod
    def enabled():
        return bool(_lib.lib.cumo_hip_pool_enable(-1))

    @staticmethod
    def free_all_blocks(stream=None):
        if stream is None:
            _lib.call(_lib.lib.cumo_hip_pool_free_all_blocks)
        else:
            _lib.call(_lib.lib.cumo_hip_pool_free_all_blocks_stream, stream)

    n_free_blocks = staticmethod(lambda: _lib.lib.cumo_hip_pool_n_free_blocks())
    used_bytes = staticmethod(lambda: _lib.lib.cumo_hip_pool_used_bytes())
    free_bytes = staticmethod(lambda: _lib.lib.cumo_hip_pool_free_bytes())
    total_bytes = staticmethod(lambda: _lib.lib.cumo_hip_pool_total_bytes())


def synchronize():
    _lib.call(_lib.lib.cumo_hip_synchronize)


def device_count():
    return _lib.lib.cumo_hip_device_count()


__all__ = ["SFloat", "DFloat", "Int32", "Int64", "UInt64", "Bit", "NArray", "NMath", "Fused", "MemoryPool", "ShapeError",
           "OutOfMemoryError", "RuntimeError", "synchronize", "device_count"]
