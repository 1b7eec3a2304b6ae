"""Seeded synthetic tensors of the benchmark configurations.

The generator is the C++ host layer's (``eddl_hip_synth.cpp`` in ``libeddlhip_host.so``: ``std::mt19937(seed)``,
``u = (word >> 8) * 2**-24``, explicit Box-Muller in double precision), called through ctypes, so that a C++ host
(``eddl_hip::synth_he_normal``, ``tests/host/net_driver.cpp``) and this Python host build bit-identical inputs and
parameters from a seed alone.  Values are drawn in row-major order, tensor after tensor in the order of the calls.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "host", "libeddlhip_host.so")
_lib = None


def _load():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError("%s is missing: build it with `make -C eddl_amd/host`" % _LIB_PATH)
        lib = ctypes.CDLL(_LIB_PATH)
        lib.eddl_synth_new.restype = ctypes.c_void_p
        lib.eddl_synth_new.argtypes = [ctypes.c_uint32]
        lib.eddl_synth_free.argtypes = [ctypes.c_void_p]
        lib.eddl_synth_words.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t]
        lib.eddl_synth_uniform.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_float]
        lib.eddl_synth_normal.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_float]
        _lib = lib
    return _lib


class Synth:
    """One seeded stream; every call continues it."""

    def __init__(self, seed):
        self._lib = _load()
        self._h = self._lib.eddl_synth_new(int(seed) & 0xFFFFFFFF)

    def __del__(self):
        try:
            if self._h:
                self._lib.eddl_synth_free(self._h)
                self._h = None
        except Exception:
            pass

    def words(self, n):
        out = np.empty(n, np.uint32)
        self._lib.eddl_synth_words(self._h, out.ctypes.data, n)
        return out

    def uniform(self, shape, lo=0.0, hi=1.0):
        out = np.empty(shape, np.float32)
        self._lib.eddl_synth_uniform(self._h, out.ctypes.data, out.size, lo, hi)
        return out

    def normal(self, shape, mean=0.0, stddev=1.0):
        out = np.empty(shape, np.float32)
        self._lib.eddl_synth_normal(self._h, out.ctypes.data, out.size, mean, stddev)
        return out
