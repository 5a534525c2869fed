"""ctypes wrapper of oracle/liboracle_c.so (TEST INFRASTRUCTURE ONLY)."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATH = os.path.join(_HERE, "liboracle_c.so")


def build():
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle_c.so"], check=True, capture_output=True)


def load():
    if not os.path.exists(_PATH):
        build()
    lib = ctypes.CDLL(_PATH)
    fp = ctypes.POINTER(ctypes.c_float)
    lib.oc_num_threads.restype = ctypes.c_int
    lib.oc_add_f32.argtypes = [fp, fp, fp, ctypes.c_int64]
    lib.oc_add_f32.restype = None
    lib.oc_sum_f32.argtypes = [fp, ctypes.c_int64]
    lib.oc_sum_f32.restype = ctypes.c_float
    for n in ("oc_argmax_f32", "oc_argmin_f32"):
        getattr(lib, n).argtypes = [fp, ctypes.c_int64]
        getattr(lib, n).restype = ctypes.c_int64
    return lib


def _p(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


class OracleC:
    def __init__(self):
        self.lib = load()
        self.threads = self.lib.oc_num_threads()

    def add(self, a, b, out=None):
        out = np.empty_like(a) if out is None else out
        self.lib.oc_add_f32(_p(a), _p(b), _p(out), a.size)
        return out

    def sum(self, x):
        return np.float32(self.lib.oc_sum_f32(_p(x), x.size))

    def argmax(self, x):
        return int(self.lib.oc_argmax_f32(_p(x), x.size))

    def argmin(self, x):
        return int(self.lib.oc_argmin_f32(_p(x), x.size))
