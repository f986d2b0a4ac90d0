"""Python front end of the MI355X build of Mini-Caffe's forward path.

Same surface as the reference's `minicaffe` package (python/minicaffe/__init__.py):
Net, Blob, set_mode helpers and the profiler, bound through ctypes to libcaffe.so.
"""
from .base import LIB, LIB_PATH, MiniCaffeError, check_call  # noqa: F401
from .blob import Blob  # noqa: F401
from .net import Net  # noqa: F401
from . import kernels  # noqa: F401  (declares the prototypes of the mc* kernel entry points)


def check_gpu_available():
    return LIB.CaffeGPUAvailable() == 1


def set_runtime_mode(mode, device=0):
    """mode: 0 = CPU (build/reshape only), 1 = GPU (HIP)."""
    check_call(LIB.CaffeSetMode(mode, device))


def memory_pool_clear():
    check_call(LIB.CaffeMemoryPoolClear())


class Profiler(object):
    """chrome://tracing profiler (reference python/minicaffe/profiler.py)."""

    @staticmethod
    def enable():
        check_call(LIB.CaffeProfilerEnable())

    @staticmethod
    def disable():
        check_call(LIB.CaffeProfilerDisable())

    @staticmethod
    def open_scope(name):
        check_call(LIB.CaffeProfilerScopeStart(name.encode("utf-8")))

    @staticmethod
    def close_scope():
        check_call(LIB.CaffeProfilerScopeEnd())

    @staticmethod
    def dump(fn):
        check_call(LIB.CaffeProfilerDump(fn.encode("utf-8")))
