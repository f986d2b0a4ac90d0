"""Loads libcaffe.so, the HIP build of Mini-Caffe's forward path.

Mirrors the loader of the reference's ctypes binding (reference
python/minicaffe/base.py:17-47): find the shared library next to the package,
declare the return types ctypes cannot guess, and turn a non-zero return code
into a Python exception carrying CaffeGetLastError().
There is no fallback: if the library is missing or does not load, importing
this module raises.
"""
import ctypes
import os

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_PKG), "lib", "libcaffe.so")


class MiniCaffeError(RuntimeError):
    """Raised when a library call reports failure."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise MiniCaffeError(
            "libcaffe.so not found at %s: build it first (python -c 'import __graft_entry__ as g; "
            "g.build()' or make -C mini-caffe_amd/csrc)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    lib.mcLastError.restype = ctypes.c_char_p
    return lib


LIB = _load()


def check_mc(ret):
    """Kernel-level ABI: 0 is success, anything else carries mcLastError()."""
    if ret != 0:
        raise MiniCaffeError(LIB.mcLastError().decode("utf-8", "replace"))
