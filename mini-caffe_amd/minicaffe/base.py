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
    _declare_c_api(lib)
    return lib


NetHandle = ctypes.c_void_p
BlobHandle = ctypes.c_void_p
_int_p = ctypes.POINTER(ctypes.c_int)


def _declare_c_api(lib):
    """Argument and return types of include/caffe/c_api.h."""
    lib.CaffeGetLastError.restype = ctypes.c_char_p
    lib.CaffeBlobData.restype = ctypes.POINTER(ctypes.c_float)
    for fn in ("CaffeBlobNum", "CaffeBlobChannels", "CaffeBlobHeight", "CaffeBlobWidth",
               "CaffeBlobCount", "CaffeBlobData"):
        getattr(lib, fn).argtypes = [BlobHandle]
    lib.CaffeBlobReshape.argtypes = [BlobHandle, ctypes.c_int, _int_p]
    lib.CaffeBlobShape.argtypes = [BlobHandle, _int_p, ctypes.POINTER(_int_p)]
    lib.CaffeNetCreate.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.POINTER(NetHandle)]
    lib.CaffeNetCreateFromBuffer.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_char_p,
                                             ctypes.c_int, ctypes.POINTER(NetHandle)]
    lib.CaffeNetDestroy.argtypes = [NetHandle]
    lib.CaffeNetMarkOutput.argtypes = [NetHandle, ctypes.c_char_p]
    lib.CaffeNetForward.argtypes = [NetHandle]
    lib.CaffeNetGetBlob.argtypes = [NetHandle, ctypes.c_char_p, ctypes.POINTER(BlobHandle)]
    names_p = ctypes.POINTER(ctypes.POINTER(ctypes.c_char_p))
    handles_p = ctypes.POINTER(ctypes.POINTER(BlobHandle))
    lib.CaffeNetListBlob.argtypes = [NetHandle, _int_p, names_p, handles_p]
    lib.CaffeNetListParam.argtypes = [NetHandle, _int_p, names_p, handles_p]
    lib.CaffeProfilerScopeStart.argtypes = [ctypes.c_char_p]
    lib.CaffeProfilerDump.argtypes = [ctypes.c_char_p]
    lib.CaffeSetMode.argtypes = [ctypes.c_int, ctypes.c_int]
    lib.mcCurrentStream.restype = ctypes.c_void_p


LIB = _load()


def check_call(ret):
    """Net/Blob C ABI: 0 is success, -1 carries CaffeGetLastError()
    (reference python/minicaffe/base.py:67-78)."""
    if ret != 0:
        raise MiniCaffeError(LIB.CaffeGetLastError().decode("utf-8", "replace"))


def c_str(string):
    return ctypes.c_char_p(string.encode("utf-8"))


def py_str(cstr):
    return cstr.decode("utf-8")


def check_mc(ret):
    """Kernel-level ABI: 0 is success, anything else carries mcLastError()."""
    if ret != 0:
        raise MiniCaffeError(LIB.mcLastError().decode("utf-8", "replace"))
