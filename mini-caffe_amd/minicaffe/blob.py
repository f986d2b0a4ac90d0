"""Blob: numpy view of a net's blob (mirror of reference python/minicaffe/blob.py:9-66)."""
import ctypes

import numpy as np

from .base import LIB, check_call, MiniCaffeError


class Blob(object):
    """Reference to a blob owned by a Net; never constructed by users."""

    def __init__(self, handle):
        self.handle = handle

    @property
    def shape(self):
        n = ctypes.c_int()
        shape = ctypes.POINTER(ctypes.c_int)()
        check_call(LIB.CaffeBlobShape(self.handle, ctypes.byref(n), ctypes.byref(shape)))
        return [shape[i] for i in range(n.value)]

    def reshape(self, *shape):
        """Change the blob's shape; arrays returned by `data` before become invalid."""
        arr = (ctypes.c_int * len(shape))(*shape)
        check_call(LIB.CaffeBlobReshape(self.handle, len(shape), arr))

    @property
    def count(self):
        return LIB.CaffeBlobCount(self.handle)

    @property
    def data(self):
        """float32 array sharing the blob's host memory.  Asking for it marks the
        host copy as the valid one (device results are copied back first)."""
        shape = self.shape
        ptr = LIB.CaffeBlobData(self.handle)
        if not ptr:
            raise MiniCaffeError(LIB.CaffeGetLastError().decode("utf-8", "replace"))
        count = int(np.prod(shape)) if shape else 1
        if count == 0:
            return np.zeros(shape, np.float32)
        return np.ctypeslib.as_array(ptr, shape=(count,)).reshape(shape)
