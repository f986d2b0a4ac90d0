"""Net: mirror of the reference's ctypes Net (reference python/minicaffe/net.py:13-122)."""
import ctypes
from collections import defaultdict

from .base import LIB, BlobHandle, NetHandle, c_str, check_call, py_str
from .blob import Blob


class Net(object):
    """A network built from a prototxt (+ optional caffemodel).

    Net(prototxt_path, caffemodel_path) as in the reference, or
    Net.from_buffers(prototxt_text, caffemodel_bytes) for in-memory definitions.
    """

    def __init__(self, prototxt, caffemodel):
        self.handle = NetHandle()
        check_call(LIB.CaffeNetCreate(c_str(prototxt), c_str(caffemodel),
                                      ctypes.byref(self.handle)))

    @classmethod
    def from_buffers(cls, prototxt_text, caffemodel_bytes=b""):
        self = cls.__new__(cls)
        self.handle = NetHandle()
        if isinstance(prototxt_text, str):
            prototxt_text = prototxt_text.encode("utf-8")
        check_call(LIB.CaffeNetCreateFromBuffer(prototxt_text, len(prototxt_text),
                                                caffemodel_bytes or None, len(caffemodel_bytes),
                                                ctypes.byref(self.handle)))
        return self

    def __del__(self):
        if getattr(self, "handle", None):
            LIB.CaffeNetDestroy(self.handle)
            self.handle = None

    def get_blob(self, name):
        handle = BlobHandle()
        check_call(LIB.CaffeNetGetBlob(self.handle, c_str(name), ctypes.byref(handle)))
        return Blob(handle)

    def _list(self, fn):
        n = ctypes.c_int()
        names = ctypes.POINTER(ctypes.c_char_p)()
        handles = ctypes.POINTER(BlobHandle)()
        check_call(fn(self.handle, ctypes.byref(n), ctypes.byref(names), ctypes.byref(handles)))
        return [(py_str(names[i]), Blob(BlobHandle(handles[i]))) for i in range(n.value)]

    @property
    def blobs(self):
        """dict name -> Blob of every internal blob."""
        return dict(self._list(LIB.CaffeNetListBlob))

    @property
    def params(self):
        """dict layer name -> [(param name, Blob)], in layer order."""
        params = defaultdict(list)
        for name, blob in self._list(LIB.CaffeNetListParam):
            params["_".join(name.split("_")[:-1])].append((name, blob))
        return params

    @property
    def param_list(self):
        """[(param name, Blob)] in net order."""
        return self._list(LIB.CaffeNetListParam)

    def mark_output(self, name):
        """Keep an internal blob's memory from being recycled so it can be read after forward."""
        check_call(LIB.CaffeNetMarkOutput(self.handle, c_str(name)))

    def forward(self, **kwargs):
        """Fill the named input blobs from numpy arrays, then run the net."""
        for k, v in kwargs.items():
            blob = self.get_blob(k)
            blob.reshape(*v.shape)
            blob.data[...] = v
        check_call(LIB.CaffeNetForward(self.handle))
