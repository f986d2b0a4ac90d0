"""ctypes access to oracle/_ref/libref_math.so: the reference's own
src/util/{im2col,math_functions}.cpp compiled as they lie and linked against the
OpenBLAS bundled with scipy.  Used only to pin the oracle."""
import ctypes
import os

import numpy as np

_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref",
                     "libref_math.so")
fp = ctypes.POINTER(ctypes.c_float)


def available():
    return os.path.exists(_PATH)


def load():
    lib = ctypes.CDLL(_PATH)
    # mangled names of caffe::im2col_cpu<float>, caffe::col2im_cpu<float> and friends
    lib.im2col = lib._ZN5caffe10im2col_cpuIfEEvPKT_iiiiiiiiiiiPS1_
    lib.col2im = lib._ZN5caffe10col2im_cpuIfEEvPKT_iiiiiiiiiiiPS1_
    lib.im2col.argtypes = [fp] + [ctypes.c_int] * 11 + [fp]
    lib.col2im.argtypes = [fp] + [ctypes.c_int] * 11 + [fp]
    lib.gemm = lib._ZN5caffe14caffe_cpu_gemmE15CBLAS_TRANSPOSES0_iiifPKfS2_fPf
    lib.gemm.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                         ctypes.c_float, fp, fp, ctypes.c_float, fp]
    lib.exp = lib._ZN5caffe9caffe_expEiPKfPf
    lib.exp.argtypes = [ctypes.c_int, fp, fp]
    lib.powx = lib._ZN5caffe10caffe_powxEiPKffPf
    lib.powx.argtypes = [ctypes.c_int, fp, ctypes.c_float, fp]
    lib.div = lib._ZN5caffe9caffe_divEiPKfS1_Pf
    lib.div.argtypes = [ctypes.c_int, fp, fp, fp]
    lib.axpy = lib._ZN5caffe10caffe_axpyEifPKfPf
    lib.axpy.argtypes = [ctypes.c_int, ctypes.c_float, fp, fp]
    lib.scale = lib._ZN5caffe15caffe_cpu_scaleEifPKfPf
    lib.scale.argtypes = [ctypes.c_int, ctypes.c_float, fp, fp]
    return lib


def p(a):
    return a.ctypes.data_as(fp)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)
