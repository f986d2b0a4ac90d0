"""ctypes/numpy front end of the CPU checker (oracle/mc_oracle*.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py.  The product package never imports it.

Arrays are float32, C-contiguous, in the reference's NCHW blob layout.
"""
import ctypes
import glob
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmcoracle.so")

c_float_p = ctypes.POINTER(ctypes.c_float)
c_int_p = ctypes.POINTER(ctypes.c_int)


def build(force=False):
    """Compile the checker (and oracle/_ref when the reference checkout exists)."""
    if force:
        subprocess.check_call(["make", "-C", _HERE, "clean"], stdout=subprocess.DEVNULL)
    subprocess.check_call(["make", "-C", _HERE], stdout=subprocess.DEVNULL)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()


def _fp(a):
    return a.ctypes.data_as(c_float_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class ConvGeom(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "channels_in", "height_in", "width_in", "channels_out", "kernel_h", "kernel_w",
        "stride_h", "stride_w", "pad_h", "pad_w", "dilation_h", "dilation_w", "group",
        "transposed")]


def conv_geom(cin, h, w, cout, kernel, stride=1, pad=0, dilation=1, group=1, transposed=False):
    def two(v):
        return (v, v) if isinstance(v, int) else tuple(v)
    kh, kw = two(kernel)
    sh, sw = two(stride)
    ph, pw = two(pad)
    dh, dw = two(dilation)
    return ConvGeom(cin, h, w, cout, kh, kw, sh, sw, ph, pw, dh, dw, group, int(transposed))


# ---- BLAS plug -------------------------------------------------------------

_blas_handle = None


def find_openblas():
    """Path of the OpenBLAS bundled with scipy (CBLAS symbols prefixed scipy_), or None."""
    try:
        import scipy
    except ImportError:
        return None
    root = os.path.dirname(os.path.dirname(scipy.__file__))
    hits = sorted(glob.glob(os.path.join(root, "scipy.libs", "libscipy_openblas-*.so")))
    return hits[0] if hits else None


def use_openblas(enable=True, threads=None):
    """Route orc_gemm through OpenBLAS's cblas_sgemm, as the reference does
    (src/util/math_functions.cpp:8-16).  Returns the library path or None."""
    global _blas_handle
    if not enable:
        _lib.orc_set_sgemm(None)
        return None
    path = find_openblas()
    if path is None:
        return None
    if _blas_handle is None:
        _blas_handle = ctypes.CDLL(path)
    if threads is not None:
        _blas_handle.scipy_openblas_set_num_threads(int(threads))
    fn = ctypes.cast(_blas_handle.scipy_cblas_sgemm, ctypes.c_void_p)
    _lib.orc_set_sgemm(fn)
    return path


def openblas_threads():
    if _blas_handle is None:
        return 0
    return int(_blas_handle.scipy_openblas_get_num_threads())


# ---- prototypes --------------------------------------------------------------

_lib.orc_set_sgemm.argtypes = [ctypes.c_void_p]
_lib.orc_gemm.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                          ctypes.c_float, c_float_p, c_float_p, ctypes.c_float, c_float_p]
_lib.orc_im2col.argtypes = [c_float_p] + [ctypes.c_int] * 11 + [c_float_p]
_lib.orc_col2im.argtypes = [c_float_p] + [ctypes.c_int] * 11 + [c_float_p]
_lib.orc_conv_output_shape.argtypes = [ctypes.POINTER(ConvGeom), c_int_p, c_int_p]
_lib.orc_conv_forward.argtypes = [ctypes.POINTER(ConvGeom), ctypes.c_int, c_float_p, c_float_p,
                                  c_float_p, c_float_p]
_lib.orc_deconv_forward.argtypes = _lib.orc_conv_forward.argtypes
_lib.orc_inner_product.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, c_float_p, c_float_p,
                                   c_float_p, ctypes.c_int, c_float_p]
_lib.orc_exp.argtypes = [ctypes.c_int, c_float_p, c_float_p]
_lib.orc_powx.argtypes = [ctypes.c_int, c_float_p, ctypes.c_float, c_float_p]
_lib.orc_batch_norm.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, c_float_p, c_float_p,
                                c_float_p, c_float_p, ctypes.c_int, ctypes.c_float, c_float_p]
_lib.orc_scale.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, c_float_p, c_float_p,
                           c_float_p, c_float_p]
_lib.orc_bias.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, c_float_p, c_float_p,
                          c_float_p]
_lib.orc_relu.argtypes = [ctypes.c_size_t, c_float_p, ctypes.c_float, c_float_p]
_lib.orc_tanh.argtypes = [ctypes.c_size_t, c_float_p, c_float_p]
_lib.orc_sigmoid.argtypes = [ctypes.c_size_t, c_float_p, c_float_p]
_lib.orc_pooling_output_shape.argtypes = [ctypes.c_int] * 8 + [c_int_p, c_int_p]
_lib.orc_pooling.argtypes = [ctypes.c_int] * 10 + [c_float_p, c_float_p]
_lib.orc_eltwise.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(c_float_p), c_float_p,
                             ctypes.c_size_t, c_float_p]
_lib.orc_softmax.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, c_float_p, c_float_p]


# ---- numpy API ---------------------------------------------------------------

def gemm(transa, transb, M, N, K, alpha, A, B, beta, C):
    A, B = _f32(A), _f32(B)
    _lib.orc_gemm(int(transa), int(transb), M, N, K, alpha, _fp(A), _fp(B), beta, _fp(C))
    return C


def im2col(im, kernel, pad, stride, dilation):
    im = _f32(im)
    C, H, W = im.shape
    (kh, kw), (ph, pw), (sh, sw), (dh, dw) = kernel, pad, stride, dilation
    Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1
    Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1
    col = np.empty((C * kh * kw, Ho, Wo), np.float32)
    _lib.orc_im2col(_fp(im), C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, _fp(col))
    return col


def col2im(col, C, H, W, kernel, pad, stride, dilation):
    col = _f32(col)
    (kh, kw), (ph, pw), (sh, sw), (dh, dw) = kernel, pad, stride, dilation
    im = np.empty((C, H, W), np.float32)
    _lib.orc_col2im(_fp(col), C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, _fp(im))
    return im


def conv_output_shape(geom):
    ho, wo = ctypes.c_int(), ctypes.c_int()
    _lib.orc_conv_output_shape(ctypes.byref(geom), ctypes.byref(ho), ctypes.byref(wo))
    return ho.value, wo.value


def conv_forward(geom, x, w, bias=None):
    """Convolution (geom.transposed == 0) or Deconvolution forward of x [N,Cin,H,W]."""
    x, w = _f32(x), _f32(w)
    b = _f32(bias) if bias is not None else None
    ho, wo = conv_output_shape(geom)
    y = np.empty((x.shape[0], geom.channels_out, ho, wo), np.float32)
    fn = _lib.orc_deconv_forward if geom.transposed else _lib.orc_conv_forward
    fn(ctypes.byref(geom), x.shape[0], _fp(x), _fp(w), _fp(b) if b is not None else None, _fp(y))
    return y


def inner_product(x, w, bias=None, transpose=False):
    x, w = _f32(x), _f32(w)
    M, K = x.shape[0], int(np.prod(x.shape[1:]))
    N = w.shape[1] if transpose else w.shape[0]
    b = _f32(bias) if bias is not None else None
    y = np.empty((M, N), np.float32)
    _lib.orc_inner_product(M, N, K, _fp(x), _fp(w), _fp(b) if b is not None else None,
                           int(transpose), _fp(y))
    return y


def exp(a):
    a = _f32(a)
    y = np.empty_like(a)
    _lib.orc_exp(a.size, _fp(a), _fp(y))
    return y


def powx(a, b):
    a = _f32(a)
    y = np.empty_like(a)
    _lib.orc_powx(a.size, _fp(a), b, _fp(y))
    return y


def batch_norm(x, blob0, blob1, blob2, use_global_stats=True, eps=1e-5):
    x = _f32(x)
    num, ch = x.shape[0], (x.shape[1] if x.ndim > 1 else 1)
    spatial = x.size // (num * ch)
    y = np.empty_like(x)
    b0, b1, b2 = _f32(blob0), _f32(blob1), _f32(blob2)
    _lib.orc_batch_norm(num, ch, spatial, _fp(x), _fp(b0), _fp(b1), _fp(b2),
                        int(use_global_stats), eps, _fp(y))
    return y


def scale(x, gamma, beta=None, axis=1):
    x, gamma = _f32(x), _f32(gamma)
    outer = int(np.prod(x.shape[:axis]))
    inner = int(np.prod(x.shape[axis + gamma.ndim:]))
    b = _f32(beta) if beta is not None else None
    y = np.empty_like(x)
    _lib.orc_scale(outer, gamma.size, inner, _fp(x), _fp(gamma),
                   _fp(b) if b is not None else None, _fp(y))
    return y


def bias(x, beta, axis=1):
    x, beta = _f32(x), _f32(beta)
    outer = int(np.prod(x.shape[:axis]))
    inner = int(np.prod(x.shape[axis + beta.ndim:]))
    y = np.empty_like(x)
    _lib.orc_bias(outer, beta.size, inner, _fp(x), _fp(beta), _fp(y))
    return y


def relu(x, negative_slope=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_relu(x.size, _fp(x), negative_slope, _fp(y))
    return y


def tanh(x):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_tanh(x.size, _fp(x), _fp(y))
    return y


def sigmoid(x):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_sigmoid(x.size, _fp(x), _fp(y))
    return y


def pooling_output_shape(H, W, kernel, stride, pad):
    ho, wo = ctypes.c_int(), ctypes.c_int()
    _lib.orc_pooling_output_shape(H, W, kernel[0], kernel[1], stride[0], stride[1], pad[0], pad[1],
                                  ctypes.byref(ho), ctypes.byref(wo))
    return ho.value, wo.value


def pooling(x, method, kernel, stride=(1, 1), pad=(0, 0), global_pooling=False):
    """method: 'MAX' or 'AVE'; x [N,C,H,W]."""
    x = _f32(x)
    N, C, H, W = x.shape
    if global_pooling:
        kernel = (H, W)
    ho, wo = pooling_output_shape(H, W, kernel, stride, pad)
    y = np.empty((N, C, ho, wo), np.float32)
    _lib.orc_pooling({"MAX": 0, "AVE": 1}[method], N * C, H, W, kernel[0], kernel[1], stride[0],
                     stride[1], pad[0], pad[1], _fp(x), _fp(y))
    return y


def eltwise(bottoms, op="SUM", coeffs=None):
    bs = [_f32(b) for b in bottoms]
    arr = (c_float_p * len(bs))(*[_fp(b) for b in bs])
    co = _f32(coeffs) if coeffs is not None and len(coeffs) else None
    y = np.empty_like(bs[0])
    _lib.orc_eltwise({"PROD": 0, "SUM": 1, "MAX": 2}[op], len(bs), arr,
                     _fp(co) if co is not None else None, bs[0].size, _fp(y))
    return y


def softmax(x, axis=1):
    x = _f32(x)
    axis = axis % x.ndim
    outer = int(np.prod(x.shape[:axis]))
    inner = int(np.prod(x.shape[axis + 1:]))
    y = np.empty_like(x)
    _lib.orc_softmax(outer, x.shape[axis], inner, _fp(x), _fp(y))
    return y


# ---- detection tail (mc_oracle_det.cc) -----------------------------------------

_lib.orc_normalize.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, c_float_p, c_float_p,
                               ctypes.c_int, ctypes.c_int, ctypes.c_float, c_float_p]
_lib.orc_prior_box.argtypes = [ctypes.c_int] * 4 + [c_float_p, ctypes.c_int, c_float_p, ctypes.c_int,
                                                    c_float_p, ctypes.c_int, c_float_p, ctypes.c_int,
                                                    ctypes.c_int, ctypes.c_float, ctypes.c_float,
                                                    ctypes.c_float, c_float_p]
_lib.orc_generate_anchors.argtypes = [ctypes.c_int, c_float_p, ctypes.c_int, c_float_p, ctypes.c_int,
                                      c_float_p]
_lib.orc_generate_proposals.argtypes = [c_float_p, c_float_p, c_float_p, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_float,
                                        ctypes.c_int, c_float_p]
_lib.orc_sort_bbox.argtypes = [c_float_p, ctypes.c_int, ctypes.c_int]
_lib.orc_nms_pixel.argtypes = [ctypes.c_int, c_float_p, ctypes.c_float, ctypes.c_int, c_int_p]
_lib.orc_proposal.argtypes = [c_float_p, c_float_p, c_float_p, ctypes.c_int, ctypes.c_int,
                              ctypes.c_int, c_float_p, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                              ctypes.c_int, ctypes.c_float, c_float_p, c_float_p, c_int_p, c_float_p]
_lib.orc_detection_output.argtypes = [c_float_p, c_float_p, c_float_p] + [ctypes.c_int] * 8 + \
    [ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_int, c_float_p, ctypes.c_int]


_lib.orc_roi_pooling.argtypes = [c_float_p] + [ctypes.c_int] * 4 + [c_float_p] + [ctypes.c_int] * 3 + \
                                 [ctypes.c_float, c_float_p]
_lib.orc_psroi_pooling.argtypes = [c_float_p] + [ctypes.c_int] * 5 + [c_float_p, ctypes.c_int,
                                                                      ctypes.c_float, c_float_p]


def roi_pooling(x, rois, pooled_h, pooled_w, spatial_scale):
    """ROIPooling (roi_pooling_layer.cpp:37-110): x (N,C,H,W), rois (R,5) -> (R,C,ph,pw)."""
    x, rois = _f32(x), _f32(rois).reshape(-1, 5)
    n, c, h, w = x.shape
    y = np.empty((rois.shape[0], c, pooled_h, pooled_w), np.float32)
    rc = _lib.orc_roi_pooling(_fp(x), n, c, h, w, _fp(rois), rois.shape[0], pooled_h, pooled_w,
                              spatial_scale, _fp(y))
    if rc:
        raise ValueError("roi batch index outside [0, %d)" % n)
    return y


def psroi_pooling(x, rois, output_dim, group_size, spatial_scale):
    """PSROIPooling (psroi_pooling_layer.cpp:45-122): x (N, dim*g*g, H, W), rois (R,5) -> (R,dim,g,g)."""
    x, rois = _f32(x), _f32(rois).reshape(-1, 5)
    n, c, h, w = x.shape
    if c != output_dim * group_size * group_size:
        raise ValueError("input channel number does not match layer parameters")
    y = np.empty((rois.shape[0], output_dim, group_size, group_size), np.float32)
    rc = _lib.orc_psroi_pooling(_fp(x), n, output_dim, group_size, h, w, _fp(rois), rois.shape[0],
                                spatial_scale, _fp(y))
    if rc:
        raise ValueError("roi batch index outside [0, %d)" % n)
    return y


def normalize(x, scale, across_spatial=True, channel_shared=True, eps=1e-10):
    x, scale = _f32(x), _f32(scale).reshape(-1)
    n, c = x.shape[0], x.shape[1]
    y = np.empty_like(x)
    _lib.orc_normalize(n, c, x.size // (n * c), _fp(x), _fp(scale), int(across_spatial),
                       int(channel_shared), eps, _fp(y))
    return y


def _as_list(v):
    if v is None:
        return []
    return list(v) if isinstance(v, (list, tuple)) else [v]


def prior_box_aspect_ratios(param):
    """The list PriorBoxLayer::LayerSetUp builds (prior_box_layer.cpp:21-37)."""
    ars = [np.float32(1.0)]
    flip = param.get("flip", True)
    for ar in _as_list(param.get("aspect_ratio")):
        ar = np.float32(ar)
        if any(abs(float(ar) - float(a)) < 1e-6 for a in ars):
            continue
        ars.append(ar)
        if flip:
            ars.append(np.float32(1.0 / float(ar)))
    return np.array(ars, np.float32)


def prior_box(param, feat_shape, img_shape):
    mins = _f32(_as_list(param["min_size"]))
    maxs = _f32(_as_list(param.get("max_size")))
    ars = prior_box_aspect_ratios(param)
    var = _f32(_as_list(param.get("variance")) or [0.1])
    lh, lw = feat_shape[2], feat_shape[3]
    if "img_size" in param:
        ih = iw = int(param["img_size"])
    elif "img_h" in param:
        ih, iw = int(param["img_h"]), int(param["img_w"])
    else:
        ih, iw = img_shape[2], img_shape[3]
    if "step" in param:
        sh = sw = float(param["step"])
    else:
        sh, sw = float(param.get("step_h", 0)), float(param.get("step_w", 0))
    num_priors = len(ars) * len(mins) + len(maxs)
    dim = lh * lw * num_priors * 4
    out = np.empty((1, 2, dim), np.float32)
    _lib.orc_prior_box(lh, lw, ih, iw, _fp(mins), len(mins), _fp(maxs) if len(maxs) else None,
                       len(maxs), _fp(ars), len(ars), _fp(var), len(var), int(param.get("clip", False)),
                       sh, sw, float(param.get("offset", 0.5)), _fp(out))
    return out


def generate_anchors(base_size=16, ratios=(0.5, 1, 2), scales=(8, 16, 32)):
    r, s = _f32(ratios), _f32(scales)
    out = np.empty((len(r) * len(s), 4), np.float32)
    _lib.orc_generate_anchors(base_size, _fp(r), len(r), _fp(s), len(s), _fp(out))
    return out


def generate_proposals(fg_scores, bbox, anchors, im_h, im_w, min_bbox_size, feat_stride):
    fg_scores, bbox, anchors = _f32(fg_scores), _f32(bbox), _f32(anchors)
    A, (H, W) = anchors.shape[0], fg_scores.shape[-2:]
    out = np.empty((A * H * W, 5), np.float32)
    _lib.orc_generate_proposals(_fp(fg_scores), _fp(bbox), _fp(anchors), A, H, W, im_h, im_w,
                                min_bbox_size, feat_stride, _fp(out))
    return out


def sort_bbox(rois, num_top):
    rois = _f32(rois).copy()
    _lib.orc_sort_bbox(_fp(rois), rois.shape[0], num_top)
    return rois


def nms_pixel(proposals, thr, max_rois):
    proposals = _f32(proposals)
    kept = np.empty(max_rois, np.int32)
    n = _lib.orc_nms_pixel(proposals.shape[0], _fp(proposals), thr, max_rois,
                           kept.ctypes.data_as(c_int_p))
    return kept[:n].copy()


def proposal(param, scores, bbox, im_info, ntop=1, details=False):
    """ProposalLayer forward.  Returns [rois] or [rois, scores]; with details=True
    also the kept indices (positions in the sorted table) and the sorted table."""
    scores, bbox, im_info = _f32(scores), _f32(bbox), _f32(im_info).reshape(-1)
    assert scores.shape[0] == 1, "Only support single scale."
    ratios = _as_list(param.get("ratio")) or [0.5, 1, 2]
    scales = _as_list(param.get("scale")) or [8, 16, 32]
    anchors = generate_anchors(int(param.get("base_size", 16)), ratios, scales)
    A, H, W = anchors.shape[0], scores.shape[2], scores.shape[3]
    post = int(param.get("post_nms_topn", 300))
    rois = np.empty((post, 5), np.float32)
    rs = np.empty(post, np.float32)
    kept = np.empty(post, np.int32)
    table = np.empty((A * H * W, 5), np.float32)
    r = _lib.orc_proposal(_fp(scores), _fp(bbox), _fp(im_info), A, H, W, _fp(anchors),
                          int(param.get("feat_stride", 16)), int(param.get("min_size", 16)),
                          int(param.get("pre_nms_topn", 6000)), post,
                          float(param.get("nms_thresh", 0.7)), _fp(rois), _fp(rs),
                          kept.ctypes.data_as(c_int_p), _fp(table))
    tops = [rois[:r].copy()] + ([rs[:r].copy()] if ntop > 1 else [])
    if details:
        return tops, kept[:r].copy(), table
    return tops


_CODE = {"CORNER": 1, "CENTER_SIZE": 2, "CORNER_SIZE": 3}


def detection_output(param, loc, conf, prior):
    loc, conf, prior = _f32(loc), _f32(conf), _f32(prior)
    num = loc.shape[0]
    num_classes = int(param["num_classes"])
    share = bool(param.get("share_location", True))
    num_priors = prior.shape[2] // 4
    nms = param.get("nms_param", {})
    max_rows = max(num, num * num_priors * num_classes)
    keep = int(param.get("keep_top_k", -1))
    if keep > -1:
        max_rows = max(num, min(max_rows, num * max(keep, num_classes * max(1, int(nms.get("top_k", num_priors))))))
    out = np.empty((max_rows, 7), np.float32)
    n = _lib.orc_detection_output(
        _fp(loc), _fp(conf), _fp(prior), num, num_priors, num_classes, int(share),
        int(param.get("background_label_id", 0)), _CODE[str(param.get("code_type", "CORNER"))],
        int(param.get("variance_encoded_in_target", False)), keep,
        float(param.get("confidence_threshold", -3.4028234663852886e38)),
        float(nms.get("nms_threshold", 0.3)), float(nms.get("eta", 1.0)), int(nms.get("top_k", -1)),
        _fp(out), max_rows)
    if n == -2:
        raise ValueError("Could not find location predictions for label -1")  # the reference's LOG(FATAL)
    assert n >= 0, "detection_output: row buffer too small"
    return out[:n].copy()


# ---- less common layers (mc_oracle_zoo.c) ------------------------------------------

_I, _F, _Z = ctypes.c_int, ctypes.c_float, ctypes.c_size_t
_lib.orc_bn.argtypes = [_I, _I, _I] + [c_float_p] * 6
_lib.orc_conv_dw.argtypes = [_I] * 12 + [c_float_p] * 4
_lib.orc_power.argtypes = [_Z, c_float_p, _F, _F, _F, c_float_p]
_lib.orc_exp_layer.argtypes = [_Z, c_float_p, _F, _F, _F, c_float_p]
_lib.orc_log_layer.argtypes = [_Z, c_float_p, _F, _F, _F, c_float_p]
_lib.orc_absval.argtypes = [_Z, c_float_p, c_float_p]
_lib.orc_bnll.argtypes = [_Z, c_float_p, c_float_p]
_lib.orc_elu.argtypes = [_Z, c_float_p, _F, c_float_p]
_lib.orc_threshold.argtypes = [_Z, c_float_p, _F, c_float_p]
_lib.orc_prelu.argtypes = [_I, _I, _I, c_float_p, c_float_p, _I, c_float_p]
_lib.orc_lrn_across.argtypes = [_I] * 5 + [_F] * 3 + [c_float_p, c_float_p]
_lib.orc_argmax.argtypes = [_I] * 5 + [c_float_p, c_float_p]
_lib.orc_reduction.argtypes = [_I, _I, _I, _F, c_float_p, c_float_p]
_lib.orc_mvn.argtypes = [_I, _I, _I, _F, c_float_p, c_float_p]
_lib.orc_embed.argtypes = [_I, _I] + [c_float_p] * 4
_lib.orc_shuffle_channel.argtypes = [_I] * 4 + [c_float_p, c_float_p]


def _two(v):
    return (v, v) if np.isscalar(v) else tuple(v)


def bn(x, slope, bias, mean, mult):
    """BN layer (bn_layer.cpp:77-147): (x - mean) * mult * slope + bias per channel."""
    x = _f32(x)
    num, ch = x.shape[0], x.shape[1]
    y = np.empty_like(x)
    s, b, m, v = (_f32(a).reshape(-1) for a in (slope, bias, mean, mult))
    _lib.orc_bn(num, ch, x.size // (num * ch), _fp(x), _fp(s), _fp(b), _fp(m), _fp(v), _fp(y))
    return y


def conv_dw(x, w, bias=None, stride=1, pad=0, dilation=1):
    """ConvolutionDepthwise (conv_dw_layer.cpp:105-158): x (N,C,H,W), w (C,1,kh,kw)."""
    x, w = _f32(x), _f32(w)
    n, c, h, wd = x.shape
    kh, kw = w.shape[2], w.shape[3]
    (sh, sw), (ph, pw), (dh, dw) = _two(stride), _two(pad), _two(dilation)
    ho = (h + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1
    wo = (wd + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1
    y = np.empty((n, c, ho, wo), np.float32)
    b = _f32(bias) if bias is not None else None
    _lib.orc_conv_dw(n, c, h, wd, kh, kw, sh, sw, ph, pw, dh, dw, _fp(x), _fp(w),
                     _fp(b) if b is not None else None, _fp(y))
    return y


def power(x, power=1.0, scale=1.0, shift=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_power(x.size, _fp(x), scale, shift, power, _fp(y))
    return y


def exp_layer(x, base=-1.0, scale=1.0, shift=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_exp_layer(x.size, _fp(x), base, scale, shift, _fp(y))
    return y


def log_layer(x, base=-1.0, scale=1.0, shift=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_log_layer(x.size, _fp(x), base, scale, shift, _fp(y))
    return y


def absval(x):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_absval(x.size, _fp(x), _fp(y))
    return y


def bnll(x):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_bnll(x.size, _fp(x), _fp(y))
    return y


def elu(x, alpha=1.0):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_elu(x.size, _fp(x), alpha, _fp(y))
    return y


def threshold(x, threshold=0.0):
    x = _f32(x)
    y = np.empty_like(x)
    _lib.orc_threshold(x.size, _fp(x), threshold, _fp(y))
    return y


def prelu(x, slope, channel_shared=False):
    x, slope = _f32(x), _f32(slope).reshape(-1)
    y = np.empty_like(x)
    num, ch = x.shape[0], x.shape[1]
    _lib.orc_prelu(num, ch, x.size // max(1, num * ch), _fp(x), _fp(slope), int(channel_shared),
                   _fp(y))
    return y


def lrn(x, local_size=5, alpha=1.0, beta=0.75, k=1.0, norm_region="ACROSS_CHANNELS"):
    """LRN (lrn_layer.cpp:112-164).  The within-channel region is the reference's own
    chain: Power(2) -> average Pooling -> Power(1 + alpha*., -beta) -> Eltwise PROD."""
    x = _f32(x)
    if str(norm_region) == "ACROSS_CHANNELS":
        n, c, h, w = x.shape
        y = np.empty_like(x)
        _lib.orc_lrn_across(n, c, h, w, local_size, alpha, beta, k, _fp(x), _fp(y))
        return y
    pre_pad = (local_size - 1) // 2
    sq = power(x, power=2.0)
    pooled = pooling(sq, "AVE", (local_size, local_size), (1, 1), (pre_pad, pre_pad))
    denom = power(pooled, power=-beta, scale=alpha, shift=1.0)
    return eltwise([x, denom], "PROD")


def argmax(x, top_k=1, out_max_val=False, axis=None):
    """ArgMax (argmax_layer.cpp:36-93)."""
    x = _f32(x)
    if axis is not None:
        axis = axis % x.ndim
        dim = x.shape[axis]
        dist = int(np.prod(x.shape[axis + 1:]))
        shape = list(x.shape)
        shape[axis] = top_k
        layout = 1 if out_max_val else 0
    else:
        dim = int(np.prod(x.shape[1:]))
        dist = 1
        shape = [1] * max(3, x.ndim)
        shape[0], shape[2] = x.shape[0], top_k
        if out_max_val:
            shape[1] = 2
        layout = 2 if out_max_val else 0
    y = np.empty(shape, np.float32)
    _lib.orc_argmax(x.size, dim, dist, top_k, layout, _fp(x), _fp(y))
    return y


def reduction(x, operation="SUM", axis=0, coeff=1.0):
    x = _f32(x)
    axis = axis % x.ndim if x.ndim else 0
    num = int(np.prod(x.shape[:axis]))
    y = np.empty(x.shape[:axis], np.float32)
    _lib.orc_reduction({"SUM": 1, "ASUM": 2, "SUMSQ": 3, "MEAN": 4}[str(operation)], num,
                       x.size // max(1, num), coeff, _fp(x), _fp(y))
    return y


def mvn(x, normalize_variance=True, across_channels=False, eps=1e-9):
    x = _f32(x)
    x4 = x.reshape(x.shape + (1,) * (4 - x.ndim))
    num = x4.shape[0] if across_channels else x4.shape[0] * x4.shape[1]
    y = np.empty_like(x4)
    _lib.orc_mvn(num, x4.size // num, int(normalize_variance), eps, _fp(x4), _fp(y))
    return y


def embed(x, weight, bias=None):
    x, weight = _f32(x), _f32(weight)
    b = _f32(bias) if bias is not None else None
    n_out = weight.shape[1]
    y = np.empty(x.shape + (n_out,), np.float32)
    _lib.orc_embed(x.size, n_out, _fp(x), _fp(weight), _fp(b) if b is not None else None, _fp(y))
    return y


def shuffle_channel(x, group):
    x = _f32(x)
    y = np.empty_like(x)
    n, c = x.shape[0], x.shape[1]
    _lib.orc_shuffle_channel(n, c, x.size // (n * c), group, _fp(x), _fp(y))
    return y


def spp(x, pyramid_height, pool="MAX"):
    """SPP (spp_layer.cpp:16-199): per level 2^l bins per side through the Pooling layer's
    own arithmetic, flattened and concatenated on axis 1."""
    x = _f32(x)
    h, w = x.shape[2], x.shape[3]
    outs = []
    for level in range(pyramid_height):
        bins = 2 ** level
        kh, kw = -(-h // bins), -(-w // bins)
        ph, pw = (kh * bins - h + 1) // 2, (kw * bins - w + 1) // 2
        outs.append(pooling(x, str(pool), (kh, kw), (kh, kw), (ph, pw)))
    if pyramid_height == 1:
        return outs[0]
    return np.ascontiguousarray(np.concatenate([o.reshape(o.shape[0], -1) for o in outs], axis=1))
