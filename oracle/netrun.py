"""Runs a net description (minicaffe.craft spec) on the CPU oracle.

TEST INFRASTRUCTURE ONLY.  Walks the layers in file order as the reference's
Net::Forward does (reference src/net.cpp:212-233: in-place tops overwrite their
bottoms) and evaluates each with the restated CPU arithmetic of oracle/.
"""
import numpy as np

import oracle

def _pair(p, rep, h, w, default):
    if h in p or w in p:
        return int(p.get(h, default)), int(p.get(w, default))
    v = p.get(rep, default)
    if isinstance(v, (list, tuple)):
        return (int(v[0]), int(v[0])) if len(v) == 1 else (int(v[0]), int(v[1]))
    return int(v), int(v)


def _conv(layer, x, transposed):
    p = layer["convolution_param"]
    k = _pair(p, "kernel_size", "kernel_h", "kernel_w", 0)
    s = _pair(p, "stride", "stride_h", "stride_w", 1)
    pad = _pair(p, "pad", "pad_h", "pad_w", 0)
    d = _pair(p, "dilation", "_", "_", 1)
    g = oracle.conv_geom(x.shape[1], x.shape[2], x.shape[3], p["num_output"], k, s, pad, d,
                         p.get("group", 1), transposed)
    blobs = layer["blobs"]
    bias = blobs[1] if p.get("bias_term", True) else None
    return oracle.conv_forward(g, x, blobs[0], bias)


def _canon(axis, ndim):
    return axis + ndim if axis < 0 else axis


def run_layer(layer, bottoms):
    """Returns the list of top arrays of one layer."""
    t = layer["type"]
    x = bottoms[0] if bottoms else None
    if t == "Convolution":
        return [_conv(layer, x, False)]
    if t == "Deconvolution":
        return [_conv(layer, x, True)]
    if t == "InnerProduct":
        p = layer["inner_product_param"]
        axis = _canon(p.get("axis", 1), x.ndim)
        x2 = x.reshape(int(np.prod(x.shape[:axis])), -1)
        b = layer["blobs"]
        y = oracle.inner_product(x2, b[0], b[1] if p.get("bias_term", True) else None,
                                 p.get("transpose", False))
        return [y.reshape(tuple(x.shape[:axis]) + (p["num_output"],))]
    if t == "BatchNorm":
        p = layer.get("batch_norm_param", {})
        b = layer["blobs"]
        return [oracle.batch_norm(x, b[0], b[1], b[2], p.get("use_global_stats", True),
                                  p.get("eps", 1e-5))]
    if t == "Scale":
        p = layer.get("scale_param", {})
        b = layer["blobs"]
        axis = _canon(p.get("axis", 1), x.ndim)
        return [oracle.scale(x, b[0], b[1] if p.get("bias_term", False) else None, axis)]
    if t == "Bias":
        p = layer.get("bias_param", {})
        return [oracle.bias(x, layer["blobs"][0], _canon(p.get("axis", 1), x.ndim))]
    if t == "ReLU":
        slope = layer.get("relu_param", {}).get("negative_slope", 0.0)
        return [oracle.relu(x, slope)]
    if t == "TanH":
        return [oracle.tanh(x)]
    if t == "Sigmoid":
        return [oracle.sigmoid(x)]
    if t == "Pooling":
        p = layer["pooling_param"]
        g = p.get("global_pooling", False)
        k = (0, 0) if g else _pair(p, "kernel_size", "kernel_h", "kernel_w", 0)
        return [oracle.pooling(x, str(p.get("pool", "MAX")), k,
                               _pair(p, "stride", "stride_h", "stride_w", 1),
                               _pair(p, "pad", "pad_h", "pad_w", 0), g)]
    if t == "Eltwise":
        p = layer.get("eltwise_param", {})
        return [oracle.eltwise(bottoms, str(p.get("operation", "SUM")), p.get("coeff"))]
    if t == "Softmax":
        return [oracle.softmax(x, layer.get("softmax_param", {}).get("axis", 1))]
    if t == "Concat":
        axis = _canon(layer.get("concat_param", {}).get("axis", 1), x.ndim)
        return [np.ascontiguousarray(np.concatenate(bottoms, axis=axis))]
    if t == "Slice":
        p = layer.get("slice_param", {})
        axis = _canon(p.get("axis", 1), x.ndim)
        pts = p.get("slice_point")
        ntop = len(layer["top"])
        if pts is None:
            parts = np.split(x, ntop, axis=axis)
        else:
            parts = np.split(x, list(pts) if isinstance(pts, (list, tuple)) else [pts], axis=axis)
        return [np.ascontiguousarray(a) for a in parts]
    if t == "Flatten":
        p = layer.get("flatten_param", {})
        a0, a1 = _canon(p.get("axis", 1), x.ndim), _canon(p.get("end_axis", -1), x.ndim)
        return [x.reshape(x.shape[:a0] + (-1,) + x.shape[a1 + 1:])]
    if t == "Reshape":
        p = layer["reshape_param"]
        dims = list(p["shape"]["dim"])
        axis = p.get("axis", 0)
        start = axis if axis >= 0 else x.ndim + axis + 1
        na = p.get("num_axes", -1)
        end = x.ndim if na == -1 else start + na
        new = [x.shape[start + i] if d == 0 else d for i, d in enumerate(dims)]
        shape = list(x.shape[:start]) + new + list(x.shape[end:])
        return [x.reshape(shape)]
    if t == "Permute":
        order = list(layer["permute_param"]["order"])
        order += [i for i in range(x.ndim) if i not in order]
        return [np.ascontiguousarray(np.transpose(x, order))]
    if t == "Split":
        return [x.copy() for _ in layer["top"]]
    if t == "Normalize":
        p = layer.get("norm_param", {})
        return [oracle.normalize(x, layer["blobs"][0], p.get("across_spatial", True),
                                 p.get("channel_shared", True), p.get("eps", 1e-10))]
    if t == "PriorBox":
        return [oracle.prior_box(layer["prior_box_param"], x.shape, bottoms[1].shape)]
    if t == "Proposal":
        return oracle.proposal(layer.get("proposal_param", {}), bottoms[0], bottoms[1], bottoms[2],
                               len(layer["top"]))
    if t == "DetectionOutput":
        return [oracle.detection_output(layer["detection_output_param"], bottoms[0], bottoms[1],
                                        bottoms[2])]
    if t == "ROIPooling":
        p = layer["roi_pooling_param"]
        return [oracle.roi_pooling(x, bottoms[1], p["pooled_h"], p["pooled_w"],
                                   p.get("spatial_scale", 1.0))]
    if t == "PSROIPooling":
        p = layer["psroi_pooling_param"]
        return [oracle.psroi_pooling(x, bottoms[1], p["output_dim"], p["group_size"],
                                     p["spatial_scale"])]
    if t == "ConvolutionDepthwise":
        p = layer["convolution_param"]
        blobs = layer["blobs"]
        return [oracle.conv_dw(x, blobs[0], blobs[1] if p.get("bias_term", True) else None,
                               _pair(p, "stride", "stride_h", "stride_w", 1),
                               _pair(p, "pad", "pad_h", "pad_w", 0), _pair(p, "dilation", "_", "_", 1))]
    if t == "BN":
        b = layer["blobs"]
        return [oracle.bn(x, b[0], b[1], b[2], b[3])]
    if t == "Dropout":
        return [x.copy()]
    if t == "Power":
        p = layer.get("power_param", {})
        return [oracle.power(x, p.get("power", 1.0), p.get("scale", 1.0), p.get("shift", 0.0))]
    if t == "Exp":
        p = layer.get("exp_param", {})
        return [oracle.exp_layer(x, p.get("base", -1.0), p.get("scale", 1.0), p.get("shift", 0.0))]
    if t == "Log":
        p = layer.get("log_param", {})
        return [oracle.log_layer(x, p.get("base", -1.0), p.get("scale", 1.0), p.get("shift", 0.0))]
    if t == "AbsVal":
        return [oracle.absval(x)]
    if t == "BNLL":
        return [oracle.bnll(x)]
    if t == "ELU":
        return [oracle.elu(x, layer.get("elu_param", {}).get("alpha", 1.0))]
    if t == "Threshold":
        return [oracle.threshold(x, layer.get("threshold_param", {}).get("threshold", 0.0))]
    if t == "PReLU":
        shared = layer.get("prelu_param", {}).get("channel_shared", False)
        return [oracle.prelu(x, layer["blobs"][0], shared)]
    if t == "LRN":
        p = layer.get("lrn_param", {})
        return [oracle.lrn(x, p.get("local_size", 5), p.get("alpha", 1.0), p.get("beta", 0.75),
                           p.get("k", 1.0), p.get("norm_region", "ACROSS_CHANNELS"))]
    if t == "ArgMax":
        p = layer.get("argmax_param", {})
        return [oracle.argmax(x, p.get("top_k", 1), p.get("out_max_val", False), p.get("axis"))]
    if t == "Reduction":
        p = layer.get("reduction_param", {})
        return [oracle.reduction(x, p.get("operation", "SUM"), p.get("axis", 0), p.get("coeff", 1.0))]
    if t == "MVN":
        p = layer.get("mvn_param", {})
        return [oracle.mvn(x, p.get("normalize_variance", True), p.get("across_channels", False),
                           p.get("eps", 1e-9))]
    if t == "Embed":
        p = layer["embed_param"]
        b = layer["blobs"]
        return [oracle.embed(x, b[0], b[1] if p.get("bias_term", True) else None)]
    if t == "Crop":
        # crop_layer.cpp:29-107: axes from `axis` on take bottom[1]'s extent at the offset
        p = layer.get("crop_param", {})
        axis = _canon(p.get("axis", 2), x.ndim)
        offs = p.get("offset", [])
        offs = list(offs) if isinstance(offs, (list, tuple)) else [offs]
        index = [slice(None)] * x.ndim
        for i in range(axis, x.ndim):
            o = 0 if not offs else (offs[0] if len(offs) == 1 else offs[i - axis])
            index[i] = slice(o, o + bottoms[1].shape[i])
        return [np.ascontiguousarray(x[tuple(index)])]
    if t == "Tile":
        # tile_layer.cpp:24-35
        p = layer["tile_param"]
        axis = _canon(p.get("axis", 1), x.ndim)
        reps = [1] * x.ndim
        reps[axis] = p["tiles"]
        return [np.ascontiguousarray(np.tile(x, reps))]
    if t == "ShuffleChannel":
        return [oracle.shuffle_channel(x, layer.get("shuffle_channel_param", {}).get("group", 1))]
    if t == "SPP":
        p = layer["spp_param"]
        return [oracle.spp(x, p["pyramid_height"], p.get("pool", "MAX"))]
    if t == "Parameter":
        return [layer["blobs"][0].copy()]
    raise NotImplementedError(t)


def oracle_forward(spec, inputs, keep=None):
    """Run the spec on the CPU oracle.  inputs: dict blob name -> array.
    Returns dict blob name -> final array (in-place layers overwrite).
    keep: optional set of blob names to retain (all are kept when None)."""
    blobs = {k: np.ascontiguousarray(v, dtype=np.float32) for k, v in inputs.items()}
    # Proposal shrinks its tops to the kept count in Forward, after every layer's
    # Reshape has run: a region pooling layer's top keeps the row count the rois had
    # at Reshape time and fills the rows it does not pool
    # (roi_pooling_layer.cpp:46 -FLT_MAX, psroi_pooling_layer.cpp:54 zero).
    reshape_rows = {}
    for layer in spec:
        if layer["type"] == "Input":
            for name in layer["top"]:
                assert name in blobs, "missing input %s" % name
            continue
        bottoms = [blobs[b] for b in layer.get("bottom", [])]
        tops = run_layer(layer, bottoms)
        if layer["type"] == "Proposal":
            rows = bottoms[0].shape[0] * layer.get("proposal_param", {}).get("post_nms_topn", 300)
            for name in layer["top"]:
                reshape_rows[name] = rows
        if layer["type"] in ("ROIPooling", "PSROIPooling"):
            rows = reshape_rows.get(layer["bottom"][1], tops[0].shape[0])
            if rows > tops[0].shape[0]:
                fill = np.float32(-3.4028234663852886e38 if layer["type"] == "ROIPooling" else 0.0)
                pad = np.full((rows - tops[0].shape[0],) + tops[0].shape[1:], fill, np.float32)
                tops = [np.concatenate([tops[0], pad])]
        for name, arr in zip(layer["top"], tops):
            blobs[name] = np.ascontiguousarray(arr, dtype=np.float32)
    if keep is not None:
        blobs = {k: v for k, v in blobs.items() if k in keep}
    return blobs


def rel_err(got, want, floor=1e-2):
    """max |got - want| / max(|want|, tau) with tau = floor * max|want|.

    Plain elementwise relative error is ill-posed at ReLU zeros and wherever a
    long fp32 sum cancels: two correct fp32 evaluations of the same K=576 dot
    product that merely add in a different order (OpenBLAS vs. plain loops, see
    tests/test_oracle.py::test_blas_order_noise) already differ by ~2e-4 of an
    output that is 1e-3 of the blob's peak.  The floor keeps the metric about the
    implementation rather than about summation order."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    if want.size == 0:
        return 0.0
    tau = floor * max(np.abs(want).max(), 1e-30)
    return float((np.abs(got - want) / np.maximum(np.abs(want), tau)).max())
