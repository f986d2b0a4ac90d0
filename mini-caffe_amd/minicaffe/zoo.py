"""Builders for the benchmark configurations as minicaffe.craft layer lists.

Weights are drawn here from seeded numpy generators with the distributions the
configurations name; mini-caffe's own fillers are all constant
(reference src/filler.hpp:51-71), so weights are always injected.
"""
import numpy as np

from .craft import Enum, input_layer


def _rng(seed, *names):
    """One generator per (seed, tensor name): tensors do not depend on creation order."""
    h = np.random.SeedSequence([seed] + [sum(ord(c) * (i + 1) for i, c in enumerate(n)) % (2 ** 31)
                                         for n in names])
    return np.random.default_rng(h)


def conv_layer(name, bottom, top, cin, cout, k, stride=1, pad=0, dilation=1, group=1, bias=True,
               seed=0, std=None, bias_value=0.0, deconv=False):
    std = std if std is not None else float(np.sqrt(2.0 / (cin // group * k * k)))
    shape = (cin, cout // group, k, k) if deconv else (cout, cin // group, k, k)
    w = (_rng(seed, name, "w").standard_normal(shape) * std).astype(np.float32)
    p = {"num_output": cout, "kernel_size": k}
    if stride != 1:
        p["stride"] = stride
    if pad:
        p["pad"] = pad
    if dilation != 1:
        p["dilation"] = dilation
    if group != 1:
        p["group"] = group
    blobs = [w]
    if bias:
        blobs.append(np.full((cout,), bias_value, np.float32))
    else:
        p["bias_term"] = False
    return {"name": name, "type": "Deconvolution" if deconv else "Convolution", "bottom": [bottom],
            "top": [top], "convolution_param": p, "blobs": blobs}


def bn_layer(name, blob, channels, use_global_stats=None, seed=None):
    """In-place BatchNorm.  Default statistics: mean 0, var 1, factor 1; with a
    seed, non-trivial statistics so that a wrong formula cannot pass."""
    if seed is None:
        mean = np.zeros(channels, np.float32)
        var = np.ones(channels, np.float32)
        factor = np.ones(1, np.float32)
    else:
        r = _rng(seed, name, "bn")
        factor = np.array([1.7], np.float32)
        mean = (r.standard_normal(channels) * 0.3 * 1.7).astype(np.float32)
        var = ((0.5 + r.random(channels)) * 1.7).astype(np.float32)
    layer = {"name": name, "type": "BatchNorm", "bottom": [blob], "top": [blob],
             "blobs": [mean, var, factor]}
    if use_global_stats is not None:
        layer["batch_norm_param"] = {"use_global_stats": use_global_stats}
    return layer


def scale_layer(name, blob, channels, seed=None):
    if seed is None:
        gamma = np.ones(channels, np.float32)
        beta = np.zeros(channels, np.float32)
    else:
        r = _rng(seed, name, "scale")
        gamma = (0.5 + r.random(channels)).astype(np.float32)
        beta = (r.standard_normal(channels) * 0.2).astype(np.float32)
    return {"name": name, "type": "Scale", "bottom": [blob], "top": [blob],
            "scale_param": {"bias_term": True}, "blobs": [gamma, beta]}


def relu_layer(name, blob, slope=None):
    layer = {"name": name, "type": "ReLU", "bottom": [blob], "top": [blob]}
    if slope is not None:
        layer["relu_param"] = {"negative_slope": slope}
    return layer


def c1_spec(seed=0):
    """Config 1: 3x3 s1 p1 convolution 64->64 on 1x64x56x56 with bias 0.01, then ReLU."""
    spec = [input_layer({"data": (1, 64, 56, 56)}),
            conv_layer("conv", "data", "conv", 64, 64, 3, pad=1, seed=seed, bias_value=0.01),
            relu_layer("relu", "conv")]
    x = np.random.default_rng(seed).standard_normal((1, 64, 56, 56)).astype(np.float32)
    return spec, {"data": x}


def resnet50_spec(batch=64, size=224, seed=0, num_classes=1000, stages=(3, 4, 6, 3),
                  width=64, bn_seed=None):
    """Caffe ResNet-50 v1 deploy graph: Conv+BatchNorm+Scale+ReLU units, stride on the
    first 1x1 of a stage, Eltwise SUM + ReLU, 3x3 s2 max pool (ceil mode), global
    average pool, InnerProduct, Softmax.  `stages`/`width` shrink it for tests."""
    spec = [input_layer({"data": (batch, 3, size, size)})]

    def unit(conv_name, bn_suffix, bottom, top, cin, cout, k, stride, pad, relu, bias=False):
        spec.append(conv_layer(conv_name, bottom, top, cin, cout, k, stride, pad, bias=bias,
                               seed=seed))
        spec.append(bn_layer("bn" + bn_suffix, top, cout, seed=bn_seed))
        spec.append(scale_layer("scale" + bn_suffix, top, cout, seed=bn_seed))
        if relu:
            spec.append(relu_layer(conv_name + "_relu", top))

    unit("conv1", "_conv1", "data", "conv1", 3, width, 7, 2, 3, True, bias=True)
    spec.append({"name": "pool1", "type": "Pooling", "bottom": ["conv1"], "top": ["pool1"],
                 "pooling_param": {"pool": Enum("MAX"), "kernel_size": 3, "stride": 2}})
    prev, cin = "pool1", width
    for si, nblocks in enumerate(stages):
        mid = width * (2 ** si)
        cout = mid * 4
        for bi in range(nblocks):
            tag = "%d%s" % (si + 2, "abcdefghij"[bi])
            stride = 2 if (bi == 0 and si > 0) else 1
            if bi == 0:
                unit("res%s_branch1" % tag, "%s_branch1" % tag, prev, "res%s_branch1" % tag, cin,
                     cout, 1, stride, 0, False)
                shortcut = "res%s_branch1" % tag
            else:
                shortcut = prev
            unit("res%s_branch2a" % tag, "%s_branch2a" % tag, prev, "res%s_branch2a" % tag, cin,
                 mid, 1, stride, 0, True)
            unit("res%s_branch2b" % tag, "%s_branch2b" % tag, "res%s_branch2a" % tag,
                 "res%s_branch2b" % tag, mid, mid, 3, 1, 1, True)
            unit("res%s_branch2c" % tag, "%s_branch2c" % tag, "res%s_branch2b" % tag,
                 "res%s_branch2c" % tag, mid, cout, 1, 1, 0, False)
            spec.append({"name": "res%s" % tag, "type": "Eltwise",
                         "bottom": [shortcut, "res%s_branch2c" % tag], "top": ["res%s" % tag]})
            spec.append(relu_layer("res%s_relu" % tag, "res%s" % tag))
            prev, cin = "res%s" % tag, cout
    spec.append({"name": "pool5", "type": "Pooling", "bottom": [prev], "top": ["pool5"],
                 "pooling_param": {"pool": Enum("AVE"), "global_pooling": True}})
    wfc = (_rng(seed, "fc1000", "w").standard_normal((num_classes, cin)) *
           np.sqrt(2.0 / cin)).astype(np.float32)
    spec.append({"name": "fc1000", "type": "InnerProduct", "bottom": ["pool5"], "top": ["fc1000"],
                 "inner_product_param": {"num_output": num_classes},
                 "blobs": [wfc, np.zeros(num_classes, np.float32)]})
    spec.append({"name": "prob", "type": "Softmax", "bottom": ["fc1000"], "top": ["prob"]})
    x = np.random.default_rng(seed + 1).uniform(-1, 1, (batch, 3, size, size)).astype(np.float32)
    return spec, {"data": x}


def _pool_out(n, k, s, pad):
    """Caffe's ceil-mode pooled extent with the last-window clip."""
    import math
    o = int(math.ceil(float(n + 2 * pad - k) / s)) + 1
    if pad and (o - 1) * s >= n + pad:
        o -= 1
    return o


def conv_flops(spec, inputs):
    """Algorithmic FLOPs of the Convolution / Deconvolution / InnerProduct layers of a
    spec: 2*N*Cout*Ho*Wo*(Cin/g)*kh*kw (deconv: 2*N*Cin*Hin*Win*(Cout/g)*kh*kw), 2*M*N*K."""
    shapes = {k: tuple(v.shape) for k, v in inputs.items()}
    total = {"conv": 0.0, "fc": 0.0}
    for layer in spec:
        t = layer["type"]
        if t == "Input":
            continue
        # shape inference for the layer types used by the configs
        b = [shapes[n] for n in layer.get("bottom", [])]
        if t in ("Convolution", "Deconvolution"):
            p = layer["convolution_param"]
            k, s, pad = p["kernel_size"], p.get("stride", 1), p.get("pad", 0)
            d, g = p.get("dilation", 1), p.get("group", 1)
            n, cin, h, w = b[0]
            ext = d * (k - 1) + 1
            if t == "Convolution":
                ho, wo = (h + 2 * pad - ext) // s + 1, (w + 2 * pad - ext) // s + 1
                total["conv"] += 2.0 * n * p["num_output"] * ho * wo * (cin // g) * k * k
            else:
                ho, wo = s * (h - 1) + ext - 2 * pad, s * (w - 1) + ext - 2 * pad
                total["conv"] += 2.0 * n * cin * h * w * (p["num_output"] // g) * k * k
            shapes[layer["top"][0]] = (n, p["num_output"], ho, wo)
        elif t == "InnerProduct":
            n_out = layer["inner_product_param"]["num_output"]
            m = b[0][0]
            kk = int(np.prod(b[0][1:]))
            total["fc"] += 2.0 * m * n_out * kk
            shapes[layer["top"][0]] = (m, n_out)
        elif t == "Pooling":
            p = layer["pooling_param"]
            n, c, h, w = b[0]
            if p.get("global_pooling", False):
                ho = wo = 1
            else:
                k, s, pad = p["kernel_size"], p.get("stride", 1), p.get("pad", 0)
                ho, wo = _pool_out(h, k, s, pad), _pool_out(w, k, s, pad)
            shapes[layer["top"][0]] = (n, c, ho, wo)
        elif t == "Reshape":
            dims = list(layer["reshape_param"]["shape"]["dim"])
            cnt = int(np.prod(b[0]))
            new = [b[0][i] if d == 0 else d for i, d in enumerate(dims)]
            if -1 in new:
                new[new.index(-1)] = cnt // int(-np.prod(new))
            shapes[layer["top"][0]] = tuple(new)
        else:
            for name in layer["top"]:
                shapes[name] = b[0]
    return total


def rpn_spec(seed=0, feat_shape=(1, 1024, 38, 63), im_info=(600.0, 1000.0, 1.0), std=0.01,
             pre_nms_topn=6000, post_nms_topn=300, nms_thresh=0.7, mid=512):
    """Config 4: region-proposal stage of a Faster R-CNN / R-FCN detector on a
    stride-16 feature map: 3x3 conv + ReLU, 1x1 score and box heads for 9 anchors,
    2-way softmax over (background, foreground), Proposal."""
    n, c, h, w = feat_shape
    A = 9
    spec = [input_layer({"feat": feat_shape, "im_info": (1, 3)}),
            conv_layer("rpn_conv/3x3", "feat", "rpn/output", c, mid, 3, pad=1, seed=seed, std=std),
            relu_layer("rpn_relu/3x3", "rpn/output"),
            conv_layer("rpn_cls_score", "rpn/output", "rpn_cls_score", mid, 2 * A, 1, seed=seed,
                       std=std),
            conv_layer("rpn_bbox_pred", "rpn/output", "rpn_bbox_pred", mid, 4 * A, 1, seed=seed,
                       std=std),
            {"name": "rpn_cls_score_reshape", "type": "Reshape", "bottom": ["rpn_cls_score"],
             "top": ["rpn_cls_score_reshape"], "reshape_param": {"shape": {"dim": [0, 2, -1, 0]}}},
            {"name": "rpn_cls_prob", "type": "Softmax", "bottom": ["rpn_cls_score_reshape"],
             "top": ["rpn_cls_prob"]},
            {"name": "rpn_cls_prob_reshape", "type": "Reshape", "bottom": ["rpn_cls_prob"],
             "top": ["rpn_cls_prob_reshape"],
             "reshape_param": {"shape": {"dim": [0, 2 * A, -1, 0]}}},
            {"name": "proposal", "type": "Proposal",
             "bottom": ["rpn_cls_prob_reshape", "rpn_bbox_pred", "im_info"], "top": ["rois"],
             "proposal_param": {"feat_stride": 16, "base_size": 16, "min_size": 16,
                                "ratio": [0.5, 1.0, 2.0], "scale": [8.0, 16.0, 32.0],
                                "pre_nms_topn": pre_nms_topn, "post_nms_topn": post_nms_topn,
                                "nms_thresh": nms_thresh}}]
    x = np.random.default_rng(seed + 1).standard_normal(feat_shape).astype(np.float32)
    return spec, {"feat": x, "im_info": np.array([im_info], np.float32)}


def dcgan_spec(batch=128, seed=0, zdim=100, base=1024, use_global_stats=False, std=0.02):
    """Config 5: DCGAN/WGAN generator: InnerProduct to 4x4xbase, three 4x4 stride-2
    Deconvolutions halving the channels with BatchNorm + Scale + ReLU, a last one to
    3 channels with TanH (64x64 output for base 1024)."""
    spec = [input_layer({"z": (batch, zdim)})]
    w = (_rng(seed, "fc", "w").standard_normal((base * 16, zdim)) * std).astype(np.float32)
    spec.append({"name": "fc", "type": "InnerProduct", "bottom": ["z"], "top": ["fc"],
                 "inner_product_param": {"num_output": base * 16},
                 "blobs": [w, np.zeros(base * 16, np.float32)]})
    spec.append({"name": "fc_reshape", "type": "Reshape", "bottom": ["fc"], "top": ["g0"],
                 "reshape_param": {"shape": {"dim": [0, base, 4, 4]}}})
    prev, cin = "g0", base
    for i in range(1, 4):
        cout = cin // 2
        name = "gconv%d" % i
        spec.append(conv_layer(name, prev, name, cin, cout, 4, stride=2, pad=1, bias=False,
                               seed=seed, std=std, deconv=True))
        bn = bn_layer("gbn%d" % i, name, cout, use_global_stats=use_global_stats,
                      seed=(seed + 11) if use_global_stats else None)
        if not use_global_stats:
            bn["blobs"] = [np.zeros(cout, np.float32), np.zeros(cout, np.float32),
                           np.zeros(1, np.float32)]
        spec.append(bn)
        spec.append(scale_layer("gbn%d_scale" % i, name, cout, seed=seed + 13))
        spec.append(relu_layer("gact%d" % i, name))
        prev, cin = name, cout
    spec.append(conv_layer("gconv4", prev, "gconv4", cin, 3, 4, stride=2, pad=1, bias=False,
                           seed=seed, std=std, deconv=True))
    spec.append({"name": "gact4", "type": "TanH", "bottom": ["gconv4"], "top": ["gconv4"]})
    z = np.random.default_rng(seed + 1).standard_normal((batch, zdim)).astype(np.float32)
    return spec, {"z": z}


SSD_SOURCES = [  # (source blob, channels, priors, min_size, max_size, aspect ratios, step)
    ("conv4_3_norm", 512, 4, 30.0, 60.0, [2.0], 8),
    ("fc7", 1024, 6, 60.0, 111.0, [2.0, 3.0], 16),
    ("conv6_2", 512, 6, 111.0, 162.0, [2.0, 3.0], 32),
    ("conv7_2", 256, 6, 162.0, 213.0, [2.0, 3.0], 64),
    ("conv8_2", 256, 4, 213.0, 264.0, [2.0], 100),
    ("conv9_2", 256, 4, 264.0, 315.0, [2.0], 300),
]


def _multibox_tail(spec, sources, num_classes, seed, head_kernel, nms_top_k, keep_top_k,
                   confidence_threshold):
    """Appends the SSD heads (loc / conf convolutions -> Permute -> Flatten, PriorBox per
    source), their concatenations, the class softmax and DetectionOutput.
    sources: (blob, channels, priors per cell, min_size, max_size or None, aspect ratios,
    step or None)."""
    locs, confs, priors = [], [], []
    for src, c, npri, mn, mx, ars, step in sources:
        for kind, per in (("loc", 4), ("conf", num_classes)):
            name = "%s_mbox_%s" % (src, kind)
            spec.append(conv_layer(name, src, name, c, npri * per, head_kernel,
                                   pad=head_kernel // 2, seed=seed))
            spec.append({"name": name + "_perm", "type": "Permute", "bottom": [name],
                         "top": [name + "_perm"], "permute_param": {"order": [0, 2, 3, 1]}})
            spec.append({"name": name + "_flat", "type": "Flatten", "bottom": [name + "_perm"],
                         "top": [name + "_flat"], "flatten_param": {"axis": 1}})
            (locs if kind == "loc" else confs).append(name + "_flat")
        pname = "%s_mbox_priorbox" % src
        pb = {"min_size": mn}
        if mx is not None:
            pb["max_size"] = mx
        pb.update({"aspect_ratio": ars, "flip": True, "clip": False,
                   "variance": [0.1, 0.1, 0.2, 0.2]})
        if step is not None:
            pb["step"] = float(step)
        pb["offset"] = 0.5
        spec.append({"name": pname, "type": "PriorBox", "bottom": [src, "data"], "top": [pname],
                     "prior_box_param": pb})
        priors.append(pname)
    spec.append({"name": "mbox_loc", "type": "Concat", "bottom": locs, "top": ["mbox_loc"],
                 "concat_param": {"axis": 1}})
    spec.append({"name": "mbox_conf", "type": "Concat", "bottom": confs, "top": ["mbox_conf"],
                 "concat_param": {"axis": 1}})
    spec.append({"name": "mbox_priorbox", "type": "Concat", "bottom": priors,
                 "top": ["mbox_priorbox"], "concat_param": {"axis": 2}})
    spec.append({"name": "mbox_conf_reshape", "type": "Reshape", "bottom": ["mbox_conf"],
                 "top": ["mbox_conf_reshape"],
                 "reshape_param": {"shape": {"dim": [0, -1, num_classes]}}})
    spec.append({"name": "mbox_conf_softmax", "type": "Softmax", "bottom": ["mbox_conf_reshape"],
                 "top": ["mbox_conf_softmax"], "softmax_param": {"axis": 2}})
    spec.append({"name": "mbox_conf_flatten", "type": "Flatten", "bottom": ["mbox_conf_softmax"],
                 "top": ["mbox_conf_flatten"], "flatten_param": {"axis": 1}})
    spec.append({"name": "detection_out", "type": "DetectionOutput",
                 "bottom": ["mbox_loc", "mbox_conf_flatten", "mbox_priorbox"],
                 "top": ["detection_out"],
                 "detection_output_param": {
                     "num_classes": num_classes, "share_location": True,
                     "background_label_id": 0,
                     "nms_param": {"nms_threshold": 0.45, "top_k": nms_top_k},
                     "code_type": Enum("CENTER_SIZE"), "keep_top_k": keep_top_k,
                     "confidence_threshold": confidence_threshold}})


def ssd300_spec(batch=8, seed=0, num_classes=21, size=300, width=64):
    """Config 3: SSD300 on VGG16 (atrous fc6, extra layers conv6-conv9, six multibox
    heads with 4/6/6/6/4/4 priors, 8732 priors at 300x300), DetectionOutput with
    NMS 0.45, top_k 400, keep_top_k 200.  `width` scales the channel counts for
    small test nets (64 is the real model)."""
    s = width / 64.0
    ch = lambda c: max(4, int(round(c * s)))  # noqa: E731
    spec = [input_layer({"data": (batch, 3, size, size)})]
    prev, cin = "data", 3

    def conv_relu(name, cout, k, stride=1, pad=0, dilation=1):
        nonlocal prev, cin
        spec.append(conv_layer(name, prev, name, cin, cout, k, stride, pad, dilation, seed=seed))
        spec.append(relu_layer("relu" + name[4:] if name.startswith("conv") else name + "_relu",
                               name))
        prev, cin = name, cout

    def pool(name, k, stride, pad=0):
        nonlocal prev
        p = {"pool": Enum("MAX"), "kernel_size": k, "stride": stride}
        if pad:
            p["pad"] = pad
        spec.append({"name": name, "type": "Pooling", "bottom": [prev], "top": [name],
                     "pooling_param": p})
        prev = name

    for blk, (n_conv, c) in enumerate([(2, 64), (2, 128), (3, 256), (3, 512), (3, 512)], 1):
        for i in range(1, n_conv + 1):
            conv_relu("conv%d_%d" % (blk, i), ch(c), 3, pad=1)
        if blk < 5:
            pool("pool%d" % blk, 2, 2)
        else:
            pool("pool5", 3, 1, 1)
    conv_relu("fc6", ch(1024), 3, pad=6, dilation=6)
    conv_relu("fc7", ch(1024), 1)
    conv_relu("conv6_1", ch(256), 1)
    conv_relu("conv6_2", ch(512), 3, stride=2, pad=1)
    conv_relu("conv7_1", ch(128), 1)
    conv_relu("conv7_2", ch(256), 3, stride=2, pad=1)
    conv_relu("conv8_1", ch(128), 1)
    conv_relu("conv8_2", ch(256), 3)
    conv_relu("conv9_1", ch(128), 1)
    conv_relu("conv9_2", ch(256), 3)
    c43 = ch(512)
    spec.append({"name": "conv4_3_norm", "type": "Normalize", "bottom": ["conv4_3"],
                 "top": ["conv4_3_norm"],
                 "norm_param": {"across_spatial": False, "channel_shared": False,
                                "scale_filler": {"type": "constant", "value": 20.0}},
                 "blobs": [np.full(c43, 20.0, np.float32)]})
    _multibox_tail(spec, [(src, ch(c), npri, mn, mx, ars, step)
                          for src, c, npri, mn, mx, ars, step in SSD_SOURCES],
                   num_classes, seed, head_kernel=3, nms_top_k=400, keep_top_k=200,
                   confidence_threshold=0.01)
    x = np.random.default_rng(seed + 1).uniform(-1, 1, (batch, 3, size, size)).astype(np.float32)
    return spec, {"data": x}



# MobileNet-SSD sources: blob, channels, priors per cell, min_size, max_size, aspect ratios.
MOBILENET_SSD_SOURCES = [
    ("conv11", 512, 3, 60.0, None, [2.0]),
    ("conv13", 1024, 6, 105.0, 150.0, [2.0, 3.0]),
    ("conv14_2", 512, 6, 150.0, 195.0, [2.0, 3.0]),
    ("conv15_2", 256, 6, 195.0, 240.0, [2.0, 3.0]),
    ("conv16_2", 256, 6, 240.0, 285.0, [2.0, 3.0]),
    ("conv17_2", 128, 6, 285.0, 300.0, [2.0, 3.0]),
]


def mobilenet_ssd_spec(batch=1, seed=0, num_classes=21, size=300, width=1.0, depthwise_type=False):
    """MobileNet-v1 SSD in its deploy form (batch norm merged into the convolutions), the
    graph of the reference's ssd example (example/models/ssd/MobileNetSSD_deploy.prototxt):
    conv0, 13 depthwise-separable blocks (`Convolution` with group == channels, then 1x1),
    four extra stride-2 stages, six 1x1 multibox heads, 1917 priors at 300x300,
    DetectionOutput with NMS 0.45, top_k 100, keep_top_k 100, confidence 0.25.
    depthwise_type=True declares the depthwise layers as `ConvolutionDepthwise` instead."""
    ch = lambda c: max(8, int(round(c * width)))  # noqa: E731
    spec = [input_layer({"data": (batch, 3, size, size)})]

    def conv_relu(name, bottom, cin, cout, k, stride=1, group=1):
        layer = conv_layer(name, bottom, name, cin, cout, k, stride, k // 2, group=group, seed=seed)
        if group != 1 and depthwise_type:
            layer["type"] = "ConvolutionDepthwise"
            del layer["convolution_param"]["group"]
        spec.append(layer)
        spec.append(relu_layer(name + "/relu", name))

    conv_relu("conv0", "data", 3, ch(32), 3, 2)
    prev, cin = "conv0", ch(32)
    for i, (cout, stride) in enumerate([(64, 1), (128, 2), (128, 1), (256, 2), (256, 1), (512, 2),
                                        (512, 1), (512, 1), (512, 1), (512, 1), (512, 1),
                                        (1024, 2), (1024, 1)], 1):
        conv_relu("conv%d/dw" % i, prev, cin, cin, 3, stride, group=cin)
        conv_relu("conv%d" % i, "conv%d/dw" % i, cin, ch(cout), 1)
        prev, cin = "conv%d" % i, ch(cout)
    for i, (mid, cout) in enumerate([(256, 512), (128, 256), (128, 256), (64, 128)], 14):
        conv_relu("conv%d_1" % i, prev, cin, ch(mid), 1)
        conv_relu("conv%d_2" % i, "conv%d_1" % i, ch(mid), ch(cout), 3, 2)
        prev, cin = "conv%d_2" % i, ch(cout)
    _multibox_tail(spec, [(src, ch(c), npri, mn, mx, ars, None)
                          for src, c, npri, mn, mx, ars in MOBILENET_SSD_SOURCES],
                   num_classes, seed, head_kernel=1, nms_top_k=100, keep_top_k=100,
                   confidence_threshold=0.25)
    x = np.random.default_rng(seed + 1).uniform(-1, 1, (batch, 3, size, size)).astype(np.float32)
    return spec, {"data": x}


def _pool(name, bottom, method, k, stride=1, pad=0, global_pooling=False):
    p = {"pool": Enum(method)}
    if global_pooling:
        p["global_pooling"] = True
    else:
        p["kernel_size"] = k
        p["stride"] = stride
        if pad:
            p["pad"] = pad
    return {"name": name, "type": "Pooling", "bottom": [bottom], "top": [name], "pooling_param": p}


def googlenet_spec(batch=2, size=96, seed=0, num_classes=10,
                   modules=((64, 96, 128, 16, 32, 32), (128, 128, 192, 32, 96, 64))):
    """The front of bvlc_googlenet (one of the three nets the reference's own test program
    runs, tests/run_net.cpp:175-236): 7x7/2 stem, LRN, 1x1 + 3x3, LRN, then inception
    modules (1x1 | 1x1 -> 3x3 | 1x1 -> 5x5 | 3x3/1 max pool -> 1x1, Concat), global
    average pool, Dropout, InnerProduct, Softmax.  `modules` lists (1x1, 3x3 reduce, 3x3,
    5x5 reduce, 5x5, pool proj) outputs; the default is inception 3a and 3b."""
    spec = [input_layer({"data": (batch, 3, size, size)})]

    def conv_relu(name, bottom, cin, cout, k, stride=1, pad=0):
        spec.append(conv_layer(name, bottom, name, cin, cout, k, stride, pad, seed=seed, bias_value=0.2))
        spec.append(relu_layer("relu_" + name, name))

    lrn = lambda name, bottom: {"name": name, "type": "LRN", "bottom": [bottom], "top": [name],  # noqa: E731
                                "lrn_param": {"local_size": 5, "alpha": 1e-4, "beta": 0.75}}
    conv_relu("conv1/7x7_s2", "data", 3, 64, 7, 2, 3)
    spec.append(_pool("pool1/3x3_s2", "conv1/7x7_s2", "MAX", 3, 2))
    spec.append(lrn("pool1/norm1", "pool1/3x3_s2"))
    conv_relu("conv2/3x3_reduce", "pool1/norm1", 64, 64, 1)
    conv_relu("conv2/3x3", "conv2/3x3_reduce", 64, 192, 3, 1, 1)
    spec.append(lrn("conv2/norm2", "conv2/3x3"))
    spec.append(_pool("pool2/3x3_s2", "conv2/norm2", "MAX", 3, 2))
    prev, cin = "pool2/3x3_s2", 192
    for i, (c1, c3r, c3, c5r, c5, cp) in enumerate(modules):
        m = "inception_%d" % i
        conv_relu(m + "/1x1", prev, cin, c1, 1)
        conv_relu(m + "/3x3_reduce", prev, cin, c3r, 1)
        conv_relu(m + "/3x3", m + "/3x3_reduce", c3r, c3, 3, 1, 1)
        conv_relu(m + "/5x5_reduce", prev, cin, c5r, 1)
        conv_relu(m + "/5x5", m + "/5x5_reduce", c5r, c5, 5, 1, 2)
        spec.append(_pool(m + "/pool", prev, "MAX", 3, 1, 1))
        conv_relu(m + "/pool_proj", m + "/pool", cin, cp, 1)
        spec.append({"name": m + "/output", "type": "Concat",
                     "bottom": [m + "/1x1", m + "/3x3", m + "/5x5", m + "/pool_proj"], "top": [m + "/output"]})
        prev, cin = m + "/output", c1 + c3 + c5 + cp
    spec.append(_pool("pool5", prev, "AVE", 0, global_pooling=True))
    spec.append({"name": "pool5/drop", "type": "Dropout", "bottom": ["pool5"], "top": ["pool5"],
                 "dropout_param": {"dropout_ratio": 0.4}})
    w = (_rng(seed, "loss3/classifier", "w").standard_normal((num_classes, cin)) * np.sqrt(2.0 / cin)).astype(np.float32)
    spec.append({"name": "loss3/classifier", "type": "InnerProduct", "bottom": ["pool5"], "top": ["loss3/classifier"],
                 "inner_product_param": {"num_output": num_classes},
                 "blobs": [w, np.zeros(num_classes, np.float32)]})
    spec.append({"name": "prob", "type": "Softmax", "bottom": ["loss3/classifier"], "top": ["prob"]})
    x = np.random.default_rng(seed + 1).uniform(-1, 1, (batch, 3, size, size)).astype(np.float32)
    return spec, {"data": x}


def nin_spec(batch=2, size=67, seed=0, num_classes=10, width=32):
    """Network-in-Network (another of the reference's test nets): every block is a
    spatial convolution followed by two 1x1 "cccp" convolutions, all with ReLU; max
    pools with Dropout between blocks; the classifier is a 1x1 convolution, a global
    average pool and Softmax (no InnerProduct)."""
    spec = [input_layer({"data": (batch, 3, size, size)})]

    def conv_relu(name, bottom, cin, cout, k, stride=1, pad=0):
        spec.append(conv_layer(name, bottom, name, cin, cout, k, stride, pad, seed=seed, bias_value=0.1))
        spec.append(relu_layer("relu_" + name, name))

    conv_relu("conv1", "data", 3, width * 3, 11, 4)
    conv_relu("cccp1", "conv1", width * 3, width * 3, 1)
    conv_relu("cccp2", "cccp1", width * 3, width * 3, 1)
    spec.append(_pool("pool0", "cccp2", "MAX", 3, 2))
    conv_relu("conv2", "pool0", width * 3, width * 8, 5, 1, 2)
    conv_relu("cccp3", "conv2", width * 8, width * 8, 1)
    conv_relu("cccp4", "cccp3", width * 8, width * 8, 1)
    spec.append(_pool("pool2", "cccp4", "MAX", 3, 2))
    spec.append({"name": "drop", "type": "Dropout", "bottom": ["pool2"], "top": ["pool2"],
                 "dropout_param": {"dropout_ratio": 0.5}})
    conv_relu("conv4-1024", "pool2", width * 8, width * 16, 3, 1, 1)
    conv_relu("cccp7-1024", "conv4-1024", width * 16, width * 16, 1)
    conv_relu("cccp8-1024", "cccp7-1024", width * 16, num_classes, 1)
    spec.append(_pool("pool4", "cccp8-1024", "AVE", 0, global_pooling=True))
    spec.append({"name": "prob", "type": "Softmax", "bottom": ["pool4"], "top": ["prob"]})
    x = np.random.default_rng(seed + 1).uniform(-1, 1, (batch, 3, size, size)).astype(np.float32)
    return spec, {"data": x}
