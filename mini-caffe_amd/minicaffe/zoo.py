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
