"""Host-side behaviour of libcaffe.so through its C ABI; no GPU needed.

Covers what the reference's tests/run_net.c asserts on a CPU box (creation,
blob shapes, listing, the -1 + CaffeGetLastError error convention) plus the
prototxt / caffemodel reader that replaces protobuf.
"""
import ctypes
import json
import os
import re

import numpy as np
import pytest

import minicaffe as mc
from minicaffe import craft, zoo
from minicaffe.base import LIB

import wire

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"
needs_ref = pytest.mark.skipif(not os.path.isdir(REF), reason="reference checkout not present")


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:Caffe|mc)[A-Z]\w*)\s*\(", text)))


@pytest.mark.parametrize("header", ["caffe/c_api.h", "mchip/kernels.h"])
def test_library_exports_every_declared_symbol(header):
    names = declared_functions(header)
    assert len(names) >= 20
    missing = [n for n in names if not hasattr(LIB, n)]
    assert not missing, missing


def test_c_api_has_the_reference_entry_points():
    # the 25 functions of the reference's include/caffe/c_api.h:26-162
    want = """CaffeBlobNum CaffeBlobChannels CaffeBlobHeight CaffeBlobWidth CaffeBlobData
    CaffeBlobCount CaffeBlobReshape CaffeBlobShape CaffeNetCreate CaffeNetCreateFromBuffer
    CaffeNetDestroy CaffeNetMarkOutput CaffeNetForward CaffeNetGetBlob CaffeNetListBlob
    CaffeNetListParam CaffeProfilerEnable CaffeProfilerDisable CaffeProfilerScopeStart
    CaffeProfilerScopeEnd CaffeProfilerDump CaffeGPUAvailable CaffeSetMode CaffeGetLastError
    CaffeMemoryPoolClear""".split()
    assert len(want) == 25
    assert set(want) <= set(declared_functions("caffe/c_api.h"))


TRICKY = """
# comment line
name: 'tricky'   # trailing comment
input: "data"
input_dim: 2
input_dim: 3
input_dim: 12
input_dim: 10
layer {
  name: "conv1" type: "Convolution" bottom: "data" top: "conv1"
  param { lr_mult: 1.0 decay_mult: 1.0 }
  param { lr_mult: 2.0 decay_mult: 0 }
  convolution_param: {
    num_output: 8; kernel_h: 3, kernel_w: 2
    stride_h: 2 stride_w: 1 pad_h: 1 pad_w: 0
    weight_filler { type: "xavier" } bias_filler { type: "constant" value: 0.25 }
  }
}
layer { name: "pool" type: "Pooling" bottom: "conv1" top: "pool"
        pooling_param { pool: AVE kernel_size: 2 stride: 2 } include { phase: TEST } }
layer { name: "relu" type: "ReLU" bottom: "pool" top: "pool" relu_param { negative_slope: 1e-1 } }
layer { name: "ip" type: "InnerProduct" bottom: "pool" top: "ip"
        inner_product_param { num_output: 5 bias_term: false } }
layer { name: "prob" type: "Softmax" bottom: "ip" top: "prob" }
"""


def test_prototxt_reader_and_shape_inference():
    net = mc.Net.from_buffers(TRICKY)
    shapes = {k: v.shape for k, v in net.blobs.items()}
    # conv: H (12+2-3)/2+1 = 6, W (10-2)/1+1 = 9; pool (ceil): 3 x 5
    assert shapes == {"data": [2, 3, 12, 10], "conv1": [2, 8, 6, 9], "pool": [2, 8, 3, 5],
                      "ip": [2, 5], "prob": [2, 5]}
    params = net.param_list
    assert [n for n, _ in params] == ["conv1_0", "conv1_1", "ip_0"]
    assert params[0][1].shape == [8, 3, 3, 2] and params[2][1].shape == [5, 120]
    # every filler is a constant fill; "xavier" without value gives zeros
    assert np.all(params[0][1].data == 0) and np.all(params[1][1].data == 0.25)
    blob = net.get_blob("data")
    assert (LIB.CaffeBlobNum(blob.handle), LIB.CaffeBlobChannels(blob.handle),
            LIB.CaffeBlobHeight(blob.handle), LIB.CaffeBlobWidth(blob.handle),
            LIB.CaffeBlobCount(blob.handle)) == (2, 3, 12, 10, 720)


def err(fn):
    with pytest.raises(mc.MiniCaffeError) as e:
        fn()
    return str(e.value)


def test_error_convention():
    assert "Unknown layer type: Nope" in err(lambda: mc.Net.from_buffers(
        'layer { name: "d" type: "Input" top: "d" input_param { shape { dim: 1 } } }'
        'layer { name: "x" type: "Nope" bottom: "d" top: "x" }'))
    # nonexistent files must give -1 and a message (reference tests/run_net.c:73-74)
    assert "File not found" in err(lambda: mc.Net("/nonexistent.prototxt", "/nonexistent.caffemodel"))
    assert "takes 1 bottom blob" in err(lambda: mc.Net.from_buffers(
        'layer { name: "r" type: "ReLU" top: "r" }'))
    two = ('layer { name: "d" type: "Input" top: "d" input_param { shape { dim: 1 dim: 2 } } }'
           'layer { name: "a" type: "ReLU" bottom: "d" top: "x" }'
           'layer { name: "b" type: "ReLU" bottom: "d" top: "x" }')
    assert "produced by multiple sources" in err(lambda: mc.Net.from_buffers(two))
    assert "Unknown bottom blob 'nope'" in err(lambda: mc.Net.from_buffers(
        'layer { name: "d" type: "Input" top: "d" input_param { shape { dim: 1 } } }'
        'layer { name: "a" type: "ReLU" bottom: "nope" top: "x" }'))
    assert "parse error at 1:" in err(lambda: mc.Net.from_buffers('layer { name "x" }'))
    assert "missing closing brace" in err(lambda: mc.Net.from_buffers('layer { name: "x" '))
    net = mc.Net.from_buffers(TRICKY)
    assert "is not availiable" in err(lambda: net.mark_output("nope"))
    assert "Unknown blob name" in err(lambda: net.get_blob("nope"))
    assert "mode must be 0" in err(lambda: mc.set_runtime_mode(7, 0))


def test_forward_without_gpu_mode_fails_loudly():
    mc.set_runtime_mode(0, -1)
    net = mc.Net.from_buffers(TRICKY)
    msg = err(lambda: net.forward())
    assert "HIP device path only" in msg


def test_caffemodel_reader_and_weight_copy():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((8, 3, 3, 2)).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    ipw = rng.standard_normal((5, 120)).astype(np.float32)
    for kw in ({}, {"packed": False}, {"as_double": True}):
        model = wire.net("m", [wire.layer("conv1", "Convolution", [w, b], **kw),
                               wire.layer("not_in_net", "ReLU", []),
                               wire.layer("ip", "InnerProduct", [ipw], **kw)])
        net = mc.Net.from_buffers(TRICKY, model)
        params = dict(net.param_list)
        assert np.array_equal(params["conv1_0"].data, w)
        assert np.array_equal(params["conv1_1"].data, b)
        assert np.array_equal(params["ip_0"].data, ipw)
    # legacy 4-D blob dims: bias (1,1,1,8) and ip weight (1,1,5,120) match N-d targets
    model = wire.net("m", [wire.layer("conv1", "Convolution", [w, b], legacy=True),
                           wire.layer("ip", "InnerProduct", [ipw], legacy=True)])
    net = mc.Net.from_buffers(TRICKY, model)
    assert np.array_equal(dict(net.param_list)["ip_0"].data, ipw)
    # shape mismatch is fatal and names both shapes
    bad = wire.net("m", [wire.layer("conv1", "Convolution", [w[:, :, :2], b])])
    msg = err(lambda: mc.Net.from_buffers(TRICKY, bad))
    assert "shape mismatch" in msg and "8 3 2 2" in msg and "8 3 3 2" in msg
    bad = wire.net("m", [wire.layer("conv1", "Convolution", [w])])
    assert "Incompatible number of blobs" in err(lambda: mc.Net.from_buffers(TRICKY, bad))
    assert "truncated" in err(lambda: mc.Net.from_buffers(TRICKY, model[:-3]))


def test_create_from_files(tmp_path):
    w = np.arange(8 * 3 * 3 * 2, dtype=np.float32).reshape(8, 3, 3, 2)
    b = np.ones(8, np.float32)
    (tmp_path / "n.prototxt").write_text(TRICKY)
    (tmp_path / "n.caffemodel").write_bytes(
        wire.net("m", [wire.layer("conv1", "Convolution", [w, b])]))
    net = mc.Net(str(tmp_path / "n.prototxt"), str(tmp_path / "n.caffemodel"))
    assert np.array_equal(dict(net.param_list)["conv1_0"].data, w)


def test_layer_argument_checks():
    base = 'layer { name: "d" type: "Input" top: "d" input_param { shape { dim: 1 dim: 4 dim: 6 dim: 6 } } }'

    def conv(body):
        return base + 'layer { name: "c" type: "Convolution" bottom: "d" top: "c" convolution_param { %s } }' % body
    assert "kernel_size must be specified" in err(lambda: mc.Net.from_buffers(conv("num_output: 2")))
    assert "multiples of group" in err(lambda: mc.Net.from_buffers(conv("num_output: 3 kernel_size: 1 group: 2")))
    assert "not both" in err(lambda: mc.Net.from_buffers(conv("num_output: 2 kernel_size: 3 kernel_h: 3")))
    assert "Stride dimensions must be nonzero" in err(lambda: mc.Net.from_buffers(conv("num_output: 2 kernel_size: 3 stride: 0")))
    pool = base + 'layer { name: "p" type: "Pooling" bottom: "d" top: "p" pooling_param { %s } }'
    assert "Filter size cannot specified" in err(lambda: mc.Net.from_buffers(pool % "global_pooling: true kernel_size: 2"))
    assert "Unknown pooling method" in err(lambda: mc.Net.from_buffers(pool % "pool: STOCHASTIC kernel_size: 2"))
    elt = base + ('layer { name: "e" type: "Eltwise" bottom: "d" bottom: "d" top: "e" '
                  'eltwise_param { operation: PROD coeff: 1 coeff: 2 } }')
    assert "only takes coefficients for summation" in err(lambda: mc.Net.from_buffers(elt))
    assert "takes at least 2 bottom" in err(lambda: mc.Net.from_buffers(
        base + 'layer { name: "e" type: "Eltwise" bottom: "d" top: "e" }'))
    assert "Unknown filler name" in err(lambda: mc.Net.from_buffers(
        conv('num_output: 2 kernel_size: 1 weight_filler { type: "fancy" }')))
    resh = base + 'layer { name: "r" type: "Reshape" bottom: "d" top: "r" reshape_param { shape { dim: 0 dim: -1 dim: 5 } } }'
    assert "must be divisible" in err(lambda: mc.Net.from_buffers(resh))


def test_resnet50_graph_builds_with_reference_shapes():
    spec, inputs = zoo.resnet50_spec(batch=2, size=224)
    assert len(spec) == 229   # Input, 53 conv/BN/Scale, 49 ReLU, 16 Eltwise, 2 pool, IP, softmax
    net = mc.Net.from_buffers(craft.to_prototxt(spec))
    shapes = {k: v.shape for k, v in net.blobs.items()}
    assert shapes["conv1"] == [2, 64, 112, 112] and shapes["pool1"] == [2, 64, 56, 56]
    assert shapes["res3a"] == [2, 512, 28, 28] and shapes["res5c"] == [2, 2048, 7, 7]
    assert shapes["pool5"] == [2, 2048, 1, 1] and shapes["prob"] == [2, 1000]
    # 7.712 GFLOP per image in the convolutions
    assert abs(zoo.conv_flops(spec, inputs)["conv"] / 2 / 1e9 - 7.712) < 0.01


def test_profiler_dump(tmp_path):
    mc.Profiler.enable()
    mc.Profiler.open_scope("outer")
    mc.Profiler.open_scope("inner")
    mc.Profiler.close_scope()
    mc.Profiler.close_scope()
    mc.Profiler.disable()
    fn = str(tmp_path / "profile.json")
    mc.Profiler.dump(fn)
    events = json.load(open(fn))["traceEvents"]
    names = [e["name"] for e in events if e["ph"] == "B"]
    assert "outer" in names and "outer:inner" in names
    assert "not running" in err(mc.Profiler.disable)


def test_memory_pool_clear_and_gpu_flag():
    mc.memory_pool_clear()
    assert LIB.CaffeGPUAvailable() in (0, 1)


@needs_ref
@pytest.mark.parametrize("name", ["1_F", "2_LE1", "2_N2", "2_RM2"])
def test_reads_the_reference_example_models(name):
    """Real prototxt + binary caffemodel pairs shipped with the reference's
    deeplandmark example (example/models/deeplandmark): only files in the tree
    with trained weights.  They must load; weights must be finite and non-trivial."""
    d = os.path.join(REF, "example", "models", "deeplandmark")
    net = mc.Net(os.path.join(d, name + ".prototxt"), os.path.join(d, name + ".caffemodel"))
    params = net.param_list
    assert len(params) >= 6
    for _, blob in params:
        a = blob.data
        assert np.isfinite(a).all()
    assert any(np.abs(b.data).max() > 1e-3 for _, b in params)


@needs_ref
def test_reads_the_reference_wgan_prototxt():
    net = mc.Net.from_buffers(open(os.path.join(REF, "example", "models", "wgan", "g.prototxt")).read())
    shapes = {k: v.shape for k, v in net.blobs.items()}
    assert list(shapes.values())[-1][1:] == [3, 64, 64]


def test_region_pooling_layers_setup_errors_and_shapes():
    """ROIPooling / PSROIPooling construction (roi_pooling_layer.cpp:15-36,
    psroi_pooling_layer.cpp:18-44): parameter checks and the top shape taken from the
    rois blob's row count."""
    from minicaffe import MiniCaffeError
    base = [craft.input_layer({"feat": (1, 18, 6, 8), "rois": (7, 5)})]
    ok = base + [{"name": "ps", "type": "PSROIPooling", "bottom": ["feat", "rois"], "top": ["ps"],
                  "psroi_pooling_param": {"spatial_scale": 0.0625, "output_dim": 2, "group_size": 3}},
                 {"name": "rp", "type": "ROIPooling", "bottom": ["feat", "rois"], "top": ["rp"],
                  "roi_pooling_param": {"pooled_h": 2, "pooled_w": 4, "spatial_scale": 0.0625}}]
    net = mc.Net.from_buffers(craft.to_prototxt(ok))
    assert tuple(net.get_blob("ps").shape) == (7, 2, 3, 3)
    assert tuple(net.get_blob("rp").shape) == (7, 18, 2, 4)
    bad = base + [{"name": "ps", "type": "PSROIPooling", "bottom": ["feat", "rois"], "top": ["ps"],
                   "psroi_pooling_param": {"spatial_scale": 0.0625, "output_dim": 4, "group_size": 3}}]
    with pytest.raises(MiniCaffeError, match="input channel number does not match"):
        mc.Net.from_buffers(craft.to_prototxt(bad))
    bad = base + [{"name": "rp", "type": "ROIPooling", "bottom": ["feat", "rois"], "top": ["rp"],
                   "roi_pooling_param": {"pooled_h": 0, "pooled_w": 4}}]
    with pytest.raises(MiniCaffeError, match="pooled_h must be > 0"):
        mc.Net.from_buffers(craft.to_prototxt(bad))


# Every type string the reference registers (REGISTER_LAYER_CLASS / _CREATOR in
# src/layers/*.cpp).
REFERENCE_LAYER_TYPES = """AbsVal ArgMax BN BNLL BatchNorm Bias Concat Convolution ConvolutionDepthwise
Crop Deconvolution DetectionOutput Dropout ELU Eltwise Embed Exp Filter Flatten InnerProduct Input LRN
Log MVN Normalize PReLU PSROIPooling Parameter Permute Pooling Power PriorBox Proposal ROIPooling ReLU
Reduction Reshape SPP Scale ShuffleChannel Sigmoid Slice Softmax Split TanH Threshold Tile""".split()


def test_registry_holds_every_reference_layer_type():
    msg = err(lambda: mc.Net.from_buffers('layer { name: "x" type: "NoSuchLayer" top: "x" }'))
    assert "Unknown layer type: NoSuchLayer" in msg
    known = msg.split("known types:")[1].strip(" )").split(", ")
    assert sorted(known) == sorted(REFERENCE_LAYER_TYPES)


def test_zoo_layers_shapes_params_and_setup_errors():
    E = craft.Enum
    base = [craft.input_layer({"d": (2, 6, 8, 8), "small": (2, 6, 4, 5), "idx": (3, 4), "sel": (2,)})]

    def one(ltype, bottoms, tops, **params):
        return base + [dict({"name": "l", "type": ltype, "bottom": bottoms, "top": tops}, **params)]

    def shape_of(spec, top="t"):
        net = mc.Net.from_buffers(craft.to_prototxt(spec))   # must outlive the blob view
        return tuple(net.get_blob(top).shape)

    for ltype in ("Dropout", "Power", "Exp", "Log", "AbsVal", "BNLL", "ELU", "Threshold", "PReLU",
                  "LRN", "MVN", "ShuffleChannel", "BN"):
        assert shape_of(one(ltype, ["d"], ["t"])) == (2, 6, 8, 8), ltype
    # parameter blobs: PReLU slope (default filler 0.25), BN's four, Embed, ConvolutionDepthwise
    net = mc.Net.from_buffers(craft.to_prototxt(one("PReLU", ["d"], ["t"])))
    assert [(n, b.shape) for n, b in net.param_list] == [("l_0", [6])]
    assert np.all(net.param_list[0][1].data == 0.25)
    net = mc.Net.from_buffers(craft.to_prototxt(
        one("PReLU", ["d"], ["t"], prelu_param={"channel_shared": True, "filler": {"value": 0.1}})))
    assert net.param_list[0][1].shape == [] and np.allclose(net.param_list[0][1].data, 0.1)
    net = mc.Net.from_buffers(craft.to_prototxt(one("BN", ["d"], ["t"])))
    assert [b.shape for _, b in net.param_list] == [[1, 6]] * 4
    assert [float(b.data.ravel()[0]) for _, b in net.param_list] == [0.0, 0.0, 0.0, 1.0]
    net = mc.Net.from_buffers(craft.to_prototxt(
        one("ConvolutionDepthwise", ["d"], ["t"],
            convolution_param={"num_output": 99, "kernel_size": 3, "stride": 2, "pad": 1})))
    assert tuple(net.get_blob("t").shape) == (2, 6, 4, 4)
    assert [b.shape for _, b in net.param_list] == [[6, 1, 3, 3], [6]]
    net = mc.Net.from_buffers(craft.to_prototxt(
        one("Embed", ["idx"], ["t"], embed_param={"num_output": 5, "input_dim": 9})))
    assert tuple(net.get_blob("t").shape) == (3, 4, 5)
    assert [b.shape for _, b in net.param_list] == [[9, 5], [5]]
    # shapes
    assert shape_of(one("ArgMax", ["d"], ["t"])) == (2, 1, 1, 1)
    assert shape_of(one("ArgMax", ["d"], ["t"], argmax_param={"top_k": 3, "out_max_val": True})) == (2, 2, 3, 1)
    assert shape_of(one("ArgMax", ["d"], ["t"], argmax_param={"top_k": 2, "axis": 1})) == (2, 2, 8, 8)
    assert shape_of(one("Reduction", ["d"], ["t"], reduction_param={"axis": 2})) == (2, 6)
    assert shape_of(one("Reduction", ["d"], ["t"])) == ()
    assert shape_of(one("Crop", ["d", "small"], ["t"], crop_param={"offset": [2, 1]})) == (2, 6, 4, 5)
    assert shape_of(one("Crop", ["d", "small"], ["t"], crop_param={"axis": 1, "offset": 0})) == (2, 6, 4, 5)
    assert shape_of(one("Tile", ["d"], ["t"], tile_param={"tiles": 3})) == (2, 18, 8, 8)
    assert shape_of(one("Tile", ["d"], ["t"], tile_param={"tiles": 2, "axis": -1})) == (2, 6, 8, 16)
    assert shape_of(one("SPP", ["d"], ["t"], spp_param={"pyramid_height": 3})) == (2, 6 * 21)
    assert shape_of(one("SPP", ["d"], ["t"], spp_param={"pyramid_height": 1, "pool": E("AVE")})) == (2, 6, 1, 1)
    # Net::Init reshapes twice (SetUp, then PlaceMemory): the second time the all-zero
    # selector keeps no item, as in the reference (net.cpp:52,72,149).
    assert shape_of(one("Filter", ["d", "sel"], ["t"])) == (0, 6, 8, 8)
    par = base + [{"name": "p", "type": "Parameter", "top": ["t"], "parameter_param": {"shape": {"dim": [3, 2]}}}]
    net = mc.Net.from_buffers(craft.to_prototxt(par))
    assert tuple(net.get_blob("t").shape) == (3, 2) and net.param_list[0][1].shape == [3, 2]
    # set-up errors carry the reference's messages
    bad = lambda *a, **k: err(lambda: mc.Net.from_buffers(craft.to_prototxt(one(*a, **k))))
    assert "odd values for local_size" in bad("LRN", ["d"], ["t"], lrn_param={"local_size": 4})
    assert "base must be strictly positive" in bad("Exp", ["d"], ["t"], exp_param={"base": -2.0})
    assert "base must be strictly positive" in bad("Log", ["d"], ["t"], log_param={"base": 0.0})
    assert "top_k must be less than or equal" in bad("ArgMax", ["d"], ["t"], argmax_param={"top_k": 7, "axis": 1})
    assert "top k must not be less than 1" in bad("ArgMax", ["d"], ["t"], argmax_param={"top_k": 0})
    assert "Number of tiles must be specified" in bad("Tile", ["d"], ["t"])
    assert "out-of-bounds" in bad("Crop", ["d", "small"], ["t"], crop_param={"offset": 5})
    assert "number of offset values" in bad("Crop", ["d", "small"], ["t"], crop_param={"offset": [1, 1, 1]})
    assert "group must be greater than 0" in bad("ShuffleChannel", ["d"], ["t"], shuffle_channel_param={"group": 0})
    assert "Wrong group size" in bad("ShuffleChannel", ["d"], ["t"], shuffle_channel_param={"group": 4})
    assert "input_dim must be positive" in bad("Embed", ["idx"], ["t"], embed_param={"num_output": 5})
    assert "shape mismatch" in err(lambda: mc.Net.from_buffers(
        craft.to_prototxt(one("PReLU", ["d"], ["t"])), wire.net("m", [wire.layer("l", "PReLU", [np.zeros(5, np.float32)])])))
    assert "Selector blob dimensions must be singletons" in bad("Filter", ["d", "idx"], ["t"])
    assert "Unknown reduction op" in bad("Reduction", ["d"], ["t"], reduction_param={"operation": E("PRODUCT")})


V1_NET = """
name: "v1"
input: "data"
input_dim: 2 input_dim: 3 input_dim: 12 input_dim: 10
layers { name: "conv1" type: CONVOLUTION bottom: "data" top: "conv1"
         blobs_lr: 1 blobs_lr: 2 weight_decay: 1 weight_decay: 0
         convolution_param { num_output: 8 kernel_h: 3 kernel_w: 2 stride_h: 2 stride_w: 1 pad_h: 1 pad_w: 0 } }
layers { name: "relu" type: RELU bottom: "conv1" top: "conv1" }
layers { name: "norm" type: LRN bottom: "conv1" top: "norm" lrn_param { local_size: 3 alpha: 0.1 } }
layers { name: "pool" type: POOLING bottom: "norm" top: "pool" pooling_param { pool: AVE kernel_size: 2 stride: 2 } }
layers { name: "drop" type: DROPOUT bottom: "pool" top: "pool" dropout_param { dropout_ratio: 0.3 } }
layers { name: "ip" type: INNER_PRODUCT bottom: "pool" top: "ip" inner_product_param { num_output: 5 bias_term: false } }
layers { name: "prob" type: 20 bottom: "ip" top: "prob" }
"""


def test_v1_layers_definition_is_upgraded():
    """V1 `layers { type: ENUM }` prototxt and caffemodel (upgrade_proto.cpp:60-265)."""
    net = mc.Net.from_buffers(V1_NET)
    shapes = {k: v.shape for k, v in net.blobs.items()}
    assert shapes == {"data": [2, 3, 12, 10], "conv1": [2, 8, 6, 9], "norm": [2, 8, 6, 9],
                      "pool": [2, 8, 3, 5], "ip": [2, 5], "prob": [2, 5]}
    assert [n for n, _ in net.param_list] == ["conv1_0", "conv1_1", "ip_0"]
    rng = np.random.default_rng(0)
    w = rng.standard_normal((8, 3, 3, 2)).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    ipw = rng.standard_normal((5, 120)).astype(np.float32)
    model = wire.net("m", [], v1_layers=[wire.v1_layer("conv1", 4, [w, b], legacy=True),
                                         wire.v1_layer("ip", 14, [ipw], legacy=True)])
    net = mc.Net.from_buffers(V1_NET, model)
    params = dict(net.param_list)
    assert np.array_equal(params["conv1_0"].data, w) and np.array_equal(params["ip_0"].data, ipw)
    assert "Unknown V1LayerParameter layer type: ARGMAX" in err(
        lambda: mc.Net.from_buffers(V1_NET.replace("type: RELU", "type: ARGMAX")))
    assert "both 'layer' and 'layers'" in err(
        lambda: mc.Net.from_buffers(V1_NET + 'layer { name: "x" type: "ReLU" bottom: "ip" top: "ip" }'))


@needs_ref
def test_mobilenet_ssd_builder_matches_the_reference_prototxt():
    """zoo.mobilenet_ssd_spec builds the graph of example/models/ssd/MobileNetSSD_deploy.prototxt:
    same blobs, shapes and parameter blobs, 1917 priors."""
    spec, _ = zoo.mobilenet_ssd_spec()
    mine = mc.Net.from_buffers(craft.to_prototxt(spec))
    ref = mc.Net.from_buffers(open(os.path.join(REF, "example", "models", "ssd",
                                                "MobileNetSSD_deploy.prototxt")).read())
    assert {k: v.shape for k, v in mine.blobs.items()} == {k: v.shape for k, v in ref.blobs.items()}
    assert [(n, b.shape) for n, b in mine.param_list] == [(n, b.shape) for n, b in ref.param_list]
    assert mine.get_blob("mbox_priorbox").shape == [1, 2, 1917 * 4]
    # the ConvolutionDepthwise spelling of the same graph has the same blobs and parameters
    spec_dw, _ = zoo.mobilenet_ssd_spec(depthwise_type=True)
    dw = mc.Net.from_buffers(craft.to_prototxt(spec_dw))
    assert [(n, b.shape) for n, b in dw.param_list] == [(n, b.shape) for n, b in ref.param_list]


def test_benchmark_tool_is_built_against_public_headers(tmp_path):
    """The reference's timing tool (tools/benchmark.cpp) rebuilt from the public C++ headers:
    same command line; without a device it builds the net and then refuses to run it."""
    import subprocess
    exe = os.path.join(ROOT, "mini-caffe_amd", "bin", "benchmark")
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    from minicaffe import craft, zoo
    spec, _ = zoo.c1_spec()
    proto = tmp_path / "net.prototxt"
    proto.write_text(craft.to_prototxt(spec))
    r = subprocess.run([exe], capture_output=True, text=True, cwd=tmp_path)
    assert r.returncode != 0 and "Usage" in (r.stdout + r.stderr)
    r = subprocess.run([exe, str(proto), "1", "-1"], capture_output=True, text=True, cwd=tmp_path)
    out = r.stdout + r.stderr
    assert r.returncode == 1 and "net forward iterations: 1" in out and "HIP device path only" in out


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def landmark_level2_spec(batch=1):
    """Net definition of the reference's level-2 landmark nets (example/models/deeplandmark/2_*.prototxt),
    written from its description: 1x15x15 patch, 4x4 conv to 20, 2x2 max pool, 3x3 conv to 40,
    2x2 max pool, 60 hidden units, 2 outputs, ReLU after every parameter layer."""
    from minicaffe.craft import Enum, input_layer
    conv = lambda n, b, c, k: {"name": n, "type": "Convolution", "bottom": [b], "top": [n],  # noqa: E731
                               "convolution_param": {"num_output": c, "kernel_size": k}}
    relu = lambda n, b: {"name": n, "type": "ReLU", "bottom": [b], "top": [b]}  # noqa: E731
    pool = lambda n, b: {"name": n, "type": "Pooling", "bottom": [b], "top": [n],  # noqa: E731
                         "pooling_param": {"pool": Enum("MAX"), "kernel_size": 2, "stride": 2}}
    ip = lambda n, b, c: {"name": n, "type": "InnerProduct", "bottom": [b], "top": [n],  # noqa: E731
                          "inner_product_param": {"num_output": c}}
    return [input_layer({"data": (batch, 1, 15, 15)}), conv("conv1", "data", 20, 4), relu("relu1", "conv1"),
            pool("pool1", "conv1"), conv("conv2", "pool1", 40, 3), relu("relu2", "conv2"), pool("pool2", "conv2"),
            ip("fc1", "pool2", 60), relu("relu_fc1", "fc1"), ip("fc2", "fc1", 2), relu("relu_fc2", "fc2")]


def test_golden_caffemodel_loads_into_the_landmark_net():
    """tests/golden holds trained weights from the reference's example data.  The library's
    caffemodel reader must give the values an independent wire-format walk finds."""
    from minicaffe import craft
    model = open(os.path.join(GOLDEN, "deeplandmark_2_LE1.caffemodel"), "rb").read()
    want = wire.read_net_blobs(model)
    assert sorted(want) == ["conv1", "conv2", "fc1", "fc2"]
    net = mc.Net.from_buffers(craft.to_prototxt(landmark_level2_spec()), model)
    params = dict(net.param_list)
    for layer, blobs in want.items():
        for j, arr in enumerate(blobs):
            got = params["%s_%d" % (layer, j)].data
            assert got.shape == arr.shape and np.array_equal(got, arr), (layer, j)
    assert net.blobs["fc2"].shape == [1, 2]


def test_net_to_proto_round_trip(tmp_path):
    """Net::ToProto (reference src/net.cpp:293-301): the definition with the current weights
    builds an equal net, survives the wire-format writer and reader, and the written bytes
    hold the trained values when walked by the independent reader of tests/wire.py."""
    import subprocess
    from minicaffe import craft
    exe = os.path.join(ROOT, "mini-caffe_amd", "bin", "net_roundtrip")
    assert os.path.exists(exe), "run __graft_entry__.build() first"
    proto = tmp_path / "net.prototxt"
    proto.write_text(craft.to_prototxt(landmark_level2_spec(), "landmark"))
    model = os.path.join(GOLDEN, "deeplandmark_2_LE1.caffemodel")
    out = tmp_path / "out.caffemodel"
    r = subprocess.run([exe, str(proto), model, str(out)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "roundtrip ok: 8 parameter blobs" in r.stdout
    want = wire.read_net_blobs(open(model, "rb").read())
    got = wire.read_net_blobs(out.read_bytes())
    assert sorted(got) == sorted(want)
    for layer in want:
        assert len(got[layer]) == len(want[layer])
        for a, b in zip(got[layer], want[layer]):
            assert a.shape == b.shape and np.array_equal(a, b), layer
    # and the library reads its own bytes back as weights through the C ABI
    net = mc.Net.from_buffers(proto.read_text(), out.read_bytes())
    params = dict(net.param_list)
    assert np.array_equal(params["fc2_0"].data, want["fc2"][0])


@needs_ref
def test_landmark_spec_equals_the_reference_prototxt():
    from minicaffe import craft
    ref = mc.Net.from_buffers(open(os.path.join(REF, "example", "models", "deeplandmark", "2_LE1.prototxt")).read())
    own = mc.Net.from_buffers(craft.to_prototxt(landmark_level2_spec()))
    assert [(k, v.shape) for k, v in ref.blobs.items()] == [(k, v.shape) for k, v in own.blobs.items()]
    assert [(k, v.shape) for k, v in ref.param_list] == [(k, v.shape) for k, v in own.param_list]
    # and the fixture is the reference's file
    a = open(os.path.join(REF, "example", "models", "deeplandmark", "2_LE1.caffemodel"), "rb").read()
    assert a == open(os.path.join(GOLDEN, "deeplandmark_2_LE1.caffemodel"), "rb").read()


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asking for more ends with a message instead of a number."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "one GPU" in (r.stdout + r.stderr)
    assert "{" not in r.stdout
