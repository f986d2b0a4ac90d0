"""End-to-end parity through the reference's own C ABI on the MI355X: build a net
from prototxt text, inject seeded weights through CaffeNetListParam, run
CaffeNetForward, compare blobs with the CPU oracle walking the same layers.

Tolerance: relative error (netrun.rel_err) 1e-4 for single layers, 1e-3 for deep
nets, as the configurations state.
"""
import numpy as np
import pytest

import oracle
from oracle import netrun

pytestmark = pytest.mark.gpu


def run_net(mc, spec, inputs, marks=()):
    from minicaffe import craft
    net = mc.Net.from_buffers(craft.to_prototxt(spec))
    craft.load_weights(net, spec)
    for m in marks:
        net.mark_output(m)
    net.forward(**inputs)
    return net


def test_config1_conv_relu(gpu_mode):
    from minicaffe import zoo
    oracle.use_openblas(False)
    spec, inputs = zoo.c1_spec()
    net = run_net(gpu_mode, spec, inputs)
    got = net.get_blob("conv").data.copy()
    want = netrun.oracle_forward(spec, inputs)["conv"]
    assert netrun.rel_err(got, want) < 1e-4
    assert (got >= 0).all() and (got == 0).mean() > 0.3   # the ReLU really ran
    # against an exact (float64) evaluation the HIP result is as good as the oracle's
    import torch
    x64 = torch.from_numpy(inputs["data"]).double()
    exact = torch.relu(torch.nn.functional.conv2d(
        x64, torch.from_numpy(spec[1]["blobs"][0]).double(),
        torch.from_numpy(spec[1]["blobs"][1]).double(), padding=1)).numpy()
    assert netrun.rel_err(got, exact) < 2 * max(netrun.rel_err(want, exact), 1e-5)


def test_small_resnet_every_marked_blob(gpu_mode):
    """All ResNet layer types with non-trivial BatchNorm statistics and Scale
    parameters: a wrong fold (dropped mean, swapped gamma/beta, missing eps) shows."""
    from minicaffe import zoo
    oracle.use_openblas(False)
    spec, inputs = zoo.resnet50_spec(batch=3, size=65, stages=(2, 2, 1, 1), width=16,
                                     num_classes=10, bn_seed=3)
    marks = ["conv1", "pool1", "res2a_branch1", "res2a", "res2b", "res3a", "res5a", "pool5", "fc1000"]
    net = run_net(gpu_mode, spec, inputs, marks)
    want = netrun.oracle_forward(spec, inputs)
    for name in marks + ["prob"]:
        got = net.get_blob(name).data
        assert got.shape == want[name].shape
        assert netrun.rel_err(got, want[name]) < 1e-3, name
    assert np.allclose(net.get_blob("prob").data.sum(axis=1), 1, atol=1e-5)


def test_forward_twice_and_weight_update(gpu_mode):
    """A second forward reuses packed filters and folded epilogues; changing a
    parameter blob through the C ABI must invalidate both."""
    from minicaffe import zoo
    oracle.use_openblas(False)
    spec, inputs = zoo.resnet50_spec(batch=1, size=33, stages=(1, 1, 1, 1), width=8,
                                     num_classes=5, bn_seed=1)
    net = run_net(gpu_mode, spec, inputs, ["fc1000"])
    first = net.get_blob("fc1000").data.copy()
    net.forward()
    assert np.array_equal(net.get_blob("fc1000").data, first)
    params = dict(net.param_list)
    spec[1]["blobs"][0] = spec[1]["blobs"][0] * 0.5            # conv1 filter
    params["conv1_0"].data[...] = spec[1]["blobs"][0]
    spec[3]["blobs"][0] = spec[3]["blobs"][0] + 0.25           # scale_conv1 gamma
    params["scale_conv1_0"].data[...] = spec[3]["blobs"][0]
    spec[2]["blobs"][0] = spec[2]["blobs"][0] + 0.1            # bn_conv1 mean
    params["bn_conv1_0"].data[...] = spec[2]["blobs"][0]
    net.forward()
    got = net.get_blob("fc1000").data.copy()
    assert not np.allclose(got, first)
    want = netrun.oracle_forward(spec, inputs)["fc1000"]
    assert netrun.rel_err(got, want) < 1e-3


def test_reshape_and_batch_invariance(gpu_mode):
    """The reference's one numeric test (tests/run_net.cpp:274-321): the output for
    an image does not depend on the batch it rides in, across input reshapes."""
    from minicaffe import zoo
    spec, inputs = zoo.resnet50_spec(batch=1, size=64, stages=(1, 1, 1, 1), width=16,
                                     num_classes=10, bn_seed=2)
    net = run_net(gpu_mode, spec, inputs)
    x = inputs["data"]
    p1 = net.get_blob("prob").data.copy()
    x2 = np.concatenate([x, x], axis=0)
    net.forward(data=x2)
    p2 = net.get_blob("prob").data.copy()
    assert p2.shape == (2, 10)
    net.forward(data=x)
    p3 = net.get_blob("prob").data.copy()
    assert np.abs(p2[0] - p1[0]).max() < 1e-6 and np.abs(p2[1] - p1[0]).max() < 1e-6
    assert np.abs(p3 - p1).max() < 1e-6
    # a different spatial size re-plans the convolutions
    xs = np.random.default_rng(3).uniform(-1, 1, (2, 3, 48, 40)).astype(np.float32)
    net.forward(data=xs)
    want = netrun.oracle_forward(spec, {"data": xs})["prob"]
    assert netrun.rel_err(net.get_blob("prob").data, want) < 1e-3


def test_unfused_layers_standalone(gpu_mode):
    """BatchNorm / Scale / Bias / ReLU / TanH / Sigmoid / Eltwise that do NOT follow a
    contraction run as their own kernels; Split, Slice, Concat, Flatten, Reshape,
    Permute move data."""
    from minicaffe.craft import Enum, input_layer
    rng = np.random.default_rng(4)
    C = 6
    spec = [input_layer({"data": (2, C, 5, 7)}),
            {"name": "split", "type": "Split", "bottom": ["data"], "top": ["a", "b"]},
            {"name": "bn", "type": "BatchNorm", "bottom": ["a"], "top": ["bn"],
             "batch_norm_param": {"eps": 1e-3},
             "blobs": [rng.standard_normal(C).astype(np.float32), (rng.random(C) + 0.5).astype(np.float32),
                       np.array([0.8], np.float32)]},
            {"name": "sc", "type": "Scale", "bottom": ["bn"], "top": ["bn"], "scale_param": {"bias_term": True},
             "blobs": [rng.standard_normal(C).astype(np.float32), rng.standard_normal(C).astype(np.float32)]},
            {"name": "th", "type": "TanH", "bottom": ["bn"], "top": ["th"]},
            {"name": "bnb", "type": "BatchNorm", "bottom": ["b"], "top": ["bnb"],
             "batch_norm_param": {"use_global_stats": False},
             "blobs": [np.zeros(C, np.float32), np.zeros(C, np.float32), np.zeros(1, np.float32)]},
            {"name": "bias", "type": "Bias", "bottom": ["bnb"], "top": ["bnb"],
             "blobs": [rng.standard_normal(C).astype(np.float32)]},
            {"name": "sg", "type": "Sigmoid", "bottom": ["bnb"], "top": ["sg"]},
            {"name": "elt", "type": "Eltwise", "bottom": ["th", "sg", "data"], "top": ["elt"],
             "eltwise_param": {"operation": Enum("SUM"), "coeff": [1.0, -0.5, 2.0]}},
            {"name": "lrelu", "type": "ReLU", "bottom": ["elt"], "top": ["elt"],
             "relu_param": {"negative_slope": 0.3}},
            {"name": "mx", "type": "Eltwise", "bottom": ["elt", "data"], "top": ["mx"],
             "eltwise_param": {"operation": Enum("MAX")}},
            {"name": "slice", "type": "Slice", "bottom": ["mx"], "top": ["s0", "s1", "s2"],
             "slice_param": {"axis": 1, "slice_point": [1, 4]}},
            {"name": "cat", "type": "Concat", "bottom": ["s2", "s0", "s1"], "top": ["cat"]},
            {"name": "perm", "type": "Permute", "bottom": ["cat"], "top": ["perm"],
             "permute_param": {"order": [0, 2, 3, 1]}},
            {"name": "flat", "type": "Flatten", "bottom": ["perm"], "top": ["flat"]},
            {"name": "resh", "type": "Reshape", "bottom": ["flat"], "top": ["resh"],
             "reshape_param": {"shape": {"dim": [0, -1, C]}}},
            {"name": "sm", "type": "Softmax", "bottom": ["resh"], "top": ["sm"], "softmax_param": {"axis": 2}}]
    inputs = {"data": rng.standard_normal((2, C, 5, 7)).astype(np.float32)}
    marks = ["th", "sg", "elt", "mx", "cat", "perm", "resh"]
    net = run_net(gpu_mode, spec, inputs, marks)
    want = netrun.oracle_forward(spec, inputs)
    for name in marks + ["sm"]:
        got = net.get_blob(name).data
        assert got.shape == want[name].shape, name
        assert netrun.rel_err(got, want[name]) < 1e-5, name


def test_resnet50_full_graph_two_images(gpu_mode):
    """The real ResNet-50 graph at 224x224 (229 layers); the oracle uses OpenBLAS for
    its sgemm, as the reference does."""
    from minicaffe import zoo
    oracle.use_openblas(True)
    try:
        spec, inputs = zoo.resnet50_spec(batch=2, size=224, seed=0, bn_seed=7)
        net = run_net(gpu_mode, spec, inputs, ["res3d", "res5c", "fc1000"])
        want = netrun.oracle_forward(spec, inputs, keep={"res3d", "res5c", "fc1000", "prob"})
    finally:
        oracle.use_openblas(False)
    for name in ("res3d", "res5c", "fc1000", "prob"):
        assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-3, name


def test_resnet50_b64_properties(gpu_mode):
    """Full benchmark size: size-independent properties instead of a CPU run.
    Rows of the batch-64 result equal the batch-1 result of the same image, rows
    sum to one, and duplicated images give identical rows."""
    from minicaffe import zoo
    spec, inputs = zoo.resnet50_spec(batch=64, size=224, seed=0)
    x = inputs["data"]
    x[63] = x[5]
    net = run_net(gpu_mode, spec, {"data": x})
    p64 = net.get_blob("prob").data.copy()
    assert p64.shape == (64, 1000) and np.isfinite(p64).all()
    assert np.allclose(p64.sum(axis=1), 1, atol=1e-4)
    assert np.array_equal(p64[63], p64[5])
    net.forward(data=x[17:18])
    p1 = net.get_blob("prob").data.copy()
    assert np.abs(p1[0] - p64[17]).max() < 1e-6
