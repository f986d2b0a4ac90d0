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


def test_nets_with_every_3x3_layer_on_the_winograd_path(gpu_mode):
    """The library takes the Winograd path by size, which small test nets never reach:
    with mcConvWinogradDefault(1) every 3x3 stride-1 convolution of a small ResNet (folded
    BatchNorm / Scale / ReLU and residual sums in the output transform), of it again at another
    batch size and after a weight update, and of a quarter-width SSD300 runs through it."""
    from minicaffe import zoo
    from minicaffe.base import LIB
    oracle.use_openblas(False)
    LIB.mcConvWinogradDefault(1)
    try:
        spec, inputs = zoo.resnet50_spec(batch=3, size=65, stages=(2, 2, 1, 1), width=16,
                                         num_classes=10, bn_seed=3)
        marks = ["conv1", "res2a", "res2b", "res3a", "res5a", "fc1000"]
        net = run_net(gpu_mode, spec, inputs, marks)
        want = netrun.oracle_forward(spec, inputs)
        for name in marks + ["prob"]:
            assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-3, name
        # a filter of a Winograd layer changes: its transformed copy must follow
        params = dict(net.param_list)
        idx = next(i for i, layer in enumerate(spec) if layer["name"] == "res2a_branch2b")
        spec[idx]["blobs"][0] = spec[idx]["blobs"][0] * -0.7
        params["res2a_branch2b_0"].data[...] = spec[idx]["blobs"][0]
        net.forward()
        want = netrun.oracle_forward(spec, inputs)
        assert netrun.rel_err(net.get_blob("fc1000").data, want["fc1000"]) < 1e-3
        # another batch size through the same plans
        spec2, inputs2 = zoo.resnet50_spec(batch=5, size=65, stages=(2, 2, 1, 1), width=16,
                                           num_classes=10, bn_seed=3)
        spec2[idx]["blobs"][0] = spec[idx]["blobs"][0]
        net.forward(**inputs2)
        want2 = netrun.oracle_forward(spec2, inputs2)
        assert netrun.rel_err(net.get_blob("fc1000").data, want2["fc1000"]) < 1e-3
        del net

        spec, inputs = zoo.ssd300_spec(batch=2, seed=4, width=16)
        net = run_net(gpu_mode, spec, inputs, ["conv4_3_norm", "fc7", "mbox_loc", "mbox_conf"])
        want = netrun.oracle_forward(spec, inputs)
        for name in ("conv4_3_norm", "fc7", "mbox_loc", "mbox_conf"):
            assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-3, name
    finally:
        LIB.mcConvWinogradDefault(-1)


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


def test_three_threads_each_with_their_own_net(gpu_mode):
    """The reference's concurrency smoke test (tests/run_net.cpp:238-246): every
    thread selects the device itself, builds and runs its own net and clears its
    own memory pool.  Here each thread's result is also checked against the oracle."""
    import threading
    from minicaffe import zoo
    oracle.use_openblas(False)
    jobs = []
    for t in range(3):
        spec, inputs = zoo.resnet50_spec(batch=2 + t, size=48 + 16 * t, stages=(1, 1, 1, 1), width=8,
                                         num_classes=7, bn_seed=10 + t, seed=20 + t)
        jobs.append((spec, inputs, netrun.oracle_forward(spec, inputs)["prob"]))
    got, errors = [None] * 3, []

    def work(t):
        try:
            gpu_mode.set_runtime_mode(1, 0)
            spec, inputs, _ = jobs[t]
            net = run_net(gpu_mode, spec, inputs)
            for _ in range(3):
                net.forward()
            got[t] = net.get_blob("prob").data.copy()
            del net                      # a net is destroyed on the thread that ran it
            gpu_mode.memory_pool_clear()
        except Exception as e:           # noqa: BLE001 - reported by the main thread
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=work, args=(t,)) for t in range(3)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    for t in range(3):
        assert got[t] is not None and got[t].shape == jobs[t][2].shape
        assert netrun.rel_err(got[t], jobs[t][2]) < 1e-3, t


def test_two_threads_running_forwards_at_the_same_time_keep_their_bits(gpu_mode):
    """Two threads, each with its own net (different sizes and weights), run forty forwards
    each at the same time on their own streams: launches of the two streams share the chip,
    and the partial sums and arrival counters of sliced contractions belong to the (thread,
    stream) pair.  Every forward must give the bits the same net gave when it ran alone."""
    import threading
    from minicaffe import zoo
    jobs = [zoo.resnet50_spec(batch=6, size=96, stages=(1, 2, 1, 1), width=64, num_classes=9, bn_seed=5, seed=6),
            zoo.resnet50_spec(batch=4, size=128, stages=(2, 1, 1, 1), width=32, num_classes=11, bn_seed=7, seed=8)]
    alone = []
    for spec, inputs in jobs:
        net = run_net(gpu_mode, spec, inputs)
        alone.append({k: net.get_blob(k).data.copy() for k in ("prob", "fc1000")})
        del net
    bar = threading.Barrier(2)
    errors = []

    def work(t):
        try:
            gpu_mode.set_runtime_mode(1, 0)
            spec, inputs = jobs[t]
            net = run_net(gpu_mode, spec, inputs)
            bar.wait(timeout=60)
            for it in range(40):
                net.forward()
                for k, want in alone[t].items():
                    got = net.get_blob(k).data
                    if not np.array_equal(got, want):
                        errors.append((t, it, k, float(np.abs(got - want).max())))
                        return
            del net
            gpu_mode.memory_pool_clear()
        except Exception as e:           # noqa: BLE001 - reported by the main thread
            errors.append((t, repr(e)))
            bar.abort()

    threads = [threading.Thread(target=work, args=(t,)) for t in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors


def test_short_lived_thread_leaves_no_device_memory(gpu_mode):
    """A thread that builds a net, runs it (contractions whose channel loop is cut into
    slices take partial-sum scratch and arrival counters from the kernel library, blobs
    come from the thread's pool) and ends WITHOUT clearing anything: what it allocated
    belongs to the thread and goes back to the device when the thread ends."""
    import threading
    import torch
    from minicaffe import zoo
    spec, inputs = zoo.resnet50_spec(batch=4, size=64, stages=(1, 1, 1, 1), width=32, num_classes=7,
                                     bn_seed=3, seed=4)
    errors = []

    def work():
        try:
            gpu_mode.set_runtime_mode(1, 0)
            net = run_net(gpu_mode, spec, inputs)
            for _ in range(2):
                net.forward()
            del net
        except Exception as e:           # noqa: BLE001 - reported by the main thread
            errors.append(repr(e))

    def one_thread():
        th = threading.Thread(target=work)
        th.start()
        th.join(timeout=100)
        assert not errors, errors
        torch.cuda.synchronize()
        return torch.cuda.mem_get_info()[0]

    one_thread()                          # (first use: code objects, the runtime's own pools)
    free_before = one_thread()
    for _ in range(6):
        free_after = one_thread()
    # the net, its weights and its scratch are some 20 MB per thread; the HIP runtime's own
    # pools grow in steps of 2 MiB now and then (seen: 4 MiB over three threads, once)
    assert free_before - free_after < (8 << 20), (free_before, free_after)


def test_flatten_and_reshape_as_views(gpu_mode):
    """Flatten and Reshape take over their bottom's memory when they are its last
    reader; a bottom that is read again, is a net input or is a marked output is
    copied.  All variants give the reference's values, on repeated passes and
    across a reshape of the input."""
    from minicaffe.craft import input_layer
    rng = np.random.default_rng(5)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    spec = [
        input_layer({"data": (2, 3, 6, 5)}),
        {"name": "in_flat", "type": "Flatten", "bottom": ["data"], "top": ["in_flat"]},          # input: copied
        {"name": "conv", "type": "Convolution", "bottom": ["data"], "top": ["conv"],
         "convolution_param": {"num_output": 4, "kernel_size": 3, "pad": 1}, "blobs": [f(4, 3, 3, 3) * 0.3, f(4)]},
        {"name": "perm", "type": "Permute", "bottom": ["conv"], "top": ["perm"], "permute_param": {"order": [0, 2, 3, 1]}},
        {"name": "flat", "type": "Flatten", "bottom": ["perm"], "top": ["flat"]},                  # view
        {"name": "resh", "type": "Reshape", "bottom": ["flat"], "top": ["resh"],
         "reshape_param": {"shape": {"dim": [0, -1, 4]}}},                                         # view of a view
        {"name": "sm", "type": "Softmax", "bottom": ["resh"], "top": ["sm"], "softmax_param": {"axis": 2}},
        {"name": "sm_flat", "type": "Flatten", "bottom": ["sm"], "top": ["sm_flat"]},              # view
        {"name": "relu", "type": "ReLU", "bottom": ["sm_flat"], "top": ["sm_flat"]},               # in place on a view
        {"name": "conv_flat", "type": "Flatten", "bottom": ["conv"], "top": ["conv_flat"]},        # conv read again below
        {"name": "pool", "type": "Pooling", "bottom": ["conv"], "top": ["pool"],
         "pooling_param": {"kernel_size": 2, "stride": 2}},
        {"name": "pool_flat", "type": "Flatten", "bottom": ["pool"], "top": ["pool_flat"]},        # pool is marked
        {"name": "cat", "type": "Concat", "bottom": ["in_flat", "sm_flat", "conv_flat", "pool_flat"], "top": ["cat"]},
    ]
    x = f(2, 3, 6, 5)
    net = run_net(gpu_mode, spec, {"data": x}, ["pool", "resh"])
    want = netrun.oracle_forward(spec, {"data": x})
    for _ in range(2):
        assert netrun.rel_err(net.get_blob("cat").data, want["cat"]) < 1e-5
        assert netrun.rel_err(net.get_blob("pool").data, want["pool"]) < 1e-5
        assert netrun.rel_err(net.get_blob("resh").data, want["resh"]) < 1e-5
        net.forward()
    x3 = f(3, 3, 9, 4)
    net.forward(data=x3)
    want = netrun.oracle_forward(spec, {"data": x3})
    assert net.get_blob("cat").data.shape == want["cat"].shape
    assert netrun.rel_err(net.get_blob("cat").data, want["cat"]) < 1e-5
    assert netrun.rel_err(net.get_blob("resh").data, want["resh"]) < 1e-5


def test_googlenet_front_and_nin(gpu_mode):
    """The other two nets the reference's test program runs (tests/run_net.cpp:175-236), at
    reduced size: GoogLeNet's stem and first two inception modules (a blob feeding four
    branches, 5x5 filters, LRN, 3x3/1 padded max pools, four-way Concat) and
    Network-in-Network (11x11/4 filters, 1x1 chains, Dropout, global average pool as the
    classifier).  Every stage against the oracle, and batch invariance as in
    run_net.cpp:274-321."""
    from minicaffe import zoo
    oracle.use_openblas(False)
    spec, inputs = zoo.googlenet_spec(batch=3, size=96, seed=4)
    marks = ["pool1/norm1", "conv2/norm2", "pool2/3x3_s2", "inception_0/5x5", "inception_0/pool_proj",
             "inception_0/output", "inception_1/output", "pool5", "loss3/classifier"]
    net = run_net(gpu_mode, spec, inputs, marks)
    want = netrun.oracle_forward(spec, inputs)
    for name in marks + ["prob"]:
        got = net.get_blob(name).data
        assert got.shape == want[name].shape, name
        assert netrun.rel_err(got, want[name]) < 1e-3, name
    p3 = net.get_blob("prob").data.copy()
    net.forward(data=inputs["data"][1:2])
    assert np.abs(net.get_blob("prob").data[0] - p3[1]).max() < 1e-6

    spec, inputs = zoo.nin_spec(batch=2, size=67, seed=5)
    marks = ["conv1", "cccp2", "pool0", "conv2", "pool2", "cccp8-1024", "pool4"]
    net = run_net(gpu_mode, spec, inputs, marks)
    want = netrun.oracle_forward(spec, inputs)
    for name in marks + ["prob"]:
        got = net.get_blob(name).data
        assert got.shape == want[name].shape, name
        assert netrun.rel_err(got, want[name]) < 1e-3, name
    assert np.allclose(net.get_blob("prob").data.reshape(2, -1).sum(axis=1), 1, atol=1e-5)


def test_sibling_convolutions_run_as_one_launch(gpu_mode):
    """Convolutions that read the same blob with the same window (SSD's loc / conf heads, the
    RPN's cls / bbox heads) are computed by one launch over the concatenated filters.  Pairs
    with and without bias, a third sibling that stays alone, and neighbours that must not be
    merged (other window, an in-place ReLU folded in, groups); later parameter updates of
    either partner and a new input size are honoured."""
    from minicaffe import zoo
    from minicaffe.craft import input_layer
    oracle.use_openblas(False)
    C = 12
    conv = lambda name, cout, k, pad, bias=True, group=1, seed=3: zoo.conv_layer(  # noqa: E731
        name, "feat", name, C, cout, k, 1, pad, group=group, bias=bias, seed=seed, bias_value=0.3)
    spec = [
        input_layer({"data": (2, 3, 13, 11)}),
        zoo.conv_layer("feat", "data", "feat", 3, C, 3, 1, 1, seed=3),
        zoo.relu_layer("feat_relu", "feat"),
        conv("loc", 8, 3, 1), conv("conf", 42, 3, 1),            # merged, both with bias
        conv("third", 5, 3, 1),                                  # same window: no partner left
        conv("a_nobias", 7, 1, 0, bias=False), conv("b_bias", 9, 1, 0),   # merged, one bias only
        conv("c_nobias", 4, 5, 2, bias=False), conv("d_nobias", 6, 5, 2, bias=False),  # merged, no bias at all
        conv("relu_head", 6, 3, 1), zoo.relu_layer("relu_head_relu", "relu_head"),   # has a follower: alone
        conv("grouped", 6, 3, 1, group=3),
    ]
    tops = ["loc", "conf", "third", "a_nobias", "b_bias", "c_nobias", "d_nobias", "relu_head", "grouped"]
    spec.append({"name": "cat", "type": "Concat", "bottom": tops, "top": ["cat"]})
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 3, 13, 11)).astype(np.float32)
    net = run_net(gpu_mode, spec, {"data": x}, tops)
    want = netrun.oracle_forward(spec, {"data": x})
    for name in tops + ["cat"]:
        assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-4, name
    # which layers ran on their own: the profiler opens a scope per executed layer
    import json
    import tempfile
    gpu_mode.Profiler.enable()
    net.forward()
    gpu_mode.Profiler.disable()
    with tempfile.TemporaryDirectory() as d:
        gpu_mode.Profiler.dump(d + "/p.json")
        ran = {e["name"] for e in json.load(open(d + "/p.json"))["traceEvents"]}
    assert {"loc", "third", "a_nobias", "c_nobias", "relu_head", "grouped"} <= ran
    assert not ({"conf", "b_bias", "d_nobias", "relu_head_relu"} & ran)
    # the second partner's filter and the first partner's bias change
    params = dict(net.param_list)
    by_name = {l["name"]: l for l in spec}
    by_name["conf"]["blobs"][0] = by_name["conf"]["blobs"][0] * -0.5
    params["conf_0"].data[...] = by_name["conf"]["blobs"][0]
    by_name["loc"]["blobs"][1] = by_name["loc"]["blobs"][1] + 1.0
    params["loc_1"].data[...] = by_name["loc"]["blobs"][1]
    x2 = rng.standard_normal((3, 3, 9, 14)).astype(np.float32)
    net.forward(data=x2)
    want = netrun.oracle_forward(spec, {"data": x2})
    for name in tops + ["cat"]:
        got = net.get_blob(name).data
        assert got.shape == want[name].shape and netrun.rel_err(got, want[name]) < 1e-4, name


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


def test_batch_norm_head_takes_only_scale_bias_followers(gpu_mode):
    """A BatchNorm that runs as its own pass absorbs an in-place Scale / Bias and an
    activation; an in-place BN or a second BatchNorm behind it carries a subtraction of
    its own and must run as its own pass.  Both statistics modes."""
    from minicaffe.craft import input_layer
    rng = np.random.default_rng(14)
    C = 5

    def stats():
        return [rng.standard_normal(C).astype(np.float32), (rng.random(C) + 0.5).astype(np.float32),
                np.array([0.7], np.float32)]

    def bn_blobs():
        return [a.reshape(1, C) for a in (rng.standard_normal(C).astype(np.float32),
                                          rng.standard_normal(C).astype(np.float32),
                                          rng.standard_normal(C).astype(np.float32),
                                          (rng.random(C) + 0.5).astype(np.float32))]

    spec = [input_layer({"data": (3, C, 4, 6)}),
            {"name": "split", "type": "Split", "bottom": ["data"], "top": ["a", "b", "c"]},
            # batch statistics head, BN follower, ReLU
            {"name": "bn_a", "type": "BatchNorm", "bottom": ["a"], "top": ["ya"],
             "batch_norm_param": {"use_global_stats": False},
             "blobs": [np.zeros(C, np.float32), np.zeros(C, np.float32), np.zeros(1, np.float32)]},
            {"name": "fused_a", "type": "BN", "bottom": ["ya"], "top": ["ya"], "blobs": bn_blobs()},
            {"name": "relu_a", "type": "ReLU", "bottom": ["ya"], "top": ["ya"]},
            # stored statistics head (first layer on its blob, so it is the head), BatchNorm follower
            {"name": "bn_b", "type": "BatchNorm", "bottom": ["b"], "top": ["yb"], "blobs": stats()},
            {"name": "bn_b2", "type": "BatchNorm", "bottom": ["yb"], "top": ["yb"],
             "batch_norm_param": {"eps": 1e-2}, "blobs": stats()},
            {"name": "tanh_b", "type": "TanH", "bottom": ["yb"], "top": ["yb"]},
            # the supported run for comparison: Scale + ReLU ride along
            {"name": "bn_c", "type": "BatchNorm", "bottom": ["c"], "top": ["yc"], "blobs": stats()},
            {"name": "sc_c", "type": "Scale", "bottom": ["yc"], "top": ["yc"], "scale_param": {"bias_term": True},
             "blobs": [rng.standard_normal(C).astype(np.float32), rng.standard_normal(C).astype(np.float32)]},
            {"name": "relu_c", "type": "ReLU", "bottom": ["yc"], "top": ["yc"]}]
    inputs = {"data": rng.standard_normal((3, C, 4, 6)).astype(np.float32)}
    net = run_net(gpu_mode, spec, inputs, ["ya", "yb", "yc"])
    want = netrun.oracle_forward(spec, inputs)
    for name in ("ya", "yb", "yc"):
        assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-5, name


def test_view_behind_detection_output_sees_the_final_rows(gpu_mode):
    """DetectionOutput sizes its top after the device has counted the rows; a Flatten
    behind it must copy those rows (not alias the block the top had before Forward)."""
    from minicaffe.craft import Enum, input_layer
    rng = np.random.default_rng(15)
    num, P, C = 2, 40, 4
    c = rng.random((P, 2)) * 0.8 + 0.1
    wh = rng.random((P, 2)) * 0.3 + 0.05
    prior = np.concatenate([np.concatenate([c - wh / 2, c + wh / 2], 1).reshape(-1),
                            np.tile([0.1, 0.1, 0.2, 0.2], P)]).reshape(1, 2, P * 4).astype(np.float32)
    loc = (rng.standard_normal((num, P * 4)) * 0.5).astype(np.float32)
    conf = oracle.softmax((rng.standard_normal((num, P, C)) * 2).astype(np.float32), 2).reshape(num, P * C)
    param = {"num_classes": C, "share_location": True, "background_label_id": 0,
             "code_type": Enum("CENTER_SIZE"), "keep_top_k": 20, "confidence_threshold": 0.05,
             "nms_param": {"nms_threshold": 0.45, "top_k": 15}}
    spec = [input_layer({"loc": loc.shape, "conf": conf.shape, "prior": prior.shape}),
            {"name": "det", "type": "DetectionOutput", "bottom": ["loc", "conf", "prior"], "top": ["det"],
             "detection_output_param": param},
            {"name": "flat", "type": "Flatten", "bottom": ["det"], "top": ["flat"],
             "flatten_param": {"axis": 0}}]
    net = run_net(gpu_mode, spec, {"loc": loc, "conf": conf, "prior": prior})
    want = oracle.detection_output(dict(param, code_type="CENTER_SIZE"), loc, conf, prior)
    assert want.shape[0] > 5
    assert np.array_equal(net.get_blob("flat").data.reshape(-1, 7), want)
    net.forward(loc=loc, conf=conf, prior=prior)          # and on a repeated call
    assert np.array_equal(net.get_blob("flat").data.reshape(-1, 7), want)


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
    """Full benchmark size.  Rows 0, 17 and 63 of the batch-64 result are compared with
    the CPU oracle walking the same three images (`res5c` and `prob`); for the rest,
    size-independent properties: rows of the batch-64 result equal the batch-1 result
    of the same image, rows sum to one, and duplicated images give identical rows."""
    from minicaffe import zoo
    spec, inputs = zoo.resnet50_spec(batch=64, size=224, seed=0)
    x = inputs["data"]
    x[63] = x[5]
    net = run_net(gpu_mode, spec, {"data": x}, ["res5c"])
    p64 = net.get_blob("prob").data.copy()
    r64 = net.get_blob("res5c").data.copy()
    assert p64.shape == (64, 1000) and np.isfinite(p64).all()
    assert np.allclose(p64.sum(axis=1), 1, atol=1e-4)
    assert np.array_equal(p64[63], p64[5])
    rows = [0, 17, 63]
    oracle.use_openblas(True)
    try:
        want = netrun.oracle_forward(spec, {"data": x[rows]}, keep={"res5c", "prob"})
    finally:
        oracle.use_openblas(False)
    assert r64.shape == (64, 2048, 7, 7)
    for k, row in enumerate(rows):
        assert netrun.rel_err(r64[row], want["res5c"][k]) < 1e-3, row
        assert netrun.rel_err(p64[row], want["prob"][k]) < 1e-3, row
    net.forward(data=x[17:18])
    p1 = net.get_blob("prob").data.copy()
    assert np.abs(p1[0] - p64[17]).max() < 1e-6


def test_config4_rpn_proposal_full_size(gpu_mode):
    """RPN head + Proposal at the benchmark size (1x1024x38x63, 21 546 anchors ->
    top 6000 -> NMS 0.7 -> 300).  The dense part is compared within tolerance; the
    tail is compared bit for bit on identical tail inputs (the blobs the device
    produced), which is the only well-posed form of "same kept indices"."""
    from minicaffe import zoo
    oracle.use_openblas(True)
    try:
        spec, inputs = zoo.rpn_spec()
        net = run_net(gpu_mode, spec, inputs, ["rpn_cls_prob_reshape", "rpn_bbox_pred"])
        want = netrun.oracle_forward(spec[:-1], inputs)
    finally:
        oracle.use_openblas(False)
    prob = net.get_blob("rpn_cls_prob_reshape").data.copy()
    bbox = net.get_blob("rpn_bbox_pred").data.copy()
    # two stacked contractions, the first with K = 9216: summation-order noise alone
    # is above 1e-4 here, so the multi-layer tolerance applies
    assert netrun.rel_err(prob, want["rpn_cls_prob_reshape"]) < 1e-3
    assert netrun.rel_err(bbox, want["rpn_bbox_pred"]) < 1e-3
    rois = net.get_blob("rois").data.copy()
    (ref_rois,), kept, table = oracle.proposal(spec[-1]["proposal_param"], prob, bbox,
                                               inputs["im_info"], 1, details=True)
    assert rois.shape == ref_rois.shape and rois.shape[0] <= 300 and rois.shape[1] == 5
    assert np.array_equal(rois, ref_rois)
    # NMS invariants on the result itself: kept boxes are pairwise below the threshold
    b = rois[:, 1:]
    area = (b[:, 2] - b[:, 0] + 1) * (b[:, 3] - b[:, 1] + 1)
    for i in range(min(50, len(b))):
        xx1, yy1 = np.maximum(b[i, 0], b[:, 0]), np.maximum(b[i, 1], b[:, 1])
        xx2, yy2 = np.minimum(b[i, 2], b[:, 2]), np.minimum(b[i, 3], b[:, 3])
        inter = np.maximum(0, xx2 - xx1 + 1) * np.maximum(0, yy2 - yy1 + 1)
        iou = inter / (area[i] + area - inter)
        iou[i] = 0
        assert iou.max() <= 0.7 + 1e-6


def test_proposal_layer_with_score_ties_and_two_tops(gpu_mode):
    """Quantised scores force ties inside the top-N prefix: the device must replay
    the reference's quicksort order.  Also the optional second top (scores)."""
    from minicaffe.craft import input_layer
    rng = np.random.default_rng(5)
    A, H, W = 9, 14, 17
    spec = [input_layer({"prob": (1, 2 * A, H, W), "bbox": (1, 4 * A, H, W), "im_info": (1, 3)}),
            {"name": "proposal", "type": "Proposal", "bottom": ["prob", "bbox", "im_info"],
             "top": ["rois", "scores"],
             "proposal_param": {"pre_nms_topn": 1500, "post_nms_topn": 80, "nms_thresh": 0.6,
                                "min_size": 24}}]
    prob = (np.round(rng.random((1, 2 * A, H, W)) * 40) / 40).astype(np.float32)
    bbox = (rng.standard_normal((1, 4 * A, H, W)) * 0.4).astype(np.float32)
    inputs = {"prob": prob, "bbox": bbox, "im_info": np.array([[H * 16, W * 16, 1.5]], np.float32)}
    net = run_net(gpu_mode, spec, inputs)
    ref = oracle.proposal(spec[1]["proposal_param"], prob, bbox, inputs["im_info"], 2)
    assert np.array_equal(net.get_blob("rois").data, ref[0])
    assert np.array_equal(net.get_blob("scores").data, ref[1])


@pytest.mark.parametrize("use_global_stats", [False, True])
def test_config5_dcgan_generator_full_size(gpu_mode, use_global_stats):
    """DCGAN generator at batch 128: InnerProduct, Reshape, three stride-2
    Deconvolutions with BatchNorm (batch statistics as in the reference's WGAN
    graph, and stored statistics) + Scale + ReLU, Deconvolution + TanH."""
    from minicaffe import zoo
    oracle.use_openblas(True)
    try:
        spec, inputs = zoo.dcgan_spec(batch=128, use_global_stats=use_global_stats)
        net = run_net(gpu_mode, spec, inputs, ["g0", "gconv1", "gconv3"])
        want = netrun.oracle_forward(spec, inputs, keep={"g0", "gconv1", "gconv3", "gconv4"})
    finally:
        oracle.use_openblas(False)
    for name in ("g0", "gconv1", "gconv3", "gconv4"):
        got = net.get_blob(name).data
        assert got.shape == want[name].shape
        assert netrun.rel_err(got, want[name]) < 1e-3, name
    out = net.get_blob("gconv4").data
    assert out.shape == (128, 3, 64, 64) and np.abs(out).max() <= 1.0


def _check_ssd_tail(net, spec):
    """DetectionOutput rows of the device against the oracle run on the device's own
    mbox_loc / softmaxed confidences / priors: must be identical."""
    loc = net.get_blob("mbox_loc").data.copy()
    conf = net.get_blob("mbox_conf_flatten").data.copy()
    prior = net.get_blob("mbox_priorbox").data.copy()
    want = oracle.detection_output(spec[-1]["detection_output_param"], loc, conf, prior)
    got = net.get_blob("detection_out").data.copy()
    assert got.shape == want.shape
    assert np.array_equal(got, want)
    # the one order the reference leaves undefined (equal scores on both sides of the
    # keep_top_k cut) does not occur in these inputs: the kernel-level call says so
    from minicaffe import kernels
    from test_kernels_gpu import run_detection_output
    p = dict(spec[-1]["detection_output_param"])
    p["code_type"] = str(p.get("code_type", "CORNER"))
    rows, cut_tie = run_detection_output(kernels, p, loc, conf, prior)
    assert not (cut_tie & 1) and np.array_equal(rows, want)
    return got


def test_config3_ssd_small_width_every_stage(gpu_mode):
    """The SSD300 graph (all 102 layers, 300x300 input, 8732 priors) at 1/4 width so
    the CPU oracle can walk all of it: dilated fc6, Normalize, Permute / Flatten /
    Concat, PriorBox, Reshape + Softmax(axis 2), DetectionOutput."""
    from minicaffe import zoo
    oracle.use_openblas(True)
    try:
        spec, inputs = zoo.ssd300_spec(batch=2, width=16)
        marks = ["conv4_3_norm", "fc7", "conv9_2", "mbox_loc", "mbox_conf", "mbox_conf_flatten",
                 "mbox_priorbox"]
        net = run_net(gpu_mode, spec, inputs, marks)
        want = netrun.oracle_forward(spec[:-1], inputs, keep=set(marks))
    finally:
        oracle.use_openblas(False)
    assert np.array_equal(net.get_blob("mbox_priorbox").data, want["mbox_priorbox"])
    assert want["mbox_priorbox"].shape == (1, 2, 8732 * 4)
    for name in marks[:-1]:
        assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-3, name
    rows = _check_ssd_tail(net, spec)
    assert rows.shape[1] == 7 and rows.shape[0] <= 2 * 200


def test_config3_ssd_full_size_b8(gpu_mode):
    """Benchmark size (VGG16 widths, batch 8): the dense part of image 0 (Normalize,
    fc7, the last extra layer and the concatenated heads before and after the softmax)
    against the oracle walking that image at full width, the tail bit for bit on all
    8 images."""
    from minicaffe import zoo
    spec, inputs = zoo.ssd300_spec(batch=8)
    dense = ["conv4_3_norm", "fc7", "conv9_2", "mbox_loc", "mbox_conf", "mbox_conf_flatten"]
    net = run_net(gpu_mode, spec, inputs, dense + ["mbox_priorbox"])
    rows = _check_ssd_tail(net, spec)
    assert set(np.unique(rows[:, 0]).astype(int)) <= set(range(8))
    counts = np.bincount(rows[:, 0].astype(int), minlength=8)
    assert counts.max() <= 200
    # labels ascending within an image, scores descending within a label
    for i in range(8):
        r = rows[rows[:, 0] == i]
        assert (np.diff(r[:, 1]) >= 0).all()
        for lab in np.unique(r[:, 1]):
            assert (np.diff(r[r[:, 1] == lab][:, 2]) <= 0).all()
    oracle.use_openblas(True)
    try:
        want = netrun.oracle_forward(spec[:-1], {"data": inputs["data"][:1]},
                                     keep=set(dense + ["mbox_priorbox"]))
    finally:
        oracle.use_openblas(False)
    assert np.array_equal(net.get_blob("mbox_priorbox").data, want["mbox_priorbox"])
    for name in dense:
        got = net.get_blob(name).data[:1].copy()
        assert got.shape == want[name].shape, name
        assert netrun.rel_err(got, want[name]) < 1e-3, name


def test_rfcn_second_stage_on_proposal_rois(gpu_mode):
    """Config 4 continued into a detector head: the rois of Proposal feed a
    position-sensitive pooling branch (R-FCN: 1x1 conv -> PSROIPooling -> global
    average) and a ROIPooling branch.  Tops keep post_nms_topn rows with the
    reference's fill in the rows past the kept count."""
    import minicaffe as mc
    from minicaffe import zoo
    from minicaffe.craft import Enum
    spec, inputs = zoo.rpn_spec(seed=3, feat_shape=(1, 64, 20, 30), im_info=(320.0, 480.0, 1.0), mid=32,
                                post_nms_topn=50, nms_thresh=0.5)
    dim, g = 5, 3
    spec += [zoo.conv_layer("rfcn_cls", "feat", "rfcn_cls", 64, dim * g * g, 1, seed=4, std=0.05),
             {"name": "psroipooled_cls_rois", "type": "PSROIPooling", "bottom": ["rfcn_cls", "rois"],
              "top": ["psroipooled_cls_rois"],
              "psroi_pooling_param": {"spatial_scale": 0.0625, "output_dim": dim, "group_size": g}},
             {"name": "ave_cls_score_rois", "type": "Pooling", "bottom": ["psroipooled_cls_rois"],
              "top": ["cls_score"], "pooling_param": {"pool": Enum("AVE"), "kernel_size": g, "stride": g}},
             {"name": "roi_pool", "type": "ROIPooling", "bottom": ["feat", "rois"], "top": ["roi_pool"],
              "roi_pooling_param": {"pooled_h": 4, "pooled_w": 4, "spatial_scale": 0.0625}}]
    marks = ("rpn_cls_prob_reshape", "rpn_bbox_pred", "rfcn_cls", "rois", "psroipooled_cls_rois", "cls_score",
             "roi_pool")
    net = run_net(mc, spec, inputs, marks)
    # the dense part within tolerance ...
    dense = netrun.oracle_forward([l for l in spec if l["type"] not in ("Proposal", "PSROIPooling", "ROIPooling")
                                   and l["name"] != "ave_cls_score_rois"], inputs)
    for name in ("rpn_cls_prob_reshape", "rpn_bbox_pred", "rfcn_cls"):
        assert netrun.rel_err(net.get_blob(name).data, dense[name]) < 1e-3
    # ... the tail bit for bit on the blobs the device produced
    tail_in = {name: net.get_blob(name).data.copy() for name in ("rpn_cls_prob_reshape", "rpn_bbox_pred", "rfcn_cls")}
    tail_in.update(feat=inputs["feat"], im_info=inputs["im_info"])
    tail = [{"name": "in", "type": "Input", "top": list(tail_in)}] + \
           [l for l in spec if l["type"] in ("Proposal", "PSROIPooling", "ROIPooling") or l["name"] == "ave_cls_score_rois"]
    want = netrun.oracle_forward(tail, tail_in)
    rois = net.get_blob("rois").data
    r = rois.shape[0]
    assert np.array_equal(rois, want["rois"]) and 0 < r <= 50
    ps = net.get_blob("psroipooled_cls_rois").data
    assert ps.shape == (50, dim, g, g) == want["psroipooled_cls_rois"].shape
    assert np.array_equal(ps, want["psroipooled_cls_rois"])        # same sums in the same order
    if r < 50:
        assert np.array_equal(ps[r:], np.zeros_like(ps[r:]))       # rows past the kept count
    rp = net.get_blob("roi_pool").data
    assert rp.shape == (50, 64, 4, 4) and np.array_equal(rp, want["roi_pool"])
    assert netrun.rel_err(net.get_blob("cls_score").data, want["cls_score"]) < 1e-5


def test_zoo_layers_in_a_net(gpu_mode):
    """The less common layer types wired into one graph, every top compared with the
    CPU oracle walking the same layers: a MobileNet-style block (ConvolutionDepthwise
    -> BN -> PReLU, the BN folded into the convolution's epilogue), AlexNet-style
    LRN + Dropout, and the rest of the registry as side branches."""
    from minicaffe.craft import Enum, input_layer
    rng = np.random.default_rng(11)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    C = 8
    spec = [
        input_layer({"data": (2, C, 12, 10), "ref": (2, C, 7, 6), "words": (2, 5)}),
        {"name": "dw", "type": "ConvolutionDepthwise", "bottom": ["data"], "top": ["dw"],
         "convolution_param": {"num_output": C, "kernel_size": 3, "pad": 1, "bias_term": False},
         "blobs": [f(C, 1, 3, 3) * 0.3]},
        {"name": "dw_bn", "type": "BN", "bottom": ["dw"], "top": ["dw"],
         "blobs": [f(1, C), f(1, C), f(1, C) * 0.1, (rng.random((1, C)) + 0.5).astype(np.float32)]},
        {"name": "dw_prelu", "type": "PReLU", "bottom": ["dw"], "top": ["dw"], "blobs": [f(C) * 0.3]},
        {"name": "pw", "type": "Convolution", "bottom": ["dw"], "top": ["pw"],
         "convolution_param": {"num_output": 12, "kernel_size": 1}, "blobs": [f(12, C, 1, 1) * 0.3, f(12)]},
        {"name": "pw_elu", "type": "ELU", "bottom": ["pw"], "top": ["pw"], "elu_param": {"alpha": 0.7}},
        {"name": "shuf", "type": "ShuffleChannel", "bottom": ["pw"], "top": ["shuf"],
         "shuffle_channel_param": {"group": 3}},
        {"name": "lrn", "type": "LRN", "bottom": ["shuf"], "top": ["lrn"],
         "lrn_param": {"local_size": 5, "alpha": 1e-2, "beta": 0.75, "k": 2.0}},
        {"name": "drop", "type": "Dropout", "bottom": ["lrn"], "top": ["lrn"], "dropout_param": {"dropout_ratio": 0.5}},
        {"name": "lrn_w", "type": "LRN", "bottom": ["lrn"], "top": ["lrn_w"],
         "lrn_param": {"local_size": 3, "alpha": 0.5, "norm_region": Enum("WITHIN_CHANNEL")}},
        {"name": "bn_alone", "type": "BN", "bottom": ["lrn_w"], "top": ["bn_alone"],
         "blobs": [f(1, 12), f(1, 12), f(1, 12) * 0.1, (rng.random((1, 12)) + 0.5).astype(np.float32)]},
        {"name": "crop", "type": "Crop", "bottom": ["bn_alone", "ref"], "top": ["crop"],
         "crop_param": {"axis": 2, "offset": [3, 2]}},
        {"name": "mvn", "type": "MVN", "bottom": ["crop"], "top": ["mvn"], "mvn_param": {"eps": 1e-3}},
        {"name": "abs", "type": "AbsVal", "bottom": ["mvn"], "top": ["abs"]},
        {"name": "pow", "type": "Power", "bottom": ["abs"], "top": ["pow"],
         "power_param": {"power": 0.5, "scale": 2.0, "shift": 0.25}},
        {"name": "log", "type": "Log", "bottom": ["pow"], "top": ["log"], "log_param": {"base": 2.0, "shift": 1.0}},
        {"name": "exp", "type": "Exp", "bottom": ["log"], "top": ["exp"], "exp_param": {"scale": -0.5}},
        {"name": "bnll", "type": "BNLL", "bottom": ["mvn"], "top": ["bnll"]},
        {"name": "thr", "type": "Threshold", "bottom": ["mvn"], "top": ["thr"],
         "threshold_param": {"threshold": 0.1}},
        {"name": "tile", "type": "Tile", "bottom": ["exp"], "top": ["tile"], "tile_param": {"axis": 1, "tiles": 2}},
        {"name": "spp", "type": "SPP", "bottom": ["data"], "top": ["spp"], "spp_param": {"pyramid_height": 2}},
        {"name": "red", "type": "Reduction", "bottom": ["spp"], "top": ["red"],
         "reduction_param": {"operation": Enum("SUMSQ"), "axis": 1, "coeff": 0.1}},
        {"name": "am", "type": "ArgMax", "bottom": ["bnll"], "top": ["am"], "argmax_param": {"axis": 1, "top_k": 2}},
        {"name": "am_flat", "type": "ArgMax", "bottom": ["spp"], "top": ["am_flat"],
         "argmax_param": {"top_k": 3, "out_max_val": True}},
        {"name": "emb", "type": "Embed", "bottom": ["words"], "top": ["emb"],
         "embed_param": {"num_output": 4, "input_dim": 9}, "blobs": [f(9, 4), f(4)]},
        {"name": "par", "type": "Parameter", "top": ["par"], "parameter_param": {"shape": {"dim": [2, 3]}},
         "blobs": [f(2, 3)]},
    ]
    inputs = {"data": f(2, C, 12, 10), "ref": np.zeros((2, C, 7, 6), np.float32),
              "words": rng.integers(0, 9, (2, 5)).astype(np.float32)}
    marks = ["dw", "pw", "shuf", "lrn", "lrn_w", "bn_alone", "crop", "mvn", "abs", "pow", "log", "exp",
             "bnll", "thr", "tile", "spp", "red", "am", "am_flat", "emb", "par"]
    net = run_net(gpu_mode, spec, inputs, marks)
    # device-produced inputs for the index-valued tops, so that "same indices" is well posed
    bnll_dev = net.get_blob("bnll").data.copy()
    spp_dev = net.get_blob("spp").data.copy()
    want = netrun.oracle_forward(spec, inputs)
    for name in marks:
        got = net.get_blob(name).data
        assert tuple(got.shape) == want[name].shape, name
        if name in ("am", "am_flat", "thr"):
            continue
        # MVN subtracts a mean several times the spread it keeps: from there on the
        # deep-net tolerance applies
        deep = name in ("mvn", "abs", "pow", "log", "exp", "bnll", "tile")
        assert netrun.rel_err(got, want[name]) < (1e-3 if deep else 1e-4), name
    assert np.array_equal(net.get_blob("am").data, oracle.argmax(bnll_dev, 2, False, 1))
    assert np.array_equal(net.get_blob("am_flat").data, oracle.argmax(spp_dev, 3, True))
    assert np.array_equal(net.get_blob("thr").data, oracle.threshold(net.get_blob("mvn").data, 0.1))
    assert np.array_equal(net.get_blob("spp").data, want["spp"])      # max pooling moves values
    assert np.array_equal(net.get_blob("emb").data, want["emb"])
    assert np.array_equal(net.get_blob("par").data, spec[-1]["blobs"][0])
    # a second forward with another batch size re-plans every layer
    x3 = f(3, C, 12, 10)
    in3 = {"data": x3, "ref": np.zeros((3, C, 7, 6), np.float32),
           "words": rng.integers(0, 9, (3, 5)).astype(np.float32)}
    net.forward(**in3)
    want3 = netrun.oracle_forward(spec, in3)
    for name in ("tile", "red", "bn_alone", "emb"):
        assert netrun.rel_err(net.get_blob(name).data, want3[name]) < 1e-4, name


def test_filter_layer_selects_items_at_reshape(gpu_mode):
    """Filter reads its selector when the net is reshaped (filter_layer.cpp:19-59): the
    selector is an input written before Forward(reshape=True), as a caller of the
    reference has to do."""
    from minicaffe.craft import input_layer
    rng = np.random.default_rng(12)
    spec = [input_layer({"a": (5, 3, 4), "b": (5, 2), "sel": (5,)}),
            {"name": "flt", "type": "Filter", "bottom": ["a", "b", "sel"], "top": ["fa", "fb"]}]
    a, b = rng.standard_normal((5, 3, 4)).astype(np.float32), rng.standard_normal((5, 2)).astype(np.float32)
    sel = np.array([0, 1, 0, 2, 1], np.float32)
    net = run_net(gpu_mode, spec, {"a": a, "b": b, "sel": sel})
    keep = sel != 0
    assert np.array_equal(net.get_blob("fa").data, a[keep])
    assert np.array_equal(net.get_blob("fb").data, b[keep])
    net.forward(a=a, b=b, sel=np.zeros(5, np.float32))
    assert tuple(net.get_blob("fa").shape) == (0, 3, 4)


@pytest.mark.parametrize("depthwise_type", [False, True])
def test_mobilenet_ssd_full_size(gpu_mode, depthwise_type):
    """MobileNet-SSD at its real size (300x300, 47 convolutions of which 13 depthwise,
    1917 priors), the graph of the reference's ssd example with seeded weights: the
    dense part against the oracle, the DetectionOutput rows bit for bit on the device's
    own tail inputs.  The confidence heads are sharpened so that detections pass the
    0.25 threshold.  Both spellings of the depthwise layers give the same numbers."""
    from minicaffe import zoo
    spec, inputs = zoo.mobilenet_ssd_spec(batch=2, depthwise_type=depthwise_type)
    for layer in spec:
        if layer["name"].endswith("_mbox_conf"):
            layer["blobs"][0] = layer["blobs"][0] * 6
    marks = ["conv1/dw", "conv6", "conv13", "conv17_2", "mbox_loc", "mbox_conf_flatten", "mbox_priorbox"]
    net = run_net(gpu_mode, spec, inputs, marks)
    oracle.use_openblas(True)
    try:
        want = netrun.oracle_forward(spec[:-1], inputs, keep=set(marks))
    finally:
        oracle.use_openblas(False)
    assert np.array_equal(net.get_blob("mbox_priorbox").data, want["mbox_priorbox"])
    for name in marks[:-1]:
        assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-3, name
    rows = _check_ssd_tail(net, spec)
    assert rows.shape == (200, 7) and (rows[:, 2] >= 0.25).all()


def test_ssh_context_module_upsample_crop_and_two_top_proposal(gpu_mode):
    """The motif of the reference's ssh example (example/models/ssh/test_ssh.prototxt):
    1x1 reduction of the stride-16 map, bilinear 2x upsampling by a Deconvolution with
    group == channels, Crop to the stride-8 map, Eltwise SUM, 3x3 convolutions, 2-anchor
    score / box heads, Reshape -> Softmax -> Reshape, and a Proposal with two tops
    (boxes and their scores).  Dense blobs within tolerance; the Proposal tops bit for
    bit on the device's own score / box blobs."""
    from minicaffe import zoo
    from minicaffe.craft import Enum, input_layer
    C, R, A = 24, 16, 2
    h8, w8 = 37, 50                      # stride-8 map; the stride-16 map is 19 x 25
    h16, w16 = (h8 + 1) // 2, (w8 + 1) // 2
    # bilinear upsampling filter (factor 2, kernel 4), one per channel
    f = np.array([0.25, 0.75, 0.75, 0.25], np.float32)
    up = np.tile(np.outer(f, f).reshape(1, 1, 4, 4), (R, 1, 1, 1))
    spec = [input_layer({"conv4_3": (1, C, h8, w8), "conv5_3": (1, C, h16, w16), "im_info": (1, 3)}),
            zoo.conv_layer("conv5_128", "conv5_3", "conv5_128", C, R, 1, seed=1),
            zoo.relu_layer("conv5_128_relu", "conv5_128"),
            {"name": "conv5_128_up", "type": "Deconvolution", "bottom": ["conv5_128"], "top": ["conv5_128_up"],
             "convolution_param": {"kernel_size": 4, "stride": 2, "num_output": R, "group": R, "pad": 1,
                                   "bias_term": False}, "blobs": [up]},
            zoo.conv_layer("conv4_128", "conv4_3", "conv4_128", C, R, 1, seed=2),
            zoo.relu_layer("conv4_128_relu", "conv4_128"),
            {"name": "conv5_128_crop", "type": "Crop", "bottom": ["conv5_128_up", "conv4_128"],
             "top": ["conv5_128_crop"], "crop_param": {"axis": 2, "offset": 0}},
            {"name": "conv4_fuse", "type": "Eltwise", "bottom": ["conv5_128_crop", "conv4_128"],
             "top": ["conv4_fuse"], "eltwise_param": {"operation": Enum("SUM")}},
            zoo.conv_layer("conv4_fuse_final", "conv4_fuse", "conv4_fuse_final", R, R, 3, pad=1, seed=3),
            zoo.relu_layer("conv4_fuse_final_relu", "conv4_fuse_final"),
            zoo.conv_layer("m1@ssh_3x3", "conv4_fuse_final", "m1@ssh_3x3_output", R, R, 3, pad=1, seed=4),
            zoo.conv_layer("m1@ssh_dimred", "conv4_fuse_final", "m1@ssh_dimred_output", R, R // 2, 3, pad=1, seed=5),
            zoo.relu_layer("m1@ssh_dimred_relu", "m1@ssh_dimred_output"),
            zoo.conv_layer("m1@ssh_5x5", "m1@ssh_dimred_output", "m1@ssh_5x5_output", R // 2, R // 2, 3, pad=1, seed=6),
            {"name": "m1@ssh_output", "type": "Concat", "bottom": ["m1@ssh_3x3_output", "m1@ssh_5x5_output"],
             "top": ["m1@ssh_output"], "concat_param": {"axis": 1}},
            zoo.relu_layer("m1@ssh_output_relu", "m1@ssh_output"),
            zoo.conv_layer("m1@ssh_cls_score", "m1@ssh_output", "m1@ssh_cls_score_output", R + R // 2, 2 * A, 1,
                           seed=7, std=0.3),
            zoo.conv_layer("m1@ssh_bbox_pred", "m1@ssh_output", "m1@ssh_bbox_pred_output", R + R // 2, 4 * A, 1,
                           seed=8, std=0.02),
            {"name": "m1@ssh_cls_reshape", "type": "Reshape", "bottom": ["m1@ssh_cls_score_output"],
             "top": ["m1@ssh_cls_score_reshape_output"], "reshape_param": {"shape": {"dim": [0, 2, -1, 0]}}},
            {"name": "m1@ssh_cls_prob", "type": "Softmax", "bottom": ["m1@ssh_cls_score_reshape_output"],
             "top": ["m1@ssh_cls_prob_output"]},
            {"name": "m1@ssh_cls_prob_reshape", "type": "Reshape", "bottom": ["m1@ssh_cls_prob_output"],
             "top": ["m1@ssh_cls_prob_reshape_output"], "reshape_param": {"shape": {"dim": [0, 2 * A, -1, 0]}}},
            {"name": "m1@ssh_proposal", "type": "Proposal",
             "bottom": ["m1@ssh_cls_prob_reshape_output", "m1@ssh_bbox_pred_output", "im_info"],
             "top": ["m1@ssh_boxes", "m1@ssh_cls_prob"],
             "proposal_param": {"feat_stride": 8, "scale": [1.0, 2.0], "ratio": [1.0], "min_size": 4,
                                "nms_thresh": 0.3}}]
    rng = np.random.default_rng(21)
    inputs = {"conv4_3": rng.standard_normal((1, C, h8, w8)).astype(np.float32),
              "conv5_3": rng.standard_normal((1, C, h16, w16)).astype(np.float32),
              "im_info": np.array([[h8 * 8.0, w8 * 8.0, 1.0]], np.float32)}
    marks = ["conv5_128_up", "conv5_128_crop", "conv4_fuse", "m1@ssh_output",
             "m1@ssh_cls_prob_reshape_output", "m1@ssh_bbox_pred_output"]
    net = run_net(gpu_mode, spec, inputs, marks)
    want = netrun.oracle_forward(spec[:-1], inputs)
    assert want["conv5_128_up"].shape == (1, R, 2 * h16, 2 * w16) and want["conv5_128_crop"].shape == (1, R, h8, w8)
    for name in marks:
        assert netrun.rel_err(net.get_blob(name).data, want[name]) < 1e-3, name
    scores = net.get_blob("m1@ssh_cls_prob_reshape_output").data.copy()
    boxes = net.get_blob("m1@ssh_bbox_pred_output").data.copy()
    rois, probs = oracle.proposal(spec[-1]["proposal_param"], scores, boxes, inputs["im_info"], 2)
    n = rois.shape[0]
    assert 10 < n <= 300
    assert np.array_equal(net.get_blob("m1@ssh_boxes").data[:n], rois)
    assert np.array_equal(net.get_blob("m1@ssh_cls_prob").data.reshape(-1)[:n], probs)


def test_benchmark_tool_runs_a_prototxt(gpu_mode, tmp_path):
    """tools/benchmark.cpp of the reference, rebuilt here: net from the prototxt alone,
    N timed passes, layer scopes in ./profile.json."""
    import json
    import os
    import subprocess
    from minicaffe import craft, zoo
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "mini-caffe_amd", "bin", "benchmark")
    spec, _ = zoo.resnet50_spec(batch=2, size=64, stages=(1, 1, 1, 1), width=16, num_classes=10)
    proto = tmp_path / "net.prototxt"
    proto.write_text(craft.to_prototxt(spec))
    r = subprocess.run([exe, str(proto), "3", "0"], capture_output=True, text=True, cwd=tmp_path, timeout=100)
    out = r.stdout + r.stderr
    assert r.returncode == 0, out
    assert out.count("Forward costs") == 3 and "run on device 0" in out
    events = json.load(open(tmp_path / "profile.json"))["traceEvents"]
    names = {e["name"] for e in events}
    assert {"conv1", "pool1", "fc1000", "prob"} <= names


def test_c_program_through_the_c_abi(gpu_mode, tmp_path):
    """A C99 program (csrc/tools/run_net_c.c, the counterpart of the reference's
    tests/run_net.c) creates a net from files and from buffers, fills the input, runs it
    and lists blobs; the sum it prints for the last blob equals the oracle's."""
    import os
    import re
    import subprocess
    import wire
    from minicaffe import craft, zoo
    oracle.use_openblas(False)
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "mini-caffe_amd", "bin", "run_net_c")
    spec, _ = zoo.resnet50_spec(batch=2, size=40, stages=(1, 1, 1, 1), width=8, num_classes=6, bn_seed=9)
    (tmp_path / "n.prototxt").write_text(craft.to_prototxt(spec))
    (tmp_path / "n.caffemodel").write_bytes(wire.net("m", [
        wire.layer(l["name"], l["type"], l["blobs"]) for l in spec if l.get("blobs")]))
    r = subprocess.run([exe, str(tmp_path / "n.prototxt"), str(tmp_path / "n.caffemodel")],
                       capture_output=True, text=True, cwd=tmp_path, timeout=100)
    out = r.stdout + r.stderr
    assert r.returncode == 0 and "run_net_c: ok" in out, out
    assert "data: 4 axes, [2, 3, 40, 40], 9600 values" in out
    assert "expected error:" in out and "prob: [2, 6, 1, 1]" in out
    # the program's deterministic input, through the oracle
    i = np.arange(9600)
    x = ((i * 37 % 101) / 50.0 - 1.0).astype(np.float32).reshape(2, 3, 40, 40)
    want = netrun.oracle_forward(spec, {"data": x})["prob"]
    m = re.search(r"sum of the last blob: ([-0-9.e]+), first value: ([-0-9.e]+)", out)
    assert abs(float(m.group(1)) - float(want.sum())) < 1e-4
    assert abs(float(m.group(2)) - float(want.flat[0])) < 1e-4 * float(want.max())


def test_trained_landmark_net_from_the_golden_caffemodel(gpu_mode):
    """Real trained weights (tests/golden, from the reference's deeplandmark example) through
    CaffeNetCreateFromBuffer; forward at batch 1, as the reference's example calls it, and at
    batch 6 after a reshape, against the oracle on the same weights."""
    import os
    import wire
    from minicaffe import craft
    from test_host_api import landmark_level2_spec
    oracle.use_openblas(False)
    here = os.path.dirname(os.path.abspath(__file__))
    model = open(os.path.join(here, "golden", "deeplandmark_2_LE1.caffemodel"), "rb").read()
    weights = wire.read_net_blobs(model)
    rng = np.random.default_rng(31)
    net = gpu_mode.Net.from_buffers(craft.to_prototxt(landmark_level2_spec()), model)
    for name in ("pool1", "pool2", "fc1"):
        net.mark_output(name)
    for batch in (1, 6, 1):
        spec = landmark_level2_spec(batch)
        for layer in spec:
            if layer["name"] in weights:
                layer["blobs"] = weights[layer["name"]]
        x = rng.uniform(-1, 1, (batch, 1, 15, 15)).astype(np.float32)
        net.forward(data=x)
        want = netrun.oracle_forward(spec, {"data": x})
        for name in ("pool1", "pool2", "fc1", "fc2"):
            got = net.get_blob(name).data
            assert got.shape == want[name].shape, name
            assert netrun.rel_err(got, want[name]) < 1e-4, (batch, name)
        assert np.abs(want["fc2"]).max() > 1e-3   # the trained net answers with something
