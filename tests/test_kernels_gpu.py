"""Kernel-level parity on the MI355X: every entry point of include/mchip/kernels.h is
called through the C ABI with device pointers (torch only owns the memory) and
compared with the CPU oracle on the same seeded inputs.

Tolerances: the dense contraction differs from the oracle only by fp32 summation
order (see netrun.rel_err): 1e-4.  Pure data movement (pooling MAX, copy,
permute, concat) must be bit-exact.
"""
import ctypes

import numpy as np
import pytest

import oracle
from oracle import netrun

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")


@pytest.fixture(scope="module")
def K(gpu_mode):
    from minicaffe import kernels
    oracle.use_openblas(False)
    return kernels


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def fptr(t):
    return ctypes.c_void_p(t.data_ptr())


K_ACT_NONE, K_ACT_RELU, K_ACT_TANH = 0, 1, 2

CONV_CASES = [
    # cin, h, w, cout, k, s, p, d, g, transposed, batch
    (64, 56, 56, 64, 3, 1, 1, 1, 1, False, 1),      # config 1
    (3, 33, 31, 64, 7, 2, 3, 1, 1, False, 2),       # ResNet conv1 geometry, odd extents
    (64, 14, 14, 256, 1, 1, 0, 1, 1, False, 3),     # 1x1
    (256, 14, 14, 128, 1, 2, 0, 1, 1, False, 2),    # strided 1x1
    (32, 19, 19, 64, 3, 1, 6, 6, 1, False, 2),      # dilated (SSD fc6 geometry)
    (32, 20, 20, 64, 3, 1, 1, 1, 4, False, 2),      # groups
    (8, 9, 11, 8, (3, 2), (2, 1), (1, 0), 1, 8, False, 2),   # depthwise, non-square
    (16, 5, 5, 24, 3, 1, 1, 1, 1, False, 2),        # odd M (SSD head)
    (100, 1, 1, 1000, 1, 1, 0, 1, 1, False, 7),     # inner-product shape
    (40, 10, 10, 130, 3, 2, 1, 1, 1, False, 2),     # M and K not multiples of the tile
    (1024, 4, 4, 512, 4, 2, 1, 1, 1, True, 2),      # DCGAN deconv 4 -> 8
    (16, 5, 7, 3, 4, 2, 1, 1, 1, True, 3),          # deconv to 3 channels
    (8, 6, 6, 8, 3, 1, 1, 1, 1, True, 2),           # stride-1 deconv
    (8, 6, 6, 12, 2, 3, 0, 1, 1, True, 2),          # kernel < stride: tapless output classes
    (8, 6, 6, 12, 5, 2, 2, 1, 2, True, 2),          # grouped deconv
    (8, 6, 6, 12, 3, 2, 1, 2, 1, True, 2),          # dilated deconv
    (32, 28, 28, 32, 3, 1, 1, 1, 32, False, 3),     # depthwise 3x3 (MobileNet): direct kernel
    (32, 29, 27, 32, 3, 2, 1, 1, 32, False, 2),     # depthwise, stride 2, odd extents
    (16, 12, 12, 32, 5, 1, 2, 1, 16, False, 2),     # depthwise 5x5 with channel multiplier 2
    (16, 12, 12, 16, 3, 1, 2, 2, 16, False, 2),     # depthwise, dilated
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("cfg", [-1, 0, 3, 5])
def test_conv_forward(K, case, cfg):
    cin, h, w, cout, k, s, p, d, g, tr, n = case
    rng = np.random.default_rng(1)
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    kk = (k, k) if isinstance(k, int) else k
    wshape = (cin, cout // g) + kk if tr else (cout, cin // g) + kk
    wt = (rng.standard_normal(wshape) * 0.1).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    want = oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, k, s, p, d, g, tr), x, wt, b)
    plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, k, s, p, d, g, tr))
    plan.force_config(cfg)
    assert plan.output_shape() == want.shape[2:]
    xd, wd, bd = dev(x), dev(wt), dev(b)
    yd = torch.full(want.shape, float("nan"), device="cuda")
    plan.set_weights(wd.data_ptr())
    plan.forward(n, xd.data_ptr(), yd.data_ptr(), shift=bd.data_ptr())
    torch.cuda.synchronize()
    assert netrun.rel_err(yd.cpu().numpy(), want) < 1e-4


@pytest.mark.parametrize("case", [
    # cin, h, w, cout, k, s, p, transposed, n, images per run
    (24, 13, 11, 40, 3, 1, 1, False, 8, 3),      # runs of 3, 3, 2 images
    (32, 9, 9, 70, 1, 1, 0, False, 7, 2),        # pointwise
    (16, 7, 6, 20, 4, 2, 1, True, 5, 2),         # deconvolution: four parity classes per run
    (24, 13, 11, 40, 3, 2, 1, False, 4, 1),      # one image per run
])
def test_conv_batch_cut_into_image_runs(K, case):
    """A batch the buffer descriptors cannot address in one launch is cut into runs of
    whole images (forced here with a small run length): every run must equal a call of
    its own on those images bit for bit, epilogue and residual rows included, and the
    whole result the oracle's."""
    cin, h, w, cout, k, st, p, tr, n, per = case
    rng = np.random.default_rng(51)
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cin, cout, k, k) if tr else (cout, cin, k, k)) * 0.1).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    sc = (rng.random(cout) + 0.5).astype(np.float32)
    geom = oracle.conv_geom(cin, h, w, cout, k, st, p, 1, 1, tr)
    raw = oracle.conv_forward(geom, x, wt, None)
    res = rng.standard_normal(raw.shape).astype(np.float32)
    want = np.maximum(raw * sc.reshape(1, -1, 1, 1) + b.reshape(1, -1, 1, 1) + res, 0)
    plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, k, st, p, 1, 1, tr))
    xd, wd, bd, sd, rd = dev(x), dev(wt), dev(b), dev(sc), dev(res)
    plan.set_weights(wd.data_ptr())
    ep = dict(scale=sd.data_ptr(), shift=bd.data_ptr(), activation=K_ACT_RELU)
    plan.force_chunk(per)
    cut = torch.full(raw.shape, float("nan"), device="cuda")
    plan.forward(n, xd.data_ptr(), cut.data_ptr(), residual=rd.data_ptr(), **ep)
    plan.force_chunk(0)
    runs = -(-n // per)
    run_len = -(-n // runs)
    parts = torch.full(raw.shape, float("nan"), device="cuda")
    for n0 in range(0, n, run_len):
        m = min(run_len, n - n0)
        plan.forward(m, xd[n0:].data_ptr(), parts[n0:].data_ptr(), residual=rd[n0:].data_ptr(), **ep)
    torch.cuda.synchronize()
    assert torch.equal(cut, parts)
    assert netrun.rel_err(cut.cpu().numpy(), want) < 1e-4
    if not tr:
        # two tops: each top advances by its own image size
        c_first = 13
        plan.force_chunk(per)
        first = torch.full((n, c_first) + raw.shape[2:], float("nan"), device="cuda")
        second = torch.full((n, cout - c_first) + raw.shape[2:], float("nan"), device="cuda")
        plan.forward_two_tops(n, xd.data_ptr(), first.data_ptr(), c_first, second.data_ptr(), **ep)
        torch.cuda.synchronize()
        both = torch.cat([first, second], 1).cpu().numpy()
        want2 = np.maximum(raw * sc.reshape(1, -1, 1, 1) + b.reshape(1, -1, 1, 1), 0)
        assert netrun.rel_err(both, want2) < 1e-4


def test_conv_blob_beyond_two_to_the_29_elements(K):
    """A 1x1 convolution whose bottom and top hold more than 2^29 elements each (the
    reference's per-image loop takes any size): the call cuts the batch itself, and
    every image equals the result of a small call on that image."""
    cin = cout = 64
    h = w = 56
    n = (1 << 29) // (cin * h * w) + 30          # 2705 images, 542.9M elements, 2.2 GB per blob
    assert n * cin * h * w > (1 << 29)
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.empty((n, cin, h, w), device="cuda").uniform_(-1, 1, generator=g)
    wt = (torch.randn((cout, cin, 1, 1), device="cuda", generator=g) * 0.1).contiguous()
    b = torch.randn(cout, device="cuda", generator=g)
    plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, 1, 1, 0))
    plan.set_weights(wt.data_ptr())
    y = torch.full((n, cout, h, w), float("nan"), device="cuda")
    plan.forward(n, x.data_ptr(), y.data_ptr(), shift=b.data_ptr(), activation=K_ACT_RELU)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(y).all())
    # the run length the library chose, and images on both sides of every cut
    per = ((1 << 29) - 1) // (cin * h * w)
    runs = -(-n // per)
    run_len = -(-n // runs)
    probe = sorted({0, 1, run_len - 1, run_len, run_len + 1, n - 2, n - 1})
    small = torch.empty((1, cout, h, w), device="cuda")
    for i in probe:
        plan.forward(1, x[i:].data_ptr(), small.data_ptr(), shift=b.data_ptr(), activation=K_ACT_RELU)
        torch.cuda.synchronize()
        assert netrun.rel_err(y[i].cpu().numpy(), small[0].cpu().numpy()) < 1e-5, i
    # and one image against the CPU oracle
    i = run_len
    want = np.maximum(oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, 1, 1, 0), x[i:i + 1].cpu().numpy(),
                                          wt.cpu().numpy(), b.cpu().numpy()), 0)
    assert netrun.rel_err(y[i:i + 1].cpu().numpy(), want) < 1e-4
    del x, y
    torch.cuda.empty_cache()


THIN_CASES = [
    (8, 96, 90, 3, 3, 1, 1, 1, 1, False, 8),        # 3x3 to 3 channels (one validity mask per tap pair)
    (16, 96, 90, 1, 1, 1, 0, 1, 1, False, 8),       # 1x1 score map: pointwise path
    (8, 40, 44, 3, 4, 2, 1, 1, 1, True, 10),        # generator's last layer: deconv 4x4/2 to RGB, 4 output classes
    (8, 64, 64, 8, 3, 2, 1, 1, 2, False, 33),       # two groups of 4 outputs, stride 2
    (3, 200, 180, 4, 7, 2, 3, 1, 1, False, 8),      # 7x7/2 from 3 channels (row and column masks)
    (4, 90, 100, 2, 3, 1, 2, 2, 1, False, 8),       # dilated
]


@pytest.mark.parametrize("case", THIN_CASES)
@pytest.mark.parametrize("act", [K_ACT_NONE, K_ACT_TANH])
def test_conv_few_output_channels(K, case, act):
    """At most 4 output channels per group over many pixels: the per-pixel kernel,
    with the whole epilogue, against the oracle's convolution + the same tail."""
    cin, h, w, cout, k, s, p, d, g, tr, n = case
    rng = np.random.default_rng(12)
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    wshape = (cin, cout // g, k, k) if tr else (cout, cin // g, k, k)
    wt = (rng.standard_normal(wshape) * 0.2).astype(np.float32)
    sc = (rng.random(cout) + 0.5).astype(np.float32)
    sh = rng.standard_normal(cout).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, k, s, p, d, g, tr), x, wt, None)
    res = rng.standard_normal(y.shape).astype(np.float32)
    want = y * sc[None, :, None, None] + sh[None, :, None, None] + res
    if act == K_ACT_TANH:
        want = np.tanh(want.astype(np.float64)).astype(np.float32)
    plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, k, s, p, d, g, tr))
    assert plan.kernel_name(n) == "thin_f32"
    xd, wd, scd, shd, rd = dev(x), dev(wt), dev(sc), dev(sh), dev(res)
    yd = torch.full(want.shape, float("nan"), device="cuda")
    plan.set_weights(wd.data_ptr())
    plan.forward(n, xd.data_ptr(), yd.data_ptr(), scale=scd.data_ptr(), shift=shd.data_ptr(),
                 residual=rd.data_ptr(), activation=act)
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    # tanh outputs near 0 carry the absolute error of sums of magnitude ~10: absolute bound there
    close = (lambda a, b: np.abs(a - b).max() < 1e-5) if act == K_ACT_TANH else \
        (lambda a, b: netrun.rel_err(a, b) < 1e-4)
    assert close(got, want)
    # the matrix-core kernel on the same problem agrees
    plan.force_config(4)
    y2 = torch.full(want.shape, float("nan"), device="cuda")
    plan.forward(n, xd.data_ptr(), y2.data_ptr(), scale=scd.data_ptr(), shift=shd.data_ptr(),
                 residual=rd.data_ptr(), activation=act)
    torch.cuda.synchronize()
    assert close(y2.cpu().numpy(), got)


@pytest.mark.parametrize("c_first", [8, 64, 100, 149])
@pytest.mark.parametrize("split", [1, 0, 3])
def test_conv_two_tops_equals_one_top_cut_in_two(K, split, c_first):
    """mcConvForwardTwoTops writes the same values as mcConvForward, channel ranges
    [0, c) and [c, C) each into a blob of its own (cuts inside the first, at the edge
    of and inside a later 32-row block, and one channel before the end): with the
    plan's own choice of K slices, with three forced slices, and with one requested
    (two tops always run as at least two slices, so that case is compared with the
    two-slice single-top result)."""
    n, cin, h, w, cout, k, c_first = 3, 48, 9, 7, 150, 3, c_first
    rng = np.random.default_rng(31)
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, cin, k, k)) * 0.1).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, k, 1, 1))
    xd, wd, bd = dev(x), dev(wt), dev(b)
    plan.set_weights(wd.data_ptr())
    whole = torch.full((n, cout, h, w), float("nan"), device="cuda")
    plan.force_split(max(split, 2) if split else 0)
    plan.forward(n, xd.data_ptr(), whole.data_ptr(), shift=bd.data_ptr(), activation=K_ACT_RELU)
    plan.force_split(split)
    first = torch.full((n, c_first, h, w), float("nan"), device="cuda")
    second = torch.full((n, cout - c_first, h, w), float("nan"), device="cuda")
    plan.forward_two_tops(n, xd.data_ptr(), first.data_ptr(), c_first, second.data_ptr(),
                          shift=bd.data_ptr(), activation=K_ACT_RELU)
    torch.cuda.synchronize()
    assert torch.equal(first, whole[:, :c_first]) and torch.equal(second, whole[:, c_first:])
    want = np.maximum(oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, k, 1, 1), x, wt, b), 0)
    assert netrun.rel_err(whole.cpu().numpy(), want) < 1e-4
    with pytest.raises(Exception, match="TwoTops"):
        plan.forward_two_tops(n, xd.data_ptr(), first.data_ptr(), cout, second.data_ptr())


def test_conv_epilogue_matches_unfused_chain(K):
    """scale/shift/residual/activation of the epilogue against Conv -> BatchNorm ->
    Scale -> (+residual) -> ReLU evaluated layer by layer on the oracle."""
    rng = np.random.default_rng(2)
    n, cin, cout, h = 2, 24, 40, 9
    x = rng.standard_normal((n, cin, h, h)).astype(np.float32)
    wt = (rng.standard_normal((cout, cin, 3, 3)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(cout).astype(np.float32)
    mean = rng.standard_normal(cout).astype(np.float32)
    var = (rng.random(cout) + 0.5).astype(np.float32)
    gamma = (rng.random(cout) + 0.5).astype(np.float32)
    beta = rng.standard_normal(cout).astype(np.float32)
    res = rng.standard_normal((n, cout, h, h)).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(cin, h, h, cout, 3, 1, 1), x, wt, bias)
    y = oracle.batch_norm(y, mean, var, np.ones(1, np.float32), True, 1e-5)
    y = oracle.scale(y, gamma, beta)
    want = oracle.relu(oracle.eltwise([y, res], "SUM"), 0.1)
    # fold BN + Scale on the device
    LIB = K.LIB
    meand, stdd = torch.empty(cout, device="cuda"), torch.empty(cout, device="cuda")
    b0, b1, b2 = dev(mean), dev(var), dev(np.ones(1, np.float32))   # keep the tensors alive
    K.check_mc(LIB.mcBatchNormStored(fptr(b0), fptr(b1), fptr(b2),
                                     ctypes.c_float(1e-5), cout, fptr(meand), fptr(stdd), None))
    gd, bd, biasd = dev(gamma), dev(beta), dev(bias)
    stages = (K.ChannelOp * 2)(K.ChannelOp(meand.data_ptr(), stdd.data_ptr(), None, None, 0, 0.0),
                               K.ChannelOp(None, None, gd.data_ptr(), bd.data_ptr(), 0, 0.0))
    sc, sh = torch.empty(cout, device="cuda"), torch.empty(cout, device="cuda")
    K.check_mc(LIB.mcFoldChannelOps(fptr(biasd), stages, 2, cout, fptr(sc), fptr(sh), None))
    plan = K.ConvPlan(K.conv_geom(cin, h, h, cout, 3, 1, 1))
    wd, xd, rd = dev(wt), dev(x), dev(res)
    yd = torch.empty(want.shape, device="cuda")
    plan.set_weights(wd.data_ptr())
    plan.forward(n, xd.data_ptr(), yd.data_ptr(), scale=sc.data_ptr(), shift=sh.data_ptr(),
                 residual=rd.data_ptr(), activation=K.ACT_RELU, negative_slope=0.1)
    torch.cuda.synchronize()
    assert netrun.rel_err(yd.cpu().numpy(), want) < 1e-4



def _run_plan(K, plan, n, x, wt, out_shape, **ep):
    xd, wd = dev(x), dev(wt)
    keep = {k: dev(v) for k, v in ep.items() if isinstance(v, np.ndarray)}
    args = {k: (keep[k].data_ptr() if k in keep else v) for k, v in ep.items()}
    yd = torch.full(out_shape, float("nan"), device="cuda")
    plan.set_weights(wd.data_ptr())
    plan.forward(n, xd.data_ptr(), yd.data_ptr(), **args)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


@pytest.mark.parametrize("case", [
    # cin, h, w, cout, stride, batch: 1x1 kernels without padding
    (64, 14, 14, 256, 1, 3), (256, 14, 14, 128, 2, 2), (100, 1, 1, 1000, 1, 7), (40, 9, 7, 24, 1, 2),
    (70, 5, 5, 64, 3, 2),
    # stride 1, plane a multiple of four pixels, channels a multiple of 16: four pixels per load;
    # tiles that straddle images (plane 20), a ragged last tile, then planes and channel counts
    # that rule the form out
    (32, 4, 5, 40, 1, 7), (48, 6, 6, 70, 1, 3), (16, 8, 8, 16, 1, 1), (32, 7, 7, 40, 1, 3), (24, 4, 4, 40, 1, 3)])
def test_conv_pointwise_path_equals_tap_table_path(K, case):
    """A 1x1 unpadded convolution takes a K loop without tap table (in two forms: one
    pixel of four channels, or four pixels of one channel per thread); pinned to the
    general loop (configuration + 100) it must give the same bits: all add the same
    products in the same order."""
    cin, h, w, cout, s, n = case
    rng = np.random.default_rng(3)
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, cin, 1, 1)) * 0.1).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    want = oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, 1, s, 0), x, wt, b)
    got = {}
    for cfg in (3, 103):
        plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, 1, s, 0))
        plan.force_config(cfg)
        plan.force_split(1)
        got[cfg] = _run_plan(K, plan, n, x, wt, want.shape, shift=b)
    assert np.array_equal(got[3], got[103])
    assert netrun.rel_err(got[3], want) < 1e-4


@pytest.mark.parametrize("slices", [2, 3, 5, 64])
@pytest.mark.parametrize("geom", [(96, 14, 14, 64, 3, 1, 1), (512, 7, 7, 96, 1, 1, 0), (20, 6, 5, 40, 3, 2, 1)])
def test_conv_split_k_with_epilogue(K, geom, slices):
    """K cut into slices whose partial sums the last workgroup of each tile adds in slice
    order, then scale, shift, residual and activation: against the oracle and against
    the unsliced launch (slices beyond the K tile count are clamped)."""
    cin, h, w, cout, k, s, p = geom
    n = 2
    rng = np.random.default_rng(4)
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, cin, k, k)) * 0.1).astype(np.float32)
    sc = (rng.random(cout) + 0.5).astype(np.float32)
    sh = rng.standard_normal(cout).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, k, s, p), x, wt, None)
    res = rng.standard_normal(y.shape).astype(np.float32)
    want = oracle.relu(oracle.eltwise([oracle.scale(y, sc, sh), res], "SUM"), 0.0)
    outs = []
    for S in (1, slices):
        plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, k, s, p))
        plan.force_split(S)
        outs.append(_run_plan(K, plan, n, x, wt, want.shape, scale=sc, shift=sh, residual=res,
                              activation=K.ACT_RELU, negative_slope=0.0))
    assert netrun.rel_err(outs[0], want) < 1e-4
    assert netrun.rel_err(outs[1], want) < 1e-4
    assert netrun.rel_err(outs[1], outs[0]) < 1e-4   # summation order only


WINOGRAD_CASES = [
    # cin, h, w, cout, pad, batch: odd and even maps, every padding, one-pixel maps,
    # channel counts off every tile size, more blocks than one plane row of the inner blob
    (8, 6, 6, 8, 1, 1), (20, 7, 7, 33, 1, 3), (16, 14, 15, 16, 0, 2), (5, 9, 4, 7, 2, 2),
    (64, 13, 13, 70, 1, 5), (3, 1, 1, 4, 1, 2), (7, 3, 3, 5, 0, 1), (130, 28, 28, 128, 1, 2),
    (4, 200, 190, 6, 1, 2)]


@pytest.mark.parametrize("case", WINOGRAD_CASES)
def test_conv_winograd_path(K, case):
    """3x3 stride-1 convolutions pinned to the Winograd path, with the whole epilogue,
    against the oracle's direct sum; the same plan pinned to the direct path as well."""
    cin, h, w, cout, pad, n = case
    rng = np.random.default_rng(17)
    x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
    wt = (rng.standard_normal((cout, cin, 3, 3)) * 0.2).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    sc = (rng.random(cout) + 0.5).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, 3, 1, pad), x, wt, None)
    res = rng.standard_normal(y.shape).astype(np.float32)
    want = oracle.relu(oracle.eltwise([oracle.scale(y, sc, b), res], "SUM"), 0.1)
    plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, 3, 1, pad))
    ep = dict(scale=sc, shift=b, residual=res, activation=K.ACT_RELU, negative_slope=0.1)
    tol = 4e-6 * max(1.0, float(np.abs(y).max()))
    for mode in (1, 0):
        plan.force_winograd(mode)
        got = _run_plan(K, plan, n, x, wt, want.shape, **ep)
        assert np.abs(got - want).max() < tol, (case, mode)
    # no epilogue at all
    plan.force_winograd(1)
    got = _run_plan(K, plan, n, x, wt, y.shape)
    assert np.abs(got - y).max() < tol


@pytest.mark.parametrize("case", [(512, 19, 512, 2), (128, 28, 128, 3), (1024, 13, 256, 1)])
def test_conv_winograd_error_at_layer_sizes(K, case):
    """Sums over thousands of products, post-ReLU bottoms and He-scaled filters: the direct
    path, the Winograd path and the reference's own algorithm (im2col + OpenBLAS sgemm, the
    oracle) are all held against a float64 convolution with the parity metric (floor 1e-2 of
    the largest output, bar 1e-4); the Winograd path may not be further from float64 than
    three times the reference's algorithm is."""
    cin, hw, cout, n = case
    rng = np.random.default_rng(23)
    x = np.maximum(rng.standard_normal((n, cin, hw, hw)), 0).astype(np.float32)
    wt = (rng.standard_normal((cout, cin, 3, 3)) * np.sqrt(2.0 / (9 * cin))).astype(np.float32)
    oracle.use_openblas(True)
    try:
        want = oracle.conv_forward(oracle.conv_geom(cin, hw, hw, cout, 3, 1, 1), x, wt, None)
    finally:
        oracle.use_openblas(False)
    exact = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(),
                                       padding=1).numpy()
    plan = K.ConvPlan(K.conv_geom(cin, hw, hw, cout, 3, 1, 1))
    err = {}
    for mode in (0, 1):
        plan.force_winograd(mode)
        got = _run_plan(K, plan, n, x, wt, want.shape)
        err[mode] = netrun.rel_err(got, exact)
        assert err[mode] < 1e-4 and netrun.rel_err(got, want) < 1e-4, (case, mode, err)
    assert err[1] < 3 * max(netrun.rel_err(want, exact), 1e-5), (case, err)
    # the same comparison with the denominator floor at 1e-3 of the largest output (the
    # floor the parity metric of a whole net may use at its loosest): reported, and held
    # to the whole-net bar
    plan.force_winograd(1)
    got = _run_plan(K, plan, n, x, wt, want.shape)
    floor = 1e-3 * float(np.abs(exact).max())
    at_1e3 = float((np.abs(got - exact) / np.maximum(np.abs(exact), floor)).max())
    print("winograd %s: max relative error %.2e at floor 1e-3 of max, %.2e at floor 1e-2" % (case, at_1e3, err[1]))
    assert at_1e3 < 1e-3, (case, at_1e3)


@pytest.mark.parametrize("c_first", [1, 16, 50, 99])
def test_conv_winograd_two_tops(K, c_first):
    """The Winograd path with the output channels split over two blobs (merged sibling
    layers): the same values as with one top, odd and even maps, batch cut into runs."""
    rng = np.random.default_rng(19)
    for h, w, n in ((9, 7, 3), (10, 12, 5)):
        cin, cout = 24, 100
        x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
        wt = (rng.standard_normal((cout, cin, 3, 3)) * 0.2).astype(np.float32)
        b = rng.standard_normal(cout).astype(np.float32)
        sc = (rng.random(cout) + 0.5).astype(np.float32)
        plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, 3, 1, 1))
        plan.force_winograd(1)
        xd, wd, bd, sd = dev(x), dev(wt), dev(b), dev(sc)
        plan.set_weights(wd.data_ptr())
        ep = dict(scale=sd.data_ptr(), shift=bd.data_ptr(), activation=K_ACT_RELU)
        whole = torch.full((n, cout, h, w), float("nan"), device="cuda")
        plan.forward(n, xd.data_ptr(), whole.data_ptr(), **ep)
        for per_run in (0, 2):
            plan.force_chunk(per_run)
            first = torch.full((n, c_first, h, w), float("nan"), device="cuda")
            second = torch.full((n, cout - c_first, h, w), float("nan"), device="cuda")
            plan.forward_two_tops(n, xd.data_ptr(), first.data_ptr(), c_first, second.data_ptr(), **ep)
            torch.cuda.synchronize()
            assert torch.equal(first, whole[:, :c_first]) and torch.equal(second, whole[:, c_first:])
        plan.force_chunk(0)
        want = np.maximum(oracle.scale(oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, 3, 1, 1), x, wt, None),
                                       sc, b), 0)
        assert netrun.rel_err(whole.cpu().numpy(), want) < 1e-4
        with pytest.raises(Exception, match="TwoTops"):
            plan.forward_two_tops(n, xd.data_ptr(), first.data_ptr(), cout, second.data_ptr())


def test_conv_winograd_runs_batches_and_new_weights(K):
    """One plan on the Winograd path over changing batch sizes, with the batch cut into
    runs of images, and after the weights change."""
    cin, h, w, cout = 12, 10, 11, 9
    rng = np.random.default_rng(18)
    plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, 3, 1, 1))
    plan.force_winograd(1)
    for round_, n in enumerate((5, 2, 7, 5, 1)):
        plan.force_chunk(2 if round_ % 2 else 0)
        x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
        wt = (rng.standard_normal((cout, cin, 3, 3)) * 0.2).astype(np.float32)
        b = rng.standard_normal(cout).astype(np.float32)
        res = rng.standard_normal((n, cout, h, w)).astype(np.float32)
        want = oracle.conv_forward(oracle.conv_geom(cin, h, w, cout, 3, 1, 1), x, wt, b) + res
        got = _run_plan(K, plan, n, x, wt, want.shape, shift=b, residual=res)
        assert np.abs(got - want).max() < 1e-5, (round_, n)


def test_conv_winograd_refused_where_it_does_not_apply(K):
    for geom in (K.conv_geom(8, 9, 9, 8, 3, 2, 1), K.conv_geom(8, 9, 9, 8, 5, 1, 2),
                 K.conv_geom(8, 9, 9, 8, 3, 1, 1, group=2), K.conv_geom(8, 9, 9, 8, 3, 1, 1, dilation=2),
                 K.conv_geom(8, 9, 9, 8, 3, 1, 1, transposed=True)):
        plan = K.ConvPlan(geom)
        with pytest.raises(Exception, match="not a 3x3 stride-1 convolution"):
            plan.force_winograd(1)
        plan.force_winograd(0)
        plan.force_winograd(-1)


def test_conv_slices_summed_in_launch_over_many_launches(K):
    """The last workgroup of a tile to arrive adds the K slices of all of them, out of a
    workspace and arrival counters that every sliced launch on the stream shares: 60
    launches in a row, alternating between three geometries and slice counts with new
    values each time, must each equal the launch whose slices a separate pass adds
    (two tops: bit for bit, same partial sums in the same order) and agree with the
    unsliced launch (summation order only).  A partial sum read before it arrived, or
    left over from an earlier launch, would be off by whole terms."""
    cases = [((64, 14, 14, 128, 3, 1, 1), 4, 5), ((256, 7, 7, 64, 1, 1, 0), 8, 3), ((32, 20, 12, 96, 3, 2, 1), 2, 9)]
    plans = []
    gen = torch.Generator(device="cuda").manual_seed(5)
    for geom, slices, n in cases:
        cin, h, w, cout, k, s, p = geom
        ho, wo = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
        wd = torch.randn(cout, cin, k, k, device="cuda", generator=gen) * 0.1
        pl = [K.ConvPlan(K.conv_geom(*geom)) for _ in range(3)]
        for q in pl:
            q.set_weights(wd.data_ptr())
        pl[0].force_split(slices)
        pl[1].force_split(slices)
        pl[2].force_split(1)
        plans.append((pl, wd, (n, cin, h, w), (n, cout, ho, wo)))
    for it in range(60):
        pl, wd, xs, ys = plans[it % 3]
        n, cout = ys[0], ys[1]
        xd = torch.randn(*xs, device="cuda", generator=gen)
        bd = torch.randn(cout, device="cuda", generator=gen)
        whole = torch.full(ys, float("nan"), device="cuda")
        first = torch.full((n, 40) + ys[2:], float("nan"), device="cuda")
        second = torch.full((n, cout - 40) + ys[2:], float("nan"), device="cuda")
        plain = torch.full(ys, float("nan"), device="cuda")
        pl[0].forward(n, xd.data_ptr(), whole.data_ptr(), shift=bd.data_ptr(), activation=K_ACT_RELU)
        pl[1].forward_two_tops(n, xd.data_ptr(), first.data_ptr(), 40, second.data_ptr(),
                               shift=bd.data_ptr(), activation=K_ACT_RELU)
        pl[2].forward(n, xd.data_ptr(), plain.data_ptr(), shift=bd.data_ptr(), activation=K_ACT_RELU)
        torch.cuda.synchronize()
        assert torch.equal(first, whole[:, :40]) and torch.equal(second, whole[:, 40:]), it
        assert netrun.rel_err(whole.cpu().numpy(), plain.cpu().numpy()) < 1e-4, it


SLICED_IN_THE_CONFIGS = [
    # cin, h, w, cout, k, s, p, d, transposed, batch: the launches of the five configurations
    # (and their sizes) that leave workgroup slots empty and so cut their channel loop
    (64, 56, 56, 64, 3, 1, 1, 1, False, 1),          # config 1
    (1024, 14, 14, 256, 1, 1, 0, 1, False, 64),      # ResNet-50 b64, 784 tiles
    (512, 28, 28, 256, 1, 2, 0, 1, False, 64),
    (2048, 7, 7, 512, 1, 1, 0, 1, False, 64),        # 392 tiles
    (1024, 14, 14, 512, 1, 2, 0, 1, False, 64),
    (2048, 1, 1, 1000, 1, 1, 0, 1, False, 64),       # the classifier
    (512, 7, 7, 512, 3, 1, 1, 1, False, 64),         # Winograd path, two slices
    (512, 19, 19, 1024, 3, 1, 6, 6, False, 8),       # SSD300 b8: fc6 (dilated), fc7, the extra layers
    (1024, 19, 19, 1024, 1, 1, 0, 1, False, 8),
    (1024, 19, 19, 256, 1, 1, 0, 1, False, 8),
    (256, 19, 19, 512, 3, 2, 1, 1, False, 8),
    (512, 10, 10, 128, 1, 1, 0, 1, False, 8),
    (128, 10, 10, 256, 3, 2, 1, 1, False, 8),
    (128, 5, 5, 256, 3, 1, 0, 1, False, 8),
    (128, 3, 3, 256, 3, 1, 0, 1, False, 8),
    (512, 19, 19, 512, 3, 1, 1, 1, False, 8),        # conv5_x: Winograd path, sliced
    (1024, 38, 63, 512, 3, 1, 1, 1, False, 1),       # RPN head: Winograd path, three slices
    (1024, 4, 4, 512, 4, 2, 1, 1, True, 128),        # DCGAN b128: first deconvolution
]


def test_conv_sliced_launches_of_the_configurations_in_rotation(K):
    """Every launch of the five configurations whose channel loop the library cuts into
    slices (summed inside the launch out of a workspace and arrival counters that all
    sliced launches of a stream share), by the library's own choice of slices, three
    rounds in rotation: the three results of a geometry must be the same bit for bit (a
    partial sum read before it arrived, or left over from another launch, would differ)
    and agree with the unsliced launch (summation order only: two fp32 sums over up to
    9216 terms, bar 3e-4 against 1e-4 for a result against the oracle)."""
    gen = torch.Generator(device="cuda").manual_seed(15)
    work = []
    for cin, h, w, cout, k, st, p, d, tr, n in SLICED_IN_THE_CONFIGS:
        plan = K.ConvPlan(K.conv_geom(cin, h, w, cout, k, st, p, d, 1, tr))
        plain = K.ConvPlan(K.conv_geom(cin, h, w, cout, k, st, p, d, 1, tr))
        plain.force_split(1)
        wshape = (cin, cout, k, k) if tr else (cout, cin, k, k)
        wd = torch.randn(*wshape, device="cuda", generator=gen) * (2.0 / (cin * k * k)) ** 0.5
        plan.set_weights(wd.data_ptr())
        plain.set_weights(wd.data_ptr())
        ho, wo = plan.output_shape()
        xd = torch.randn(n, cin, h, w, device="cuda", generator=gen)
        bd = torch.randn(cout, device="cuda", generator=gen)
        work.append((plan, plain, wd, xd, bd, (n, cout, ho, wo), []))
    for _ in range(3):
        for plan, plain, wd, xd, bd, ys, outs in work:
            y = torch.full(ys, float("nan"), device="cuda")
            plan.forward(ys[0], xd.data_ptr(), y.data_ptr(), shift=bd.data_ptr(), activation=K_ACT_RELU)
            outs.append(y)
    torch.cuda.synchronize()
    for (plan, plain, wd, xd, bd, ys, outs), geom in zip(work, SLICED_IN_THE_CONFIGS):
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2]), geom
        ref = torch.full(ys, float("nan"), device="cuda")
        plain.forward(ys[0], xd.data_ptr(), ref.data_ptr(), shift=bd.data_ptr(), activation=K_ACT_RELU)
        torch.cuda.synchronize()
        assert netrun.rel_err(outs[0].cpu().numpy(), ref.cpu().numpy()) < 3e-4, geom


@pytest.mark.parametrize("act,slope", [("none", 0.0), ("relu", 0.0), ("relu", 0.2), ("tanh", 0.0),
                                       ("sigmoid", 0.0)])
def test_conv_epilogue_activations_full_channel_blocks(K, act, slope):
    """64 output channels: every 32-row block takes the batched epilogue path."""
    rng = np.random.default_rng(5)
    n, cin, cout, h = 2, 16, 64, 7
    x = rng.standard_normal((n, cin, h, h)).astype(np.float32)
    wt = (rng.standard_normal((cout, cin, 3, 3)) * 0.1).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(cin, h, h, cout, 3, 1, 1), x, wt, b)
    want = {"none": lambda v: v, "relu": lambda v: oracle.relu(v, slope), "tanh": oracle.tanh,
            "sigmoid": oracle.sigmoid}[act](y)
    code = {"none": K.ACT_NONE, "relu": K.ACT_RELU, "tanh": K.ACT_TANH, "sigmoid": K.ACT_SIGMOID}[act]
    plan = K.ConvPlan(K.conv_geom(cin, h, h, cout, 3, 1, 1))
    got = _run_plan(K, plan, n, x, wt, want.shape, shift=b, activation=code, negative_slope=slope)
    assert netrun.rel_err(got, want) < 1e-4


def test_depthwise_with_epilogue(K):
    """group == channels takes the direct kernel; scale, shift, residual and ReLU as for the
    implicit-GEMM path."""
    rng = np.random.default_rng(6)
    n, c, h = 3, 48, 19
    x = rng.standard_normal((n, c, h, h)).astype(np.float32)
    wt = (rng.standard_normal((c, 1, 3, 3)) * 0.3).astype(np.float32)
    sc = (rng.random(c) + 0.5).astype(np.float32)
    sh = rng.standard_normal(c).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(c, h, h, c, 3, 1, 1, 1, c), x, wt, None)
    res = rng.standard_normal(y.shape).astype(np.float32)
    want = oracle.relu(oracle.eltwise([oracle.scale(y, sc, sh), res], "SUM"), 0.1)
    plan = K.ConvPlan(K.conv_geom(c, h, h, c, 3, 1, 1, 1, c))
    assert plan.kernel_name(n) == "depthwise_f32"
    got = _run_plan(K, plan, n, x, wt, want.shape, scale=sc, shift=sh, residual=res,
                    activation=K.ACT_RELU, negative_slope=0.1)
    assert netrun.rel_err(got, want) < 1e-4


@pytest.mark.parametrize("c,h,w,s,p,n", [
    (48, 19, 19, 1, 1, 3), (7, 10, 10, 1, 0, 5), (6, 60, 60, 1, 1, 2),
    (5, 150, 150, 1, 1, 1),    # MobileNet conv1/dw
    (4, 75, 75, 2, 1, 2),      # stride 2, odd extents
    (3, 8, 585, 2, 0, 2), (3, 33, 130, 1, 1, 2), (2, 6, 1024, 1, 1, 1), (2, 6, 1025, 2, 1, 1),
    (3, 200, 40, 2, 1, 1),     # stride 2 with 16 output rows per thread (100 rows: 6 groups + 4)
    (2, 97, 9, 1, 0, 2),       # stride 1, 95 output rows: 8 per thread, ragged last group
    # MobileNet's 38x38 stride 2 and 19x19 stride 2, one pixel, two rows, many small planes
    (5, 38, 38, 2, 1, 3), (9, 19, 19, 2, 1, 2), (3, 1, 1, 1, 1, 2), (4, 2, 40, 1, 1, 2),
    (6, 5, 200, 2, 1, 2), (4, 43, 43, 1, 1, 1), (4, 44, 44, 1, 1, 1), (700, 5, 5, 1, 1, 30),
])
def test_depthwise_3x3_shapes(K, c, h, w, s, p, n):
    """3x3 depthwise at stride 1 and 2 (4, 8 or 16 output rows per thread by map height): small
    and large planes, odd extents, rows wider than a workgroup, with the whole epilogue."""
    rng = np.random.default_rng(21)
    x = rng.standard_normal((n, c, h, w)).astype(np.float32)
    wt = (rng.standard_normal((c, 1, 3, 3)) * 0.3).astype(np.float32)
    sc = (rng.random(c) + 0.5).astype(np.float32)
    sh = rng.standard_normal(c).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(c, h, w, c, 3, s, p, 1, c), x, wt, None)
    res = rng.standard_normal(y.shape).astype(np.float32)
    want = oracle.relu(oracle.eltwise([oracle.scale(y, sc, sh), res], "SUM"), 0.1)
    plan = K.ConvPlan(K.conv_geom(c, h, w, c, 3, s, p, 1, c))
    got = _run_plan(K, plan, n, x, wt, want.shape, scale=sc, shift=sh, residual=res,
                    activation=K.ACT_RELU, negative_slope=0.1)
    assert netrun.rel_err(got, want) < 1e-4


def test_conv_limits_are_errors(K):
    from minicaffe import MiniCaffeError
    with pytest.raises(MiniCaffeError, match="31 taps"):
        K.ConvPlan(K.conv_geom(1, 40, 40, 1, 33))
    # a bottom blob of 2^29 elements or more cannot be addressed: refused before any launch
    plan = K.ConvPlan(K.conv_geom(1024, 1024, 1024, 1, 1))
    dummy = torch.zeros(16, device="cuda")
    with pytest.raises(MiniCaffeError, match="2\\^29"):
        plan.forward(1, dummy.data_ptr(), dummy.data_ptr())

def test_conv_rejects_bad_geometry(K):
    from minicaffe import MiniCaffeError
    with pytest.raises(MiniCaffeError, match="multiples of group"):
        K.ConvPlan(K.conv_geom(6, 8, 8, 4, 3, group=4))
    with pytest.raises(MiniCaffeError, match="empty output"):
        K.ConvPlan(K.conv_geom(3, 2, 2, 4, 5))
    with pytest.raises(MiniCaffeError, match="Stride"):
        K.ConvPlan(K.conv_geom(3, 8, 8, 4, 3, stride=0))


@pytest.mark.parametrize("shape", [(2, 5, 7, 8), (3, 4, 1, 1), (1, 6, 3, 5), (2, 3, 16, 16)])
def test_channel_transform(K, shape):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(shape).astype(np.float32)
    c = shape[1]
    mean, var = rng.standard_normal(c).astype(np.float32), (rng.random(c) + 0.5).astype(np.float32)
    gamma, beta = rng.standard_normal(c).astype(np.float32), rng.standard_normal(c).astype(np.float32)
    want = oracle.relu(oracle.scale(oracle.batch_norm(x, mean, var, np.ones(1, np.float32), True, 1e-5),
                                    gamma, beta), 0.2)
    std = np.sqrt(var + np.float32(1e-5)).astype(np.float32)
    xd, yd = dev(x), torch.empty(shape, device="cuda")
    md, sd, gd, bd = dev(mean), dev(std), dev(gamma), dev(beta)
    op = K.ChannelOp(md.data_ptr(), sd.data_ptr(), gd.data_ptr(), bd.data_ptr(), K.ACT_RELU, 0.2)
    inner = int(np.prod(shape[2:]))
    K.check_mc(K.LIB.mcChannelTransform(fptr(xd), fptr(yd), shape[0], c, inner, ctypes.byref(op), None))
    torch.cuda.synchronize()
    assert netrun.rel_err(yd.cpu().numpy(), want) < 1e-5
    # activations alone, in place
    for act, fn in ((K.ACT_TANH, oracle.tanh), (K.ACT_SIGMOID, oracle.sigmoid)):
        zd = dev(x)
        op = K.ChannelOp(None, None, None, None, act, 0.0)
        K.check_mc(K.LIB.mcChannelTransform(fptr(zd), fptr(zd), 1, 1, x.size, ctypes.byref(op), None))
        torch.cuda.synchronize()
        assert np.abs(zd.cpu().numpy() - fn(x)).max() < 2e-7


def test_batch_norm_batch_stats(K):
    rng = np.random.default_rng(4)
    x = (rng.standard_normal((16, 12, 8, 8)) * 2 + 1).astype(np.float32)
    want = oracle.batch_norm(x, np.zeros(12), np.zeros(12), np.zeros(1), False, 1e-5)
    xd, yd = dev(x), torch.empty(x.shape, device="cuda")
    md, sd = torch.empty(12, device="cuda"), torch.empty(12, device="cuda")
    K.check_mc(K.LIB.mcBatchNormBatchStats(fptr(xd), 16, 12, 64, ctypes.c_float(1e-5), fptr(md), fptr(sd), None))
    op = K.ChannelOp(md.data_ptr(), sd.data_ptr(), None, None, 0, 0.0)
    K.check_mc(K.LIB.mcChannelTransform(fptr(xd), fptr(yd), 16, 12, 64, ctypes.byref(op), None))
    torch.cuda.synchronize()
    assert netrun.rel_err(yd.cpu().numpy(), want) < 1e-5
    assert np.abs(md.cpu().numpy() - x.mean(axis=(0, 2, 3))).max() < 1e-5


@pytest.mark.parametrize("shape", [(37, 6, 32, 32), (130, 3, 24, 20), (150, 5, 9, 13), (128, 16, 64, 64),
                                   (3, 2, 128, 128)])
def test_batch_norm_batch_stats_of_few_channels(K, shape):
    """With few channels each channel's images are cut into parts that run as workgroups of
    their own and are merged afterwards (part sizes that do not divide the batch, planes that
    are not a multiple of four, a batch too small to cut): mean and deviation against float64,
    on data whose mean is 60 deviations away from zero."""
    n, c, h, w = shape
    rng = np.random.default_rng(41)
    x = (rng.standard_normal(shape) * 0.5 + 30 + np.arange(c)[None, :, None, None]).astype(np.float32)
    xd = dev(x)
    md, sd = torch.empty(c, device="cuda"), torch.empty(c, device="cuda")
    K.check_mc(K.LIB.mcBatchNormBatchStats(fptr(xd), n, c, h * w, ctypes.c_float(1e-5), fptr(md), fptr(sd), None))
    torch.cuda.synchronize()
    x64 = x.astype(np.float64)
    assert np.abs(md.cpu().numpy() - x64.mean(axis=(0, 2, 3))).max() < 1e-4
    want_sd = np.sqrt(x64.var(axis=(0, 2, 3)) + 1e-5)
    assert np.abs(sd.cpu().numpy() / want_sd - 1).max() < 1e-4


@pytest.mark.parametrize("method", ["MAX", "AVE"])
@pytest.mark.parametrize("hw,k,s,p", [((112, 112), 3, 2, 0), ((75, 75), 2, 2, 0), ((19, 19), 3, 1, 1),
                                      ((7, 7), 7, 1, 0), ((6, 6), 2, 2, 1), ((9, 13), 3, 3, 1),
                                      # fixed-window max kernels: odd output heights, padding, 1-wide maps
                                      ((10, 7), 2, 2, 0), ((13, 9), 3, 2, 0), ((5, 9), 3, 2, 1), ((6, 1), 3, 1, 1),
                                      ((3, 3), 3, 2, 0), ((300, 300), 2, 2, 0),
                                      # MAX 3x3/2 on widths that are multiples of 4 (2 x 2 outputs per thread):
                                      # odd and even output extents, the clipped last window, one block only
                                      ((9, 12), 3, 2, 0), ((10, 16), 3, 2, 0), ((3, 4), 3, 2, 0), ((4, 8), 3, 2, 0),
                                      ((56, 56), 3, 2, 0)])
def test_pooling(K, method, hw, k, s, p):
    x = np.random.default_rng(5).standard_normal((2, 5) + hw).astype(np.float32)
    want = oracle.pooling(x, method, (k, k), (s, s), (p, p))
    ho, wo = ctypes.c_int(), ctypes.c_int()
    K.check_mc(K.LIB.mcPoolingOutputShape(hw[0], hw[1], k, k, s, s, p, p, ctypes.byref(ho), ctypes.byref(wo)))
    assert (ho.value, wo.value) == want.shape[2:]
    xd, yd = dev(x), torch.full(want.shape, float("nan"), device="cuda")
    K.check_mc(K.LIB.mcPooling(0 if method == "MAX" else 1, fptr(xd), fptr(yd), 10, hw[0], hw[1],
                               k, k, s, s, p, p, None))
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    if method == "MAX":
        assert np.array_equal(got, want)
    else:
        assert np.abs(got - want).max() < 1e-5


@pytest.mark.parametrize("method", ["MAX", "AVE"])
@pytest.mark.parametrize("hw", [(1, 1), (2, 3), (5, 5), (4, 8), (7, 7), (8, 8), (9, 9), (10, 13), (19, 19)])
def test_global_pooling_plane_sizes(K, method, hw):
    """A window that covers the whole plane: planes of 1 to 361 values (8, 16, 32 or 64 lanes
    per plane), a plane count that fills no workgroup evenly."""
    x = np.random.default_rng(15).standard_normal((3, 37) + hw).astype(np.float32)
    want = x.max(axis=(2, 3)) if method == "MAX" else x.astype(np.float64).mean(axis=(2, 3))
    xd, yd = dev(x), torch.full((3, 37, 1, 1), float("nan"), device="cuda")
    K.check_mc(K.LIB.mcPooling(0 if method == "MAX" else 1, fptr(xd), fptr(yd), 3 * 37, hw[0], hw[1],
                               hw[0], hw[1], 1, 1, 0, 0, None))
    torch.cuda.synchronize()
    got = yd.cpu().numpy().reshape(3, 37)
    if method == "MAX":
        assert np.array_equal(got, want)
    else:
        assert np.abs(got - want).max() < 1e-6


@pytest.mark.parametrize("op,coeffs", [("SUM", None), ("SUM", [1.0, -2.0, 0.5]), ("PROD", None), ("MAX", None)])
@pytest.mark.parametrize("count", [4096, 1001])
def test_eltwise(K, op, coeffs, count):
    rng = np.random.default_rng(6)
    xs = [rng.standard_normal(count).astype(np.float32) for _ in range(3)]
    want = oracle.eltwise(xs, op, coeffs)
    ds = [dev(a) for a in xs]
    ptrs = (ctypes.c_void_p * 3)(*[d.data_ptr() for d in ds])
    co = (ctypes.c_float * 3)(*coeffs) if coeffs else None
    yd = torch.empty(count, device="cuda")
    K.check_mc(K.LIB.mcEltwise({"PROD": 0, "SUM": 1, "MAX": 2}[op], 3, ptrs, co, count, fptr(yd), 0,
                               ctypes.c_float(0), None))
    torch.cuda.synchronize()
    assert np.abs(yd.cpu().numpy() - want).max() < 1e-6


@pytest.mark.parametrize("shape,axis", [((64, 1000), 1), ((8, 873, 21), 2), ((1, 2, 342, 63), 1),
                                        ((3, 5, 7), 1), ((4, 1500), 1),
                                        # rows that share a wavefront: every group width, ragged last wavefront
                                        ((7, 1), 1), ((13, 2), 1), ((67, 4), 1), ((9, 5), 1), ((131, 16), 1),
                                        ((5, 17), 1), ((3, 33), 1), ((6, 64), 1), ((6, 65), 1)])
def test_softmax(K, shape, axis):
    x = (np.random.default_rng(7).standard_normal(shape) * 3).astype(np.float32)
    want = oracle.softmax(x, axis)
    outer, inner = int(np.prod(shape[:axis])), int(np.prod(shape[axis + 1:]))
    xd, yd = dev(x), torch.empty(shape, device="cuda")
    K.check_mc(K.LIB.mcSoftmax(fptr(xd), fptr(yd), outer, shape[axis], inner, None))
    torch.cuda.synchronize()
    assert np.abs(yd.cpu().numpy() - want).max() < 1e-6


@pytest.mark.parametrize("shape,order", [((8, 84, 38, 38), (0, 2, 3, 1)), ((2, 3, 4, 5), (0, 3, 1, 2)),
                                         ((2, 3, 4, 5), (3, 2, 1, 0)), ((2, 3, 4, 5), (0, 1, 2, 3)),
                                         ((3, 70, 65), (0, 2, 1)), ((5, 6), (1, 0)),
                                         # 16-byte form of the tiled transpose: both extents multiples of 4,
                                         # ragged tiles on both sides; then extents that rule it out
                                         ((2, 68, 132), (0, 2, 1)), ((3, 256, 28, 28), (0, 2, 3, 1)),
                                         ((2, 4, 4), (0, 2, 1)), ((2, 68, 130), (0, 2, 1)), ((2, 66, 132), (0, 2, 1)),
                                         ((8, 24, 19, 19), (0, 2, 3, 1))])
def test_permute_bit_exact(K, shape, order):
    x = np.random.default_rng(8).standard_normal(shape).astype(np.float32)
    want = np.ascontiguousarray(np.transpose(x, order))
    xd, yd = dev(x), torch.full(want.shape, float("nan"), device="cuda")
    sh = (ctypes.c_int * len(shape))(*shape)
    od = (ctypes.c_int * len(order))(*order)
    K.check_mc(K.LIB.mcPermute(fptr(xd), fptr(yd), len(shape), sh, od, None))
    torch.cuda.synchronize()
    assert np.array_equal(yd.cpu().numpy(), want)


def test_copy2d_and_fill(K):
    x = np.random.default_rng(9).standard_normal((7, 33)).astype(np.float32)
    xd = dev(x)
    yd = torch.zeros((7, 50), device="cuda")
    K.check_mc(K.LIB.mcCopy2D(fptr(xd), 33, ctypes.c_void_p(yd.data_ptr() + 4 * 10), 50, 33, 7, None))
    K.check_mc(K.LIB.mcFill(fptr(yd), 5, ctypes.c_float(2.5), None))
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    assert np.array_equal(got[:, 10:43], x) and np.all(got[0, :5] == 2.5) and np.all(got[1:, :10] == 0)


@pytest.mark.parametrize("widths,rows", [
    ((4, 8, 12), 5),                                  # every width and offset a multiple of four: 16-byte accesses
    ((3, 0, 7, 1), 6),                                # ragged widths, an empty source
    ((16, 24, 24, 24, 16, 16, 84, 126, 126, 126, 84, 84), 8),   # more than eight sources: two launches
    ((5,), 3), ((34928, 8664, 2400, 600, 144, 16), 8)])        # one source; SSD300's six location heads
def test_concat_in_one_launch(K, widths, rows):
    rng = np.random.default_rng(14)
    xs = [rng.standard_normal((rows, w)).astype(np.float32) for w in widths]
    keep = [dev(x) if x.size else None for x in xs]
    srcs = (ctypes.c_void_p * len(xs))(*[k.data_ptr() if k is not None else None for k in keep])
    ws = (ctypes.c_long * len(xs))(*widths)
    yd = torch.full((rows, sum(widths)), float("nan"), device="cuda")
    K.check_mc(K.LIB.mcConcat(srcs, ws, len(xs), fptr(yd), rows, None))
    torch.cuda.synchronize()
    assert np.array_equal(yd.cpu().numpy(), np.concatenate(xs, axis=1))


@pytest.mark.parametrize("shape", [(2, 12, 5, 7),       # a thread keeps its channels in registers (<= 128)
                                   (2, 512, 9, 11),     # SSD's 512 channels, ragged pixel tile (<= 512)
                                   (1, 130, 6, 6), (1, 515, 3, 5)])   # > 512 channels: read twice
def test_normalize(K, shape):
    rng = np.random.default_rng(10)
    x = rng.standard_normal(shape).astype(np.float32)
    num, ch, spatial = shape[0], shape[1], shape[2] * shape[3]
    for across, shared in ((0, 0), (0, 1), (1, 0), (1, 1)):
        s = (rng.random(1 if shared else ch) + 0.5).astype(np.float32)
        want = oracle.normalize(x, s, bool(across), bool(shared), 1e-10)
        xd, sd, yd = dev(x), dev(s), torch.full(x.shape, float("nan"), device="cuda")
        K.check_mc(K.LIB.mcNormalize(fptr(xd), fptr(yd), num, ch, spatial, across, shared, ctypes.c_float(1e-10),
                                     fptr(sd), None))
        torch.cuda.synchronize()
        assert np.abs(yd.cpu().numpy() - want).max() < 1e-6


def run_proposal(K, scores, bbox, im_info, param, mode="both"):
    """mode "both": mcProposal (head of the table, then the full-size path, which skips itself
    on the device when the head settled the result); "rest": the full-size path alone
    (mcProposalRest); "steps": the layer's way, mcProposalHead, then mcProposalRest only if
    the head's state word says the result is not final.  Returns rois, scores, the
    equal-score replay flag and whether the head step alone gave the result."""
    anchors = oracle.generate_anchors()
    A, H, W = 9, scores.shape[2], scores.shape[3]
    pre, post = param["pre_nms_topn"], param["post_nms_topn"]
    sz = ctypes.c_size_t()
    K.check_mc(K.LIB.mcProposalWorkspaceSize(A * H * W, pre, post, ctypes.byref(sz)))
    ws = torch.empty(sz.value, dtype=torch.uint8, device="cuda")
    sd, bd, idv, ad = dev(scores), dev(bbox), dev(im_info), dev(anchors)
    rois = torch.full((post, 5), float("nan"), device="cuda")
    rs = torch.zeros(post, device="cuda")
    cnt = torch.zeros(3, dtype=torch.int32, device="cuda")

    def call(fn):
        K.check_mc(fn(fptr(sd), fptr(bd), fptr(idv), fptr(ad), A, H, W, 16,
                      ctypes.c_float(param.get("min_size", 16)), pre, post,
                      ctypes.c_float(param["nms_thresh"]), fptr(ws), sz.value, fptr(rois),
                      fptr(rs), ctypes.c_void_p(cnt.data_ptr()),
                      ctypes.c_void_p(cnt.data_ptr() + 4), None))
        torch.cuda.synchronize()

    head_final = False
    if mode == "both":
        call(K.LIB.mcProposal)
    elif mode == "rest":
        call(K.LIB.mcProposalRest)
        assert int(cnt[2].item()) == 1
    else:
        call(K.LIB.mcProposalHead)
        head_final = int(cnt[2].item()) == 1
        if not head_final:
            call(K.LIB.mcProposalRest)
            assert int(cnt[2].item()) == 1
    n, ties = int(cnt[0].item()), int(cnt[1].item())
    return rois[:n].cpu().numpy(), rs[:n].cpu().numpy(), ties, head_final


@pytest.mark.parametrize("hw,pre,post,thr,quant", [
    ((38, 63), 6000, 300, 0.7, 0),       # config 4 size, tie-free
    ((38, 63), 6000, 300, 0.7, 2000),    # ties inside the top 6000
    ((38, 63), 300, 2000, 0.9, 0),       # fewer candidates than post_nms_topn
    ((10, 12), 2000, 50, 0.5, 0),        # pre_nms_topn > proposals: zero-score ties
    ((20, 20), 6000, 300, 0.7, 7),       # heavy ties
    ((5, 4), 100, 300, 0.3, 0),
    ((50, 60), 6000, 300, 0.7, 0),       # 27000 proposals: sort through global scratch
    ((50, 60), 6000, 300, 0.7, 5000),    # ... with ties: replay starts outside LDS
    # the greedy scan's super-blocks of 512 boxes
    ((50, 60), 12000, 1000, 0.7, 0),     # 188 mask words per row: more words than lanes
    ((38, 63), 513, 600, 0.1, 0),        # one box into the second super-block, heavy suppression
    ((38, 63), 512, 600, 0.95, 0),       # exactly one super-block, almost everything kept
    ((38, 63), 6000, 37, 0.7, 0),        # post_nms_topn reached inside the first block
    ((38, 63), 6000, 5000, 0.3, 0),      # every super-block walked, post_nms_topn never reached
    ((38, 63), 6000, 700, 0.8, 0),       # post_nms_topn reached in a later super-block
])
def test_proposal_bit_exact(K, hw, pre, post, thr, quant):
    """Kept rois and scores equal the CPU path's bit for bit, with and without
    score ties (ties replay the reference's quicksort on the device)."""
    rng = np.random.default_rng(11)
    A, (H, W) = 9, hw
    n = A * H * W
    scores = rng.random((1, 2 * A, H, W)).astype(np.float32)
    scores[0, A:] = (rng.permutation(n).astype(np.float32) / n * 0.9 + 0.05).reshape(A, H, W)
    if quant:
        scores[0, A:] = np.round(scores[0, A:] * quant) / quant
    bbox = (rng.standard_normal((1, 4 * A, H, W)) * 0.3).astype(np.float32)
    im_info = np.array([H * 16, W * 16, 1.0], np.float32)
    param = {"pre_nms_topn": pre, "post_nms_topn": post, "nms_thresh": thr}
    want_rois, want_scores = oracle.proposal(param, scores, bbox, im_info, 2)
    for mode in ("rest", "both", "steps"):
        rois, rs, ties, _ = run_proposal(K, scores, bbox, im_info, param, mode)
        assert np.array_equal(rois, want_rois), mode
        assert np.array_equal(rs, want_scores), mode
        if quant and mode == "rest":
            assert ties & 1


@pytest.mark.parametrize("hw,pre,post,thr,pairs,seed", [
    ((38, 63), 6000, 300, 0.7, 1, 0),        # config 4 size, a single pair of equal scores
    ((38, 63), 6000, 300, 0.7, 20, 1),       # about as many as the configuration's own scores hold
    ((38, 63), 6000, 300, 0.7, 120, 2),
    ((38, 63), 6000, 300, 0.7, 480, 3),      # close to the most the few-ties kernel takes
    ((38, 63), 6000, 300, 0.7, 520, 4),      # just beyond: the general kernel
    ((38, 63), 300, 100, 0.7, 200, 5),       # most pairs lie beyond the cut
    ((20, 20), 6000, 300, 0.7, 60, 6),       # pre_nms_topn > proposals
    ((5, 4), 100, 300, 0.3, 30, 7),          # partitions of a few places only
    ((11, 9), 500, 60, 0.5, 8, 8),
    ((39, 64), 6000, 300, 0.7, 25, 9),       # 22 464 proposals: the largest map the kernel holds
    ((40, 63), 6000, 300, 0.7, 25, 10),      # 22 680: beyond it
])
@pytest.mark.parametrize("general", [False, True])
def test_proposal_with_few_equal_scores(K, hw, pre, post, thr, pairs, seed, general):
    """A few equal scores among otherwise distinct ones (what real score maps look like):
    some pairs, some runs of three to five, some straddling the pre_nms_topn cut.  The kernel
    that follows only the partitions holding equal scores and the general level-by-level
    kernel must both leave the reference quicksort's order."""
    rng = np.random.default_rng(100 + seed)
    A, (H, W) = 9, hw
    n = A * H * W
    fg = (rng.permutation(n).astype(np.float32) / n * 0.9 + 0.05)
    best = np.argsort(-fg)[:min(pre, n) // 2]
    for g in range(pairs):
        size = 2 if g % 5 else int(rng.integers(3, 6))
        idx = rng.choice(best if g == 0 else n, size, replace=False)   # the first group among the best
        fg[idx] = fg[idx[0]]
    if pairs >= 8:                          # equal scores right at the cut
        order = np.argsort(-fg, kind="stable")
        cut = min(pre, n) - 1
        fg[order[cut:cut + 3]] = fg[order[cut]]
    scores = rng.random((1, 2 * A, H, W)).astype(np.float32)
    scores[0, A:] = fg.reshape(H, W, A).transpose(2, 0, 1)
    bbox = (rng.standard_normal((1, 4 * A, H, W)) * 0.3).astype(np.float32)
    im_info = np.array([H * 16, W * 16, 1.0], np.float32)
    param = {"pre_nms_topn": pre, "post_nms_topn": post, "nms_thresh": thr}
    want_rois, want_scores = oracle.proposal(param, scores, bbox, im_info, 2)
    K.check_mc(K.LIB.mcProposalForceGeneralReplay(int(general)))
    try:
        for mode in ("both", "steps", "rest"):
            rois, rs, ties, _ = run_proposal(K, scores, bbox, im_info, param, mode)
            assert np.array_equal(rois, want_rois), mode
            assert np.array_equal(rs, want_scores), mode
    finally:
        K.check_mc(K.LIB.mcProposalForceGeneralReplay(0))
    # which kernel did it: 3 = the few-ties one (at most 22 528 proposals and 500 equal
    # neighbour pairs among the best pre_nms_topn + 1 sorted scores), 1 = the general one
    props = oracle.generate_proposals(scores[0, A:], bbox[0], oracle.generate_anchors(), float(im_info[0]),
                                      float(im_info[1]), 16.0, 16)
    skey = np.sort(props[:, 4])[::-1]       # too small boxes score 0: more equal scores at the end
    counted = int((skey[:-1] == skey[1:])[:min(pre, n)].sum())
    assert counted > 0
    assert ties == (3 if (not general and n <= 22528 and counted <= 500) else 1)


@pytest.mark.parametrize("seed", range(12))
def test_proposal_head_with_equal_scores_among_the_best(K, seed):
    """The head step (best 512 proposals) may only call its result final when the order of
    equal scores cannot matter.  Equal scores are planted among the best few hundred
    proposals, half of the groups on proposals of one anchor position and shape (boxes
    that overlap: one suppresses the other, which one depends on the reference's order),
    half on proposals far apart (both kept: the order of the rows depends on it), some
    below a box that suppresses them (dead: no order matters).  Whatever the head decides,
    the rows must equal the reference's bit for bit; over the seeds both outcomes occur."""
    rng = np.random.default_rng(500 + seed)
    A, H, W = 9, 38, 63
    n = A * H * W
    fg = (rng.permutation(n).astype(np.float32) / n * 0.9 + 0.05).reshape(H, W, A)
    bbox = (rng.standard_normal((1, 4 * A, H, W)) * 0.05).astype(np.float32)
    flat = fg.reshape(-1)
    best = np.argsort(-flat)[:400]
    groups = int(rng.integers(0, 4)) if seed % 3 else 0
    for g in range(groups):
        i = int(rng.choice(best[20:]))
        h, w, k = np.unravel_index(i, (H, W, A))
        if g % 2 == 0:      # neighbour position, same anchor shape: heavy overlap
            j = np.ravel_multi_index((h, min(w + 1, W - 1) if w + 1 < W else w - 1, k), (H, W, A))
        else:               # far away
            j = np.ravel_multi_index(((h + H // 2) % H, (w + W // 2) % W, k), (H, W, A))
        flat[j] = flat[i]
    scores = rng.random((1, 2 * A, H, W)).astype(np.float32)
    scores[0, A:] = fg.transpose(2, 0, 1)
    im_info = np.array([H * 16, W * 16, 1.0], np.float32)
    param = {"pre_nms_topn": 6000, "post_nms_topn": int(rng.choice([50, 300])), "nms_thresh": 0.7}
    want_rois, want_scores = oracle.proposal(param, scores, bbox, im_info, 2)
    outcomes = []
    for mode in ("steps", "both"):
        rois, rs, ties, head_final = run_proposal(K, scores, bbox, im_info, param, mode)
        assert np.array_equal(rois, want_rois), (mode, head_final)
        assert np.array_equal(rs, want_scores), (mode, head_final)
        outcomes.append(head_final)
    if groups == 0:
        assert outcomes[0]          # distinct scores: the head settles it


def test_detection_output_shared_locations_without_background_fail(K):
    """share_location with background_label_id -1 aborts in the reference ("Could not find
    location predictions for label -1", detection_output_layer.cpp:122-126): an error here."""
    rng = np.random.default_rng(3)
    P, C = 6, 3
    loc = rng.standard_normal((1, P * 4)).astype(np.float32)
    conf = oracle.softmax(rng.standard_normal((1, P, C)).astype(np.float32), 2).reshape(1, P * C)
    prior = np.tile(np.float32([0.1, 0.1, 0.4, 0.4]), 2 * P).reshape(1, 2, P * 4)
    param = {"num_classes": C, "share_location": True, "background_label_id": -1,
             "nms_param": {"nms_threshold": 0.5}}
    with pytest.raises(Exception, match="label -1"):
        run_detection_output(K, param, loc, conf, prior)


@pytest.mark.parametrize("num,P,C,share,code,keep,thr,nms,eta,topk,sigma", [
    (2, 64, 4, True, "CENTER_SIZE", 10, 0.01, 0.45, 1.0, 20, 2.0),
    (8, 8732, 21, True, "CENTER_SIZE", 200, 0.01, 0.45, 1.0, 400, 2.0),   # config 3 tail, logits N(0, sigma=2)
    (3, 500, 5, False, "CORNER", -1, None, 0.3, 1.0, None, 2.0),          # per-class boxes, no limits
    (2, 300, 6, True, "CORNER_SIZE", 50, 0.05, 0.6, 0.9, 100, 2.0),       # adaptive threshold (eta < 1)
    (2, 100, 3, True, "CENTER_SIZE", 10, 0.999999, 0.45, 1.0, 20, 2.0),   # nothing kept -> rows of -1
    (1, 2000, 21, True, "CENTER_SIZE", 200, 0.01, 0.45, 1.0, 400, 0.5),
    (1, 13000, 3, True, "CENTER_SIZE", 100, 0.01, 0.45, 1.0, 1500, 2.0),   # sort through global scratch,
                                                                           # more candidates than cached
    # candidate counts around the limits of the block-wise form of the greedy pass (constant threshold)
    (2, 3000, 3, True, "CENTER_SIZE", -1, 0.001, 0.45, 1.0, 576, 1.0),     # nine blocks: more later blocks than wavefronts
    (2, 3000, 3, True, "CENTER_SIZE", -1, 0.001, 0.45, 1.0, 577, 1.0),     # a last block of one candidate
    (2, 3000, 3, True, "CENTER_SIZE", -1, 0.001, 0.45, 1.0, 1024, 1.0),    # as many candidates as LDS caches
    (2, 3000, 3, True, "CENTER_SIZE", -1, 0.001, 0.45, 1.0, 1025, 1.0),    # one more: one-wavefront pass
    (2, 3000, 3, True, "CENTER_SIZE", -1, 0.001, 0.3, 1.0, 64, 1.0),       # exactly one block
    (2, 3000, 3, True, "CENTER_SIZE", -1, 0.001, 0.3, 1.0, 65, 1.0),
    (1, 3000, 3, True, "CENTER_SIZE", -1, 0.001, 0.95, 1.0, 300, 1.0),     # nearly everything kept
    # keep_top_k over more kept boxes than the selection holds in registers (8192): through global scratch
    (1, 6000, 12, True, "CENTER_SIZE", 300, 0.001, 0.95, 1.0, 900, 1.0),
    (1, 6000, 12, True, "CENTER_SIZE", -1, 0.001, 0.95, 1.0, 900, 1.0),    # ... and without a cut
    (2, 700, 13, True, "CENTER_SIZE", 0, 0.001, 0.6, 1.0, 100, 1.0),       # keep_top_k 0: nothing kept
    (2, 3000, 4, False, "CORNER", -1, 0.001, 0.7, 1.0, 1, 1.0),            # a single candidate per class
    (1, 400, 2, True, "CENTER_SIZE", -1, None, 0.05, 1.0, None, 1.0),      # low threshold: long reject chains
])
def test_detection_output_bit_exact(K, num, P, C, share, code, keep, thr, nms, eta, topk, sigma):
    rng = np.random.default_rng(12)
    lc = 1 if share else C
    loc = (rng.standard_normal((num, P * lc * 4)) * 0.5).astype(np.float32)
    conf = oracle.softmax((rng.standard_normal((num, P, C)) * sigma).astype(np.float32), 2).reshape(num, P * C)
    c = rng.random((P, 2)) * 0.8 + 0.1
    wh = rng.random((P, 2)) * 0.3 + 0.05
    prior = np.concatenate([np.concatenate([c - wh / 2, c + wh / 2], 1).reshape(-1),
                            np.tile([0.1, 0.1, 0.2, 0.2], P)]).reshape(1, 2, P * 4).astype(np.float32)
    param = {"num_classes": C, "share_location": share, "background_label_id": 0, "code_type": code,
             "keep_top_k": keep, "nms_param": {"nms_threshold": nms, "eta": eta}}
    if thr is not None:
        param["confidence_threshold"] = thr
    if topk is not None:
        param["nms_param"]["top_k"] = topk
    want = oracle.detection_output(param, loc, conf, prior)
    got, flag = run_detection_output(K, param, loc, conf, prior)
    assert got.shape == want.shape
    assert np.array_equal(got, want)
    want_flag = cut_tie_expected(param, loc, conf, prior)
    assert flag == want_flag and not (want_flag & 1)      # no case here is undefined at the cut


def run_detection_output(K, param, loc, conf, prior):
    """mcDetectionOutput on host arrays -> (rows, cut-tie flag)."""
    num, C = loc.shape[0], param["num_classes"]
    P = prior.shape[2] // 4
    nmsp = param.get("nms_param", {})
    tk, keep = nmsp.get("top_k", -1), param.get("keep_top_k", -1)
    share = param.get("share_location", True)
    sz = ctypes.c_size_t()
    K.check_mc(K.LIB.mcDetectionOutputWorkspaceSize(num, P, C, int(share), tk, ctypes.byref(sz)))
    max_rows = K.LIB.mcDetectionOutputMaxRows(num, P, C, tk, keep)
    ws = torch.empty(sz.value, dtype=torch.uint8, device="cuda")
    ld, cd, pd = dev(loc), dev(conf), dev(prior)
    code = {"CORNER": 1, "CENTER_SIZE": 2, "CORNER_SIZE": 3}[str(param.get("code_type", "CORNER"))]
    results = []
    # every input twice: three launches per class wherever the input allows it, then pinned
    # to the one-launch-per-class kernels; same rows, same flag
    for split in (2, 0):
        out = torch.full((max_rows, 7), float("nan"), device="cuda")
        cnt = torch.full((2,), -5, dtype=torch.int32, device="cuda")
        K.check_mc(K.LIB.mcDetectionOutputSplit(split))
        try:
            K.check_mc(K.LIB.mcDetectionOutput(
                fptr(ld), fptr(cd), fptr(pd), num, P, C, int(share), param.get("background_label_id", 0), code,
                int(param.get("variance_encoded_in_target", False)), keep,
                ctypes.c_float(param.get("confidence_threshold", -3.4028234663852886e38)),
                ctypes.c_float(nmsp.get("nms_threshold", 0.3)), ctypes.c_float(nmsp.get("eta", 1.0)), tk, fptr(ws),
                sz.value, fptr(out), max_rows, ctypes.c_void_p(cnt.data_ptr()), ctypes.c_void_p(cnt.data_ptr() + 4),
                None))
            torch.cuda.synchronize()
        finally:
            K.check_mc(K.LIB.mcDetectionOutputSplit(1))
        results.append((out[:int(cnt[0].item())].cpu().numpy(), int(cnt[1].item())))
    assert np.array_equal(results[0][0], results[1][0], equal_nan=True) and results[0][1] == results[1][1]
    return results[0]


def cut_tie_expected(param, loc, conf, prior):
    """The flag's bits from the CPU side.  Over the images that keep_top_k cuts: 1 when the
    keep_top_k-th and the next score of the per-class NMS survivors are equal, 2 when two
    kept rows of one label have equal scores (std::sort defines neither order)."""
    keep = param.get("keep_top_k", -1)
    if keep < 0:
        return 0
    rows = oracle.detection_output(dict(param, keep_top_k=-1), loc, conf, prior)
    flag = 0
    for i in range(loc.shape[0]):
        r = rows[(rows[:, 0] == i) & (rows[:, 1] >= 0)]
        sc = np.sort(r[:, 2])[::-1]
        if not len(sc) > keep > 0:
            continue
        if sc[keep - 1] == sc[keep]:
            flag |= 1
        for lab in np.unique(r[:, 1]):
            s = r[(r[:, 1] == lab) & (r[:, 2] >= sc[keep - 1]), 2]
            # of a run of equal scores at the cut only a prefix is kept: count what survives
            room = keep - int((r[:, 2] > sc[keep - 1]).sum())
            at_cut = r[r[:, 2] == sc[keep - 1]]
            taken = at_cut[np.argsort(at_cut[:, 1], kind="stable")][:room]
            s = np.concatenate([r[(r[:, 1] == lab) & (r[:, 2] > sc[keep - 1]), 2],
                                taken[taken[:, 1] == lab, 2]])
            if len(np.unique(s)) < len(s):
                flag |= 2
    return flag


def test_detection_output_flags_equal_scores_at_the_keep_top_k_cut(K):
    """Quantised confidences: some images have equal scores on both sides of the cut.
    The flag says so (bit 1 = tie at the cut, bit 2 = equal scores within a kept label);
    the rows above the tied score are the oracle's up to the order of equal scores, and
    the kept scores are the same multiset either way."""
    rng = np.random.default_rng(40)
    num, P, C = 6, 300, 4
    loc = (rng.standard_normal((num, P * 4)) * 0.5).astype(np.float32)
    conf = (np.round(rng.random((num, P * C)) * 50) / 50).astype(np.float32)
    c = rng.random((P, 2)) * 0.8 + 0.1
    wh = rng.random((P, 2)) * 0.1 + 0.02
    prior = np.concatenate([np.concatenate([c - wh / 2, c + wh / 2], 1).reshape(-1),
                            np.tile([0.1, 0.1, 0.2, 0.2], P)]).reshape(1, 2, P * 4).astype(np.float32)
    param = {"num_classes": C, "share_location": True, "background_label_id": 0, "code_type": "CENTER_SIZE",
             "keep_top_k": 40, "confidence_threshold": 0.3, "nms_param": {"nms_threshold": 0.45, "top_k": 100}}
    got, flag = run_detection_output(K, param, loc, conf, prior)
    assert flag == 3 and cut_tie_expected(param, loc, conf, prior) == 3
    want = oracle.detection_output(param, loc, conf, prior)
    assert got.shape == want.shape
    for i in range(num):
        g, w = got[got[:, 0] == i], want[want[:, 0] == i]
        assert np.array_equal(np.sort(g[:, 2]), np.sort(w[:, 2]))
        cut = g[:, 2].min()                       # rows strictly above the tied score are defined
        ga, wa = g[g[:, 2] > cut], w[w[:, 2] > cut]
        assert np.array_equal(ga[np.lexsort(ga.T[::-1])], wa[np.lexsort(wa.T[::-1])])
    # without a cut there is nothing to flag
    got, flag = run_detection_output(K, dict(param, keep_top_k=-1), loc, conf, prior)
    assert flag == 0 and np.array_equal(got, oracle.detection_output(dict(param, keep_top_k=-1), loc, conf, prior))


def _random_rois(rng, n_rois, num, img_h, img_w):
    """Proposal-like rows [batch, x1, y1, x2, y2] in image coordinates, with some tiny,
    some reaching past the image and some wholly outside."""
    b = rng.integers(0, num, n_rois).astype(np.float32)
    cx, cy = rng.random(n_rois) * img_w, rng.random(n_rois) * img_h
    w, h = rng.random(n_rois) ** 2 * img_w, rng.random(n_rois) ** 2 * img_h
    rois = np.stack([b, cx - w / 2, cy - h / 2, cx + w / 2, cy + h / 2], 1).astype(np.float32)
    rois[0, 1:] = [0, 0, img_w - 1, img_h - 1]
    rois[1, 1:] = [img_w + 5, img_h + 5, img_w + 40, img_h + 40]      # outside
    rois[2, 1:] = [3.2, 4.7, 3.4, 4.9]                                # below one cell
    rois[3, 1:] = [-30.5, -12.5, 20.5, 17.5]                          # negative corner, half-way values
    return rois


@pytest.mark.parametrize("shape,pooled,scale", [((2, 5, 38, 63), (6, 6), 0.0625), ((1, 3, 9, 7), (2, 3), 1.0),
                                                ((3, 4, 20, 20), (7, 7), 0.125)])
def test_roi_pooling_bit_exact(K, shape, pooled, scale):
    rng = np.random.default_rng(20)
    x = rng.standard_normal(shape).astype(np.float32)
    rois = _random_rois(rng, 64, shape[0], shape[2] / scale, shape[3] / scale)
    want = oracle.roi_pooling(x, rois, pooled[0], pooled[1], scale)
    xd, rd = dev(x), dev(rois)
    out = torch.full(want.shape, float("nan"), device="cuda")
    K.check_mc(K.LIB.mcROIPooling(fptr(xd), *shape, fptr(rd), rois.shape[0], pooled[0], pooled[1],
                                  ctypes.c_float(scale), fptr(out), None, None))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)


@pytest.mark.parametrize("num,dim,g,hw,scale", [(1, 21, 7, (38, 63), 0.0625), (2, 8, 3, (20, 20), 0.125),
                                                (1, 4, 1, (6, 6), 1.0)])
def test_psroi_pooling_bit_exact(K, num, dim, g, hw, scale):
    rng = np.random.default_rng(21)
    x = rng.standard_normal((num, dim * g * g) + hw).astype(np.float32)
    rois = _random_rois(rng, 64, num, hw[0] / scale, hw[1] / scale)
    want = oracle.psroi_pooling(x, rois, dim, g, scale)
    xd, rd = dev(x), dev(rois)
    out = torch.full(want.shape, float("nan"), device="cuda")
    flag = torch.zeros(1, dtype=torch.int32, device="cuda")
    K.check_mc(K.LIB.mcPSROIPooling(fptr(xd), num, dim, g, hw[0], hw[1], fptr(rd), rois.shape[0],
                                    ctypes.c_float(scale), fptr(out), ctypes.c_void_p(flag.data_ptr()), None))
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), want)     # same expressions, same summation order
    assert int(flag.item()) == 0
    # a batch index outside the blob: zeros and the flag, where the reference's CPU code CHECK-fails
    bad = rois[:4].copy()
    bad[1, 0] = num
    rd2 = dev(bad)
    out2 = torch.full((4, dim, g, g), float("nan"), device="cuda")
    K.check_mc(K.LIB.mcPSROIPooling(fptr(xd), num, dim, g, hw[0], hw[1], fptr(rd2), 4,
                                    ctypes.c_float(scale), fptr(out2), ctypes.c_void_p(flag.data_ptr()), None))
    torch.cuda.synchronize()
    got = out2.cpu().numpy()
    assert int(flag.item()) == 1 and np.array_equal(got[1], np.zeros((dim, g, g), np.float32))
    assert np.array_equal(got[[0, 2, 3]], want[[0, 2, 3]])


# ---- less common layers ------------------------------------------------------------

def close(got, want, tol=1e-5):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    return np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max())


UNARY = {"POWER": 0, "EXP": 1, "LOG": 2, "ABS": 3, "BNLL": 4, "ELU": 5, "THRESHOLD": 6}


def run_unary(K, op, x, p0=0.0, p1=0.0, p2=0.0, offset=0):
    xd = dev(x.reshape(-1))
    yd = torch.full((x.size + offset,), float("nan"), device="cuda")
    K.check_mc(K.LIB.mcUnary(UNARY[op], fptr(xd), ctypes.c_void_p(yd.data_ptr() + 4 * offset), x.size,
                             p0, p1, p2, None))
    torch.cuda.synchronize()
    return yd[offset:].cpu().numpy().reshape(x.shape)


@pytest.mark.parametrize("n", [1, 3, 1021, 4096, 100003])
def test_unary_functions(K, n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    pos = (rng.random(n) * 4 + 0.05).astype(np.float32)
    assert close(run_unary(K, "POWER", pos, 2.0, 1.0, 0.5), oracle.power(pos, 0.5, 2.0, 1.0))
    assert close(run_unary(K, "POWER", pos, 1e-2, 1.0, -0.75), oracle.power(pos, -0.75, 1e-2, 1.0))
    assert close(run_unary(K, "POWER", x, 1.0, 0.0, 2.0), oracle.power(x, 2.0), 1e-6)
    assert np.array_equal(run_unary(K, "POWER", x, 1.0, 0.0, 1.0), x)
    assert close(run_unary(K, "EXP", x, 1.0, 1.0), oracle.exp_layer(x))
    assert close(run_unary(K, "EXP", x, np.float32(np.log(np.float32(2.0))) * np.float32(0.5), 8.0),
                 oracle.exp_layer(x, 2.0, 0.5, 3.0))
    assert close(run_unary(K, "LOG", pos, 1.0, 0.0, 1.0), oracle.log_layer(pos))
    assert close(run_unary(K, "LOG", pos, 2.0, 1.0, 1.0 / np.log(np.float32(10.0))),
                 oracle.log_layer(pos, 10.0, 2.0, 1.0))
    assert np.array_equal(run_unary(K, "ABS", x), oracle.absval(x))
    big = np.concatenate([x, np.array([90.0, -90.0, 0.0], np.float32)])
    assert close(run_unary(K, "BNLL", big), oracle.bnll(big), 1e-6)
    assert close(run_unary(K, "ELU", x, 1.5), oracle.elu(x, 1.5), 1e-6)
    assert np.array_equal(run_unary(K, "THRESHOLD", x, 0.25), oracle.threshold(x, 0.25))
    # a destination that is not 16-byte aligned takes the scalar walk
    assert np.array_equal(run_unary(K, "ABS", x, offset=1), oracle.absval(x))


def test_unary_in_place_and_bad_op(K):
    x = np.random.default_rng(0).standard_normal(777).astype(np.float32)
    xd = dev(x)
    K.check_mc(K.LIB.mcUnary(UNARY["ABS"], fptr(xd), fptr(xd), x.size, 0.0, 0.0, 0.0, None))
    assert np.array_equal(xd.cpu().numpy(), np.abs(x))
    assert K.LIB.mcUnary(42, fptr(xd), fptr(xd), x.size, 0.0, 0.0, 0.0, None) != 0


@pytest.mark.parametrize("shape,shared", [((2, 5, 7, 3), False), ((3, 4), False), ((2, 6, 9, 9), True)])
def test_prelu(K, shape, shared):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(shape).astype(np.float32)
    slope = rng.standard_normal(1 if shared else shape[1]).astype(np.float32)
    xd, sd = dev(x), dev(slope)
    yd = torch.empty_like(xd)
    inner = int(np.prod(shape[2:]))
    K.check_mc(K.LIB.mcPReLU(fptr(xd), fptr(yd), shape[0], shape[1], inner, fptr(sd), int(shared), None))
    assert np.array_equal(yd.cpu().numpy(), oracle.prelu(x, slope, shared))


@pytest.mark.parametrize("case", [(2, 96, 27, 27, 5), (1, 7, 3, 5, 3), (2, 40, 6, 6, 9), (1, 3, 4, 4, 1),
                                  (1, 2, 5, 5, 7),
                                  # chunks of 32 channels walked in blocks of 8: ragged last chunk and block
                                  (1, 33, 5, 5, 5), (2, 64, 4, 4, 7), (1, 100, 3, 3, 3), (1, 45, 2, 3, 5)])
def test_lrn_across_channels(K, case):
    n, c, h, w, size = case
    x = (np.random.default_rng(2).standard_normal((n, c, h, w)) * 4).astype(np.float32)
    xd = dev(x)
    yd = torch.full_like(xd, float("nan"))
    K.check_mc(K.LIB.mcLRNAcrossChannels(fptr(xd), fptr(yd), n, c, h, w, size, 1e-2, 0.75, 2.0, None))
    assert close(yd.cpu().numpy(), oracle.lrn(x, size, 1e-2, 0.75, 2.0), 1e-5)
    assert K.LIB.mcLRNAcrossChannels(fptr(xd), fptr(yd), n, c, h, w, 4, 1e-2, 0.75, 2.0, None) != 0


@pytest.mark.parametrize("case", [(6, 13, 11, 3), (2, 5, 5, 5), (3, 2, 9, 7)])
def test_lrn_within_channel(K, case):
    planes, h, w, size = case
    x = (np.random.default_rng(3).standard_normal((1, planes, h, w)) * 3).astype(np.float32)
    xd = dev(x)
    yd = torch.full_like(xd, float("nan"))
    K.check_mc(K.LIB.mcLRNWithinChannel(fptr(xd), fptr(yd), planes, h, w, size, 0.5, 0.75, None))
    assert close(yd.cpu().numpy(), oracle.lrn(x, size, 0.5, 0.75, norm_region="WITHIN_CHANNEL"), 1e-5)


ARGMAX_CASES = [
    # shape, top_k, out_max_val, axis
    ((4, 1000), 1, False, None),
    ((4, 1000), 5, True, None),
    ((2, 21, 30, 40), 1, False, 1),       # segmentation argmax: many short lines
    ((2, 21, 30, 40), 3, True, 1),
    ((3, 7, 300), 4, False, 2),           # long lines, inner == 1
    ((2, 3000, 4), 2, False, 1),          # long strided lines: one workgroup each
    ((2, 5, 6), 30, True, None),          # top_k = whole flattened instance
    ((70, 33), 33, False, 1),
]


@pytest.mark.parametrize("shape,top_k,omv,axis", ARGMAX_CASES)
@pytest.mark.parametrize("ties", [False, True])
def test_argmax_indices_bit_exact(K, shape, top_k, omv, axis, ties):
    rng = np.random.default_rng(4)
    x = rng.standard_normal(shape).astype(np.float32)
    if ties:
        x = np.round(x * 2) / 2            # few distinct values: order among equals matters
    want = oracle.argmax(x, top_k, omv, axis)
    xd = dev(x)
    yd = torch.full(want.shape, float("nan"), device="cuda")
    if axis is None:
        outer, dim, inner, layout = shape[0], int(np.prod(shape[1:])), 1, 2 if omv else 0
    else:
        outer, dim, inner = int(np.prod(shape[:axis])), shape[axis], int(np.prod(shape[axis + 1:]))
        layout = 1 if omv else 0
    K.check_mc(K.LIB.mcArgMax(fptr(xd), fptr(yd), outer, dim, inner, top_k, layout, None))
    assert np.array_equal(yd.cpu().numpy(), want)


@pytest.mark.parametrize("num,dim", [(1, 100000), (7, 300), (2048, 9), (5, 1), (3000, 64)])
def test_reduction(K, num, dim):
    x = np.random.default_rng(5).standard_normal((num, dim)).astype(np.float32)
    xd = dev(x)
    for op, name in ((1, "SUM"), (2, "ASUM"), (3, "SUMSQ"), (4, "MEAN")):
        yd = torch.full((num,), float("nan"), device="cuda")
        K.check_mc(K.LIB.mcReduction(op, fptr(xd), fptr(yd), num, dim, 0.5, None))
        want = oracle.reduction(x, name, 1, 0.5)
        scale = np.abs(x).sum(axis=1).max() * (0.5 / dim if name == "MEAN" else 0.5)
        got = yd.cpu().numpy()
        if dim <= 300:
            assert np.abs(got - want).max() <= 1e-5 * max(scale, 1e-6), name
        # Long rows: the oracle adds in index order in fp32, as plain loops do, and drifts;
        # both are held against the float64 sum, the device's tree sum being the closer.
        x64 = x.astype(np.float64)
        exact = 0.5 * {"SUM": x64.sum(1), "ASUM": np.abs(x64).sum(1), "SUMSQ": (x64 ** 2).sum(1),
                       "MEAN": x64.mean(1)}[name]
        if name == "SUMSQ":
            scale = (x64 ** 2).sum(1).max() * 0.5
        assert np.abs(got - exact).max() <= 1e-5 * max(scale, 1e-6), name
        assert np.abs(got - exact).max() <= np.abs(want - exact).max() + 1e-6 * max(scale, 1e-6), name
    assert K.LIB.mcReduction(9, fptr(xd), fptr(xd), num, dim, 1.0, None) != 0


@pytest.mark.parametrize("num,dim,norm", [(6, 35, True), (2, 5000, True), (6, 35, False), (3, 1, True)])
def test_mvn(K, num, dim, norm):
    x = (np.random.default_rng(6).standard_normal((num, dim, 1, 1)) * 2 + 3).astype(np.float32)
    xd = dev(x)
    yd = torch.full_like(xd, float("nan"))
    K.check_mc(K.LIB.mcMVN(fptr(xd), fptr(yd), num, dim, int(norm), 0.1, None))
    want = oracle.mvn(x.reshape(1, num, dim, 1), norm, False, 0.1).reshape(x.shape)
    assert close(yd.cpu().numpy(), want, 1e-5)


def test_gather_rows_embed_and_out_of_range(K):
    rng = np.random.default_rng(7)
    w = rng.standard_normal((50, 33)).astype(np.float32)
    b = rng.standard_normal(33).astype(np.float32)
    idx = rng.integers(0, 50, 200).astype(np.float32)
    wd, bd, idd = dev(w), dev(b), dev(idx)
    yd = torch.full((200, 33), float("nan"), device="cuda")
    K.check_mc(K.LIB.mcGatherRows(fptr(wd), 50, 33, fptr(idd), 200, fptr(bd), fptr(yd), None))
    assert np.array_equal(yd.cpu().numpy(), oracle.embed(idx, w, b))
    K.check_mc(K.LIB.mcGatherRows(fptr(wd), 50, 33, fptr(idd), 200, None, fptr(yd), None))
    assert np.array_equal(yd.cpu().numpy(), w[idx.astype(int)])
    bad = dev(np.array([3, 50, -1, 0], np.float32))
    K.check_mc(K.LIB.mcGatherRows(fptr(wd), 50, 33, fptr(bad), 4, None, fptr(yd), None))
    got = yd[:4].cpu().numpy()
    assert np.array_equal(got[[0, 3]], w[[3, 0]]) and np.isnan(got[[1, 2]]).all()


def test_crop_and_tile_bit_exact(K):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 5, 9, 11)).astype(np.float32)
    xd = dev(x)
    arr = lambda v: (ctypes.c_int * len(v))(*v)
    for top, off in [((2, 5, 4, 6), (0, 0, 3, 2)), ((1, 2, 9, 11), (1, 3, 0, 0)), ((2, 5, 9, 11), (0, 0, 0, 0)),
                     ((2, 5, 1, 1), (0, 0, 8, 10))]:
        yd = torch.full(top, float("nan"), device="cuda")
        K.check_mc(K.LIB.mcCrop(fptr(xd), fptr(yd), 4, arr(x.shape), arr(top), arr(off), None))
        want = x[tuple(slice(o, o + t) for o, t in zip(off, top))]
        assert np.array_equal(yd.cpu().numpy(), want)
    yd = torch.empty((2, 5, 4, 6), device="cuda")
    assert K.LIB.mcCrop(fptr(xd), fptr(yd), 4, arr(x.shape), arr((2, 5, 4, 6)), arr((0, 0, 6, 0)), None) != 0
    assert "out-of-bounds" in K.LIB.mcLastError().decode()
    for axis, tiles in [(1, 3), (0, 2), (3, 4)]:
        shape = list(x.shape)
        shape[axis] *= tiles
        yd = torch.full(shape, float("nan"), device="cuda")
        K.check_mc(K.LIB.mcTile(fptr(xd), fptr(yd), int(np.prod(x.shape[:axis])),
                                int(np.prod(x.shape[axis:])), tiles, None))
        reps = [1] * 4
        reps[axis] = tiles
        assert np.array_equal(yd.cpu().numpy(), np.tile(x, reps))
