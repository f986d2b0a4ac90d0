"""Pins the CPU oracle (oracle/mc_oracle.c) before anything is checked against it.

Three kinds of evidence, chosen so that a dropped term, a wrong sign or index or
a transposed operand fails at least one:
  * bit equality with the reference's own compiled im2col / col2im / gemm / exp /
    powx (oracle/_ref, built from the reference checkout; skipped where absent);
  * float64 brute force written independently of the oracle's loop structure;
  * identities (adjointness of conv/deconv, 1x1 conv == matmul, softmax sums).
"""
import numpy as np
import pytest

import oracle
import ref_math

ref = pytest.mark.skipif(not ref_math.available(), reason="oracle/_ref not built (no reference checkout)")


def rng(seed):
    return np.random.default_rng(seed)


# ---- against the compiled reference ------------------------------------------

CONV_CASES = [
    # C, H, W, kh, kw, ph, pw, sh, sw, dh, dw
    (3, 7, 9, 3, 3, 1, 1, 1, 1, 1, 1),
    (2, 8, 8, 3, 2, 0, 1, 2, 1, 1, 1),
    (4, 11, 5, 3, 3, 2, 2, 1, 1, 2, 2),
    (1, 6, 6, 1, 1, 0, 0, 1, 1, 1, 1),
    (2, 9, 9, 5, 5, 2, 2, 3, 3, 1, 1),
    (3, 5, 5, 2, 2, 1, 1, 2, 2, 1, 1),
]


@ref
@pytest.mark.parametrize("case", CONV_CASES)
def test_im2col_matches_reference(case):
    lib = ref_math.load()
    C, H, W, kh, kw, ph, pw, sh, sw, dh, dw = case
    im = rng(1).standard_normal((C, H, W)).astype(np.float32)
    col = oracle.im2col(im, (kh, kw), (ph, pw), (sh, sw), (dh, dw))
    want = np.full_like(col, np.nan)
    lib.im2col(ref_math.p(im), C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, ref_math.p(want))
    assert np.array_equal(col, want)


@ref
@pytest.mark.parametrize("case", CONV_CASES)
def test_col2im_matches_reference(case):
    lib = ref_math.load()
    C, H, W, kh, kw, ph, pw, sh, sw, dh, dw = case
    Ho = (H + 2 * ph - (dh * (kh - 1) + 1)) // sh + 1
    Wo = (W + 2 * pw - (dw * (kw - 1) + 1)) // sw + 1
    col = rng(2).standard_normal((C * kh * kw, Ho, Wo)).astype(np.float32)
    im = oracle.col2im(col, C, H, W, (kh, kw), (ph, pw), (sh, sw), (dh, dw))
    want = np.full_like(im, np.nan)
    lib.col2im(ref_math.p(col), C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, ref_math.p(want))
    assert np.array_equal(im, want)


@ref
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_gemm_matches_reference_within_rounding(ta, tb):
    """caffe_cpu_gemm's argument convention (lda/ldb/ldc, transposes, alpha/beta)."""
    lib = ref_math.load()
    M, N, K = 7, 13, 11
    r = rng(3)
    A = r.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = r.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    C0 = r.standard_normal((M, N)).astype(np.float32)
    mine, theirs = C0.copy(), C0.copy()
    oracle.use_openblas(False)
    oracle.gemm(ta, tb, M, N, K, 0.75, A, B, -0.5, mine)
    lib.gemm(112 if ta else 111, 112 if tb else 111, M, N, K, 0.75, ref_math.p(A), ref_math.p(B),
             -0.5, ref_math.p(theirs))
    exact = 0.75 * ((A.T if ta else A).astype(np.float64) @ (B.T if tb else B).astype(np.float64)) \
        - 0.5 * C0
    assert np.abs(mine - exact).max() < 1e-5
    assert np.abs(theirs - exact).max() < 1e-5


@ref
def test_exp_powx_div_axpy_bit_exact():
    """The float overloads selected through <math.h> in mkl_alternate.hpp."""
    lib = ref_math.load()
    a = (rng(4).standard_normal(4096) * 3).astype(np.float32)
    want = np.empty_like(a)
    lib.exp(a.size, ref_math.p(a), ref_math.p(want))
    assert np.array_equal(oracle.exp(a), want)
    pos = np.abs(a) + 1e-3
    for b in (0.5, 2.0):
        lib.powx(pos.size, ref_math.p(pos), b, ref_math.p(want))
        assert np.array_equal(oracle.powx(pos, b), want)
    # eltwise SUM accumulates with axpy: y = a*x + y
    x = rng(5).standard_normal(1000).astype(np.float32)
    y = rng(6).standard_normal(1000).astype(np.float32)
    acc = np.zeros(1000, np.float32)
    lib.axpy(1000, 1.0, ref_math.p(x), ref_math.p(acc))
    lib.axpy(1000, 1.0, ref_math.p(y), ref_math.p(acc))
    assert np.array_equal(oracle.eltwise([x, y], "SUM"), acc)
    # scale layer multiplies with caffe_cpu_scale (copy + scal)
    out = np.empty_like(x)
    lib.scale(1000, 1.7, ref_math.p(x), ref_math.p(out))
    assert np.array_equal(oracle.scale(x.reshape(1, 1, 1000), np.array([1.7], np.float32)).ravel(),
                          out)


def test_blas_order_noise():
    """Two correct fp32 evaluations of config 1 that only differ in summation order
    (plain loops vs OpenBLAS) already disagree by more than 1e-4 of small outputs:
    this is why the parity metric floors the denominator at 1e-2 of the blob peak."""
    if oracle.find_openblas() is None:
        pytest.skip("no OpenBLAS to compare with")
    from oracle import netrun
    r = rng(0)
    x = r.standard_normal((1, 64, 56, 56)).astype(np.float32)
    w = (r.standard_normal((64, 64, 3, 3)) * np.sqrt(2 / 576)).astype(np.float32)
    g = oracle.conv_geom(64, 56, 56, 64, 3, 1, 1)
    oracle.use_openblas(False)
    a = oracle.conv_forward(g, x, w)
    oracle.use_openblas(True)
    b = oracle.conv_forward(g, x, w)
    oracle.use_openblas(False)
    assert netrun.rel_err(a, b, floor=1e-2) < 1e-4
    assert netrun.rel_err(a, b, floor=0.0) > 1e-4   # raw relative error is order-dominated


# ---- brute force and identities ------------------------------------------------

def brute_conv(x, w, b, stride, pad, dil, group):
    """Direct float64 sum over (ci, i, j) per output, written with explicit loops."""
    N, Cin, H, W = x.shape
    Cout, Cg, kh, kw = w.shape
    Ho = (H + 2 * pad[0] - (dil[0] * (kh - 1) + 1)) // stride[0] + 1
    Wo = (W + 2 * pad[1] - (dil[1] * (kw - 1) + 1)) // stride[1] + 1
    y = np.zeros((N, Cout, Ho, Wo))
    og = Cout // group
    for n in range(N):
        for co in range(Cout):
            g = co // og
            for ho in range(Ho):
                for wo in range(Wo):
                    s = 0.0
                    for ci in range(Cg):
                        for i in range(kh):
                            for j in range(kw):
                                h = ho * stride[0] - pad[0] + i * dil[0]
                                ww = wo * stride[1] - pad[1] + j * dil[1]
                                if 0 <= h < H and 0 <= ww < W:
                                    s += float(x[n, g * Cg + ci, h, ww]) * float(w[co, ci, i, j])
                    y[n, co, ho, wo] = s + (float(b[co]) if b is not None else 0.0)
    return y


@pytest.mark.parametrize("cin,cout,k,s,p,d,g", [
    (4, 6, (3, 3), (1, 1), (1, 1), (1, 1), 1),
    (4, 6, (3, 2), (2, 1), (0, 1), (1, 1), 2),
    (3, 5, (3, 3), (1, 1), (2, 2), (2, 2), 1),
    (6, 6, (1, 1), (2, 2), (0, 0), (1, 1), 3),
    (2, 4, (5, 5), (3, 3), (2, 2), (1, 1), 1),
])
def test_conv_brute_force(cin, cout, k, s, p, d, g):
    oracle.use_openblas(False)
    r = rng(7)
    x = r.standard_normal((2, cin, 7, 8)).astype(np.float32)
    w = r.standard_normal((cout, cin // g) + k).astype(np.float32)
    b = r.standard_normal(cout).astype(np.float32)
    got = oracle.conv_forward(oracle.conv_geom(cin, 7, 8, cout, k, s, p, d, g), x, w, b)
    want = brute_conv(x, w, b, s, p, d, g)
    assert got.shape == want.shape
    assert np.abs(got - want).max() < 1e-4


def test_conv_1x1_is_matmul_and_identity_kernel():
    oracle.use_openblas(False)
    r = rng(8)
    x = r.standard_normal((2, 5, 4, 3)).astype(np.float32)
    w = r.standard_normal((7, 5, 1, 1)).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(5, 4, 3, 7, 1), x, w)
    want = np.einsum("oc,nchw->nohw", w[:, :, 0, 0].astype(np.float64), x.astype(np.float64))
    assert np.abs(y - want).max() < 1e-5
    # a centred delta filter per channel reproduces the input
    wd = np.zeros((5, 5, 3, 3), np.float32)
    for c in range(5):
        wd[c, c, 1, 1] = 1
    assert np.array_equal(oracle.conv_forward(oracle.conv_geom(5, 4, 3, 5, 3, 1, 1), x, wd), x)


@pytest.mark.parametrize("cin,cout,k,s,p,d,g", [
    (4, 6, 4, 2, 1, 1, 1), (4, 6, 3, 1, 1, 1, 2), (3, 3, 2, 3, 0, 1, 1), (4, 2, 3, 2, 1, 2, 1),
])
def test_deconv_is_adjoint_of_conv(cin, cout, k, s, p, d, g):
    """<conv_W(u), v> == <u, deconv_W(v)> for the same weight blob: Deconvolution with
    weights [Cin_d, Cout_d/g, k, k] is the transpose of the Convolution Cout_d -> Cin_d."""
    oracle.use_openblas(False)
    r = rng(9)
    h, w_ = 5, 6
    gd = oracle.conv_geom(cin, h, w_, cout, k, s, p, d, g, True)
    Ho, Wo = oracle.conv_output_shape(gd)
    W = r.standard_normal((cin, cout // g, k, k)).astype(np.float32)
    v = r.standard_normal((1, cin, h, w_)).astype(np.float32)
    u = r.standard_normal((1, cout, Ho, Wo)).astype(np.float32)
    dv = oracle.conv_forward(gd, v, W)
    gc = oracle.conv_geom(cout, Ho, Wo, cin, k, s, p, d, g, False)
    assert oracle.conv_output_shape(gc) == (h, w_)
    cu = oracle.conv_forward(gc, u, W)
    lhs = float((cu.astype(np.float64) * v).sum())
    rhs = float((u.astype(np.float64) * dv).sum())
    assert abs(lhs - rhs) < 1e-3 * max(1.0, abs(lhs))


def test_deconv_matches_torch():
    torch = pytest.importorskip("torch")
    oracle.use_openblas(False)
    r = rng(10)
    x = r.standard_normal((2, 8, 4, 4)).astype(np.float32)
    W = r.standard_normal((8, 3, 4, 4)).astype(np.float32)
    b = r.standard_normal(6).astype(np.float32)
    y = oracle.conv_forward(oracle.conv_geom(8, 4, 4, 6, 4, 2, 1, 1, 2, True), x, W, b)
    want = torch.nn.functional.conv_transpose2d(
        torch.from_numpy(x).double(), torch.from_numpy(W).double(), torch.from_numpy(b).double(),
        stride=2, padding=1, groups=2).numpy()
    assert y.shape == want.shape == (2, 6, 8, 8)
    assert np.abs(y - want).max() < 1e-4


def test_inner_product():
    oracle.use_openblas(False)
    r = rng(11)
    x = r.standard_normal((5, 3, 2, 2)).astype(np.float32)
    W = r.standard_normal((7, 12)).astype(np.float32)
    b = r.standard_normal(7).astype(np.float32)
    want = x.reshape(5, 12).astype(np.float64) @ W.T + b
    assert np.abs(oracle.inner_product(x, W, b) - want).max() < 1e-5
    assert np.abs(oracle.inner_product(x, np.ascontiguousarray(W.T), b, transpose=True) - want).max() < 1e-5


def test_batch_norm_closed_forms():
    r = rng(12)
    x = r.standard_normal((3, 4, 5, 2)).astype(np.float32)
    mean_sum = r.standard_normal(4).astype(np.float32)
    var_sum = (r.random(4) + 0.5).astype(np.float32)
    factor = np.array([2.5], np.float32)
    y = oracle.batch_norm(x, mean_sum, var_sum, factor, True, 1e-3)
    m = (mean_sum / 2.5).reshape(1, 4, 1, 1).astype(np.float64)
    v = (var_sum / 2.5).reshape(1, 4, 1, 1).astype(np.float64)
    assert np.abs(y - (x - m) / np.sqrt(v + 1e-3)).max() < 1e-5
    # a zero moving-average factor zeroes the statistics (batch_norm_layer.cpp:85-90)
    y0 = oracle.batch_norm(x, mean_sum, var_sum, np.zeros(1, np.float32), True, 1e-3)
    assert np.abs(y0 - x / np.sqrt(1e-3)).max() < 1e-3
    # batch statistics: biased variance over (n, h, w)
    yb = oracle.batch_norm(x, mean_sum, var_sum, factor, False, 1e-5)
    mu = x.astype(np.float64).mean(axis=(0, 2, 3), keepdims=True)
    var = x.astype(np.float64).var(axis=(0, 2, 3), keepdims=True)
    assert np.abs(yb - (x - mu) / np.sqrt(var + 1e-5)).max() < 1e-5


def test_scale_bias_relu_tanh_sigmoid():
    r = rng(13)
    x = r.standard_normal((2, 3, 4, 5)).astype(np.float32)
    g = r.standard_normal(3).astype(np.float32)
    b = r.standard_normal(3).astype(np.float32)
    assert np.allclose(oracle.scale(x, g, b), x * g.reshape(1, 3, 1, 1) + b.reshape(1, 3, 1, 1),
                       atol=1e-6)
    assert np.allclose(oracle.bias(x, b), x + b.reshape(1, 3, 1, 1), atol=1e-6)
    assert np.array_equal(oracle.relu(x), np.maximum(x, 0))
    assert np.allclose(oracle.relu(x, 0.1), np.where(x > 0, x, 0.1 * x), atol=1e-7)
    # |slope| < 1e-6 counts as zero (relu_layer.cpp:18)
    assert np.array_equal(oracle.relu(x, 1e-7), np.maximum(x, 0))
    assert np.allclose(oracle.tanh(x), np.tanh(x.astype(np.float64)), atol=1e-7)
    assert np.allclose(oracle.sigmoid(x), 1 / (1 + np.exp(-x.astype(np.float64))), atol=1e-7)


def brute_pool(x, method, k, s, p):
    N, C, H, W = x.shape
    ho = int(np.ceil((H + 2 * p[0] - k[0]) / s[0])) + 1
    wo = int(np.ceil((W + 2 * p[1] - k[1]) / s[1])) + 1
    if p[0] or p[1]:
        if (ho - 1) * s[0] >= H + p[0]:
            ho -= 1
        if (wo - 1) * s[1] >= W + p[1]:
            wo -= 1
    y = np.zeros((N, C, ho, wo))
    for i in range(ho):
        for j in range(wo):
            h0, w0 = i * s[0] - p[0], j * s[1] - p[1]
            if method == "MAX":
                win = x[:, :, max(h0, 0):min(h0 + k[0], H), max(w0, 0):min(w0 + k[1], W)]
                y[:, :, i, j] = win.max(axis=(2, 3))
            else:
                h1, w1 = min(h0 + k[0], H + p[0]), min(w0 + k[1], W + p[1])
                area = (h1 - h0) * (w1 - w0)   # padded extent, not the valid count
                win = x[:, :, max(h0, 0):min(h1, H), max(w0, 0):min(w1, W)]
                y[:, :, i, j] = win.astype(np.float64).sum(axis=(2, 3)) / area
    return y


@pytest.mark.parametrize("method", ["MAX", "AVE"])
@pytest.mark.parametrize("hw,k,s,p", [
    ((112, 112), (3, 3), (2, 2), (0, 0)),   # ResNet pool1: ceil mode gives 56
    ((75, 75), (2, 2), (2, 2), (0, 0)),     # SSD pool3: 75 -> 38 needs ceil
    ((19, 19), (3, 3), (1, 1), (1, 1)),     # SSD pool5
    ((7, 9), (3, 2), (2, 3), (1, 1)),
    ((6, 6), (2, 2), (2, 2), (1, 1)),       # last window clipped away
])
def test_pooling_brute_force(method, hw, k, s, p):
    x = rng(14).standard_normal((2, 3) + hw).astype(np.float32)
    got = oracle.pooling(x, method, k, s, p)
    want = brute_pool(x, method, k, s, p)
    assert got.shape == want.shape
    assert np.abs(got - want).max() < 1e-5


def test_pooling_known_shapes_and_global():
    assert oracle.pooling_output_shape(112, 112, (3, 3), (2, 2), (0, 0)) == (56, 56)
    assert oracle.pooling_output_shape(75, 75, (2, 2), (2, 2), (0, 0)) == (38, 38)
    assert oracle.pooling_output_shape(19, 19, (3, 3), (1, 1), (1, 1)) == (19, 19)
    x = rng(15).standard_normal((2, 4, 7, 7)).astype(np.float32)
    assert np.allclose(oracle.pooling(x, "AVE", (0, 0), global_pooling=True)[:, :, 0, 0],
                       x.mean(axis=(2, 3)), atol=1e-6)


def test_eltwise_and_softmax():
    r = rng(16)
    a, b, c = (r.standard_normal((2, 3, 4)).astype(np.float32) for _ in range(3))
    assert np.allclose(oracle.eltwise([a, b, c], "SUM", [1, -2, 0.5]), a - 2 * b + 0.5 * c, atol=1e-6)
    assert np.allclose(oracle.eltwise([a, b, c], "PROD"), a * b * c, atol=1e-6)
    assert np.array_equal(oracle.eltwise([a, b, c], "MAX"), np.maximum(np.maximum(a, b), c))
    for axis in (1, 2, -1):
        y = oracle.softmax(a * 5, axis)
        e = np.exp((a * 5 - (a * 5).max(axis=axis, keepdims=True)).astype(np.float64))
        assert np.allclose(y, e / e.sum(axis=axis, keepdims=True), atol=1e-6)
        assert np.allclose(y.sum(axis=axis), 1, atol=1e-6)
