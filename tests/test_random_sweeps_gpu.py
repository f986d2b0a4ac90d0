"""Seeded random sweeps of the kernel-level C ABI against the oracle: geometries and
parameter combinations nobody wrote down by hand (the hand-picked cases live in
test_kernels_gpu.py).  Every sweep is deterministic and takes about a second."""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from oracle import netrun

import test_kernels_gpu as T
from test_kernels_gpu import K  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu
dev, fptr = T.dev, T.fptr


def test_random_convolutions(K):
    """Convolution / Deconvolution with random extents, kernel, stride, pad, dilation and
    groups (depthwise included), random tile configuration and K slices (3x3 stride-1 cases
    left to the automatic choice run on the Winograd path half of the time), and a random
    epilogue (scale, shift, residual, ReLU / leaky ReLU / TanH)."""
    rng = np.random.default_rng(2024)
    done = 0
    for _ in range(260):
        tr = bool(rng.integers(0, 4) == 0)
        g = int(rng.choice([1, 1, 1, 2, 4]))
        cin, cout = g * int(rng.integers(1, 20)), g * int(rng.integers(1, 40))
        if rng.integers(0, 6) == 0:
            cin = cout = g = int(rng.integers(2, 24))      # depthwise
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        if rng.integers(0, 3) == 0:
            kw = kh
        if rng.integers(0, 5) == 0:
            kh = kw = 3
        sh, sw = (1, 1) if rng.integers(0, 3) == 0 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        dh, dw = (int(rng.integers(1, 3)), int(rng.integers(1, 3))) if rng.integers(0, 4) == 0 else (1, 1)
        ph, pw = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        h, w = int(rng.integers(1, 30)), int(rng.integers(1, 30))
        n = int(rng.integers(1, 6))
        if tr:
            ho, wo = sh * (h - 1) + dh * (kh - 1) + 1 - 2 * ph, sw * (w - 1) + dw * (kw - 1) + 1 - 2 * pw
        else:
            ho = (h + 2 * ph - dh * (kh - 1) - 1) // sh + 1 if h + 2 * ph - dh * (kh - 1) - 1 >= 0 else 0
            wo = (w + 2 * pw - dw * (kw - 1) - 1) // sw + 1 if w + 2 * pw - dw * (kw - 1) - 1 >= 0 else 0
        if ho <= 0 or wo <= 0:
            continue
        geom = (cin, h, w, cout, (kh, kw), (sh, sw), (ph, pw), (dh, dw), g, tr)
        x = rng.standard_normal((n, cin, h, w)).astype(np.float32)
        wshape = (cin, cout // g, kh, kw) if tr else (cout, cin // g, kh, kw)
        wt = (rng.standard_normal(wshape) * 0.2).astype(np.float32)
        b = rng.standard_normal(cout).astype(np.float32)
        sc = (rng.random(cout) + 0.5).astype(np.float32)
        y = oracle.conv_forward(oracle.conv_geom(*geom), x, wt, None)
        use_res = bool(rng.integers(0, 2))
        act = int(rng.choice([K.ACT_NONE, K.ACT_RELU, K.ACT_RELU, K.ACT_TANH]))
        slope = float(rng.choice([0.0, 0.0, 0.1]))
        res = rng.standard_normal(y.shape).astype(np.float32)
        want = oracle.scale(y, sc, b)
        if use_res:
            want = oracle.eltwise([want, res], "SUM")
        if act == K.ACT_RELU:
            want = oracle.relu(want, slope)
        elif act == K.ACT_TANH:
            want = oracle.tanh(want)
        plan = K.ConvPlan(K.conv_geom(*geom))
        slices, config = int(rng.choice([0, 0, 1, 2, 3, 7])), int(rng.choice([-1, -1, 0, 1, 2, 3, 4, 5, 6, 7]))
        plan.force_split(slices)
        plan.force_config(config)
        if (kh, kw, sh, sw, dh, dw, g, tr) == (3, 3, 1, 1, 1, 1, 1, False) and slices == 0 and config == -1:
            plan.force_winograd(int(rng.integers(0, 2)))
        ep = dict(scale=sc, shift=b, activation=act, negative_slope=slope)
        if use_res:
            ep["residual"] = res
        got = T._run_plan(K, plan, n, x, wt, want.shape, **ep)
        # absolute against the largest pre-activation value: TanH squeezes a sum of
        # hundreds of products into [-1, 1] without shrinking its rounding noise
        scale_of_sums = max(1.0, float(np.abs(y).max()))
        assert np.abs(got - want).max() < 3e-6 * scale_of_sums + 1e-6, (geom, n, slices, config, act, use_res)
        done += 1
    assert done > 200


def test_random_pooling_permute_normalize(K):
    rng = np.random.default_rng(77)
    for _ in range(200):
        method = str(rng.choice(["MAX", "AVE"]))
        hh, ww = int(rng.integers(1, 40)), int(rng.choice([1, 2, 3, 4, 7, 8, 12, 13, 16, 20, 28, 33]))
        k, s = int(rng.integers(1, 5)), int(rng.integers(1, 4))
        p = int(rng.integers(0, k))
        n, c = int(rng.integers(1, 4)), int(rng.integers(1, 7))
        x = rng.standard_normal((n, c, hh, ww)).astype(np.float32)
        try:
            want = oracle.pooling(x, method, (k, k), (s, s), (p, p))
        except ValueError:
            continue   # window larger than the padded map: no output
        if want.size == 0:
            continue
        xd, yd = dev(x), torch.full(want.shape, float("nan"), device="cuda")
        K.check_mc(K.LIB.mcPooling(0 if method == "MAX" else 1, fptr(xd), fptr(yd), n * c, hh, ww, k, k, s, s,
                                   p, p, None))
        torch.cuda.synchronize()
        got = yd.cpu().numpy()
        # (an unpadded window that starts past the map is empty: -FLT_MAX, or 0 / 0 = NaN for AVE,
        # as pooling_layer.cpp:141-177 computes it)
        if method == "MAX":
            assert np.array_equal(got, want), (method, hh, ww, k, s, p)
        else:
            assert np.allclose(got, want, rtol=0, atol=1e-5, equal_nan=True), (method, hh, ww, k, s, p)
    for _ in range(200):
        nd = int(rng.integers(2, 5))
        shape = tuple(int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 19, 33, 64, 68])) for _ in range(nd))
        if np.prod(shape) > 2_000_000:
            continue
        order = tuple(int(v) for v in rng.permutation(nd))
        x = rng.standard_normal(shape).astype(np.float32)
        want = np.ascontiguousarray(np.transpose(x, order))
        xd, yd = dev(x), torch.full(want.shape, float("nan"), device="cuda")
        K.check_mc(K.LIB.mcPermute(fptr(xd), fptr(yd), nd, (ctypes.c_int * nd)(*shape), (ctypes.c_int * nd)(*order),
                                   None))
        torch.cuda.synchronize()
        assert np.array_equal(yd.cpu().numpy(), want), (shape, order)
    for _ in range(100):
        n, c = int(rng.integers(1, 4)), int(rng.choice([1, 3, 12, 64, 129, 512, 515]))
        hh, ww = int(rng.integers(1, 12)), int(rng.integers(1, 12))
        x = rng.standard_normal((n, c, hh, ww)).astype(np.float32)
        across, shared = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        s = (rng.random(1 if shared else c) + 0.5).astype(np.float32)
        want = oracle.normalize(x, s, bool(across), bool(shared), 1e-10)
        xd, sd, yd = dev(x), dev(s), torch.full(x.shape, float("nan"), device="cuda")
        K.check_mc(K.LIB.mcNormalize(fptr(xd), fptr(yd), n, c, hh * ww, across, shared, ctypes.c_float(1e-10),
                                     fptr(sd), None))
        torch.cuda.synchronize()
        assert np.abs(yd.cpu().numpy() - want).max() < 1e-6, (n, c, hh, ww, across, shared)


def test_random_proposals(K):
    """Map sizes, pre / post_nms_topn around the scan's 512-box super-blocks, thresholds
    from 0.05 to 0.99, tight and loose boxes, with and without equal scores."""
    rng = np.random.default_rng(123)
    for case in range(120):
        H, W = int(rng.integers(3, 45)), int(rng.integers(3, 64))
        A = 9
        n = A * H * W
        pre = int(rng.choice([64, 300, 511, 512, 513, 1000, 2000, 6000, 12000]))
        post = int(rng.choice([1, 37, 64, 300, 700, 2000, 5000]))
        thr = float(rng.choice([0.05, 0.3, 0.5, 0.7, 0.9, 0.99]))
        spread = float(rng.choice([0.05, 0.3, 1.0]))
        quant = int(rng.choice([0, 0, 0, 50, 3000]))
        scores = rng.random((1, 2 * A, H, W)).astype(np.float32)
        scores[0, A:] = (rng.permutation(n).astype(np.float32) / n * 0.9 + 0.05).reshape(A, H, W)
        if quant:
            scores[0, A:] = np.round(scores[0, A:] * quant) / quant
        bbox = (rng.standard_normal((1, 4 * A, H, W)) * spread).astype(np.float32)
        im_info = np.array([H * 16, W * 16, 1.0], np.float32)
        param = {"pre_nms_topn": pre, "post_nms_topn": post, "nms_thresh": thr}
        want_rois, want_scores = oracle.proposal(param, scores, bbox, im_info, 2)
        rois, rs, _, _ = T.run_proposal(K, scores, bbox, im_info, param, ("both", "steps", "rest")[case % 3])
        assert np.array_equal(rois, want_rois) and np.array_equal(rs, want_scores), (H, W, pre, post, thr, spread, quant)


def test_random_detection_outputs(K):
    """All code types, shared and per-class boxes, any background label, keep_top_k from
    none to 0, top_k around the 64-candidate blocks and the 1024 cached boxes, adaptive eta."""
    rng = np.random.default_rng(321)
    for _ in range(110):
        num, P = int(rng.integers(1, 5)), int(rng.choice([40, 64, 65, 300, 1917, 3000, 8732]))
        C = int(rng.choice([2, 3, 5, 21]))
        share, code = bool(rng.integers(0, 2)), str(rng.choice(["CORNER", "CENTER_SIZE", "CORNER_SIZE"]))
        keep = int(rng.choice([-1, 0, 1, 10, 200, 1000]))
        thr = [None, 0.001, 0.01, 0.05, 0.3][int(rng.integers(0, 5))]
        nms, eta = float(rng.choice([0.05, 0.3, 0.45, 0.6, 0.95])), float(rng.choice([1.0, 1.0, 1.0, 0.9]))
        topk = [None, 1, 64, 65, 400, 1024, 1025][int(rng.integers(0, 7))]
        sigma = float(rng.choice([0.5, 1.0, 2.0]))
        bg = int(rng.choice([0, 0, 1, -1]))
        if bg == -1 and share:
            bg = 0          # that combination is an error (the reference aborts)
        lc = 1 if share else C
        loc = (rng.standard_normal((num, P * lc * 4)) * 0.5).astype(np.float32)
        conf = oracle.softmax((rng.standard_normal((num, P, C)) * sigma).astype(np.float32), 2).reshape(num, P * C)
        c = rng.random((P, 2)) * 0.8 + 0.1
        wh = rng.random((P, 2)) * 0.3 + 0.05
        prior = np.concatenate([np.concatenate([c - wh / 2, c + wh / 2], 1).reshape(-1),
                                np.tile([0.1, 0.1, 0.2, 0.2], P)]).reshape(1, 2, P * 4).astype(np.float32)
        param = {"num_classes": C, "share_location": share, "background_label_id": bg, "code_type": code,
                 "keep_top_k": keep, "nms_param": {"nms_threshold": nms, "eta": eta}}
        if thr is not None:
            param["confidence_threshold"] = thr
        if topk is not None:
            param["nms_param"]["top_k"] = topk
        want = oracle.detection_output(param, loc, conf, prior)
        got, flag = T.run_detection_output(K, param, loc, conf, prior)
        want_flag = T.cut_tie_expected(param, loc, conf, prior)
        case = (num, P, C, share, code, keep, thr, nms, eta, topk, sigma, bg)
        assert got.shape == want.shape and flag == want_flag, case
        if not want_flag:
            assert np.array_equal(got, want), case
        elif not (want_flag & 1):   # equal scores inside a kept label only: the same rows in some order
            assert np.array_equal(got[np.lexsort(got.T[::-1])], want[np.lexsort(want.T[::-1])]), case
