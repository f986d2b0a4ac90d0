"""Pins the oracle of the less common layers (oracle/mc_oracle_zoo.c) with evidence
that does not come from the oracle itself: float64 closed forms in numpy, torch
library routines, brute force over windows, and defining invariants."""
import numpy as np
import pytest

import oracle


def rng(seed):
    return np.random.default_rng(seed)


def close(got, want, tol=1e-6):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    return np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max())


def test_bn_is_affine_in_stored_multiplier():
    r = rng(0)
    x = r.standard_normal((3, 5, 4, 6)).astype(np.float32)
    slope, bias, mean = (r.standard_normal(5).astype(np.float32) for _ in range(3))
    mult = (r.random(5) + 0.5).astype(np.float32)
    got = oracle.bn(x, slope, bias, mean, mult)
    c = lambda a: a.astype(np.float64).reshape(1, 5, 1, 1)
    want = (x.astype(np.float64) - c(mean)) * c(mult) * c(slope) + c(bias)
    assert close(got, want)
    # not BatchNorm's 1/sqrt(var + eps): with mult = 4 the output scales by 4, not 1/2
    four = oracle.bn(x, np.ones(5), np.zeros(5), np.zeros(5), np.full(5, 4.0))
    assert np.array_equal(four, x * 4)


def test_conv_dw_against_torch_and_grouped_oracle():
    import torch
    r = rng(1)
    for (C, H, W, k, s, p, d, with_bias) in [(6, 9, 11, 3, 1, 1, 1, True), (4, 12, 10, 3, 2, 1, 1, False),
                                             (5, 13, 9, (3, 5), (2, 1), (1, 2), (2, 1), True)]:
        kh, kw = (k, k) if np.isscalar(k) else k
        x = r.standard_normal((2, C, H, W)).astype(np.float32)
        w = r.standard_normal((C, 1, kh, kw)).astype(np.float32)
        b = r.standard_normal(C).astype(np.float32) if with_bias else None
        got = oracle.conv_dw(x, w, b, s, p, d)
        want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                                          torch.from_numpy(b).double() if with_bias else None,
                                          stride=s, padding=p, dilation=d, groups=C).numpy()
        assert close(got, want, 1e-5)
        g = oracle.conv_geom(C, H, W, C, (kh, kw), s, p, d, C)
        assert close(got, oracle.conv_forward(g, x, w, b), 1e-5)


def test_power_closed_forms_and_constant_cases():
    r = rng(2)
    x = (r.random(1000) * 3 + 0.1).astype(np.float32)
    assert close(oracle.power(x, 0.5, 2.0, 1.0), np.sqrt(1.0 + 2.0 * x.astype(np.float64)))
    assert np.array_equal(oracle.power(x, 1.0, 1.0, 0.0), x)
    assert close(oracle.power(x, 2.0), x.astype(np.float64) ** 2)
    assert close(oracle.power(x, -0.75, 1e-2, 1.0), (1 + 1e-2 * x.astype(np.float64)) ** -0.75)
    # scale 0 -> shift^power everywhere; power 0 -> 1 everywhere
    assert np.array_equal(oracle.power(x, 2.0, 0.0, 3.0), np.full_like(x, 9.0))
    assert np.array_equal(oracle.power(x, 0.0, 5.0, 3.0), np.ones_like(x))


def test_exp_and_log_with_bases():
    r = rng(3)
    x = r.standard_normal(500).astype(np.float32)
    x64 = x.astype(np.float64)
    assert close(oracle.exp_layer(x), np.exp(x64))
    assert close(oracle.exp_layer(x, base=2.0, scale=0.5, shift=3.0), 2.0 ** (3.0 + 0.5 * x64), 1e-5)
    assert close(oracle.exp_layer(x, scale=-2.0, shift=1.0), np.exp(1.0 - 2.0 * x64), 1e-5)
    pos = (r.random(500) * 10 + 0.01).astype(np.float32)
    assert close(oracle.log_layer(pos), np.log(pos.astype(np.float64)))
    assert close(oracle.log_layer(pos, base=10.0, scale=2.0, shift=1.0),
                 np.log10(1.0 + 2.0 * pos.astype(np.float64)), 1e-5)
    # exp and log with the same base undo each other
    assert close(oracle.log_layer(oracle.exp_layer(x, base=3.0), base=3.0), x64, 1e-5)


def test_simple_unary_closed_forms():
    r = rng(4)
    x = (r.standard_normal(2000) * 5).astype(np.float32)
    x[:4] = [0.0, -0.0, 40.0, -40.0]
    x64 = x.astype(np.float64)
    assert np.array_equal(oracle.absval(x), np.abs(x))
    assert close(oracle.bnll(x), np.logaddexp(0.0, x64))
    assert close(oracle.elu(x, 1.5), np.where(x64 > 0, x64, 1.5 * np.expm1(np.minimum(x64, 0))))
    assert np.array_equal(oracle.threshold(x, 0.5), (x > 0.5).astype(np.float32))
    assert np.array_equal(oracle.threshold(np.array([0.5], np.float32), 0.5), [0.0])  # strict


def test_prelu_per_channel_and_shared():
    r = rng(5)
    x = r.standard_normal((2, 4, 3, 5)).astype(np.float32)
    slope = r.standard_normal(4).astype(np.float32)
    want = np.where(x > 0, x, x * slope.reshape(1, 4, 1, 1))
    assert np.array_equal(oracle.prelu(x, slope), want.astype(np.float32))
    assert np.array_equal(oracle.prelu(x, [0.25], True), np.where(x > 0, x, x * np.float32(0.25)))


def lrn_brute(x, size, alpha, beta, k, within):
    x = x.astype(np.float64)
    N, C, H, W = x.shape
    pre = (size - 1) // 2
    y = np.empty_like(x)
    if not within:
        for c in range(C):
            lo, hi = max(0, c - pre), min(C, c + size - pre)
            s = (x[:, lo:hi] ** 2).sum(axis=1)
            y[:, c] = x[:, c] * (k + alpha / size * s) ** -beta
        return y
    for h in range(H):
        for w in range(W):
            hs, ws = h - pre, w - pre
            he, we = min(hs + size, H + pre), min(ws + size, W + pre)
            area = (he - hs) * (we - ws)            # counts the padding
            s = (x[:, :, max(hs, 0):min(he, H), max(ws, 0):min(we, W)] ** 2).sum(axis=(2, 3))
            y[:, :, h, w] = x[:, :, h, w] * (1 + alpha * s / area) ** -beta
    return y


@pytest.mark.parametrize("size,C", [(5, 16), (3, 4), (7, 5), (1, 3)])
def test_lrn_across_channels_brute_force(size, C):
    x = (rng(6).standard_normal((2, C, 4, 5)) * 3).astype(np.float32)
    got = oracle.lrn(x, size, 1e-1, 0.75, 2.0)
    assert close(got, lrn_brute(x, size, 1e-1, 0.75, 2.0, False), 1e-5)


@pytest.mark.parametrize("size", [3, 5])
def test_lrn_within_channel_brute_force(size):
    x = (rng(7).standard_normal((2, 3, 7, 6)) * 3).astype(np.float32)
    got = oracle.lrn(x, size, 0.5, 0.75, norm_region="WITHIN_CHANNEL")
    assert close(got, lrn_brute(x, size, 0.5, 0.75, 1.0, True), 1e-5)


def test_argmax_layouts_and_ties():
    r = rng(8)
    x = r.permutation(2 * 3 * 4 * 5).reshape(2, 3, 4, 5).astype(np.float32)
    # no axis: flattened per instance
    flat = x.reshape(2, -1)
    order = np.argsort(-flat, axis=1)[:, :4]
    got = oracle.argmax(x, 4)
    assert got.shape == (2, 1, 4, 1) and np.array_equal(got.reshape(2, 4), order)
    both = oracle.argmax(x, 4, out_max_val=True)
    assert both.shape == (2, 2, 4, 1)
    assert np.array_equal(both[:, 0, :, 0], order)
    assert np.array_equal(both[:, 1, :, 0], np.take_along_axis(flat, order, 1))
    # along an axis
    got = oracle.argmax(x, 2, axis=1)
    assert got.shape == (2, 2, 4, 5)
    assert np.array_equal(got, np.argsort(-x, axis=1)[:, :2].astype(np.float32))
    vals = oracle.argmax(x, 2, out_max_val=True, axis=-1)
    assert np.array_equal(vals, -np.sort(-x, axis=-1)[..., :2])
    # ties: std::greater on (value, index) pairs puts the larger index first
    t = np.array([[1, 3, 3, 2, 3]], np.float32)
    assert np.array_equal(oracle.argmax(t, 4).reshape(-1), [4, 2, 1, 3])


def test_reduction_ops():
    r = rng(9)
    x = r.standard_normal((3, 4, 50)).astype(np.float32)
    x64 = x.astype(np.float64)
    assert close(oracle.reduction(x, "SUM", 1), x64.sum(axis=(1, 2)), 1e-5)
    assert close(oracle.reduction(x, "ASUM", 2, 0.5), 0.5 * np.abs(x64).sum(axis=2), 1e-5)
    assert close(oracle.reduction(x, "SUMSQ", -1), (x64 ** 2).sum(axis=2), 1e-5)
    assert close(oracle.reduction(x, "MEAN", 1, 3.0), 3.0 * x64.mean(axis=(1, 2)), 1e-5)
    assert oracle.reduction(x, "SUM", 0).shape == ()


def test_mvn_eps_outside_the_root():
    r = rng(10)
    x = (r.standard_normal((2, 3, 4, 5)) * 2 + 1).astype(np.float32)
    x64 = x.astype(np.float64)
    m = x64.mean(axis=(2, 3), keepdims=True)
    sd = np.sqrt(((x64 - m) ** 2).mean(axis=(2, 3), keepdims=True))
    assert close(oracle.mvn(x, eps=0.5), (x64 - m) / (sd + 0.5), 1e-5)
    assert close(oracle.mvn(x, normalize_variance=False), x64 - m, 1e-5)
    ma = x64.mean(axis=(1, 2, 3), keepdims=True)
    sda = np.sqrt(((x64 - ma) ** 2).mean(axis=(1, 2, 3), keepdims=True))
    assert close(oracle.mvn(x, across_channels=True), (x64 - ma) / (sda + 1e-9), 1e-5)


def test_embed_rows_plus_bias():
    r = rng(11)
    w = r.standard_normal((7, 4)).astype(np.float32)
    b = r.standard_normal(4).astype(np.float32)
    idx = r.integers(0, 7, (3, 5)).astype(np.float32)
    got = oracle.embed(idx, w, b)
    assert got.shape == (3, 5, 4)
    assert np.array_equal(got, w[idx.astype(int)] + b)
    assert np.array_equal(oracle.embed(idx, w), w[idx.astype(int)])


def test_shuffle_channel_is_a_transposition():
    x = rng(12).standard_normal((2, 12, 3, 2)).astype(np.float32)
    got = oracle.shuffle_channel(x, 3)
    want = x.reshape(2, 3, 4, 3, 2).transpose(0, 2, 1, 3, 4).reshape(x.shape)
    assert np.array_equal(got, want)
    assert np.array_equal(oracle.shuffle_channel(got, 4), x)
    assert np.array_equal(oracle.shuffle_channel(x, 1), x)


def test_spp_levels_are_block_maxima():
    x = rng(13).standard_normal((2, 3, 8, 8)).astype(np.float32)
    got = oracle.spp(x, 3)
    assert got.shape == (2, 3 * (1 + 4 + 16))
    l0 = x.max(axis=(2, 3)).reshape(2, -1)
    l1 = x.reshape(2, 3, 2, 4, 2, 4).max(axis=(3, 5)).reshape(2, -1)
    l2 = x.reshape(2, 3, 4, 2, 4, 2).max(axis=(3, 5)).reshape(2, -1)
    assert np.array_equal(got, np.concatenate([l0, l1, l2], axis=1))
    ave = oracle.spp(x, 2, "AVE")
    assert close(ave[:, :3], x.astype(np.float64).mean(axis=(2, 3)), 1e-6)
    assert oracle.spp(x, 1).shape == (2, 3, 1, 1)
