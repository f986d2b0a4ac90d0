"""Pins the detection-tail oracle (oracle/mc_oracle_det.cc) with evidence that does
not come from the oracle itself: published anchor tables, float64 closed forms,
brute-force greedy NMS, and the defining invariants of NMS and of a partial sort."""
import numpy as np
import pytest

import oracle


def rng(seed):
    return np.random.default_rng(seed)


def test_anchor_table_is_py_faster_rcnn():
    """generate_anchors(base 16, ratios .5/1/2, scales 8/16/32) of py-faster-rcnn."""
    want = np.array([[-84, -40, 99, 55], [-176, -88, 191, 103], [-360, -184, 375, 199],
                     [-56, -56, 71, 71], [-120, -120, 135, 135], [-248, -248, 263, 263],
                     [-36, -80, 51, 95], [-80, -168, 95, 183], [-168, -344, 183, 359]], np.float32)
    assert np.array_equal(oracle.generate_anchors(16, (0.5, 1, 2), (8, 16, 32)), want)


def test_proposal_decode_closed_form():
    r = rng(1)
    A, H, W = 9, 6, 7
    anchors = oracle.generate_anchors()
    fg = r.random((A, H, W)).astype(np.float32)
    bbox = (r.standard_normal((4 * A, H, W)) * 0.2).astype(np.float32)
    im_h, im_w = 2000.0, 2000.0      # far away: no clipping except at 0
    props = oracle.generate_proposals(fg, bbox, anchors, im_h, im_w, 16.0, 16)
    assert props.shape == (A * H * W, 5)
    for h, w, k in [(0, 0, 0), (3, 4, 5), (5, 6, 8), (2, 1, 3)]:
        i = (h * W + w) * A + k          # order h, w, anchor
        a = anchors[k].astype(np.float64) + np.array([w * 16, h * 16, w * 16, h * 16])
        aw, ah = a[2] - a[0] + 1, a[3] - a[1] + 1
        cx, cy = a[0] + 0.5 * aw, a[1] + 0.5 * ah
        dx, dy, dw, dh = (float(bbox[k * 4 + j, h, w]) for j in range(4))
        pcx, pcy, pw, ph = dx * aw + cx, dy * ah + cy, np.exp(dw) * aw, np.exp(dh) * ah
        box = np.clip([pcx - 0.5 * pw, pcy - 0.5 * ph, pcx + 0.5 * pw, pcy + 0.5 * ph], 0, 1999)
        assert np.abs(props[i, :4] - box).max() < 1e-3
        ok = (box[2] - box[0] + 1 >= 16) and (box[3] - box[1] + 1 >= 16)
        assert props[i, 4] == (fg[k, h, w] if ok else 0)
    # a huge min size masks every score
    none = oracle.generate_proposals(fg, bbox, anchors, im_h, im_w, 1e6, 16)
    assert np.all(none[:, 4] == 0)


def test_sort_bbox_contract():
    """Descending and complete on the first num_top rows; a permutation overall."""
    r = rng(2)
    n, top = 3000, 700
    rois = r.standard_normal((n, 5)).astype(np.float32)
    rois[:, 4] = r.permutation(n).astype(np.float32)     # tie-free
    out = oracle.sort_bbox(rois, top)
    assert np.array_equal(out[:top, 4], np.arange(n - 1, n - 1 - top, -1, dtype=np.float32))
    order = np.argsort(-rois[:, 4], kind="stable")
    assert np.array_equal(out[:top], rois[order[:top]])
    assert np.array_equal(np.sort(out[:, 4]), np.sort(rois[:, 4]))
    # with ties the scores are still descending on the prefix and rows stay intact
    rois[:, 4] = r.integers(0, 20, n).astype(np.float32)
    rois[:, 0] = np.arange(n)
    out = oracle.sort_bbox(rois, top)
    assert (np.diff(out[:top, 4]) <= 0).all()
    assert np.array_equal(rois[out[:, 0].astype(int)], out)


def brute_nms_pixel(boxes, thr, max_keep):
    b = boxes.astype(np.float64)
    area = (b[:, 2] - b[:, 0] + 1) * (b[:, 3] - b[:, 1] + 1)
    keep = []
    for i in range(len(b)):
        ok = True
        for k in keep:
            w = max(0.0, min(b[i, 2], b[k, 2]) - max(b[i, 0], b[k, 0]) + 1)
            h = max(0.0, min(b[i, 3], b[k, 3]) - max(b[i, 1], b[k, 1]) + 1)
            if w * h / (area[i] + area[k] - w * h) > thr:
                ok = False
                break
        if ok:
            keep.append(i)
            if len(keep) == max_keep:
                break
    return np.array(keep, np.int32)


@pytest.mark.parametrize("thr,max_keep", [(0.7, 300), (0.3, 300), (0.5, 20)])
def test_nms_pixel_brute_force(thr, max_keep):
    r = rng(3)
    n = 400
    c = r.random((n, 2)) * 200
    wh = r.random((n, 2)) * 80 + 5
    # integer coordinates keep every IoU exactly representable away from thr
    boxes = np.round(np.concatenate([c, c + wh, r.random((n, 1))], 1)).astype(np.float32)
    got = oracle.nms_pixel(boxes, thr, max_keep)
    assert np.array_equal(got, brute_nms_pixel(boxes, thr, max_keep))


def test_proposal_end_to_end_small():
    r = rng(4)
    A, H, W = 9, 5, 6
    scores = r.random((1, 2 * A, H, W)).astype(np.float32)
    bbox = (r.standard_normal((1, 4 * A, H, W)) * 0.3).astype(np.float32)
    im_info = np.array([[H * 16, W * 16, 1.0]], np.float32)
    param = {"pre_nms_topn": 100, "post_nms_topn": 30, "nms_thresh": 0.5}
    (rois, rs), kept, table = oracle.proposal(param, scores, bbox, im_info, 2, details=True)
    props = oracle.generate_proposals(scores[0, A:], bbox[0], oracle.generate_anchors(), H * 16.0,
                                      W * 16.0, 16.0, 16)
    order = np.argsort(-props[:, 4], kind="stable")
    if len(np.unique(props[:, 4])) == len(props):        # tie-free: order is unique
        assert np.array_equal(table[:100], props[order[:100]])
    assert np.array_equal(kept, brute_nms_pixel(table[:100], 0.5, 30))
    assert np.array_equal(rois[:, 1:], table[kept, :4]) and np.all(rois[:, 0] == 0)
    assert np.array_equal(rs, table[kept, 4])


def test_prior_box_ssd300():
    # SSD300: 38^2*4 + 19^2*6 + 10^2*6 + 5^2*6 + 3^2*4 + 1*4 = 8732 priors
    cfg = [(38, 4, 30., 60., [2.], 8), (19, 6, 60., 111., [2., 3.], 16), (10, 6, 111., 162., [2., 3.], 32),
           (5, 6, 162., 213., [2., 3.], 64), (3, 4, 213., 264., [2.], 100), (1, 4, 264., 315., [2.], 300)]
    total = 0
    for fm, npri, mn, mx, ars, step in cfg:
        p = {"min_size": mn, "max_size": mx, "aspect_ratio": ars, "flip": True, "clip": False,
             "variance": [0.1, 0.1, 0.2, 0.2], "step": float(step), "offset": 0.5}
        out = oracle.prior_box(p, (1, 8, fm, fm), (1, 3, 300, 300))
        assert out.shape == (1, 2, fm * fm * npri * 4)
        total += fm * fm * npri
        boxes = out[0, 0].reshape(fm, fm, npri, 4).astype(np.float64)
        # centres at (w + 0.5) * step / 300, first prior is the min_size square
        h, w = fm // 2, fm // 3
        cx, cy = (w + 0.5) * step / 300, (h + 0.5) * step / 300
        assert np.allclose(boxes[h, w, 0], [cx - mn / 600, cy - mn / 600, cx + mn / 600, cy + mn / 600], atol=1e-6)
        s2 = np.sqrt(mn * mx) / 600
        assert np.allclose(boxes[h, w, 1], [cx - s2, cy - s2, cx + s2, cy + s2], atol=1e-6)
        # third prior: aspect ratio 2 -> width min*sqrt(2), height min/sqrt(2)
        assert np.allclose(boxes[h, w, 2, 2] - boxes[h, w, 2, 0], mn * np.sqrt(2) / 300, atol=1e-6)
        assert np.allclose(boxes[h, w, 3, 3] - boxes[h, w, 3, 1], mn * np.sqrt(2) / 300, atol=1e-6)
        assert np.array_equal(out[0, 1].reshape(-1, 4), np.tile(np.float32([0.1, 0.1, 0.2, 0.2]), (fm * fm * npri, 1)))
    assert total == 8732
    clipped = oracle.prior_box({"min_size": 200., "clip": True}, (1, 1, 2, 2), (1, 3, 100, 100))
    assert clipped[0, 0].min() == 0 and clipped[0, 0].max() == 1


def brute_detection_output(param, loc, conf, prior):
    """Independent float64 walk: decode (CENTER_SIZE), per-class greedy NMS, keep_top_k."""
    num, P, C = loc.shape[0], prior.shape[2] // 4, param["num_classes"]
    pb = prior[0, 0].reshape(P, 4).astype(np.float64)
    var = prior[0, 1].reshape(P, 4).astype(np.float64)
    nms = param["nms_param"]
    rows = []
    for i in range(num):
        l = loc[i].reshape(P, 4).astype(np.float64)
        pw, ph = pb[:, 2] - pb[:, 0], pb[:, 3] - pb[:, 1]
        pcx, pcy = (pb[:, 0] + pb[:, 2]) / 2, (pb[:, 1] + pb[:, 3]) / 2
        cx, cy = var[:, 0] * l[:, 0] * pw + pcx, var[:, 1] * l[:, 1] * ph + pcy
        w, h = np.exp(var[:, 2] * l[:, 2]) * pw, np.exp(var[:, 3] * l[:, 3]) * ph
        box = np.stack([cx - w / 2, cy - h / 2, cx + w / 2, cy + h / 2], 1)
        area = np.where((box[:, 2] < box[:, 0]) | (box[:, 3] < box[:, 1]), 0, (box[:, 2] - box[:, 0]) * (box[:, 3] - box[:, 1]))
        sc = conf[i].reshape(P, C)
        kept = {}
        for c in range(1, C):
            cand = [p for p in np.argsort(-sc[:, c], kind="stable") if sc[p, c] > param["confidence_threshold"]]
            cand = cand[:nms["top_k"]]
            ks = []
            for p in cand:
                ok = True
                for k in ks:
                    iw = min(box[p, 2], box[k, 2]) - max(box[p, 0], box[k, 0])
                    ih = min(box[p, 3], box[k, 3]) - max(box[p, 1], box[k, 1])
                    if iw > 0 and ih > 0 and iw * ih / (area[p] + area[k] - iw * ih) > nms["nms_threshold"]:
                        ok = False
                        break
                if ok:
                    ks.append(p)
            kept[c] = ks
        allk = [(sc[p, c], c, p) for c in kept for p in kept[c]]
        if len(allk) > param["keep_top_k"]:
            allk = sorted(allk, key=lambda t: -t[0])[:param["keep_top_k"]]
            sel = {(c, p) for _, c, p in allk}
            kept = {c: [p for p in kept[c] if (c, p) in sel] for c in kept}
        for c in sorted(kept):
            for p in kept[c]:
                rows.append([i, c, sc[p, c], *box[p]])
    return np.array(rows, np.float64).reshape(-1, 7)


def test_detection_output_brute_force():
    r = rng(5)
    num, P, C = 3, 64, 5
    c = r.random((P, 2)) * 0.8 + 0.1
    wh = r.random((P, 2)) * 0.3 + 0.05
    prior = np.concatenate([np.concatenate([c - wh / 2, c + wh / 2], 1).reshape(-1),
                            np.tile([0.1, 0.1, 0.2, 0.2], P)]).reshape(1, 2, P * 4).astype(np.float32)
    loc = (r.standard_normal((num, P * 4)) * 0.5).astype(np.float32)
    conf = oracle.softmax((r.standard_normal((num, P, C)) * 2).astype(np.float32), 2).reshape(num, P * C)
    param = {"num_classes": C, "share_location": True, "background_label_id": 0,
             "code_type": "CENTER_SIZE", "keep_top_k": 30, "confidence_threshold": 0.05,
             "nms_param": {"nms_threshold": 0.45, "top_k": 20}}
    got = oracle.detection_output(param, loc, conf, prior)
    want = brute_detection_output(param, loc, conf, prior)
    assert got.shape == want.shape and got.shape[0] > 10
    assert np.array_equal(got[:, :2], want[:, :2])
    assert np.abs(got - want).max() < 1e-5
    # nothing above the threshold: one row of -1 per image with the image id
    param["confidence_threshold"] = 2.0
    none = oracle.detection_output(param, loc, conf, prior)
    assert np.array_equal(none, np.array([[i, -1, -1, -1, -1, -1, -1] for i in range(num)], np.float32))


def test_normalize_closed_form():
    r = rng(6)
    x = r.standard_normal((2, 5, 3, 4)).astype(np.float32)
    s = (r.random(5) + 0.5).astype(np.float32)
    y = oracle.normalize(x, s, across_spatial=False, channel_shared=False, eps=1e-10)
    want = x / np.sqrt((x.astype(np.float64) ** 2).sum(axis=1, keepdims=True) + 1e-10) * s.reshape(1, 5, 1, 1)
    assert np.abs(y - want).max() < 1e-6
    y = oracle.normalize(x, s[:1], across_spatial=True, channel_shared=True, eps=1e-10)
    want = x / np.sqrt((x.astype(np.float64) ** 2).sum(axis=(1, 2, 3), keepdims=True) + 1e-10) * s[0]
    assert np.abs(y - want).max() < 1e-6


# ---- region pooling (roi_pooling_layer.cpp, psroi_pooling_layer.cpp) --------------------
# Pinned through cases that reduce to numpy routines, chosen so that a wrong rounding
# rule, a missing "+1", a transposed bin index or a wrong channel map fails one of them.

def _blocks(a, bh, bw):
    """(C, H, W) -> (C, H/bh, W/bw, bh*bw) blocks."""
    c, h, w = a.shape
    return a.reshape(c, h // bh, bh, w // bw, bw).transpose(0, 1, 3, 2, 4).reshape(c, h // bh, w // bw, -1)


def test_roi_pooling_reduces_to_numpy_cases():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 3, 8, 12)).astype(np.float32)
    whole = [[1, 0, 0, 11, 7]]                       # x1, y1, x2, y2 inclusive
    assert np.array_equal(oracle.roi_pooling(x, whole, 1, 1, 1.0)[0, :, 0, 0], x[1].max(axis=(1, 2)))
    assert np.array_equal(oracle.roi_pooling(x, whole, 8, 12, 1.0)[0], x[1])        # one bin per cell
    assert np.array_equal(oracle.roi_pooling(x, whole, 4, 3, 1.0)[0], _blocks(x[1], 2, 4).max(-1))
    # an aligned sub-region: rows 2..5, columns 4..9 (inclusive ends: the "+1" of the extent)
    sub = oracle.roi_pooling(x, [[0, 4, 2, 9, 5]], 2, 3, 1.0)[0]
    assert np.array_equal(sub, _blocks(x[0][:, 2:6, 4:10], 2, 2).max(-1))
    # spatial_scale: image coordinates 16x the map's, rounded after scaling (40/16 = 2.5 -> 3)
    scaled = oracle.roi_pooling(x, [[0, 40, 0, 191, 127]], 1, 1, 1 / 16.0)[0, :, 0, 0]
    assert np.array_equal(scaled, x[0][:, 0:8, 3:12].max(axis=(1, 2)))
    # a roi outside the map: every bin empty -> 0; a bad batch index is an error
    assert np.array_equal(oracle.roi_pooling(x, [[0, 50, 50, 60, 60]], 2, 2, 1.0), np.zeros((1, 3, 2, 2)))
    with pytest.raises(ValueError):
        oracle.roi_pooling(x, [[2, 0, 0, 1, 1]], 1, 1, 1.0)


def test_psroi_pooling_reduces_to_numpy_cases():
    rng = np.random.default_rng(1)
    dim, g = 3, 2
    x = rng.standard_normal((2, dim * g * g, 8, 12)).astype(np.float32)
    whole = [[1, 0, 0, 11, 7]]
    got = oracle.psroi_pooling(x, whole, dim, g, 1.0)[0]
    # bin (ph, pw) of output c = mean of the (ph, pw) block of input channel (c*g + ph)*g + pw
    for c in range(dim):
        for ph in range(g):
            for pw in range(g):
                blk = x[1, (c * g + ph) * g + pw, ph * 4:(ph + 1) * 4, pw * 6:(pw + 1) * 6]
                assert abs(got[c, ph, pw] - blk.astype(np.float64).mean()) < 1e-6
    # group_size 1: plain mean over the region, end corner x2 + 1 exclusive
    x1 = rng.standard_normal((1, 4, 6, 6)).astype(np.float32)
    got = oracle.psroi_pooling(x1, [[0, 1, 2, 4, 3]], 4, 1, 1.0)[0, :, 0, 0]
    assert np.allclose(got, x1[0][:, 2:4, 1:5].astype(np.float64).mean(axis=(1, 2)), atol=1e-6)
    # corners are rounded BEFORE scaling: x1 = 7.6 -> 8 -> 0.5 on a 1/16 map, i.e. bin start floor(0.5) = 0
    got = oracle.psroi_pooling(x1, [[0, 7.6, 0, 31.4, 15.2]], 4, 1, 1 / 16.0)[0, :, 0, 0]
    assert np.allclose(got, x1[0][:, 0:1, 0:2].astype(np.float64).mean(axis=(1, 2)), atol=1e-6)
    # outside the map -> 0
    assert np.array_equal(oracle.psroi_pooling(x1, [[0, 100, 100, 120, 120]], 4, 1, 1.0), np.zeros((1, 4, 1, 1)))
    with pytest.raises(ValueError):
        oracle.psroi_pooling(x1, [[0, 0, 0, 1, 1]], 3, 1, 1.0)      # channel count mismatch
