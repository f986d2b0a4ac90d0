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


# Literal vectors for the order SortBBox leaves EQUAL scores in.  Each expected order was
# traced by hand from proposal_layer.cpp:88-111 (first element is the pivot "key"; `last`
# walks left over scores <= key, the row there moves into the hole at `first`; `first` walks
# right over scores >= key, the row there moves into the hole at `last`; the key lands where
# they meet; recurse left, then right only while the right part starts before num_top).
# Rows are named a, b, c ... in input order; the trace of each case is in its comment.
_TIE_CASES = [
    # [a5 b5 c5], top 3.  key a: last walks 2->1->0 (5<=5 each), a stays at 0.  Right part
    # (1,2): key b, last walks 2->1, b stays.  All-equal input keeps its order.
    # A `<` in the last-walk would instead move c to the front: c b a.
    ([5, 5, 5], 3, "abc"),
    # [a3 b5 c3 d4], top 4.  key a(3): last=3 (4<=3 no) -> d into hole 0; first walks 0(d4)
    # 1(b5) 2(c3: 3>=3) and meets last at 3; a lands at 3: d b c a.  Left part (0,2): key d(4):
    # last 2(c3<=4)->1 (b5<=4 no) -> b into hole 0; first 0->1 meets; d lands at 1: b d c a.
    # The equal pair ends up c before a: NOT the stable order (a before c).
    ([3, 5, 3, 4], 4, "bdca"),
    # [a4 b6 c4 d6 e2], top 5.  key a(4): last 4(e2<=4)->3 (d6 no) -> d into hole 0; first walks
    # 0(d6) 1(b6) 2(c4>=4) to 3; a lands at 3: d b c a e.  Left (0,2): key d(6): last 2(c4)->1
    # (b6<=6)->0, d stays; its right part (1,2): key b: last 2->1, b stays.  Result d b c a e:
    # both equal pairs reversed.  A `>` in the first-walk would stop at c and give d b a c e.
    ([4, 6, 4, 6, 2], 5, "dbcae"),
    # [a5 b1 c2 d3 e4], top 2: the right recursion is cut by num_top.  key a(5): last walks to
    # 0, a stays, first=0; right part (1,4) is sorted because 1 < 2: key b(1): last=4 (e4<=1 no)
    # -> e into hole 1; first walks 1,2,3 to 4; b lands at 4: a e c d b, first=4.  Its left part
    # (1,3): key e(4): last 3(d3)->2(c2)->1, e stays, first=1; right part (2,3) is NOT sorted
    # because first+1 = 2 is not < num_top = 2.  c2 stays before d3.
    ([5, 1, 2, 3, 4], 2, "aecdb"),
    # same input, top 1: after the first partition first+1 = 1 is not < 1: nothing else moves.
    ([5, 1, 2, 3, 4], 1, "abcde"),
    # [a2 b7 c2 d7 e2 f7], top 3: equal scores on both sides of the cut.  key a(2): last=5
    # (f7<=2 no) -> f into hole 0; first walks 0..4 (7,7,2,7,2 all >= 2) to 5; a lands at 5:
    # f b c d e a.  Left (0,4): key f(7): last walks 4,3,2,1 (2,7,2,7 all <= 7) to 0, f stays,
    # first=0.  Right (1,4) (1<3): key b(7): last walks 4,3,2 to 1, b stays, first=1.  Right
    # (2,4) (2<3): key c(2): last 4(e2<=2)->3 (d7 no) -> d into hole 2; first 2(d7)->3 meets;
    # c lands at 3: f b d c e a, first=3; left (2,2) and right (4<3 fails) end.  Top three are
    # f b d (the stable order would be b d f).
    ([2, 7, 2, 7, 2, 7], 3, "fbdcea"),
    # [a3 b1 c3 d5 e3 f0 g5 h3], top 8: equal scores left and right of the pivot, two hole
    # moves.  key a(3): last 7(h3<=3)->6 (g5 no) -> g into hole 0; first 0(g5)->1 (b1>=3 no) ->
    # b into hole 6; last 6(b1)->5(f0)->4(e3<=3)->3 (d5 no) -> d into hole 1; first 1(d5)->2
    # (c3>=3)->3 meets; a lands at 3: g d c a e f b h.  Left (0,2): key g(5): last 2(c3)->1
    # (d5<=5)->0, g stays; right part (1,2): key d(5): last 2->1, d stays.  Right of a, (4,7)
    # = e3 f0 b1 h3: key e(3): last 7(h3<=3)->6->5->4, e stays, first=4; right (5,7) = f0 b1 h3:
    # key f(0): last=7 (h3<=0 no) -> h into hole 5; first 5(h3)->6(b1>=0)->7 meets; f lands at
    # 7: h b f, first=7; left (5,6) = h3 b1: key h: last 6->5, h stays.  Result g d c a e h b f.
    ([3, 1, 3, 5, 3, 0, 5, 3], 8, "gdcaehbf"),
]


@pytest.mark.parametrize("scores,top,want", _TIE_CASES)
def test_sort_bbox_tie_order_hand_traced(scores, top, want):
    n = len(scores)
    rois = np.zeros((n, 5), np.float32)
    rois[:, 0] = np.arange(n)                 # row identity travels in column 0
    rois[:, 1] = np.arange(n) * 10 + 1        # and the other columns must travel with it
    rois[:, 4] = scores
    out = oracle.sort_bbox(rois, top)
    got = "".join("abcdefgh"[int(i)] for i in out[:, 0])
    assert got == want
    assert np.array_equal(out, rois[out[:, 0].astype(int)])


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


def test_order_of_equal_scores_is_irrelevant_with_one_live_member():
    """The rule the device's head step relies on: a group of equal scores may stand in any
    order when at most one of its members is alive where the greedy pass reaches the group
    (alive: overlaps no box kept before the group by more than the threshold).  Checked on
    the CPU against every order of planted groups; and the converse happens: with two live
    members some order changes the kept rows."""
    import itertools
    r = rng(9)
    changed_with_two_live = 0
    checked_with_one_live = 0
    for trial in range(120):
        n = 60
        c = r.random((n, 2)) * 120
        wh = r.random((n, 2)) * 60 + 10
        boxes = np.round(np.concatenate([c, c + wh], 1)).astype(np.float32)
        scores = np.sort(r.random(n).astype(np.float32))[::-1].copy()
        start, size = int(r.integers(5, 40)), int(r.integers(2, 4))
        scores[start:start + size] = scores[start]
        thr, max_keep = float(r.choice([0.3, 0.5])), int(r.choice([8, 60]))
        table = np.concatenate([boxes, scores[:, None]], 1).astype(np.float32)
        kept_before = [k for k in brute_nms_pixel(table, thr, n) if k < start]

        def iou(a, b):
            w = min(a[2], b[2]) - max(a[0], b[0]) + 1
            h = min(a[3], b[3]) - max(a[1], b[1]) + 1
            if w <= 0 or h <= 0:
                return 0.0
            inter = w * h
            return inter / ((a[2] - a[0] + 1) * (a[3] - a[1] + 1) + (b[2] - b[0] + 1) * (b[3] - b[1] + 1) - inter)

        live = [z for z in range(start, start + size)
                if not any(iou(boxes[k], boxes[z]) > thr for k in kept_before)]
        results = set()
        for perm in itertools.permutations(range(start, start + size)):
            order = list(range(start)) + list(perm) + list(range(start + size, n))
            kept = brute_nms_pixel(table[order], thr, max_keep)
            results.add(tuple(map(tuple, table[order][kept])))
        reached = len(kept_before) < max_keep
        if len(live) <= 1 or not reached:
            assert len(results) == 1, (trial, live)
            checked_with_one_live += 1
        elif len(results) > 1:
            changed_with_two_live += 1
    assert checked_with_one_live > 20 and changed_with_two_live > 20


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


def brute_decode(code_type, var_in_target, pb, var, l):
    """Float64 decode of P boxes for the three code types (bbox_util.cpp:242-330)."""
    if var_in_target:
        var = np.ones_like(var)
    pw, ph = pb[:, 2] - pb[:, 0], pb[:, 3] - pb[:, 1]
    if code_type == "CORNER":
        return pb + var * l
    if code_type == "CORNER_SIZE":
        return pb + var * l * np.stack([pw, ph, pw, ph], 1)
    assert code_type == "CENTER_SIZE"
    pcx, pcy = (pb[:, 0] + pb[:, 2]) / 2, (pb[:, 1] + pb[:, 3]) / 2
    cx, cy = var[:, 0] * l[:, 0] * pw + pcx, var[:, 1] * l[:, 1] * ph + pcy
    w, h = np.exp(var[:, 2] * l[:, 2]) * pw, np.exp(var[:, 3] * l[:, 3]) * ph
    return np.stack([cx - w / 2, cy - h / 2, cx + w / 2, cy + h / 2], 1)


def brute_detection_output(param, loc, conf, prior):
    """Independent float64 walk of detection_output_layer.cpp:74-226: decode (any code type,
    variance in the prior or in the target, shared or per-class locations), per-class greedy
    NMS with the adaptive threshold (bbox_util.cpp:696-715), keep_top_k."""
    num, P, C = loc.shape[0], prior.shape[2] // 4, param["num_classes"]
    share = param.get("share_location", True)
    bg = param.get("background_label_id", 0)
    pb = prior[0, 0].reshape(P, 4).astype(np.float64)
    var = prior[0, 1].reshape(P, 4).astype(np.float64)
    nms = param["nms_param"]
    eta = nms.get("eta", 1.0)
    rows = []
    for i in range(num):
        l_all = loc[i].reshape(P, 1 if share else C, 4).astype(np.float64)
        sc = conf[i].reshape(P, C)
        kept, boxes = {}, {}
        for c in range(C):
            if c == bg:
                continue
            box = brute_decode(param["code_type"], param.get("variance_encoded_in_target", False),
                               pb, var, l_all[:, 0 if share else c])
            boxes[c] = box
            area = np.where((box[:, 2] < box[:, 0]) | (box[:, 3] < box[:, 1]), 0,
                            (box[:, 2] - box[:, 0]) * (box[:, 3] - box[:, 1]))
            cand = [p for p in np.argsort(-sc[:, c], kind="stable") if sc[p, c] > param["confidence_threshold"]]
            if nms.get("top_k", -1) > -1:
                cand = cand[:nms["top_k"]]
            thr = nms["nms_threshold"]
            ks = []
            for p in cand:
                iw = np.minimum(box[p, 2], box[ks, 2]) - np.maximum(box[p, 0], box[ks, 0])
                ih = np.minimum(box[p, 3], box[ks, 3]) - np.maximum(box[p, 1], box[ks, 1])
                inter = np.where((iw > 0) & (ih > 0), iw * ih, 0.0)
                if not (inter / (area[p] + area[ks] - inter + 1e-300) > thr).any():
                    ks.append(p)
                    if eta < 1 and thr > 0.5:
                        thr *= eta
            kept[c] = ks
        allk = [(sc[p, c], c, p) for c in kept for p in kept[c]]
        if -1 < param["keep_top_k"] < len(allk):
            allk = sorted(allk, key=lambda t: -t[0])[:param["keep_top_k"]]
            kept = {c: [p for s_, c_, p in allk if c_ == c] for c in kept}
        for c in sorted(kept):
            for p in kept[c]:
                rows.append([i, c, sc[p, c], *boxes[c][p]])
    return np.array(rows, np.float64).reshape(-1, 7)


def _detection_case(seed, num=3, P=64, C=5, per_class=False, loc_scale=0.5):
    r = rng(seed)
    c = r.random((P, 2)) * 0.8 + 0.1
    wh = r.random((P, 2)) * 0.3 + 0.05
    # four different variances so that a transposed or dropped variance shows
    prior = np.concatenate([np.concatenate([c - wh / 2, c + wh / 2], 1).reshape(-1),
                            np.tile([0.1, 0.15, 0.2, 0.3], P)]).reshape(1, 2, P * 4).astype(np.float32)
    loc = (r.standard_normal((num, P * (C if per_class else 1) * 4)) * loc_scale).astype(np.float32)
    conf = oracle.softmax((r.standard_normal((num, P, C)) * 2).astype(np.float32), 2).reshape(num, P * C)
    return loc, conf, prior


def _assert_rows(got, want, min_rows=10):
    assert got.shape == want.shape and got.shape[0] > min_rows
    assert np.array_equal(got[:, :2], want[:, :2])
    assert np.abs(got - want).max() < 1e-5


def test_detection_output_brute_force():
    loc, conf, prior = _detection_case(5)
    num = loc.shape[0]
    param = {"num_classes": 5, "share_location": True, "background_label_id": 0,
             "code_type": "CENTER_SIZE", "keep_top_k": 30, "confidence_threshold": 0.05,
             "nms_param": {"nms_threshold": 0.45, "top_k": 20}}
    _assert_rows(oracle.detection_output(param, loc, conf, prior),
                 brute_detection_output(param, loc, conf, prior))
    # nothing above the threshold: one row of -1 per image with the image id
    param["confidence_threshold"] = 2.0
    none = oracle.detection_output(param, loc, conf, prior)
    assert np.array_equal(none, np.array([[i, -1, -1, -1, -1, -1, -1] for i in range(num)], np.float32))


@pytest.mark.parametrize("code_type", ["CORNER", "CENTER_SIZE", "CORNER_SIZE"])
@pytest.mark.parametrize("var_in_target", [False, True])
@pytest.mark.parametrize("per_class", [False, True])
def test_detection_output_decode_branches_brute_force(code_type, var_in_target, per_class):
    """CORNER / CORNER_SIZE decode, variance_encoded_in_target and share_location: false
    (bbox_util.cpp:242-330, 348-401) against the float64 walk; kept (image, label) rows
    must be identical, scores and corners within 1e-5."""
    loc, conf, prior = _detection_case(11 + 2 * var_in_target + per_class, per_class=per_class,
                                       loc_scale=0.08 if code_type == "CORNER" else 0.5)
    param = {"num_classes": 5, "share_location": not per_class, "background_label_id": 0,
             "code_type": code_type, "variance_encoded_in_target": var_in_target,
             "keep_top_k": 40, "confidence_threshold": 0.03,
             "nms_param": {"nms_threshold": 0.45, "top_k": 25}}
    got = oracle.detection_output(param, loc, conf, prior)
    want = brute_detection_output(param, loc, conf, prior)
    _assert_rows(got, want)
    # the branch must matter: the other variance convention decodes different boxes
    other = dict(param, variance_encoded_in_target=not var_in_target)
    assert np.abs(brute_detection_output(other, loc, conf, prior)[:5, 3:] - want[:5, 3:]).max() > 1e-3


def test_detection_output_shared_locations_without_background_fail():
    """share_location with background_label_id -1: the reference skips the shared boxes
    (label -1) as background and aborts (bbox_util.cpp:366-371,
    detection_output_layer.cpp:122-126); the restatement reports it."""
    rng = np.random.default_rng(3)
    P, C = 6, 3
    loc = rng.standard_normal((1, P * 4)).astype(np.float32)
    conf = oracle.softmax(rng.standard_normal((1, P, C)).astype(np.float32), 2).reshape(1, P * C)
    prior = np.tile(np.float32([0.1, 0.1, 0.4, 0.4]), 2 * P).reshape(1, 2, P * 4)
    param = {"num_classes": C, "share_location": True, "background_label_id": -1,
             "nms_param": {"nms_threshold": 0.5}}
    with pytest.raises(ValueError, match="label -1"):
        oracle.detection_output(param, loc, conf, prior)


@pytest.mark.parametrize("bg", [0, 2, -1])
def test_detection_output_background_label_brute_force(bg):
    """Any class can be the background (skipped); -1 keeps every class."""
    loc, conf, prior = _detection_case(21, per_class=True)
    param = {"num_classes": 5, "share_location": False, "background_label_id": bg,
             "code_type": "CENTER_SIZE", "keep_top_k": -1, "confidence_threshold": 0.1,
             "nms_param": {"nms_threshold": 0.4, "top_k": 30}}
    got = oracle.detection_output(param, loc, conf, prior)
    _assert_rows(got, brute_detection_output(param, loc, conf, prior))
    assert bg not in got[:, 1]                            # the background label never appears
    assert set(np.unique(got[:, 1]).astype(int)) == set(range(5)) - {bg}


@pytest.mark.parametrize("eta,thr0", [(0.8, 0.9), (0.95, 0.7), (0.6, 0.55)])
def test_detection_output_adaptive_eta_brute_force(eta, thr0):
    """eta < 1: the overlap threshold is multiplied by eta after every kept box while it is
    above 0.5 (bbox_util.cpp:696-715).  Overlapping priors and small offsets make the kept
    set depend on the decaying threshold."""
    r = rng(31)
    num, P, C = 2, 96, 3
    centre = r.random((P // 8, 2)) * 0.6 + 0.2                     # 12 clusters of 8 boxes
    c = np.repeat(centre, 8, 0) + r.standard_normal((P, 2)) * 0.02
    wh = 0.25 + r.random((P, 2)) * 0.05
    prior = np.concatenate([np.concatenate([c - wh / 2, c + wh / 2], 1).reshape(-1),
                            np.tile([0.1, 0.1, 0.2, 0.2], P)]).reshape(1, 2, P * 4).astype(np.float32)
    loc = (r.standard_normal((num, P * 4)) * 0.3).astype(np.float32)
    conf = oracle.softmax((r.standard_normal((num, P, C)) * 2).astype(np.float32), 2).reshape(num, P * C)
    param = {"num_classes": C, "share_location": True, "background_label_id": 0,
             "code_type": "CENTER_SIZE", "keep_top_k": -1, "confidence_threshold": 0.01,
             "nms_param": {"nms_threshold": thr0, "top_k": -1, "eta": eta}}
    got = oracle.detection_output(param, loc, conf, prior)
    want = brute_detection_output(param, loc, conf, prior)
    _assert_rows(got, want)
    fixed = dict(param, nms_param=dict(param["nms_param"], eta=1.0))
    assert oracle.detection_output(fixed, loc, conf, prior).shape[0] > got.shape[0]   # eta bites


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
