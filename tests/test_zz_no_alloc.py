"""mcProposalStatic (the entry point that allocates nothing) against mcProposal: same
rois, scores, counts and tie flags, bit for bit, on consecutive calls that share the
library's built-in scratch buffer, the second call on a smaller problem; and a clear
error for a problem the buffer cannot hold."""
import ctypes

import numpy as np
import pytest

import oracle

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from minicaffe import kernels
    return kernels


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _inputs(seed, H, W, quant):
    r = np.random.default_rng(seed)
    A = 9
    scores = r.random((1, 2 * A, H, W)).astype(np.float32)
    if quant:
        scores = np.round(scores * quant) / np.float32(quant)
    bbox = (r.standard_normal((1, 4 * A, H, W)) * 0.3).astype(np.float32)
    im_info = np.array([[H * 16, W * 16, 1.0]], np.float32)
    return scores.astype(np.float32), bbox, im_info


def _run(K, static, scores, bbox, im_info, pre, post, thr):
    A, H, W = 9, scores.shape[2], scores.shape[3]
    dev = [torch.from_numpy(np.ascontiguousarray(a)).cuda()
           for a in (scores, bbox, im_info, oracle.generate_anchors())]
    rois = torch.full((post, 5), float("nan"), device="cuda")
    rs = torch.full((post,), float("nan"), device="cuda")
    cnt = torch.full((2,), -7, dtype=torch.int32, device="cuda")
    head = [_ptr(d) for d in dev] + [A, H, W, 16, ctypes.c_float(16), pre, post, ctypes.c_float(thr)]
    tail = [_ptr(rois), _ptr(rs), ctypes.c_void_p(cnt.data_ptr()), ctypes.c_void_p(cnt.data_ptr() + 4),
            None]
    if static:
        K.check_mc(K.LIB.mcProposalStatic(*head, *tail))
    else:
        sz = ctypes.c_size_t()
        K.check_mc(K.LIB.mcProposalWorkspaceSize(A * H * W, pre, post, ctypes.byref(sz)))
        ws = torch.empty(sz.value, dtype=torch.uint8, device="cuda")
        K.check_mc(K.LIB.mcProposal(*head, _ptr(ws), sz.value, *tail))
    torch.cuda.synchronize()
    n, ties = int(cnt[0].item()), int(cnt[1].item())
    return n, ties, rois[:n].cpu().numpy(), rs[:n].cpu().numpy()


def test_static_scratch_matches_workspace_entry_point_on_consecutive_calls(K):
    # large (config-4 size, with score ties), then smaller, then large again: the buffer
    # keeps the previous call's contents and every call must still be exact
    calls = [(1, 38, 63, 2000, 6000, 300, 0.7), (2, 10, 12, 0, 2000, 50, 0.5),
             (3, 20, 20, 7, 6000, 300, 0.7), (4, 38, 63, 0, 6000, 300, 0.7)]
    for seed, H, W, quant, pre, post, thr in calls:
        scores, bbox, im_info = _inputs(seed, H, W, quant)
        want = _run(K, False, scores, bbox, im_info, pre, post, thr)
        got = _run(K, True, scores, bbox, im_info, pre, post, thr)
        assert got[0] == want[0] and got[0] > 0 and got[1] == want[1]
        assert np.array_equal(got[2], want[2]) and np.array_equal(got[3], want[3])
        # and against the CPU checker, as the workspace entry point's own test does
        (rois, rs), _, _ = oracle.proposal({"pre_nms_topn": pre, "post_nms_topn": post,
                                            "nms_thresh": thr}, scores, bbox, im_info, 2, details=True)
        assert np.array_equal(got[2], rois) and np.array_equal(got[3], rs)


def test_static_scratch_allocates_nothing(K):
    """What the entry point is for: after one call on the device (the first looks up the
    buffer's address, which may load the code object: it must happen outside a capture),
    further calls leave the device's free memory as it is."""
    scores, bbox, im_info = _inputs(6, 38, 63, 0)
    A, H, W, pre, post = 9, 38, 63, 6000, 300
    dev = [torch.from_numpy(np.ascontiguousarray(a)).cuda()
           for a in (scores, bbox, im_info, oracle.generate_anchors())]
    rois = torch.empty((post, 5), device="cuda")
    rs = torch.empty((post,), device="cuda")
    cnt = torch.zeros(2, dtype=torch.int32, device="cuda")
    args = [_ptr(d) for d in dev] + [A, H, W, 16, ctypes.c_float(16), pre, post, ctypes.c_float(0.7), _ptr(rois),
                                     _ptr(rs), ctypes.c_void_p(cnt.data_ptr()), ctypes.c_void_p(cnt.data_ptr() + 4), None]
    K.check_mc(K.LIB.mcProposalStatic(*args))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(5):
        K.check_mc(K.LIB.mcProposalStatic(*args))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert int(cnt[0].item()) > 0


def test_static_scratch_refuses_what_it_cannot_hold(K):
    scores, bbox, im_info = _inputs(5, 60, 80, 0)          # 43200 proposals
    with pytest.raises(Exception, match="scratch"):
        _run(K, True, scores, bbox, im_info, 12000, 300, 0.7)
