#!/usr/bin/env python3
"""Headline benchmark: ResNet-50 v1 forward, fp32, batch 64, 3x224x224, on one MI355X.

A step is one Net::Forward through the C ABI (CaffeNetForward) on a batch that
already sits in HBM: seeded synthetic input, He-normal random weights of the
real architecture.  Prints one JSON line with images/s, the roofline figures of
the dominant kernel (the fp32 MFMA implicit-GEMM convolution) measured with HIP
events on the library's stream, and the CPU baseline (the oracle's restatement
of the reference's per-image im2col + OpenBLAS sgemm path) timed on a bounded
sample on this box's host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "mini-caffe_amd"))

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0
CONV_SOURCES = [os.path.join(ROOT, "mini-caffe_amd", "csrc", "kernels", f)
                for f in ("conv_igemm.hip", "conv_winograd.hip")]
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "igemm_resnet50_b64_pmc_traffic.txt")
MFMA_PROFILE = os.path.join(ROOT, "profiles", "igemm_resnet50_b64_pmc_mfma_util.txt")


def counter_figure(path, key):
    """A figure that only a rocprofv3 --pmc run can give (HBM bytes per launch, MFMA
    utilisation), read from the committed summary of that run.  The summary ends with
    `key: value` lines, among them the SHA-256 of the convolution kernel sources it was
    taken with; a summary of another kernel version is reported as stale instead of being quoted.
    Returns (value or None, note)."""
    import hashlib
    fields = {}
    try:
        for line in open(path):
            k, sep, v = line.partition(":")
            if sep and " " not in k.strip():
                fields[k.strip()] = v.strip()
    except OSError as e:
        return None, "no counter summary (%s)" % e
    have = hashlib.sha256(b"".join(open(f, "rb").read() for f in CONV_SOURCES)).hexdigest()
    rel = os.path.relpath(path, ROOT)
    if key not in fields or "conv_sources_sha256" not in fields:
        return None, "%s holds no '%s' line" % (rel, key)
    if fields["conv_sources_sha256"] != have:
        msg = ("%s was taken with another version of conv_igemm.hip + conv_winograd.hip (sha256 %s..., tree "
               "has %s...): re-run the command it names" % (rel, fields["conv_sources_sha256"][:12], have[:12]))
        print("bench.py: STALE COUNTER SUMMARY: " + msg, file=sys.stderr)
        return None, "stale: " + msg
    return float(fields[key]), "%s, taken %s" % (rel, fields.get("date", "?"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-batch", type=int, default=8)
    ap.add_argument("--no-winograd", action="store_true",
                    help="keep every convolution on the direct implicit-GEMM path (3x3 stride-1 layers with "
                         "128 or more channels otherwise run as F(2x2,3x3) Winograd)")
    ap.add_argument("--no-direct-comparison", action="store_true",
                    help="skip the second, shorter measurement with every convolution on the direct path "
                         "(and the two-thread run: profiling commands see the one net's launches only)")
    ap.add_argument("--no-detection-tails", action="store_true",
                    help="skip the NMS / Proposal / DetectionOutput timings (profiling runs of the "
                         "ResNet-50 forward alone)")
    ap.add_argument("--no-two-threads", action="store_true",
                    help="skip the run with two host threads, each with its own net and stream")
    ap.add_argument("--configs-report", metavar="PATH",
                    help="also time all five BASELINE configurations (whole forward, contraction "
                         "launches, Proposal / DetectionOutput layers) and write a text table to PATH")
    ap.add_argument("--layer-scaling", metavar="PATH",
                    help="also time representative ResNet-50 convolutions alone at batch 16..512 "
                         "(how far a single launch is from the kernel's steady state) and write a "
                         "text table to PATH")
    ap.add_argument("--layer-roofline", metavar="PATH",
                    help="also time the 20 distinct ResNet-50 convolutions alone at the bench batch "
                         "and write, per layer, FLOPs, algorithmic bytes, the roofline that binds "
                         "(fp32 MFMA or HBM) and the fraction reached to PATH")
    ap.add_argument("--bandwidth-report", metavar="PATH",
                    help="also time the HBM-bound kernels (pooling, eltwise, channel transform, "
                         "softmax, permute, normalize, LRN, copies, depthwise convolution) alone at "
                         "the shapes of the configurations and write GB/s against the 8 TB/s "
                         "roofline to PATH")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run one plain 256 MiB device copy (mcCopy2D): under rocprofv3 --pmc "
                         "its FETCH_SIZE / WRITE_SIZE reading calibrates the counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported "
                 "(the forward path shards over the batch with no exchange)" % args.gpus)

    import numpy as np
    import minicaffe as mc
    from minicaffe import craft, zoo
    from minicaffe.base import LIB

    if not mc.check_gpu_available():
        sys.exit("bench.py: no HIP device visible")
    mc.set_runtime_mode(1, 0)

    if args.copy_calibration:
        import torch
        from minicaffe import kernels  # noqa: F401  (declares the mc* prototypes: 64-bit pointers)
        n = 64 << 20                      # floats: 256 MiB read, 256 MiB written
        src = torch.ones(n, device="cuda")
        dst = torch.empty(n, device="cuda")
        for _ in range(2):
            rc = LIB.mcCopy2D(ctypes.c_void_p(src.data_ptr()), n, ctypes.c_void_p(dst.data_ptr()), n, n, 1, None)
            assert rc == 0, LIB.mcLastError()
        torch.cuda.synchronize()
        del src, dst

    spec, inputs = zoo.resnet50_spec(batch=args.batch, size=224, seed=0)
    flops = zoo.conv_flops(spec, inputs)
    if args.no_winograd:
        LIB.mcConvWinogradDefault(0)
    net = mc.Net.from_buffers(craft.to_prototxt(spec, "ResNet-50"))
    craft.load_weights(net, spec)
    net.forward(**inputs)          # uploads input + weights, packs filters
    for _ in range(max(0, args.warmup - 1)):
        net.forward()

    import torch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        net.forward()              # ends with a stream synchronisation
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = 1e3 * elapsed / args.steps
    prob = net.get_blob("prob").data
    assert np.isfinite(prob).all() and abs(float(prob.sum()) - args.batch) < 1e-2 * args.batch

    # Roofline of the dominant kernel: same steps again with every contraction
    # launch bracketed by HIP events on the launch stream.
    LIB.mcConvTimingEnable(1)
    for _ in range(args.steps):
        net.forward()
    tot_ms, launches, fl = ctypes.c_double(), ctypes.c_long(), ctypes.c_double()
    issued, wino = ctypes.c_double(), ctypes.c_long()
    LIB.mcConvTimingCollectDetail(ctypes.byref(tot_ms), ctypes.byref(launches), ctypes.byref(fl),
                                  ctypes.byref(issued), ctypes.byref(wino))
    LIB.mcConvTimingEnable(0)
    # achieved: the layers' algorithmic FLOPs (2 x MACs of the direct sum) over the device time
    # of their launches (one launch per contraction).  A 3x3 layer on the Winograd path counts
    # with its direct-sum FLOPs; mfma_issued_* is what the matrix pipe was actually handed in
    # the same time (2.25 times fewer products for those layers).
    secs = tot_ms.value * 1e-3
    achieved = fl.value / secs / 1e12 if secs > 0 else 0.0
    issued_tflops = issued.value / secs / 1e12 if secs > 0 else 0.0
    traffic, traffic_note = counter_figure(TRAFFIC_PROFILE, "traffic_bytes_per_launch")
    mfma_util, mfma_note = counter_figure(MFMA_PROFILE, "mfma_util_pct")
    steps = max(1, args.steps)
    roofline = {"bound": "mfma", "achieved": round(achieved, 2), "peak": FP32_MFMA_PEAK_TFLOPS,
                "unit": "TFLOP/s", "frac": round(achieved / FP32_MFMA_PEAK_TFLOPS, 4),
                "frac_is": "direct-sum FLOPs of all contractions over their device time, against the fp32 MFMA peak: what "
                           "the layers are worth; the matrix pipe's own utilisation is mfma_issued_frac (the Winograd "
                           "layers hand it 2.25 times fewer products)",
                "traffic": traffic, "traffic_source": traffic_note,
                "kernel": "igemm_f32 / winograd_fused (Convolution + InnerProduct, fused BN/Scale/ReLU epilogue; "
                          "%d of the %d contractions per step are 3x3 stride-1 layers run as F(2x2,3x3) Winograd "
                          "in one launch each)" % (wino.value // steps, launches.value // steps),
                "launches_per_step": launches.value // steps,
                "winograd_per_step": wino.value // steps,
                "kernel_ms_per_step": round(tot_ms.value / steps, 3),
                "gflop_per_step": round(fl.value / steps / 1e9, 1),
                "mfma_issued_gflop_per_step": round(issued.value / steps / 1e9, 1),
                "mfma_issued_tflops": round(issued_tflops, 2),
                "mfma_issued_frac": round(issued_tflops / FP32_MFMA_PEAK_TFLOPS, 4)}
    # The same step with the input handed over as a host buffer every time, as a caller of
    # CaffeNetForward with fresh images does: the copy over PCIe is inside the time.
    n_h2d = max(5, min(args.steps, 20))
    net.forward(**inputs)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n_h2d):
        net.forward(**inputs)
    torch.cuda.synchronize()
    el_h2d = time.perf_counter() - t0
    with_h2d = {"value_with_h2d": round(args.batch * n_h2d / el_h2d, 1),
                "ms_per_step_with_h2d": round(1e3 * el_h2d / n_h2d, 3), "steps_with_h2d": n_h2d,
                "h2d_bytes_per_step": int(sum(v.nbytes for v in inputs.values()))}

    # The same net with every convolution on the direct path (no Winograd), shorter: what
    # the implicit-GEMM kernel alone gives, for comparison with the figures above.
    direct = None
    if not args.no_winograd and not args.no_direct_comparison:
        LIB.mcConvWinogradDefault(0)
        net0 = mc.Net.from_buffers(craft.to_prototxt(spec, "ResNet-50"))
        craft.load_weights(net0, spec)
        net0.forward(**inputs)
        n0 = max(10, args.steps // 2)
        for _ in range(max(5, args.warmup // 2)):
            net0.forward()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n0):
            net0.forward()
        torch.cuda.synchronize()
        el0 = time.perf_counter() - t0
        LIB.mcConvTimingEnable(1)
        for _ in range(n0):
            net0.forward()
        LIB.mcConvTimingCollectDetail(ctypes.byref(tot_ms), ctypes.byref(launches), ctypes.byref(fl),
                                      ctypes.byref(issued), ctypes.byref(wino))
        LIB.mcConvTimingEnable(0)
        LIB.mcConvWinogradDefault(-1)
        rate0 = fl.value / (tot_ms.value * 1e-3) / 1e12
        direct = {"value": round(args.batch * n0 / el0, 1), "unit": "images/s", "steps": n0,
                  "ms_per_step": round(1e3 * el0 / n0, 3), "kernel_ms_per_step": round(tot_ms.value / n0, 3),
                  "achieved": round(rate0, 2), "frac": round(rate0 / FP32_MFMA_PEAK_TFLOPS, 4),
                  "note": "same net, mcConvWinogradDefault(0): all 53 convolutions on the direct implicit-GEMM path"}
        del net0

    two_threads = None if args.no_two_threads or args.no_direct_comparison else two_thread_throughput(mc, craft, zoo, args.batch,
                                                                         max(10, args.steps // 2))

    if args.configs_report:
        configs_report(args.configs_report, mc, craft, zoo, LIB)
    if args.layer_scaling:
        layer_scaling(args.layer_scaling)
    if args.layer_roofline:
        layer_roofline(args.layer_roofline, args.batch)
    if args.bandwidth_report:
        bandwidth_report(args.bandwidth_report)

    # the other two figures of the metric: convolution MFMA utilisation (hardware
    # counters, quoted from the committed counter run) and the detection tails
    del net
    tails = {} if args.no_detection_tails else detection_tails(mc, craft, zoo, LIB)
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(args.cpu_batch)

    out = {"metric": "images/sec at 1 MI355X (ResNet-50 b64 fp32)",
           "value": round(args.batch * args.steps / elapsed, 1), "unit": "images/s",
           "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
           "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak",
           "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": "ResNet-50 v1 forward, batch %d, 3x224x224, fp32 "
                                  "(BASELINE configs[1])" % args.batch,
                      "conv_gflop_per_step": round(flops["conv"] / 1e9, 1),
                      "api": "CaffeNetForward (Net::Forward(reshape=true))"},
           "timing_note": "the device needs about a second of load to settle: 20 steps after 5 warm-up steps read "
                          "2-3 % slower than the default 100 after 50 (the same library, the same box)",
           "roofline": roofline, "cpu_baseline": cpu,
           "conv_mfma_util_pct": mfma_util, "conv_mfma_util_source": mfma_note,
           "direct_path_only": direct, "two_host_threads": two_threads}
    out.update(with_h2d)
    out.update(tails)
    print(json.dumps(out))


def two_thread_throughput(mc, craft, zoo, batch, steps):
    """Two host threads, each with its own net of the same batch and its own stream (the
    runtime's context is per thread, as in the reference: tests/run_net.cpp:238-246 runs
    three such threads).  Launches of the two streams fill each other's last, partly
    empty rounds of workgroups.  Reported beside `value`, never as `value`: two batches
    are in flight and a step takes nearly twice as long."""
    import threading
    bar = threading.Barrier(2)
    took, errors = [0.0, 0.0], []

    def work(idx):
        try:
            mc.set_runtime_mode(1, 0)
            spec, inputs = zoo.resnet50_spec(batch=batch, size=224, seed=idx)
            net = mc.Net.from_buffers(craft.to_prototxt(spec, "ResNet-50"))
            craft.load_weights(net, spec)
            net.forward(**inputs)
            for _ in range(max(5, steps // 2)):
                net.forward()
            bar.wait()
            t0 = time.perf_counter()
            for _ in range(steps):
                net.forward()
            took[idx] = time.perf_counter() - t0
            bar.wait()
            prob = net.get_blob("prob").data
            assert abs(float(prob.sum()) - batch) < 1e-2 * batch
            del net
            mc.memory_pool_clear()
        except Exception as e:  # noqa: BLE001 - reported by the caller
            errors.append(repr(e))
            bar.abort()

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    if errors:
        return {"error": errors[0]}
    return {"value": round(2 * batch * steps / max(took), 1), "unit": "images/s", "threads": 2,
            "steps_per_thread": steps, "ms_per_step_per_thread": round(1e3 * max(took) / steps, 3),
            "note": "two host threads, each its own ResNet-50 b%d net, context and HIP stream, forwards "
                    "running concurrently; not the headline figure (two batches in flight)" % batch}


def detection_tails(mc, craft, zoo, LIB):
    """NMS / Proposal / DetectionOutput device time at the sizes of configurations 4 and 3,
    medians in microseconds.  Proposal: the layer inside the RPN net, through its stage hook.
    DetectionOutput: the SSD net runs once for locations and priors, the confidences are the
    softmax of N(0, sigma = 2) logits as configuration 3 states (the net's own confidences
    give a second figure); the tail is called alone through the kernel-level C ABI, 5 warm-up
    + 30 calls, each call between HIP events on its stream."""
    import statistics
    import numpy as np
    import torch
    from minicaffe import kernels as K
    P = ctypes.c_void_p
    stream = torch.cuda.current_stream().cuda_stream
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    out = {}

    # configuration 4: 1x1024x38x63 -> 21 546 anchors -> best 6000 -> NMS 0.7 -> 300 rois
    spec, inputs = zoo.rpn_spec(seed=0)
    net = mc.Net.from_buffers(craft.to_prototxt(spec, "rpn"))
    craft.load_weights(net, spec)
    net.mark_output("rpn_bbox_pred")
    net.forward(**inputs)
    bbox = net.get_blob("rpn_bbox_pred").data
    pp = spec[-1]["proposal_param"]
    pre, post, thr = pp.get("pre_nms_topn", 6000), pp.get("post_nms_topn", 300), pp.get("nms_thresh", 0.7)
    A, H, W = bbox.shape[1] // 4, bbox.shape[2], bbox.shape[3]
    # The Proposal layer of the net itself is what is timed (its own anchor table, its own
    # sequence of calls: the head of the score table first, the counters read back, the
    # full-size path only if the head did not settle the result).  The stage hook records
    # HIP events inside every call the layer makes.
    for _ in range(5):
        net.forward()
    stages, calls_seen = [], set()
    for _ in range(30):
        LIB.mcProposalTimingEnable(1)
        net.forward()
        LIB.mcProposalTimingEnable(0)
        ms, calls = (ctypes.c_double * 4)(), ctypes.c_long()
        K.check_mc(LIB.mcProposalTimingCollect(ms, ctypes.byref(calls)))
        stages.append([1e3 * v for v in ms])
        calls_seen.add(calls.value)
    kept = int(net.get_blob(spec[-1]["top"][0]).data.shape[0])
    del net
    med = [statistics.median(s[k] for s in stages) for k in range(4)]
    out["nms_us"] = round(med[1] + med[3], 1)
    out["proposal_us"] = round(statistics.median(sum(s) for s in stages), 1)
    out["proposal_detail"] = {
        "workload": "config 4: %d anchors -> best %d -> NMS %.1f -> <= %d rois (kept %d; the layer made %s "
                    "call(s) per forward: 1 = the head of the table settled the result, 2 = the full-size path "
                    "ran too)" % (A * H * W, pre, thr, post, kept, "/".join(str(c) for c in sorted(calls_seen))),
        "decode_head_order_us": round(med[0], 1), "head_nms_check_gather_us": round(med[1], 1),
        "full_sort_replay_us": round(med[2], 1), "full_nms_gather_us": round(med[3], 1),
        "nms_us_is": "head_nms_check_gather_us + full_nms_gather_us",
        "method": "the net's Proposal layer on the net's own scores, HIP events between the stages of each "
                  "call the layer makes (device time; the read-back between the calls is not in it), median of "
                  "30 forwards"}

    # configuration 3: SSD300 b8, 8732 priors x 21 classes, top_k 400, NMS 0.45, keep 200
    spec, inputs = zoo.ssd300_spec(batch=8, seed=0)
    net = mc.Net.from_buffers(craft.to_prototxt(spec, "ssd"))
    craft.load_weights(net, spec)
    for m in ("mbox_loc", "mbox_conf_flatten", "mbox_priorbox"):
        net.mark_output(m)
    net.forward(**inputs)
    loc, conf, prior = (dev(net.get_blob(m).data.copy()) for m in ("mbox_loc", "mbox_conf_flatten", "mbox_priorbox"))
    del net
    dp = spec[-1]["detection_output_param"]
    num, Pn, C = loc.shape[0], prior.shape[2] // 4, dp["num_classes"]
    nmsp = dp["nms_param"]
    code = {"CORNER": 1, "CENTER_SIZE": 2, "CORNER_SIZE": 3}[str(dp.get("code_type", "CORNER"))]
    sz = ctypes.c_size_t()
    cnt = torch.zeros(2, dtype=torch.int32, device="cuda")
    K.check_mc(LIB.mcDetectionOutputWorkspaceSize(num, Pn, C, 1, nmsp["top_k"], ctypes.byref(sz)))
    max_rows = LIB.mcDetectionOutputMaxRows(num, Pn, C, nmsp["top_k"], dp["keep_top_k"])
    ws = torch.empty(sz.value, dtype=torch.uint8, device="cuda")
    rows = torch.empty((max_rows, 7), device="cuda")

    thr_conf = dp.get("confidence_threshold", -3.4028234663852886e38)

    def detect():
        K.check_mc(LIB.mcDetectionOutput(
            P(loc.data_ptr()), P(conf.data_ptr()), P(prior.data_ptr()), num, Pn, C, 1, dp.get("background_label_id", 0),
            code, 0, dp["keep_top_k"], ctypes.c_float(thr_conf),
            ctypes.c_float(nmsp["nms_threshold"]), ctypes.c_float(nmsp.get("eta", 1.0)), nmsp["top_k"],
            P(ws.data_ptr()), sz.value, P(rows.data_ptr()), max_rows, P(cnt.data_ptr()), P(cnt.data_ptr() + 4),
            P(stream)))

    def timed_detect():
        for _ in range(5):
            detect()
        torch.cuda.synchronize()
        spans = []
        for _ in range(30):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            detect()
            e1.record()
            spans.append((e0, e1))
        torch.cuda.synchronize()
        return round(1e3 * statistics.median(a.elapsed_time(b) for a, b in spans), 1), int(cnt[0])

    own_us, own_rows = timed_detect()
    # configuration 3's confidences: logits ~ N(0, sigma = 2) per (image, prior, class), softmax over classes
    logits = torch.randn((num, Pn, C), generator=torch.Generator().manual_seed(3)) * 2.0
    conf = torch.softmax(logits, dim=2).reshape(num, Pn * C).contiguous().cuda()
    us, rows_n = timed_detect()
    out["detection_output_us"] = us
    out["detection_output_detail"] = {
        "workload": "config 3: %d images x %d priors x %d classes, confidences = softmax of N(0, sigma=2) logits, "
                    "confidence_threshold %.2f, top_k %d, NMS %.2f, keep %d (rows %d)"
                    % (num, Pn, C, thr_conf, nmsp["top_k"], nmsp["nms_threshold"], dp["keep_top_k"], rows_n),
        "on_the_nets_own_confidences_us": own_us, "on_the_nets_own_confidences_rows": own_rows,
        "method": "mcDetectionOutput alone (locations and priors from the net), HIP events on the launch stream, "
                  "median of 30 calls"}
    return out


def configs_report(path, mc, craft, zoo, LIB):
    """Whole-forward time, contraction TFLOP/s and detection-tail layer time of the five
    BASELINE configurations (plus MobileNet-SSD) on the GPU (synthetic inputs and weights from the zoo builders)."""
    import tempfile
    import oracle
    from oracle import netrun
    oracle.use_openblas(True)
    # (name, GPU spec, tail layers, batch, CPU-sample spec at a reduced batch, its batch)
    cases = [("C1 conv3x3+ReLU 1x64x56x56", zoo.c1_spec(seed=0), (), 1, zoo.c1_spec(seed=0), 1),
             ("C2 ResNet-50 b64", zoo.resnet50_spec(batch=64, size=224, seed=0), (), 64,
              zoo.resnet50_spec(batch=4, size=224, seed=0), 4),
             ("C3 SSD300-VGG16 b8", zoo.ssd300_spec(batch=8, seed=0), ("detection_out",), 8,
              zoo.ssd300_spec(batch=1, seed=0), 1),
             ("C4 RPN+Proposal 1x1024x38x63", zoo.rpn_spec(seed=0), ("proposal",), 1, zoo.rpn_spec(seed=0), 1),
             ("C5 DCGAN generator b128", zoo.dcgan_spec(batch=128, seed=0), (), 128,
              zoo.dcgan_spec(batch=8, seed=0), 8),
             # not a BASELINE configuration: the depthwise-separable graph of the reference's ssd example
             ("+  MobileNet-SSD b32", zoo.mobilenet_ssd_spec(batch=32, seed=0), ("detection_out",), 32,
              zoo.mobilenet_ssd_spec(batch=2, seed=0), 2)]
    lines = ["%-30s %10s %10s %12s %12s %10s %8s %12s %12s  %s"
             % ("configuration", "ms/forward", "GFLOP", "contr. ms", "dir-eq TF/s", "issued TF/s", "of peak",
                "GPU img/s", "CPU img/s", "tail layers (us, device time)")]
    for name, (spec, inputs), tails, batch, (cspec, cinputs), cbatch in cases:
        net = mc.Net.from_buffers(craft.to_prototxt(spec, "net"))
        craft.load_weights(net, spec)
        net.forward(**inputs)
        reps = 20
        for _ in range(3):
            net.forward()
        t0 = time.perf_counter()
        for _ in range(reps):
            net.forward()
        ms = 1e3 * (time.perf_counter() - t0) / reps
        LIB.mcConvTimingEnable(1)
        for _ in range(reps):
            net.forward()
        tot_ms, launches, fl = ctypes.c_double(), ctypes.c_long(), ctypes.c_double()
        issued, wino = ctypes.c_double(), ctypes.c_long()
        LIB.mcConvTimingCollectDetail(ctypes.byref(tot_ms), ctypes.byref(launches), ctypes.byref(fl),
                                      ctypes.byref(issued), ctypes.byref(wino))
        LIB.mcConvTimingEnable(0)
        tail_txt = ""
        if tails:
            # per-layer device time: the profiler synchronises the stream at every scope
            mc.Profiler.enable()
            for _ in range(reps):
                net.forward()
            mc.Profiler.disable()
            with tempfile.NamedTemporaryFile(suffix=".json") as tf:
                mc.Profiler.dump(tf.name)
                events = json.load(open(tf.name))["traceEvents"]
            begin, spans = {}, {}
            for e in events:
                if e["ph"] == "B":
                    begin[e["name"]] = e["ts"]
                elif e["name"] in begin:
                    spans.setdefault(e["name"], []).append(e["ts"] - begin.pop(e["name"]))
            # the profiler keeps the scopes of earlier configurations: the last `reps` are this net's
            last = {t: spans[t][-reps:] for t in tails if t in spans}
            tail_txt = ", ".join("%s %.0f (median of %d)" % (t, sorted(v)[len(v) // 2], len(v))
                                 for t, v in last.items())
        cms = tot_ms.value / reps
        tf_s = fl.value / (tot_ms.value * 1e-3) / 1e12 if tot_ms.value else 0.0
        is_s = issued.value / (tot_ms.value * 1e-3) / 1e12 if tot_ms.value else 0.0
        # CPU path (oracle restatement of the reference, OpenBLAS sgemm, all host cores): one
        # pass at the reduced batch
        last = cspec[-1]["top"][0]
        t0 = time.perf_counter()
        netrun.oracle_forward(cspec, cinputs, keep={last})
        cpu_rate = cbatch / (time.perf_counter() - t0)
        lines.append("%-30s %10.3f %10.2f %12.3f %12.1f %10.1f %7.1f%% %12.1f %12.2f  %s"
                     % (name, ms, fl.value / reps / 1e9, cms, tf_s, is_s, 100 * is_s / FP32_MFMA_PEAK_TFLOPS,
                        batch / (ms * 1e-3), cpu_rate, tail_txt))
        del net
    lines.append("dir-eq TF/s: the contractions' direct-sum FLOPs over the device time of their launches (a 3x3 layer on "
                 "the Winograd path counts with its direct-sum FLOPs, so this rate can pass the matrix peak); issued "
                 "TF/s / of peak: what the matrix pipe was handed in the same time, against 157.3 TFLOP/s.")
    lines.append("CPU column: one pass of the oracle (reference algorithm: per-image im2col + OpenBLAS sgemm, "
                 "unfused layers) on %d host threads at batch 1/4/1/1/8/2." % oracle.openblas_threads())
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def layer_scaling(path):
    """One convolution launch of the implicit-GEMM kernel (ReLU epilogue, pinned to the direct
    path) at growing batch sizes: time per launch and TFLOP/s, through the kernel-level C ABI
    on torch-owned device memory; the 3x3 layers that the library would run as Winograd are
    listed a second time on that path (algorithmic TFLOP/s: the direct sum's FLOPs)."""
    import torch
    from minicaffe import kernels as K
    # cin, height = width, cout, kernel, stride, pad: shapes of ResNet-50 stages 2-5
    shapes = [(64, 56, 64, 3, 1, 1), (64, 56, 256, 1, 1, 0), (256, 56, 64, 1, 1, 0), (128, 28, 128, 3, 1, 1),
              (256, 14, 256, 3, 1, 1), (1024, 14, 256, 1, 1, 0), (256, 14, 1024, 1, 1, 0),
              (512, 7, 512, 3, 1, 1), (2048, 7, 512, 1, 1, 0)]
    batches = (16, 32, 64, 128, 256, 512)
    lines = ["%-22s" % "convolution" + "".join("%16s" % ("batch %d" % n) for n in batches)]
    stream = torch.cuda.current_stream().cuda_stream
    wino = [sh + (1,) for sh in shapes if sh[3] == 3 and sh[0] >= 128]
    for cin, h, cout, k, s, p, mode in [sh + (0,) for sh in shapes] + wino:
        cells = []
        for n in batches:
            if n * max(cin, cout) * h * h > 2 ** 28 or (mode == 1 and 4 * n * max(cin, cout) * h * h >= 2 ** 29):
                cells.append("%16s" % "-")
                continue
            plan = K.ConvPlan(K.conv_geom(cin, h, h, cout, k, s, p))
            plan.force_winograd(mode)
            ho, wo = plan.output_shape()
            x = torch.randn(n, cin, h, h, device="cuda")
            w = torch.randn(cout, cin, k, k, device="cuda") * 0.05
            y = torch.empty(n, cout, ho, wo, device="cuda")
            plan.set_weights(w.data_ptr())
            for _ in range(3):
                plan.forward(n, x.data_ptr(), y.data_ptr(), activation=K.ACT_RELU, stream=stream)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 10
            e0.record()
            for _ in range(reps):
                plan.forward(n, x.data_ptr(), y.data_ptr(), activation=K.ACT_RELU, stream=stream)
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / reps
            cells.append("%8.0f us %4.0f" % (ms * 1e3, plan.flops(n) / ms / 1e9))
            del x, y, w, plan
        lines.append("%-22s" % ("%d->%d %dx%d @%d%s" % (cin, cout, k, k, h, " W" if mode else "")) + "".join(cells))
    lines.append("cells: time per launch (10 back-to-back launches between two events) and TFLOP/s; W = the layer as "
                 "F(2x2,3x3) Winograd (one fused launch; TFLOP/s in the direct sum's FLOPs, which can exceed the matrix peak)")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def layer_roofline(path, batch):
    """Every distinct convolution of ResNet-50 v1 alone (ReLU epilogue, no residual), one
    launch at a time through the kernel-level C ABI: which roofline binds it and how close
    the launch comes.  Bytes = bottom + top + filter, each once.  Two rates per layer: the
    direct sum's FLOPs over the time (what the layer is worth; a Winograd launch can exceed
    the matrix peak on this scale, so no fraction is printed for it) and the FLOPs the matrix
    pipe was handed (padding of tiles included, 2.25 times fewer products on the Winograd
    path) with their share of the fp32 peak."""
    import torch
    from minicaffe import kernels as K
    from minicaffe.base import LIB
    # cin, height = width, cout, kernel, stride, pad, number of layers of this shape
    shapes = [(3, 224, 64, 7, 2, 3, 1), (64, 56, 256, 1, 1, 0, 4), (64, 56, 64, 1, 1, 0, 1), (64, 56, 64, 3, 1, 1, 3),
              (256, 56, 64, 1, 1, 0, 2), (256, 56, 512, 1, 2, 0, 1), (256, 56, 128, 1, 2, 0, 1), (128, 28, 128, 3, 1, 1, 4),
              (128, 28, 512, 1, 1, 0, 4), (512, 28, 128, 1, 1, 0, 3), (512, 28, 1024, 1, 2, 0, 1), (512, 28, 256, 1, 2, 0, 1),
              (256, 14, 256, 3, 1, 1, 6), (256, 14, 1024, 1, 1, 0, 6), (1024, 14, 256, 1, 1, 0, 5),
              (1024, 14, 2048, 1, 2, 0, 1), (1024, 14, 512, 1, 2, 0, 1), (512, 7, 512, 3, 1, 1, 3),
              (512, 7, 2048, 1, 1, 0, 3), (2048, 7, 512, 1, 1, 0, 2)]
    stream = torch.cuda.current_stream().cuda_stream
    lines = ["%-24s %3s %8s %9s %8s %6s %9s %9s %11s %9s %8s" % (
        "convolution (batch %d)" % batch, "x", "GFLOP", "MB", "FLOP/B", "bound", "roof us", "meas. us",
        "direct-eq.", "issued", "issued")]
    lines.append("%-24s %3s %8s %9s %8s %6s %9s %9s %11s %9s %8s" % (
        "", "", "", "", "", "", "", "", "TFLOP/s", "TFLOP/s", "of peak"))
    sum_roof = sum_meas = sum_issued = 0.0
    for cin, h, cout, k, s_, p_, cnt in shapes:
        plan = K.ConvPlan(K.conv_geom(cin, h, h, cout, k, s_, p_))
        ho, wo = plan.output_shape()
        x = torch.randn(batch, cin, h, h, device="cuda")
        w = torch.randn(cout, cin, k, k, device="cuda") * 0.05
        y = torch.empty(batch, cout, ho, wo, device="cuda")
        plan.set_weights(w.data_ptr())
        fl = plan.flops(batch)
        nbytes = 4.0 * (x.numel() + y.numel() + w.numel())
        t_mfma, t_hbm = fl / (FP32_MFMA_PEAK_TFLOPS * 1e6), nbytes / (HBM_PEAK_GBS * 1e3)
        roof = max(t_mfma, t_hbm)
        winograd = plan.kernel_name(batch) == "winograd_f32"
        # a layer the library runs on the Winograd path is also timed on the direct one
        for mode in ((-1, 0) if winograd else (-1,)):
            plan.force_winograd(mode)
            for _ in range(5):
                plan.forward(batch, x.data_ptr(), y.data_ptr(), activation=K.ACT_RELU, stream=stream)
            torch.cuda.synchronize()
            reps = 20
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(reps):
                plan.forward(batch, x.data_ptr(), y.data_ptr(), activation=K.ACT_RELU, stream=stream)
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) / reps * 1e3
            # what the launch hands the matrix pipe: from the library's own count
            LIB.mcConvTimingEnable(1)
            plan.forward(batch, x.data_ptr(), y.data_ptr(), activation=K.ACT_RELU, stream=stream)
            tot_ms, launches, fl_c = ctypes.c_double(), ctypes.c_long(), ctypes.c_double()
            issued, wino = ctypes.c_double(), ctypes.c_long()
            LIB.mcConvTimingCollectDetail(ctypes.byref(tot_ms), ctypes.byref(launches), ctypes.byref(fl_c),
                                          ctypes.byref(issued), ctypes.byref(wino))
            LIB.mcConvTimingEnable(0)
            if mode == -1:
                sum_roof += roof * cnt
                sum_meas += us * cnt
                sum_issued += issued.value * cnt
            lines.append("%-24s %3d %8.2f %9.1f %8.1f %6s %9.1f %9.1f %11.1f %9.1f %7.1f%%  %s" % (
                "%d->%d %dx%d/%d @%d" % (cin, cout, k, k, s_, h), cnt, fl / 1e9, nbytes / 1e6, fl / nbytes,
                "mfma" if t_mfma >= t_hbm else "hbm", roof, us, fl / us / 1e6, issued.value / us / 1e6,
                100 * issued.value / us / 1e6 / FP32_MFMA_PEAK_TFLOPS,
                "" if not winograd else ("Winograd F(2x2,3x3), one fused launch" if mode == -1
                                         else "(same layer pinned to the direct path; not in the total)")))
        del x, y, w, plan
    lines.append("all 53 convolutions: direct-sum roofline %.0f us, measured %.0f us (direct-sum equivalent %.1f%% of the "
                 "per-layer roofline); issued to the matrix pipe: %.1f%% of the fp32 peak over the same time"
                 % (sum_roof, sum_meas, 100 * sum_roof / sum_meas,
                    100 * sum_issued / sum_meas / 1e6 / FP32_MFMA_PEAK_TFLOPS))
    lines.append("roof us = max(FLOP / 157.3 TFLOP/s, bytes / 8 TB/s) with the FLOPs and bytes of the direct sum; 20 "
                 "back-to-back calls between two events.")
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def bandwidth_report(path):
    """The kernels whose bound is HBM, alone, through the kernel-level C ABI on torch-owned
    device memory.  Two figures per kernel: `cold` rotates over enough copies of the
    operands to exceed twice the 256 MB last-level cache and times 40 back-to-back
    launches between two HIP events (what HBM gives; launch overhead amortised);
    `one launch` is the median of 100 launches of one operand set, each between its own
    two events (includes about 6 us of event and launch overhead; small operands come
    from the cache).  Algorithmic bytes = 4 * (elements read + elements written),
    parameters left out; Normalize counts its input twice (12 bytes per element)."""
    import statistics
    import torch
    from minicaffe import kernels as K
    from minicaffe.base import LIB
    stream = torch.cuda.current_stream().cuda_stream
    P = ctypes.c_void_p
    ints = lambda v: (ctypes.c_int * len(v))(*v)  # noqa: E731
    rows = []

    def sets_for(nbytes):
        return max(2, min(64, int(2 * 256e6 // max(nbytes, 1)) + 1))

    def timed(name, nbytes, make):
        """make() -> (launch, keepalive) for a fresh operand set."""
        k = sets_for(nbytes)
        launches = [make() for _ in range(k)]
        for fn, _ in launches:
            rc = fn()
            assert rc in (0, None), LIB.mcLastError()
        torch.cuda.synchronize()
        reps = 40
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for i in range(reps):
            launches[i % k][0]()
        e1.record()
        torch.cuda.synchronize()
        cold_us = e0.elapsed_time(e1) / reps * 1e3
        fn = launches[0][0]
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        spans = []
        for _ in range(100):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            spans.append((a, b))
        torch.cuda.synchronize()
        one_us = statistics.median(a.elapsed_time(b) for a, b in spans) * 1e3
        gbs = nbytes / cold_us / 1e3
        rows.append("%-58s %9.1f MB %3d sets %9.1f us %8.0f GB/s %6.1f %% %11.1f us"
                    % (name, nbytes / 1e6, k, cold_us, gbs, gbs / HBM_PEAK_GBS * 100, one_us))

    dev = lambda *shape: torch.randn(*shape, device="cuda")  # noqa: E731

    def pool(name, method, planes, h, w, k, s_, pad):
        ho, wo = ctypes.c_int(), ctypes.c_int()
        LIB.mcPoolingOutputShape(h, w, k, k, s_, s_, pad, pad, ctypes.byref(ho), ctypes.byref(wo))

        def make():
            x, y = dev(planes, h, w), dev(planes, ho.value, wo.value)
            return (lambda: LIB.mcPooling(method, P(x.data_ptr()), P(y.data_ptr()), planes, h, w, k, k, s_, s_,
                                          pad, pad, P(stream))), (x, y)
        timed(name, 4 * (planes * h * w + planes * ho.value * wo.value), make)

    pool("Pooling MAX 3x3/2, 64x64x112x112 (ResNet-50 stem)", 0, 64 * 64, 112, 112, 3, 2, 0)
    pool("Pooling MAX 2x2/2, 8x64x300x300 (SSD300 pool1)", 0, 8 * 64, 300, 300, 2, 2, 0)
    pool("Pooling MAX 3x3/1 pad 1, 8x512x19x19 (SSD300 pool5)", 0, 8 * 512, 19, 19, 3, 1, 1)
    pool("Pooling AVE 7x7 global, 64x2048x7x7 (ResNet-50 pool5)", 1, 64 * 2048, 7, 7, 7, 1, 0)

    n, c, sp = 64, 256, 56 * 56
    numel = n * c * sp

    def make_eltwise():
        a, b, y = dev(n, c, sp), dev(n, c, sp), dev(n, c, sp)
        bottoms = (ctypes.c_void_p * 2)(a.data_ptr(), b.data_ptr())
        coeffs = (ctypes.c_float * 2)(1.0, 1.0)
        return (lambda: LIB.mcEltwise(1, 2, bottoms, coeffs, numel, P(y.data_ptr()), 1, 0.0, P(stream))), (a, b, y, bottoms, coeffs)
    timed("Eltwise SUM + ReLU, 2 x 64x256x56x56 (residual, unfused)", 4 * 3 * numel, make_eltwise)
    mul, add = dev(c), dev(c)
    op = K.ChannelOp(None, None, mul.data_ptr(), add.data_ptr(), 1, 0.0)

    def unary_like(call):
        def make():
            a, y = dev(n, c, sp), dev(n, c, sp)
            return (lambda: call(a, y)), (a, y)
        return make
    timed("channel transform x*g+b, ReLU, 64x256x56x56 (BN/Scale/ReLU)", 4 * 2 * numel, unary_like(
        lambda a, y: LIB.mcChannelTransform(P(a.data_ptr()), P(y.data_ptr()), n, c, sp, ctypes.byref(op), P(stream))))
    timed("Unary ELU, 64x256x56x56", 4 * 2 * numel, unary_like(
        lambda a, y: LIB.mcUnary(5, P(a.data_ptr()), P(y.data_ptr()), numel, 1.0, 0.0, 0.0, P(stream))))
    timed("PReLU, one slope per channel, 64x256x56x56", 4 * 2 * numel, unary_like(
        lambda a, y: LIB.mcPReLU(P(a.data_ptr()), P(y.data_ptr()), n, c, sp, P(mul.data_ptr()), 0, P(stream))))
    timed("copy (Concat / Slice / Split), 64x256x56x56", 4 * 2 * numel, unary_like(
        lambda a, y: LIB.mcCopy2D(P(a.data_ptr()), numel, P(y.data_ptr()), numel, numel, 1, P(stream))))
    shape, order = ints([n, c, 56, 56]), ints([0, 2, 3, 1])
    timed("Permute (0,2,3,1), 64x256x56x56", 4 * 2 * numel, unary_like(
        lambda a, y: LIB.mcPermute(P(a.data_ptr()), P(y.data_ptr()), 4, shape, order, P(stream))))

    def simple(shape_, call):
        def make():
            x, y = dev(*shape_), dev(*shape_)
            return (lambda: call(x, y)), (x, y)
        return make
    shape2 = ints([8, 84, 38, 38])
    timed("Permute (0,2,3,1), 8x84x38x38 (SSD300 conv4_3 conf head)", 4 * 2 * 8 * 84 * 38 * 38, simple(
        (8, 84, 38, 38), lambda x, y: LIB.mcPermute(P(x.data_ptr()), P(y.data_ptr()), 4, shape2, order, P(stream))))
    timed("Softmax over 21 classes, 8x8732 rows (SSD300 mbox_conf)", 4 * 2 * 8 * 8732 * 21, simple(
        (8 * 8732, 21), lambda x, y: LIB.mcSoftmax(P(x.data_ptr()), P(y.data_ptr()), 8 * 8732, 21, 1, P(stream))))
    timed("Softmax over 1000 classes, 64 rows (ResNet-50 prob)", 4 * 2 * 64 * 1000, simple(
        (64, 1000), lambda x, y: LIB.mcSoftmax(P(x.data_ptr()), P(y.data_ptr()), 64, 1000, 1, P(stream))))
    sc = dev(512)
    timed("Normalize across channels, 8x512x38x38 (SSD300 conv4_3_norm)", 4 * 3 * 8 * 512 * 38 * 38, simple(
        (8, 512, 38 * 38), lambda x, y: LIB.mcNormalize(P(x.data_ptr()), P(y.data_ptr()), 8, 512, 38 * 38, 0, 0, 1e-10,
                                                         P(sc.data_ptr()), P(stream))))
    timed("LRN across 5 channels, 64x96x55x55 (AlexNet norm1)", 4 * 2 * 64 * 96 * 55 * 55, simple(
        (64, 96, 55, 55), lambda x, y: LIB.mcLRNAcrossChannels(P(x.data_ptr()), P(y.data_ptr()), 64, 96, 55, 55, 5, 1e-4,
                                                               0.75, 1.0, P(stream))))
    for cin, h, s_ in ((512, 19, 1), (256, 38, 2), (64, 150, 1)):
        plan = K.ConvPlan(K.conv_geom(cin, h, h, cin, 3, s_, 1, group=cin))
        ho, wo = plan.output_shape()
        w = dev(cin, 1, 3, 3)
        plan.set_weights(w.data_ptr())

        def make():
            x, y = dev(32, cin, h, h), dev(32, cin, ho, wo)
            return (lambda: plan.forward(32, x.data_ptr(), y.data_ptr(), activation=K.ACT_RELU, stream=stream)), (x, y)
        timed("depthwise 3x3/%d + ReLU, 32x%dx%dx%d (MobileNet)" % (s_, cin, h, h),
              4 * 32 * cin * (h * h + ho * wo), make)
        del plan
    # the plain copy at the sizes of the small launches above: what a launch of that size can reach at all
    for label, nel in (("the 19x19 depthwise launch", 32 * 512 * 19 * 19), ("Normalize", 8 * 512 * 38 * 38),
                       ("LRN", 64 * 96 * 55 * 55)):
        def make(nel=nel):
            a, y = dev(nel), dev(nel)
            return (lambda: LIB.mcCopy2D(P(a.data_ptr()), nel, P(y.data_ptr()), nel, nel, 1, P(stream))), (a, y)
        timed("copy of the size of %s" % label, 4 * 2 * nel, make)
    head = ["%-58s %12s %8s %12s %13s %8s %14s" % ("kernel, shape", "alg. bytes", "operands", "cold", "achieved",
                                                  "of 8 TB/s", "one launch")]
    tail = ["cold: 40 back-to-back launches between two HIP events, rotating over `operands` sets (more than 512 MB",
            "in total, twice the last-level cache), so every launch reads from and writes to HBM.",
            "one launch: median of 100 launches of one operand set, each between its own two events: includes",
            "about 6 us of event and launch overhead, and operands below 256 MB come from the last-level cache."]
    with open(path, "w") as f:
        f.write("\n".join(head + rows + tail) + "\n")


def cpu_baseline(batch):
    """The reference algorithm (per-image im2col + sgemm, unfused BN/Scale/ReLU)
    as restated by the oracle, sgemm from the OpenBLAS bundled with scipy."""
    import oracle
    from oracle import netrun
    from minicaffe import zoo
    blas = oracle.use_openblas(True)
    spec, inputs = zoo.resnet50_spec(batch=batch, size=224, seed=0)
    netrun.oracle_forward(spec, {k: v[:1] for k, v in inputs.items()}, keep={"prob"})  # warm
    t0 = time.perf_counter()
    reps = 0
    while True:
        netrun.oracle_forward(spec, inputs, keep={"prob"})
        reps += 1
        if time.perf_counter() - t0 > 10.0 or reps >= 5:
            break
    dt = time.perf_counter() - t0
    return {"value": round(batch * reps / dt, 2), "unit": "images/s",
            "cores": oracle.openblas_threads() if blas else 1, "kind": "port",
            "blas": os.path.basename(blas) if blas else "built-in loops",
            "sample": "%d pass(es) of ResNet-50 forward at batch %d (same graph, same seeds)"
                      % (reps, batch)}


if __name__ == "__main__":
    main()
