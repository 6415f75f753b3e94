#!/usr/bin/env python3
"""Benchmark of the binary-convolution forward path on one MI355X.

One step = one forward pass (binarize_data + calculate_k + XNOR/popcount convolution; the
same three-part split the reference reports in README.md:29-32) over one batch of
synthetic input that is already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--no-cold]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
# the CPU baseline's OpenMP threads stay on neighbouring cores (set before any OpenMP runtime
# starts; the GPU legs do not depend on it)
os.environ.setdefault("OMP_PROC_BIND", "close")

METRIC = "ms/forward + effective binary GOPS, AlexNet conv4 N=256 on 1 MI355X"
HBM_PEAK_GBS = 8000.0
MFMA_FP4_PEAK_TOPS = 10100.0
INFINITY_CACHE_BYTES = 256 << 20


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` on `workload`, from the committed rocprofv3 --pmc
    summary profiles/<workload>_hbm_traffic_pmc.txt (FETCH_SIZE / WRITE_SIZE in KiB per
    dispatch, each scaled by what the same counter shows for a plain copy of known size).
    The counters need profiler runs of their own, so this script cannot measure them; it
    reads the line "traffic_bytes <kernel variant> read=R written=W" of the summary and
    returns None when there is no summary or it was taken with another kernel variant."""
    path = os.path.join(ROOT, "profiles", workload + "_hbm_traffic_pmc.txt")
    if not os.path.exists(path):
        return None
    for line in open(path):
        f = line.split()
        if len(f) == 4 and f[0] == "traffic_bytes" and f[1] == kernel:
            return int(f[2].split("=")[1]) + int(f[3].split("=")[1])
    return None


def work_figures(d):
    """Algorithmic work of one forward pass (bytes for the streaming stages, binary ops
    for the convolution)."""
    mb, ic, ih, iw, oc = d["mb"], d["ic"], d["ih"], d["iw"], d["oc"]
    kh, kw, sh, sw, ph, pw = d["kh"], d["kw"], d["sh"], d["sw"], d["ph"], d["pw"]
    oh = (ih + 2 * pw - kh) // sh + 1
    ow = (iw + 2 * pw - kw) // sw + 1
    taps = 0
    for o_h in range(oh):
        for o_w in range(ow):
            vh = sum(1 for k in range(kh) if 0 <= o_h * sh - ph + k < ih)
            vw = sum(1 for k in range(kw) if 0 <= o_w * sw - pw + k < iw)
            taps += vh * vw
    bic = (ic + 7) // 8
    return {
        "oh": oh, "ow": ow,
        "nominal_ops": 2 * mb * oc * oh * ow * ic * kh * kw,
        "exact_ops": 2 * mb * oc * ic * taps,
        # fused binarize + mean|x| pass: read x once, write bits and a
        "binarize_bytes": 4 * mb * ic * ih * iw + mb * ih * iw * bic + 4 * mb * ih * iw,
        # convolution: read packed input and FP4/packed weights once, k, write fp32 output
        "conv_bytes": mb * ih * iw * bic + oc * kh * kw * bic + 4 * mb * oh * ow
                      + 4 * mb * oc * oh * ow,
        # box filter: read a, write k
        "k_bytes": 4 * mb * ih * iw + 4 * mb * oh * ow,
    }


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(d, x, w, threads):
    """The CPU path timed on this host, methodology of the reference's own benchmark
    (reference test/perf/test_simple_net.cpp:39-60: per-stage timers around repeated forward
    passes, minimum reported; the median is given beside it because this host is shared):
    the compiled upstream library when it was built (oracle/_ref, kind "reference") and the
    in-repo C restatement (oracle/, kind "port"), each on the whole workload, OpenMP on all
    host threads with OMP_PROC_BIND=close.  Baselines only; never the product.  Returns
    (headline entry, all entries): the reference when it is there, else the port."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import checkers
    reps = 7 if d["mb"] * d["oc"] * d["ih"] * d["iw"] < 5e7 else 5
    nominal = work_figures(d)["nominal_ops"]

    def entry(kind, passes):
        # passes: (t0, t1, t2, t3) per forward pass, the first one (warm-up) already dropped
        totals = sorted(1e3 * (p[3] - p[0]) for p in passes)
        best = min(passes, key=lambda p: p[3] - p[0])
        stages = [1e3 * (best[i + 1] - best[i]) for i in range(3)]
        ms, median = totals[0], totals[len(totals) // 2]
        return {
            "value": nominal / (ms * 1e-3) / 1e9, "unit": "GOPS",
            "ms_per_forward": ms, "ms_per_forward_median": median,
            "ms_per_forward_all": totals,
            "value_at_median": nominal / (median * 1e-3) / 1e9,
            "stage_ms": {"binarize_data": stages[0], "calculate_k": stages[1],
                         "forward": stages[2]},
            "cores": threads, "kind": kind, "cpu": cpu_model(),
            "sample": "whole workload, minimum (and median) of %d forward passes after one "
                      "warm-up (OpenMP, %d threads, OMP_PROC_BIND=%s%s)" % (
                          len(passes), threads, os.environ.get("OMP_PROC_BIND", "unset"),
                          ", XNOR_NN_ISA=2: AVX kernels" if kind == "reference" else ""),
        }

    entries = []
    if checkers.have_ref():
        ref = checkers.RefLib()
        out = ref.forward(d, x, w, reps=reps + 1, timer=time.perf_counter)
        entries.append(entry("reference", out["times"][1:]))
    from util import oracle_shape
    oracle = checkers.Oracle()
    s = oracle_shape(oracle, d)
    bw, alpha, opc = oracle.binarize_weights(s, w)
    passes = []
    for _ in range(reps + 1):
        t0 = time.perf_counter()
        bsrc = oracle.binarize_data(s, x)
        t1 = time.perf_counter()
        a, k = oracle.calculate_k(s, x)
        t2 = time.perf_counter()
        oracle.convolution(s, bsrc, bw, alpha, k, opc)
        t3 = time.perf_counter()
        passes.append((t0, t1, t2, t3))
    entries.append(entry("port", passes[1:]))
    return entries[0], entries


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="alexnet_conv4_mb256")
    ap.add_argument("--mb", type=int, default=None,
                    help="override the batch size of the workload (experiments only)")
    ap.add_argument("--shape", default=None, metavar="MB,IC,OC,IH,IW,KH,KW,SH,SW,PH,PW",
                    help="another layer instead of a named workload (experiments only): N(0,1) "
                         "input and N(0,0.05) weights of this shape, NCHW/OIHW/NCHW")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-cold", action="store_true",
                    help="skip the leg that rotates through more buffers than the cache holds")
    ap.add_argument("--cold-only", action="store_true",
                    help="profiling aid: every step of the run, warm-up included, rotates "
                         "through the buffer pairs, so that a kernel trace of the run holds "
                         "cold launches only")
    ap.add_argument("--binarize-only", action="store_true",
                    help="profiling aid, with --cold-only: the rotation runs the binarize "
                         "stage alone (no convolution output waiting in the caches to be "
                         "written back while it reads)")
    ap.add_argument("--no-host", action="store_true",
                    help="skip the three forward passes through host buffers")
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="after the timed region, run one plain device-to-device copy of "
                         "this many MiB (a kernel of known traffic to scale rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE readings with)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py measures one GPU: every image of the batch is independent, so "
                 "more GPUs would only split the batch; run with --gpus 1")

    import torch
    from xnor_nn_amd import Convolution, capi, synth

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the library has no CPU path)")
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(0)
    import ctypes
    c_cus, c_khz = ctypes.c_int(0), ctypes.c_int(0)
    if capi.load().xnor_nn_hip_device_info(ctypes.byref(c_cus), ctypes.byref(c_khz)) != 0:
        sys.exit("cannot query the HIP device")
    cus, clk_hz = c_cus.value, c_khz.value * 1e3

    if args.shape:
        dims = [int(v) for v in args.shape.split(",")]
        if len(dims) != 11 or min(dims) < 0:
            sys.exit("--shape takes MB,IC,OC,IH,IW,KH,KW,SH,SW,PH,PW")
        d = dict(zip(("mb", "ic", "oc", "ih", "iw", "kh", "kw", "sh", "sw", "ph", "pw"), dims))
        x = synth.normal(synth.SEED_SRC, d["mb"] * d["ic"] * d["ih"] * d["iw"]).reshape(
            d["mb"], d["ic"], d["ih"], d["iw"])
        w = synth.normal(synth.SEED_WEIGHTS, d["oc"] * d["ic"] * d["kh"] * d["kw"], 0.05).reshape(
            d["oc"], d["ic"], d["kh"], d["kw"])
        args.workload = "shape:" + args.shape
    else:
        d, x, w = synth.make_workload(args.workload, args.mb)
    wf = work_figures(d)
    xt = torch.from_numpy(x).to(dev)
    wt = torch.from_numpy(w).to(dev)
    yt = torch.empty((d["mb"], d["oc"], wf["oh"], wf["ow"]), dtype=torch.float32, device=dev)

    # a stream of its own: the legacy default stream synchronises implicitly with others
    stream = torch.cuda.Stream()
    conv = Convolution(capi.ALGORITHM_BCAST, capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW,
                       d["mb"], d["oc"], d["ic"], d["ih"], d["iw"], d["kh"], d["kw"],
                       d["sh"], d["sw"], d["ph"], d["pw"], wt, stream=stream)

    def step(src=xt, dst=yt):
        # the three executors of the C ABI, in the order of xnor_nn::Convolution::forward
        conv.stage("binarize_data", src=src, dst=dst)
        conv.stage("calculate_k")
        conv.stage("forward")

    host_us = []  # host time per step of the three executor calls (enqueue only), per leg

    def timed_steps(sets):
        """K steps over the (input, output) pairs of `sets` in turn: wall clock per step, then
        the same K steps again with HIP events attached to every kernel launch (their own
        dispatches, no marker packets between the kernels): mean duration of the binarize
        and of the convolution kernel inside the step, in ms."""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(*sets[i % len(sets)])
        host_us.append(1e6 * (time.perf_counter() - t0) / args.steps)  # all enqueued, none awaited
        torch.cuda.synchronize()
        wall_ms = 1e3 * (time.perf_counter() - t0) / args.steps
        conv.time_kernels(args.steps)
        for i in range(args.steps):
            step(*sets[i % len(sets)])
        torch.cuda.synchronize()
        tb = conv.kernel_times(capi.OP_BINARIZE_DATA)
        tc = conv.kernel_times(capi.OP_CONVOLUTION_FORWARD)
        conv.time_kernels(0)
        assert len(tb) == args.steps and len(tc) == args.steps, (len(tb), len(tc))
        return wall_ms, sum(tb) / len(tb), sum(tc) / len(tc), sorted(tb), sorted(tc)

    pair_bytes = xt.numel() * 4 + yt.numel() * 4
    nsets = max(3, -(-4 * INFINITY_CACHE_BYTES // pair_bytes))
    if args.cold_only:
        sets = [(xt, yt)] + [(xt.clone(), torch.empty_like(yt)) for _ in range(nsets - 1)]
        torch.cuda.synchronize()
        if args.binarize_only:
            for i in range(max(args.warmup, nsets) + 2 * args.steps):
                conv.stage("binarize_data", src=sets[i % nsets][0], dst=sets[i % nsets][1])
            torch.cuda.synchronize()
            print(json.dumps({"cold_only": True, "binarize_only": True,
                              "workload": args.workload, "buffer_pairs": nsets}))
            conv.close()
            return
        for i in range(max(args.warmup, nsets)):
            step(*sets[i % nsets])
        cold_ms, cbin_ms, cconv_ms, _, _ = timed_steps(sets)
        print(json.dumps({"cold_only": True, "workload": args.workload, "ms_per_step": cold_ms,
                          "buffer_pairs": nsets, "kernel_us": {"binarize": cbin_ms * 1e3,
                                                               "convolution": cconv_ms * 1e3}}))
        conv.close()
        return

    torch.cuda.synchronize()  # inputs were written on the default stream
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # ---- warm leg: the same input and output buffers every step (66 + 44 MB for the default
    # workload: they stay in the 256 MB Infinity Cache between steps).  The timed region is
    # exactly K steps, nothing but the three executor calls per step.
    ms_per_step, bin_ms, conv_ms, tb_sorted, tc_sorted = timed_steps([(xt, yt)])
    warm_host_us = host_us[-1]

    # K launches of the binarize kernel alone, back to back, one pair of events around all
    region = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    torch.cuda.synchronize()
    region[0].record(stream)
    for i in range(args.steps):
        conv.stage("binarize_data", src=xt, dst=yt)
    region[1].record(stream)
    torch.cuda.synchronize()
    bin_alone_ms = region[0].elapsed_time(region[1]) / args.steps

    # Spread of the step time: one event between consecutive steps.
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    torch.cuda.synchronize()
    marks[0].record(stream)
    for i in range(args.steps):
        step()
        marks[i + 1].record(stream)
    torch.cuda.synchronize()
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))

    # ---- cold leg: what the reference's own benchmark does with its cache flush between
    # repetitions (reference test/perf/test_simple_net.cpp:32-37).  The steps rotate through
    # enough input/output pairs that a pair's lines have left the Infinity Cache (and L2) by
    # the time it comes round again: the pairs together hold at least four times the cache.
    cold = None
    if not args.no_cold:
        sets = [(xt, yt)] + [(xt.clone(), torch.empty_like(yt)) for _ in range(nsets - 1)]
        torch.cuda.synchronize()
        for i in range(max(args.warmup, nsets)):
            step(*sets[i % nsets])
        cold_ms, cbin_ms, cconv_ms, _, _ = timed_steps(sets)
        # the binarize kernel alone over the same rotation: its input comes from HBM as in the
        # cold steps, but no convolution output is waiting in the caches to be written back
        # while it runs
        for i in range(nsets):
            conv.stage("binarize_data", src=sets[i][0], dst=sets[i][1])
        conv.time_kernels(args.steps)
        for i in range(args.steps):
            conv.stage("binarize_data", src=sets[i % nsets][0], dst=sets[i % nsets][1])
        torch.cuda.synchronize()
        alone = conv.kernel_times(capi.OP_BINARIZE_DATA)
        conv.time_kernels(0)
        cold = {"ms_per_step": cold_ms, "buffer_pairs": nsets, "bytes_per_pair": pair_bytes,
                "kernel_us": {"binarize": cbin_ms * 1e3, "convolution": cconv_ms * 1e3,
                              "binarize_without_convolutions": 1e3 * sum(alone) / len(alone)},
                "value": wf["nominal_ops"] / (cold_ms * 1e-3) / 1e9}
        del sets

    # Two descriptors, each with a stream, resources and an input/output pair of its own, fed
    # in turn from this one host thread: the binarize kernel of one forward pass (memory-bound)
    # runs beside the convolution of the other (matrix-core-bound).  Reported beside the
    # headline, never as it: ms_per_step above is one pass after the other on one stream.
    overlapped = None
    if not args.no_cold:
        stream2 = torch.cuda.Stream()
        conv2 = Convolution(capi.ALGORITHM_BCAST, capi.FMT_NCHW, capi.FMT_OIHW, capi.FMT_NCHW,
                            d["mb"], d["oc"], d["ic"], d["ih"], d["iw"], d["kh"], d["kw"],
                            d["sh"], d["sw"], d["ph"], d["pw"], wt, stream=stream2)
        x2, y2 = xt.clone(), torch.empty_like(yt)
        lanes = ((conv, xt, yt), (conv2, x2, y2))

        def step_on(lane):
            c, src, dst = lane
            c.stage("binarize_data", src=src, dst=dst)
            c.stage("calculate_k")
            c.stage("forward")

        torch.cuda.synchronize()
        for i in range(2 * max(args.warmup, 2)):
            step_on(lanes[i % 2])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(2 * args.steps):
            step_on(lanes[i % 2])
        torch.cuda.synchronize()
        pass_ms = 1e3 * (time.perf_counter() - t1) / (2 * args.steps)
        overlapped = {"ms_per_forward": pass_ms,
                      "value": wf["nominal_ops"] / (pass_ms * 1e-3) / 1e9,
                      "how": "two descriptors on two streams, %d forward passes in turn, wall "
                             "clock / passes; both input/output pairs stay in the Infinity "
                             "Cache" % (2 * args.steps)}
        conv2.close()
        del x2, y2

    # The same forward pass through host buffers (pageable numpy arrays, the way the
    # reference's own callers use the API): PCIe copies included, never the headline.
    host_ms = None
    if not args.no_host:
        import numpy as np
        yh = np.empty((d["mb"], d["oc"], wf["oh"], wf["ow"]), np.float32)
        conv.forward(x, yh)
        t2 = time.perf_counter()
        for _ in range(3):
            conv.forward(x, yh)
        host_ms = 1e3 * (time.perf_counter() - t2) / 3
    conv_s = conv_ms * 1e-3
    # Roofline of the convolution kernel.  The matrix-core kernel multiplies +-1 values as
    # FP4 operands, so its ceiling is the chip's dense FP4 MFMA rate.  The XNOR/popcount
    # kernel (very deep inputs, or XNOR_NN_HIP_CONV=valu) is bounded by the integer VALU: one
    # v_xnor_b32 + one v_bcnt_u32_b32 per lane handle 32 binary multiply-accumulates = 64
    # binary ops, i.e. CUs * 64 lanes * clock * 32 ops per lane-instruction.
    conv_kernel = conv.kernel_name(0)
    bin_kernel = conv.kernel_name(2)
    on_mfma = conv_kernel.startswith("conv_mfma")
    valu_peak_tops = cus * 64 * clk_hz * 32 / 1e12
    conv_peak = MFMA_FP4_PEAK_TOPS if on_mfma else valu_peak_tops
    conv_tops = wf["exact_ops"] / conv_s / 1e12
    profiled = args.workload if args.mb is None and not args.shape else "none"
    # The streaming stage is priced against HBM with its duration inside the cold steps, where
    # its input really comes from HBM; inside the warm steps the input of the default
    # workload is served by the Infinity Cache, which is reported beside it.
    bin_hbm_ms = cold["kernel_us"]["binarize"] * 1e-3 if cold else bin_ms
    bin_gbs = wf["binarize_bytes"] / (bin_hbm_ms * 1e-3) / 1e9

    result = {
        "metric": METRIC,
        "value": wf["nominal_ops"] / (ms_per_step * 1e-3) / 1e9,
        "unit": "GOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_cold": cold["ms_per_step"] if cold else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("fp4 (E2M1, +-1 exactly) MFMA, fp32 accumulate (exact integers), fp32 scale"
                  if on_mfma else "u32 xnor/popcount, int32 accumulate, fp32 scale"),
        "data": "synthetic (hash-based N(0,1)/N(0,sigma), seeds 1234/4321), resident in HBM",
        "config": {"workload": args.workload,
                   "shape": {k: d[k] for k in ("mb", "ic", "ih", "iw", "oc", "kh", "kw",
                                               "sh", "sw", "ph", "pw")},
                   "layout": "NCHW/OIHW/NCHW", "weights_binarized": "once, outside the step"},
        "timing": "ms_per_step: wall clock over K steps on one input/output pair (warm: the "
                  "pair stays in the Infinity Cache); ms_per_step_cold: the same over pairs "
                  "that together hold 4x the cache; kernel_us: mean duration of each kernel "
                  "inside K further steps of the same kind, from HIP events attached to the "
                  "kernels' own dispatches; binarize_alone_us: K back-to-back launches "
                  "between two events; step_ms_between_events: one event between "
                  "consecutive steps; host_buffers_ms_per_forward: three passes through "
                  "pageable host arrays; host_enqueue_per_step: host time of the executor "
                  "calls of a step (us), from the time to enqueue the K steps",
        "kernel_us": {"binarize": bin_ms * 1e3, "convolution": conv_ms * 1e3,
                      "step_minus_kernels": (ms_per_step - bin_ms - conv_ms) * 1e3,
                      # what the host spends in the three executor calls of a step (pointer
                      # queries, two mutexes, two launches), measured as the time to enqueue
                      # the K steps; the rest of step_minus_kernels is the gap between
                      # dependent dispatches on the GPU
                      "host_enqueue_per_step": warm_host_us,
                      "binarize_alone": bin_alone_ms * 1e3,
                      "binarize_min_median_max": [tb_sorted[0] * 1e3,
                                                  tb_sorted[len(tb_sorted) // 2] * 1e3,
                                                  tb_sorted[-1] * 1e3],
                      "convolution_min_median_max": [tc_sorted[0] * 1e3,
                                                     tc_sorted[len(tc_sorted) // 2] * 1e3,
                                                     tc_sorted[-1] * 1e3]},
        "cold": cold,
        "two_streams": overlapped,
        "step_ms_between_events": {"min": per_step[0], "median": per_step[len(per_step) // 2],
                                   "max": per_step[-1]},
        "host_buffers_ms_per_forward": host_ms,
        "conv_effective_gops": wf["nominal_ops"] / conv_s / 1e9,
        "roofline": {
            "kernel": conv_kernel, "bound": "mfma" if on_mfma else "valu",
            "achieved": conv_tops, "peak": conv_peak, "unit": "TFLOP/s",
            "frac": conv_tops / conv_peak,
            "traffic": measured_traffic(profiled, conv_kernel),
            "duration_us": conv_ms * 1e3,
            "cold": ({"duration_us": cold["kernel_us"]["convolution"],
                      "frac": wf["exact_ops"] / (cold["kernel_us"]["convolution"] * 1e-6)
                              / 1e12 / conv_peak} if cold else None),
            "peak_definition": (
                "MI355X dense FP4 MFMA rate, 10.1 PFLOP/s (signs are multiplied as FP4 +-1)"
                if on_mfma else
                "%d CUs x 64 lanes x %.3f GHz x 32 binary ops per VALU lane-instruction "
                "(xnor + bcnt pair = 64 ops)" % (cus, clk_hz / 1e9)),
            "ops": "exact in-bounds binary ops per launch = %d" % wf["exact_ops"],
            "hbm_view": {"bytes": wf["conv_bytes"],
                         "achieved_gbs": wf["conv_bytes"] / conv_s / 1e9,
                         "frac": wf["conv_bytes"] / conv_s / 1e9 / HBM_PEAK_GBS},
        },
        "roofline_binarize": {
            "kernel": bin_kernel, "bound": "hbm", "achieved": bin_gbs,
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bin_gbs / HBM_PEAK_GBS,
            "bytes": wf["binarize_bytes"],
            "duration_us": bin_hbm_ms * 1e3,
            "input_from": "HBM (cold steps)" if cold else "Infinity Cache where it fits",
            "warm": {"duration_us": bin_ms * 1e3,
                     "achieved": wf["binarize_bytes"] / (bin_ms * 1e-3) / 1e9,
                     "frac": wf["binarize_bytes"] / (bin_ms * 1e-3) / 1e9 / HBM_PEAK_GBS},
            "traffic": measured_traffic(profiled, bin_kernel),
        },
        "device": {"name": props.name, "cus": cus, "clock_ghz": clk_hz / 1e9},
    }
    conv.close()
    if not args.no_cold:
        # What the memory system gives a kernel that only reads (xnor_nn_hip_plain_read: 16
        # bytes per lane and load, nothing kept), for context beside the 8 TB/s the fractions
        # are priced against: 1 GiB (four times the Infinity Cache: HBM), and this workload's
        # own input re-read in place (cache-resident where it fits, as in the warm steps).
        lib = capi.load()

        def plain_read_us(tensor, passes=10):
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
            nbytes = tensor.numel() * tensor.element_size()
            with torch.cuda.stream(stream):
                for timed in (False, True):
                    if timed:
                        marks[0].record(stream)
                    for _ in range(passes):
                        if lib.xnor_nn_hip_plain_read(tensor.data_ptr(), nbytes,
                                                      stream.cuda_stream) != capi.SUCCESS:
                            sys.exit("xnor_nn_hip_plain_read failed")
                    if timed:
                        marks[1].record(stream)
                    torch.cuda.synchronize()
            return 1e3 * marks[0].elapsed_time(marks[1]) / passes

        big = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        torch.cuda.synchronize()
        big_us = plain_read_us(big)
        del big
        own_us = plain_read_us(xt)
        result["roofline_binarize"]["plain_read"] = {
            "of_1gib": {"duration_us": big_us, "achieved": (1 << 30) / (big_us * 1e-6) / 1e9,
                        "frac": (1 << 30) / (big_us * 1e-6) / 1e9 / HBM_PEAK_GBS},
            "of_this_input": {"bytes": xt.numel() * 4, "duration_us": own_us,
                              "achieved": xt.numel() * 4 / (own_us * 1e-6) / 1e9},
            "unit": "GB/s",
            "how": "xnor_nn_hip_plain_read, 10 back-to-back passes between two events"}
    if not args.no_cold and on_mfma:
        # What the matrix pipes give a kernel that only multiplies (xnor_nn_hip_mfma_only:
        # register-resident pseudo-random +-1 operands, two workgroups per compute unit like
        # the convolution, no operand traffic): the practical ceiling beside the published
        # peak, which assumes the full clock.  As long a launch as the convolution takes, and
        # a long one (the clock settles over milliseconds).
        ops_per_wave_iter = 8 * 131072
        rates = {}
        for label, iters in (("short", 100), ("long", 20000)):
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
            reps = 20 if label == "short" else 1
            with torch.cuda.stream(stream):
                for timed in (False, True):
                    if timed:
                        marks[0].record(stream)
                    for _ in range(reps):
                        if lib.xnor_nn_hip_mfma_only(2 * cus, iters,
                                                     stream.cuda_stream) != capi.SUCCESS:
                            sys.exit("xnor_nn_hip_mfma_only failed")
                    if timed:
                        marks[1].record(stream)
                    torch.cuda.synchronize()
            us = 1e3 * marks[0].elapsed_time(marks[1]) / reps
            tops = 2 * cus * 4 * iters * ops_per_wave_iter / (us * 1e-6) / 1e12
            rates[label] = {"duration_us": us, "achieved": tops, "frac": tops / conv_peak}
        result["roofline"]["matrix_instructions_only"] = dict(
            rates, unit="TFLOP/s",
            how="xnor_nn_hip_mfma_only, 2 workgroups per CU; short: 800 instructions per "
                "wave, 20 launches back to back; long: 160000 per wave, one launch")
    if args.copy_calibration_mib:
        n = args.copy_calibration_mib * (1 << 20) // 4
        src_buf = torch.ones(n, dtype=torch.float32, device=dev)
        dst_buf = torch.empty_like(src_buf)
        torch.cuda.synchronize()
        dst_buf.copy_(src_buf)
        torch.cuda.synchronize()
        result["copy_calibration_bytes_each_way"] = n * 4
    if not args.no_cpu:
        threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        cb, both = cpu_baseline(d, x, w, threads)
        result["cpu_baseline"] = cb
        result["cpu_baselines"] = both  # the real reference and the in-repo restatement
        result["speedup_vs_cpu_baseline"] = cb["ms_per_forward"] / ms_per_step
    print(json.dumps(result))


if __name__ == "__main__":
    main()
