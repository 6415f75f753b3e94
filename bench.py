#!/usr/bin/env python3
"""Benchmark of the binary-convolution forward path on one MI355X.

One step = one forward pass (binarize_data + calculate_k + XNOR/popcount convolution; the
same three-part split the reference reports in README.md:29-32) over one batch of
synthetic input that is already resident in HBM.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "ms/forward + effective binary GOPS, AlexNet conv4 N=256 on 1 MI355X"
HBM_PEAK_GBS = 8000.0
MFMA_FP4_PEAK_TOPS = 10100.0
# HBM bytes per launch read from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch),
# each scaled by what the same counter shows for a plain copy of known size; the runs and
# the scale factors are recorded in profiles/.  Not measurable from inside this script.
MEASURED_TRAFFIC = {
    # profiles/alexnet_conv4_mb256_hbm_traffic_pmc.txt: read (FETCH_SIZE x2) + written bytes
    ("alexnet_conv4_mb256", "conv_mfma_fp4_kernel"): 5956 * 1024 + 43770 * 1024,
    ("alexnet_conv4_mb256", "binarize_nchw_kernel"): 65720 * 1024 + 2197 * 1024,
}


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


def cpu_baseline(d, x, w, threads):
    """The CPU path timed on this host: the compiled upstream library when it was built
    (oracle/_ref), else the in-repo C restatement.  Baseline only; never the product."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import checkers
    reps = 5 if d["mb"] * d["oc"] * d["ih"] * d["iw"] < 5e7 else 3
    if checkers.have_ref():
        ref = checkers.RefLib()
        out = ref.forward(d, x, w, reps=reps + 1, timer=time.perf_counter)
        times = out["times"][1:]
        best = min(times, key=lambda t: t[3] - t[0])
        stages = [1e3 * (best[i + 1] - best[i]) for i in range(3)]
        kind = "reference"
    else:
        from util import oracle_shape
        oracle = checkers.Oracle()
        s = oracle_shape(oracle, d)
        bw, alpha, opc = oracle.binarize_weights(s, w)
        best = None
        for _ in range(reps):
            t0 = time.perf_counter()
            bsrc = oracle.binarize_data(s, x)
            t1 = time.perf_counter()
            a, k = oracle.calculate_k(s, x)
            t2 = time.perf_counter()
            oracle.convolution(s, bsrc, bw, alpha, k, opc)
            t3 = time.perf_counter()
            if best is None or t3 - t0 < best[3] - best[0]:
                best = (t0, t1, t2, t3)
        stages = [1e3 * (best[i + 1] - best[i]) for i in range(3)]
        kind = "port"
    ms = sum(stages)
    return {
        "value": work_figures(d)["nominal_ops"] / (ms * 1e-3) / 1e9, "unit": "GOPS",
        "ms_per_forward": ms, "stage_ms": {"binarize_data": stages[0],
                                           "calculate_k": stages[1], "forward": stages[2]},
        "cores": threads, "kind": kind,
        "sample": "whole workload, best of %d forward passes after one warm-up "
                  "(OpenMP, %d threads%s)" % (reps, threads,
                                              ", XNOR_NN_ISA=2" if kind == "reference" else ""),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="alexnet_conv4_mb256")
    ap.add_argument("--mb", type=int, default=None,
                    help="override the batch size of the workload (experiments only)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
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

    def step(events=None):
        # the three executors of the C ABI, in the order of xnor_nn::Convolution::forward
        if events:
            events[0].record(stream)
        conv.stage("binarize_data", src=xt, dst=yt)
        if events:
            events[1].record(stream)
        conv.stage("calculate_k")
        if events:
            events[2].record(stream)
        conv.stage("forward")
        if events:
            events[3].record(stream)

    torch.cuda.synchronize()  # inputs were written on the default stream
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # Timed region: exactly K steps, nothing but the three executor calls per step.
    region = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region[0].record(stream)
    for i in range(args.steps):
        step()
    region[1].record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = 1e3 * (t1 - t0) / args.steps

    # Kernel durations for the rooflines.  An event record costs the stream a few
    # microseconds, so events around single launches overstate a 13 or 25 us kernel.  One pair
    # of events spans the K steps above; a second pair spans K launches of the binarize
    # kernel alone, back to back.  The stream runs its kernels one after the other, so
    # (K steps - K binarize launches) / K is what a step spends on the only other kernel, the
    # convolution, with every gap between kernels counted against it.
    torch.cuda.synchronize()
    region[2].record(stream)
    for i in range(args.steps):
        conv.stage("binarize_data", src=xt, dst=yt)
    region[3].record(stream)
    torch.cuda.synchronize()
    step_ms_events = region[0].elapsed_time(region[1]) / args.steps
    bin_ms = region[2].elapsed_time(region[3]) / args.steps
    conv_ms = step_ms_events - bin_ms

    # A further pass of K steps with HIP events around every stage, for the per-stage view
    # (each figure includes the cost of its event records; calculate_k launches nothing, so
    # its figure is that cost alone).
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    torch.cuda.synchronize()
    for i in range(args.steps):
        step(evs[i])
    torch.cuda.synchronize()
    stage_ms = [sum(e[i].elapsed_time(e[i + 1]) for e in evs) / args.steps for i in range(3)]
    gpu_ms = sum(e[0].elapsed_time(e[3]) for e in evs) / args.steps

    # Spread of the step time: one event between consecutive steps.
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    torch.cuda.synchronize()
    marks[0].record(stream)
    for i in range(args.steps):
        step()
        marks[i + 1].record(stream)
    torch.cuda.synchronize()
    per_step = sorted(marks[i].elapsed_time(marks[i + 1]) for i in range(args.steps))

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
    # kernel (stride > 1, very wide inputs, or XNOR_NN_HIP_CONV=valu) is bounded by the
    # integer VALU: one v_xnor_b32 + one v_bcnt_u32_b32 per lane handle 32 binary
    # multiply-accumulates = 64 binary ops, i.e. CUs * 64 lanes * clock * 32 ops per
    # lane-instruction.
    conv_kernel = conv.kernel_name(0)
    on_mfma = conv_kernel.startswith("conv_mfma")
    valu_peak_tops = cus * 64 * clk_hz * 32 / 1e12
    conv_tops = wf["exact_ops"] / conv_s / 1e12
    bin_gbs = wf["binarize_bytes"] / (bin_ms * 1e-3) / 1e9

    result = {
        "metric": METRIC,
        "value": wf["nominal_ops"] / (ms_per_step * 1e-3) / 1e9,
        "unit": "GOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": ("fp4 (E2M1, +-1 exactly) MFMA, fp32 accumulate (exact integers), fp32 scale"
                  if on_mfma else "u32 xnor/popcount, int32 accumulate, fp32 scale"),
        "data": "synthetic (hash-based N(0,1)/N(0,sigma), seeds 1234/4321), resident in HBM",
        "config": {"workload": args.workload,
                   "shape": {k: d[k] for k in ("mb", "ic", "ih", "iw", "oc", "kh", "kw",
                                               "sh", "sw", "ph", "pw")},
                   "layout": "NCHW/OIHW/NCHW", "weights_binarized": "once, outside the step"},
        "timing": "ms_per_step: wall clock over the K steps; kernel_us (used by the rooflines): "
                  "one pair of HIP events over those K steps and one over K back-to-back "
                  "launches of the binarize kernel, convolution = difference; stage_ms: a "
                  "further pass with events around every stage, event cost included; "
                  "step_ms_between_events: one event between consecutive steps; "
                  "host_buffers_ms_per_forward: three passes through pageable host arrays",
        "kernel_us": {"step": step_ms_events * 1e3, "binarize": bin_ms * 1e3,
                      "convolution": conv_ms * 1e3},
        "step_ms_between_events": {"min": per_step[0], "median": per_step[len(per_step) // 2],
                                   "max": per_step[-1]},
        "host_buffers_ms_per_forward": host_ms,
        "gpu_ms_per_forward_with_events": gpu_ms,
        "stage_ms": {"binarize_data": stage_ms[0], "calculate_k": stage_ms[1],
                     "forward": stage_ms[2]},
        "conv_effective_gops": wf["nominal_ops"] / conv_s / 1e9,
        "roofline": {
            "kernel": conv_kernel, "bound": "mfma" if on_mfma else "valu",
            "achieved": conv_tops,
            "peak": MFMA_FP4_PEAK_TOPS if on_mfma else valu_peak_tops,
            "unit": "TFLOP/s",
            "frac": conv_tops / (MFMA_FP4_PEAK_TOPS if on_mfma else valu_peak_tops),
            "traffic": MEASURED_TRAFFIC.get((args.workload if args.mb is None else None,
                                             conv_kernel.split("<")[0])),
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
            "kernel": conv.kernel_name(2), "bound": "hbm", "achieved": bin_gbs,
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": bin_gbs / HBM_PEAK_GBS,
            "bytes": wf["binarize_bytes"],
            "traffic": MEASURED_TRAFFIC.get((args.workload if args.mb is None else None,
                                             conv.kernel_name(2).split("<")[0])),
        },
        "device": {"name": props.name, "cus": cus, "clock_ghz": clk_hz / 1e9},
    }
    conv.close()
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
        cb = cpu_baseline(d, x, w, threads)
        result["cpu_baseline"] = cb
        result["speedup_vs_cpu_baseline"] = cb["ms_per_forward"] / ms_per_step
    print(json.dumps(result))


if __name__ == "__main__":
    main()
