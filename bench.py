#!/usr/bin/env python3
"""Benchmark of the IMathEngine inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

A step is one forward pass of the ResNet-18-style network (BASELINE.json configs[1]: batch 64, 224x224x3, fp32)
issued as engine calls through the C ABI of libneoml_hip.so, input already resident in device memory.
Prints one JSON line: images/sec, the roofline of the dominant kernel (the 3x3 implicit-GEMM convolutions, timed
live with events on the launch stream) and the reference CPU engine (its MLAS build) timed on the same batch: one thread,
and one engine per host core with the batch split between them.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBPS = 8000.0
# Bytes crossing the L2 <-> fabric boundary per 3x3-convolution launch, mean over the 16 launches of one step at
# batch 64, 224x224: rocprofv3 --pmc FETCH_SIZE (x2.0, the factor a known-size copy gives) 71.9 MB + WRITE_SIZE (x1.0)
# 45.3 MB; profiles/resnet18_b64_conv_hbm_traffic.txt holds the two runs. Counters cannot be read from inside this
# process, so the figure is a constant of the default workload (labelled as coming from that profile) and null for any other.
CONV3X3_TRAFFIC_BYTES_B64_224 = 117.2e6
CONV3X3_TRAFFIC_SOURCE = "offline_profile: profiles/resnet18_b64_conv_hbm_traffic.txt"


def _cpu_model():
    """What /proc/cpuinfo says of the host's first processor: the model name (a virtual machine may only give the brand)
    with family / model / stepping and the clock it reports, which identify the part where the name does not."""
    fields = {}
    try:
        for line in open("/proc/cpuinfo"):
            if ":" not in line:
                if fields:
                    break
                continue
            key, value = (t.strip() for t in line.split(":", 1))
            fields.setdefault(key, value)
    except OSError:
        return "unknown"
    if "model name" not in fields:
        return "unknown"
    detail = ", ".join("%s %s" % (k, fields[k]) for k in ("cpu family", "model", "stepping") if k in fields)
    mhz = " at %.0f MHz" % float(fields["cpu MHz"]) if "cpu MHz" in fields else ""
    return "%s (%s%s)" % (fields["model name"], detail, mhz)


def cpu_baseline(batch, image, replicas):
    """The reference's own CPU engine (oracle/_ref, compiled from its sources, with the MLAS GEMM it ships with on Linux) on
    the same network and the same batch: (1) one engine, one thread, the whole batch; (2) `replicas` engines side by side,
    one thread and one network each, the batch split between them, started together
    (NeoML/test/src/InferencePerformanceMultiThreadingTest.cpp:238-262). Every engine runs in a process of its own
    (oracle/cpu_baseline.py). Returns the JSON object and the arrays of the single-thread pass (softmax, logits)."""
    import subprocess
    import tempfile
    import numpy as np
    script = os.path.join(ROOT, "oracle", "cpu_baseline.py")
    mlas = os.path.exists(os.path.join(ROOT, "oracle", "_ref", "mlas", "libengine_shim.so"))
    common = [sys.executable, script, "--image", str(image)] + (["--mlas"] if mlas else [])
    with tempfile.TemporaryDirectory() as tmp:
        saved = os.path.join(tmp, "single.npz")
        one = json.loads(subprocess.run(common + ["--images", str(batch), "--passes", "2", "--save", saved], check=True, stdout=subprocess.PIPE,
                                        text=True).stdout.strip().splitlines()[-1])
        arrays = dict(np.load(saved))
        # the first images once more on the engine's built-in GEMM (no MLAS), the build the parity tests check against:
        # how far the reference's own two backends are from each other is the scale for the GPU's distance from either
        if mlas:
            first = os.path.join(tmp, "first.npz")
            n_first = min(4, batch)
            subprocess.run([sys.executable, script, "--image", str(image), "--images", str(n_first), "--save", first], check=True,
                           stdout=subprocess.DEVNULL)
            arrays["logits_builtin_gemm"] = np.load(first)["logits"]
    base = {
        "value": round(one["images"] / one["seconds"], 3), "unit": "images/sec", "cores": 1, "kind": one["kind"],
        "sample": "the whole batch of %d images, mean of 2 passes, 1 thread, %s" % (batch, one["backend"]),
        "seconds": round(one["seconds"], 2), "cpu": _cpu_model(),
    }
    if replicas > 1:
        share = [batch // replicas + (1 if i < batch % replicas else 0) for i in range(replicas)]
        share = [n for n in share if n > 0]
        start_at = time.time() + 6.0  # past every replica's start-up (imports, weights)
        procs = [subprocess.Popen(common + ["--images", str(n), "--passes", "4", "--start-at", repr(start_at)], stdout=subprocess.PIPE, text=True)
                 for n in share]
        done = [json.loads(p.communicate()[0].strip().splitlines()[-1]) for p in procs]
        slowest = max(d["seconds"] for d in done)
        base["replicas"] = {
            "value": round(batch / slowest, 3), "unit": "images/sec", "cores": len(share),
            "sample": "the same batch split over %d engines (one thread, one network each, %d-%d images), started together, 4 passes each; "
                      "rate = batch / slowest replica's mean pass" % (len(share), min(share), max(share)),
            "seconds": round(slowest, 2),
        }
    return base, arrays


def cdnn_run_once(batch, image):
    """CDnn::RunOnce (NeoML/src/Dnn/Dnn.cpp:626-658) of the benchmark network on CHipMathEngine, measured by
    oracle/cdnn_run_once.py; None where the reference's layer library was not built."""
    import subprocess
    if not os.path.exists(os.path.join(ROOT, "oracle", "_ref", "libdnn_shim.so")):
        return None
    res = subprocess.run([sys.executable, os.path.join(ROOT, "oracle", "cdnn_run_once.py"), "--batch", str(batch), "--image", str(image)],
                         stdout=subprocess.PIPE, text=True)
    if res.returncode != 0:
        return {"error": "oracle/cdnn_run_once.py exited with %d" % res.returncode}
    fig = json.loads(res.stdout.strip().splitlines()[-1])
    fig["what"] = "NeoML's CDnn + layer classes (reference sources) on CHipMathEngine, wall time per RunOnce closed by a read-back"
    return fig


def lstm_overlap_report(be, plan, steps):
    """Did the two directions of the bidirectional layers run side by side? The same replay with nhStreamOverlapLstm on and
    off: the step time, and the span of a layer's pair of nhLstm calls (event before the first call, event behind the
    second, both on the launch stream, which waits for the side stream behind the second call)."""
    import ctypes
    import torch
    lib, ms = be.lib, ctypes.c_float(0)
    report = {}
    for mode, enable in (("in_order", 0), ("side_by_side", 1)):  # ( ends with the overlap on, as the network asked )
        be.na.check(lib.nhStreamOverlapLstm(be.stream, enable))
        for _ in range(3):
            plan.run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            plan.run()
        torch.cuda.synchronize()
        step_ms = (time.perf_counter() - t0) / steps * 1e3
        # events around each pair only: one between the two calls would be a launch between them, and the second call
        # then has to stay behind the first
        record, check = lib.nhEventRecord, be.na.check
        pairs = []
        for _ in range(steps):
            seen = 0
            for fn, fargs, tag, _, _ in plan.launches:
                if tag == "lstm" and seen % 2 == 0:
                    start, stop = ctypes.c_void_p(), ctypes.c_void_p()
                    check(lib.nhEventCreate(ctypes.byref(start)))
                    check(lib.nhEventCreate(ctypes.byref(stop)))
                    record(start, be.stream)
                check(fn(*fargs))
                if tag == "lstm":
                    seen += 1
                    if seen % 2 == 0:
                        record(stop, be.stream)
                        pairs.append((start, stop))
        torch.cuda.synchronize()
        spans = []
        for start, stop in pairs:
            check(lib.nhEventElapsedMs(start, stop, ctypes.byref(ms)))
            spans.append(ms.value * 1e3)
        report[mode] = {"ms_per_step": round(step_ms, 3), "pair_span_us": round(sum(spans) / max(len(spans), 1), 1)}
    report["ran_side_by_side"] = report["side_by_side"]["pair_span_us"] < 0.9 * report["in_order"]["pair_span_us"]
    return report


def other_workload(args):
    """BASELINE configurations 3-5 at full size: same replay + event method, one JSON line with the per-family split."""
    import torch
    from workloads import HipBackend, MobileNetV2, TransformerEncoder, LineRecognizer
    be = HipBackend()
    if args.workload == "mobilenetv2":
        net = MobileNetV2(be, batch=args.batch or 128, image=args.image, fused=args.fused)
        unit, items, name = "images/sec", net.batch, "MobileNetV2-style inference, batch %d, %dx%dx3" % (net.batch, args.image, args.image)
    elif args.workload == "transformer":
        net = TransformerEncoder(be, batch=args.batch or 32)
        unit, items, name = "sequences/sec", net.batch, "6-layer transformer encoder, d_model 512, 8 heads, FFN 2048, seq 256, batch %d" % net.batch
    else:
        net = LineRecognizer(be, batch=args.batch or 64)
        unit, items, name = "lines/sec", net.batch, "OCR line recogniser, 32x512 grey, 6 convs + 2 BiLSTM layers (hidden 256) + CTC arg-max, batch %d" % net.batch
    x = be.tensor(net.make_input())
    plan, _ = net.record_plan(x)
    tags = set(t for _, _, t, _, _ in plan.launches if t)
    steps = args.steps
    pools = plan.make_events(tags, steps)
    # what the engine adapter asks for its own stream: runs of small element-wise calls (the per-row scalars of the
    # normalisation layers) go out several per launch, and a fully connected layer's product takes its free term along;
    # every launch and wait below goes through the library
    deferring = not args.no_defer
    be.defer_small_ops(deferring)
    for _ in range(args.warmup):
        plan.run()
    be.synchronize()
    t_settle = time.perf_counter()
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        plan.run()
        be.synchronize()
    # untimed-event pass for the throughput figure, then an event pass for the per-family split
    t0 = time.perf_counter()
    for _ in range(steps):
        plan.run()
    be.synchronize()
    elapsed = time.perf_counter() - t0
    by_runs = deferring or args.time_by_runs
    for step in range(steps):
        plan.run_with_events(pools[step], by_runs=by_runs)
    be.synchronize()
    be.defer_small_ops(False)
    fam = plan.family_totals()
    split = {}
    for tag, (cnt, tms, fl, by) in sorted(fam.items(), key=lambda kv: -kv[1][1]):
        split[tag] = {"launches_per_step": cnt // steps, "ms_per_step": round(tms / steps, 4),
                      "tflops": round(fl / (tms * 1e-3) / 1e12, 2) if fl else None,
                      "gb_per_s": round(by / (tms * 1e-3) / 1e9, 1)}
        print("%-10s launches/step %4d  ms/step %8.3f  TFLOP/s %7.2f  GB/s %8.1f" % (
            tag, cnt // steps, tms / steps, fl / (tms * 1e-3) / 1e12 if fl else 0.0, by / (tms * 1e-3) / 1e9), file=sys.stderr)
    extra = {}
    if args.workload == "ocr":
        extra["lstm_overlap"] = lstm_overlap_report(be, plan, steps)
    print(json.dumps({
        "metric": "%s (not the headline metric)" % unit, "value": round(items * steps / elapsed, 1), "unit": unit, "n_gpus": 1,
        "steps": steps, "warmup": args.warmup, "ms_per_step": round(elapsed / steps * 1e3, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": name + ", fp32, engine calls through the C ABI", "launches_per_step": len(plan.launches),
                   "small_ops_deferred": deferring, "families_timed": "per run of launches" if by_runs else "per launch"},
        "families": split, **extra}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--settle-ms", type=float, default=600.0,
                    help="after the warm-up steps keep replaying the step untimed for this long, so that the timed region "
                         "starts with the GPU at its sustained clock instead of ramping up from idle")
    ap.add_argument("--fused", action="store_true",
                    help="the network as NeoML's graph optimizer rewrites it: resnet18: convolution + ReLU pairs as one "
                         "engine call; mobilenetv2: the inverted-residual blocks as fused block calls")
    ap.add_argument("--workload", default="resnet18", choices=("resnet18", "mobilenetv2", "transformer", "ocr"),
                    help="resnet18 (default) is the configuration the metric is quoted on; the others are the remaining "
                         "BASELINE configurations, measured the same way with a per-family table on stderr")
    ap.add_argument("--batch", type=int, default=None)
    ap.add_argument("--image", type=int, default=224)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--time-by-runs", action="store_true",
                    help="other workloads: the per-family split from one pair of events per run of consecutive launches of a family")
    ap.add_argument("--no-defer", action="store_true",
                    help="every call a launch of its own (nhStreamDeferSmallOps off)")
    ap.add_argument("--cpu-replicas", type=int, default=min(16, os.cpu_count() or 1),
                    help="engines of the multi-replica CPU baseline (one thread each; 16 = the host cores that go with one GPU)")
    ap.add_argument("--per-kernel", action="store_true", help="print a per-op-family timing table to stderr")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one nhVectorCopy of 2^26 floats (256 MiB read + 256 MiB written): the known-size "
                         "kernel that scales the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus)

    if args.workload != "resnet18":
        return other_workload(args)
    if args.batch is None:
        args.batch = 64

    import torch
    from workloads import HipBackend, ResNet18

    be = HipBackend()
    net = ResNet18(be, batch=args.batch, image=args.image, fused=args.fused)
    x = be.tensor(net.make_input())
    # the launches of one forward pass, arguments bound once: replaying them costs the host a few microseconds
    # per launch, so the timed region is bound by the GPU, not by the Python interpreter
    plan, out = net.record_plan(x)
    if args.calibrate_copy:
        import ctypes
        src = be.empty(1 << 26).fill_(1.0)
        dst = be.empty(1 << 26)
        be.na.check(be.lib.nhVectorCopy(be.stream, ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), 1 << 26))
        torch.cuda.synchronize()
        del src, dst
    timed_tags = None if args.per_kernel else ("conv3x3",)
    all_tags = set(t for _, _, t, _, _ in plan.launches if t)
    pools = plan.make_events(all_tags if timed_tags is None else timed_tags, args.steps)
    # The stream as the engine adapter sets its own up (nhStreamDeferSmallOps): a launch may wait for the call behind it,
    # so the ReLU that follows a convolution in place, the free term behind the classifier's product and runs of small
    # element-wise calls go out with the launch in front of them. Same calls, same results; every launch and wait of
    # the timed region goes through the library.
    deferring = not args.no_defer
    be.defer_small_ops(deferring)
    for _ in range(args.warmup):
        plan.run()
    be.synchronize()
    settle_start = time.perf_counter()
    settle_steps = 0
    while (time.perf_counter() - settle_start) * 1e3 < args.settle_ms:
        for _ in range(5):
            plan.run()
        be.synchronize()
        settle_steps += 5

    # the throughput figure: the plain replay, nothing but the step's own launches on the stream
    t0 = time.perf_counter()
    for step in range(args.steps):
        plan.run()
    host_done = time.perf_counter()
    be.synchronize()
    elapsed = time.perf_counter() - t0
    # the roofline figure: the same steps again with an event pair around every 3x3 convolution (on the launch stream;
    # an event is a call on the stream too, so here every convolution goes out as it was asked for, without its ReLU)
    for step in range(args.steps):
        plan.run_with_events(pools[step])
    be.synchronize()
    be.defer_small_ops(False)

    ms_per_step = elapsed / args.steps * 1e3
    images_per_sec = args.batch * args.steps / elapsed

    # per-family totals from the events of the second pass
    fam = plan.family_totals()
    c3 = fam.get("conv3x3", [0, 1e-9, 0, 0])
    launches, ms, flops, nbytes = c3
    achieved = flops / (ms * 1e-3) / 1e12
    roofline = {
        "bound": "mfma", "kernel": "matMulKernel<AM_ConvTaps> (3x3 convolutions, %d launches per step)" % (launches // max(args.steps, 1)),
        "achieved": round(achieved, 2), "peak": FP32_MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / FP32_MFMA_PEAK_TFLOPS, 4),
        "traffic": CONV3X3_TRAFFIC_BYTES_B64_224 if (args.batch, args.image) == (64, 224) else None,
        "traffic_unit": "bytes per launch (FETCH_SIZE + WRITE_SIZE, rocprofv3 --pmc, scaled by a known-size copy)",
        "traffic_source": CONV3X3_TRAFFIC_SOURCE if (args.batch, args.image) == (64, 224) else None,
        "algorithmic_bytes_per_launch": nbytes // max(launches, 1),
        "avg_launch_us": round(ms * 1e3 / max(launches, 1), 2),
        "flop_per_step": flops // max(args.steps, 1),
    }
    if args.per_kernel:
        for tag, (cnt, tms, fl, by) in sorted(fam.items(), key=lambda kv: -kv[1][1]):
            print("%-10s launches/step %3d  ms/step %8.3f  TFLOP/s %7.2f  GB/s %8.1f" % (
                tag, cnt // args.steps, tms / args.steps, fl / (tms * 1e-3) / 1e12 if fl else 0.0,
                by / (tms * 1e-3) / 1e9), file=sys.stderr)

    result = {
        "metric": "images/sec ResNet-18-style b64 fp32; conv TFLOPS as % of fp32 MFMA peak",
        "value": round(images_per_sec, 1), "unit": "images/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "ResNet-18-style inference, batch %d, %dx%dx3, fp32, engine calls through the C ABI%s" % (
            args.batch, args.image, args.image,
            ", graph as rewritten by OptimizeDnn (convolution + ReLU in one call)" if args.fused else ""),
            "global_batch": args.batch, "launch_waits_for_successor": deferring,
            "gflop_per_step": round(net.conv_flops() / 1e9, 2)},
        "conv_tflops_overall": round(net.conv_flops() / (ms_per_step * 1e-3) / 1e12, 2),
        "host_enqueue_ms_per_step": round((host_done - t0) / args.steps * 1e3, 3),
        "clock_settle": {"ms": args.settle_ms, "untimed_steps": settle_steps},
        "roofline": roofline,
    }

    if not args.fused:
        # beside the headline: the same network after NeoML's own graph optimizer (OptimizeDnn turns each convolution that
        # feeds only a ReLU into a rowwise chain = one engine call); same result, fewer passes over the activations
        opt = ResNet18(be, batch=args.batch, image=args.image, fused=True)
        opt_plan, opt_out = opt.record_plan(x)
        torch.cuda.synchronize()
        steps = max(10, min(args.steps, 50))
        for _ in range(10):
            opt_plan.run()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(steps):
            opt_plan.run()
        torch.cuda.synchronize()
        opt_ms = (time.perf_counter() - t1) / steps * 1e3
        result["optimized_graph"] = {"ms_per_step": round(opt_ms, 3), "images_per_sec": round(args.batch / opt_ms * 1e3, 1),
                                     "steps": steps, "max_abs_diff_vs_plain": float((opt_out - out).abs().max().item())}

    if not args.no_cpu_baseline:
        import numpy as np
        base, cpu = cpu_baseline(args.batch, args.image, args.cpu_replicas)
        result["cpu_baseline"] = base
        # parity of the whole network on the whole batch, against the CPU engine's single-thread pass: the softmax output
        # and the logits in front of it (1000 probabilities of ~1e-3 pass an absolute bar easily, the logits do not)
        y_gpu = be.to_numpy(out)
        logits_gpu = be.to_numpy(net.buffers["fc"])
        logits_cpu = cpu["logits"].reshape(logits_gpu.shape)

        def distance(a, b):
            d = np.abs(a - b)
            scale = max(1.0, float(np.abs(b).max()))  # the whole-network bar of the tests: the floor follows the output's scale
            return {"max_abs_diff": float(d.max()), "max_abs_value": float(np.abs(b).max()),
                    "worst_fraction_of_bar": round(float((d / (1e-5 + 1e-4 * np.abs(b))).max()), 3),
                    "worst_fraction_of_network_bar": round(float((d / (1e-5 * scale + 1e-4 * np.abs(b))).max()), 4),
                    "images": int(a.shape[0])}

        result["parity_max_abs_diff_vs_cpu"] = float(np.max(np.abs(y_gpu - cpu["softmax"].reshape(y_gpu.shape))))
        result["parity_logits_vs_cpu"] = dict(distance(logits_gpu, logits_cpu), bar="|a - b| <= 1e-5 + 1e-4 |b| per element",
                                              network_bar="|a - b| <= 1e-5 max(1, max|b|) + 1e-4 |b|")
        if "logits_builtin_gemm" in cpu:
            # logits near zero are sums of 512 products that cancel: their absolute error follows the size of the products,
            # not of the sum, so the per-element bar is a strict one here; the reference's two GEMM backends show the scale
            builtin = cpu["logits_builtin_gemm"].reshape(-1, logits_gpu.shape[1])
            n = builtin.shape[0]
            # ( all three on the same first images, so that the figures can be set side by side )
            result["parity_logits_vs_cpu"]["same_images_vs_mlas_engine"] = distance(logits_gpu[:n], logits_cpu[:n])
            result["parity_logits_vs_cpu"]["vs_builtin_gemm_engine"] = distance(logits_gpu[:n], builtin)
            result["parity_logits_vs_cpu"]["reference_mlas_vs_builtin_gemm"] = distance(logits_cpu[:n], builtin)
        # the same network as an application of the reference runs it: NeoML's own CDnn and layer classes (compiled from the
        # reference's sources) calling the HIP engine through IMathEngine, timed per CDnn::RunOnce in a process of its own
        result["cdnn_run_once"] = cdnn_run_once(args.batch, args.image)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
