#!/usr/bin/env python3
"""One replica of the benchmark's CPU baseline: the ResNet-18-style network (BASELINE configuration 2) on the
reference's own CPU engine, `--images` images, one thread, one engine.

    python oracle/cpu_baseline.py --images 4 [--mlas] [--passes 1] [--start-at UNIX_TIME] [--save out.npz]

--mlas      the engine built with its vendored MLAS GEMM (oracle/_ref/mlas, the backend the reference ships with on
            Linux) instead of its built-in SSE kernels
--start-at  sleep until this time before the timed pass: the N replicas of a multi-replica measurement (one engine and one
            network per replica, the batch split N ways: NeoML/test/src/InferencePerformanceMultiThreadingTest.cpp:238-262)
            start together
--save      write the softmax output and the logits in front of it to a .npz (the parity figures of the benchmark)
Prints one JSON line {"images", "seconds", "backend"}.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--images", type=int, default=4)
    ap.add_argument("--image", type=int, default=224)
    ap.add_argument("--mlas", action="store_true")
    ap.add_argument("--passes", type=int, default=1, help="timed passes, back to back; the time printed is their mean")
    ap.add_argument("--start-at", type=float, default=0.0)
    ap.add_argument("--save", default="")
    args = ap.parse_args()
    if args.mlas:
        os.environ["NHTEST_SHIM_LIB"] = os.path.join(ROOT, "oracle", "_ref", "mlas", "libengine_shim.so")
    os.environ.setdefault("OMP_NUM_THREADS", "1")
    sys.path.insert(0, ROOT)
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import numpy as np
    import nhtest
    from workloads import ResNet18

    kind = "ref" if nhtest.have_reference() else "orc"
    be = nhtest.CpuBackend(kind)
    net = ResNet18(be, batch=args.images, image=args.image)
    x = net.make_input()
    delay = args.start_at - time.time()
    if delay > 0:
        time.sleep(delay)
    t0 = time.perf_counter()
    for _ in range(max(1, args.passes)):
        y = net.forward(x)
    dt = (time.perf_counter() - t0) / max(1, args.passes)
    if args.save:
        np.savez(args.save, softmax=np.asarray(y), logits=np.asarray(net.buffers["fc"]))
    backend = "C oracle" if kind == "orc" else ("reference CCpuMathEngine, MLAS GEMM" if args.mlas else "reference CCpuMathEngine, built-in SSE GEMM")
    print(json.dumps({"images": args.images, "seconds": dt, "backend": backend, "kind": "reference" if kind == "ref" else "port"}))


if __name__ == "__main__":
    main()
