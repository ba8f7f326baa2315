#!/usr/bin/env python3
"""The benchmark network as an application of the reference sees it: a CDnn built from NeoML's own layer classes
(oracle/_ref/libNeoML.so, compiled from the reference's sources; the network is put together by oracle/dnn_shim.cpp) on
the HIP engine, timed per CDnn::RunOnce (NeoML/src/Dnn/Dnn.cpp:626-658) over `--passes` passes that a read-back of the
result closes. The reference's layer library is the caller here and the HIP engine the thing measured.

    python oracle/cdnn_run_once.py [--batch 64] [--image 224] [--passes 20]

Prints one JSON line {"ms_per_pass", "images_per_sec", "optimized_ms_per_pass", "optimized_images_per_sec"}; the
"optimized" pair is the same network after NeoML's OptimizeDnn (NeoML/include/NeoML/Dnn/DnnOptimization.h).
"""
import argparse
import ctypes
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--image", type=int, default=224)
    ap.add_argument("--passes", type=int, default=20)
    args = ap.parse_args()
    sys.path.insert(0, ROOT)
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import numpy as np
    import nhtest
    import test_dnn_layers as layers

    dims = (1, args.batch, 1, args.image, args.image, 1, 3)
    x = np.random.default_rng(7).uniform(0, 1, dims).astype(np.float32)
    lib = layers.lib()
    lib.dnn_last_pass_ms.restype = ctypes.c_double
    lib.dnn_set_timed_passes(args.passes)
    engine = nhtest.hip_engine()
    y = layers.dnn_run(engine, 5, dims, x, 1000).reshape(args.batch, 1000)
    plain = lib.dnn_last_pass_ms()
    with layers.optimized():
        y2 = layers.dnn_run(engine, 5, dims, x, 1000).reshape(args.batch, 1000)
        fused = lib.dnn_last_pass_ms()
    lib.dnn_set_timed_passes(0)
    if not (np.allclose(y.sum(axis=1), 1.0, atol=1e-5) and np.allclose(y, y2, rtol=1e-4, atol=1e-5)):
        raise SystemExit("the CDnn passes do not give the same valid softmax")
    print(json.dumps({
        "ms_per_pass": round(plain, 4), "images_per_sec": round(args.batch * 1e3 / plain, 1),
        "optimized_ms_per_pass": round(fused, 4), "optimized_images_per_sec": round(args.batch * 1e3 / fused, 1),
        "passes": args.passes,
    }))


if __name__ == "__main__":
    main()
