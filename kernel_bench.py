"""Per-kernel measurements at the sizes of the BASELINE configurations.

    python kernel_bench.py [--reps N] [--filter substring[,substring...]]

Every line is one C-ABI entry point at one shape: time per launch (events on the launch stream around a run of
back-to-back launches, after a clock warm-up), algorithmic FLOP and bytes (the formulas of the measurement
specification: conv 2*N*Ho*Wo*Cout*fh*fw*Cin and 4*(in+out+filter+bias); GEMM 2*M*N*K and 4*(MK+NK+MN); depthwise
2*N*Ho*Wo*C*fh*fw and 4*(in+out+filter+bias); pooling 4*(in+out); unary 8n, binary 12n; softmax 8*rows*width;
transpose/copy 8n), and the fraction of the bounding peak (fp32 MFMA 157.3 TFLOP/s or HBM 8 TB/s).
Buffers that are re-read on every repetition can sit in the 256 MB last-level cache; shapes whose working set is
below that are marked with '*' in the output: their GB/s is a cache-assisted figure, not an HBM one.
"""
import argparse
import ctypes
import sys

import numpy as np

MFMA_PEAK = 157.3e12
HBM_PEAK = 8.0e12
LLC_BYTES = 256e6


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=0, help="launches per measurement (default: enough for ~0.3 s)")
    ap.add_argument("--filter", default="")
    ap.add_argument("--vendor", action="store_true",
                    help="under every convolution and matrix product line, time the vendor library at the same shape "
                         "(torch.nn.functional.conv2d = MIOpen, torch.matmul / torch.bmm = hipBLASLt or rocBLAS, fp32): "
                         "a yardstick on the same device, nothing the engine calls")
    args = ap.parse_args()

    import torch
    import neoml_amd
    lib = neoml_amd.load()
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def P(t):
        return None if t is None else ctypes.c_void_p(t.data_ptr())

    def rand(*shape):
        return torch.rand(shape, device=dev, dtype=torch.float32) * 2 - 1

    def empty(*shape):
        return torch.empty(shape, device=dev, dtype=torch.float32)

    rows = []
    wanted = [w for w in args.filter.split(",") if w]

    def measure(name, fn, flops, nbytes, footprint):
        if wanted and not any(w in name for w in wanted):
            return
        neoml_amd.check(fn())
        torch.cuda.synchronize()
        # clock warm-up + estimate
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            fn()
        e1.record()
        torch.cuda.synchronize()
        est = max(e0.elapsed_time(e1) / 20, 1e-3)
        reps = args.reps or int(min(max(300.0 / est, 50), 20000))
        for _ in range(reps // 2):
            fn()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / reps * 1e3
        tf = flops / us / 1e6 if flops else 0.0
        gbs = nbytes / us / 1e3
        mfma_frac = flops / (us * 1e-6) / MFMA_PEAK if flops else 0.0
        hbm_frac = nbytes / (us * 1e-6) / HBM_PEAK
        cached = "*" if footprint < LLC_BYTES else " "
        rows.append((name, us, tf, gbs, mfma_frac, hbm_frac, cached))
        print("%-58s %9.1f us %7.1f TFLOP/s %5.1f%%  %8.1f GB/s%s %5.1f%%" % (
            name, us, tf, 100 * mfma_frac, gbs, cached, 100 * hbm_frac), flush=True)

    def vendor(name, op, flops, nbytes):
        """op() runs the vendor library's routine on torch's current stream (the one the engine's launches use here)"""
        if not args.vendor or (wanted and not any(w in name for w in wanted)):
            return
        try:
            op()
            torch.cuda.synchronize()
        except Exception as e:  # a shape the library refuses is reported, not fatal
            print("%-58s vendor library: %s" % ("  " + name[:56], str(e).splitlines()[0][:60]), flush=True)
            return

        def call():
            op()
            return 0
        measure(("  vendor: " + name)[:58], call, flops, nbytes, nbytes)

    zero = torch.zeros(1, device=dev)
    six = torch.full((1,), 6.0, device=dev)

    # ---- convolutions (config 1, 2, 3, 5)
    def conv(tag, n, h, w, cin, cout, f, p, s):
        d = neoml_amd.ConvDesc(n, h, w, cin, cout, f, f, p, p, s, s, 1, 1, 0, 0)
        neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
        x, flt, b = rand(n, h, w, cin), rand(cout, f, f, cin) * 0.05, rand(cout)
        y = empty(n, d.resultHeight, d.resultWidth, cout)
        fl = 2 * n * d.resultHeight * d.resultWidth * cout * f * f * cin
        by = 4 * (x.numel() + y.numel() + flt.numel() + cout)
        measure("BlobConvolution %s %dx%dx%dx%d->%d %dx%d/%d" % (tag, n, h, w, cin, cout, f, f, s),
                lambda: lib.nhBlobConvolution(stream, ctypes.byref(d), P(x), P(flt), P(b), P(y)), fl, by, by)
        if args.vendor:
            # the same tensors as logical NCHW views of channels-last memory, and as plain NCHW
            xl, wl = x.permute(0, 3, 1, 2), flt.permute(0, 3, 1, 2)
            vendor("conv2d channels-last %s %dx%dx%dx%d->%d %dx%d/%d" % (tag, n, h, w, cin, cout, f, f, s),
                   lambda: torch.nn.functional.conv2d(xl, wl, b, stride=s, padding=p), fl, by)
            xc, wc = xl.contiguous(), wl.contiguous()
            vendor("conv2d NCHW %s %dx%dx%dx%d->%d %dx%d/%d" % (tag, n, h, w, cin, cout, f, f, s),
                   lambda: torch.nn.functional.conv2d(xc, wc, b, stride=s, padding=p), fl, by)

    conv("cfg1", 32, 32, 32, 64, 64, 3, 1, 1)
    conv("cfg2 stem", 64, 224, 224, 3, 64, 7, 3, 2)
    conv("cfg2 s1", 64, 56, 56, 64, 64, 3, 1, 1)
    conv("cfg2 s2", 64, 28, 28, 128, 128, 3, 1, 1)
    conv("cfg2 s3", 64, 14, 14, 256, 256, 3, 1, 1)
    conv("cfg2 s4", 64, 7, 7, 512, 512, 3, 1, 1)
    conv("cfg2 s2 down", 64, 56, 56, 64, 128, 3, 1, 2)
    conv("cfg2 s2 short", 64, 56, 56, 64, 128, 1, 0, 2)
    conv("cfg3 stem", 128, 224, 224, 3, 32, 3, 1, 2)
    conv("cfg3 project", 128, 112, 112, 32, 16, 1, 0, 1)
    conv("cfg3 expand", 128, 112, 112, 16, 96, 1, 0, 1)
    conv("cfg3 project", 128, 56, 56, 96, 24, 1, 0, 1)
    conv("cfg3 expand", 128, 56, 56, 24, 144, 1, 0, 1)
    conv("cfg3 project", 128, 56, 56, 144, 24, 1, 0, 1)
    conv("cfg3 expand", 128, 28, 28, 32, 192, 1, 0, 1)
    conv("cfg3 project", 128, 28, 28, 192, 32, 1, 0, 1)
    conv("cfg3 expand", 128, 14, 14, 64, 384, 1, 0, 1)
    conv("cfg3 project", 128, 14, 14, 384, 64, 1, 0, 1)
    conv("cfg5 conv1", 64, 32, 512, 1, 64, 3, 1, 1)
    conv("cfg5 conv3", 64, 16, 256, 64, 128, 3, 1, 1)

    # ---- gradients of the convolutions (a training step of config 1 / 2)
    def conv_grad(tag, n, h, w, cin, cout, f, p, s):
        d = neoml_amd.ConvDesc(n, h, w, cin, cout, f, f, p, p, s, s, 1, 1, 0, 0)
        neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
        x, flt = rand(n, h, w, cin), rand(cout, f, f, cin) * 0.05
        g = rand(n, d.resultHeight, d.resultWidth, cout)
        dx, dflt = empty(n, h, w, cin), torch.zeros_like(flt)
        size = ctypes.c_size_t(0)
        neoml_amd.check(lib.nhBlobConvolutionBackwardWorkspaceSize(ctypes.byref(d), ctypes.byref(size)))
        work = torch.empty((size.value + 15) // 4 + 4, dtype=torch.float32, device=dev)
        fl = 2 * n * d.resultHeight * d.resultWidth * cout * f * f * cin
        by = 4 * (x.numel() + g.numel() + flt.numel())
        shape = "%s %dx%dx%dx%d->%d %dx%d/%d" % (tag, n, h, w, cin, cout, f, f, s)
        measure("BlobConvolutionBackward " + shape, lambda: lib.nhBlobConvolutionBackward(
            stream, ctypes.byref(d), P(g), P(flt), None, P(dx), P(work), size.value), fl, by, by)
        measure("BlobConvolutionLearnAdd " + shape, lambda: lib.nhBlobConvolutionLearnAdd(
            stream, ctypes.byref(d), P(x), P(g), P(dflt)), fl, by, by)

    conv_grad("cfg1", 32, 32, 32, 64, 64, 3, 1, 1)
    conv_grad("cfg2 stem", 64, 224, 224, 3, 64, 7, 3, 2)
    conv_grad("cfg2 s1", 64, 56, 56, 64, 64, 3, 1, 1)
    conv_grad("cfg2 s2", 64, 28, 28, 128, 128, 3, 1, 1)
    conv_grad("cfg2 s3", 64, 14, 14, 256, 256, 3, 1, 1)
    conv_grad("cfg2 s4", 64, 7, 7, 512, 512, 3, 1, 1)
    conv_grad("cfg2 s2 down", 64, 56, 56, 64, 128, 3, 1, 2)
    conv_grad("cfg2 s2 short", 64, 56, 56, 64, 128, 1, 0, 2)

    # ---- matrix products (config 2 FC, config 4, config 5)
    def gemm_nt(tag, m, n, k):
        a, b, c = rand(m, k), rand(n, k), empty(m, n)
        measure("MultiplyMatrixByTransposedMatrix %s %dx%dx%d" % (tag, m, n, k),
                lambda: lib.nhMultiplyMatrixByTransposedMatrix(stream, P(a), m, k, k, P(b), n, k, P(c), n, m * n),
                2 * m * n * k, 4 * (m * k + n * k + m * n), 4 * (m * k + n * k + m * n))
        vendor("matmul A B^T %s %dx%dx%d" % (tag, m, n, k), lambda: torch.matmul(a, b.t(), out=c),
               2 * m * n * k, 4 * (m * k + n * k + m * n))

    gemm_nt("cfg2 fc", 64, 1000, 512)
    gemm_nt("cfg4 qkv/out", 8192, 512, 512)
    gemm_nt("cfg4 ffn1", 8192, 2048, 512)
    gemm_nt("cfg4 ffn2", 8192, 512, 2048)
    gemm_nt("cfg5 lstm in", 8192, 1024, 256)
    gemm_nt("cfg5 fc", 8192, 101, 512)

    def gemm_batched(tag, kind, batch, m, n, k):
        fn = {"nn": lib.nhBatchMultiplyMatrixByMatrix, "tn": lib.nhBatchMultiplyTransposedMatrixByMatrix}[kind]
        a = rand(batch, m, k) if kind == "nn" else rand(batch, k, m)
        b, c = rand(batch, k, n), empty(batch, m, n)
        if kind == "nn":
            call = lambda: fn(stream, batch, P(a), m, k, P(b), n, P(c), c.numel())
        else:
            call = lambda: fn(stream, batch, P(a), k, m, P(b), n, P(c), c.numel())
        by = 4 * batch * (m * k + k * n + m * n)
        measure("%s %s b%d %dx%dx%d" % ("MultiplyMatrixByMatrix" if kind == "nn" else "MultiplyTransposedMatrixByMatrix",
                                         tag, batch, m, n, k), call, 2 * batch * m * n * k, by, by)
        if kind == "nn":
            vendor("bmm %s b%d %dx%dx%d" % (tag, batch, m, n, k), lambda: torch.bmm(a, b, out=c), 2 * batch * m * n * k, by)

    gemm_batched("cfg4 QK^T", "nn", 256, 256, 256, 64)
    gemm_batched("cfg4 PV", "nn", 256, 256, 64, 256)
    gemm_batched("fc grad", "tn", 1, 512, 2048, 8192)

    # ---- the fused block of the graph optimizer (config 3): expand 1x1 -> depthwise 3x3 -> down 1x1 (+ input)
    def block(n, h, w, cin, e, cout, stride, residual):
        d = neoml_amd.SeparableBlockDesc(n, h, w, cin, e, cout, stride, 1 if residual else 0, 1, 6.0, 1, 6.0)  # ReLU6 twice
        size = ctypes.c_size_t(0)
        neoml_amd.check(lib.nhMobileNetV2BlockWorkspaceSize(ctypes.byref(d), ctypes.byref(size)))
        work = empty((size.value + 15) // 4 + 4)
        x, ef, eb, cf, cb, df, db = rand(n, h, w, cin), rand(e, cin), rand(e), rand(3, 3, e), rand(e), rand(cout, e), rand(cout)
        ho, wo = (h + stride - 1) // stride, (w + stride - 1) // stride
        out = empty(n, ho, wo, cout)
        fl = 2 * n * (h * w * cin * e + ho * wo * e * (9 + cout))
        by = 4 * (x.numel() + out.numel() + ef.numel() + cf.numel() + df.numel() + 2 * e + cout)
        measure("MobileNetV2Block cfg3 %dx%dx%dx%d->%d->%d /%d" % (n, h, w, cin, e, cout, stride),
                lambda: lib.nhMobileNetV2Block(stream, ctypes.byref(d), P(x), P(ef), P(eb), P(cf), P(cb), P(df), P(db), P(out),
                                               P(work), size.value), fl, by, by)

    block(128, 112, 112, 16, 96, 24, 2, False)
    block(128, 56, 56, 24, 144, 24, 1, True)
    block(128, 56, 56, 24, 144, 32, 2, False)
    block(128, 28, 28, 32, 192, 32, 1, True)
    block(128, 14, 14, 64, 384, 64, 1, True)

    # ---- depthwise convolution (config 3)
    def dw(n, h, w, c, s):
        d = neoml_amd.ConvDesc(n, h, w, c, c, 3, 3, 1, 1, s, s, 1, 1, 0, 0)
        neoml_amd.check(lib.nhInitBlobChannelwiseConvolution(ctypes.byref(d)))
        x, flt, b = rand(n, h, w, c), rand(3, 3, c), rand(c)
        y = empty(n, d.resultHeight, d.resultWidth, c)
        by = 4 * (x.numel() + y.numel() + flt.numel() + c)
        measure("BlobChannelwiseConvolution cfg3 %dx%dx%dx%d 3x3/%d" % (n, h, w, c, s),
                lambda: lib.nhBlobChannelwiseConvolution(stream, ctypes.byref(d), P(x), P(flt), P(b), P(y)),
                2 * n * d.resultHeight * d.resultWidth * c * 9, by, by)
        if by >= 200e6:
            # as inside a network, where the input was written by the layer in front and is not in the last-level cache:
            # the launches rotate through enough input / output pairs to exceed it several times
            pairs = [(x, y)] + [(rand(n, h, w, c), empty(n, d.resultHeight, d.resultWidth, c)) for _ in range(max(1, int(1.2e9 // by)))]
            turn = [0]

            def cold():
                xi, yi = pairs[turn[0] % len(pairs)]
                turn[0] += 1
                return lib.nhBlobChannelwiseConvolution(stream, ctypes.byref(d), P(xi), P(flt), P(b), P(yi))
            measure("BlobChannelwiseConvolution cold %dx%dx%dx%d 3x3/%d" % (n, h, w, c, s), cold,
                    2 * n * d.resultHeight * d.resultWidth * c * 9, by, 2e9)

    def dw_gradients(n, h, w, c, s):
        d = neoml_amd.ConvDesc(n, h, w, c, c, 3, 3, 1, 1, s, s, 1, 1, 0, 0)
        neoml_amd.check(lib.nhInitBlobChannelwiseConvolution(ctypes.byref(d)))
        x, flt = rand(n, h, w, c), rand(3, 3, c)
        g = rand(n, d.resultHeight, d.resultWidth, c)
        dx, dflt, dfree = empty(n, h, w, c), torch.zeros((3, 3, c), device=dev), torch.zeros(c, device=dev)
        by = 4 * (x.numel() + g.numel())
        tag = "cfg3 %dx%dx%dx%d 3x3/%d" % (n, h, w, c, s)
        measure("BlobChannelwiseConvolutionBackward " + tag,
                lambda: lib.nhBlobChannelwiseConvolutionBackward(stream, ctypes.byref(d), P(g), P(flt), P(dx)),
                2 * g.numel() * 9, by, by)
        measure("BlobChannelwiseConvolutionLearnAdd " + tag,
                lambda: lib.nhBlobChannelwiseConvolutionLearnAdd(stream, ctypes.byref(d), P(x), P(g), P(dflt), P(dfree)),
                2 * g.numel() * 9, by, by)

    dw(128, 112, 112, 96, 2)
    dw(128, 112, 112, 32, 1)
    dw(128, 56, 56, 144, 1)
    dw(128, 28, 28, 192, 2)
    dw(128, 14, 14, 384, 1)
    dw(128, 7, 7, 960, 1)
    dw_gradients(128, 56, 56, 144, 1)
    dw_gradients(128, 112, 112, 96, 2)
    dw_gradients(128, 14, 14, 384, 1)

    # ---- pooling, padding (config 2, 5)
    def pool(tag, n, h, w, c, f_h, f_w, s_h, s_w, mean=False):
        d = neoml_amd.PoolingDesc(n, h, w, c, f_h, f_w, s_h, s_w, 0, 0)
        neoml_amd.check(lib.nhInitPooling(ctypes.byref(d)))
        x, y = rand(n, h, w, c), empty(n, d.resultHeight, d.resultWidth, c)
        by = 4 * (x.numel() + y.numel())
        if mean:
            measure("BlobMeanPooling %s %dx%dx%dx%d %dx%d/%d" % (tag, n, h, w, c, f_h, f_w, s_h),
                    lambda: lib.nhBlobMeanPooling(stream, ctypes.byref(d), P(x), P(y)), 0, by, by)
        else:
            measure("BlobMaxPooling %s %dx%dx%dx%d %dx%d/%d" % (tag, n, h, w, c, f_h, f_w, s_h),
                    lambda: lib.nhBlobMaxPooling(stream, ctypes.byref(d), P(x), None, P(y)), 0, by, by)

    pool("cfg2", 64, 114, 114, 64, 3, 3, 2, 2)
    pool("cfg5", 64, 32, 512, 64, 2, 2, 2, 2)
    pool("cfg2", 64, 114, 114, 64, 3, 3, 2, 2, mean=True)
    pool("at the depthwise shape", 128, 112, 112, 96, 3, 3, 2, 2)
    pool("at the depthwise shape", 128, 112, 112, 32, 3, 3, 1, 1)

    def pool_grad(n, h, w, c, f, s_):
        d = neoml_amd.PoolingDesc(n, h, w, c, f, f, s_, s_, 0, 0)
        neoml_amd.check(lib.nhInitPooling(ctypes.byref(d)))
        x, y = rand(n, h, w, c), empty(n, d.resultHeight, d.resultWidth, c)
        idx = torch.empty(y.shape, dtype=torch.int32, device=dev)
        neoml_amd.check(lib.nhBlobMaxPooling(stream, ctypes.byref(d), P(x), P(idx), P(y)))
        measure("BlobMaxPooling with indices cfg2 %dx%dx%dx%d %dx%d/%d" % (n, h, w, c, f, f, s_),
                lambda: lib.nhBlobMaxPooling(stream, ctypes.byref(d), P(x), P(idx), P(y)),
                0, 4 * (x.numel() + 2 * y.numel()), 4 * (x.numel() + 2 * y.numel()))
        g, dx = rand(*y.shape), empty(n, h, w, c)
        measure("BlobMaxPoolingBackward cfg2 %dx%dx%dx%d %dx%d/%d" % (n, h, w, c, f, f, s_),
                lambda: lib.nhBlobMaxPoolingBackward(stream, ctypes.byref(d), P(g), P(idx), P(dx)),
                0, 4 * (2 * g.numel() + dx.numel()), 4 * (2 * g.numel() + dx.numel()))
        measure("BlobMeanPoolingBackward cfg2 %dx%dx%dx%d %dx%d/%d" % (n, h, w, c, f, f, s_),
                lambda: lib.nhBlobMeanPoolingBackward(stream, ctypes.byref(d), P(g), P(dx)),
                0, 4 * (g.numel() + dx.numel()), 4 * (g.numel() + dx.numel()))

    pool_grad(64, 114, 114, 64, 3, 2)

    x, y = rand(64, 112, 112, 64), empty(64, 114, 114, 64)
    fd, td = neoml_amd.BlobDesc.of(1, 64, 1, 112, 112, 1, 64), neoml_amd.BlobDesc.of(1, 64, 1, 114, 114, 1, 64)
    measure("BlobResizeImage cfg2 pad 112->114 x64ch", lambda: lib.nhBlobResizeImage(
        stream, ctypes.byref(fd), P(x), 1, 1, 1, 1, 0, ctypes.c_float(0), ctypes.byref(td), P(y)),
        0, 4 * (x.numel() + y.numel()), 4 * (x.numel() + y.numel()))

    # ---- element-wise (sizes of configs 2-4)
    for n in (64 * 112 * 112 * 64, 128 * 112 * 112 * 96, 8192 * 2048, 64 * 56 * 56 * 64):
        a, b, c = rand(n), rand(n), empty(n)
        measure("VectorReLU in place n=%d" % n, lambda: lib.nhVectorReLU(stream, P(a), P(a), n, P(zero)), 0, 8 * n, 4 * n)
        measure("VectorReLU6 n=%d" % n, lambda: lib.nhVectorReLU(stream, P(a), P(c), n, P(six)), 0, 8 * n, 8 * n)
        measure("VectorAdd n=%d" % n, lambda: lib.nhVectorAdd(stream, P(a), P(b), P(c), n), 0, 12 * n, 12 * n)
        measure("VectorSigmoid n=%d" % n, lambda: lib.nhVectorSigmoid(stream, P(a), P(c), n), 0, 8 * n, 8 * n)
        measure("VectorReLUDiff n=%d" % n, lambda: lib.nhVectorReLUDiff(stream, P(a), P(b), P(c), n, P(zero)), 0, 12 * n, 12 * n)
        measure("VectorEltwiseMultiply n=%d" % n, lambda: lib.nhVectorEltwiseMultiply(stream, P(a), P(b), P(c), n), 0, 12 * n, 12 * n)
        del a, b, c
    for n in (1 << 26, 1 << 28):
        c = empty(n)
        measure("VectorFill (write only) n=%d" % n, lambda: lib.nhVectorFill(stream, P(c), ctypes.c_float(1.5), n), 0, 4 * n, 4 * n)
        a = rand(n)
        measure("VectorSum (read only) n=%d" % n, lambda: lib.nhVectorSum(stream, P(a), n, P(zero)), 0, 4 * n, 4 * n)
        del a, c
    if any("calibrate" in w for w in wanted):
        # a copy of known size (256 MiB read, 256 MiB written): the scale of the FETCH_SIZE / WRITE_SIZE counters
        n = 1 << 26
        a, c = rand(n), empty(n)
        measure("VectorCopy calibrate n=%d" % n, lambda: lib.nhVectorCopy(stream, P(c), P(a), n), 0, 8 * n, 8 * n)
        del a, c
    n = 8192 * 512
    a, c = rand(n), empty(n)
    measure("VectorTanh n=%d" % n, lambda: lib.nhVectorTanh(stream, P(a), P(c), n), 0, 8 * n, 8 * n)
    measure("VectorCopy n=%d" % n, lambda: lib.nhVectorCopy(stream, P(c), P(a), n), 0, 8 * n, 8 * n)

    # ---- row / column families (config 4 layer-norm set, bias adds, softmax, arg-max)
    h, w = 8192, 512
    m, out, vec_w, vec_h = rand(h, w), empty(h, w), rand(w), rand(h)
    by = 8 * h * w
    measure("AddVectorToMatrixRows %dx%d" % (h, w), lambda: lib.nhAddVectorToMatrixRows(stream, 1, P(m), P(out), h, w, P(vec_w)), 0, by, by)
    measure("AddVectorToMatrixColumns %dx%d" % (h, w), lambda: lib.nhAddVectorToMatrixColumns(stream, P(m), P(out), h, w, P(vec_h)), 0, by, by)
    measure("SumMatrixColumns %dx%d" % (h, w), lambda: lib.nhSumMatrixColumns(stream, P(vec_h), P(m), h, w), 0, 4 * h * w, 4 * h * w)
    measure("MultiplyDiagMatrixByMatrix %dx%d" % (h, w), lambda: lib.nhMultiplyDiagMatrixByMatrix(stream, P(vec_h), h, P(m), w, P(out), h * w), 0, by, by)
    measure("BatchMultiplyMatrixByDiagMatrix %dx%d" % (h, w), lambda: lib.nhBatchMultiplyMatrixByDiagMatrix(
        stream, 1, P(m), h, w, h * w, P(vec_w), w, P(out), h * w), 0, by, by)
    for rows_, width in ((65536, 256), (8192, 101), (64, 1000)):
        s_in, s_out = rand(rows_, width), empty(rows_, width)
        measure("MatrixSoftmaxByRows %dx%d" % (rows_, width), lambda: lib.nhMatrixSoftmaxByRows(stream, P(s_in), rows_, width, P(s_out)),
                0, 8 * rows_ * width, 8 * rows_ * width)
    s_in = rand(8192, 101)
    mv, mi = empty(8192), torch.empty(8192, dtype=torch.int32, device=dev)
    measure("FindMaxValueInRows 8192x101", lambda: lib.nhFindMaxValueInRows(stream, P(s_in), 8192, 101, P(mv), P(mi), 8192),
            0, 4 * 8192 * 101, 4 * 8192 * 101)
    t_in, t_out = rand(64 * 56 * 56, 64), empty(64)
    measure("SumMatrixRowsAdd free-term gradient 200704x64", lambda: lib.nhSumMatrixRowsAdd(stream, 1, P(t_out), P(t_in), 64 * 56 * 56, 64),
            0, 4 * t_in.numel(), 4 * t_in.numel())
    g_in, g_out = rand(64, 49, 512), empty(64, 512)
    measure("SumMatrixRows cfg2 global mean 64x49x512", lambda: lib.nhSumMatrixRows(stream, 64, P(g_out), P(g_in), 49, 512),
            0, 4 * g_in.numel(), 4 * g_in.numel())

    # ---- transposes of the attention layers (config 4), split / merge (config 5)
    t_in, t_out = rand(32, 256, 1, 8, 64), empty(32, 8, 1, 256, 64)
    measure("TransposeMatrix cfg4 [32,256,1,8,64]", lambda: lib.nhTransposeMatrix(stream, 32, P(t_in), 256, 1, 8, 64, P(t_out), t_out.numel()),
            0, 8 * t_in.numel(), 8 * t_in.numel())
    t_in, t_out = rand(32, 256, 1, 512, 1), empty(32, 512, 1, 256, 1)
    measure("TransposeMatrix cfg4 K [32,256,1,512,1]", lambda: lib.nhTransposeMatrix(stream, 32, P(t_in), 256, 1, 512, 1, P(t_out), t_out.numel()),
            0, 8 * t_in.numel(), 8 * t_in.numel())
    big = rand(64, 1024)
    parts = [empty(64, 256) for _ in range(4)]
    bd = neoml_amd.BlobDesc.of(1, 64, 1, 1, 1, 1, 1024)
    pd = (neoml_amd.BlobDesc * 4)(*[neoml_amd.BlobDesc.of(1, 64, 1, 1, 1, 1, 256)] * 4)
    ptrs = (ctypes.c_void_p * 4)(*[p.data_ptr() for p in parts])
    measure("BlobSplitByDim cfg5 gates 64x1024 -> 4x256", lambda: lib.nhBlobSplitByDim(stream, 6, ctypes.byref(bd), P(big), pd, ptrs, 4),
            0, 8 * big.numel(), 8 * big.numel())

    # ---- LSTM (config 5, one direction of layer 1)
    T, B, H, In = 128, 64, 256, 256
    w_in, w_rec, b_in, xs = rand(4 * H, In) * 0.1, rand(4 * H, H) * 0.1, rand(4 * H), rand(T, B, In)
    hs = empty(T, B, H)
    size = ctypes.c_size_t(0)
    neoml_amd.check(lib.nhLstmWorkspaceSize(H, In, T, B, ctypes.byref(size)))
    work = torch.empty((size.value + 3) // 4, dtype=torch.float32, device=dev)
    measure("Lstm cfg5 T=128 B=64 H=256 In=256", lambda: lib.nhLstm(
        stream, H, In, P(w_in), P(b_in), P(w_rec), None, 0, T, B, None, None, P(xs), None, P(hs), P(work), size.value),
        2 * T * B * 4 * H * (In + H), 4 * (xs.numel() + hs.numel() + w_in.numel() + w_rec.numel()), 1e9)
    return 0


if __name__ == "__main__":
    sys.exit(main())
