"""The benchmark configurations as sequences of engine calls.

Each network is written once, as the sequence of IMathEngine calls that NeoML's layers issue for it
(ConvLayer -> BlobConvolution, ReLULayer -> VectorReLU, EltwiseSumLayer -> VectorAdd, PoolingLayer ->
BlobMaxPooling, ImageResizeLayer -> BlobResizeImage, GlobalMeanPoolingLayer -> SumMatrixRows + VectorMultiply,
FullyConnectedLayer -> MultiplyMatrixByTransposedMatrix + AddVectorToMatrixRows, SoftmaxLayer ->
MatrixSoftmaxByRows), over a small backend interface. `HipBackend` issues them through the C ABI on
device-resident buffers; the tests and the benchmark's CPU leg plug in a host backend with the same methods.

Weights are random (He-normal, folded batch-norm as a small free term); inputs are synthetic.
"""
import ctypes

import numpy as np


def conv_out(h, w, fh, fw, ph, pw, sh, sw, dh=1, dw=1):
    return 1 + (h - (fh - 1) * dh + 2 * ph - 1) // sh, 1 + (w - (fw - 1) * dw + 2 * pw - 1) // sw


def conv_flops(n, ho, wo, cout, fh, fw, cin):
    return 2 * n * ho * wo * cout * fh * fw * cin


def conv_bytes(n, h, w, cin, ho, wo, cout, fh, fw):
    return 4 * (n * h * w * cin + n * ho * wo * cout + cout * fh * fw * cin + cout)


class HipBackend:
    """Device-resident execution through libneoml_hip.so. Tensors are torch CUDA tensors used as plain memory."""

    name = "hip"

    def __init__(self, record_events=False):
        import torch
        import neoml_amd
        if not torch.cuda.is_available():
            raise RuntimeError("HipBackend needs a GPU")
        self.torch = torch
        self.na = neoml_amd
        self.lib = neoml_amd.load()
        self.dev = torch.device("cuda:0")
        self.stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        self.zero = self.tensor(np.zeros(1, np.float32))
        self.record_events = record_events
        self.events = []  # (tag, flops, bytes, start, stop)
        self._desc_cache = {}
        self.plan = None  # when a list: every launch is also appended as (fn, args, tag, flops, bytes)

    # ---- memory
    def tensor(self, a):
        return self.torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)

    def empty(self, *shape):
        return self.torch.empty(shape, dtype=self.torch.float32, device=self.dev)

    def to_numpy(self, t):
        self.synchronize()
        return t.cpu().numpy()

    def synchronize(self):
        # through the library first: it launches what the stream may have put aside (nhStreamDeferSmallOps)
        self.na.check(self.lib.nhStreamSynchronize(self.stream))
        self.torch.cuda.synchronize()

    def defer_small_ops(self, enable):
        """Small element-wise calls of this backend's stream are launched several at a time. Only while every launch and
        every synchronisation goes through the library: switch it off before torch touches the tensors again."""
        self.na.check(self.lib.nhStreamDeferSmallOps(self.stream, 1 if enable else 0))

    @staticmethod
    def _p(t):
        return None if t is None else ctypes.c_void_p(t.data_ptr())

    def _call(self, fn, *args):
        if self.plan is not None:
            self.plan.append((fn, args, None, 0, 0))
        rc = fn(self.stream, *args)
        if rc != 0:
            self.na.check(rc)

    def _timed(self, tag, flops, nbytes, fn, *args):
        if self.plan is not None:
            self.plan.append((fn, args, tag, flops, nbytes))
            rc = fn(self.stream, *args)
            if rc != 0:
                self.na.check(rc)
            return
        if not self.record_events:
            self._call(fn, *args)
            return
        start = self.torch.cuda.Event(enable_timing=True)
        stop = self.torch.cuda.Event(enable_timing=True)
        start.record()
        self._call(fn, *args)
        stop.record()
        self.events.append((tag, flops, nbytes, start, stop))

    # ---- ops (shapes are N,H,W,C)
    def conv(self, x, filt, bias, ph, pw, sh, sw, out=None, relu=False):
        """relu: the activation in the convolution's own launch, what a rowwise chain of NeoML's graph optimizer
        (convolution + ReLU) asks of the engine; True for the plain ReLU, a number for ReLU with that upper threshold."""
        n, h, w, cin = x.shape
        cout, fh, fw, _ = filt.shape
        key = ("conv", n, h, w, cin, cout, fh, fw, ph, pw, sh, sw)
        d = self._desc_cache.get(key)
        if d is None:
            d = self.na.ConvDesc(n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, 1, 1, 0, 0)
            self.na.check(self.lib.nhInitBlobConvolution(ctypes.byref(d)))
            self._desc_cache[key] = d
        ho, wo = d.resultHeight, d.resultWidth
        if out is None:
            out = self.empty(n, ho, wo, cout)
        tag = "conv%dx%d" % (fh, fw)
        if relu:
            self._timed(tag, conv_flops(n, ho, wo, cout, fh, fw, cin), conv_bytes(n, h, w, cin, ho, wo, cout, fh, fw),
                        self.lib.nhBlobConvolutionWithActivation, ctypes.byref(d), self._p(x), self._p(filt), self._p(bias),
                        1, ctypes.c_float(0.0 if relu is True else float(relu)), self._p(out))
            return out
        self._timed(tag, conv_flops(n, ho, wo, cout, fh, fw, cin), conv_bytes(n, h, w, cin, ho, wo, cout, fh, fw),
                    self.lib.nhBlobConvolution, ctypes.byref(d), self._p(x), self._p(filt), self._p(bias), self._p(out))
        return out

    def relu_(self, x, threshold=None):
        t = self.zero if threshold is None else threshold
        self._timed("relu", 0, 8 * x.numel(), self.lib.nhVectorReLU, self._p(x), self._p(x), x.numel(), self._p(t))
        return x

    def add_(self, a, b):
        """a += b"""
        self._timed("add", 0, 12 * a.numel(), self.lib.nhVectorAdd, self._p(a), self._p(b), self._p(a), a.numel())
        return a

    def pad(self, x, dl, dr, dt, db, value=0.0, out=None):
        n, h, w, c = x.shape
        if out is None:
            out = self.empty(n, h + dt + db, w + dl + dr, c)
        fd = self.na.BlobDesc.of(1, n, 1, h, w, 1, c)
        td = self.na.BlobDesc.of(1, n, 1, h + dt + db, w + dl + dr, 1, c)
        self._timed("pad", 0, 4 * (x.numel() + out.numel()), self.lib.nhBlobResizeImage, ctypes.byref(fd), self._p(x),
                    dl, dr, dt, db, 0, ctypes.c_float(value), ctypes.byref(td), self._p(out))
        return out

    def max_pool(self, x, fh, fw, sh, sw, out=None):
        n, h, w, c = x.shape
        key = ("pool", n, h, w, c, fh, fw, sh, sw)
        d = self._desc_cache.get(key)
        if d is None:
            d = self.na.PoolingDesc(n, h, w, c, fh, fw, sh, sw, 0, 0)
            self.na.check(self.lib.nhInitPooling(ctypes.byref(d)))
            self._desc_cache[key] = d
        if out is None:
            out = self.empty(n, d.resultHeight, d.resultWidth, c)
        self._timed("maxpool", 0, 4 * (x.numel() + out.numel()), self.lib.nhBlobMaxPooling, ctypes.byref(d), self._p(x),
                    None, self._p(out))
        return out

    def global_mean(self, x, out=None):
        n, h, w, c = x.shape
        if out is None:
            out = self.empty(n, c)
        scale = self._desc_cache.setdefault(("scale", h * w), self.tensor(np.array([1.0 / (h * w)], np.float32)))
        self._timed("sumrows", 0, 4 * (x.numel() + out.numel()), self.lib.nhSumMatrixRows, n, self._p(out), self._p(x), h * w, c)
        self._call(self.lib.nhVectorMultiply, self._p(out), self._p(out), out.numel(), self._p(scale))
        return out

    def fc(self, x, weight, bias, out=None):
        m, k = x.shape
        n = weight.shape[0]
        if out is None:
            out = self.empty(m, n)
        self._timed("fc", 2 * m * n * k, 4 * (m * k + n * k + m * n), self.lib.nhMultiplyMatrixByTransposedMatrix,
                    self._p(x), m, k, k, self._p(weight), n, k, self._p(out), n, m * n)
        # ( the layer's second call; the same family, so that a stream on which the product waits for it shows both as one )
        self._timed("fc", 0, 8 * m * n, self.lib.nhAddVectorToMatrixRows, 1, self._p(out), self._p(out), m, n, self._p(bias))
        return out

    def softmax(self, x, out=None):
        if out is None:
            out = self.empty(*x.shape)
        self._timed("softmax", 0, 8 * x.numel(), self.lib.nhMatrixSoftmaxByRows, self._p(x), x.shape[0], x.shape[1], self._p(out))
        return out

    # ---- ops of the depthwise-separable, transformer and line-recogniser configurations
    def scalar(self, value):
        """A one-float device buffer: the form the engine takes multipliers, thresholds and addends in."""
        key = ("scalar", float(value))
        t = self._desc_cache.get(key)
        if t is None:
            t = self._desc_cache[key] = self.tensor(np.array([value], np.float32))
        return t

    def relu6_(self, x):
        return self.relu_(x, self.scalar(6.0))

    def channelwise_conv(self, x, filt, bias, ph, pw, sh, sw, out=None):
        n, h, w, c = x.shape
        fh, fw, _ = filt.shape
        key = ("dw", n, h, w, c, fh, fw, ph, pw, sh, sw)
        d = self._desc_cache.get(key)
        if d is None:
            d = self.na.ConvDesc(n, h, w, c, c, fh, fw, ph, pw, sh, sw, 1, 1, 0, 0)
            self.na.check(self.lib.nhInitBlobChannelwiseConvolution(ctypes.byref(d)))
            self._desc_cache[key] = d
        ho, wo = d.resultHeight, d.resultWidth
        if out is None:
            out = self.empty(n, ho, wo, c)
        self._timed("depthwise", 2 * n * ho * wo * c * fh * fw, 4 * (x.numel() + out.numel() + filt.numel() + c),
                    self.lib.nhBlobChannelwiseConvolution, ctypes.byref(d), self._p(x), self._p(filt), self._p(bias), self._p(out))
        return out

    def separable_block(self, x, expand, channelwise, down, stride, residual, out=None):
        """The fused inverted-residual block (nhMobileNetV2Block) or, without an expand stage, channelwise + 1x1
        (nhChannelwiseWith1x1), ReLU6 behind the expand and channelwise stages as the configuration has it."""
        n, h, w, cin = x.shape
        e, cout = channelwise[0].shape[2], down[0].shape[0]
        ho, wo = (h + stride - 1) // stride, (w + stride - 1) // stride
        key = ("sep", n, h, w, cin, e, cout, stride, residual, expand is not None)
        cached = self._desc_cache.get(key)
        if cached is None:
            d = self.na.SeparableBlockDesc(n, h, w, cin if expand is not None else 0, e, cout, stride, 1 if residual else 0,
                                           1, 6.0, 1, 6.0)
            size = ctypes.c_size_t(0)
            fn = self.lib.nhMobileNetV2BlockWorkspaceSize if expand is not None else self.lib.nhChannelwiseWith1x1WorkspaceSize
            self.na.check(fn(ctypes.byref(d), ctypes.byref(size)))
            cached = self._desc_cache[key] = (d, size.value)
        d, size = cached
        work = self._desc_cache.get("sep_workspace")
        if work is None or work.numel() * 4 < size:
            work = self._desc_cache["sep_workspace"] = self.torch.empty((size + 3) // 4, dtype=self.torch.float32, device=self.dev)
        if out is None:
            out = self.empty(n, ho, wo, cout)
        flops = 2 * n * ho * wo * e * (9 + cout) + (2 * n * h * w * e * cin if expand is not None else 0)
        nbytes = 4 * (x.numel() + out.numel())  # what the block has to move; the expanded tensors are its own business
        if expand is not None:
            self._timed("mbv2block", flops, nbytes, self.lib.nhMobileNetV2Block, ctypes.byref(d), self._p(x),
                        self._p(expand[0]), self._p(expand[1]), self._p(channelwise[0]), self._p(channelwise[1]),
                        self._p(down[0]), self._p(down[1]), self._p(out), self._p(work), size)
        else:
            self._timed("dw+1x1", flops, nbytes, self.lib.nhChannelwiseWith1x1, ctypes.byref(d), self._p(x),
                        self._p(channelwise[0]), self._p(channelwise[1]), self._p(down[0]), self._p(down[1]),
                        self._p(out), self._p(work), size)
        return out

    def pointwise_conv_relu6(self, x, filt, bias, out=None):
        n, h, w, cin = x.shape
        cout = filt.shape[0]
        if out is None:
            out = self.empty(n, h, w, cout)
        self._timed("conv1x1+act", conv_flops(n, h, w, cout, 1, 1, cin), conv_bytes(n, h, w, cin, h, w, cout, 1, 1),
                    self.lib.nhPointwiseConvolutionWithActivation, self._p(x), n * h * w, cin, self._p(filt), self._p(bias),
                    cout, 1, 6.0, self._p(out))
        return out

    def add(self, a, b, out=None):
        if out is None:
            out = self.empty(*a.shape)
        self._timed("add", 0, 12 * a.numel(), self.lib.nhVectorAdd, self._p(a), self._p(b), self._p(out), a.numel())
        return out

    def mul_scalar_(self, x, value, family="eltwise"):
        self._timed(family, 0, 8 * x.numel(), self.lib.nhVectorMultiply, self._p(x), self._p(x), x.numel(), self._p(self.scalar(value)))
        return x

    def transpose(self, x, out=None):
        """[b,h,m,w,c] -> [b,w,m,h,c]"""
        b, h, m, w, c = x.shape
        if out is None:
            out = self.empty(b, w, m, h, c)
        self._timed("transpose", 0, 8 * x.numel(), self.lib.nhTransposeMatrix, b, self._p(x), h, m, w, c, self._p(out), out.numel())
        return out

    def bmm_nn(self, a, b, out=None):
        """a [batch,M,K] x b [batch,K,N]"""
        batch, m, k = a.shape
        n = b.shape[2]
        if out is None:
            out = self.empty(batch, m, n)
        self._timed("bmm", 2 * batch * m * n * k, 4 * batch * (m * k + k * n + m * n), self.lib.nhBatchMultiplyMatrixByMatrix,
                    batch, self._p(a), m, k, self._p(b), n, self._p(out), out.numel())
        return out

    def layer_norm(self, x, scale, bias, out=None, eps=1e-5):
        """CObjectNormalizationLayer::runOnceImpl (NeoML/src/Dnn/Layers/ObjectNormalizationLayer.cpp:181-242):
        thirteen engine calls over a [rows x width] matrix."""
        rows, width = x.shape
        L, p = self.lib, self._p
        if out is None:
            out = self.empty(rows, width)
        key = ("ln", rows, width)
        tmp = self._desc_cache.get(key)
        if tmp is None:
            tmp = self._desc_cache[key] = (self.empty(rows), self.empty(rows), self.empty(rows, width))
        neg_mean, inv_std, sq = tmp
        inv_w, e = self.scalar(1.0 / width), self.scalar(eps)
        mat = 8 * rows * width
        t = lambda nbytes, fn, *a: self._timed("layernorm", 0, nbytes, fn, *a)
        t(mat // 2, L.nhSumMatrixColumns, p(neg_mean), p(x), rows, width)
        t(8 * rows, L.nhVectorNegMultiply, p(neg_mean), p(neg_mean), rows, p(inv_w))
        t(mat, L.nhAddVectorToMatrixColumns, p(x), p(sq), rows, width, p(neg_mean))
        t(mat // 2 * 3, L.nhVectorEltwiseMultiply, p(sq), p(sq), p(sq), rows * width)
        t(mat // 2, L.nhSumMatrixColumns, p(inv_std), p(sq), rows, width)
        t(8 * rows, L.nhVectorMultiply, p(inv_std), p(inv_std), rows, p(inv_w))
        t(8 * rows, L.nhVectorAddValue, p(inv_std), p(inv_std), rows, p(e))
        t(8 * rows, L.nhVectorSqrt, p(inv_std), p(inv_std), rows)
        t(8 * rows, L.nhVectorInv, p(inv_std), p(inv_std), rows)
        t(mat, L.nhAddVectorToMatrixColumns, p(x), p(out), rows, width, p(neg_mean))
        t(mat, L.nhMultiplyDiagMatrixByMatrix, p(inv_std), rows, p(out), width, p(out), rows * width)
        t(mat, L.nhBatchMultiplyMatrixByDiagMatrix, 1, p(out), rows, width, 0, p(scale), 0, p(out), rows * width)
        t(mat, L.nhAddVectorToMatrixRows, 1, p(out), p(out), rows, width, p(bias))
        return out

    def gelu_(self, x):
        """CGELULayer, sigmoid approximation (NeoML/src/Dnn/Layers/GELULayer.cpp:146-160): x * sigmoid(1.702 x)"""
        key = ("gelu", x.numel())
        tmp = self._desc_cache.get(key)
        if tmp is None:
            tmp = self._desc_cache[key] = self.empty(x.numel())
        n, p = x.numel(), self._p
        self._timed("gelu", 0, 8 * n, self.lib.nhVectorMultiply, p(x), p(tmp), n, p(self.scalar(1.702)))
        self._timed("gelu", 0, 8 * n, self.lib.nhVectorSigmoid, p(tmp), p(tmp), n)
        self._timed("gelu", 0, 12 * n, self.lib.nhVectorEltwiseMultiply, p(x), p(tmp), p(x), n)
        return x

    def lstm(self, x, w_in, b_in, w_rec, b_rec, reverse=False, out=None):
        """x [T,B,In] -> h [T,B,H]; zero initial state"""
        T, B, In = x.shape
        H = w_rec.shape[1]
        if out is None:
            out = self.empty(T, B, H)
        key = ("lstm", T, B, In, H, bool(reverse))
        ws = self._desc_cache.get(key)
        if ws is None:
            size = ctypes.c_size_t(0)
            self.na.check(self.lib.nhLstmWorkspaceSize(H, In, T, B, ctypes.byref(size)))
            ws = self._desc_cache[key] = (self.empty((size.value + 3) // 4), size.value)
        p = self._p
        self._timed("lstm", 2 * T * B * 4 * H * (In + H), 4 * (x.numel() + out.numel() + w_in.numel() + w_rec.numel()),
                    self.lib.nhLstm, H, In, p(w_in), p(b_in), p(w_rec), p(b_rec), 1 if reverse else 0, T, B, None, None, p(x),
                    None, p(out), p(ws[0]), ws[1])
        return out

    def merge_channels(self, parts, out=None):
        """concatenate [rows, c_i] along the channels (BlobMergeByDim on BD_Channels)"""
        rows = parts[0].shape[0]
        total = sum(t.shape[1] for t in parts)
        if out is None:
            out = self.empty(rows, total)
        key = ("merge", rows) + tuple(t.data_ptr() for t in parts)
        d = self._desc_cache.get(key)
        if d is None:
            descs = (self.na.BlobDesc * len(parts))(*[self.na.BlobDesc.of(1, rows, 1, 1, 1, 1, t.shape[1]) for t in parts])
            ptrs = (ctypes.c_void_p * len(parts))(*[t.data_ptr() for t in parts])
            d = self._desc_cache[key] = (descs, ptrs, self.na.BlobDesc.of(1, rows, 1, 1, 1, 1, total))
        self._timed("merge", 0, 8 * out.numel(), self.lib.nhBlobMergeByDim, 6, d[0], d[1], len(parts), ctypes.byref(d[2]), self._p(out))
        return out

    def log_(self, x):
        self._timed("eltwise", 0, 8 * x.numel(), self.lib.nhVectorLog, self._p(x), self._p(x), x.numel())
        return x

    def argmax_rows(self, x):
        rows, width = x.shape
        key = ("argmax", rows)
        t = self._desc_cache.get(key)
        if t is None:
            t = self._desc_cache[key] = (self.empty(rows), self.torch.empty(rows, dtype=self.torch.int32, device=self.dev))
        self._timed("argmax", 0, 4 * x.numel(), self.lib.nhFindMaxValueInRows, self._p(x), rows, width, self._p(t[0]), self._p(t[1]), rows)
        return t[1]


class LaunchPlan:
    """A recorded sequence of C-ABI launches with their arguments bound once, replayed with minimal host work
    (the position a native caller of the engine is in). Optionally brackets the launches of chosen op families
    with events recorded on the launch stream through nhEventRecord."""

    def __init__(self, backend, launches):
        self.be = backend
        self.launches = [(fn, (backend.stream,) + tuple(args), tag, flops, nbytes) for fn, args, tag, flops, nbytes in launches]
        self.keep_alive = launches  # ctypes objects referenced by the bound arguments
        self.timed = []  # (tag, flops, bytes, start, stop) of the replays run with events

    def run(self):
        for fn, args, _, _, _ in self.launches:
            rc = fn(*args)
            if rc != 0:
                self.be.na.check(rc)

    def make_events(self, tags, steps):
        lib = self.be.lib
        pools = []
        for _ in range(steps):
            step = []
            for fn, args, tag, flops, nbytes in self.launches:
                if tag in tags:
                    a, b = ctypes.c_void_p(), ctypes.c_void_p()
                    self.be.na.check(lib.nhEventCreate(ctypes.byref(a)))
                    self.be.na.check(lib.nhEventCreate(ctypes.byref(b)))
                    step.append((a, b))
                else:
                    step.append(None)
            pools.append(step)
        return pools

    def run_with_events(self, pool, by_runs=False):
        """by_runs: one pair of events around every run of consecutive launches of one family (the launches of one layer)
        rather than around every launch. An event is itself a call on the stream, so with small calls being put aside
        (HipBackend.defer_small_ops) only this way shows what the stream then does."""
        record, stream = self.be.lib.nhEventRecord, self.be.stream
        if by_runs:
            launches, i = self.launches, 0
            while i < len(launches):
                tag, j, flops, nbytes = launches[i][2], i, 0, 0
                while j < len(launches) and launches[j][2] == tag:
                    flops, nbytes, j = flops + launches[j][3], nbytes + launches[j][4], j + 1
                if tag and (tag.startswith("conv") or tag in ("depthwise", "add")) and j < len(launches) and launches[j][2] == "relu":
                    # the activation in place behind a convolution or a sum: on such a stream it is that call's own launch
                    flops, nbytes, j = flops + launches[j][3], nbytes + launches[j][4], j + 1
                if tag == "pad" and j < len(launches) and launches[j][2] == "maxpool":
                    # the pooling over a padded image: one launch with the padding on such a stream
                    flops, nbytes, j = flops + launches[j][3], nbytes + launches[j][4], j + 1
                if pool[i] is not None:
                    record(pool[i][0], stream)
                for fn, args, _, _, _ in launches[i:j]:
                    rc = fn(*args)
                    if rc != 0:
                        self.be.na.check(rc)
                if pool[i] is not None:
                    record(pool[i][1], stream)
                    self.timed.append((tag, flops, nbytes, pool[i][0], pool[i][1], j - i))
                i = j
            return
        for (fn, args, tag, flops, nbytes), ev in zip(self.launches, pool):
            if ev is None:
                rc = fn(*args)
            else:
                record(ev[0], stream)
                rc = fn(*args)
                record(ev[1], stream)
                self.timed.append((tag, flops, nbytes, ev[0], ev[1]))
            if rc != 0:
                self.be.na.check(rc)

    def family_totals(self):
        """{tag: [launches, total ms, flops, bytes]} of the replays run with events (after a synchronize)."""
        lib = self.be.lib
        fam = {}
        ms = ctypes.c_float(0)
        for tag, flops, nbytes, a, b, *count in self.timed:
            self.be.na.check(lib.nhEventElapsedMs(a, b, ctypes.byref(ms)))
            f = fam.setdefault(tag, [0, 0.0, 0, 0])
            f[0] += count[0] if count else 1
            f[1] += ms.value
            f[2] += flops
            f[3] += nbytes
        return fam


class ResNet18:
    """ResNet-18-style inference: 7x7/2 stem, pad + 3x3/2 max-pool, 4 stages of 2 basic blocks (64/128/256/512,
    batch-norm folded into the convolution free terms), global mean pool, FC -> classes, softmax."""

    STAGES = (64, 128, 256, 512)

    def __init__(self, backend, batch=64, image=224, classes=1000, seed=0xC0FFEE + 2, width_scale=1.0, fused=False):
        """fused: the network as NeoML's OptimizeDnn leaves it: every convolution that feeds a ReLU and nothing else
        (the stem and the first convolution of each block) forms a rowwise chain with it, one engine call."""
        self.be = backend
        self.fused = fused
        self.batch, self.image, self.classes = batch, image, classes
        g = np.random.default_rng(seed)
        self.widths = [max(4, int(round(c * width_scale / 4)) * 4) for c in self.STAGES]

        def conv_params(cout, fh, fw, cin):
            std = np.sqrt(2.0 / (fh * fw * cin))
            f = g.normal(0, std, (cout, fh, fw, cin)).astype(np.float32)
            b = g.normal(0, 0.01, cout).astype(np.float32)
            return f, b

        self.host = {"stem": conv_params(self.widths[0], 7, 7, 3)}
        cin = self.widths[0]
        for s, c in enumerate(self.widths):
            for blk in range(2):
                stride = 2 if (s > 0 and blk == 0) else 1
                self.host["s%db%dc1" % (s, blk)] = conv_params(c, 3, 3, cin)
                self.host["s%db%dc2" % (s, blk)] = conv_params(c, 3, 3, c)
                if stride == 2 or cin != c:
                    self.host["s%db%dsc" % (s, blk)] = conv_params(c, 1, 1, cin)
                cin = c
        self.host["fc"] = (g.normal(0, np.sqrt(1.0 / cin), (classes, cin)).astype(np.float32),
                           g.normal(0, 0.01, classes).astype(np.float32))
        self.dev = {k: (backend.tensor(f), backend.tensor(b)) for k, (f, b) in self.host.items()}
        self.buffers = {}

    def make_input(self, seed=0xC0FFEE + 102):
        g = np.random.default_rng(seed)
        return g.uniform(0, 1, (self.batch, self.image, self.image, 3)).astype(np.float32)

    def conv_flops(self):
        """Algorithmic FLOP of all convolutions + FC for one batch."""
        total = 0
        n, h = self.batch, self.image
        ho, _ = conv_out(h, h, 7, 7, 3, 3, 2, 2)
        total += conv_flops(n, ho, ho, self.widths[0], 7, 7, 3)
        h = (ho + 2 - 3) // 2 + 1
        cin = self.widths[0]
        for s, c in enumerate(self.widths):
            for blk in range(2):
                stride = 2 if (s > 0 and blk == 0) else 1
                ho, _ = conv_out(h, h, 3, 3, 1, 1, stride, stride)
                total += conv_flops(n, ho, ho, c, 3, 3, cin) + conv_flops(n, ho, ho, c, 3, 3, c)
                if ("s%db%dsc" % (s, blk)) in self.host:
                    total += conv_flops(n, ho, ho, c, 1, 1, cin)
                h, cin = ho, c
        total += 2 * n * self.classes * cin
        return total

    def record_plan(self, x):
        """Runs one forward pass while recording its launches; returns (LaunchPlan, output tensor).
        Activation buffers are allocated by this pass and reused by every replay."""
        self.forward(x)  # allocates the buffers
        self.be.plan = []
        out = self.forward(x)
        launches, self.be.plan = self.be.plan, None
        return LaunchPlan(self.be, launches), out

    def forward(self, x):
        be, B = self.be, self.buffers

        def run(key, fn, *args, **kw):
            out = fn(*args, out=B.get(key), **kw)
            B[key] = out
            return out

        f, b = self.dev["stem"]
        y = run("stem", be.conv, x, f, b, 3, 3, 2, 2, relu=self.fused)
        if not self.fused:
            be.relu_(y)
        y = run("pad", be.pad, y, 1, 1, 1, 1, 0.0)
        y = run("pool", be.max_pool, y, 3, 3, 2, 2)
        for s in range(len(self.widths)):
            for blk in range(2):
                stride = 2 if (s > 0 and blk == 0) else 1
                name = "s%db%d" % (s, blk)
                f1, b1 = self.dev[name + "c1"]
                f2, b2 = self.dev[name + "c2"]
                t = run(name + "c1", be.conv, y, f1, b1, 1, 1, stride, stride, relu=self.fused)
                if not self.fused:
                    be.relu_(t)
                t = run(name + "c2", be.conv, t, f2, b2, 1, 1, 1, 1)
                if (name + "sc") in self.dev:
                    fs, bs = self.dev[name + "sc"]
                    sc = run(name + "sc", be.conv, y, fs, bs, 0, 0, stride, stride)
                else:
                    sc = y
                be.add_(t, sc)
                be.relu_(t)
                y = t
        y = run("gap", be.global_mean, y)
        f, b = self.dev["fc"]
        y = run("fc", be.fc, y, f, b)
        return run("softmax", be.softmax, y)


class Network:
    """Shared plumbing of the configurations: named activation buffers reused across passes, plan recording."""

    def __init__(self, backend):
        self.be = backend
        self.buffers = {}

    def run(self, key, fn, *args, **kw):
        out = fn(*args, out=self.buffers.get(key), **kw)
        self.buffers[key] = out
        return out

    def record_plan(self, x):
        self.forward(x)  # allocates the buffers
        self.be.plan = []
        out = self.forward(x)
        launches, self.be.plan = self.be.plan, None
        return LaunchPlan(self.be, launches), out


class MobileNetV2(Network):
    """MobileNetV2-style inference: 3x3/2 stem, inverted residual blocks (1x1 expand x t + ReLU6, 3x3 depthwise + ReLU6,
    1x1 project, residual add when the shape is kept), 1x1 head, global mean pool, FC. Batch-norm folded into the free
    terms, He-normal weights."""

    TABLE = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1))

    def __init__(self, backend, batch=128, image=224, classes=1000, seed=0xC0FFEE + 3, head=1280, fused=False):
        super().__init__(backend)
        self.batch, self.image, self.classes = batch, image, classes
        # fused: the form NeoML's graph optimizer gives the network (one MobileNetV2Block / ChannelwiseWith1x1 call per
        # block, activations inside); same arithmetic
        self.fused = fused
        g = np.random.default_rng(seed)

        def conv(cout, f, cin):
            return (g.normal(0, np.sqrt(2.0 / (f * f * cin)), (cout, f, f, cin)).astype(np.float32),
                    g.normal(0, 0.01, cout).astype(np.float32))

        def depthwise(c):
            return g.normal(0, np.sqrt(2.0 / 9), (3, 3, c)).astype(np.float32), g.normal(0, 0.01, c).astype(np.float32)

        self.host = {"stem": conv(32, 3, 3)}
        self.blocks = []
        cin = 32
        for t, c, n, s in self.TABLE:
            for i in range(n):
                name = "b%d" % len(self.blocks)
                stride = s if i == 0 else 1
                mid = cin * t
                if t != 1:
                    self.host[name + "e"] = conv(mid, 1, cin)
                self.host[name + "d"] = depthwise(mid)
                self.host[name + "p"] = conv(c, 1, mid)
                self.blocks.append((name, t != 1, stride, stride == 1 and cin == c))
                cin = c
        self.host["head"] = conv(head, 1, cin)
        self.host["fc"] = (g.normal(0, np.sqrt(1.0 / head), (classes, head)).astype(np.float32), g.normal(0, 0.01, classes).astype(np.float32))
        self.dev = {k: (backend.tensor(f), backend.tensor(b)) for k, (f, b) in self.host.items()}

    def make_input(self, seed=0xC0FFEE + 103):
        return np.random.default_rng(seed).uniform(0, 1, (self.batch, self.image, self.image, 3)).astype(np.float32)

    def forward(self, x):
        be, run, W = self.be, self.run, self.dev
        # ( the optimizer's form: the stem and its ReLU6 are a rowwise chain = one engine call )
        y = run("stem", be.conv, x, *W["stem"], 1, 1, 2, 2, relu=6.0 if self.fused else False)
        if not self.fused:
            be.relu6_(y)
        for name, expand, stride, residual in self.blocks:
            if self.fused:
                y = run(name + "p", be.separable_block, y, W[name + "e"] if expand else None, W[name + "d"], W[name + "p"],
                        stride, residual)
                continue
            t = y
            if expand:
                t = run(name + "e", be.conv, t, *W[name + "e"], 0, 0, 1, 1)
                be.relu6_(t)
            t = run(name + "d", be.channelwise_conv, t, *W[name + "d"], 1, 1, stride, stride)
            be.relu6_(t)
            t = run(name + "p", be.conv, t, *W[name + "p"], 0, 0, 1, 1)
            if residual:
                be.add_(t, y)
            y = t
        if self.fused:
            y = run("head", be.pointwise_conv_relu6, y, *W["head"])
        else:
            y = run("head", be.conv, y, *W["head"], 0, 0, 1, 1)
            be.relu6_(y)
        y = run("gap", be.global_mean, y)
        return run("fc", be.fc, y, *W["fc"])


class TransformerEncoder(Network):
    """Stack of CTransformerEncoderLayer (post-layernorm, no mask, no dropout, GELU by sigmoid approximation) as
    the engine calls of NeoML/src/Dnn/Layers/TransformerLayer.cpp:249-329 and MultiheadAttentionLayer.cpp:145-456.
    Reshapes that the layer graph does with in-place transforms cost nothing here either."""

    def __init__(self, backend, layers=6, d_model=512, heads=8, ffn=2048, seq=256, batch=32, seed=0xC0FFEE + 4):
        super().__init__(backend)
        self.layers, self.d, self.heads, self.ffn, self.seq, self.batch = layers, d_model, heads, ffn, seq, batch
        g = np.random.default_rng(seed)

        def xavier(n_out, n_in):
            a = np.sqrt(6.0 / (n_in + n_out))
            return g.uniform(-a, a, (n_out, n_in)).astype(np.float32), g.normal(0, 0.01, n_out).astype(np.float32)

        self.host = {}
        for l in range(layers):
            for nm, shape in (("q", (d_model, d_model)), ("k", (d_model, d_model)), ("v", (d_model, d_model)), ("o", (d_model, d_model)),
                              ("f1", (ffn, d_model)), ("f2", (d_model, ffn))):
                self.host["l%d%s" % (l, nm)] = xavier(*shape)
            for nm in ("n1", "n2"):
                self.host["l%d%s" % (l, nm)] = (g.uniform(0.8, 1.2, d_model).astype(np.float32), g.normal(0, 0.05, d_model).astype(np.float32))
        self.dev = {k: (backend.tensor(a), backend.tensor(b)) for k, (a, b) in self.host.items()}

    def make_input(self, seed=0xC0FFEE + 104):
        return np.random.default_rng(seed).normal(0, 1, (self.batch * self.seq, self.d)).astype(np.float32)

    def gemm_flops(self):
        m, d, f, s = self.batch * self.seq, self.d, self.ffn, self.seq
        per_layer = 2 * m * d * d * 4 + 2 * m * d * f * 2 + 2 * 2 * self.batch * self.heads * s * s * (d // self.heads)
        return per_layer * self.layers

    def forward(self, x):
        be, run, W = self.be, self.run, self.dev
        B, S, D, h = self.batch, self.seq, self.d, self.heads
        dk = D // h
        y = x
        for l in range(self.layers):
            n = "l%d" % l
            q = run(n + "q", be.fc, y, *W[n + "q"])
            k = run(n + "k", be.fc, y, *W[n + "k"])
            v = run(n + "v", be.fc, y, *W[n + "v"])
            qt = run(n + "qt", be.transpose, q.reshape(B, S, 1, h, dk))          # [B,h,1,S,dk]
            kt = run(n + "kt", be.transpose, k.reshape(B, S, 1, D, 1))           # [B,D,1,S,1] = [B,h,dk,S]
            vt = run(n + "vt", be.transpose, v.reshape(B, S, 1, h, dk))
            sc = run(n + "sc", be.bmm_nn, qt.reshape(B * h, S, dk), kt.reshape(B * h, dk, S))
            # ( CLinearLayer behind the product, MultiheadAttentionLayer.cpp:175-183: the product's family, whose launch
            # takes the factor along on a stream that puts calls aside )
            be.mul_scalar_(sc, 1.0 / np.sqrt(dk), family="bmm")
            pr = run(n + "pr", be.softmax, sc.reshape(B * h * S, S))
            cx = run(n + "cx", be.bmm_nn, pr.reshape(B * h, S, S), vt.reshape(B * h, S, dk))
            ct = run(n + "ct", be.transpose, cx.reshape(B, h, 1, S, dk))          # [B,S,1,h,dk]
            o = run(n + "o", be.fc, ct.reshape(B * S, D), *W[n + "o"])
            a = run(n + "a", be.add, y, o)
            y1 = run(n + "n1", be.layer_norm, a, *W[n + "n1"])
            f = run(n + "f1", be.fc, y1, *W[n + "f1"])
            be.gelu_(f)
            f2 = run(n + "f2", be.fc, f, *W[n + "f2"])
            a2 = run(n + "a2", be.add, y1, f2)
            y = run(n + "n2", be.layer_norm, a2, *W[n + "n2"])
        return y


class LineRecognizer(Network):
    """OCR line recogniser: 3x3 convolution backbone that pools a 32 x W grey image down to height 1 and width W/4,
    two bidirectional LSTM layers through the fused Lstm entry point, FC to classes + blank, and the engine part of
    CCtcDecodingLayer::RunOnce (NeoML/src/Dnn/Layers/CtcLayer.cpp:205-226): transpose, softmax, log, arg-max.
    The label collapse is host code in the reference too."""

    BACKBONE = ((64, (2, 2)), (128, (2, 2)), (256, None), (256, (2, 1)), (256, (2, 1)), (256, (2, 1)))

    def __init__(self, backend, batch=64, height=32, width=512, hidden=256, classes=100, seed=0xC0FFEE + 5):
        super().__init__(backend)
        self.batch, self.height, self.width, self.hidden, self.classes = batch, height, width, hidden, classes
        if hasattr(backend, "lib") and hasattr(backend, "stream"):
            # every launch of this network goes through the library: the two directions of a bidirectional layer, two
            # nhLstm calls one behind the other with workspaces of their own, may run side by side (what the engine
            # adapter asks for its own stream)
            backend.na.check(backend.lib.nhStreamOverlapLstm(backend.stream, 1))
        g = np.random.default_rng(seed)
        self.host = {}
        cin = 1
        for i, (c, _) in enumerate(self.BACKBONE):
            self.host["c%d" % i] = (g.normal(0, np.sqrt(2.0 / (9 * cin)), (c, 3, 3, cin)).astype(np.float32), g.normal(0, 0.01, c).astype(np.float32))
            cin = c
        feat = cin
        self.lstm_host = {}
        for layer in range(2):
            for direction in ("f", "r"):
                a = 1.0 / np.sqrt(hidden)
                self.lstm_host["l%d%s" % (layer, direction)] = (
                    g.uniform(-a, a, (4 * hidden, feat)).astype(np.float32), g.uniform(-a, a, 4 * hidden).astype(np.float32),
                    g.uniform(-a, a, (4 * hidden, hidden)).astype(np.float32), g.uniform(-a, a, 4 * hidden).astype(np.float32))
            feat = 2 * hidden
        self.host["fc"] = (g.normal(0, np.sqrt(1.0 / feat), (classes + 1, feat)).astype(np.float32), g.normal(0, 0.01, classes + 1).astype(np.float32))
        self.dev = {k: tuple(backend.tensor(a) for a in v) for k, v in list(self.host.items()) + list(self.lstm_host.items())}

    def make_input(self, seed=0xC0FFEE + 105):
        return np.random.default_rng(seed).uniform(0, 1, (self.batch, self.height, self.width, 1)).astype(np.float32)

    def forward(self, x):
        """Returns (labels int32 [B][T], log-probabilities [B*T, classes+1])."""
        be, run, W = self.be, self.run, self.dev
        y = x
        for i, (_, pool) in enumerate(self.BACKBONE):
            y = run("c%d" % i, be.conv, y, *W["c%d" % i], 1, 1, 1, 1)
            be.relu_(y)
            if pool is not None:
                y = run("p%d" % i, be.max_pool, y, pool[0], pool[1], pool[0], pool[1])
        B, one, T, C = y.shape
        assert one == 1
        seq = run("seq", be.transpose, y.reshape(1, B, 1, T, C)).reshape(T, B, C)   # [T,B,C]
        for layer in range(2):
            f = run("l%df" % layer, be.lstm, seq, *W["l%df" % layer], reverse=False)
            r = run("l%dr" % layer, be.lstm, seq, *W["l%dr" % layer], reverse=True)
            H = f.shape[2]
            seq = run("l%dm" % layer, be.merge_channels, [f.reshape(T * B, H), r.reshape(T * B, H)]).reshape(T, B, 2 * H)
        logits = run("fc", be.fc, seq.reshape(T * B, seq.shape[2]), *W["fc"])
        K = logits.shape[1]
        bt = run("bt", be.transpose, logits.reshape(1, T, 1, B, K)).reshape(B * T, K)   # [B,T,K]
        prob = run("prob", be.softmax, bt)
        be.log_(prob)
        labels = be.argmax_rows(prob)
        return labels.reshape(B, T), prob
