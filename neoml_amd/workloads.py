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
        return t.cpu().numpy()

    def synchronize(self):
        self.torch.cuda.synchronize()

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
    def conv(self, x, filt, bias, ph, pw, sh, sw, out=None):
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
        self._call(self.lib.nhAddVectorToMatrixRows, 1, self._p(out), self._p(out), m, n, self._p(bias))
        return out

    def softmax(self, x, out=None):
        if out is None:
            out = self.empty(*x.shape)
        self._timed("softmax", 0, 8 * x.numel(), self.lib.nhMatrixSoftmaxByRows, self._p(x), x.shape[0], x.shape[1], self._p(out))
        return out


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

    def run_with_events(self, pool):
        record, stream = self.be.lib.nhEventRecord, self.be.stream
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
        for tag, flops, nbytes, a, b in self.timed:
            self.be.na.check(lib.nhEventElapsedMs(a, b, ctypes.byref(ms)))
            f = fam.setdefault(tag, [0, 0.0, 0, 0])
            f[0] += 1
            f[1] += ms.value
            f[2] += flops
            f[3] += nbytes
        return fam


class ResNet18:
    """ResNet-18-style inference: 7x7/2 stem, pad + 3x3/2 max-pool, 4 stages of 2 basic blocks (64/128/256/512,
    batch-norm folded into the convolution free terms), global mean pool, FC -> classes, softmax."""

    STAGES = (64, 128, 256, 512)

    def __init__(self, backend, batch=64, image=224, classes=1000, seed=0xC0FFEE + 2, width_scale=1.0):
        self.be = backend
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
        y = run("stem", be.conv, x, f, b, 3, 3, 2, 2)
        be.relu_(y)
        y = run("pad", be.pad, y, 1, 1, 1, 1, 0.0)
        y = run("pool", be.max_pool, y, 3, 3, 2, 2)
        for s in range(len(self.widths)):
            for blk in range(2):
                stride = 2 if (s > 0 and blk == 0) else 1
                name = "s%db%d" % (s, blk)
                f1, b1 = self.dev[name + "c1"]
                f2, b2 = self.dev[name + "c2"]
                t = run(name + "c1", be.conv, y, f1, b1, 1, 1, stride, stride)
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
