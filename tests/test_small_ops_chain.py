"""nhStreamDeferSmallOps: small element-wise calls that a stream puts aside and launches together must leave the very
bits that the separate launches leave, whatever the calls have to do with one another (in place, shifted views of
one buffer, a device scalar that a call in front has produced), and nothing may overtake or be overtaken by them."""
import ctypes

import numpy as np
import pytest

from test_oracle import rng

pytestmark = pytest.mark.gpu

ARENA = 1 << 19


class Streams:
    """Two streams of the library: one that launches every call by itself, one that puts small calls aside."""

    def __init__(self):
        import torch
        import neoml_amd
        self.torch, self.na, self.lib = torch, neoml_amd, neoml_amd.load()
        self.dev = torch.device("cuda:0")
        self.plain, self.deferring = ctypes.c_void_p(), ctypes.c_void_p()
        neoml_amd.check(self.lib.nhStreamCreate(ctypes.byref(self.plain)))
        neoml_amd.check(self.lib.nhStreamCreate(ctypes.byref(self.deferring)))
        neoml_amd.check(self.lib.nhStreamDeferSmallOps(self.deferring, 1))

    def close(self):
        self.na.check(self.lib.nhStreamDestroy(self.plain))
        self.na.check(self.lib.nhStreamDestroy(self.deferring))

    def run(self, stream, program, start):
        """program: [(entry point, [arguments; ("at", offset) stands for a pointer into the arena])]. Returns the arena
        afterwards, fetched through the library (a copy to the host is one of the calls that launch what was put aside)."""
        arena = self.torch.from_numpy(start).to(self.dev)
        self.torch.cuda.synchronize()
        base = arena.data_ptr()
        for name, args in program:
            real = [ctypes.c_void_p(base + 4 * a[1]) if isinstance(a, tuple) else a for a in args]
            self.na.check(getattr(self.lib, name)(stream, *real))
        out = np.empty_like(start)
        self.na.check(self.lib.nhCopyDeviceToHost(stream, out.ctypes.data_as(ctypes.c_void_p), ctypes.c_void_p(base), out.nbytes))
        return out


@pytest.fixture(scope="module")
def streams():
    s = Streams()
    yield s
    s.close()


def same_bits(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32))


def at(offset):
    return ("at", int(offset))


def test_row_normalisation_scalars_chain(streams):
    """The small calls of CObjectNormalizationLayer::runOnceImpl (NeoML/src/Dnn/Layers/ObjectNormalizationLayer.cpp:
    200-230) on one value per row, with the matrix-sized calls between them."""
    g = rng(4001)
    rows, width = 8192, 2
    start = g.uniform(0.5, 2.0, ARENA).astype(np.float32)
    x, sq, mean, inv_std, inv_w, eps = 0, rows * width, 2 * rows * width, 2 * rows * width + rows, ARENA - 8, ARENA - 4
    start[inv_w], start[eps] = 1.0 / width, 1e-5
    program = [
        ("nhSumMatrixColumns", [at(mean), at(x), rows, width]),
        ("nhVectorNegMultiply", [at(mean), at(mean), rows, at(inv_w)]),
        ("nhAddVectorToMatrixColumns", [at(x), at(sq), rows, width, at(mean)]),
        ("nhVectorEltwiseMultiply", [at(sq), at(sq), at(sq), rows * width]),
        ("nhSumMatrixColumns", [at(inv_std), at(sq), rows, width]),
        ("nhVectorMultiply", [at(inv_std), at(inv_std), rows, at(inv_w)]),
        ("nhVectorAddValue", [at(inv_std), at(inv_std), rows, at(eps)]),
        ("nhVectorSqrt", [at(inv_std), at(inv_std), rows]),
        ("nhVectorInv", [at(inv_std), at(inv_std), rows]),
        ("nhAddVectorToMatrixColumns", [at(x), at(sq), rows, width, at(mean)]),
        ("nhMultiplyDiagMatrixByMatrix", [at(inv_std), rows, at(sq), width, at(sq), rows * width]),
    ]
    want = streams.run(streams.plain, program, start)
    got = streams.run(streams.deferring, program, start)
    assert same_bits(got, want)
    # and the numbers are those of the formula
    m = start[x:x + rows * width].reshape(rows, width).astype(np.float64)
    ref = (m - m.mean(1, keepdims=True)) / np.sqrt(m.var(1, keepdims=True) + 1e-5)
    # ( two values per row: where they nearly agree the variance is a difference of close numbers, hence the loose bar;
    # the bar of this test is the line above )
    assert np.allclose(got[sq:sq + rows * width].reshape(rows, width), ref, rtol=1e-3, atol=5e-3)


UNARY = ("nhVectorSqrt", "nhVectorInv", "nhVectorNeg", "nhVectorAbs")
BINARY = ("nhVectorAdd", "nhVectorSub", "nhVectorEltwiseMultiply", "nhVectorEltwiseDivide", "nhVectorEltwiseMax", "nhVectorEltwiseMin",
          "nhVectorEltwiseMultiplyAdd", "nhVectorEltwiseNegMultiply")
WITH_SCALAR = ("nhVectorAddValue", "nhVectorMultiply", "nhVectorNegMultiply", "nhVectorReLU")
BINARY_WITH_SCALAR = ("nhVectorMultiplyAndAdd", "nhVectorMultiplyAndSub")
# activations that are put aside too, and two that are not: those are launched at once, after what was put aside
OTHER = ("nhVectorSigmoid", "nhVectorTanh", "nhVectorHSwish", "nhVectorExp", "nhVectorSquaredHinge")


def random_program(g, length):
    """Operands begin at a few fixed places of the arena, so that exact matches, shifted overlaps and disjoint operands
    all come up; a result either begins where one of the call's own operands begins or keeps clear of them (what the
    entry points ask for); scalars sit in the arena too, sometimes where a call in front writes."""
    places = [0, 0, 0, 1, 3, 4, 64, 4096, 8192, 8195, 12288, 20000, 20000, 36000, 100000, 100000, 210000]
    # ( above 16384 elements a call joins a chain only while no call in it has to wait for another; above 262144 only
    # a chain of calls of its own count )
    sizes = [1, 5, 64, 777, 1024, 4096, 8192, 8192, 16384, 16384, 20000, 70000, 200000, 300000, 300000, 300000, 280000]
    program = []
    while len(program) < length:
        n = int(g.choice(sizes))
        kind = g.integers(0, 10)
        if kind < 1:
            out = int(g.choice(places))
            program.append(("nhVectorFill", [at(out), float(g.integers(-3, 4)) * 0.5, n]))
            continue
        if kind < 3:
            name, n_in, scalar = str(g.choice(UNARY)), 1, False
        elif kind < 6:
            name, n_in, scalar = str(g.choice(BINARY)), 2, False
        elif kind < 8:
            name, n_in, scalar = str(g.choice(WITH_SCALAR)), 1, True
        elif kind < 9:
            name, n_in, scalar = str(g.choice(BINARY_WITH_SCALAR)), 2, True
        else:
            name, n_in, scalar = str(g.choice(OTHER)), 1, False
        ins = [int(g.choice(places)) for _ in range(n_in)]
        if name == "nhVectorEltwiseMultiplyAdd":
            # result += first * second: the result is the third operand
            out = int(g.choice(places))
            if any(i != out and i < out + n and out < i + n for i in ins):
                continue
        elif g.integers(0, 2) == 0:
            out = ins[int(g.integers(0, n_in))]
            if any(i != out and i < out + n and out < i + n for i in ins):
                continue
        else:
            out = int(g.choice(places))
            if any(i != out and i < out + n and out < i + n for i in ins):
                continue
        args = [at(i) for i in ins]
        if scalar:
            where = int(g.choice([ARENA - 4, ARENA - 3, 2, 4100, 8192]))
            if out <= where < out + n:
                continue  # a call may not overwrite its own scalar
            args += [at(out), n, at(where)]
        else:
            args += [at(out), n]
        program.append((name, args))
    return program


@pytest.mark.parametrize("seed", range(12))
def test_random_chains_leave_the_same_bits(streams, seed):
    g = rng(4100 + seed)
    start = g.uniform(0.25, 4.0, ARENA).astype(np.float32) * g.choice([-1.0, 1.0], ARENA).astype(np.float32)
    start[ARENA - 4:] = (1.5, -0.75, 0.0, 0.0)
    program = random_program(g, 40)
    want = streams.run(streams.plain, program, start)
    got = streams.run(streams.deferring, program, start)
    assert same_bits(got, want), [p[0] for p in program]


def test_every_way_out_of_the_queue(streams):
    """What was put aside is launched by: a ninth small call, an event, a synchronisation, switching the mode off, and
    the release of device memory."""
    import torch
    lib, na = streams.lib, streams.na
    s = streams.deferring
    x = torch.full((4096,), 2.0, device=streams.dev)
    two = torch.full((1,), 2.0, device=streams.dev)
    torch.cuda.synchronize()
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def double(times):
        for _ in range(times):
            na.check(lib.nhVectorMultiply(s, P(x), P(x), 4096, P(two)))

    double(11)  # more than one chain holds
    na.check(lib.nhStreamSynchronize(s))
    assert float(x[0]) == 2.0 * 2 ** 11 and float(x[4095]) == 2.0 * 2 ** 11
    double(2)
    event = ctypes.c_void_p()
    na.check(lib.nhEventCreate(ctypes.byref(event)))
    na.check(lib.nhEventRecord(event, s))
    na.check(lib.nhEventSynchronize(event))
    assert float(x[7]) == 2.0 * 2 ** 13
    na.check(lib.nhEventDestroy(event))
    double(1)
    na.check(lib.nhStreamDeferSmallOps(s, 0))
    torch.cuda.synchronize()
    assert float(x[9]) == 2.0 * 2 ** 14
    na.check(lib.nhStreamDeferSmallOps(s, 1))
    block = ctypes.c_void_p()
    na.check(lib.nhRawAlloc(ctypes.byref(block), 4096 * 4))
    na.check(lib.nhVectorCopy(s, block, P(x), 4096))
    na.check(lib.nhVectorMultiply(s, block, P(x), 4096, P(two)))
    na.check(lib.nhRawFree(block))  # the two calls above name the block: they run before it goes
    na.check(lib.nhStreamSynchronize(s))
    assert float(x[11]) == 2.0 * 2 ** 15


def test_small_call_between_two_lstms_keeps_its_place(streams):
    """On a stream that also lets independent one-launch LSTMs run side by side: a small call between two nhLstm calls
    that produces the second one's input is launched before it, and the second does not run beside the first."""
    import torch
    from nhtest import Cpu, assert_close
    orc = Cpu("orc")
    lib, na = streams.lib, streams.na
    s = streams.deferring
    g = rng(4200)
    T, B, In, H = 16, 16, 64, 256   # the second call's input: T * B * In = 16384 floats, a small call
    w_in = g.uniform(-0.2, 0.2, (2, 4 * H, In)).astype(np.float32)
    w_rec = g.uniform(-0.1, 0.1, (2, 4 * H, H)).astype(np.float32)
    bias = g.uniform(-0.5, 0.5, (2, 4 * H)).astype(np.float32)
    x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(streams.dev)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    d_w_in, d_w_rec, d_bias, d_x = up(w_in), up(w_rec), up(bias), up(x)
    size = ctypes.c_size_t(0)
    na.check(lib.nhLstmWorkspaceSize(H, In, T, B, ctypes.byref(size)))
    work = [torch.empty((size.value + 15) // 4, dtype=torch.float32, device=streams.dev) for _ in range(2)]
    out = [torch.zeros((T, B, H), device=streams.dev) for _ in range(2)]
    x2 = torch.zeros((T, B, In), device=streams.dev)
    half = up(np.array([0.5], np.float32))
    torch.cuda.synchronize()
    na.check(lib.nhStreamOverlapLstm(s, 1))
    try:
        for _ in range(2):
            na.check(lib.nhLstm(s, H, In, P(d_w_in[0]), P(d_bias[0]), P(d_w_rec[0]), None, 0, T, B, None, None, P(d_x), None, P(out[0]),
                                P(work[0]), size.value))
            na.check(lib.nhVectorMultiply(s, P(d_x), P(x2), x.size, P(half)))
            na.check(lib.nhLstm(s, H, In, P(d_w_in[1]), P(d_bias[1]), P(d_w_rec[1]), None, 1, T, B, None, None, P(x2), None, P(out[1]),
                                P(work[1]), size.value))
            assert lib.nhStreamSynchronize(s) == 0
            assert_close(out[0].cpu().numpy(), orc.lstm(w_in[0], bias[0], w_rec[0], None, x, False)[0], "first")
            assert_close(out[1].cpu().numpy(), orc.lstm(w_in[1], bias[1], w_rec[1], None, 0.5 * x, True)[0], "second, input from the small call")
            x2.zero_()
            torch.cuda.synchronize()
    finally:
        na.check(lib.nhStreamOverlapLstm(s, 0))


def test_nothing_is_put_aside_while_the_stream_is_captured():
    """A graph recorded from a stream that puts small calls aside holds every call: the recording ends outside the library,
    so a call left in the queue would be missing from the graph (and run once, later, outside it)."""
    import torch
    import neoml_amd
    lib = neoml_amd.load()
    dev = torch.device("cuda:0")
    x = torch.full((4096,), 1.0, device=dev)
    two = torch.full((1,), 2.0, device=dev)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    s = torch.cuda.Stream()
    ps = ctypes.c_void_p(s.cuda_stream)
    torch.cuda.synchronize()
    neoml_amd.check(lib.nhStreamDeferSmallOps(ps, 1))
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=s):
            for _ in range(3):
                neoml_amd.check(lib.nhVectorMultiply(ps, P(x), P(x), 4096, P(two)))
        torch.cuda.synchronize()
        assert float(x[0]) == 1.0 and float(x[4095]) == 1.0  # recorded, not run
        for replay in range(1, 4):
            graph.replay()
            torch.cuda.synchronize()
            assert float(x[0]) == 8.0 ** replay and float(x[4095]) == 8.0 ** replay
    finally:
        neoml_amd.check(lib.nhStreamDeferSmallOps(ps, 0))


def test_product_waits_for_its_free_term(streams):
    """On such a stream a product A * B^T is put aside as well, and an AddVectorToMatrixRows over its result in place goes
    into the same launch (the two calls of CFullyConnectedLayer::RunOnce, NeoML/src/Dnn/Layers/FullyConnectedLayer.cpp:
    91-99). Whatever else comes behind the product finds it done."""
    import torch
    from nhtest import assert_close
    lib, na = streams.lib, streams.na
    g = rng(4300)
    dev = streams.dev
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    for m, n, k in ((8192, 512, 512), (300, 101, 64), (64, 1000, 512), (1000, 24, 8), (5, 7, 3)):
        a = g.uniform(-1, 1, (m, k)).astype(np.float32)
        w = (g.uniform(-1, 1, (n, k)) / np.sqrt(k)).astype(np.float32)
        bias = g.uniform(-1, 1, n).astype(np.float32)
        want = (a.astype(np.float64) @ w.astype(np.float64).T + bias).astype(np.float32)
        d_a, d_w, d_bias = up(a), up(w), up(bias)
        outs = {}
        for name, stream in (("plain", streams.plain), ("deferring", streams.deferring)):
            c = torch.zeros((m, n), device=dev)
            torch.cuda.synchronize()
            na.check(lib.nhMultiplyMatrixByTransposedMatrix(stream, P(d_a), m, k, k, P(d_w), n, k, P(c), n, m * n))
            na.check(lib.nhAddVectorToMatrixRows(stream, 1, P(c), P(c), m, n, P(d_bias)))
            na.check(lib.nhStreamSynchronize(stream))
            outs[name] = c.cpu().numpy()
        assert_close(outs["deferring"], want, "product + free term in one launch %s" % ((m, n, k),), atol=2e-5)
        assert_close(outs["deferring"], outs["plain"], "one launch vs two %s" % ((m, n, k),), atol=2e-5)
    # other successors: the product is launched as it was asked for, before them
    m, n, k = 512, 256, 128
    a = g.uniform(-1, 1, (m, k)).astype(np.float32)
    w = g.uniform(-1, 1, (n, k)).astype(np.float32)
    bias = g.uniform(-1, 1, n).astype(np.float32)
    d_a, d_w, d_bias, zero = up(a), up(w), up(bias), up(np.zeros(1, np.float32))

    def run(stream, successor):
        c = torch.zeros((m, n), device=dev)
        other = torch.zeros((m, n), device=dev)
        torch.cuda.synchronize()
        na.check(lib.nhMultiplyMatrixByTransposedMatrix(stream, P(d_a), m, k, k, P(d_w), n, k, P(c), n, m * n))
        successor(stream, c, other)
        na.check(lib.nhStreamSynchronize(stream))
        return c.cpu().numpy(), other.cpu().numpy()

    successors = {
        "nothing but the wait": lambda s, c, o: None,
        "free term into another matrix": lambda s, c, o: na.check(lib.nhAddVectorToMatrixRows(s, 1, P(c), P(o), m, n, P(d_bias))),
        "free term of half the rows": lambda s, c, o: na.check(lib.nhAddVectorToMatrixRows(s, 1, P(c), P(c), m // 2, n, P(d_bias))),
        "a large call on the result": lambda s, c, o: na.check(lib.nhVectorReLU(s, P(c), P(o), m * n, P(zero))),
        "a small call on the result": lambda s, c, o: na.check(lib.nhVectorAbs(s, P(c), P(o), 4096)),
        "a second product": lambda s, c, o: na.check(lib.nhMultiplyMatrixByTransposedMatrix(s, P(d_a), m, k, k, P(d_w), n, k, P(o), n, m * n)),
    }
    for what, successor in successors.items():
        want_c, want_o = run(streams.plain, successor)
        got_c, got_o = run(streams.deferring, successor)
        assert same_bits(got_c, want_c) and same_bits(got_o, want_o), what
    # memory given back while a product waits: it runs first
    c = torch.zeros((m, n), device=dev)
    block = ctypes.c_void_p()
    na.check(lib.nhRawAlloc(ctypes.byref(block), 1 << 20))
    torch.cuda.synchronize()
    na.check(lib.nhMultiplyMatrixByTransposedMatrix(streams.deferring, P(d_a), m, k, k, P(d_w), n, k, P(c), n, m * n))
    na.check(lib.nhRawFree(block))
    torch.cuda.synchronize()
    assert_close(c.cpu().numpy(), (a.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32), "launched by nhRawFree", atol=2e-5)


def test_convolution_waits_for_its_relu(streams):
    """A convolution (plain or channelwise) is put aside as well, and a VectorReLU over its result in place goes into its
    launch, the threshold read from device memory: the same bits as the two launches, whatever kernel the shape takes
    (tap-step and tiled products, the short-reduction and window kernels, K slices that meet in scratch memory, the
    depthwise strips). Other successors find the convolution done."""
    import torch
    import neoml_amd
    lib, na = streams.lib, streams.na
    g = rng(4400)
    dev = streams.dev
    P = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    six, zero = up(np.array([6.0], np.float32)), up(np.array([0.0], np.float32))
    cases = [
        # n, h, w, cin, cout, f, pad, stride
        (4, 56, 56, 64, 64, 3, 1, 1), (4, 28, 28, 128, 128, 3, 1, 1), (8, 14, 14, 256, 512, 3, 1, 1), (2, 56, 56, 64, 128, 1, 0, 2),
        (4, 64, 64, 3, 64, 7, 3, 2), (8, 56, 56, 24, 144, 1, 0, 1), (2, 9, 11, 5, 6, 3, 1, 1), (16, 32, 96, 1, 64, 3, 1, 1),
    ]
    for n, h, w, cin, cout, f, pad, stride in cases:
        x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
        filt = g.normal(0, 1.0 / np.sqrt(f * f * cin), (cout, f, f, cin)).astype(np.float32)
        bias = g.uniform(-0.5, 0.5, cout).astype(np.float32)
        d = neoml_amd.ConvDesc(n, h, w, cin, cout, f, f, pad, pad, stride, stride, 1, 1, 0, 0)
        na.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
        d_x, d_f, d_b = up(x), up(filt), up(bias)
        shape = (n, d.resultHeight, d.resultWidth, cout)
        for threshold in (zero, six):
            outs = []
            for stream in (streams.plain, streams.deferring):
                y = torch.zeros(shape, device=dev)
                torch.cuda.synchronize()
                na.check(lib.nhBlobConvolution(stream, ctypes.byref(d), P(d_x), P(d_f), P(d_b), P(y)))
                na.check(lib.nhVectorReLU(stream, P(y), P(y), y.numel(), P(threshold)))
                na.check(lib.nhStreamSynchronize(stream))
                outs.append(y.cpu().numpy())
            assert same_bits(outs[0], outs[1]), (n, h, w, cin, cout, f, pad, stride, float(threshold[0]))
            assert outs[1].min() >= 0.0 and (float(threshold[0]) == 0.0 or outs[1].max() <= 6.0)
        # VectorHSwish in place is taken along in the same way
        outs = []
        for stream in (streams.plain, streams.deferring):
            y = torch.zeros(shape, device=dev)
            d_x4 = up(x * 4)  # ( values on both sides of -3 and 3 )
            torch.cuda.synchronize()
            na.check(lib.nhBlobConvolution(stream, ctypes.byref(d), P(d_x4), P(d_f), P(d_b), P(y)))
            na.check(lib.nhVectorHSwish(stream, P(y), P(y), y.numel()))
            na.check(lib.nhStreamSynchronize(stream))
            outs.append(y.cpu().numpy())
        assert same_bits(outs[0], outs[1]), ("h-swish", n, h, w, cin, cout, f, pad, stride)
    for n, h, w, c, stride in ((8, 56, 56, 144, 1), (8, 112, 112, 96, 2), (3, 9, 7, 6, 1)):
        x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
        filt = g.normal(0, 1.0 / 3, (3, 3, c)).astype(np.float32)
        bias = g.uniform(-0.5, 0.5, c).astype(np.float32)
        d = neoml_amd.ConvDesc(n, h, w, c, 0, 3, 3, 1, 1, stride, stride, 0, 0, 0, 0)
        na.check(lib.nhInitBlobChannelwiseConvolution(ctypes.byref(d)))
        d_x, d_f, d_b = up(x), up(filt), up(bias)
        outs = []
        for stream in (streams.plain, streams.deferring):
            y = torch.zeros((n, d.resultHeight, d.resultWidth, c), device=dev)
            torch.cuda.synchronize()
            na.check(lib.nhBlobChannelwiseConvolution(stream, ctypes.byref(d), P(d_x), P(d_f), P(d_b), P(y)))
            na.check(lib.nhVectorReLU(stream, P(y), P(y), y.numel(), P(six)))
            na.check(lib.nhStreamSynchronize(stream))
            outs.append(y.cpu().numpy())
        assert same_bits(outs[0], outs[1]), ("channelwise", n, h, w, c, stride)
        outs = []
        for stream in (streams.plain, streams.deferring):
            y = torch.zeros((n, d.resultHeight, d.resultWidth, c), device=dev)
            d_x4 = up(x * 6)
            torch.cuda.synchronize()
            na.check(lib.nhBlobChannelwiseConvolution(stream, ctypes.byref(d), P(d_x4), P(d_f), P(d_b), P(y)))
            na.check(lib.nhVectorHSwish(stream, P(y), P(y), y.numel()))
            na.check(lib.nhStreamSynchronize(stream))
            outs.append(y.cpu().numpy())
        assert same_bits(outs[0], outs[1]), ("channelwise h-swish", n, h, w, c, stride)
    # other successors
    n, h, w, cin, cout = 4, 28, 28, 32, 64
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    filt = g.normal(0, 1.0 / np.sqrt(9 * cin), (cout, 3, 3, cin)).astype(np.float32)
    d = neoml_amd.ConvDesc(n, h, w, cin, cout, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)
    na.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
    d_x, d_f = up(x), up(filt)
    count = n * h * w * cout

    def run(stream, successor):
        y = torch.zeros((n, h, w, cout), device=dev)
        other = torch.zeros((n, h, w, cout), device=dev)
        torch.cuda.synchronize()
        na.check(lib.nhBlobConvolution(stream, ctypes.byref(d), P(d_x), P(d_f), None, P(y)))
        successor(stream, y, other)
        na.check(lib.nhStreamSynchronize(stream))
        return y.cpu().numpy(), other.cpu().numpy()

    successors = {
        "nothing but the wait": lambda s, y, o: None,
        "ReLU into another blob": lambda s, y, o: na.check(lib.nhVectorReLU(s, P(y), P(o), count, P(zero))),
        "ReLU over a part": lambda s, y, o: na.check(lib.nhVectorReLU(s, P(y), P(y), count // 2, P(zero))),
        "another activation in place": lambda s, y, o: na.check(lib.nhVectorAbs(s, P(y), P(y), count)),
        "a small call on the result": lambda s, y, o: na.check(lib.nhVectorNeg(s, P(y), P(o), 1000)),
        "a second convolution": lambda s, y, o: na.check(lib.nhBlobConvolution(s, ctypes.byref(d), P(d_x), P(d_f), None, P(o))),
    }
    for what, successor in successors.items():
        want_y, want_o = run(streams.plain, successor)
        got_y, got_o = run(streams.deferring, successor)
        assert same_bits(got_y, want_y) and same_bits(got_o, want_o), what


def test_large_sum_waits_for_its_relu(streams):
    """VectorAdd over more elements than a chain takes waits for the call behind it too: a VectorReLU over the sum in place
    (CEltwiseSumLayer + CReLULayer at the end of a residual block) is the same pass. Same bits; other successors find
    the sum done."""
    import torch
    lib, na = streams.lib, streams.na
    g = rng(4500)
    dev = streams.dev
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    n = 3 * 1000 * 1000 + 7
    a, b = g.normal(0, 3, n).astype(np.float32), g.normal(0, 3, n).astype(np.float32)
    a[5], b[5] = np.nan, 1.0  # NaN becomes 0, as in VectorReLU
    zero, six = up(np.zeros(1, np.float32)), up(np.array([6.0], np.float32))

    def run(stream, in_place, successor):
        d_a, d_b = up(a), up(b)
        out = d_a if in_place else torch.zeros(n, device=dev)
        other = torch.zeros(n, device=dev)
        torch.cuda.synchronize()
        na.check(lib.nhVectorAdd(stream, P(d_a), P(d_b), P(out), n))
        successor(stream, out, other)
        na.check(lib.nhStreamSynchronize(stream))
        return out.cpu().numpy(), other.cpu().numpy()

    successors = {
        "ReLU in place": lambda s, y, o: na.check(lib.nhVectorReLU(s, P(y), P(y), n, P(zero))),
        "ReLU6 in place": lambda s, y, o: na.check(lib.nhVectorReLU(s, P(y), P(y), n, P(six))),
        "nothing but the wait": lambda s, y, o: None,
        "ReLU into another vector": lambda s, y, o: na.check(lib.nhVectorReLU(s, P(y), P(o), n, P(zero))),
        "ReLU over a part": lambda s, y, o: na.check(lib.nhVectorReLU(s, P(y), P(y), n - 8, P(zero))),
        "a second sum": lambda s, y, o: na.check(lib.nhVectorAdd(s, P(y), P(y), P(o), n)),
        "a small call": lambda s, y, o: na.check(lib.nhVectorNeg(s, P(y), P(o), 100)),
    }
    for in_place in (False, True):
        for what, successor in successors.items():
            want = run(streams.plain, in_place, successor)
            got = run(streams.deferring, in_place, successor)
            assert same_bits(got[0], want[0]) and same_bits(got[1], want[1]), (what, in_place)
    # a copy to the host through the library is the call behind it (what a test of the engine does with a result)
    d_a, d_b, d_out = up(a), up(b), torch.zeros(n, device=dev)
    torch.cuda.synchronize()
    na.check(lib.nhVectorAdd(streams.deferring, P(d_a), P(d_b), P(d_out), n))
    fetched = np.empty(n, np.float32)
    na.check(lib.nhCopyDeviceToHost(streams.deferring, fetched.ctypes.data_as(ctypes.c_void_p), P(d_out), fetched.nbytes))
    assert same_bits(np.delete(fetched, 5), np.delete(a + b, 5)) and np.isnan(fetched[5])
    y, _ = run(streams.deferring, False, successors["ReLU6 in place"])
    assert y[5] == 0.0 and y.min() >= 0.0 and y.max() <= 6.0
    assert np.array_equal(np.delete(y, 5), np.clip(np.delete(a + b, 5), 0.0, 6.0))


def test_large_calls_of_one_count_go_as_one_pass(streams):
    """Calls over more elements than a mixed chain takes wait too, for calls of the same count: the three calls of
    CGELULayer::runFastApproximate (NeoML/src/Dnn/Layers/GELULayer.cpp:145-160), in the layer's own form and with the
    product written over the input, and a solver's passes over one parameter blob
    (CDnnSimpleGradientSolver::TrainLayer, NeoML/src/Dnn/DnnSolver.cpp) leave the bits of the separate launches: on
    16-byte boundaries with a count that is a multiple of four (four elements per thread), and off them."""
    import torch
    lib, na = streams.lib, streams.na
    g = rng(4600)
    dev = streams.dev
    P = lambda t, o=0: ctypes.c_void_p(t.data_ptr() + 4 * o)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    scale, rate, moment, decay = (up(np.array([v], np.float32)) for v in (1.702, -0.01, 0.9, 1e-4))

    def gelu_layer(s, x, y, z, n, o):
        na.check(lib.nhVectorMultiply(s, P(x, o), P(y, o), n, P(scale)))
        na.check(lib.nhVectorSigmoid(s, P(y, o), P(y, o), n))
        na.check(lib.nhVectorEltwiseMultiply(s, P(x, o), P(y, o), P(y, o), n))

    def gelu_over_input(s, x, y, z, n, o):
        na.check(lib.nhVectorMultiply(s, P(x, o), P(y, o), n, P(scale)))
        na.check(lib.nhVectorSigmoid(s, P(y, o), P(y, o), n))
        na.check(lib.nhVectorEltwiseMultiply(s, P(x, o), P(y, o), P(x, o), n))

    def gelu_into_a_third(s, x, y, z, n, o):
        na.check(lib.nhVectorMultiply(s, P(x, o), P(y, o), n, P(scale)))
        na.check(lib.nhVectorSigmoid(s, P(y, o), P(y, o), n))
        na.check(lib.nhVectorEltwiseMultiply(s, P(y, o), P(x, o), P(z, o), n))

    def solver(s, x, y, z, n, o):
        # x: parameters, y: their gradient, z: the moving mean of the steps
        na.check(lib.nhVectorMultiply(s, P(z, o), P(z, o), n, P(moment)))
        na.check(lib.nhVectorMultiplyAndAdd(s, P(y, o), P(x, o), P(y, o), n, P(decay)))
        na.check(lib.nhVectorMultiplyAndAdd(s, P(z, o), P(y, o), P(z, o), n, P(rate)))
        na.check(lib.nhVectorAdd(s, P(x, o), P(z, o), P(x, o), n))

    def momentum_solver(s, x, y, z, n, o):
        # the order of CDnnSimpleGradientSolver::TrainLayer (NeoML/src/Dnn/DnnSolver.cpp:481-507) with L2 regularisation
        na.check(lib.nhVectorMultiply(s, P(z, o), P(z, o), n, P(moment)))
        na.check(lib.nhVectorMultiplyAndAdd(s, P(z, o), P(y, o), P(z, o), n, P(rate)))
        na.check(lib.nhVectorMultiplyAndAdd(s, P(z, o), P(x, o), P(z, o), n, P(decay)))
        na.check(lib.nhVectorAdd(s, P(x, o), P(z, o), P(x, o), n))

    def momentum_solver_plain(s, x, y, z, n, o):
        # ... and without it, twice in a row ( two steps )
        for _ in range(2):
            na.check(lib.nhVectorMultiply(s, P(z, o), P(z, o), n, P(moment)))
            na.check(lib.nhVectorMultiplyAndAdd(s, P(z, o), P(y, o), P(z, o), n, P(rate)))
            na.check(lib.nhVectorAdd(s, P(z, o), P(x, o), P(x, o), n))

    def gradient_blob(s, x, y, z, n, o):
        # how NeoML's layers treat a blob of gradients: cleared, copied into, copied out of, cleared again. Only the last
        # value of z and the copy in y need to reach memory.
        na.check(lib.nhVectorFill(s, P(z, o), ctypes.c_float(0.0), n))
        na.check(lib.nhVectorCopy(s, P(z, o), P(x, o), n))
        na.check(lib.nhVectorCopy(s, P(y, o), P(z, o), n))
        na.check(lib.nhVectorFill(s, P(z, o), ctypes.c_float(0.0), n))

    def overwritten_but_read_from_memory(s, x, y, z, n, o):
        # z is overwritten by the last call, but the call in front of that reads it, and not from a register: it must be there
        na.check(lib.nhVectorCopy(s, P(z, o), P(y, o), n))
        na.check(lib.nhVectorNeg(s, P(x, o), P(x, o), n))
        na.check(lib.nhVectorAbs(s, P(z, o), P(x, o), n))
        na.check(lib.nhVectorFill(s, P(z, o), ctypes.c_float(0.5), n))

    def overwritten_and_read_from_a_register(s, x, y, z, n, o):
        # x is what the first call read: the thread keeps it, and what is written over it since
        na.check(lib.nhVectorAbs(s, P(x, o), P(y, o), n))
        na.check(lib.nhVectorNeg(s, P(y, o), P(x, o), n))
        na.check(lib.nhVectorSqrt(s, P(y, o), P(y, o), n))
        na.check(lib.nhVectorCopy(s, P(z, o), P(x, o), n))
        na.check(lib.nhVectorFill(s, P(x, o), ctypes.c_float(1.0), n))

    def two_counts(s, x, y, z, n, o):
        # a call of another count, and a small one, between calls of one count: each run goes out before the next begins
        na.check(lib.nhVectorMultiply(s, P(x, o), P(y, o), n, P(scale)))
        na.check(lib.nhVectorTanh(s, P(y, o), P(y, o), n - 4))
        na.check(lib.nhVectorNeg(s, P(y, o), P(z, o), 1000))
        na.check(lib.nhVectorHSwish(s, P(x, o), P(x, o), n))
        na.check(lib.nhVectorReLU(s, P(x, o), P(x, o), n, P(moment)))

    def shifted(s, x, y, z, n, o):
        # the second call reads what the first wrote one element further on: it may not join the first
        na.check(lib.nhVectorMultiply(s, P(x, o), P(y, o), n, P(scale)))
        na.check(lib.nhVectorAbs(s, P(y, o + 1), P(z, o), n))

    def alone(s, x, y, z, n, o):
        # one large call and then a call that is no element-wise one: the large one goes out as its own launch
        na.check(lib.nhVectorSigmoid(s, P(x, o), P(y, o), n))
        na.check(lib.nhSumMatrixColumns(s, P(z, o), P(y, o), 1000, 64))

    total = 3 * 1000 * 1000 + 16
    data = [g.normal(0, 2, total).astype(np.float32) for _ in range(3)]
    for what in (gelu_layer, gelu_over_input, gelu_into_a_third, solver, momentum_solver, momentum_solver_plain, gradient_blob,
                 overwritten_but_read_from_memory, overwritten_and_read_from_a_register, two_counts, shifted, alone):
        for n, o in ((3 * 1000 * 1000, 0), (3 * 1000 * 1000, 4), (3 * 1000 * 1000 + 2, 0), (3 * 1000 * 1000, 3), (262148, 8)):
            results = []
            for stream in (streams.plain, streams.deferring):
                x, y, z = (up(d) for d in data)
                torch.cuda.synchronize()
                what(stream, x, y, z, n, o)
                na.check(lib.nhStreamSynchronize(stream))
                results.append([t.cpu().numpy() for t in (x, y, z)])
            for got, want in zip(results[1], results[0]):
                assert same_bits(got, want), (what.__name__, n, o)
    # and the values are the layer's: x * sigmoid( 1.702 x ) within the sigmoid's own bar
    x, y, z = (up(d) for d in data)
    gelu_layer(streams.deferring, x, y, z, 3 * 1000 * 1000, 0)
    na.check(lib.nhStreamSynchronize(streams.deferring))
    v = data[0][:3 * 1000 * 1000].astype(np.float64)
    assert np.allclose(y.cpu().numpy()[:3 * 1000 * 1000], v / (1.0 + np.exp(-1.702 * v)), rtol=2e-6, atol=1e-6)


def test_batch_of_products_waits_for_its_factor(streams):
    """nhBatchMultiplyMatrixByMatrix followed by nhVectorMultiply over the whole result in place (CMatrixMultiplicationLayer
    + CLinearLayer: the scores of an attention layer and their 1/sqrt(d), NeoML/src/Dnn/Layers/MultiheadAttentionLayer.cpp:
    168-183) is one launch where the kernel for batches of small products takes the batch, two launches as ever where it
    does not; the bits are those of the two launches, and every other successor finds the products done."""
    import torch
    lib, na = streams.lib, streams.na
    g = rng(4700)
    dev = streams.dev
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    factor = up(np.array([0.125], np.float32))
    # ( batch, M, K, N ): an attention layer's scores, a ragged batch, one too small for the strip kernel, a long reduction
    for batch, m, k, n in ((256, 256, 64, 256), (70, 200, 36, 132), (3, 64, 16, 64), (16, 128, 320, 64)):
        a = g.normal(0, 1, (batch, m, k)).astype(np.float32)
        b = g.normal(0, 1, (batch, k, n)).astype(np.float32)
        count = batch * m * n

        def run(stream, successor):
            d_a, d_b = up(a), up(b)
            out, other = torch.zeros(count, device=dev), torch.zeros(count, device=dev)
            torch.cuda.synchronize()
            na.check(lib.nhBatchMultiplyMatrixByMatrix(stream, batch, P(d_a), m, k, P(d_b), n, P(out), count))
            successor(stream, out, other)
            na.check(lib.nhStreamSynchronize(stream))
            return out.cpu().numpy(), other.cpu().numpy()

        successors = {
            "the factor in place": lambda s, y, o: na.check(lib.nhVectorMultiply(s, P(y), P(y), count, P(factor))),
            "nothing but the wait": lambda s, y, o: None,
            "the factor into another vector": lambda s, y, o: na.check(lib.nhVectorMultiply(s, P(y), P(o), count, P(factor))),
            "the factor over a part": lambda s, y, o: na.check(lib.nhVectorMultiply(s, P(y), P(y), count - n, P(factor))),
            "a softmax": lambda s, y, o: na.check(lib.nhMatrixSoftmaxByRows(s, P(y), batch * m, n, P(o))),
            "a small call": lambda s, y, o: na.check(lib.nhVectorNeg(s, P(y), P(o), 100)),
            "the factor twice": lambda s, y, o: (na.check(lib.nhVectorMultiply(s, P(y), P(y), count, P(factor))),
                                                 na.check(lib.nhVectorMultiply(s, P(y), P(y), count, P(factor)))),
        }
        for what, successor in successors.items():
            want = run(streams.plain, successor)
            got = run(streams.deferring, successor)
            assert same_bits(got[0], want[0]) and same_bits(got[1], want[1]), (what, batch, m, k, n)
        got, _ = run(streams.deferring, successors["the factor in place"])
        want = np.matmul(a.astype(np.float64), b.astype(np.float64)).reshape(-1) * 0.125
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5 * np.sqrt(k))


def test_passes_over_a_matrix_with_vectors_spread_over_it(streams):
    """The thirteen calls of CObjectNormalizationLayer::runOnceImpl (NeoML/src/Dnn/Layers/ObjectNormalizationLayer.cpp:
    181-242) at the size of a transformer layer: the calls that add a vector to the columns or rows of the matrix, or
    multiply by a diagonal matrix, are element-wise calls with a vector spread over the matrix and join the chain of large
    calls of one count (the layer's last four calls become one pass, the centring and squaring in front of the variance
    another). Same bits as the separate launches: widths that are and are not multiples of four, in place and not,
    off the 16-byte boundaries, and with other calls between them."""
    import torch
    lib, na = streams.lib, streams.na
    g = rng(4800)
    dev = streams.dev
    P = lambda t, o=0: ctypes.c_void_p(t.data_ptr() + 4 * o)
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def layer(s, x, out, sq, neg_mean, inv_std, scale, bias, inv_w, eps, rows, width, o):
        n = rows * width
        na.check(lib.nhSumMatrixColumns(s, P(neg_mean), P(x, o), rows, width))
        na.check(lib.nhVectorNegMultiply(s, P(neg_mean), P(neg_mean), rows, P(inv_w)))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(x, o), P(sq, o), rows, width, P(neg_mean)))
        na.check(lib.nhVectorEltwiseMultiply(s, P(sq, o), P(sq, o), P(sq, o), n))
        na.check(lib.nhSumMatrixColumns(s, P(inv_std), P(sq, o), rows, width))
        na.check(lib.nhVectorMultiply(s, P(inv_std), P(inv_std), rows, P(inv_w)))
        na.check(lib.nhVectorAddValue(s, P(inv_std), P(inv_std), rows, P(eps)))
        na.check(lib.nhVectorSqrt(s, P(inv_std), P(inv_std), rows))
        na.check(lib.nhVectorInv(s, P(inv_std), P(inv_std), rows))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(x, o), P(out, o), rows, width, P(neg_mean)))
        na.check(lib.nhMultiplyDiagMatrixByMatrix(s, P(inv_std), rows, P(out, o), width, P(out, o), n))
        na.check(lib.nhBatchMultiplyMatrixByDiagMatrix(s, 1, P(out, o), rows, width, 0, P(scale), 0, P(out, o), n))
        na.check(lib.nhAddVectorToMatrixRows(s, 1, P(out, o), P(out, o), rows, width, P(bias)))

    def tail_into_two_blobs(s, x, out, sq, neg_mean, inv_std, scale, bias, inv_w, eps, rows, width, o):
        # the layer with a blob of its own for the normalised input ( what it keeps for the backward pass ), and in place
        n = rows * width
        na.check(lib.nhSumMatrixColumns(s, P(neg_mean), P(x, o), rows, width))
        na.check(lib.nhSumMatrixColumns(s, P(inv_std), P(x, o + 1), rows, width - 1))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(x, o), P(sq, o), rows, width, P(neg_mean)))
        na.check(lib.nhMultiplyDiagMatrixByMatrix(s, P(inv_std), rows, P(sq, o), width, P(sq, o), n))
        na.check(lib.nhBatchMultiplyMatrixByDiagMatrix(s, 1, P(sq, o), rows, width, 0, P(scale), 0, P(out, o), n))
        na.check(lib.nhAddVectorToMatrixRows(s, 1, P(out, o), P(out, o), rows, width, P(bias)))
        na.check(lib.nhSumMatrixColumns(s, P(neg_mean), P(out, o), rows, width))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(x, o), P(x, o), rows, width, P(neg_mean)))
        na.check(lib.nhMultiplyDiagMatrixByMatrix(s, P(inv_std), rows, P(x, o), width, P(x, o), n))
        na.check(lib.nhBatchMultiplyMatrixByDiagMatrix(s, 1, P(x, o), rows, width, 0, P(scale), 0, P(x, o), n))
        na.check(lib.nhAddVectorToMatrixRows(s, 1, P(x, o), P(x, o), rows, width, P(bias)))
        na.check(lib.nhSumMatrixColumns(s, P(inv_std), P(x, o), rows, width))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(out, o), P(out, o), rows, width, P(inv_std)))
        na.check(lib.nhVectorEltwiseMultiply(s, P(out, o), P(out, o), P(out, o), n))
        # sums over fewer rows than the squares have, and sums that would land in the vector the squares were centred with:
        # the squares go out by themselves
        na.check(lib.nhSumMatrixColumns(s, P(neg_mean), P(out, o), rows - 1, width))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(x, o), P(sq, o), rows, width, P(inv_std)))
        na.check(lib.nhVectorEltwiseMultiply(s, P(sq, o), P(sq, o), P(sq, o), n))
        na.check(lib.nhSumMatrixColumns(s, P(inv_std), P(sq, o), rows, width))

    def residual_sum_in_front(s, x, out, sq, neg_mean, inv_std, scale, bias, inv_w, eps, rows, width, o):
        # the sum of two matrices that waits on the stream and the sums of its rows are one pass; in place and not, and a
        # reduction over fewer rows than the sum has, which leaves the two apart
        n = rows * width
        na.check(lib.nhVectorAdd(s, P(x, o), P(x, o), P(out, o), n))
        na.check(lib.nhSumMatrixColumns(s, P(neg_mean), P(out, o), rows, width))
        na.check(lib.nhVectorNegMultiply(s, P(neg_mean), P(neg_mean), rows, P(inv_w)))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(out, o), P(sq, o), rows, width, P(neg_mean)))
        na.check(lib.nhVectorAdd(s, P(x, o), P(sq, o), P(x, o), n))
        na.check(lib.nhSumMatrixColumns(s, P(inv_std), P(x, o), rows, width))
        na.check(lib.nhVectorAdd(s, P(out, o), P(sq, o), P(out, o), n))
        na.check(lib.nhSumMatrixColumns(s, P(neg_mean), P(out, o), rows - 1, width))

    def other_orders(s, x, out, sq, neg_mean, inv_std, scale, bias, inv_w, eps, rows, width, o):
        n = rows * width
        na.check(lib.nhSumMatrixColumns(s, P(neg_mean), P(x, o), rows, width))
        # a vector per row and one per column into different results, then a call that reads the spread vector's memory as a
        # matrix ( no hazard: reads only ), then one that writes where a call in front read its vector ( goes out alone )
        na.check(lib.nhAddVectorToMatrixRows(s, 1, P(x, o), P(out, o), rows, width, P(bias)))
        na.check(lib.nhMultiplyDiagMatrixByMatrix(s, P(neg_mean), rows, P(out, o), width, P(sq, o), n))
        na.check(lib.nhVectorAbs(s, P(sq, o), P(sq, o), n))
        na.check(lib.nhBatchMultiplyMatrixByDiagMatrix(s, 1, P(sq, o), rows, width, 0, P(sq, o), 0, P(out, o), n))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(out, o), P(x, o), rows, width, P(out, o)))
        na.check(lib.nhVectorFill(s, P(neg_mean), ctypes.c_float(0.5), rows))
        na.check(lib.nhAddVectorToMatrixColumns(s, P(x, o), P(x, o), rows, width, P(neg_mean)))

    for rows, width, o in ((8192, 512, 0), (1000, 300, 0), (1000, 300, 3), (999, 263, 0), (700, 376, 4)):
        n = rows * width
        x0 = g.normal(0.3, 1.5, n + 8).astype(np.float32)
        scale0, bias0 = g.normal(1, 0.2, width).astype(np.float32), g.normal(0, 0.5, width).astype(np.float32)
        for what in (layer, tail_into_two_blobs, residual_sum_in_front, other_orders):
            results = []
            for stream in (streams.plain, streams.deferring):
                x, scale, bias = up(x0), up(scale0), up(bias0)
                out, sq = torch.zeros(n + 8, device=dev), torch.zeros(n + 8, device=dev)
                neg_mean, inv_std = torch.zeros(rows, device=dev), torch.zeros(rows, device=dev)
                inv_w, eps = up(np.array([1.0 / width], np.float32)), up(np.array([1e-5], np.float32))
                torch.cuda.synchronize()
                what(stream, x, out, sq, neg_mean, inv_std, scale, bias, inv_w, eps, rows, width, o)
                na.check(lib.nhStreamSynchronize(stream))
                results.append([t.cpu().numpy() for t in (x, out, sq, neg_mean, inv_std)])
            for got, want in zip(results[1], results[0]):
                assert same_bits(got, want), (what.__name__, rows, width, o)
            if what is layer:
                v = x0[o:o + n].astype(np.float64).reshape(rows, width)
                ref = (v - v.mean(1, keepdims=True)) / np.sqrt(v.var(1, keepdims=True) + 1e-5) * scale0 + bias0
                assert np.allclose(results[1][1][o:o + n].reshape(rows, width), ref, rtol=1e-4, atol=1e-4)


def test_padded_image_waits_for_its_pooling(streams):
    """nhBlobResizeImage that pads with a constant, followed by nhBlobMaxPooling 3x3 over the padded blob (CImageResizeLayer +
    CMaxPoolingLayer: how a ResNet's first pooling gets its border), is one launch that writes both blobs. Same bits in
    both as the two launches leave, for strides 1 to 3, borders of 0 to 2 pixels of any constant (above and below the
    image's values), image sizes that leave rows and columns behind the last window, NaN in the image; any other successor
    finds the padded blob done."""
    import torch
    lib, na = streams.lib, streams.na
    g = rng(4900)
    dev = streams.dev
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    def blob(n, h, w, c):
        return na.BlobDesc.of(1, n, 1, h, w, 1, c)

    cases = (
        # batch, height, width, channels, (left, right, top, bottom), constant, filter, stride
        (4, 24, 24, 64, (1, 1, 1, 1), 0.0, 3, 2),
        (3, 17, 23, 8, (1, 1, 1, 1), -100.0, 3, 2),
        (2, 16, 21, 12, (2, 0, 0, 2), 7.5, 3, 3),
        (2, 9, 12, 4, (0, 1, 2, 1), 0.25, 3, 1),
        (1, 7, 7, 16, (0, 0, 0, 0), 0.0, 3, 2),
        (2, 12, 12, 8, (1, 1, 1, 1), 0.0, 2, 2),      # not a 3 x 3 window: two launches as ever
        (2, 12, 12, 6, (1, 1, 1, 1), 0.0, 3, 2),      # channels not a multiple of four: two launches as ever
    )
    for n, h, w, c, (dl, dr, dt, db), value, f, stride in cases:
        image = g.normal(0, 2, (n, h, w, c)).astype(np.float32)
        image[0, 0, 0, 0] = np.nan
        image[0, h // 2, w // 2, c - 1] = np.nan
        th, tw = h + dt + db, w + dl + dr
        pool = na.PoolingDesc(n, th, tw, c, f, f, stride, stride, 0, 0)
        na.check(lib.nhInitPooling(ctypes.byref(pool)))
        rh, rw = pool.resultHeight, pool.resultWidth
        src, dst = blob(n, h, w, c), blob(n, th, tw, c)

        def run(stream, successor):
            d_image = up(image)
            padded = torch.full((n * th * tw * c,), -7.0, device=dev)
            pooled = torch.full((n * rh * rw * c,), -7.0, device=dev)
            torch.cuda.synchronize()
            na.check(lib.nhBlobResizeImage(stream, ctypes.byref(src), P(d_image), dl, dr, dt, db, 0, ctypes.c_float(value),
                                           ctypes.byref(dst), P(padded)))
            successor(stream, padded, pooled)
            na.check(lib.nhStreamSynchronize(stream))
            return padded.cpu().numpy(), pooled.cpu().numpy()

        def pooling(s, padded, pooled):
            na.check(lib.nhBlobMaxPooling(s, ctypes.byref(pool), P(padded), None, P(pooled)))

        def pooling_with_indices(s, padded, pooled):
            indices = torch.zeros(n * rh * rw * c, dtype=torch.int32, device=dev)
            na.check(lib.nhBlobMaxPooling(s, ctypes.byref(pool), P(padded), P(indices), P(pooled)))

        def mean_pooling(s, padded, pooled):
            na.check(lib.nhBlobMeanPooling(s, ctypes.byref(pool), P(padded), P(pooled)))

        def nothing(s, padded, pooled):
            pass

        def small_call(s, padded, pooled):
            na.check(lib.nhVectorNeg(s, P(padded), P(pooled), 16))

        for successor in (pooling, pooling_with_indices, mean_pooling, nothing, small_call):
            want = run(streams.plain, successor)
            got = run(streams.deferring, successor)
            assert same_bits(got[0], want[0]) and same_bits(got[1], want[1]), (successor.__name__, n, h, w, c, stride)
        # and the padded blob is the image inside its border
        padded, pooled = run(streams.deferring, pooling)
        padded = padded.reshape(n, th, tw, c)
        assert same_bits(np.ascontiguousarray(padded[:, dt:dt + h, dl:dl + w, :]), image)
        border = np.ones((th, tw), bool)
        border[dt:dt + h, dl:dl + w] = False
        assert np.all(padded[:, border, :] == np.float32(value))


def test_row_sums_wait_for_the_calls_over_them(streams):
    """nhSumMatrixColumns followed by element-wise calls with one operand in place over the sums (the mean and the inverse
    deviation of CObjectNormalizationLayer, NeoML/src/Dnn/Layers/ObjectNormalizationLayer.cpp:190-214) is one launch;
    same bits as the separate launches, also when the call behind the sums is no such call: over a part of them, into
    another vector, with two operands, with its scalar among the sums, or more calls than a chain holds."""
    g = rng(5000)
    rows, width = 3000, 36
    start = g.uniform(0.5, 2.0, ARENA).astype(np.float32)
    x, sums, other, inv_w, eps = 0, 200000, 210000, ARENA - 8, ARENA - 4
    start[inv_w], start[eps] = 1.0 / width, 1e-5
    tails = {
        "mean": [("nhVectorNegMultiply", [at(sums), at(sums), rows, at(inv_w)])],
        "deviation": [("nhVectorMultiply", [at(sums), at(sums), rows, at(inv_w)]), ("nhVectorAddValue", [at(sums), at(sums), rows, at(eps)]),
                      ("nhVectorSqrt", [at(sums), at(sums), rows]), ("nhVectorInv", [at(sums), at(sums), rows])],
        "nothing": [],
        "a part": [("nhVectorSqrt", [at(sums), at(sums), rows - 1])],
        "into another vector": [("nhVectorSqrt", [at(sums), at(other), rows])],
        "two operands": [("nhVectorAdd", [at(sums), at(sums), at(sums), rows])],
        "its scalar among the sums": [("nhVectorMultiply", [at(sums), at(sums), rows, at(sums + 5)])],
        "ten calls": [("nhVectorAbs" if k % 2 else "nhVectorNeg", [at(sums), at(sums), rows]) for k in range(10)],
        "a second sum": [("nhVectorSqrt", [at(sums), at(sums), rows]), ("nhSumMatrixColumns", [at(other), at(x), rows, width]),
                         ("nhVectorInv", [at(other), at(other), rows])],
    }
    for what, tail in tails.items():
        for w in (width, width + 1):
            program = [("nhSumMatrixColumns", [at(sums), at(x), rows, w])] + tail
            want = streams.run(streams.plain, program, start)
            got = streams.run(streams.deferring, program, start)
            assert same_bits(got, want), (what, w)
    got = streams.run(streams.deferring, [("nhSumMatrixColumns", [at(sums), at(x), rows, width])] + tails["mean"], start)
    mean = start[:rows * width].astype(np.float64).reshape(rows, width).mean(1)
    assert np.allclose(got[sums:sums + rows], -mean, rtol=1e-5, atol=1e-6)
