"""NeoML's own layer classes, unchanged, on the HIP engine.

oracle/_ref/libNeoML.so is the reference's layer library compiled from its sources; oracle/dnn_shim.cpp builds small
CDnn networks from its CConvLayer, CChannelwiseConvLayer, CFullyConnectedLayer, CMaxPoolingLayer, CMeanPoolingLayer,
CTransformerEncoderLayer and CLstmLayer on the engine it is handed. The same network (same CRandom seed for the
initialisers, same input) runs on the reference's CCpuMathEngine and on CHipMathEngine; outputs must agree within
|a-b| <= 1e-5 + 1e-4 |b|. These tests need the reference build (they are skipped where it is absent).
"""
import ctypes
import os

import numpy as np
import pytest

import nhtest
from nhtest import assert_close, f32, fp, ip, i32

DNN_SHIM = os.path.join(nhtest.ORACLE_DIR, "_ref", "libdnn_shim.so")
pytestmark = pytest.mark.skipif(not (nhtest.have_reference() and os.path.exists(DNN_SHIM)),
                                reason="reference NeoML build (oracle/_ref) not present")

_lib = None


def lib():
    global _lib
    if _lib is None:
        nhtest.shim()  # loads libNeoMathEngine.so first
        _lib = ctypes.CDLL(DNN_SHIM, mode=ctypes.RTLD_GLOBAL)
        _lib.dnn_last_error.restype = ctypes.c_char_p
    return _lib


def dnn_run(engine, kind, dims, x, param=0, seed=451):
    out = np.empty(1 << 22, np.float32)
    out_dims = np.zeros(7, np.int32)
    x = f32(x)
    assert x.size == int(np.prod(dims))
    rc = lib().dnn_run(engine, kind, seed, param, ip(i32(dims)), fp(x), fp(out), out.size, ip(out_dims))
    if rc != 0:
        raise RuntimeError("dnn_run kind %d: %s" % (kind, lib().dnn_last_error().decode()))
    return out[:int(np.prod(out_dims))].reshape(tuple(out_dims)).copy()


CASES = {
    # kind, input dims [BL, BW, LS, H, W, D, C], param
    "cnn": (0, (1, 3, 1, 16, 20, 1, 8), 0),
    "transformer": (1, (1, 3, 24, 1, 1, 1, 32), 32),
    "lstm": (2, (9, 5, 1, 1, 1, 1, 24), 32),
    "resnet_block": (3, (1, 2, 1, 40, 48, 1, 3), 0),
    "recognizer_tail": (4, (12, 4, 1, 1, 1, 1, 16), 20),
    "resnet18": (5, (1, 2, 1, 64, 64, 1, 3), 100),
}


def make_input(name):
    kind, dims, param = CASES[name]
    g = np.random.default_rng(0xC0FFEE + kind)
    return g.uniform(-1, 1, dims).astype(np.float32)


@pytest.mark.parametrize("name", sorted(CASES))
def test_networks_run_on_the_reference_cpu_engine(name):
    kind, dims, param = CASES[name]
    y = dnn_run(nhtest.cpu_engine(), kind, dims, make_input(name), param)
    assert np.isfinite(y).all() and y.size > 0
    if name in ("cnn", "resnet_block", "resnet18"):
        assert y.shape[1] == dims[1] and y.shape[6] == (100 if name == "resnet18" else 10)
        assert np.allclose(y.reshape(dims[1], -1).sum(axis=1), 1.0, atol=1e-5)
    # the initialisers are seeded: a second build of the same network gives the same numbers
    assert np.array_equal(y, dnn_run(nhtest.cpu_engine(), kind, dims, make_input(name), param))


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_layers_unchanged_on_hip_engine(name):
    kind, dims, param = CASES[name]
    x = make_input(name)
    want = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    got = dnn_run(nhtest.hip_engine(), kind, dims, x, param)
    assert got.shape == want.shape
    assert_close(got, want, "CDnn %s on CHipMathEngine vs CCpuMathEngine" % name)


def dnn_run_ctc(engine, dims, x, classes, seed=451):
    T, B = dims[0], dims[1]
    labels = np.full(B * T, -1, np.int32)
    lengths = np.zeros(B, np.int32)
    rc = lib().dnn_run_ctc(engine, seed, classes, ip(i32(dims)), fp(f32(x)), ip(labels), ip(lengths))
    if rc != 0:
        raise RuntimeError("dnn_run_ctc: %s" % lib().dnn_last_error().decode())
    return [labels[b * T:b * T + lengths[b]].tolist() for b in range(B)]


def test_ctc_decoding_layer_agrees_with_oracle_collapse():
    """CCtcDecodingLayer::GetBestSequence on the CPU engine = arg-max of the FC output + the oracle's greedy collapse."""
    kind, dims, classes = CASES["recognizer_tail"]
    x = make_input("recognizer_tail")
    logits = dnn_run(nhtest.cpu_engine(), kind, dims, x, classes)      # [T, B, 1, 1, 1, 1, classes + 1]
    T, B = dims[0], dims[1]
    best = logits.reshape(T, B, classes + 1).argmax(axis=2).T             # [B][T]
    assert dnn_run_ctc(nhtest.cpu_engine(), dims, x, classes) == nhtest.ctc_greedy_collapse(best, blank=classes)


@pytest.mark.gpu
def test_ctc_decoding_layer_labels_bit_exact_on_hip_engine():
    kind, dims, classes = CASES["recognizer_tail"]
    x = make_input("recognizer_tail")
    assert dnn_run_ctc(nhtest.hip_engine(), dims, x, classes) == dnn_run_ctc(nhtest.cpu_engine(), dims, x, classes)


@pytest.mark.gpu
def test_resnet18_through_cdnn_at_benchmark_size(capsys):
    """The benchmark network at its full size (batch 64, 224x224x3) as a CDnn of the reference's layers on the HIP
    engine: the drop-in path an application takes. Prints the time per CDnn::RunOnce; the result must be a valid
    softmax and must equal what the same network gives at batch 2 for its first two images."""
    dims = (1, 64, 1, 224, 224, 1, 3)
    g = np.random.default_rng(0xC0FFEE + 102)
    x = g.uniform(0, 1, dims).astype(np.float32)
    lib().dnn_set_timed_passes(20)
    lib().dnn_last_pass_ms.restype = ctypes.c_double
    try:
        y = dnn_run(nhtest.hip_engine(), 5, dims, x, 1000).reshape(64, 1000)
        ms = lib().dnn_last_pass_ms()
    finally:
        lib().dnn_set_timed_passes(0)
    with capsys.disabled():
        print("\nResNet-18-style, batch 64, CDnn::RunOnce on CHipMathEngine: %.3f ms per pass = %.0f images/sec" % (ms, 64e3 / ms))
    assert np.allclose(y.sum(axis=1), 1.0, atol=1e-5)
    small = dnn_run(nhtest.hip_engine(), 5, (1, 2, 1, 224, 224, 1, 3), x[:, :2], 1000).reshape(2, 1000)
    assert_close(y[:2], small, "batch 64 vs batch 2")
    want = dnn_run(nhtest.cpu_engine(), 5, (1, 1, 1, 224, 224, 1, 3), x[:, :1], 1000).reshape(1, 1000)
    assert_close(y[:1], want, "first image vs the CPU engine")


# ---------------------------------------------------------------------------------------------------------
# CHipLstmLayer (neoml_amd/engine/HipLstmLayer.h): CLstmLayer whose RunOnce reaches IMathEngine::Lstm on a non-CPU
# engine. Same weights (same CRandom seed), so it must reproduce CLstmLayer on the CPU engine.

class fused_lstm:
    def __init__(self, hidden=32):
        self.hidden = hidden

    def __enter__(self):
        lib().dnn_set_fused_lstm(1)
        lib().dnn_set_tail_hidden(self.hidden)

    def __exit__(self, *exc):
        lib().dnn_set_fused_lstm(0)
        lib().dnn_set_tail_hidden(32)


def test_hip_lstm_layer_is_clstmlayer_on_the_cpu_engine():
    # on the CPU engine the subclass defers to its base class: identical numbers
    for name in ("lstm", "recognizer_tail"):
        kind, dims, param = CASES[name]
        x = make_input(name)
        want = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
        with fused_lstm():
            got = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
        assert np.array_equal(got, want), name


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["lstm", "recognizer_tail"])
def test_hip_lstm_layer_matches_clstmlayer(name):
    kind, dims, param = CASES[name]
    x = make_input(name)
    want = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    with fused_lstm():
        got = dnn_run(nhtest.hip_engine(), kind, dims, x, param)
    assert_close(got, want, "CHipLstmLayer on CHipMathEngine vs CLstmLayer on CCpuMathEngine (%s)" % name)
    if name == "recognizer_tail":
        with fused_lstm():
            labels = dnn_run_ctc(nhtest.hip_engine(), dims, x, param)
        assert labels == dnn_run_ctc(nhtest.cpu_engine(), dims, x, param)


# ---------------------------------------------------------------------------------------------------------
# Threads. "The math engine interface is thread-safe; the same instance may be used in different networks and different
# threads" (the reference's README.md:116-118); its own idiom is one engine and one CDnn per thread
# (NeoML/test/src/InferencePerformanceMultiThreadingTest.cpp:236-262). Both are run here: every thread builds its own
# CDnn, all threads run their passes at once, calling GetPeakMemoryUsage() and CleanUp() between passes, and every
# thread's result must be what the same network gives when it runs alone.

THREAD_CASES = [
    # kind, input dims, param: the small ResNet, the BiLSTM tail of the recogniser at its real width (CHipLstmLayer:
    # the one-launch LSTM, both directions side by side), a transformer encoder layer, the small CNN
    (5, (1, 2, 1, 64, 64, 1, 3), 100),
    (4, (32, 64, 1, 1, 1, 1, 256), 100),
    (1, (1, 3, 24, 1, 1, 1, 32), 32),
    (0, (1, 3, 1, 16, 20, 1, 8), 0),
]


def thread_inputs():
    g = np.random.default_rng(0xC0FFEE + 77)
    return [g.uniform(-1, 1, dims).astype(np.float32) for _, dims, _ in THREAD_CASES]


def dnn_run_threads(engines, inputs, passes=4, seed=451):
    n = len(THREAD_CASES)
    outs = [np.empty(1 << 20, np.float32) for _ in range(n)]
    out_dims = np.zeros(7 * n, np.int32)
    rc = lib().dnn_run_threads(
        n, (ctypes.c_void_p * n)(*[e.value for e in engines]), ip(i32([c[0] for c in THREAD_CASES])),
        ip(i32([c[2] for c in THREAD_CASES])), seed, ip(i32(np.concatenate([c[1] for c in THREAD_CASES]))),
        (ctypes.c_void_p * n)(*[x.ctypes.data for x in inputs]), (ctypes.c_void_p * n)(*[o.ctypes.data for o in outs]),
        ip(i32([o.size for o in outs])), ip(out_dims), passes)
    if rc != 0:
        raise RuntimeError("dnn_run_threads: %s" % lib().dnn_last_error().decode())
    return [o[:int(np.prod(out_dims[7 * t:7 * t + 7]))].copy() for t, o in enumerate(outs)]


def alone(engine, inputs):
    return [dnn_run(engine, kind, dims, x, param).ravel() for (kind, dims, param), x in zip(THREAD_CASES, inputs)]


@pytest.mark.gpu
def test_four_threads_share_one_engine():
    """Four threads, four networks, ONE CHipMathEngine: the same stream, pool and scratch under all of them. The kernels
    on this path are deterministic (K slices meet in a fixed order), so every result must be bit for bit what the
    network gives alone; any give-up of a one-launch LSTM would surface as an exception from the read-back."""
    inputs = thread_inputs()
    engine = nhtest.hip_engine()
    with fused_lstm(256):
        want = alone(engine, inputs)
        for _ in range(2):
            got = dnn_run_threads([engine] * len(THREAD_CASES), inputs)
            for t, (a, b) in enumerate(zip(got, want)):
                assert np.array_equal(a, b), "thread %d differs from the single-threaded run (max |diff| %g)" % (t, np.abs(a - b).max())
        # ... and against the reference engine
        cpu = alone(nhtest.cpu_engine(), inputs)
    for t, (a, b) in enumerate(zip(got, cpu)):
        assert_close(a, b, "thread %d vs the CPU engine" % t)


@pytest.mark.gpu
def test_one_engine_per_thread_on_one_device():
    """The reference's idiom: every thread its own engine (own stream, own pool) on the one GPU. The one-launch LSTMs of
    different engines are ordered behind one another on the device, their give-up words belong to their own streams:
    every thread's read-back, which checks its own stream's word, must come back clean and with the right numbers."""
    inputs = thread_inputs()
    elib = ctypes.CDLL(nhtest.ENGINE_LIB, mode=ctypes.RTLD_GLOBAL)
    first = nhtest.hip_engine()
    elib.CreateHipMathEngine.restype = ctypes.c_void_p
    elib.CreateHipMathEngine.argtypes = [ctypes.c_int, ctypes.c_size_t, ctypes.c_int]
    extra = [ctypes.c_void_p(elib.CreateHipMathEngine(0, 0, 0)) for _ in range(len(THREAD_CASES) - 1)]
    assert all(e.value for e in extra)
    try:
        with fused_lstm(256):
            want = alone(first, inputs)
            for _ in range(2):
                got = dnn_run_threads([first] + extra, inputs)
                for t, (a, b) in enumerate(zip(got, want)):
                    assert np.array_equal(a, b), "thread %d differs from the single-threaded run (max |diff| %g)" % (t, np.abs(a - b).max())
            # two engines, both running the BiLSTM tail at once: their one-launch LSTMs meet on the device
            both = [THREAD_CASES[1]] * 2
            x = inputs[1]
            outs = [np.empty(1 << 20, np.float32) for _ in both]
            out_dims = np.zeros(14, np.int32)
            rc = lib().dnn_run_threads(
                2, (ctypes.c_void_p * 2)(first.value, extra[0].value), ip(i32([c[0] for c in both])), ip(i32([c[2] for c in both])),
                451, ip(i32(np.concatenate([c[1] for c in both]))), (ctypes.c_void_p * 2)(x.ctypes.data, x.ctypes.data),
                (ctypes.c_void_p * 2)(*[o.ctypes.data for o in outs]), ip(i32([o.size for o in outs])), ip(out_dims), 6)
            assert rc == 0, lib().dnn_last_error().decode()
            for o in outs:
                assert np.array_equal(o[:want[1].size], want[1])
    finally:
        for e in extra:
            nhtest.shim().shim_destroy_engine(e)


@pytest.mark.gpu
def test_recognizer_tail_at_benchmark_size_fused_vs_composite(capsys):
    """The BiLSTM tail of the line recogniser at its full size (128 steps, 64 lines, 256 -> 2 x 256 hidden, FC to 101)
    as a CDnn: CLstmLayer (composite per-step graph on this engine) against CHipLstmLayer (IMathEngine::Lstm).
    Same weights, so the outputs must agree; the time per CDnn::RunOnce of both is printed."""
    dims = (128, 64, 1, 1, 1, 1, 256)
    g = np.random.default_rng(0xC0FFEE + 105)
    x = g.uniform(-1, 1, dims).astype(np.float32)
    lib().dnn_last_pass_ms.restype = ctypes.c_double
    lib().dnn_set_timed_passes(5)
    try:
        lib().dnn_set_tail_hidden(256)
        composite = dnn_run(nhtest.hip_engine(), 4, dims, x, 100)
        composite_ms = lib().dnn_last_pass_ms()
        with fused_lstm(256):
            fused = dnn_run(nhtest.hip_engine(), 4, dims, x, 100)
            fused_ms = lib().dnn_last_pass_ms()
    finally:
        lib().dnn_set_timed_passes(0)
        lib().dnn_set_tail_hidden(32)
    with capsys.disabled():
        print("\nBiLSTM(256) tail, 128 steps x 64 lines, CDnn::RunOnce on CHipMathEngine: CLstmLayer %.2f ms, "
              "CHipLstmLayer %.2f ms" % (composite_ms, fused_ms))
    assert_close(fused, composite, "CHipLstmLayer vs CLstmLayer on the same engine")


# ---------------------------------------------------------------------------------------------------------
# The graph optimizer's fused layers: NeoML's OptimizeDnn rewrites the plain layers of a depthwise-separable network
# into CMobileNetV2BlockLayer / CChannelwiseWith1x1Layer / CRowwiseOperationChainLayer, whose RunOnce calls
# IMathEngine::MobileNetV2Block, ChannelwiseWith1x1 and RowwiseExecute.

CASES["separable_net"] = (6, (1, 3, 1, 32, 40, 1, 3), 10)


class optimized:
    def __enter__(self):
        lib().dnn_set_optimize(1)

    def __exit__(self, *exc):
        lib().dnn_set_optimize(0)


def last_optimization():
    counts = [ctypes.c_int(0) for _ in range(3)]
    lib().dnn_last_optimization(*[ctypes.byref(c) for c in counts])
    return tuple(c.value for c in counts)


def test_optimizer_rewrites_the_separable_network_on_the_cpu_engine():
    kind, dims, param = CASES["separable_net"]
    x = make_input("separable_net")
    plain = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    with optimized():
        fused = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    blocks, with1x1, chains = last_optimization()
    assert blocks == 2 and with1x1 >= 1 and chains >= 1  # (the 1x1 pass also counts the pairs inside the two blocks)
    assert_close(fused, plain, "optimized vs plain network on the CPU engine")


@pytest.mark.gpu
def test_optimized_separable_network_on_hip_engine():
    kind, dims, param = CASES["separable_net"]
    x = make_input("separable_net")
    want = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    with optimized():
        got = dnn_run(nhtest.hip_engine(), kind, dims, x, param)
    blocks, with1x1, chains = last_optimization()
    assert blocks == 2 and with1x1 >= 1 and chains >= 1  # (the 1x1 pass also counts the pairs inside the two blocks)
    assert_close(got, want, "optimized network on CHipMathEngine vs plain network on CCpuMathEngine")


@pytest.mark.gpu
def test_optimized_separable_network_on_hip_engine_with_blocks_too_large_for_the_caches():
    """The same network on 16 images of 224 x 224: the expanded tensors of its two CMobileNetV2BlockLayers (16 x 112 x 112 x 96,
    77 MB) are beyond the size at which the engine runs the expand and depthwise stages as one launch (both strides)."""
    kind, _, param = CASES["separable_net"]
    dims = (1, 16, 1, 224, 224, 1, 3)
    x = np.random.default_rng(0xC0FFEE + 61).uniform(-1, 1, dims).astype(np.float32)
    want = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    with optimized():
        got = dnn_run(nhtest.hip_engine(), kind, dims, x, param)
    blocks, with1x1, chains = last_optimization()
    assert blocks == 2
    assert_close(got, want, "optimized network on CHipMathEngine vs plain network on CCpuMathEngine, 16 x 224 x 224")


# the MobileNetV3-style network: squeeze-and-excite branches multiplied back through COnnxEltwiseLayer
SQUEEZE_EXCITE_NET = (7, (1, 3, 1, 32, 40, 1, 3), 10)


def test_optimizer_rewrites_the_squeeze_excite_network_on_the_cpu_engine():
    kind, dims, param = SQUEEZE_EXCITE_NET
    x = np.random.default_rng(0xC0FFEE + kind).uniform(-1, 1, dims).astype(np.float32)
    plain = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    assert np.allclose(plain.reshape(dims[1], -1).sum(axis=1), 1.0, atol=1e-5)
    with optimized():
        fused = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    assert lib().dnn_last_optimization_mobilenetv3_blocks() == 2
    assert_close(fused, plain, "optimized vs plain network on the CPU engine")


@pytest.mark.gpu
def test_plain_squeeze_excite_network_on_hip_engine():
    # COnnxEltwiseLayer's multiplication of [N, H, W, C] by [N, 1, 1, C] goes through BroadcastCopy
    kind, dims, param = SQUEEZE_EXCITE_NET
    x = np.random.default_rng(0xC0FFEE + kind).uniform(-1, 1, dims).astype(np.float32)
    assert_close(dnn_run(nhtest.hip_engine(), kind, dims, x, param), dnn_run(nhtest.cpu_engine(), kind, dims, x, param),
                 "plain squeeze-and-excite network on CHipMathEngine vs CCpuMathEngine")


@pytest.mark.gpu
def test_optimized_squeeze_excite_network_on_hip_engine():
    kind, dims, param = SQUEEZE_EXCITE_NET
    x = np.random.default_rng(0xC0FFEE + kind).uniform(-1, 1, dims).astype(np.float32)
    want = dnn_run(nhtest.cpu_engine(), kind, dims, x, param)
    with optimized():
        got = dnn_run(nhtest.hip_engine(), kind, dims, x, param)
    assert lib().dnn_last_optimization_mobilenetv3_blocks() == 2
    assert_close(got, want, "optimized network on CHipMathEngine vs plain network on CCpuMathEngine")


@pytest.mark.gpu
def test_optimized_resnet18_through_cdnn_at_benchmark_size(capsys):
    """The benchmark network after NeoML's OptimizeDnn: its convolution + ReLU pairs become rowwise operation chains,
    which the engine runs as one launch per pair. Same result as the plain network; time per CDnn::RunOnce printed."""
    dims = (1, 64, 1, 224, 224, 1, 3)
    g = np.random.default_rng(0xC0FFEE + 102)
    x = g.uniform(0, 1, dims).astype(np.float32)
    lib().dnn_last_pass_ms.restype = ctypes.c_double
    lib().dnn_set_timed_passes(20)
    try:
        plain = dnn_run(nhtest.hip_engine(), 5, dims, x, 1000).reshape(64, 1000)
        plain_ms = lib().dnn_last_pass_ms()
        with optimized():
            fused = dnn_run(nhtest.hip_engine(), 5, dims, x, 1000).reshape(64, 1000)
            fused_ms = lib().dnn_last_pass_ms()
    finally:
        lib().dnn_set_timed_passes(0)
    chains = last_optimization()[2]
    with capsys.disabled():
        print("\nResNet-18-style, batch 64, CDnn::RunOnce on CHipMathEngine: plain layers %.3f ms, after OptimizeDnn "
              "(%d rowwise chains) %.3f ms = %.0f images/sec" % (plain_ms, chains, fused_ms, 64e3 / fused_ms))
    assert chains >= 1
    assert_close(fused, plain, "optimized vs plain ResNet-18 on the HIP engine")


# ---------------------------------------------------------------------------------------------------------
# training: CDnn::RunAndLearnOnce (backward and learn passes of the layers, the loss layer, the solvers)

# name: (kind, input dims, solver: 0 SGD with momentum / 1 Adam, learning rate)
TRAIN_CASES = {
    "mlp_sgd": (0, (1, 16, 1, 1, 1, 1, 24), 0, 0.05),
    "mlp_adam": (0, (1, 16, 1, 1, 1, 1, 24), 1, 0.01),
    "cnn_sgd": (1, (1, 6, 1, 12, 12, 1, 3), 0, 0.05),
    "residual_cnn_adam": (2, (1, 4, 1, 10, 10, 1, 3), 1, 0.01),
    "residual_cnn_sgd_wide": (2, (1, 8, 1, 32, 32, 1, 16), 0, 0.02),
    "lstm_adam": (3, (7, 5, 1, 1, 1, 1, 12), 1, 0.01),
    "resnet18_sgd": (4, (1, 2, 1, 64, 64, 1, 3), 0, 0.002),
    "separable_sgd": (5, (1, 3, 1, 24, 24, 1, 3), 0, 0.02),
    "transformer_adam": (6, (1, 2, 8, 1, 1, 1, 32), 1, 0.003),
    "transformer_dropout_adam": (7, (1, 2, 8, 1, 1, 1, 32), 1, 0.003),
    "batchnorm_cnn_sgd": (8, (1, 8, 1, 12, 12, 1, 3), 0, 0.05),
}


def dnn_train(engine, name, classes=5, steps=4, case=None, timed_steps=0):
    kind, dims, solver, rate = case or TRAIN_CASES[name]
    g = np.random.default_rng(0xC0FFEE + 7 * kind + solver)
    x = g.uniform(-1, 1, dims).astype(np.float32)
    n = dims[0] * dims[1] * dims[2]
    labels = np.zeros((n, classes), np.float32)
    labels[np.arange(n), g.integers(0, classes, n)] = 1
    losses = np.zeros(steps, np.float32)
    out = np.zeros(n * classes, np.float32)
    ms = ctypes.c_float(0)
    rc = lib().dnn_train(engine, kind, solver, 11, classes, steps, ctypes.c_float(rate), ip(i32(dims)), fp(x), fp(labels),
                         fp(losses), fp(out), out.size, timed_steps, ctypes.byref(ms))
    if rc != 0:
        raise RuntimeError("dnn_train %s: %s" % (name, lib().dnn_last_error().decode()))
    return (losses, out, ms.value) if timed_steps else (losses, out)


@pytest.mark.parametrize("name", sorted(TRAIN_CASES))
def test_training_reduces_the_loss_on_the_reference_cpu_engine(name):
    losses, out = dnn_train(nhtest.cpu_engine(), name)
    assert np.isfinite(out).all() and losses[-1] < losses[0], losses
    if not name.startswith("transformer"):  # (Adam's first steps overshoot on the transformer)
        assert (np.diff(losses) < 0).all(), losses
    assert abs(losses[0] - np.log(5)) < 1.5  # an untrained 5-class classifier (the deep networks start further off)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(TRAIN_CASES))
def test_training_on_hip_engine_follows_the_cpu_engine(name):
    want_losses, want = dnn_train(nhtest.cpu_engine(), name)
    losses, got = dnn_train(nhtest.hip_engine(), name)
    # four steps of forward, backward, learn and solver: every gradient kernel feeds the weights of the next step
    assert_close(losses, want_losses, "loss per step, %s" % name, atol=2e-5)
    assert_close(got, want, "logits after training, %s" % name, atol=1e-4, rtol=1e-3)


@pytest.mark.gpu
def test_resnet18_training_step_at_benchmark_size(capsys):
    # forward, backward, learn and the SGD update of the ResNet-18-style network, batch 64 of 224 x 224 x 3
    case = (4, (1, 64, 1, 224, 224, 1, 3), 0, 0.002)
    losses, out, ms = dnn_train(nhtest.hip_engine(), "resnet18 batch 64", classes=100, steps=3, case=case, timed_steps=10)
    assert np.isfinite(losses).all() and np.isfinite(out).all()
    assert abs(losses[0] - np.log(100)) < 1.0
    with capsys.disabled():
        print("\nResNet-18-style, batch 64, CDnn::RunAndLearnOnce on CHipMathEngine: %.2f ms per step = %.0f images/sec"
              % (ms, 64 / ms * 1e3))
