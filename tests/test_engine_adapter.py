"""The drop-in boundary: CHipMathEngine (neoml_amd/engine) driven through NeoML's virtual IMathEngine interface by
the same shim calls that drive the reference's CCpuMathEngine, both engines living in one process. Every case
compares the two engines on identical inputs (and with the C oracle)."""
import ctypes

import numpy as np
import pytest

import nhtest
from nhtest import Cpu, assert_close
from test_oracle import (UNARY_CASES, BINARY_CASES, DIFF_CASES, HARD_SIGMOID_BIAS, DROPOUT_CASES, BROADCAST_CASES,
                         MOBILENETV3_CASES, diff_operands, mobilenetv3_operands, unary_input, rng)

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(not nhtest.have_engine_adapter(), reason="engine adapter or oracle/_ref not built")]


def engines():
    return Cpu("hipeng"), Cpu("ref")


def test_engine_identity_and_memory_interface():
    hip, _ = engines()
    s = nhtest.shim()
    assert s.shim_engine_type(nhtest.hip_engine()) == 2  # MET_Cuda: the generic GPU value of TMathEngineType
    peak, cur, pools = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    x = np.ones(1000, np.float32)
    hip.unary("relu", x)  # allocates and frees blobs through HeapAlloc / HeapFree
    assert s.shim_memory_stats(nhtest.hip_engine(), ctypes.byref(peak), ctypes.byref(cur), ctypes.byref(pools)) == 0
    assert peak.value >= 4096 and pools.value > 0 and cur.value >= pools.value  # freed blobs stay cached
    assert s.shim_clean_up(nhtest.hip_engine()) == 0
    assert s.shim_memory_stats(nhtest.hip_engine(), ctypes.byref(peak), ctypes.byref(cur), ctypes.byref(pools)) == 0
    assert pools.value == 0


def test_performance_counters_measure_the_device_work_between_synchronise_calls():
    """IPerformanceCounters as CDnn::EnableProfile uses them (PerformanceCounters.h:27-60): counter 0 is "time ns", its
    value is the time since the previous Synchronise(), and Synchronise() drains the stream first, so device work shows
    up in it: 20 passes over 64 M floats (0.5 GB each way per pass, >= 3 ms of HBM time) must read far longer than 20
    passes over 1 K floats, and longer than the memory system could possibly make them."""
    s = nhtest.shim()
    name = ctypes.create_string_buffer(64)
    count = ctypes.c_int()
    small, large = ctypes.c_ulonglong(), ctypes.c_ulonglong()
    n_large = 64 << 20
    rc = s.shim_performance_counters(nhtest.hip_engine(), 1024, n_large, 20, name, ctypes.byref(count),
                                     ctypes.byref(small), ctypes.byref(large))
    assert rc == 0, s.shim_last_error().decode()
    assert count.value == 1 and name.value == b"time ns"
    assert small.value > 0
    floor_ns = 20 * 8 * n_large / 8e12 * 1e9  # 20 passes at the 8 TB/s peak
    assert large.value > floor_ns, (large.value, floor_ns)
    assert large.value > 5 * small.value, (small.value, large.value)
    assert large.value < 2e9  # and it is a time in nanoseconds, not in another unit


def _create_engine(limit):
    lib = ctypes.CDLL(nhtest.ENGINE_LIB, mode=ctypes.RTLD_GLOBAL)
    lib.CreateHipMathEngine.restype = ctypes.c_void_p
    lib.CreateHipMathEngine.argtypes = [ctypes.c_int, ctypes.c_size_t, ctypes.c_int]
    ptr = lib.CreateHipMathEngine(0, limit, 0)
    assert ptr
    return ctypes.c_void_p(ptr)


def test_memory_limit_covers_the_scratch_of_sliced_convolutions():
    """Everything the engine allocates counts against memoryLimit (MemoryEngineMixin.cpp:99-115), also the block in
    which the K slices of a convolution meet. The last ResNet-18 stage at batch 64 (392 tiles, cut into 5 slices) asks
    for a 30.6 MiB block next to 28 MiB of blobs: without a limit the block shows in the peak and CleanUp gives it
    back; with a limit that holds the blobs but not the block the convolution still gives the right answer (its slices
    then meet through atomic adds) and the peak stays under the limit."""
    nhtest.hip_engine()  # loads the libraries
    s = nhtest.shim()
    g = rng(77)
    x = g.uniform(-1, 1, (64, 7, 7, 512)).astype(np.float32)
    f = g.normal(0, 1.0 / 68.0, (512, 3, 3, 512)).astype(np.float32)
    bias = g.uniform(-0.5, 0.5, 512).astype(np.float32)
    peak, cur, pools = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    stats = lambda e: (s.shim_memory_stats(e, ctypes.byref(peak), ctypes.byref(cur), ctypes.byref(pools)),
                       peak.value, cur.value, pools.value)[1:]
    results = {}
    MiB = 1 << 20
    for limit in (0, 40 * MiB):
        eng = _create_engine(limit)
        try:
            hip = Cpu("hipeng")
            hip.eng = (eng,)
            results[limit] = hip.conv(x, f, bias, 1, 1, 1, 1)
            p, c, _ = stats(eng)
            if limit == 0:
                assert p >= 58 * MiB, p      # blobs (8 + 12 + 8 MiB size classes) and the 32 MiB class of the block
                assert c >= 30 * MiB, c      # the block stays with the stream ...
                assert s.shim_clean_up(eng) == 0
                assert stats(eng)[1] == 0    # ... until CleanUp returns it with the cached blobs
            else:
                assert p <= limit, (p, limit)
        finally:
            s.shim_destroy_engine(eng)
    want = Cpu("orc").conv(x[:4], f, bias, 1, 1, 1, 1)
    assert_close(results[0][:4], want, "sliced convolution, scratch from the pool")
    assert_close(results[40 * MiB], results[0], "sliced convolution under a memory limit vs without")
    # a limit below the blobs themselves is the caller's memory error, as on every engine
    eng = _create_engine(16 * MiB)
    try:
        hip = Cpu("hipeng")
        hip.eng = (eng,)
        with pytest.raises(RuntimeError, match="memory"):
            hip.conv(x, f, bias, 1, 1, 1, 1)
    finally:
        s.shim_destroy_engine(eng)


@pytest.mark.parametrize("op,p0,p1", UNARY_CASES)
def test_unary(op, p0, p1):
    hip, ref = engines()
    x = unary_input(op, 4099, 3)
    assert_close(hip.unary(op, x, p0, p1), ref.unary(op, x, p0, p1), op)


@pytest.mark.parametrize("op", BINARY_CASES)
def test_binary(op):
    hip, ref = engines()
    g = rng(2)
    a = g.uniform(-10, 10, 5003).astype(np.float32)
    b = g.uniform(0.5, 10, 5003).astype(np.float32)
    r = g.uniform(-10, 10, 5003).astype(np.float32)
    assert_close(hip.binary(op, a, b, 0.37, result=r), ref.binary(op, a, b, 0.37, result=r), op)


def test_blas_family():
    hip, ref = engines()
    g = rng(5)
    m = g.uniform(-10, 10, (3, 17, 64)).astype(np.float32)
    v = g.uniform(-10, 10, (3, 64)).astype(np.float32)
    col = g.uniform(-1, 1, 17).astype(np.float32)
    assert_close(hip.add_vector_to_matrix_rows(m, v), ref.add_vector_to_matrix_rows(m, v), "add rows")
    assert_close(hip.add_vector_to_matrix_columns(m[0], col), ref.add_vector_to_matrix_columns(m[0], col), "add cols")
    assert_close(hip.sum_matrix_rows(m), ref.sum_matrix_rows(m), "sum rows", atol=1e-4)
    assert_close(hip.sum_matrix_columns(m[0]), ref.sum_matrix_columns(m[0]), "sum cols", atol=1e-4)
    assert_close(hip.multiply_diag_matrix_by_matrix(col, m[0]), ref.multiply_diag_matrix_by_matrix(col, m[0]), "diag")
    assert_close(hip.batch_multiply_matrix_by_diag_matrix(3, m, 17, 64, 17 * 64, v, 64),
                 ref.batch_multiply_matrix_by_diag_matrix(3, m, 17, 64, 17 * 64, v, 64), "diag right")
    assert_close(hip.softmax_rows(m[0]), ref.softmax_rows(m[0]), "softmax")
    p = g.permutation(64 * 101).reshape(64, 101).astype(np.float32)
    hv, hi = hip.find_max_in_rows(p)
    rv, ri = ref.find_max_in_rows(p)
    assert np.array_equal(hi, ri) and np.array_equal(hv, rv)
    x = g.uniform(-1, 1, (2, 16, 1, 8, 64)).astype(np.float32)
    assert np.array_equal(hip.transpose(x), ref.transpose(x))


def test_matrix_products():
    hip, ref = engines()
    g = rng(9)
    M, N, K = 130, 70, 96
    a = g.uniform(-1, 1, (M, K)).astype(np.float32)
    b = g.uniform(-1, 1, (N, K)).astype(np.float32)
    kw = dict(lda=K, ldb=K, ldc=N, M=M, N=N, K=K)
    assert_close(hip.matmul("nt", a, b, **kw), ref.matmul("nt", a, b, **kw), "nt")
    a3 = g.uniform(-1, 1, (4, 33, 20)).astype(np.float32)
    bn = g.uniform(-1, 1, (4, 20, 24)).astype(np.float32)
    bt = g.uniform(-1, 1, (4, 24, 20)).astype(np.float32)
    at = g.uniform(-1, 1, (4, 20, 33)).astype(np.float32)
    for kind, x, y in (("bnn", a3, bn), ("bnt", a3, bt), ("btn", at, bn)):
        kw = dict(M=33, N=24, K=20, batch=4)
        assert_close(hip.matmul(kind, x, y, **kw), ref.matmul(kind, x, y, **kw), kind)


def test_convolution_pooling_resize_split():
    hip, ref = engines()
    g = rng(10)
    x = g.uniform(-1, 1, (2, 16, 16, 32)).astype(np.float32)
    f = g.normal(0, 0.1, (48, 3, 3, 32)).astype(np.float32)
    bias = g.uniform(-1, 1, 48).astype(np.float32)
    assert_close(hip.conv(x, f, bias, 1, 1, 1, 1), ref.conv(x, f, bias, 1, 1, 1, 1), "conv 3x3")
    assert_close(hip.conv(x, f, None, 1, 1, 2, 2), ref.conv(x, f, None, 1, 1, 2, 2), "conv 3x3/2, no free term")
    xs = g.uniform(0, 1, (2, 20, 20, 3)).astype(np.float32)
    fs = g.normal(0, 0.1, (16, 7, 7, 3)).astype(np.float32)
    assert_close(hip.conv(xs, fs, None, 3, 3, 2, 2), ref.conv(xs, fs, None, 3, 3, 2, 2), "conv 7x7/2")
    fc = g.normal(0, 1, (3, 3, 32)).astype(np.float32)
    cb = g.uniform(-1, 1, 32).astype(np.float32)
    assert_close(hip.channelwise_conv(x, fc, cb, 1, 1, 2, 2), ref.channelwise_conv(x, fc, cb, 1, 1, 2, 2), "channelwise")
    assert np.array_equal(hip.max_pool(x, 3, 3, 2, 2), ref.max_pool(x, 3, 3, 2, 2))
    hy, hidx = hip.max_pool(x, 2, 2, 2, 2, with_indices=True)
    ry, ridx = ref.max_pool(x, 2, 2, 2, 2, with_indices=True)
    assert np.array_equal(hy, ry) and np.array_equal(hidx, ridx)
    assert_close(hip.mean_pool(x, 2, 2, 2, 2), ref.mean_pool(x, 2, 2, 2, 2), "mean pool")
    assert np.array_equal(hip.resize_image(x, 1, 1, 1, 1, 0, 0.0), ref.resize_image(x, 1, 1, 1, 1, 0, 0.0))
    big = g.uniform(-1, 1, (1, 8, 1, 1, 1, 1, 64)).astype(np.float32)
    dims = [(1, 8, 1, 1, 1, 1, 16)] * 4
    for p, q in zip(hip.split(big, 6, dims), ref.split(big, 6, dims)):
        assert np.array_equal(p, q)


@pytest.mark.parametrize("reverse", [False, True])
def test_lstm_through_the_interface(reverse):
    hip, ref = engines()
    g = rng(18)
    T, B, In, H = 6, 8, 32, 64
    w_in = g.uniform(-0.2, 0.2, (4 * H, In)).astype(np.float32)
    w_rec = g.uniform(-0.2, 0.2, (4 * H, H)).astype(np.float32)
    b_in = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
    b_rec = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
    x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
    hh, hc = hip.lstm(w_in, b_in, w_rec, b_rec, x, reverse)
    rh, rc = ref.lstm(w_in, b_in, w_rec, b_rec, x, reverse)
    assert_close(hh, rh, "lstm h")
    assert_close(hc, rc, "lstm c")


def test_unimplemented_method_asserts_like_the_reference_gpu_engine():
    # SingularValueDecomposition is one of the four members left as generated bodies: it raises through NeoML's exception
    # handler, which the shim turns into an error code instead of letting it cross the C boundary
    s = nhtest.shim()
    a = np.array([[3.0, 1.0], [1.0, 2.0]], np.float32)
    sv = np.empty(2, np.float32)
    assert s.shim_singular_value_decomposition(nhtest.hip_engine(), nhtest.fp(a), 2, 2, nhtest.fp(sv)) == 1


def test_vector_top_k_on_both_engines():
    # descending values with their positions; of equal values the one met first comes first
    s = nhtest.shim()
    x = np.array([1.0, 7.0, 3.0, 7.0, -2.0, 5.0, 7.0, 0.5], np.float32)
    got, want = np.empty(5, np.float32), np.empty(5, np.float32)
    got_idx, want_idx = np.empty(5, np.int32), np.empty(5, np.int32)
    ip = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_int))
    assert s.shim_vector_top_k(nhtest.hip_engine(), nhtest.fp(x), 8, 5, nhtest.fp(got), ip(got_idx)) == 0
    assert s.shim_vector_top_k(nhtest.cpu_engine(), nhtest.fp(x), 8, 5, nhtest.fp(want), ip(want_idx)) == 0
    assert list(want_idx) == [1, 3, 6, 5, 2]
    assert np.array_equal(got, want) and np.array_equal(got_idx, want_idx)


def test_vector_power_on_both_engines():
    s = nhtest.shim()
    x = np.linspace(0.5, 3.0, 8).astype(np.float32)
    y = np.empty(8, np.float32)
    z = np.empty(8, np.float32)
    assert s.shim_vector_power(nhtest.hip_engine(), ctypes.c_float(2.5), nhtest.fp(x), nhtest.fp(y), 8) == 0
    assert s.shim_vector_power(nhtest.cpu_engine(), ctypes.c_float(2.5), nhtest.fp(x), nhtest.fp(z), 8) == 0
    assert_close(y, z, "VectorPower")


@pytest.mark.parametrize("with_expand", [True, False])
def test_fused_separable_blocks_through_the_interface(with_expand):
    """InitRowwiseMobileNetV2 / InitRowwiseChWith1x1 + MobileNetV2Block / ChannelwiseWith1x1 on both engines."""
    from test_oracle import SEPARABLE_CASES, separable_operands
    hip, ref = engines()
    for case in SEPARABLE_CASES:
        x, expand, channelwise, down, stride, residual = separable_operands(case, with_expand)
        want = ref.separable_block(x, expand, channelwise, down, stride, residual)
        assert_close(hip.separable_block(x, expand, channelwise, down, stride, residual), want,
                     "separable block %s expand=%s" % (case, with_expand))
        if residual and with_expand:
            assert_close(hip.separable_block(x, expand, channelwise, down, stride, residual, in_place=True), want,
                         "separable block in place %s" % (case,))


# ---- what the backward and learn passes of the layers call, through the interface -----------------------------

@pytest.mark.parametrize("op,p", DIFF_CASES)
def test_activation_derivatives_through_the_interface(op, p):
    hip, ref = engines()
    a, b = diff_operands(op, 4099, 3)
    assert_close(hip.binary(op, a, b, p, p1=HARD_SIGMOID_BIAS), ref.binary(op, a, b, p, p1=HARD_SIGMOID_BIAS), op)


def test_gradients_through_the_interface():
    hip, ref = engines()
    g = rng(501)
    # convolution: stride 2 with an odd size (class-by-class input gradient), free terms on both sides
    n, h, w, cin, cout, fh, fw, ph, pw, sh, sw = 2, 15, 13, 8, 12, 3, 3, 1, 1, 2, 2
    ho, wo = nhtest.conv_out(h, w, fh, fw, ph, pw, sh, sw)
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 0.2, (cout, fh, fw, cin)).astype(np.float32)
    grad = g.uniform(-1, 1, (n, ho, wo, cout)).astype(np.float32)
    bias = g.uniform(-1, 1, cin).astype(np.float32)
    assert_close(hip.conv_backward(grad, f, bias, x.shape, ph, pw, sh, sw), ref.conv_backward(grad, f, bias, x.shape, ph, pw, sh, sw),
                 "BlobConvolutionBackward", atol=2e-5)
    start, ft0 = g.uniform(-1, 1, f.shape).astype(np.float32), g.uniform(-1, 1, cout).astype(np.float32)
    got, want = (e.conv_learn_add(x, grad, start, ph, pw, sh, sw, free_term_diff=ft0) for e in (hip, ref))
    assert_close(got[0], want[0], "BlobConvolutionLearnAdd", atol=1e-4)
    assert_close(got[1], want[1], "free term gradient", atol=1e-4)
    # channelwise convolution
    fc = g.normal(0, 0.5, (3, 3, cin)).astype(np.float32)
    gc = g.uniform(-1, 1, (n, ho, wo, cin)).astype(np.float32)
    assert_close(hip.channelwise_conv_backward(gc, fc, x.shape, 1, 1, 2, 2), ref.channelwise_conv_backward(gc, fc, x.shape, 1, 1, 2, 2),
                 "BlobChannelwiseConvolutionBackward")
    got, want = (e.channelwise_conv_learn_add(x, gc, fc, 1, 1, 2, 2, free_term_diff=bias) for e in (hip, ref))
    assert_close(got[0], want[0], "BlobChannelwiseConvolutionLearnAdd", atol=1e-4)
    assert_close(got[1], want[1], "channelwise free term gradient", atol=1e-4)
    # pooling
    gp = g.uniform(-1, 1, (n, 7, 6, cin)).astype(np.float32)
    assert_close(hip.max_pool_backward(x, gp, 3, 3, 2, 2), ref.max_pool_backward(x, gp, 3, 3, 2, 2), "BlobMaxPoolingBackward")
    assert_close(hip.mean_pool_backward(x.shape, gp, 3, 3, 2, 2), ref.mean_pool_backward(x.shape, gp, 3, 3, 2, 2), "BlobMeanPoolingBackward")
    # softmax derivative, row products, diagonal accumulation
    y = ref.softmax_rows(g.uniform(-3, 3, (33, 101)).astype(np.float32))
    d = g.uniform(-1, 1, y.shape).astype(np.float32)
    assert_close(hip.softmax_diff_rows(y, d), ref.softmax_diff_rows(y, d), "MatrixSoftmaxDiffOpByRows", atol=1e-6)
    assert_close(hip.row_dot(y, d), ref.row_dot(y, d), "RowMultiplyMatrixByMatrix")
    diag, m, acc = g.uniform(-1, 1, (2, 9)).astype(np.float32), g.uniform(-1, 1, (2, 9, 20)).astype(np.float32), g.uniform(-1, 1, (9, 20)).astype(np.float32)
    assert_close(hip.diag_by_matrix_add(diag, m, acc), ref.diag_by_matrix_add(diag, m, acc), "MultiplyDiagMatrixByMatrixAndAdd")


@pytest.mark.parametrize("dims,rate,spatial,batchwise", DROPOUT_CASES[:5])
def test_dropout_through_the_interface(dims, rate, spatial, batchwise):
    hip, ref = engines()
    x = rng(502).uniform(0.5, 1.5, dims).astype(np.float32)
    got, want = hip.dropout(x, rate, spatial, batchwise, 77), ref.dropout(x, rate, spatial, batchwise, 77)
    assert np.array_equal(got != 0, want != 0)
    assert_close(got, want, "Dropout")


@pytest.mark.parametrize("from_dims,to_dims,width", BROADCAST_CASES)
def test_broadcast_copy_through_the_interface(from_dims, to_dims, width):
    hip, ref = engines()
    x = rng(503).uniform(-1, 1, from_dims + (width,)).astype(np.float32)
    assert np.array_equal(hip.broadcast_copy(x, to_dims, width), ref.broadcast_copy(x, to_dims, width))


@pytest.mark.parametrize("case", MOBILENETV3_CASES[:3])
def test_mobilenetv3_blocks_through_the_interface(case):
    hip, ref = engines()
    n, h, w, cin, e, cout, fsize, stride, residual, ex_act, ch_act, gate_act = case
    x, expand, channelwise, gate, down = mobilenetv3_operands(case)
    pre = ref.mobilenetv3_pre_se(x, expand, channelwise, stride)
    assert_close(hip.mobilenetv3_pre_se(x, expand, channelwise, stride), pre, "MobileNetV3PreSEBlock", atol=2e-5)
    res = x if residual and stride == 1 and cin == cout else None
    assert_close(hip.mobilenetv3_post_se(pre, gate, res, gate_act[0], gate_act[1], down),
                 ref.mobilenetv3_post_se(pre, gate, res, gate_act[0], gate_act[1], down), "MobileNetV3PostSEBlock", atol=2e-5)
