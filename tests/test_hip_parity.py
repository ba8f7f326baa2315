"""Parity of the HIP kernels (through the C ABI of libneoml_hip.so) with the CPU oracle.

Bar: int / index results bit-exact; fp32 within |a - b| <= 1e-5 + 1e-4 * |b| (nhtest.ATOL / nhtest.RTOL).
Where oracle/_ref is present, the reference's own CPU engine is compared as well.
"""
import ctypes

import numpy as np
import pytest

import nhtest
from nhtest import Cpu, assert_close
from test_oracle import (HARD_SIGMOID_BIAS, UNARY_CASES, BINARY_CASES, CONV_CASES, CHANNELWISE_CASES, POOL_CASES, SEPARABLE_CASES,
                         BROADCAST_CASES, DIFF_CASES, DROPOUT_CASES, MOBILENETV3_CASES, diff_operands, mobilenetv3_operands, separable_operands, unary_input, rng)

pytestmark = pytest.mark.gpu

orc = Cpu("orc")
_hip = None


def hip():
    global _hip
    if _hip is None:
        _hip = nhtest.Hip()
    return _hip


def ref_or_none():
    return Cpu("ref") if nhtest.have_reference() else None


# ---------------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("op,p0,p1", UNARY_CASES)
def test_unary(op, p0, p1):
    for n, offset, inplace in ((1, 0, False), (3, 0, False), (1003, 0, False), (4096, 0, True), (70001, 1, False),
                               (1 << 20, 0, False)):
        x = unary_input(op, max(n, 8), n)[:n]
        want = orc.unary(op, x, p0, p1)
        got = hip().unary(op, x, p0, p1, inplace=inplace, offset=offset)
        assert_close(got, want, "%s n=%d offset=%d inplace=%s" % (op, n, offset, inplace))
    r = ref_or_none()
    if r is not None:
        x = unary_input(op, 1003, 5)
        assert_close(hip().unary(op, x, p0, p1), r.unary(op, x, p0, p1), op + " vs reference")


def test_relu_nan_and_threshold():
    x = np.array([np.nan, -1.0, 0.5, 7.0, np.inf, -np.inf, 6.0, 0.0], np.float32)
    assert np.array_equal(hip().unary("relu", x, 0.0), np.array([0, 0, 0.5, 7, np.inf, 0, 6, 0], np.float32))
    assert np.array_equal(hip().unary("relu", x, 6.0), np.array([0, 0, 0.5, 6, 6, 0, 6, 0], np.float32))


@pytest.mark.parametrize("op", BINARY_CASES)
def test_binary(op):
    g = rng(2)
    for n in (1, 5, 1000, 300003):
        a = g.uniform(-10, 10, n).astype(np.float32)
        b = g.uniform(0.5, 10, n).astype(np.float32) * np.where(g.random(n) < 0.5, -1, 1).astype(np.float32)
        r = g.uniform(-10, 10, n).astype(np.float32)
        want = orc.binary(op, a, b, 0.37, result=r)
        assert_close(hip().binary(op, a, b, 0.37, result=r), want, "%s n=%d" % (op, n))
    if op == "add":  # residual connections write into their first operand
        assert_close(hip().binary(op, a, b, inplace_first=True), a + b, "add in place")


@pytest.mark.parametrize("op,p", DIFF_CASES)
def test_activation_derivatives(op, p):
    for n in (1, 5, 1003, 300003):
        a, b = diff_operands(op, n, 70 + n)
        assert_close(hip().binary(op, a, b, p, p1=HARD_SIGMOID_BIAS), orc.binary(op, a, b, p, p1=HARD_SIGMOID_BIAS), "%s n=%d" % (op, n))
    a, b = diff_operands(op, 4099, 3)
    assert_close(hip().binary(op, a, b, p, inplace_first=True, p1=HARD_SIGMOID_BIAS), orc.binary(op, a, b, p, p1=HARD_SIGMOID_BIAS),
                 op + " into its first operand")


def test_row_products_softmax_derivative_and_diag_accumulation():
    g = rng(81)
    for h, w in ((1, 1), (3, 5), (17, 64), (40, 101), (9, 300), (8192, 256), (2048, 1000)):
        a = g.uniform(-1, 1, (h, w)).astype(np.float32)
        b = g.uniform(-1, 1, (h, w)).astype(np.float32)
        assert_close(hip().row_dot(a, b), orc.row_dot(a, b), "row dot %s" % ((h, w),), atol=1e-5 * np.sqrt(w))
        y = orc.softmax_rows(a)
        want = orc.softmax_diff_rows(y, b)
        assert_close(hip().softmax_diff_rows(y, b), want, "softmax derivative %s" % ((h, w),), atol=1e-6)
        assert_close(hip().softmax_diff_rows(y, b, inplace=True), want, "softmax derivative into the gradient", atol=1e-6)
    for batch, n, w in ((1, 1, 1), (1, 7, 5), (3, 6, 33), (2, 40, 64), (1, 8192, 512)):
        diag = g.uniform(-1, 1, (batch, n)).astype(np.float32)
        m = g.uniform(-1, 1, (batch, n, w)).astype(np.float32)
        start = g.uniform(-1, 1, (n, w)).astype(np.float32)
        assert_close(hip().diag_by_matrix_add(diag, m, start), orc.diag_by_matrix_add(diag, m, start), "diag accumulate %s" % ((batch, n, w),))


def test_int_ops_fill_convert():
    g = rng(3)
    a = g.integers(-1000, 1000, 100003).astype(np.int32)
    b = g.integers(-1000, 1000, 100003).astype(np.int32)
    for op in ("add", "sub", "multiply"):
        assert np.array_equal(hip().binary_int(op, a, b), orc.binary_int(op, a, b))
    x = g.uniform(-100, 100, 100003).astype(np.float32)
    assert np.array_equal(hip().float_to_int(x), orc.float_to_int(x))
    assert np.array_equal(hip().int_to_float(a), orc.int_to_float(a))
    for n in (1, 7, 4099):
        assert np.array_equal(hip().fill(n, 2.5), np.full(n, 2.5, np.float32))
        assert np.array_equal(hip().fill(n, -3, integer=True), np.full(n, -3, np.int32))
        assert np.array_equal(hip().fill(n, 1.5, from_handle=True), np.full(n, 1.5, np.float32))
        assert np.array_equal(hip().fill(n, 9, from_handle=True, integer=True), np.full(n, 9, np.int32))


def test_sum_and_dot():
    g = rng(4)
    for n in (1, 2, 3, 5, 1000, 1003, 4099, 1 << 20, (1 << 22) + 7):
        a = g.uniform(-1, 1, n).astype(np.float32)
        b = g.uniform(-1, 1, n).astype(np.float32)
        assert_close(hip().vector_sum(a), orc.vector_sum(a), "sum n=%d" % n, atol=1e-2 if n > 1000 else 1e-4)
        assert_close(hip().dot(a, b), orc.dot(a, b), "dot n=%d" % n, atol=1e-2 if n > 1000 else 1e-4)
    # every element counted exactly once, whatever the vector / tail split: sums of small integers are exact in fp32
    for n in (7, 1026, 70001):
        a = g.integers(0, 4, n).astype(np.float32)
        assert hip().vector_sum(a) == a.sum(dtype=np.float64)
        assert hip().dot(a, np.ones_like(a)) == a.sum(dtype=np.float64)


def test_broadcasts_and_sums():
    g = rng(5)
    for b, h, w in ((1, 1, 1), (2, 3, 5), (3, 17, 64), (1, 40, 7), (2, 300, 512), (1, 4096, 12), (64, 49, 512)):
        m = g.uniform(-10, 10, (b, h, w)).astype(np.float32)
        v = g.uniform(-10, 10, (b, w)).astype(np.float32)
        col = g.uniform(-10, 10, h).astype(np.float32)
        tag = str((b, h, w))
        assert_close(hip().add_vector_to_matrix_rows(m, v), orc.add_vector_to_matrix_rows(m, v), "add rows " + tag)
        assert_close(hip().add_vector_to_matrix_rows(m, v, inplace=True), orc.add_vector_to_matrix_rows(m, v), "add rows in place")
        assert_close(hip().set_vector_to_matrix_rows(h, w, v[0]), orc.set_vector_to_matrix_rows(h, w, v[0]), "set rows")
        assert_close(hip().add_vector_to_matrix_columns(m[0], col), orc.add_vector_to_matrix_columns(m[0], col), "add cols")
        assert_close(hip().add_vector_to_matrix_columns(m[0], col, -1), orc.add_vector_to_matrix_columns(m[0], col, -1), "sub cols")
        assert_close(hip().sum_matrix_rows(m), orc.sum_matrix_rows(m), "sum rows " + tag, atol=1e-3)
        assert_close(hip().sum_matrix_rows(m, add_to=v), orc.sum_matrix_rows(m, add_to=v), "sum rows add", atol=1e-3)
        assert_close(hip().sum_matrix_columns(m[0]), orc.sum_matrix_columns(m[0]), "sum cols", atol=1e-3)
        assert_close(hip().multiply_diag_matrix_by_matrix(col, m[0]), orc.multiply_diag_matrix_by_matrix(col, m[0]), "diag")
        assert_close(hip().batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v, w),
                     orc.batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v, w), "diag right")
        assert_close(hip().batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v[0], 0),
                     orc.batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v[0], 0), "diag right broadcast")


@pytest.mark.parametrize("b,h,w", [(1, 2048, 4), (1, 12544, 64), (2, 5000, 12), (1, 3000, 256), (3, 2049, 100), (1, 100352, 128)])
def test_sums_over_the_rows_of_tall_matrices(b, h, w):
    # the free-term gradient of a convolution: one row per pixel of the batch, one column per filter
    g = rng(55 + w)
    m = g.uniform(-1, 1, (b, h, w)).astype(np.float32)
    v = g.uniform(-10, 10, (b, w)).astype(np.float32)
    want = m.astype(np.float64).sum(axis=1)
    tol = 1e-5 * np.sqrt(h)
    assert_close(hip().sum_matrix_rows(m), want, "sum rows %s" % ((b, h, w),), atol=tol)
    assert_close(hip().sum_matrix_rows(m, add_to=v), want + v, "sum rows add", atol=tol)


def test_softmax_logsumexp():
    g = rng(6)
    for h, w in ((1, 1), (3, 2), (7, 64), (9, 101), (513, 256), (64, 1000), (5, 1500), (8192, 101)):
        m = g.uniform(-10, 10, (h, w)).astype(np.float32)
        assert_close(hip().softmax_rows(m), orc.softmax_rows(m), "softmax %s" % ((h, w),))
        assert_close(hip().softmax_rows(m, inplace=True), orc.softmax_rows(m), "softmax in place")
        assert_close(hip().log_sum_exp_rows(m), orc.log_sum_exp_rows(m), "logsumexp")


def test_argmax_bit_exact():
    g = rng(7)
    for h, w in ((1, 1), (5, 3), (64, 101), (9, 257), (8192, 101), (3, 5000)):
        m = g.permutation(h * w).reshape(h, w).astype(np.float32)  # tie-free
        v, i = hip().find_max_in_rows(m)
        ov, oi = orc.find_max_in_rows(m)
        assert np.array_equal(i, oi) and np.array_equal(v, ov)
        v2, _ = hip().find_max_in_rows(m, with_indices=False)
        assert np.array_equal(v2, ov)
    # ties take the first index, as the oracle (and the reference's own test) do
    t = np.zeros((4, 300), np.float32)
    t[1, 200] = t[1, 77] = 1.0
    assert np.array_equal(hip().find_max_in_rows(t)[1], orc.find_max_in_rows(t)[1])
    for b, h, w in ((1, 1, 1), (3, 17, 9), (2, 128, 300)):
        m = g.permutation(b * h * w).reshape(b, h, w).astype(np.float32)
        v, i = hip().find_max_in_columns(m)
        ov, oi = orc.find_max_in_columns(m)
        assert np.array_equal(i, oi) and np.array_equal(v, ov)


def test_ctc_greedy_pipeline_bit_exact():
    # softmax -> log -> arg-max -> collapse, as the decoding layer does (CtcLayer.cpp:205-226,342-369)
    g = rng(20)
    T, B, C = 32, 8, 101
    logits = g.uniform(-5, 5, (B * T, C)).astype(np.float32)
    h = hip()
    p = h.softmax_rows(logits)
    lp = h.unary("log", p)
    _, labels = h.find_max_in_rows(lp.reshape(B * T, C))
    _, want = orc.find_max_in_rows(orc.unary("log", orc.softmax_rows(logits)).reshape(B * T, C))
    assert np.array_equal(labels, want)
    assert nhtest.ctc_greedy_collapse(labels.reshape(B, T), blank=100) == nhtest.ctc_greedy_collapse(want.reshape(B, T), blank=100)


def test_transpose():
    g = rng(8)
    for shape in ((1, 1, 1, 1, 1), (2, 3, 1, 5, 1), (2, 4, 3, 5, 2), (1, 1, 3, 4, 2), (3, 7, 1, 1, 4), (2, 16, 1, 8, 64),
                  (2, 100, 1, 130, 1), (4, 256, 1, 8, 64), (2, 70, 2, 33, 3),
                  # plain matrices whose sides are multiples of 4 ( 128-bit accesses ): partial and whole 64 x 64 tiles
                  (3, 100, 1, 132, 1), (2, 256, 1, 512, 1), (1, 4, 1, 68, 1)):
        x = g.uniform(-1, 1, shape).astype(np.float32)
        assert np.array_equal(hip().transpose(x), orc.transpose(x)), shape
    xi = g.integers(-5, 5, (2, 9, 2, 7, 3)).astype(np.int32)
    assert np.array_equal(hip().transpose(xi, integer=True), np.transpose(xi, (0, 3, 2, 1, 4)))
    xi = g.integers(-5, 5, (2, 72, 1, 60, 1)).astype(np.int32)
    assert np.array_equal(hip().transpose(xi, integer=True), np.transpose(xi, (0, 3, 2, 1, 4)))


# ---------------------------------------------------------------------------------------------------------

MATMUL_SHAPES = [(1, 1, 1), (3, 5, 7), (17, 33, 65), (64, 101, 48), (128, 128, 16), (129, 65, 17), (200, 300, 100),
                 (64, 1000, 512), (256, 64, 576), (70, 31, 250)]


@pytest.mark.parametrize("shape", MATMUL_SHAPES)
def test_matmul_strided(shape):
    M, N, K = shape
    g = rng(9 + M)
    for pad_a, pad_b, pad_c in ((0, 0, 0), (3, 2, 1), (4, 8, 4)):
        a = g.uniform(-1, 1, (M, K + pad_a)).astype(np.float32)
        b = g.uniform(-1, 1, (N, K + pad_b)).astype(np.float32)
        kw = dict(lda=K + pad_a, ldb=K + pad_b, ldc=N + pad_c, M=M, N=N, K=K)
        got, want = hip().matmul("nt", a, b, **kw), orc.matmul("nt", a, b, **kw)
        assert_close(got, want, "nt %s pads %s" % (shape, (pad_a, pad_b, pad_c)))
        at = g.uniform(-1, 1, (K, M + pad_a)).astype(np.float32)
        bn = g.uniform(-1, 1, (K, N + pad_b)).astype(np.float32)
        c0 = g.uniform(-1, 1, ((M - 1) * (N + pad_c) + N,)).astype(np.float32)
        kw = dict(c=c0, lda=M + pad_a, ldb=N + pad_b, ldc=N + pad_c, M=M, N=N, K=K)
        assert_close(hip().matmul("tn_add", at, bn, **kw), orc.matmul("tn_add", at, bn, **kw), "tn_add %s" % (shape,))


# results of a few hundred 128 x 128 tiles with reductions of eight steps and more: the tile of eight wavefronts. Rows
# and columns that end inside a tile, reductions that end inside a step ( multiples of 4: the vector path ), row strides
# with padding, exactly one workgroup per compute unit ( two sets of load registers ) and more
LONG_PRODUCT_SHAPES = [(2000, 1990, 264), (2048, 2048, 128), (3000, 2040, 132), (1990, 2000, 1000), (8192, 512, 520),
                       (1200, 4000, 136), (4096, 1024, 2048)]


@pytest.mark.parametrize("shape", LONG_PRODUCT_SHAPES)
def test_matmul_long_products(shape):
    M, N, K = shape
    g = rng(77 + M + K)
    for pad_a, pad_b, pad_c in ((0, 0, 0), (4, 8, 3)):
        a = g.uniform(-1, 1, (M, K + pad_a)).astype(np.float32)
        b = g.uniform(-1, 1, (N, K + pad_b)).astype(np.float32)
        kw = dict(lda=K + pad_a, ldb=K + pad_b, ldc=N + pad_c, M=M, N=N, K=K)
        got, want = hip().matmul("nt", a, b, **kw), orc.matmul("nt", a, b, **kw)
        # sums of K products of values below one: two summation orders differ by a few ulps of sqrt( K )
        assert_close(got, want, "nt %s pads %s" % (shape, (pad_a, pad_b, pad_c)), atol=1e-5 * max(1.0, np.sqrt(K / 64.0)))
        if pad_c:
            continue
        # every k counted exactly once, every row and column in its place: a one-hot A picks columns of B
        a[:] = 0
        a[np.arange(M), (np.arange(M) * 7) % K] = 1
        got = hip().matmul("nt", a, b, **kw).reshape(M, N)
        assert np.array_equal(got, b[:, (np.arange(M) * 7) % K].T)


def test_matmul_long_product_batched_and_fused():
    # the same tile behind the batched entry point and behind the pointwise convolution with its epilogue
    g = rng(78)
    batch, M, N, K = 3, 1024, 1100, 160
    a = g.uniform(-1, 1, (batch, M, K)).astype(np.float32)
    bt = g.uniform(-1, 1, (batch, N, K)).astype(np.float32)
    kw = dict(M=M, N=N, K=K, batch=batch)
    assert_close(hip().matmul("bnt", a, bt, **kw), orc.matmul("bnt", a, bt, **kw), "bnt long")
    # free term, residual and no activation in the epilogue: the down convolution of a gated block, 12 544 pixels 128 -> 256
    n, h, w, c, cout = 4, 56, 56, 128, 256
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    gate = g.uniform(0, 1, (n, c)).astype(np.float32)
    res = g.uniform(-1, 1, (n, h, w, cout)).astype(np.float32)
    down = (g.normal(0, 0.1, (cout, c)).astype(np.float32), g.uniform(-1, 1, cout).astype(np.float32))
    assert_close(hip().mobilenetv3_post_se(x, gate, res, "hswish", 0.0, down),
                 orc.mobilenetv3_post_se(x, gate, res, "hswish", 0.0, down), "down convolution with residual, long tile", atol=2e-5)


def test_matmul_k_halves_in_one_workgroup():
    # 448 tiles and 32 K steps: the two halves of K run in the two wave groups of one workgroup. Positive operands: over
    # 1.8 M sums of 512 products the few that cancel to almost nothing would otherwise sit at the edge of the absolute bar
    M, N, K = 1792, 1024, 512
    g = rng(91)
    a = g.uniform(0, 1, (M, K)).astype(np.float32)
    b = g.uniform(0, 1, (N, K)).astype(np.float32)
    kw = dict(lda=K, ldb=K, ldc=N, M=M, N=N, K=K)
    got = hip().matmul("nt", a, b, **kw)
    assert_close(got, orc.matmul("nt", a, b, **kw), "nt, K halves")
    # every k must be counted once: a one-hot column of A picks one column of B
    a[:] = 0
    a[np.arange(M), np.arange(M) % K] = 1
    got = hip().matmul("nt", a, b, **kw).reshape(M, N)
    assert np.array_equal(got, b[:, np.arange(M) % K].T)


@pytest.mark.parametrize("batch,M,N,K", [(1, 2, 3, 4), (3, 16, 8, 5), (4, 33, 17, 9), (8, 64, 64, 16), (6, 100, 64, 100),
                                         (5, 64, 256, 64), (2, 130, 36, 72),
                                         # many small products (the strips of 64 rows that walk over all of their tiles): the two
                                         # products of an attention head, ragged rows, columns and reductions, one and several k chunks
                                         (256, 256, 256, 64), (256, 256, 64, 256), (130, 200, 52, 36), (600, 50, 132, 100),
                                         (512, 64, 68, 256), (300, 70, 4, 4)])
def test_matmul_batched(batch, M, N, K):
    g = rng(30 + M)
    a = g.uniform(-1, 1, (batch, M, K)).astype(np.float32)
    bt = g.uniform(-1, 1, (batch, N, K)).astype(np.float32)
    bn = g.uniform(-1, 1, (batch, K, N)).astype(np.float32)
    at = g.uniform(-1, 1, (batch, K, M)).astype(np.float32)
    for kind, x, y in (("bnt", a, bt), ("bnn", a, bn), ("btn", at, bn)):
        kw = dict(M=M, N=N, K=K, batch=batch)
        assert_close(hip().matmul(kind, x, y, **kw), orc.matmul(kind, x, y, **kw), "%s %s" % (kind, (batch, M, N, K)))


def test_matmul_vs_reference_engine():
    r = ref_or_none()
    if r is None:
        pytest.skip("oracle/_ref is not built")
    g = rng(31)
    M, N, K = 300, 200, 160
    a = g.uniform(-1, 1, (M, K)).astype(np.float32)
    b = g.uniform(-1, 1, (N, K)).astype(np.float32)
    kw = dict(lda=K, ldb=K, ldc=N, M=M, N=N, K=K)
    assert_close(hip().matmul("nt", a, b, **kw), r.matmul("nt", a, b, **kw), "nt vs reference")


# ---------------------------------------------------------------------------------------------------------

GPU_CONV_CASES = CONV_CASES + [
    (2, 16, 16, 64, 64, 3, 3, 1, 1, 1, 1, 1, 1),    # vector path, Cin % 16 == 0
    (2, 14, 14, 32, 48, 3, 3, 1, 1, 2, 2, 1, 1),
    (1, 12, 12, 8, 16, 3, 3, 1, 1, 1, 1, 1, 1),     # Cin % 4 == 0, taps straddle a K step
    (1, 10, 10, 20, 130, 3, 3, 2, 2, 1, 1, 2, 2),   # Cin % 4 == 0, not % 16; N tail; dilation
    (3, 9, 9, 128, 200, 1, 1, 0, 0, 1, 1, 1, 1),    # 1x1
    (2, 14, 14, 128, 256, 1, 1, 0, 0, 2, 2, 1, 1),  # 1x1 stride 2 shortcut
    (2, 32, 32, 3, 64, 7, 7, 3, 3, 2, 2, 1, 1),     # stem
    (2, 8, 32, 1, 64, 3, 3, 1, 1, 1, 1, 1, 1),      # single input channel
    # channel counts that are not a multiple of 4: filter rows fetched as contiguous runs
    (2, 9, 13, 6, 10, 3, 5, 1, 2, 1, 2, 2, 1),      # height dilation, width stride
    (1, 7, 7, 2, 5, 3, 3, 1, 1, 1, 1, 1, 1),
    (3, 24, 40, 3, 32, 3, 3, 1, 1, 2, 2, 1, 1),     # RGB 3x3/2 stem
    (1, 6, 5, 7, 9, 2, 4, 0, 3, 1, 1, 1, 1),        # run longer than the image row is wide
    (2, 11, 9, 5, 70, 1, 3, 0, 1, 1, 1, 1, 1),      # N tail
    (4, 32, 64, 1, 64, 3, 3, 1, 1, 1, 1, 1, 1),     # grey line image, split over many tiles
    # pointwise convolutions over many pixels with a short reduction: the row-resident kernel
    (4, 64, 64, 24, 144, 1, 1, 0, 0, 1, 1, 1, 1),   # expand
    (4, 64, 64, 144, 24, 1, 1, 0, 0, 1, 1, 1, 1),   # project, N < 32
    (2, 96, 96, 16, 96, 1, 1, 0, 0, 1, 1, 1, 1),
    (1, 131, 127, 32, 20, 1, 1, 0, 0, 1, 1, 1, 1),  # pixel count not a multiple of 32
    (1, 128, 130, 192, 40, 1, 1, 0, 0, 1, 1, 1, 1), # longest reduction it takes, N tail
    (7, 64, 64, 64, 64, 3, 3, 1, 1, 1, 1, 1, 1),    # 448 tiles, 36 K steps: the two halves of K share a workgroup
    # channel counts that are a multiple of the K step: the filter tap is kept in scalar registers
    (2, 13, 11, 48, 40, 3, 5, 2, 4, 2, 1, 2, 3),    # dilation, padding wider than the filter's reach, stride along the height
    (1, 7, 7, 32, 64, 5, 5, 2, 2, 1, 1, 1, 1),      # one tile, 50 K steps: K slices that begin in the middle of a tap
    (3, 10, 10, 16, 24, 2, 2, 0, 0, 1, 1, 1, 1),    # a tap per K step
]


@pytest.mark.parametrize("case", GPU_CONV_CASES)
def test_convolution(case):
    n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw = case
    g = rng(10 + h * w + cin)
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 1.0 / np.sqrt(fh * fw * cin), (cout, fh, fw, cin)).astype(np.float32)
    bias = g.uniform(-1, 1, cout).astype(np.float32)
    want = orc.conv(x, f, bias, ph, pw, sh, sw, dh, dw)
    assert_close(hip().conv(x, f, bias, ph, pw, sh, sw, dh, dw), want, "conv %s" % (case,))
    assert_close(hip().conv(x, f, None, ph, pw, sh, sw, dh, dw), orc.conv(x, f, None, ph, pw, sh, sw, dh, dw), "conv, no free term")


@pytest.mark.parametrize("case", [
    (2, 16, 16, 64, 64, 3, 3, 1, 1, 1, 1, 1, 1),     # whole tiles, activation in the epilogue
    (1, 7, 7, 512, 96, 3, 3, 1, 1, 1, 1, 1, 1),      # few tiles, long reduction: K slices, activation as a pass of its own
    (3, 9, 9, 128, 200, 1, 1, 0, 0, 1, 1, 1, 1),     # 1x1 through the matrix-product path
    (2, 32, 32, 3, 64, 7, 7, 3, 3, 2, 2, 1, 1),      # stem
    (4, 64, 64, 24, 144, 1, 1, 0, 0, 1, 1, 1, 1),    # the row-resident pointwise kernel
    (7, 64, 64, 64, 64, 3, 3, 1, 1, 1, 1, 1, 1),     # two K groups in a workgroup: activation in the epilogue again
])
@pytest.mark.parametrize("activation,param", [("relu", 0.0), ("relu", 0.5), ("hswish", 0.0)])
def test_convolution_with_activation(case, activation, param):
    n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw = case
    g = rng(310 + cin + fh)
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 1.0 / np.sqrt(fh * fw * cin), (cout, fh, fw, cin)).astype(np.float32)
    bias = g.uniform(-1, 1, cout).astype(np.float32)
    plain = orc.conv(x, f, bias, ph, pw, sh, sw, dh, dw)
    want = orc.unary(activation, plain, param).reshape(plain.shape)
    got = hip().conv(x, f, bias, ph, pw, sh, sw, dh, dw, activation=activation, param=param)
    assert_close(got, want, "conv + %s %s" % (activation, case))


# the training-step shapes on top of the forward cases: whole tiles, strides that leave holes in the input gradient,
# a stem with few input channels, 1x1 shortcuts
GPU_CONV_GRADIENT_CASES = CONV_CASES + [
    (2, 16, 16, 64, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    (2, 14, 14, 32, 48, 3, 3, 1, 1, 2, 2, 1, 1),
    (2, 15, 15, 32, 48, 3, 3, 1, 1, 2, 2, 1, 1),    # stride 2 over an odd size: the last input row has no window of its own
    (1, 10, 10, 20, 130, 3, 3, 2, 2, 1, 1, 2, 2),
    (3, 9, 9, 128, 200, 1, 1, 0, 0, 1, 1, 1, 1),
    (2, 14, 14, 128, 256, 1, 1, 0, 0, 2, 2, 1, 1),
    (2, 32, 32, 3, 64, 7, 7, 3, 3, 2, 2, 1, 1),
    (2, 8, 32, 1, 64, 3, 3, 1, 1, 1, 1, 1, 1),
    (2, 9, 13, 6, 10, 3, 5, 1, 2, 1, 2, 2, 1),
    (1, 6, 5, 7, 9, 2, 4, 0, 3, 1, 1, 1, 1),
    (2, 12, 12, 8, 16, 3, 3, 0, 0, 3, 3, 1, 1),     # stride as large as the filter
    (8, 32, 32, 64, 64, 3, 3, 1, 1, 1, 1, 1, 1),    # many pixels: the filter gradient's reduction is split over the grid
    # strided: the input gradient runs class by class of ( pixel + padding ) mod stride
    (1, 11, 10, 8, 12, 3, 3, 0, 0, 2, 2, 3, 3),     # dilation 3 against stride 2
    (2, 12, 12, 8, 16, 2, 2, 0, 0, 2, 2, 1, 1),     # one tap per class
    (2, 13, 9, 4, 8, 3, 3, 1, 1, 2, 1, 1, 1),       # stride along the height only, odd size: classes of 7 and 6 rows
    (2, 9, 14, 4, 8, 3, 4, 1, 2, 1, 2, 1, 1),       # stride along the width only
    (1, 9, 9, 4, 8, 5, 5, 2, 2, 2, 2, 2, 2),        # dilation and stride share a factor: the masked form
    (1, 13, 13, 4, 8, 3, 3, 1, 1, 3, 3, 1, 1),      # stride 3: the masked form
    (1, 3, 3, 4, 8, 3, 3, 0, 0, 2, 2, 1, 1),        # a single window: classes without pixels of their own
    (1, 13, 13, 4, 16, 3, 3, 1, 1, 3, 3, 1, 1),     # the masked form over 16 gradient channels: taps in scalar registers
    (1, 9, 9, 4, 32, 5, 5, 2, 2, 2, 2, 2, 2),
    (8, 14, 14, 256, 512, 3, 3, 1, 1, 2, 2, 1, 1),  # few tiles per class, long reduction: K slices over a preset result
    # the 7x7/2 stem from 3 to 64 channels at sizes that take the window-summing input gradient: tiles of 32 x 32 input
    # pixels that fit exactly, even sizes with partial tiles, odd sizes
    (1, 224, 224, 3, 64, 7, 7, 3, 3, 2, 2, 1, 1),
    (3, 70, 100, 3, 64, 7, 7, 3, 3, 2, 2, 1, 1),
    (6, 63, 65, 3, 64, 7, 7, 3, 3, 2, 2, 1, 1),
]


@pytest.mark.parametrize("case", GPU_CONV_GRADIENT_CASES)
def test_convolution_gradients(case):
    n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw = case
    g = rng(410 + h * w + cin)
    ho, wo = nhtest.conv_out(h, w, fh, fw, ph, pw, sh, sw, dh, dw)
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 1.0 / np.sqrt(fh * fw * cin), (cout, fh, fw, cin)).astype(np.float32)
    grad = g.uniform(-1, 1, (n, ho, wo, cout)).astype(np.float32)
    bias = g.uniform(-1, 1, cin).astype(np.float32)
    want = orc.conv_backward(grad, f, None, x.shape, ph, pw, sh, sw, dh, dw)
    assert_close(hip().conv_backward(grad, f, None, x.shape, ph, pw, sh, sw, dh, dw), want, "backward %s" % (case,), atol=2e-5)
    assert_close(hip().conv_backward(grad, f, bias, x.shape, ph, pw, sh, sw, dh, dw), want + bias, "backward + free term", atol=2e-5)
    start = g.uniform(-1, 1, f.shape).astype(np.float32)
    want = orc.conv_learn_add(x, grad, start, ph, pw, sh, sw, dh, dw)
    # sums over every pixel of the batch: the bar is relative to the size of the terms, as for the dot product
    scale = np.sqrt(n * ho * wo)
    assert_close(hip().conv_learn_add(x, grad, start, ph, pw, sh, sw, dh, dw), want, "learn %s" % (case,), atol=1e-5 * scale)


def _random_conv_case(g):
    """A convolution whose result is not empty: channel counts drawn from the loader's three regimes (not a multiple of
    4, a multiple of 4, a multiple of the K step), any filter, stride, dilation and padding up to beyond the filter."""
    cin = int(g.choice([1, 3, 5, 4, 8, 12, 20, 16, 32, 48, 64]))
    cout = int(g.choice([1, 7, 16, 33, 64, 70]))
    fh, fw = int(g.integers(1, 6)), int(g.integers(1, 6))
    dh, dw = int(g.integers(1, 4)), int(g.integers(1, 4))
    sh, sw = int(g.integers(1, 4)), int(g.integers(1, 4))
    ph, pw = int(g.integers(0, fh * dh + 1)), int(g.integers(0, fw * dw + 1))
    h = int(g.integers(max(1, (fh - 1) * dh + 1 - 2 * ph), 20))
    w = int(g.integers(max(1, (fw - 1) * dw + 1 - 2 * pw), 20))
    n = int(g.integers(1, 5))
    return n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw


@pytest.mark.parametrize("seed", range(8))
def test_convolution_and_gradients_on_random_shapes(seed):
    g = rng(7000 + seed)
    for _ in range(12):
        case = _random_conv_case(g)
        n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw = case
        ho, wo = nhtest.conv_out(h, w, fh, fw, ph, pw, sh, sw, dh, dw)
        x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
        f = g.normal(0, 1.0 / np.sqrt(fh * fw * cin), (cout, fh, fw, cin)).astype(np.float32)
        bias = g.uniform(-1, 1, cout).astype(np.float32)
        grad = g.uniform(-1, 1, (n, ho, wo, cout)).astype(np.float32)
        assert_close(hip().conv(x, f, bias, ph, pw, sh, sw, dh, dw), orc.conv(x, f, bias, ph, pw, sh, sw, dh, dw), "conv %s" % (case,))
        assert_close(hip().conv_backward(grad, f, None, x.shape, ph, pw, sh, sw, dh, dw),
                     orc.conv_backward(grad, f, None, x.shape, ph, pw, sh, sw, dh, dw), "backward %s" % (case,), atol=2e-5)
        start = g.uniform(-1, 1, f.shape).astype(np.float32)
        assert_close(hip().conv_learn_add(x, grad, start, ph, pw, sh, sw, dh, dw),
                     orc.conv_learn_add(x, grad, start, ph, pw, sh, sw, dh, dw), "learn %s" % (case,), atol=1e-5 * np.sqrt(n * ho * wo))


@pytest.mark.parametrize("seed", range(4))
def test_matmul_on_random_shapes(seed):
    # row strides with padding, reductions that are and are not multiples of the K step, long reductions over few
    # tiles ( K slices ), all three operand orders
    g = rng(7100 + seed)
    for _ in range(10):
        M, N = int(g.integers(1, 200)), int(g.integers(1, 200))
        K = int(g.choice([1, 3, 16, 17, 64, 100, 512, 1000, 2048]))
        pa, pb, pc = (int(v) for v in g.integers(0, 5, 3))
        a = g.uniform(-1, 1, (M, K + pa)).astype(np.float32)
        b = g.uniform(-1, 1, (N, K + pb)).astype(np.float32)
        kw = dict(lda=K + pa, ldb=K + pb, ldc=N + pc, M=M, N=N, K=K)
        tol = dict(atol=1e-5 * max(1.0, np.sqrt(K / 64.0)))
        assert_close(hip().matmul("nt", a, b, **kw), orc.matmul("nt", a, b, **kw), "nt %s" % ((M, N, K, pa, pb, pc),), **tol)
        at = g.uniform(-1, 1, (K, M + pa)).astype(np.float32)
        bn = g.uniform(-1, 1, (K, N + pb)).astype(np.float32)
        c0 = g.uniform(-1, 1, ((M - 1) * (N + pc) + N,)).astype(np.float32)
        kw = dict(c=c0, lda=M + pa, ldb=N + pb, ldc=N + pc, M=M, N=N, K=K)
        assert_close(hip().matmul("tn_add", at, bn, **kw), orc.matmul("tn_add", at, bn, **kw), "tn_add %s" % ((M, N, K),), **tol)


def test_convolution_gradients_are_adjoints_at_full_size():
    # the single-layer configuration, batch 32: <conv(x, f), g> == <x, backward(g, f)> == <f, learn(x, g)>
    h = hip()
    g = rng(41)
    x = g.uniform(-1, 1, (32, 32, 32, 64)).astype(np.float32)
    f = g.normal(0, 1.0 / 24, (64, 3, 3, 64)).astype(np.float32)
    grad = g.uniform(-1, 1, (32, 32, 32, 64)).astype(np.float32)
    y = h.conv(x, f, None, 1, 1, 1, 1).astype(np.float64)
    pairing = np.vdot(y, grad)
    size = np.abs(y * grad).sum()
    dx = h.conv_backward(grad, f, None, x.shape, 1, 1, 1, 1)
    assert abs(np.vdot(dx.astype(np.float64), x) - pairing) <= 1e-5 * size
    df = h.conv_learn_add(x, grad, np.zeros_like(f), 1, 1, 1, 1)
    assert abs(np.vdot(df.astype(np.float64), f) - pairing) <= 1e-5 * size


@pytest.mark.parametrize("case", CHANNELWISE_CASES + [(2, 28, 28, 96, 3, 3, 1, 1, 1, 1), (2, 28, 28, 96, 3, 3, 1, 1, 2, 2),
                                                      (1, 15, 13, 6, 3, 3, 1, 1, 2, 2), (1, 9, 30, 32, 5, 5, 2, 2, 1, 1),
                                                      (2, 21, 13, 20, 3, 3, 0, 2, 2, 2), (1, 3, 3, 4, 3, 3, 1, 1, 1, 1),
                                                      (4, 14, 14, 384, 3, 3, 1, 1, 1, 1), (16, 56, 56, 144, 3, 3, 1, 1, 1, 1),
                                                      # stride 1 with padding 0, 2 and mixed: the input gradient runs as a forward pass with the filter turned
                                                      (2, 12, 10, 8, 3, 3, 0, 0, 1, 1), (2, 9, 11, 12, 3, 3, 2, 2, 1, 1), (1, 7, 16, 4, 3, 3, 0, 2, 1, 1),
                                                      # stride 2: strips of 8 columns and of row pairs, with even and odd sizes, padding 0, 1 and 2, rows
                                                      # and columns that no window reaches, several row chunks per image
                                                      (2, 16, 16, 8, 3, 3, 0, 0, 2, 2), (3, 57, 45, 32, 3, 3, 1, 1, 2, 2), (1, 5, 4, 4, 3, 3, 2, 1, 2, 2),
                                                      (2, 18, 35, 12, 3, 3, 1, 0, 2, 2), (16, 112, 112, 96, 3, 3, 1, 1, 2, 2)])
def test_channelwise_convolution_gradients(case):
    n, h, w, c, fh, fw, ph, pw, sh, sw = case
    g = rng(212 + c)
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    f = g.normal(0, 1, (fh, fw, c)).astype(np.float32)
    ho, wo = nhtest.conv_out(h, w, fh, fw, ph, pw, sh, sw)
    grad = g.uniform(-1, 1, (n, ho, wo, c)).astype(np.float32)
    assert_close(hip().channelwise_conv_backward(grad, f, x.shape, ph, pw, sh, sw),
                 orc.channelwise_conv_backward(grad, f, x.shape, ph, pw, sh, sw), "backward %s" % (case,))
    start, ft0 = g.uniform(-1, 1, f.shape).astype(np.float32), g.uniform(-1, 1, c).astype(np.float32)
    want, want_ft = orc.channelwise_conv_learn_add(x, grad, start, ph, pw, sh, sw, free_term_diff=ft0)
    got, got_ft = hip().channelwise_conv_learn_add(x, grad, start, ph, pw, sh, sw, free_term_diff=ft0)
    scale = np.sqrt(n * ho * wo)  # sums over every pixel of the batch
    assert_close(got, want, "learn %s" % (case,), atol=1e-5 * scale)
    assert_close(got_ft, want_ft, "free term gradient %s" % (case,), atol=1e-5 * scale)
    assert_close(hip().channelwise_conv_learn_add(x, grad, start, ph, pw, sh, sw), want, "learn, no free term", atol=1e-5 * scale)


@pytest.mark.parametrize("case", POOL_CASES + [(2, 57, 57, 64, 3, 3, 2, 2), (3, 16, 64, 7, 2, 2, 2, 2), (2, 23, 19, 8, 3, 3, 1, 1),
                                               (2, 9, 9, 4, 4, 4, 1, 1), (2, 10, 10, 6, 2, 2, 3, 3)])
def test_pooling_gradients(case):
    n, h, w, c, fh, fw, sh, sw = case
    g = rng(113 + h)
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    ho, wo = (h - fh) // sh + 1, (w - fw) // sw + 1
    grad = g.uniform(-1, 1, (n, ho, wo, c)).astype(np.float32)
    assert_close(hip().max_pool_backward(x, grad, fh, fw, sh, sw), orc.max_pool_backward(x, grad, fh, fw, sh, sw),
                 "max pooling backward %s" % (case,))
    assert_close(hip().mean_pool_backward(x.shape, grad, fh, fw, sh, sw), orc.mean_pool_backward(x.shape, grad, fh, fw, sh, sw),
                 "mean pooling backward %s" % (case,))


def test_k_sliced_convolutions_are_bit_reproducible():
    # K slices meet through partial tiles that the last slice to arrive adds up in slice order: whichever slice that is,
    # the sum has one order. Alternating shapes also checks that every launch leaves the arrival counters at zero.
    h = hip()
    g = rng(93)
    cases = [(4, 14, 14, 256, 256), (2, 7, 7, 512, 512), (24, 28, 28, 128, 128)]  # 3 slices; 8 slices; whole tiles + sliced tail
    data = []
    for n, hw, _, cin, cout in cases:
        x = g.uniform(-1, 1, (n, hw, hw, cin)).astype(np.float32)
        f = g.normal(0, 1.0 / np.sqrt(9 * cin), (cout, 3, 3, cin)).astype(np.float32)
        b = g.uniform(-1, 1, cout).astype(np.float32)
        data.append((x, f, b, h.conv(x, f, b, 1, 1, 1, 1)))
    for _ in range(3):
        for x, f, b, first in data:
            assert np.array_equal(h.conv(x, f, b, 1, 1, 1, 1), first)
    x, f, b, first = data[0]
    assert_close(first, orc.conv(x, f, b, 1, 1, 1, 1), "sliced convolution vs oracle")
    relu = h.conv(x, f, b, 1, 1, 1, 1, activation="relu")
    assert np.array_equal(relu, np.maximum(first, 0)), "activation in the last slice's epilogue"


def test_k_sliced_convolution_replays_from_a_captured_graph():
    # A launch recorded into a HIP graph must not keep the address of the slices' scratch block (a later, larger launch
    # frees it): under capture the slices meet in the result through atomic adds instead. The graph holds kernels only;
    # it is replayed several times with eager launches of other sizes between the replays.
    import ctypes
    import torch
    import neoml_amd
    lib = neoml_amd.load()
    g = rng(95)
    n, hw, cin, cout = 4, 14, 256, 256
    x = g.uniform(-1, 1, (n, hw, hw, cin)).astype(np.float32)
    f = g.normal(0, 1.0 / np.sqrt(9 * cin), (cout, 3, 3, cin)).astype(np.float32)
    b = g.uniform(-1, 1, cout).astype(np.float32)
    want = orc.conv(x, f, b, 1, 1, 1, 1)
    dev = torch.device("cuda:0")
    dx, df, db = (torch.from_numpy(a).to(dev) for a in (x, f, b))
    dy = torch.zeros((n, hw, hw, cout), device=dev)
    d = neoml_amd.ConvDesc(n, hw, hw, cin, cout, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)
    neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
    P = lambda t: ctypes.c_void_p(t.data_ptr())

    def launch():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        neoml_amd.check(lib.nhBlobConvolution(stream, ctypes.byref(d), P(dx), P(df), P(db), P(dy)))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert_close(dy.cpu().numpy(), want, "eager, slices meeting in scratch memory")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        launch()
    for replay in range(3):
        dy.zero_()
        # eager work between the replays: a larger sliced convolution, which grows the scratch block
        big = g.uniform(-1, 1, (8 + 8 * replay, hw, hw, cin)).astype(np.float32)
        assert_close(hip().conv(big, f, b, 1, 1, 1, 1)[:1], orc.conv(big[:1], f, b, 1, 1, 1, 1), "eager between replays")
        graph.replay()
        torch.cuda.synchronize()
        assert_close(dy.cpu().numpy(), want, "replay %d" % replay)


def test_k_sliced_convolutions_from_two_threads_on_one_stream():
    # The engine interface is thread-safe: two threads may enqueue on the engine's one stream at the same time. K-sliced
    # launches of one stream share a scratch block, which is replaced by larger ones while the other thread is launching
    # (the stream is new, so its block starts empty); every result must still be the one a single thread gets, bit for
    # bit: the slices are summed in a fixed order.
    import ctypes
    import threading
    import torch
    import neoml_amd
    lib = neoml_amd.load()
    g = rng(96)
    dev = torch.device("cuda:0")
    side = torch.cuda.Stream()
    stream = ctypes.c_void_p(side.cuda_stream)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    cin = cout = 256
    f = torch.from_numpy(g.normal(0, 1.0 / 48, (cout, 3, 3, cin)).astype(np.float32)).to(dev)
    b = torch.from_numpy(g.uniform(-1, 1, cout).astype(np.float32)).to(dev)

    def make(n):
        x = torch.from_numpy(g.uniform(-1, 1, (n, 14, 14, cin)).astype(np.float32)).to(dev)
        d = neoml_amd.ConvDesc(n, 14, 14, cin, cout, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)
        neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
        return d, x, torch.zeros((n, 14, 14, cout), device=dev)

    jobs = [[make(n) for n in sizes] for sizes in ((1, 3, 6, 12, 20), (2, 4, 8, 16, 24))]
    torch.cuda.synchronize()
    errors = []

    def worker(thread_jobs):
        try:
            for _ in range(20):
                for d, x, y in thread_jobs:
                    neoml_amd.check(lib.nhBlobConvolution(stream, ctypes.byref(d), P(x), P(f), P(b), P(y)))
        except Exception as e:  # reported by the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(tj,)) for tj in jobs]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    side.synchronize()
    assert not errors, errors
    threaded = [[y.cpu().numpy().copy() for _, _, y in tj] for tj in jobs]
    for thread_jobs, got in zip(jobs, threaded):
        for (d, x, y), have in zip(thread_jobs, got):
            y.zero_()
            torch.cuda.synchronize()
            neoml_amd.check(lib.nhBlobConvolution(stream, ctypes.byref(d), P(x), P(f), P(b), P(y)))
            side.synchronize()
            assert np.array_equal(y.cpu().numpy(), have)
    d, x, _ = jobs[1][2]
    assert_close(threaded[1][2], orc.conv(x.cpu().numpy(), f.cpu().numpy(), b.cpu().numpy(), 1, 1, 1, 1), "vs oracle")


def test_stream_destroy_frees_the_slices_scratch():
    # an application that makes an engine (= a stream) per request must not pile up scratch blocks
    import ctypes
    import torch
    import neoml_amd
    lib = neoml_amd.load()
    g = rng(97)
    dev = torch.device("cuda:0")
    n, hw, cin, cout = 16, 14, 256, 256   # 3 slices x 392 tiles x 16 KB = 19 MB of partial tiles
    x = torch.from_numpy(g.uniform(-1, 1, (n, hw, hw, cin)).astype(np.float32)).to(dev)
    f = torch.from_numpy(g.normal(0, 1.0 / 48, (cout, 3, 3, cin)).astype(np.float32)).to(dev)
    y = torch.zeros((n, hw, hw, cout), device=dev)
    d = neoml_amd.ConvDesc(n, hw, hw, cin, cout, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)
    neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    torch.cuda.synchronize()

    def once():
        stream = ctypes.c_void_p()
        neoml_amd.check(lib.nhStreamCreate(ctypes.byref(stream)))
        neoml_amd.check(lib.nhBlobConvolution(stream, ctypes.byref(d), P(x), P(f), None, P(y)))
        neoml_amd.check(lib.nhStreamSynchronize(stream))
        neoml_amd.check(lib.nhStreamDestroy(stream))
        return y.cpu().numpy().copy()

    first = once()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(12):
        assert np.array_equal(once(), first)
    free_after = torch.cuda.mem_get_info()[0]
    assert free_before - free_after < 32 * 1024 * 1024, (free_before, free_after)  # 12 leaked blocks would be 230 MB
    assert_close(first[:1], orc.conv(x[:1].cpu().numpy(), f.cpu().numpy(), None, 1, 1, 1, 1), "vs oracle")


def test_vector_sum_is_reproducible_and_may_write_into_its_operand():
    """Sums over many workgroups: the same bits on every run (the partial sums are added in a fixed order), and a result
    that lies inside the operand is read before it is written (the CPU engine computes first and stores last)."""
    import ctypes
    import torch
    import neoml_amd
    lib = neoml_amd.load()
    g = rng(123)
    n = 5_000_011
    host = g.normal(0, 1, n).astype(np.float32)
    dev = torch.device("cuda:0")
    x = torch.from_numpy(host).to(dev)
    y = torch.from_numpy(g.normal(0, 1, n).astype(np.float32)).to(dev)
    out = torch.zeros(4, device=dev)
    P = lambda t, offset=0: ctypes.c_void_p(t.data_ptr() + 4 * offset)
    runs = []
    for _ in range(5):
        neoml_amd.check(lib.nhVectorSum(None, P(x), n, P(out)))
        neoml_amd.check(lib.nhVectorDotProduct(None, P(x), P(y), n, P(out, 1)))
        torch.cuda.synchronize()
        runs.append(out[:2].cpu().numpy().copy())
    assert all(np.array_equal(r, runs[0]) for r in runs[1:]), runs
    assert abs(runs[0][0] - host.astype(np.float64).sum()) < 1.0
    # the result in the middle of the operand
    want = float(host.astype(np.float64).sum())
    neoml_amd.check(lib.nhVectorSum(None, P(x), n, P(x, 2_500_000)))
    torch.cuda.synchronize()
    got = float(x[2_500_000].item())
    assert abs(got - want) < 1.0 and got == float(runs[0][0]), (got, want, runs[0][0])
    # adding onto a value
    out[2] = 10.0
    neoml_amd.check(lib.nhVectorSumAdd(None, P(y), n, P(out, 2)))
    neoml_amd.check(lib.nhVectorSum(None, P(y), n, P(out, 3)))
    torch.cuda.synchronize()
    assert abs(float(out[2].item()) - 10.0 - float(out[3].item())) < 1e-3 * max(1.0, abs(float(out[3].item())))


def test_convolution_ignores_pixels_outside_the_windows():
    # stride 4 with a 3-wide filter never touches image columns 3 and 7; whatever they hold (here: infinities)
    # must not leak into the result through the vector fetches that run past a window's last value
    g = rng(77)
    x = g.uniform(-1, 1, (2, 6, 11, 3)).astype(np.float32)
    x[:, :, 3, :] = np.inf
    x[:, :, 7, :] = -np.inf
    f = g.normal(0, 0.3, (8, 3, 3, 3)).astype(np.float32)
    want = orc.conv(np.nan_to_num(x, posinf=0.0, neginf=0.0), f, None, 0, 0, 1, 4)
    got = hip().conv(x, f, None, 0, 0, 1, 4)
    assert np.isfinite(got).all()
    assert_close(got, want, "unused columns")


# The first layer of an image network: one or three channels, 3 x 3 or 7 x 7 filter, up to 64 filters, 16384 output
# pixels or more. These go through the window loader of the short-reduction kernel (128-bit loads at 4-byte alignment
# that bring along what lies next to a window; zeros by masks and by the memory unit's range check).
# (n, h, w, cin, cout, fh, fw, ph, pw, sh, sw)
WINDOW_CASES = [
    (2, 184, 200, 3, 32, 3, 3, 1, 1, 2, 2),   # the depthwise-separable network's stem, reduced
    (2, 190, 182, 3, 64, 7, 7, 3, 3, 2, 2),   # the residual network's stem, reduced: two rows of pixels begin in front of the blob
    (2, 96, 100, 1, 64, 3, 3, 1, 1, 1, 1),    # the line recogniser's first layer, reduced
    (1, 130, 140, 3, 20, 3, 3, 0, 0, 1, 1),   # no padding, a filter count that fills no column block
    (1, 400, 400, 3, 48, 3, 3, 2, 2, 3, 3),   # padding beyond the filter's reach on the left and at the top
    (1, 130, 131, 3, 8, 7, 7, 3, 3, 1, 1),    # windows that hang over the right border by up to three pixels
    (3, 151, 149, 1, 36, 3, 3, 1, 1, 2, 2),   # odd sizes: the last row block is ragged
    (1, 136, 129, 3, 64, 7, 7, 0, 5, 1, 1),   # wide padding on the left only
]


@pytest.mark.parametrize("case", WINDOW_CASES)
def test_first_layer_convolution(case):
    n, h, w, cin, cout, fh, fw, ph, pw, sh, sw = case
    g = rng(sum(case))
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 1.0 / np.sqrt(fh * fw * cin), (cout, fh, fw, cin)).astype(np.float32)
    bias = g.uniform(-1, 1, cout).astype(np.float32)
    want = orc.conv(x, f, bias, ph, pw, sh, sw)
    assert want.shape[0] * want.shape[1] * want.shape[2] >= 16384
    assert_close(hip().conv(x, f, bias, ph, pw, sh, sw), want, "first layer %s" % (case,))
    assert_close(hip().conv(x, f, None, ph, pw, sh, sw), want - bias, "without free term", atol=2e-5)
    assert_close(hip().conv(x, f, bias, ph, pw, sh, sw, activation="relu", param=0.5),
                 np.clip(want, 0.0, 0.5), "with ReLU clipped at 0.5")


def test_first_layer_convolution_reads_nothing_beside_its_windows():
    """Infinities in the image columns that no window touches (stride 4, filter 3 wide), and the image blob placed
    between two blocks of infinities: nothing of either may reach the result."""
    import ctypes
    import torch
    import neoml_amd
    lib = neoml_amd.load()
    g = rng(79)
    n, h, w, cin, cout = 2, 130, 267, 3, 24
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    x[:, :, 3::4, :] = np.inf
    f = g.normal(0, 0.3, (cout, 3, 3, cin)).astype(np.float32)
    want = orc.conv(np.nan_to_num(x, posinf=0.0), f, None, 0, 0, 1, 4)
    assert want.shape == (n, 128, 67, cout)
    dev = torch.device("cuda:0")
    guard = 1024  # floats, keeps the blob 16-byte aligned
    room = torch.full((guard + x.size + guard,), float("inf"), device=dev)
    room[guard:guard + x.size] = torch.from_numpy(x.reshape(-1)).to(dev)
    y = torch.zeros(want.shape, device=dev)
    fd = torch.from_numpy(f).to(dev)
    d = neoml_amd.ConvDesc(n, h, w, cin, cout, 3, 3, 0, 0, 1, 4, 1, 1, 0, 0)
    neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
    torch.cuda.synchronize()
    neoml_amd.check(lib.nhBlobConvolution(None, ctypes.byref(d), ctypes.c_void_p(room.data_ptr() + 4 * guard),
                                          ctypes.c_void_p(fd.data_ptr()), None, ctypes.c_void_p(y.data_ptr())))
    torch.cuda.synchronize()
    got = y.cpu().numpy()
    assert np.isfinite(got).all()
    assert_close(got, want, "unused columns and guards")
    # with padding: the windows of the first pixels begin in front of the blob, those of the last ones end behind it
    x2 = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    room[guard:guard + x.size] = torch.from_numpy(x2.reshape(-1)).to(dev)
    want2 = orc.conv(x2, f, None, 1, 1, 1, 1)
    y2 = torch.zeros(want2.shape, device=dev)
    d2 = neoml_amd.ConvDesc(n, h, w, cin, cout, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)
    neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d2)))
    neoml_amd.check(lib.nhBlobConvolution(None, ctypes.byref(d2), ctypes.c_void_p(room.data_ptr() + 4 * guard),
                                          ctypes.c_void_p(fd.data_ptr()), None, ctypes.c_void_p(y2.data_ptr())))
    torch.cuda.synchronize()
    got2 = y2.cpu().numpy()
    assert np.isfinite(got2).all()
    assert_close(got2, want2, "padded windows between guards")


def test_convolution_config1_vs_reference_engine():
    # the single-layer configuration at reduced batch: 32x32x64 image, 3x3 64 -> 64, pad 1, + free term, then ReLU
    g = rng(1)
    x = g.uniform(-1, 1, (2, 32, 32, 64)).astype(np.float32)
    f = g.normal(0, 1.0 / np.sqrt(576.0), (64, 3, 3, 64)).astype(np.float32)
    bias = np.zeros(64, np.float32)
    y = hip().conv(x, f, bias, 1, 1, 1, 1)
    y = hip().unary("relu", y, 0.0).reshape(2, 32, 32, 64)
    r = ref_or_none() or orc
    want = r.unary("relu", r.conv(x, f, bias, 1, 1, 1, 1), 0.0).reshape(2, 32, 32, 64)
    assert_close(y, want, "config 1")


def test_convolution_is_linear_at_full_size():
    # full single-layer configuration (batch 32): conv(a x1 + x2) == a conv(x1) + conv(x2), and the 1x1
    # identity filter returns the image; both hold for any size without a CPU pass over it
    h = hip()
    g = rng(40)
    x1 = g.uniform(-1, 1, (32, 32, 32, 64)).astype(np.float32)
    x2 = g.uniform(-1, 1, (32, 32, 32, 64)).astype(np.float32)
    f = g.normal(0, 1.0 / 24, (64, 3, 3, 64)).astype(np.float32)
    y1, y2 = h.conv(x1, f, None, 1, 1, 1, 1), h.conv(x2, f, None, 1, 1, 1, 1)
    y12 = h.conv(0.5 * x1 + x2, f, None, 1, 1, 1, 1)
    assert_close(y12, 0.5 * y1 + y2, "linearity", atol=1e-4)
    eye = np.eye(64, dtype=np.float32).reshape(64, 1, 1, 64)
    assert np.array_equal(h.conv(x1, eye, None, 0, 0, 1, 1), x1)


@pytest.mark.parametrize("case", CHANNELWISE_CASES + [(2, 28, 28, 96, 3, 3, 1, 1, 1, 1), (2, 28, 28, 96, 3, 3, 1, 1, 2, 2),
                                                      (1, 15, 13, 6, 3, 3, 1, 1, 2, 2), (1, 9, 30, 32, 5, 5, 2, 2, 1, 1),
                                                      # the 3x3 strip kernel: ragged row chunks and strip widths, no / wide / uneven padding
                                                      (2, 30, 17, 8, 3, 3, 1, 1, 1, 1), (1, 11, 11, 4, 3, 3, 0, 0, 1, 1),
                                                      (1, 7, 9, 12, 3, 3, 2, 2, 2, 2), (3, 13, 21, 16, 3, 3, 2, 0, 1, 1),
                                                      (2, 21, 13, 20, 3, 3, 0, 2, 2, 2), (1, 3, 3, 4, 3, 3, 1, 1, 1, 1),
                                                      # one strip of 12 rows per work item (a full-size MobileNet layer)
                                                      (128, 112, 112, 32, 3, 3, 1, 1, 1, 1)])
def test_channelwise_convolution(case):
    n, h, w, c, fh, fw, ph, pw, sh, sw = case
    g = rng(12 + c)
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    f = g.normal(0, 1, (fh, fw, c)).astype(np.float32)
    bias = g.uniform(-1, 1, c).astype(np.float32)
    assert_close(hip().channelwise_conv(x, f, bias, ph, pw, sh, sw), orc.channelwise_conv(x, f, bias, ph, pw, sh, sw), str(case))
    assert_close(hip().channelwise_conv(x, f, None, ph, pw, sh, sw), orc.channelwise_conv(x, f, None, ph, pw, sh, sw), str(case))


@pytest.mark.parametrize("case", POOL_CASES + [(2, 57, 57, 64, 3, 3, 2, 2), (3, 16, 64, 7, 2, 2, 2, 2), (2, 4, 128, 256, 2, 1, 2, 1),
                                               (2, 23, 19, 8, 3, 3, 1, 1), (1, 31, 9, 12, 2, 2, 2, 2), (2, 9, 9, 4, 4, 4, 1, 1),
                                               (64, 114, 114, 64, 3, 3, 2, 2)])
def test_pooling(case):
    n, h, w, c, fh, fw, sh, sw = case
    g = rng(13 + h)
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    assert np.array_equal(hip().max_pool(x, fh, fw, sh, sw), orc.max_pool(x, fh, fw, sh, sw))
    assert_close(hip().mean_pool(x, fh, fw, sh, sw), orc.mean_pool(x, fh, fw, sh, sw), "mean %s" % (case,))
    y, idx = hip().max_pool(x, fh, fw, sh, sw, with_indices=True)
    oy, oidx = orc.max_pool(x, fh, fw, sh, sw, with_indices=True)
    assert np.array_equal(y, oy)
    assert np.array_equal(idx, oidx), "pooling indices must be bit-exact"


def test_pooling_index_ties_bit_exact():
    g = rng(15)
    x = np.maximum(g.uniform(-1, 0.3, (2, 16, 16, 8)), 0).astype(np.float32)  # many all-zero windows, as after ReLU
    x = np.round(x * 4) / 4
    r = ref_or_none() or orc
    for fh, fw, sh, sw in ((2, 2, 2, 2), (3, 3, 2, 2), (3, 3, 1, 1)):
        y, idx = hip().max_pool(x, fh, fw, sh, sw, with_indices=True)
        ry, ridx = r.max_pool(x, fh, fw, sh, sw, with_indices=True)
        assert np.array_equal(y, ry) and np.array_equal(idx, ridx)


def test_resize_image():
    g = rng(16)
    for shape in ((2, 5, 6, 3), (2, 9, 7, 8)):
        x = g.uniform(-1, 1, shape).astype(np.float32)
        for dl, dr, dt, db in ((1, 1, 1, 1), (2, 0, 0, 3), (0, 0, 0, 0), (3, 2, 1, 4), (-1, -2, -1, 0), (-1, 2, 1, -2)):
            for mode in (0, 1, 2):
                if mode != 0 and min(dl, dr, dt, db) < 0:
                    continue
                assert np.array_equal(hip().resize_image(x, dl, dr, dt, db, mode, 0.5), orc.resize_image(x, dl, dr, dt, db, mode, 0.5))


@pytest.mark.parametrize("from_dims,to_dims,width", BROADCAST_CASES + [((1, 64, 1, 1, 1, 1, 96), (1, 64, 1, 28, 28, 1, 96), 1)])
def test_broadcast_copy(from_dims, to_dims, width):
    g = rng(170 + sum(from_dims))
    x = g.uniform(-1, 1, from_dims + (width,)).astype(np.float32)
    assert np.array_equal(hip().broadcast_copy(x, to_dims, width), np.broadcast_to(x, to_dims + (width,)))


@pytest.mark.parametrize("dims,rate,spatial,batchwise", DROPOUT_CASES + [((1, 64, 1, 28, 28, 1, 96), 0.2, False, False),
                                                                          ((1, 64, 1, 28, 28, 1, 96), 0.2, True, False)])
def test_dropout_mask_bit_exact(dims, rate, spatial, batchwise):
    g = rng(180 + sum(dims))
    x = g.uniform(0.5, 1.5, dims).astype(np.float32)
    for seed in (1, 12345, -7):
        want = orc.dropout(x, rate, spatial, batchwise, seed)
        got = hip().dropout(x, rate, spatial, batchwise, seed)
        assert np.array_equal(got != 0, want != 0), "dropout mask"
        assert_close(got, want, "dropout values")
    assert np.array_equal(hip().dropout(x, rate, spatial, batchwise, 5, inplace=True) != 0, orc.dropout(x, rate, spatial, batchwise, 5) != 0)


def test_split_and_merge():
    g = rng(17)
    big = g.uniform(-1, 1, (2, 3, 1, 4, 5, 1, 12)).astype(np.float32)
    for dim, sizes in ((6, (4, 8)), (6, (3, 4, 5)), (4, (2, 3)), (3, (1, 3)), (0, (1, 1)), (1, (2, 1))):
        part_dims = []
        for s in sizes:
            d = list(big.shape)
            d[dim] = s
            part_dims.append(tuple(d))
        want = orc.split(big, dim, part_dims)
        got = hip().split(big, dim, part_dims)
        for p, q in zip(got, want):
            assert np.array_equal(p, q), (dim, sizes)
        assert np.array_equal(hip().merge(want, dim, big.shape), big)
    # LSTM gate split: 4H -> 4 x H along channels
    gates = g.uniform(-1, 1, (1, 64, 1, 1, 1, 1, 1024)).astype(np.float32)
    parts = hip().split(gates, 6, [(1, 64, 1, 1, 1, 1, 256)] * 4)
    for i, p in enumerate(parts):
        assert np.array_equal(p, gates[..., 256 * i:256 * (i + 1)])


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("with_init", [False, True])
def test_lstm(reverse, with_init):
    g = rng(18)
    for T, B, In, H in ((5, 3, 6, 4), (7, 16, 32, 64), (4, 64, 256, 256), (6, 70, 48, 96), (33, 5, 16, 32)):
        w_in = g.uniform(-0.2, 0.2, (4 * H, In)).astype(np.float32)
        w_rec = g.uniform(-0.2, 0.2, (4 * H, H)).astype(np.float32)
        b_in = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
        b_rec = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
        x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
        c0 = g.uniform(-1, 1, (B, H)).astype(np.float32) if with_init else None
        h0 = g.uniform(-1, 1, (B, H)).astype(np.float32) if with_init else None
        for bi, br in ((b_in, b_rec), (None, b_rec), (None, None)):
            h, c = hip().lstm(w_in, bi, w_rec, br, x, reverse, c0, h0)
            oh, oc = orc.lstm(w_in, bi, w_rec, br, x, reverse, c0, h0)
            assert_close(h, oh, "lstm h %s" % ((T, B, In, H),))
            assert_close(c, oc, "lstm c")
            h2, _ = hip().lstm(w_in, bi, w_rec, br, x, reverse, c0, h0, want_state=False)
            assert_close(h2, oh, "lstm h without state output")


GPU_SEPARABLE_CASES = SEPARABLE_CASES + [
    (2, 56, 56, 24, 144, 24, 1, True, ("relu", 6.0), ("relu", 6.0)),    # the row-resident pointwise kernel on both 1x1 stages
    (1, 112, 112, 16, 96, 24, 2, False, ("relu", 6.0), ("relu", 6.0)),
    (4, 14, 14, 64, 384, 64, 1, True, ("hswish", 0.0), ("hswish", 0.0)),  # the tiled kernel with an epilogue
]


@pytest.mark.parametrize("case", GPU_SEPARABLE_CASES)
@pytest.mark.parametrize("with_expand", [True, False])
def test_separable_blocks(case, with_expand):
    for with_free_terms in (True, False):
        x, expand, channelwise, down, stride, residual = separable_operands(case, with_expand, with_free_terms)
        want = orc.separable_block(x, expand, channelwise, down, stride, residual)
        got = hip().separable_block(x, expand, channelwise, down, stride, residual)
        assert_close(got, want, "separable block %s expand=%s" % (case, with_expand))
        if residual and with_expand:  # the layer of the MobileNetV2 block reuses its input blob
            got = hip().separable_block(x, expand, channelwise, down, stride, residual, in_place=True)
            assert_close(got, want, "separable block in place %s" % (case,))


# Blocks whose expanded tensor would be far larger than the caches: expand and depthwise stage run as one launch that
# keeps the expanded values of a patch of pixels in LDS (32 expanded channels at a time). Sizes that are and are not
# multiples of the patch, a last chunk of 16 and of 4 channels, both strides, 16 / 24 / 32 input channels, with and
# without free terms, a residual, also one that reuses the input blob.
LARGE_SEPARABLE_CASES = [
    (16, 112, 112, 16, 96, 24, 2, False, ("relu", 6.0), ("relu", 6.0)),
    (40, 56, 56, 24, 144, 24, 1, True, ("relu", 6.0), ("relu", 6.0)),
    (40, 56, 56, 24, 144, 32, 2, False, ("relu", 6.0), ("relu", 6.0)),
    (128, 28, 28, 32, 192, 32, 1, True, ("relu", 6.0), ("relu", 6.0)),
    (24, 100, 90, 16, 100, 24, 1, False, ("hswish", 0.0), ("relu", 0.0)),
    (24, 101, 91, 16, 96, 24, 2, False, ("relu", 6.0), (None, 0.0)),
    # 32 input channels, without and with a residual
    (48, 60, 52, 32, 128, 16, 1, False, ("hswish", 0.0), ("relu", 0.0)),
    (48, 60, 52, 32, 192, 32, 1, True, ("relu", 6.0), ("relu", 6.0)),
]


@pytest.mark.parametrize("case", LARGE_SEPARABLE_CASES)
def test_separable_blocks_without_the_expanded_tensor(case):
    for with_free_terms in (True, False):
        x, expand, channelwise, down, stride, residual = separable_operands(case, True, with_free_terms)
        want = orc.separable_block(x, expand, channelwise, down, stride, residual)
        got = hip().separable_block(x, expand, channelwise, down, stride, residual)
        assert_close(got, want, "separable block %s free terms=%s" % (case, with_free_terms))
        if residual:
            got = hip().separable_block(x, expand, channelwise, down, stride, residual, in_place=True)
            assert_close(got, want, "separable block in place %s" % (case,))


def test_fused_expand_depthwise_treats_nan_like_the_separate_launches():
    """ReLU turns NaN into 0 (VectorReLU's rule, the vector maximum of the CPU engine): the one-launch expand + depthwise
    stage must do so as well. The same images run in one large batch (one launch) and two at a time (three launches)."""
    case = (16, 112, 112, 16, 96, 24, 2, False, ("relu", 6.0), ("relu", 6.0))
    x, expand, channelwise, down, stride, residual = separable_operands(case, True, True)
    x[:, 5, 7, 3] = np.nan
    x[3, 111, 111, 0] = np.inf
    whole = hip().separable_block(x, expand, channelwise, down, stride, residual)
    parts = np.concatenate([hip().separable_block(x[i:i + 2], expand, channelwise, down, stride, residual) for i in range(0, 16, 2)])
    assert np.isfinite(whole).all() and np.isfinite(parts).all()
    assert_close(whole, parts, "one launch vs three launches, NaN and infinity in the input")


@pytest.mark.parametrize("case", MOBILENETV3_CASES + [
    (4, 28, 28, 40, 120, 40, 5, 1, True, ("relu", 0.0), ("relu", 0.0), ("relu", 0.0)),
    (2, 14, 14, 80, 480, 112, 3, 1, False, ("hswish", 0.0), ("hswish", 0.0), ("hswish", 0.0)),
    (2, 14, 14, 112, 672, 160, 5, 2, False, ("hswish", 0.0), ("hswish", 0.0), ("hswish", 0.0)),
    # an expanded tensor far larger than the caches behind a 3x3 depthwise stage: expand and depthwise in one launch
    (32, 112, 112, 16, 64, 24, 3, 2, False, ("relu", 0.0), ("hswish", 0.0), ("relu", 0.0)),
    (72, 56, 56, 24, 72, 24, 3, 1, True, ("hswish", 0.0), ("relu", 0.0), ("hswish", 0.0))])
def test_mobilenetv3_blocks(case):
    n, h, w, cin, e, cout, fsize, stride, residual, ex_act, ch_act, gate_act = case
    x, expand, channelwise, gate, down = mobilenetv3_operands(case)
    pre = orc.mobilenetv3_pre_se(x, expand, channelwise, stride)
    assert_close(hip().mobilenetv3_pre_se(x, expand, channelwise, stride), pre, "pre-SE %s" % (case,), atol=2e-5)
    res = x if residual and stride == 1 and cin == cout else None
    want = orc.mobilenetv3_post_se(pre, gate, res, gate_act[0], gate_act[1], down)
    assert_close(hip().mobilenetv3_post_se(pre, gate, res, gate_act[0], gate_act[1], down), want, "post-SE %s" % (case,), atol=2e-5)
    assert_close(hip().mobilenetv3_post_se(pre, gate, None, gate_act[0], gate_act[1], (down[0], None)),
                 orc.mobilenetv3_post_se(pre, gate, None, gate_act[0], gate_act[1], (down[0], None)), "post-SE, bare", atol=2e-5)
    if res is not None:  # the layer may hand the residual blob over as the output blob
        got = hip().mobilenetv3_post_se(pre, gate, res, gate_act[0], gate_act[1], down, in_place_residual=True)
        assert_close(got, want, "post-SE into its residual", atol=2e-5)


def test_lstm_layout_by_xcds_ragged_and_full():
    """The one-launch kernel that lays the sequences out by XCDs ( H = 64, 128, 256, 512 ): sequence counts that are no
    multiple of a workgroup's four, one that leaves whole XCDs without work and the most that fit the eight XCDs, with and
    without initial state, both directions, cell state asked for."""
    g = rng(186)
    for T, B, In, H in ((9, 13, 24, 64), (5, 130, 16, 128), (4, 128, 32, 256), (6, 127, 8, 256), (3, 1, 8, 512), (12, 64, 16, 512)):
        w_in = g.uniform(-0.2, 0.2, (4 * H, In)).astype(np.float32)
        w_rec = g.uniform(-2.0 / H ** 0.5, 2.0 / H ** 0.5, (4 * H, H)).astype(np.float32)
        b_in = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
        x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
        for reverse, with_init in ((False, True), (True, False)):
            c0 = g.uniform(-1, 1, (B, H)).astype(np.float32) if with_init else None
            h0 = g.uniform(-1, 1, (B, H)).astype(np.float32) if with_init else None
            h, c = hip().lstm(w_in, b_in, w_rec, None, x, reverse, c0, h0)
            oh, oc = orc.lstm(w_in, b_in, w_rec, None, x, reverse, c0, h0)
            assert_close(h, oh, "lstm h %s" % ((T, B, In, H, reverse),))
            assert_close(c, oc, "lstm c %s" % ((T, B, In, H, reverse),))


def test_lstm_long_sequence():
    # 128 steps through the one-launch path (H a multiple of 16 and a grid that fits the device), H = 512 through
    # its 16-wavefront shape, plus a shape whose grid does not fit and takes the launch-per-step path
    g = rng(181)
    for T, B, In, H in ((128, 20, 24, 128), (6, 20, 16, 512), (3, 40, 16, 1024)):
        w_in = g.uniform(-0.2, 0.2, (4 * H, In)).astype(np.float32)
        w_rec = g.uniform(-2.0 / H ** 0.5, 2.0 / H ** 0.5, (4 * H, H)).astype(np.float32)
        b_in = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
        x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
        for reverse in (False, True):
            h, c = hip().lstm(w_in, b_in, w_rec, None, x, reverse)
            oh, oc = orc.lstm(w_in, b_in, w_rec, None, x, reverse)
            assert_close(h, oh, "lstm h %s" % ((T, B, In, H),))
            assert_close(c, oc, "lstm c %s" % ((T, B, In, H),))


def test_lstm_bounded_wait_gives_up(monkeypatch):
    # The step wait of the one-launch LSTM is bounded. With a spin limit of zero, forced from the host, a
    # wavefront that finds a value of the previous step not yet published raises the abort word and every
    # workgroup leaves: the launch ends normally and the word is visible in the workspace. (If every value
    # happens to be there in time, the word stays zero and the output is the regular one.)
    g = rng(182)
    T, B, In, H = 64, 64, 16, 256
    w_in = g.uniform(-0.2, 0.2, (4 * H, In)).astype(np.float32)
    w_rec = g.uniform(-0.1, 0.1, (4 * H, H)).astype(np.float32)
    x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
    monkeypatch.setenv("NH_LSTM_SPIN_LIMIT", "0")
    h, _, word = hip().lstm(w_in, None, w_rec, None, x, want_state=False, return_sync=True)
    monkeypatch.delenv("NH_LSTM_SPIN_LIMIT")
    assert word in (0, 1)
    # the give-up is also reported, once, by the next synchronising call of the library
    import neoml_amd
    rc = neoml_amd.load().nhStreamSynchronize(hip().stream())
    assert rc == (2 if word == 1 else 0)
    if word == 1:
        assert "gave up" in neoml_amd.last_error()
    assert neoml_amd.load().nhStreamSynchronize(hip().stream()) == 0
    h2, _, word2 = hip().lstm(w_in, None, w_rec, None, x, want_state=False, return_sync=True)
    assert word2 == 0
    oh, _ = orc.lstm(w_in, None, w_rec, None, x)
    assert_close(h2, oh, "lstm after a forced give-up")


def _enqueue_lstm(h, stream, w_in, w_rec, x):
    """nhLstm on `stream` without waiting for it; returns the output tensor and what must stay alive."""
    import torch
    T, B, In = x.shape
    H = w_rec.shape[1]
    with torch.cuda.stream(stream):
        ws = [h.up(a) for a in (w_in, w_rec, x)]
        out = h.empty((T, B, H))
        size = ctypes.c_size_t(0)
        h.na.check(h.lib.nhLstmWorkspaceSize(H, In, T, B, ctypes.byref(size)))
        work = torch.empty((size.value + 15) // 4, dtype=torch.float32, device=h.dev)
        h.call("nhLstm", H, In, h.p(ws[0]), None, h.p(ws[1]), None, 0, T, B, None, None, h.p(ws[2]), None, h.p(out),
               h.p(work), size.value)
    return out, (ws, work)


def test_lstm_on_two_streams_and_give_up_reported_to_its_own_stream(monkeypatch):
    """Two one-launch LSTMs issued on two streams without a wait between them: the library orders the second behind the
    first on the device (each needs the whole device resident), both give the oracle's result. Then a give-up forced
    from the host (spin limit zero) on the first stream is reported by that stream's next synchronising call only: the
    other stream's synchronise stays clean."""
    import torch
    import neoml_amd
    h = hip()
    lib = neoml_amd.load()
    g = rng(183)
    T, B, In, H = 48, 64, 32, 256
    w_in = g.uniform(-0.2, 0.2, (4 * H, In)).astype(np.float32)
    w_rec = g.uniform(-0.1, 0.1, (4 * H, H)).astype(np.float32)
    xa = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
    xb = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    pa, pb = ctypes.c_void_p(sa.cuda_stream), ctypes.c_void_p(sb.cuda_stream)
    torch.cuda.synchronize()
    out_a, keep_a = _enqueue_lstm(h, sa, w_in, w_rec, xa)
    out_b, keep_b = _enqueue_lstm(h, sb, w_in, w_rec, xb)
    assert lib.nhStreamSynchronize(pa) == 0 and lib.nhStreamSynchronize(pb) == 0
    assert_close(out_a.cpu().numpy(), orc.lstm(w_in, None, w_rec, None, xa)[0], "lstm on stream a")
    assert_close(out_b.cpu().numpy(), orc.lstm(w_in, None, w_rec, None, xb)[0], "lstm on stream b")
    # forced give-up on stream a, a regular run on stream b
    monkeypatch.setenv("NH_LSTM_SPIN_LIMIT", "0")
    out_a2, keep_a2 = _enqueue_lstm(h, sa, w_in, w_rec, xa)
    monkeypatch.delenv("NH_LSTM_SPIN_LIMIT")
    out_b2, keep_b2 = _enqueue_lstm(h, sb, w_in, w_rec, xb)
    rc_b = lib.nhStreamSynchronize(pb)
    rc_a = lib.nhStreamSynchronize(pa)
    assert rc_b == 0
    assert_close(out_b2.cpu().numpy(), out_b.cpu().numpy(), "lstm on stream b beside a give-up on stream a")
    assert rc_a in (0, 2)  # 0: every value happened to be there in time
    if rc_a == 2:
        assert "gave up" in neoml_amd.last_error()
    assert lib.nhStreamSynchronize(pa) == 0  # reported once
    del keep_a, keep_b, keep_a2, keep_b2


def test_independent_lstms_side_by_side(capsys):
    """nhStreamOverlapLstm: the two directions of a bidirectional layer, two nhLstm calls one behind the other on one
    stream with workspaces of their own, run side by side and give what the calls give in order. A second call that
    reads the first one's result, or whose input is produced by a launch in between, does not overtake anything."""
    import torch
    import neoml_amd
    h = hip()
    lib = neoml_amd.load()
    g = rng(185)
    T, B, In, H = 64, 64, 256, 256
    dev = h.dev

    def operands(n_in):
        w_in = g.uniform(-0.2, 0.2, (4 * H, n_in)).astype(np.float32)
        w_rec = g.uniform(-0.1, 0.1, (4 * H, H)).astype(np.float32)
        bias = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
        return w_in, w_rec, bias

    fwd, rev = operands(In), operands(In)
    x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
    s = torch.cuda.Stream()
    ps = ctypes.c_void_p(s.cuda_stream)
    size = ctypes.c_size_t(0)
    neoml_amd.check(lib.nhLstmWorkspaceSize(H, In, T, B, ctypes.byref(size)))
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    d_fwd, d_rev, d_x = [up(a) for a in fwd], [up(a) for a in rev], up(x)
    work = [torch.empty((size.value + 15) // 4, dtype=torch.float32, device=dev) for _ in range(2)]
    out = [torch.zeros((T, B, H), device=dev) for _ in range(3)]
    torch.cuda.synchronize()

    def lstm(weights, source, reverse, result, workspace):
        neoml_amd.check(lib.nhLstm(ps, H, In, P(weights[0]), P(weights[2]), P(weights[1]), None, reverse, T, B, None, None, P(source),
                                   None, P(result), P(workspace), size.value))

    def both_directions():
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record(s)
        lstm(d_fwd, d_x, 0, out[0], work[0])
        lstm(d_rev, d_x, 1, out[1], work[1])
        stop.record(s)
        assert lib.nhStreamSynchronize(ps) == 0
        return start.elapsed_time(stop), out[0].cpu().numpy().copy(), out[1].cpu().numpy().copy()

    def best_of(times):
        runs = [both_directions() for _ in range(times)]
        return (min(r[0] for r in runs),) + runs[-1][1:]

    both_directions()
    in_order_ms, f0, r0 = best_of(4)
    neoml_amd.check(lib.nhStreamOverlapLstm(ps, 1))
    try:
        both_directions()
        side_by_side_ms, f1, r1 = best_of(4)
        with capsys.disabled():
            print("\ntwo LSTM directions, %d steps, %d sequences, %d units: %.0f us in order, %.0f us side by side" % (
                T, B, H, in_order_ms * 1e3, side_by_side_ms * 1e3))
        want_f = orc.lstm(fwd[0], fwd[2], fwd[1], None, x, False)[0]
        want_r = orc.lstm(rev[0], rev[2], rev[1], None, x, True)[0]
        assert_close(f1, want_f, "forward direction, side by side")
        assert_close(r1, want_r, "reverse direction, side by side")
        assert_close(f1, f0, "forward direction: side by side vs in order")
        assert_close(r1, r0, "reverse direction: side by side vs in order")
        # the second reads what the first writes ( In == H ): it must wait
        lstm(d_fwd, d_x, 0, out[0], work[0])
        lstm(d_rev, out[0], 1, out[1], work[1])
        assert lib.nhStreamSynchronize(ps) == 0
        assert_close(out[1].cpu().numpy(), orc.lstm(rev[0], rev[2], rev[1], None, want_f, True)[0], "stacked: the second reads the first",
                     atol=2e-5)
        # a launch between the two produces the second one's input
        lstm(d_fwd, d_x, 0, out[0], work[0])
        neoml_amd.check(lib.nhVectorCopy(ps, P(out[2]), P(d_x), d_x.numel()))
        lstm(d_rev, out[2], 1, out[1], work[1])
        assert lib.nhStreamSynchronize(ps) == 0
        assert_close(out[1].cpu().numpy(), want_r, "a launch between the two")
        # the same workspace for both: in order again
        lstm(d_fwd, d_x, 0, out[0], work[0])
        lstm(d_rev, d_x, 1, out[1], work[0])
        assert lib.nhStreamSynchronize(ps) == 0
        assert_close(out[0].cpu().numpy(), want_f, "shared workspace, first")
        assert_close(out[1].cpu().numpy(), want_r, "shared workspace, second")
    finally:
        neoml_amd.check(lib.nhStreamOverlapLstm(ps, 0))


# ---------------------------------------------------------------------------------------------------------
# error convention and allocator on the device

def test_empty_inputs_are_accepted():
    """Zero-sized operands (an empty batch, a vector of no elements, a product over no terms) return NH_OK and leave
    memory they do not own alone; a product over K = 0 terms is the free term / zero."""
    import neoml_amd
    h = hip()
    lib, P = h.lib, h.p
    guard = h.up(np.full(64, 7.0, np.float32))
    zero = h.scalar(0.0)
    ok = lambda rc: neoml_amd.check(rc)
    ok(lib.nhVectorAdd(h.stream(), P(guard), P(guard), P(guard), 0))
    ok(lib.nhVectorReLU(h.stream(), P(guard), P(guard), 0, P(zero)))
    ok(lib.nhVectorCopy(h.stream(), P(guard), P(guard), 0))
    total = h.up(np.full(1, 5.0, np.float32))
    ok(lib.nhVectorSum(h.stream(), P(guard), 0, P(total)))
    assert h.down(total)[0] == 0.0
    ok(lib.nhMatrixSoftmaxByRows(h.stream(), P(guard), 0, 16, P(guard)))
    ok(lib.nhSumMatrixRows(h.stream(), 0, P(guard), P(guard), 4, 4))
    ok(lib.nhMultiplyMatrixByTransposedMatrix(h.stream(), P(guard), 0, 8, 8, P(guard), 4, 8, P(guard), 4, 0))
    d = neoml_amd.ConvDesc(0, 8, 8, 4, 4, 3, 3, 1, 1, 1, 1, 1, 1, 0, 0)
    ok(lib.nhInitBlobConvolution(ctypes.byref(d)))
    ok(lib.nhBlobConvolution(h.stream(), ctypes.byref(d), P(guard), P(guard), None, P(guard)))
    p = neoml_amd.PoolingDesc(0, 8, 8, 4, 2, 2, 2, 2, 0, 0)
    ok(lib.nhInitPooling(ctypes.byref(p)))
    ok(lib.nhBlobMaxPooling(h.stream(), ctypes.byref(p), P(guard), None, P(guard)))
    ok(lib.nhBlobMeanPoolingBackward(h.stream(), ctypes.byref(p), P(guard), P(guard)))
    assert np.array_equal(h.down(guard), np.full(64, 7.0, np.float32))
    # K = 0: [4 x 0] * [0 x 5] is a matrix of zeros
    a = np.zeros((4, 0), np.float32)
    b = np.zeros((5, 0), np.float32)
    out = h.up(np.full(20, 3.0, np.float32))
    ok(lib.nhMultiplyMatrixByTransposedMatrix(h.stream(), P(guard), 4, 0, 0, P(guard), 5, 0, P(out), 5, 20))
    assert np.array_equal(h.down(out), np.zeros(20, np.float32))


def test_argument_errors_are_reported_not_thrown():
    import neoml_amd
    lib = neoml_amd.load()
    d = neoml_amd.ConvDesc(1, 4, 4, 3, 2, 5, 5, 0, 0, 1, 1, 1, 1, 0, 0)  # filter larger than the image
    assert lib.nhInitBlobConvolution(ctypes.byref(d)) == 1
    assert "requirement failed" in neoml_amd.last_error()
    assert lib.nhVectorReLU(None, None, None, -1, None) == 1


def test_device_pool():
    import neoml_amd
    lib = neoml_amd.load()
    pool = ctypes.c_void_p()
    neoml_amd.check(lib.nhPoolCreate(ctypes.byref(pool), 0, 64 << 20))
    p1, p2 = ctypes.c_void_p(), ctypes.c_void_p()
    neoml_amd.check(lib.nhPoolHeapAlloc(pool, 1000, ctypes.byref(p1)))
    neoml_amd.check(lib.nhPoolHeapFree(pool, p1))
    neoml_amd.check(lib.nhPoolHeapAlloc(pool, 900, ctypes.byref(p2)))
    assert p1.value == p2.value  # same size class: the cached block comes back without a raw allocation
    big = ctypes.c_void_p()
    assert lib.nhPoolHeapAlloc(pool, 128 << 20, ctypes.byref(big)) == 3  # over the limit: NH_ERR_MEMORY
    # the block is usable device memory
    h = hip()
    neoml_amd.check(lib.nhVectorFill(h.stream(), p2, ctypes.c_float(3.0), 225))
    host = (ctypes.c_float * 225)()
    neoml_amd.check(lib.nhCopyDeviceToHost(h.stream(), host, p2, 900))
    assert list(host) == [3.0] * 225
    neoml_amd.check(lib.nhPoolHeapFree(pool, p2))
    neoml_amd.check(lib.nhPoolDestroy(pool))
