"""Pins the CPU oracle (oracle/oracle.c).

Two independent anchors for every function:
  1. the reference's own CCpuMathEngine, compiled from its sources into oracle/_ref (skipped only when that
     build is absent), called through oracle/engine_shim.cpp;
  2. formulations that do not share code with the oracle: numpy / scipy routines, closed forms, brute force.
A dropped term, swapped index or transposed operand in the oracle fails at least one of them.
"""
import numpy as np
import pytest
import scipy.signal
import scipy.special

import nhtest
from nhtest import Cpu, assert_close

orc = Cpu("orc")
needs_ref = pytest.mark.skipif(not nhtest.have_reference(), reason="oracle/_ref is not built")


def ref():
    return Cpu("ref")


def rng(seed):
    return np.random.default_rng(0xC0FFEE + seed)


# ---------------------------------------------------------------------------------------------------------
# element-wise

UNARY_CASES = [
    ("relu", 0.0, 0.0), ("relu", 6.0, 0.0), ("elu", 0.7, 0.0), ("leaky_relu", 0.1, 0.0), ("hswish", 0, 0),
    ("abs", 0, 0), ("hard_tanh", 0, 0), ("hard_sigmoid", 0.2, 0.5), ("neg", 0, 0), ("exp", 0, 0), ("log", 0, 0),
    ("erf", 0, 0), ("sqrt", 0, 0), ("inv", 0, 0), ("minmax", -0.5, 1.5), ("sigmoid", 0, 0), ("tanh", 0, 0),
    ("add_value", 1.25, 0), ("multiply", -2.5, 0), ("neg_multiply", 1.702, 0), ("copy", 0, 0), ("neg_log", 0, 0),
    ("sub_value", 0.75, 0), ("value_sub", 0.75, 0), ("hinge", 0, 0), ("squared_hinge", 0, 0), ("huber", 0, 0),
    ("huber_derivative", 0, 0),
]


def unary_input(op, n, seed):
    x = rng(seed).uniform(-10, 10, n).astype(np.float32)
    if op in ("log", "sqrt", "neg_log"):
        x = np.abs(x) + 1e-3
    # special values: zeros, tiny, huge
    x[:8] = [0.0, -0.0, 1e-38, -1e-38, 3.0, -3.0, 87.0, -87.0]
    if op in ("log", "sqrt", "neg_log"):
        x[:8] = np.abs(x[:8])
    return x


NUMPY_UNARY = {
    "relu": lambda x, p0, p1: np.minimum(np.maximum(x, 0), p0) if p0 > 0 else np.maximum(x, 0),
    "elu": lambda x, p0, p1: np.where(x >= 0, x, p0 * np.expm1(np.minimum(x, 0).astype(np.float64))),
    "leaky_relu": lambda x, p0, p1: np.where(x > 0, x, p0 * x),
    "hswish": lambda x, p0, p1: x * np.clip(x + 3, 0, 6) / 6,
    "abs": lambda x, p0, p1: np.abs(x),
    "hard_tanh": lambda x, p0, p1: np.clip(x, -1, 1),
    "hard_sigmoid": lambda x, p0, p1: np.clip(x * p0 + p1, 0, 1),
    "neg": lambda x, p0, p1: -x,
    "exp": lambda x, p0, p1: np.exp(x.astype(np.float64)),
    "log": lambda x, p0, p1: np.log(np.clip(x.astype(np.float64), np.finfo(np.float32).tiny, None)),
    "erf": lambda x, p0, p1: scipy.special.erf(x.astype(np.float64)),
    "sqrt": lambda x, p0, p1: np.sqrt(x.astype(np.float64)),
    "minmax": lambda x, p0, p1: np.clip(x, p0, p1),
    "sigmoid": lambda x, p0, p1: scipy.special.expit(x.astype(np.float64)),
    "tanh": lambda x, p0, p1: np.tanh(x.astype(np.float64)),
    "add_value": lambda x, p0, p1: x + np.float32(p0),
    "multiply": lambda x, p0, p1: x * np.float32(p0),
    "neg_multiply": lambda x, p0, p1: -x * np.float32(p0),
    "copy": lambda x, p0, p1: x,
    "neg_log": lambda x, p0, p1: -np.log(np.clip(x.astype(np.float64), np.finfo(np.float32).tiny, None)),
    "sub_value": lambda x, p0, p1: x - np.float32(p0),
    "value_sub": lambda x, p0, p1: np.float32(p0) - x,
    "hinge": lambda x, p0, p1: np.maximum(0, 1 - x),
    "squared_hinge": lambda x, p0, p1: np.where(x < -1, -4 * x, np.maximum(0, 1 - x.astype(np.float64)) ** 2),
    "huber": lambda x, p0, p1: np.where(np.abs(x) > 1, np.abs(x) - 0.5, x.astype(np.float64) ** 2 / 2),
    "huber_derivative": lambda x, p0, p1: np.clip(x, -1, 1),
}


@pytest.mark.parametrize("op,p0,p1", UNARY_CASES)
def test_unary_vs_numpy(op, p0, p1):
    x = unary_input(op, 1003, 1)
    y = orc.unary(op, x, p0, p1)
    if op == "inv":
        big = np.abs(x) > 1e-30
        assert_close(y[big], 1.0 / x[big].astype(np.float64), op)
        fmax = np.finfo(np.float32).max
        # saturation of 0 and of denormals; with denormals-are-zero a negative denormal counts as +0
        assert y[0] == fmax and y[2] == fmax and y[3] == fmax
        tiny = np.finfo(np.float32).tiny
        edge = orc.unary("inv", np.array([tiny, -tiny, 2 * tiny], np.float32))
        assert edge[0] == fmax and edge[1] == -fmax and edge[2] == np.float32(1.0) / np.float32(2 * tiny)
        return
    assert_close(y, NUMPY_UNARY[op](x, p0, p1), op)


@needs_ref
@pytest.mark.parametrize("op,p0,p1", UNARY_CASES)
def test_unary_vs_reference(op, p0, p1):
    for n in (1, 3, 4, 7, 64, 1003):
        x = unary_input(op, max(n, 8), n)[:n] if n < 8 else unary_input(op, n, n)
        assert_close(orc.unary(op, x, p0, p1), ref().unary(op, x, p0, p1), "%s n=%d" % (op, n))


def test_vector_log_and_exp_clamps():
    fmin, fmax = np.finfo(np.float32).tiny, np.finfo(np.float32).max
    y = orc.unary("log", np.array([0.0, -5.0, fmin, np.inf], np.float32))
    assert_close(y, [np.log(np.float64(fmin))] * 3 + [np.log(np.float64(fmax))], "log clamp")
    e = orc.unary("exp", np.array([-100.0, -87.4, 88.5, 0.0], np.float32))
    assert e[0] == 0 and e[1] == 0 and e[2] == fmax and e[3] == 1


BINARY_CASES = ["add", "sub", "eltwise_multiply", "eltwise_neg_multiply", "eltwise_divide", "eltwise_max",
                "eltwise_min", "multiply_and_add", "multiply_and_sub", "eltwise_multiply_add"]
NUMPY_BINARY = {
    "add": lambda a, b, p, r: a + b, "sub": lambda a, b, p, r: a - b, "eltwise_multiply": lambda a, b, p, r: a * b,
    "eltwise_neg_multiply": lambda a, b, p, r: -a * b, "eltwise_divide": lambda a, b, p, r: a / b,
    "eltwise_max": lambda a, b, p, r: np.maximum(a, b), "eltwise_min": lambda a, b, p, r: np.minimum(a, b),
    "multiply_and_add": lambda a, b, p, r: a + np.float32(p) * b,
    "multiply_and_sub": lambda a, b, p, r: a - np.float32(p) * b,
    "eltwise_multiply_add": lambda a, b, p, r: r + a * b,
}


@pytest.mark.parametrize("op", BINARY_CASES)
def test_binary(op):
    g = rng(2)
    for n in (1, 5, 1000):
        a = g.uniform(-10, 10, n).astype(np.float32)
        b = g.uniform(0.5, 10, n).astype(np.float32) * np.where(g.random(n) < 0.5, -1, 1).astype(np.float32)
        r = g.uniform(-10, 10, n).astype(np.float32)
        y = orc.binary(op, a, b, 0.37, result=r)
        assert_close(y, NUMPY_BINARY[op](a, b, 0.37, r), op)
        if nhtest.have_reference():
            assert_close(y, ref().binary(op, a, b, 0.37, result=r), op + " vs reference")


# derivatives of the activations: first = the activation's input (or its output for the _op forms), second = the
# gradient that arrives from above, p = ReLU's upper threshold
DIFF_CASES = [("relu_diff", 0.0), ("relu_diff", 6.0), ("hswish_diff", 0.0), ("sigmoid_diff", 0.0), ("sigmoid_diff_op", 0.0),
              ("tanh_diff", 0.0), ("tanh_diff_op", 0.0), ("elu_diff", 0.7), ("elu_diff_op", 0.7), ("leaky_relu_diff", 0.1),
              ("hard_tanh_diff", 0.0), ("hard_sigmoid_diff", 0.2), ("hard_sigmoid_diff_op", 0.2), ("abs_diff", 0.0),
              ("hinge_diff", 0.0), ("squared_hinge_diff", 0.0), ("l1_diff_add", 0.3)]
HARD_SIGMOID_BIAS = 0.5  # second parameter of the hard sigmoid cases
_expit = lambda a: scipy.special.expit(a.astype(np.float64))
NUMPY_DIFF = {
    "relu_diff": lambda a, b, p: np.where((a > 0) & ((a < p) if p > 0 else True), b, 0),
    "hswish_diff": lambda a, b, p: np.where(a <= -3, 0, np.where(a >= 3, b, b * (2 * a.astype(np.float64) + 3) / 6)),
    "sigmoid_diff": lambda a, b, p: _expit(a) * (1 - _expit(a)) * b,
    "sigmoid_diff_op": lambda a, b, p: a.astype(np.float64) * (1 - a) * b,
    "tanh_diff": lambda a, b, p: (1 - np.tanh(a.astype(np.float64)) ** 2) * b,
    "tanh_diff_op": lambda a, b, p: (1 - a.astype(np.float64) ** 2) * b,
    "elu_diff": lambda a, b, p: np.where(a >= 0, b, b * p * np.exp(np.minimum(a, 0).astype(np.float64))),
    "elu_diff_op": lambda a, b, p: np.where(a >= 0, b, b * (a.astype(np.float64) + p)),
    "leaky_relu_diff": lambda a, b, p: np.where(a > 0, b, b * np.float32(p)),
    "hard_tanh_diff": lambda a, b, p: np.where(np.abs(a) < 1, b, 0),
    "hard_sigmoid_diff": lambda a, b, p: np.where((a * p + HARD_SIGMOID_BIAS > 0) & (a * p + HARD_SIGMOID_BIAS < 1), b * np.float32(p), 0),
    "hard_sigmoid_diff_op": lambda a, b, p: np.where((a > 0) & (a < 1), b * np.float32(p), 0),
    "abs_diff": lambda a, b, p: np.where(a > 0, b, -b),
    "hinge_diff": lambda a, b, p: np.where(a < 1, -b, 0),
    "squared_hinge_diff": lambda a, b, p: np.where(a < -1, -4 * b, -2 * np.maximum(0, 1 - a.astype(np.float64)) * b),
    # (p = the clamp threshold; the multiplier travels as the second parameter, HARD_SIGMOID_BIAS in these tests)
    "l1_diff_add": lambda a, b, p: a + np.float32(HARD_SIGMOID_BIAS) * np.clip(b, -np.float32(p), np.float32(p)),
}
# the activation each derivative belongs to, for the finite-difference check
DIFF_FORWARD = {"relu_diff": "relu", "hswish_diff": "hswish", "sigmoid_diff": "sigmoid", "tanh_diff": "tanh", "elu_diff": "elu",
                "leaky_relu_diff": "leaky_relu", "hard_tanh_diff": "hard_tanh", "hard_sigmoid_diff": "hard_sigmoid", "abs_diff": "abs",
                "hinge_diff": "hinge", "squared_hinge_diff": "squared_hinge"}


def diff_operands(op, n, seed):
    g = rng(seed)
    a = g.uniform(-8, 8, n).astype(np.float32)
    if op in ("sigmoid_diff_op", "tanh_diff_op"):
        a = g.uniform(-0.99 if op.startswith("tanh") else 0.01, 0.99, n).astype(np.float32)
    elif op in ("elu_diff_op", "hard_sigmoid_diff_op"):  # outputs of the activation: ELU above -alpha, hard sigmoid in [0, 1]
        a = g.uniform(-0.69, 3, n).astype(np.float32) if op == "elu_diff_op" else np.clip(g.uniform(-0.5, 1.5, n), 0, 1).astype(np.float32)
    elif op in ("leaky_relu_diff", "abs_diff"):
        pass  # no special values: at exactly 0 the reference's vector lanes and its scalar tail disagree
    elif n >= 8:
        a[:8] = [0.0, 3.0, -3.0, 6.0, 2.999, -2.999, 40.0, -40.0]
    b = g.uniform(-2, 2, n).astype(np.float32)
    return a, b


@pytest.mark.parametrize("op,p", DIFF_CASES)
def test_activation_derivatives(op, p):
    for n in (1, 5, 1003):
        a, b = diff_operands(op, n, 70 + n)
        y = orc.binary(op, a, b, p, p1=HARD_SIGMOID_BIAS)
        assert_close(y, NUMPY_DIFF[op](a, b, p), "%s n=%d" % (op, n))
        if nhtest.have_reference():
            assert_close(ref().binary(op, a, b, p, p1=HARD_SIGMOID_BIAS), y, "%s vs reference n=%d" % (op, n))


@pytest.mark.parametrize("op,p", [c for c in DIFF_CASES if c[0] in DIFF_FORWARD])
def test_activation_derivatives_are_the_slopes_of_the_activations(op, p):
    # central differences of the forward function in float64-friendly ranges, away from the kinks
    g = rng(75)
    a = g.uniform(-2.9, 2.9, 500).astype(np.float32)
    a = a[(np.abs(a) > 0.05)]
    eps = np.float32(1.0 / 256)
    fwd = DIFF_FORWARD[op]
    if op in ("hard_tanh_diff", "hard_sigmoid_diff", "hinge_diff", "squared_hinge_diff"):
        a = a[np.abs(np.abs(a) - (2.5 if op == "hard_sigmoid_diff" else 1.0)) > 0.05]  # away from their kinks as well
    slope = (orc.unary(fwd, a + eps, p, HARD_SIGMOID_BIAS).astype(np.float64) - orc.unary(fwd, a - eps, p, HARD_SIGMOID_BIAS)) / (2.0 * float(eps))
    y = orc.binary(op, a, np.ones_like(a), p, p1=HARD_SIGMOID_BIAS)
    np.testing.assert_allclose(y, slope, rtol=2e-3, atol=2e-4)
    if op in ("sigmoid_diff", "tanh_diff"):  # the _op form on the activation's output is the same derivative
        out = orc.unary(fwd, a)
        assert_close(orc.binary(op + "_op", out, np.ones_like(a)), y, op + " through the output", atol=1e-5)


def test_row_products_softmax_derivative_and_diag_accumulation():
    g = rng(81)
    for h, w in ((1, 1), (3, 5), (17, 64), (40, 101), (9, 300)):
        a = g.uniform(-1, 1, (h, w)).astype(np.float32)
        b = g.uniform(-1, 1, (h, w)).astype(np.float32)
        dot = orc.row_dot(a, b)
        assert_close(dot, np.einsum("rc,rc->r", a.astype(np.float64), b), "row dot %s" % ((h, w),))
        y = scipy.special.softmax(a.astype(np.float64), axis=1).astype(np.float32)
        d = orc.softmax_diff_rows(y, b)
        # the Jacobian of softmax, written out: diag(y) - y y^T, applied to the incoming gradient
        want = np.stack([(np.diag(y[r].astype(np.float64)) - np.outer(y[r], y[r])) @ b[r] for r in range(h)])
        assert_close(d, want, "softmax derivative %s" % ((h, w),), atol=1e-6)
        if nhtest.have_reference():
            assert_close(ref().row_dot(a, b), dot, "row dot vs reference")
            assert_close(ref().softmax_diff_rows(y, b), d, "softmax derivative vs reference", atol=1e-6)
    for batch, n, w in ((1, 1, 1), (1, 7, 5), (3, 6, 33), (2, 40, 64)):
        diag = g.uniform(-1, 1, (batch, n)).astype(np.float32)
        m = g.uniform(-1, 1, (batch, n, w)).astype(np.float32)
        start = g.uniform(-1, 1, (n, w)).astype(np.float32)
        got = orc.diag_by_matrix_add(diag, m, start)
        assert_close(got, start + np.einsum("bn,bnw->nw", diag.astype(np.float64), m), "diag accumulate %s" % ((batch, n, w),))
        if nhtest.have_reference():
            assert_close(ref().diag_by_matrix_add(diag, m, start), got, "diag accumulate vs reference")


def test_int_ops_and_conversions():
    g = rng(3)
    a = g.integers(-1000, 1000, 257).astype(np.int32)
    b = g.integers(-1000, 1000, 257).astype(np.int32)
    for op, fn in (("add", np.add), ("sub", np.subtract), ("multiply", np.multiply)):
        assert np.array_equal(orc.binary_int(op, a, b), fn(a, b))
        if nhtest.have_reference():
            assert np.array_equal(ref().binary_int(op, a, b), fn(a, b))
    x = g.uniform(-100, 100, 257).astype(np.float32)
    assert np.array_equal(orc.float_to_int(x), np.trunc(x).astype(np.int32))
    assert np.array_equal(orc.int_to_float(a), a.astype(np.float32))
    if nhtest.have_reference():
        assert np.array_equal(ref().float_to_int(x), orc.float_to_int(x))
        assert np.array_equal(ref().int_to_float(a), orc.int_to_float(a))


def test_sum_and_dot():
    g = rng(4)
    a = g.uniform(-1, 1, 10007).astype(np.float32)
    b = g.uniform(-1, 1, 10007).astype(np.float32)
    assert_close(orc.vector_sum(a), np.sum(a.astype(np.float64)), "sum", atol=1e-4)
    assert_close(orc.dot(a, b), np.dot(a.astype(np.float64), b.astype(np.float64)), "dot", atol=1e-4)
    if nhtest.have_reference():
        assert_close(ref().vector_sum(a), orc.vector_sum(a), "sum vs reference", atol=1e-3)
        assert_close(ref().dot(a, b), orc.dot(a, b), "dot vs reference", atol=1e-3)


# ---------------------------------------------------------------------------------------------------------
# broadcasts, reductions, softmax, arg-max, transpose

def test_broadcasts_and_sums():
    g = rng(5)
    for b, h, w in ((1, 1, 1), (2, 3, 5), (3, 17, 64), (1, 40, 7)):
        m = g.uniform(-10, 10, (b, h, w)).astype(np.float32)
        v = g.uniform(-10, 10, (b, w)).astype(np.float32)
        got = {
            "add_rows": orc.add_vector_to_matrix_rows(m, v),
            "set_rows": orc.set_vector_to_matrix_rows(h, w, v[0]),
            "add_cols": orc.add_vector_to_matrix_columns(m[0], v[0, :1].repeat(h) + np.arange(h, dtype=np.float32)),
            "sub_cols": orc.add_vector_to_matrix_columns(m[0], np.arange(h, dtype=np.float32), sign=-1),
            "sum_rows": orc.sum_matrix_rows(m),
            "sum_rows_add": orc.sum_matrix_rows(m, add_to=v),
            "sum_cols": orc.sum_matrix_columns(m[0]),
            "diag_left": orc.multiply_diag_matrix_by_matrix(np.arange(h, dtype=np.float32) - 1, m[0]),
            "diag_right": orc.batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v, w),
            "diag_right_bcast": orc.batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v[0], 0),
        }
        col = v[0, :1].repeat(h) + np.arange(h, dtype=np.float32)
        want = {
            "add_rows": m + v[:, None, :], "set_rows": np.broadcast_to(v[0], (h, w)),
            "add_cols": m[0] + col[:, None], "sub_cols": m[0] - np.arange(h, dtype=np.float32)[:, None],
            "sum_rows": m.sum(axis=1, dtype=np.float64), "sum_rows_add": v + m.sum(axis=1, dtype=np.float64),
            "sum_cols": m[0].sum(axis=1, dtype=np.float64),
            "diag_left": (np.arange(h, dtype=np.float32) - 1)[:, None] * m[0],
            "diag_right": m * v[:, None, :], "diag_right_bcast": m * v[0][None, None, :],
        }
        for k in got:
            assert_close(got[k], want[k], "%s %s" % (k, (b, h, w)), atol=1e-4)
        if nhtest.have_reference():
            r = ref()
            assert_close(r.add_vector_to_matrix_rows(m, v), got["add_rows"], "add_rows ref")
            assert_close(r.set_vector_to_matrix_rows(h, w, v[0]), got["set_rows"], "set_rows ref")
            assert_close(r.add_vector_to_matrix_columns(m[0], col), got["add_cols"], "add_cols ref")
            assert_close(r.add_vector_to_matrix_columns(m[0], np.arange(h, dtype=np.float32), sign=-1), got["sub_cols"], "sub ref")
            assert_close(r.sum_matrix_rows(m), got["sum_rows"], "sum_rows ref", atol=1e-4)
            assert_close(r.sum_matrix_rows(m, add_to=v), got["sum_rows_add"], "sum_rows_add ref", atol=1e-4)
            assert_close(r.sum_matrix_columns(m[0]), got["sum_cols"], "sum_cols ref", atol=1e-4)
            assert_close(r.multiply_diag_matrix_by_matrix(np.arange(h, dtype=np.float32) - 1, m[0]), got["diag_left"], "diag ref")
            assert_close(r.batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v, w), got["diag_right"], "diagr ref")
            assert_close(r.batch_multiply_matrix_by_diag_matrix(b, m, h, w, h * w, v[0], 0), got["diag_right_bcast"], "diagb ref")


def test_softmax_and_logsumexp():
    g = rng(6)
    for h, w in ((1, 1), (3, 2), (7, 101), (5, 256), (2, 1000), (2, 1500)):
        m = g.uniform(-10, 10, (h, w)).astype(np.float32)
        assert_close(orc.softmax_rows(m), scipy.special.softmax(m.astype(np.float64), axis=1), "softmax %s" % ((h, w),))
        assert_close(orc.log_sum_exp_rows(m), scipy.special.logsumexp(m.astype(np.float64), axis=1), "lse %s" % ((h, w),))
        if nhtest.have_reference():
            assert_close(ref().softmax_rows(m), orc.softmax_rows(m), "softmax ref")
            assert_close(ref().log_sum_exp_rows(m), orc.log_sum_exp_rows(m), "lse ref")
    # rows sum to one; shifting a row by a constant changes nothing
    m = g.uniform(-5, 5, (4, 33)).astype(np.float32)
    assert_close(orc.softmax_rows(m).sum(axis=1), np.ones(4), "row sums")
    assert_close(orc.softmax_rows(m + 3.0), orc.softmax_rows(m), "shift invariance")


def test_argmax_rows_and_columns():
    g = rng(7)
    for h, w in ((1, 1), (5, 3), (64, 101), (9, 257)):
        m = g.permutation(h * w).reshape(h, w).astype(np.float32)  # tie-free
        v, i = orc.find_max_in_rows(m)
        assert np.array_equal(i, np.argmax(m, axis=1)) and np.array_equal(v, m.max(axis=1))
        if nhtest.have_reference():
            rv, ri = ref().find_max_in_rows(m)
            assert np.array_equal(ri, i) and np.array_equal(rv, v)
    m = g.permutation(3 * 17 * 9).reshape(3, 17, 9).astype(np.float32)
    v, i = orc.find_max_in_columns(m)
    assert np.array_equal(i, np.argmax(m, axis=1)) and np.array_equal(v, m.max(axis=1))
    # ties: the first row wins in columns (strict >), the first column wins in rows for the oracle
    t = np.zeros((1, 4, 5), np.float32)
    assert np.array_equal(orc.find_max_in_columns(t)[1], np.zeros((1, 5), np.int32))
    if nhtest.have_reference():
        rv, ri = ref().find_max_in_columns(m)
        assert np.array_equal(ri, i) and np.array_equal(rv, v)
        assert np.array_equal(ref().find_max_in_columns(t)[1], np.zeros((1, 5), np.int32))


def test_transpose():
    g = rng(8)
    for shape in ((1, 1, 1, 1, 1), (2, 3, 1, 5, 1), (2, 4, 3, 5, 2), (1, 1, 3, 4, 2), (3, 7, 1, 1, 4), (2, 16, 1, 8, 64)):
        x = g.uniform(-1, 1, shape).astype(np.float32)
        y = orc.transpose(x)
        assert np.array_equal(y, np.transpose(x, (0, 3, 2, 1, 4)))
        if nhtest.have_reference():
            assert np.array_equal(ref().transpose(x), y), shape


# ---------------------------------------------------------------------------------------------------------
# matrix products

def test_matmul_vs_numpy_and_reference():
    g = rng(9)
    for M, N, K in ((1, 1, 1), (3, 5, 7), (17, 33, 65), (64, 101, 48)):
        a = g.uniform(-1, 1, (M, K + 3)).astype(np.float32)  # strided rows
        b = g.uniform(-1, 1, (N, K + 2)).astype(np.float32)
        out = orc.matmul("nt", a, b, lda=K + 3, ldb=K + 2, ldc=N + 1, M=M, N=N, K=K)
        want = a[:, :K].astype(np.float64) @ b[:, :K].astype(np.float64).T
        got = np.pad(out, (0, M * (N + 1) - out.size)).reshape(M, N + 1)[:, :N]
        assert_close(got, want, "nt %s" % ((M, N, K),))
        if nhtest.have_reference():
            r = ref().matmul("nt", a, b, lda=K + 3, ldb=K + 2, ldc=N + 1, M=M, N=N, K=K)
            assert_close(np.pad(r, (0, M * (N + 1) - r.size)).reshape(M, N + 1)[:, :N], got, "nt ref")
        # accumulate A^T B into C
        at = g.uniform(-1, 1, (K, M + 1)).astype(np.float32)
        bn = g.uniform(-1, 1, (K, N + 2)).astype(np.float32)
        c0 = g.uniform(-1, 1, (M, N)).astype(np.float32)
        out = orc.matmul("tn_add", at, bn, c=c0, lda=M + 1, ldb=N + 2, ldc=N, M=M, N=N, K=K)
        assert_close(out.reshape(M, N), c0 + at[:, :M].astype(np.float64).T @ bn[:, :N].astype(np.float64), "tn_add")
        if nhtest.have_reference():
            r = ref().matmul("tn_add", at, bn, c=c0, lda=M + 1, ldb=N + 2, ldc=N, M=M, N=N, K=K)
            assert_close(r, out, "tn_add ref")
    for batch, M, N, K in ((1, 2, 3, 4), (3, 16, 8, 5), (4, 33, 17, 9)):
        a = g.uniform(-1, 1, (batch, M, K)).astype(np.float32)
        bt = g.uniform(-1, 1, (batch, N, K)).astype(np.float32)
        bn = g.uniform(-1, 1, (batch, K, N)).astype(np.float32)
        at = g.uniform(-1, 1, (batch, K, M)).astype(np.float32)
        cases = {
            "bnt": (a, bt, np.einsum("bmk,bnk->bmn", a.astype(np.float64), bt.astype(np.float64))),
            "bnn": (a, bn, np.einsum("bmk,bkn->bmn", a.astype(np.float64), bn.astype(np.float64))),
            "btn": (at, bn, np.einsum("bkm,bkn->bmn", at.astype(np.float64), bn.astype(np.float64))),
        }
        for kind, (x, y, want) in cases.items():
            got = orc.matmul(kind, x, y, M=M, N=N, K=K, batch=batch)
            assert_close(got, want, kind)
            if nhtest.have_reference():
                assert_close(ref().matmul(kind, x, y, M=M, N=N, K=K, batch=batch), got, kind + " ref")


# ---------------------------------------------------------------------------------------------------------
# convolution (grid after the reference's BlobConvolutionTest: 1x1, strides, dilations, pad > filter, H x 1 images)

CONV_CASES = [
    # n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw
    (1, 1, 1, 1, 1, 1, 1, 0, 0, 1, 1, 1, 1),
    (2, 5, 7, 3, 4, 3, 3, 1, 1, 1, 1, 1, 1),
    (2, 8, 8, 4, 8, 1, 1, 0, 0, 1, 1, 1, 1),
    (1, 9, 11, 5, 6, 3, 2, 2, 1, 2, 3, 1, 1),
    (2, 12, 10, 3, 5, 3, 3, 2, 2, 1, 1, 2, 3),
    (1, 5, 5, 3, 4, 3, 1, 2, 10, 2, 2, 1, 1),  # padding larger than the filter (BlobConvolutionTest.cpp:236-254)
    (1, 5, 5, 3, 4, 3, 3, 2, 10, 2, 2, 1, 1),  # BlobConvolutionTest.cpp:255-273
    (1, 40, 1, 3, 2, 5, 1, 2, 0, 1, 1, 1, 1),
    (3, 14, 14, 16, 24, 5, 5, 2, 2, 2, 2, 1, 1),
    (1, 16, 16, 3, 8, 7, 7, 3, 3, 2, 2, 1, 1),  # the stem shape at small size
    (2, 8, 8, 8, 16, 1, 1, 0, 0, 2, 2, 1, 1),   # 1x1 stride 2 shortcut
]


def conv_via_scipy(x, filt, bias, ph, pw, sh, sw, dh, dw):
    n, h, w, cin = x.shape
    cout, fh, fw, _ = filt.shape
    xp = np.pad(x.astype(np.float64), ((0, 0), (ph, ph), (pw, pw), (0, 0)))
    fd = np.zeros((cout, (fh - 1) * dh + 1, (fw - 1) * dw + 1, cin))
    fd[:, ::dh, ::dw, :] = filt
    outs = []
    for b in range(n):
        per_filter = []
        for co in range(cout):
            acc = sum(scipy.signal.correlate2d(xp[b, :, :, ci], fd[co, :, :, ci], mode="valid") for ci in range(cin))
            per_filter.append(acc[::sh, ::sw])
        outs.append(np.stack(per_filter, axis=-1))
    y = np.stack(outs)
    return y + (0 if bias is None else bias.astype(np.float64))


@pytest.mark.parametrize("case", CONV_CASES)
def test_convolution(case):
    n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw = case
    g = rng(10 + h * w)
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 1, (cout, fh, fw, cin)).astype(np.float32)
    bias = g.uniform(-1, 1, cout).astype(np.float32)
    y = orc.conv(x, f, bias, ph, pw, sh, sw, dh, dw)
    assert_close(y, conv_via_scipy(x, f, bias, ph, pw, sh, sw, dh, dw), "conv %s" % (case,))
    y0 = orc.conv(x, f, None, ph, pw, sh, sw, dh, dw)
    assert_close(y0, y - bias, "conv without free term", atol=1e-4)
    if nhtest.have_reference():
        assert_close(ref().conv(x, f, bias, ph, pw, sh, sw, dh, dw), y, "conv vs reference %s" % (case,))
        assert_close(ref().conv(x, f, None, ph, pw, sh, sw, dh, dw), y0, "conv vs reference, no free term")


@pytest.mark.parametrize("case", CONV_CASES)
def test_convolution_gradients_are_the_adjoints_of_the_forward_pass(case):
    """<conv(x, f), g> is bilinear in (x, f): its gradient by x is conv_backward(g, f), by f is learn(x, g). With the
    forward oracle pinned above, a wrong index, stride or dilation in either gradient breaks one of the identities."""
    n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw = case
    g = rng(20 + h * w)
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 1, (cout, fh, fw, cin)).astype(np.float32)
    y = orc.conv(x, f, None, ph, pw, sh, sw, dh, dw)
    grad = g.uniform(-1, 1, y.shape).astype(np.float32)
    bias = g.uniform(-1, 1, cin).astype(np.float32)
    dx = orc.conv_backward(grad, f, None, x.shape, ph, pw, sh, sw, dh, dw)
    pairing = np.vdot(y.astype(np.float64), grad)
    assert abs(np.vdot(dx.astype(np.float64), x) - pairing) <= 1e-4 * np.abs(y.astype(np.float64) * grad).sum()
    # every component, not only the pairing with x: the forward pass of a unit impulse picks one column of the adjoint
    for _ in range(6):
        at = tuple(g.integers(0, d) for d in x.shape)
        e = np.zeros_like(x)
        e[at] = 1
        assert abs(np.vdot(orc.conv(e, f, None, ph, pw, sh, sw, dh, dw).astype(np.float64), grad) - dx[at]) <= 1e-4 * (1 + abs(dx[at]))
    assert_close(orc.conv_backward(grad, f, bias, x.shape, ph, pw, sh, sw, dh, dw), dx + bias, "free term of the backward pass", atol=1e-5)
    start = g.uniform(-1, 1, f.shape).astype(np.float32)
    df = orc.conv_learn_add(x, grad, start, ph, pw, sh, sw, dh, dw)
    assert abs(np.vdot((df - start).astype(np.float64), f) - pairing) <= 2e-4 * np.abs(y.astype(np.float64) * grad).sum()
    for _ in range(6):
        at = tuple(g.integers(0, d) for d in f.shape)
        e = np.zeros_like(f)
        e[at] = 1
        want = np.vdot(orc.conv(x, e, None, ph, pw, sh, sw, dh, dw).astype(np.float64), grad) + start[at]
        assert abs(want - df[at]) <= 1e-4 * (1 + abs(want))
    if nhtest.have_reference():
        r = ref()
        assert_close(r.conv_backward(grad, f, None, x.shape, ph, pw, sh, sw, dh, dw), dx, "backward vs reference %s" % (case,), atol=1e-4)
        assert_close(r.conv_backward(grad, f, bias, x.shape, ph, pw, sh, sw, dh, dw), dx + bias, "backward + free term vs reference", atol=1e-4)
        ft0 = g.uniform(-1, 1, cout).astype(np.float32)
        rdf, rft = r.conv_learn_add(x, grad, start, ph, pw, sh, sw, dh, dw, free_term_diff=ft0)
        odf, oft = orc.conv_learn_add(x, grad, start, ph, pw, sh, sw, dh, dw, free_term_diff=ft0)
        assert_close(rdf, df, "learn vs reference %s" % (case,), atol=2e-4)
        assert_close(rft, oft, "free term diff vs reference", atol=1e-4)


def test_convolution_1x1_is_a_matrix_product():
    g = rng(11)
    x = g.uniform(-1, 1, (2, 4, 5, 6)).astype(np.float32)
    f = g.normal(0, 1, (7, 1, 1, 6)).astype(np.float32)
    y = orc.conv(x, f, None, 0, 0, 1, 1)
    assert_close(y.reshape(-1, 7), x.reshape(-1, 6).astype(np.float64) @ f.reshape(7, 6).astype(np.float64).T, "1x1")


# (n, h, w, cin, expanded, cout, stride, residual, expand activation, channelwise activation)
SEPARABLE_CASES = [
    (2, 9, 11, 8, 48, 8, 1, True, ("relu", 6.0), ("relu", 6.0)),
    (1, 12, 10, 16, 96, 24, 2, False, ("relu", 0.0), ("hswish", 0.0)),
    (2, 7, 7, 12, 20, 12, 1, True, ("hswish", 0.0), (None, 0.0)),
    (1, 5, 6, 3, 5, 7, 2, False, (None, 0.0), ("relu", 2.5)),       # channel counts not a multiple of 4
    (3, 8, 8, 24, 144, 32, 1, False, ("relu", 6.0), ("relu", 6.0)),
    # few pixels, long reductions, a residual: the down convolution's reduction is cut into slices whose last one adds the input
    (2, 7, 7, 160, 960, 160, 1, True, ("relu", 6.0), ("relu", 6.0)),
    (1, 14, 14, 96, 576, 96, 1, True, ("relu", 6.0), ("relu", 6.0)),
]


def separable_operands(case, with_expand, with_free_terms=True):
    n, h, w, cin, e, cout, stride, residual, ex_act, ch_act = case
    g = rng(40 + h * w + e)
    block_in = cin if with_expand else e
    if not with_expand and residual:
        cout = e
    x = g.uniform(-2, 2, (n, h, w, block_in)).astype(np.float32)
    ft = (lambda k: g.uniform(-0.5, 0.5, k).astype(np.float32)) if with_free_terms else (lambda k: None)
    expand = (g.normal(0, 1.0 / np.sqrt(cin), (e, cin)).astype(np.float32), ft(e), ex_act[0], ex_act[1]) if with_expand else None
    channelwise = (g.normal(0, 0.4, (3, 3, e)).astype(np.float32), ft(e), ch_act[0], ch_act[1])
    down = (g.normal(0, 1.0 / np.sqrt(e), (cout, e)).astype(np.float32), ft(cout))
    return x, expand, channelwise, down, stride, residual


@pytest.mark.parametrize("case", SEPARABLE_CASES)
@pytest.mark.parametrize("with_expand", [True, False])
def test_separable_blocks_against_the_reference_engine(case, with_expand):
    """MobileNetV2Block / ChannelwiseWith1x1: the oracle's stage-by-stage composition against the reference CPU
    engine's fused row-by-row implementation, and against an independent numpy formulation."""
    for with_free_terms in (True, False):
        x, expand, channelwise, down, stride, residual = separable_operands(case, with_expand, with_free_terms)
        y = orc.separable_block(x, expand, channelwise, down, stride, residual)
        # numpy: 1x1 convolutions as matrix products, the depthwise stage per channel through scipy
        def act(t, name, param):
            if name == "relu":
                t = np.maximum(t, 0)
                return np.minimum(t, param) if param > 0 else t
            if name == "hswish":
                return np.where(t <= -3, 0, np.where(t >= 3, t, t * (t + 3) / 6))
            return t
        t = x.astype(np.float64)
        if expand is not None:
            t = act(t @ expand[0].astype(np.float64).T + (0 if expand[1] is None else expand[1]), expand[2], expand[3])
        tp = np.pad(t, ((0, 0), (1, 1), (1, 1), (0, 0)))
        dw = np.stack([np.stack([scipy.signal.correlate2d(tp[b, :, :, c], channelwise[0][:, :, c].astype(np.float64), mode="valid")
                                 [::stride, ::stride] for c in range(t.shape[3])], axis=-1) for b in range(t.shape[0])])
        dw = act(dw + (0 if channelwise[1] is None else channelwise[1]), channelwise[2], channelwise[3])
        want = dw @ down[0].astype(np.float64).T + (0 if down[1] is None else down[1])
        if residual:
            want = want + x
        assert_close(y, want, "separable block %s expand=%s" % (case, with_expand))
        if nhtest.have_reference():
            assert_close(ref().separable_block(x, expand, channelwise, down, stride, residual), y,
                         "separable block vs reference %s expand=%s" % (case, with_expand))
            if residual and with_expand:  # only the MobileNetV2 block is specified to work in place
                assert_close(ref().separable_block(x, expand, channelwise, down, stride, residual, in_place=True), y,
                             "separable block in place vs reference")


# (n, h, w, cin, expanded, cout, filter size, stride, residual, expand activation, channelwise activation, gate activation)
MOBILENETV3_CASES = [
    (2, 9, 11, 8, 48, 8, 3, 1, True, ("hswish", 0.0), ("hswish", 0.0), ("hswish", 0.0)),
    (1, 12, 10, 16, 64, 24, 5, 2, False, ("relu", 0.0), ("relu", 6.0), ("relu", 0.0)),
    (2, 7, 7, 12, 20, 12, 5, 1, True, ("hswish", 0.0), (None, 0.0), (None, 0.0)),
    (1, 6, 5, 3, 5, 7, 3, 2, False, (None, 0.0), ("relu", 2.5), ("hswish", 0.0)),      # channel counts not a multiple of 4
    (3, 14, 14, 40, 240, 40, 5, 1, True, ("hswish", 0.0), ("hswish", 0.0), ("hswish", 0.0)),
]


def mobilenetv3_operands(case):
    n, h, w, cin, e, cout, fsize, stride, residual, ex_act, ch_act, gate_act = case
    g = rng(140 + h * w + e)
    x = g.uniform(-2, 2, (n, h, w, cin)).astype(np.float32)
    ft = lambda k: g.uniform(-0.5, 0.5, k).astype(np.float32)
    expand = (g.normal(0, 1.0 / np.sqrt(cin), (e, cin)).astype(np.float32), ft(e), ex_act[0], ex_act[1])
    channelwise = (g.normal(0, 0.4, (fsize, fsize, e)).astype(np.float32), ft(e), ch_act[0], ch_act[1])
    gate = g.uniform(0, 1, (n, e)).astype(np.float32)  # what the squeeze-and-excite branch's hard sigmoid delivers
    down = (g.normal(0, 1.0 / np.sqrt(e), (cout, e)).astype(np.float32), ft(cout))
    return x, expand, channelwise, gate, down


@needs_ref
@pytest.mark.parametrize("case", MOBILENETV3_CASES)
def test_mobilenetv3_blocks_against_the_reference_engine(case):
    n, h, w, cin, e, cout, fsize, stride, residual, ex_act, ch_act, gate_act = case
    x, expand, channelwise, gate, down = mobilenetv3_operands(case)
    pre = orc.mobilenetv3_pre_se(x, expand, channelwise, stride)
    assert_close(ref().mobilenetv3_pre_se(x, expand, channelwise, stride), pre, "pre-SE %s" % (case,), atol=2e-5)
    assert_close(ref().mobilenetv3_pre_se(x, expand[:1] + (None,) + expand[2:], channelwise[:1] + (None,) + channelwise[2:], stride),
                 orc.mobilenetv3_pre_se(x, expand[:1] + (None,) + expand[2:], channelwise[:1] + (None,) + channelwise[2:], stride),
                 "pre-SE without free terms", atol=2e-5)
    res = x[:, ::stride, ::stride, :][:, :pre.shape[1], :pre.shape[2], :] if residual and stride == 1 and cin == cout else None
    post = orc.mobilenetv3_post_se(pre, gate, res, gate_act[0], gate_act[1], down)
    assert_close(ref().mobilenetv3_post_se(pre, gate, res, gate_act[0], gate_act[1], down), post, "post-SE %s" % (case,), atol=2e-5)
    # numpy for the post-SE half: gate, activation, matrix product, sum
    t = pre.astype(np.float64) * gate.reshape(n, 1, 1, e)
    if gate_act[0] == "relu":
        t = np.clip(t, 0, gate_act[1]) if gate_act[1] > 0 else np.maximum(t, 0)
    elif gate_act[0] == "hswish":
        t = t * np.clip(t + 3, 0, 6) / 6
    want = t @ down[0].astype(np.float64).T + down[1]
    assert_close(post, want + (0 if res is None else res), "post-SE vs numpy", atol=2e-5)


CHANNELWISE_CASES = [
    # n, h, w, c, fh, fw, ph, pw, sh, sw
    (1, 3, 3, 1, 3, 3, 1, 1, 1, 1), (2, 8, 9, 16, 3, 3, 1, 1, 1, 1), (2, 8, 9, 16, 3, 3, 1, 1, 2, 2),
    (1, 7, 7, 5, 3, 3, 0, 0, 1, 1), (1, 10, 12, 12, 5, 5, 2, 2, 1, 1), (3, 9, 6, 7, 2, 3, 1, 2, 2, 1),
]


@pytest.mark.parametrize("case", CHANNELWISE_CASES)
def test_channelwise_convolution(case):
    n, h, w, c, fh, fw, ph, pw, sh, sw = case
    g = rng(12 + c)
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    f = g.normal(0, 1, (fh, fw, c)).astype(np.float32)
    bias = g.uniform(-1, 1, c).astype(np.float32)
    y = orc.channelwise_conv(x, f, bias, ph, pw, sh, sw)
    # every channel is an independent single-channel convolution
    for ch in range(c):
        want = conv_via_scipy(x[..., ch:ch + 1], f[None, :, :, ch:ch + 1], bias[ch:ch + 1], ph, pw, sh, sw, 1, 1)
        assert_close(y[..., ch:ch + 1], want, "channelwise %s ch %d" % (case, ch))
    if nhtest.have_reference():
        assert_close(ref().channelwise_conv(x, f, bias, ph, pw, sh, sw), y, "channelwise vs reference")
        assert_close(ref().channelwise_conv(x, f, None, ph, pw, sh, sw), orc.channelwise_conv(x, f, None, ph, pw, sh, sw), "no ft")


# ---------------------------------------------------------------------------------------------------------
# pooling

@pytest.mark.parametrize("case", CHANNELWISE_CASES)
def test_channelwise_convolution_gradients_are_adjoints(case):
    n, h, w, c, fh, fw, ph, pw, sh, sw = case
    g = rng(112 + c)
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    f = g.normal(0, 1, (fh, fw, c)).astype(np.float32)
    y = orc.channelwise_conv(x, f, None, ph, pw, sh, sw)
    grad = g.uniform(-1, 1, y.shape).astype(np.float32)
    pairing = np.vdot(y.astype(np.float64), grad)
    size = np.abs(y.astype(np.float64) * grad).sum()
    dx = orc.channelwise_conv_backward(grad, f, x.shape, ph, pw, sh, sw)
    assert abs(np.vdot(dx.astype(np.float64), x) - pairing) <= 1e-4 * size
    start, ft0 = g.uniform(-1, 1, f.shape).astype(np.float32), g.uniform(-1, 1, c).astype(np.float32)
    df, dft = orc.channelwise_conv_learn_add(x, grad, start, ph, pw, sh, sw, free_term_diff=ft0)
    assert abs(np.vdot((df - start).astype(np.float64), f) - pairing) <= 1e-4 * size
    assert_close(dft, ft0 + grad.reshape(-1, c).astype(np.float64).sum(axis=0), "free term gradient", atol=1e-5)
    for _ in range(6):  # single components through unit impulses
        at = tuple(g.integers(0, d) for d in x.shape)
        e = np.zeros_like(x)
        e[at] = 1
        assert abs(np.vdot(orc.channelwise_conv(e, f, None, ph, pw, sh, sw).astype(np.float64), grad) - dx[at]) <= 1e-4 * (1 + abs(dx[at]))
        at = tuple(g.integers(0, d) for d in f.shape)
        e = np.zeros_like(f)
        e[at] = 1
        want = np.vdot(orc.channelwise_conv(x, e, None, ph, pw, sh, sw).astype(np.float64), grad) + start[at]
        assert abs(want - df[at]) <= 1e-4 * (1 + abs(want))
    if nhtest.have_reference():
        assert_close(ref().channelwise_conv_backward(grad, f, x.shape, ph, pw, sh, sw), dx, "backward vs reference %s" % (case,), atol=1e-4)
        rdf, rdft = ref().channelwise_conv_learn_add(x, grad, start, ph, pw, sh, sw, free_term_diff=ft0)
        assert_close(rdf, df, "learn vs reference %s" % (case,), atol=1e-4)
        assert_close(rdft, dft, "free term gradient vs reference", atol=1e-4)
        assert_close(ref().channelwise_conv_learn_add(x, grad, start, ph, pw, sh, sw), df, "learn without free term", atol=1e-4)


POOL_CASES = [(1, 2, 2, 1, 2, 2, 2, 2), (2, 9, 11, 5, 3, 3, 2, 2), (1, 8, 8, 16, 2, 2, 2, 2), (2, 7, 10, 3, 3, 2, 1, 3),
              (1, 6, 6, 4, 6, 6, 1, 1), (1, 12, 5, 8, 2, 1, 2, 1)]


def windows(x, fh, fw, sh, sw):
    n, h, w, c = x.shape
    ho, wo = (h - fh) // sh + 1, (w - fw) // sw + 1
    out = np.empty((n, ho, wo, fh, fw, c), x.dtype)
    for y in range(ho):
        for z in range(wo):
            out[:, y, z] = x[:, y * sh:y * sh + fh, z * sw:z * sw + fw, :]
    return out


@pytest.mark.parametrize("case", POOL_CASES)
def test_pooling(case):
    n, h, w, c, fh, fw, sh, sw = case
    g = rng(13 + h)
    x = g.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
    win = windows(x, fh, fw, sh, sw)
    y = orc.max_pool(x, fh, fw, sh, sw)
    assert np.array_equal(y, win.max(axis=(3, 4)))
    assert_close(orc.mean_pool(x, fh, fw, sh, sw), win.astype(np.float64).mean(axis=(3, 4)), "mean")
    yi, idx = orc.max_pool(x, fh, fw, sh, sw, with_indices=True)
    assert np.array_equal(yi, y)
    if nhtest.have_reference():
        assert np.array_equal(ref().max_pool(x, fh, fw, sh, sw), y)
        assert_close(ref().mean_pool(x, fh, fw, sh, sw), orc.mean_pool(x, fh, fw, sh, sw), "mean vs reference")
        ry, ridx = ref().max_pool(x, fh, fw, sh, sw, with_indices=True)
        assert np.array_equal(ry, y)
        assert np.array_equal(ridx, idx), "max-pool indices differ from the reference engine"


def wo_is_one(w, fw, sw):
    return (w - fw) // sw + 1 == 1


@pytest.mark.parametrize("case", POOL_CASES)
def test_pooling_gradients(case):
    n, h, w, c, fh, fw, sh, sw = case
    g = rng(60 + h * w)
    x = g.permutation(n * h * w * c).reshape(n, h, w, c).astype(np.float32)  # distinct values: one maximum per window
    y = orc.mean_pool(x, fh, fw, sh, sw)
    grad = g.uniform(-1, 1, y.shape).astype(np.float32)
    # mean pooling is linear: its gradient is its adjoint
    dmean = orc.mean_pool_backward(x.shape, grad, fh, fw, sh, sw)
    assert abs(np.vdot(dmean.astype(np.float64), x) - np.vdot(y.astype(np.float64), grad)) <= 1e-4 * np.abs(y * grad).sum()
    for _ in range(5):
        at = tuple(g.integers(0, d) for d in x.shape)
        e = np.zeros_like(x)
        e[at] = 1
        assert abs(np.vdot(orc.mean_pool(e, fh, fw, sh, sw), grad) - dmean[at]) <= 1e-5
    # max pooling: a scatter-add of the gradient at the indices the forward pass stored (which follow the reference's
    # CPU engine literally, see the index tests below), restated with numpy's unbuffered add
    dmax = orc.max_pool_backward(x, grad, fh, fw, sh, sw)
    _, idx = orc.max_pool(x, fh, fw, sh, sw, with_indices=True)
    want = np.zeros((n, h * w * c))
    for b in range(n):
        np.add.at(want[b], idx[b].ravel(), grad[b].ravel().astype(np.float64))
    assert_close(dmax, want.reshape(x.shape), "max pooling backward", atol=1e-5)
    if wo_is_one(w, fw, sw):  # windows in the first column: the index is the arg max, the scatter the gradient
        step = g.integers(-3, 4, x.shape).astype(np.float32) / 8  # exact in fp32, below half the gap between values
        moved = orc.max_pool(x + step, fh, fw, sh, sw).astype(np.float64) - orc.max_pool(x, fh, fw, sh, sw)
        assert abs(np.vdot(moved, grad) - np.vdot(dmax.astype(np.float64), step)) <= 1e-5 * np.abs(grad).sum()
    assert abs(dmax.astype(np.float64).sum() - grad.astype(np.float64).sum()) <= 1e-3
    if nhtest.have_reference():
        assert_close(ref().mean_pool_backward(x.shape, grad, fh, fw, sh, sw), dmean, "mean pooling backward vs reference")
        assert_close(ref().max_pool_backward(x, grad, fh, fw, sh, sw), dmax, "max pooling backward vs reference", atol=1e-5)


def test_max_pool_index_first_window_points_at_the_maximum():
    # for the first window of every strip (window column 0) the reference's index is the true arg-max position
    g = rng(14)
    x = g.permutation(2 * 6 * 4 * 3).reshape(2, 6, 4, 3).astype(np.float32)
    y, idx = orc.max_pool(x, 2, 2, 2, 2, with_indices=True)
    flat = x.reshape(2, -1)
    for b in range(2):
        for r in range(y.shape[1]):
            for ch in range(3):
                assert flat[b, idx[b, r, 0, ch]] == y[b, r, 0, ch]


@needs_ref
def test_max_pool_index_ties_match_reference():
    # all-zero windows (common after ReLU) and repeated values
    g = rng(15)
    x = np.maximum(g.uniform(-1, 0.3, (2, 8, 8, 4)), 0).astype(np.float32)
    x = np.round(x * 4) / 4
    for fh, fw, sh, sw in ((2, 2, 2, 2), (3, 3, 2, 2), (3, 3, 1, 1)):
        y, idx = orc.max_pool(x, fh, fw, sh, sw, with_indices=True)
        ry, ridx = ref().max_pool(x, fh, fw, sh, sw, with_indices=True)
        assert np.array_equal(y, ry) and np.array_equal(idx, ridx)


# ---------------------------------------------------------------------------------------------------------
# data movement

def test_resize_image():
    g = rng(16)
    x = g.uniform(-1, 1, (2, 5, 6, 3)).astype(np.float32)
    modes = {0: "constant", 1: "edge", 2: "reflect"}
    for dl, dr, dt, db in ((1, 1, 1, 1), (2, 0, 0, 3), (0, 0, 0, 0), (3, 2, 1, 4)):
        for mode, name in modes.items():
            y = orc.resize_image(x, dl, dr, dt, db, mode, 0.5)
            kw = {"constant_values": 0.5} if mode == 0 else {}
            want = np.pad(x, ((0, 0), (dt, db), (dl, dr), (0, 0)), mode=name, **kw)
            assert np.array_equal(y, want), (dl, dr, dt, db, name)
            if nhtest.have_reference():
                assert np.array_equal(ref().resize_image(x, dl, dr, dt, db, mode, 0.5), y), (dl, dr, dt, db, name)
    # negative deltas crop; mixed crop and pad
    for dl, dr, dt, db in ((-1, -2, -1, 0), (-1, 2, 1, -2)):
        y = orc.resize_image(x, dl, dr, dt, db, 0, -1.0)
        cropped = x[:, max(0, -dt):x.shape[1] - max(0, -db), max(0, -dl):x.shape[2] - max(0, -dr), :]
        want = np.pad(cropped, ((0, 0), (max(dt, 0), max(db, 0)), (max(dl, 0), max(dr, 0)), (0, 0)), constant_values=-1.0)
        assert np.array_equal(y, want)
        if nhtest.have_reference():
            assert np.array_equal(ref().resize_image(x, dl, dr, dt, db, 0, -1.0), y)


BROADCAST_CASES = [
    # from dims, to dims, additional width
    ((1, 1, 1, 1, 1, 1, 1), (2, 3, 1, 4, 5, 1, 6), 1),
    ((1, 3, 1, 1, 1, 1, 6), (1, 3, 1, 4, 5, 1, 6), 1),       # a squeeze-and-excite gate over the pixels
    ((2, 1, 1, 4, 1, 1, 6), (2, 3, 1, 4, 5, 1, 6), 1),
    ((2, 3, 1, 4, 5, 1, 1), (2, 3, 1, 4, 5, 1, 6), 1),
    ((1, 3, 1, 1, 5, 1, 1), (2, 3, 2, 4, 5, 2, 3), 4),
    ((2, 3, 1, 4, 5, 1, 6), (2, 3, 1, 4, 5, 1, 6), 1),       # nothing to broadcast
]


@pytest.mark.parametrize("from_dims,to_dims,width", BROADCAST_CASES)
def test_broadcast_copy(from_dims, to_dims, width):
    g = rng(170 + sum(from_dims))
    x = g.uniform(-1, 1, from_dims + (width,)).astype(np.float32)
    y = orc.broadcast_copy(x, to_dims, width)
    assert np.array_equal(y, np.broadcast_to(x, to_dims + (width,)))
    if nhtest.have_reference():
        assert np.array_equal(ref().broadcast_copy(x, to_dims, width), y)


# blob dims, rate, spatial, batchwise
DROPOUT_CASES = [
    ((1, 4, 1, 1, 1, 1, 10), 0.3, False, False), ((3, 4, 1, 5, 6, 1, 7), 0.5, False, False),
    ((3, 4, 1, 5, 6, 1, 7), 0.5, False, True), ((2, 3, 2, 4, 4, 1, 70), 0.25, True, False),
    ((2, 3, 1, 4, 4, 1, 9), 0.6, True, True), ((1, 2, 1, 1, 1, 1, 1000), 0.1, False, False),
    ((1, 5, 1, 3, 3, 1, 130), 0.4, True, False), ((2, 2, 1, 2, 2, 1, 3), 0.0, False, False),
]


@pytest.mark.parametrize("dims,rate,spatial,batchwise", DROPOUT_CASES)
def test_dropout_draws_the_reference_mask(dims, rate, spatial, batchwise):
    g = rng(180 + sum(dims))
    x = g.uniform(0.5, 1.5, dims).astype(np.float32)
    for seed in (1, 12345, -7):
        y = orc.dropout(x, rate, spatial, batchwise, seed)
        kept = y != 0
        assert np.array_equal(y[kept], (x * np.float32(1.0 / (1.0 - rate)))[kept]) or np.allclose(y[kept], x[kept] / (1 - rate), rtol=1e-6)
        if rate == 0.0:
            assert kept.all()
        # the mask repeats over the outer slices; the spatial one also over the pixels of an object
        objects = dims[0] * dims[1] * dims[2]
        outer = objects if batchwise else dims[0]
        per = kept.reshape(outer, -1)
        assert (per == per[0]).all()
        if spatial:
            pix = kept.reshape(objects, -1, dims[6])
            assert (pix == pix[:, :1, :]).all()
        if nhtest.have_reference():
            assert np.array_equal(ref().dropout(x, rate, spatial, batchwise, seed), y), "mask differs from the reference's"
    if x.size >= 1000 and not spatial:
        frac = np.mean([(orc.dropout(x, rate, spatial, batchwise, s) != 0).mean() for s in range(20)])
        assert abs(frac - (1 - rate)) < 0.03


def test_split_and_merge():
    g = rng(17)
    big = g.uniform(-1, 1, (2, 3, 1, 4, 5, 1, 12)).astype(np.float32)
    for dim, sizes in ((6, (4, 8)), (6, (3, 4, 5)), (4, (2, 3)), (3, (1, 3)), (0, (1, 1)), (1, (2, 1))):
        part_dims = []
        for s in sizes:
            d = list(big.shape)
            d[dim] = s
            part_dims.append(tuple(d))
        parts = orc.split(big, dim, part_dims)
        want = np.split(big, np.cumsum(sizes)[:-1], axis=dim)
        for p, wnt in zip(parts, want):
            assert np.array_equal(p, wnt), (dim, sizes)
        assert np.array_equal(orc.merge(parts, dim, big.shape), big)
        if nhtest.have_reference():
            for p, q in zip(ref().split(big, dim, part_dims), parts):
                assert np.array_equal(p, q)
            assert np.array_equal(ref().merge(parts, dim, big.shape), big)


# ---------------------------------------------------------------------------------------------------------
# LSTM and CTC

def lstm_numpy(w_in, b_in, w_rec, b_rec, x, reverse, c0, h0):
    T, B, In = x.shape
    H = w_rec.shape[1]
    c = np.zeros((B, H)) if c0 is None else c0.astype(np.float64)
    h = np.zeros((B, H)) if h0 is None else h0.astype(np.float64)
    hs, cs = np.zeros((T, B, H)), np.zeros((T, B, H))
    bias = (0 if b_in is None else b_in.astype(np.float64)) + (0 if b_rec is None else b_rec.astype(np.float64))
    for i in range(T):
        t = T - 1 - i if reverse else i
        g = x[t].astype(np.float64) @ w_in.astype(np.float64).T + h @ w_rec.astype(np.float64).T + bias
        a, f, inp, o = g[:, :H], g[:, H:2 * H], g[:, 2 * H:3 * H], g[:, 3 * H:]
        c = scipy.special.expit(f) * c + scipy.special.expit(inp) * np.tanh(a)
        h = scipy.special.expit(o) * np.tanh(c)
        hs[t], cs[t] = h, c
    return hs, cs


@pytest.mark.parametrize("reverse", [False, True])
@pytest.mark.parametrize("with_init", [False, True])
def test_lstm(reverse, with_init):
    g = rng(18)
    T, B, In, H = 5, 3, 6, 4
    w_in = g.uniform(-0.5, 0.5, (4 * H, In)).astype(np.float32)
    w_rec = g.uniform(-0.5, 0.5, (4 * H, H)).astype(np.float32)
    b_in = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
    b_rec = g.uniform(-0.5, 0.5, 4 * H).astype(np.float32)
    x = g.uniform(-1, 1, (T, B, In)).astype(np.float32)
    c0 = g.uniform(-1, 1, (B, H)).astype(np.float32) if with_init else None
    h0 = g.uniform(-1, 1, (B, H)).astype(np.float32) if with_init else None
    for bi, br in ((b_in, b_rec), (b_in, None), (None, None)):
        h, c = orc.lstm(w_in, bi, w_rec, br, x, reverse, c0, h0)
        wh, wc = lstm_numpy(w_in, bi, w_rec, br, x, reverse, c0, h0)
        assert_close(h, wh, "lstm h")
        assert_close(c, wc, "lstm c")
        if nhtest.have_reference():
            rh, rc = ref().lstm(w_in, bi, w_rec, br, x, reverse, c0, h0)
            assert_close(rh, h, "lstm h vs reference")
            assert_close(rc, c, "lstm c vs reference")
            rh2, _ = ref().lstm(w_in, bi, w_rec, br, x, reverse, c0, h0, want_state=False)
            assert_close(rh2, h, "lstm h vs reference without state output")


def test_ctc_greedy_collapse():
    labels = np.array([[0, 0, 5, 1, 1, 5, 1, 2, 2, 5], [5, 5, 5, 5, 5, 5, 5, 5, 5, 5], [3, 5, 3, 3, 5, 5, 4, 4, 4, 0]], np.int32)
    got = nhtest.ctc_greedy_collapse(labels, blank=5)
    assert got == [[0, 1, 1, 2], [], [3, 3, 4, 0]]
    assert nhtest.ctc_greedy_collapse(labels, blank=5, seq_len=[3, 10, 4]) == [[0], [], [3, 3]]
    # brute force: itertools.groupby then drop blanks
    import itertools
    g = rng(19)
    rnd = g.integers(0, 4, (6, 40)).astype(np.int32)
    want = [[k for k, _ in itertools.groupby(row.tolist()) if k != 3] for row in rnd]
    assert nhtest.ctc_greedy_collapse(rnd, blank=3) == want
