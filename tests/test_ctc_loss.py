"""IMathEngine::CtcLossForward (NeoMathEngine.h:1033-1036; src/CPU/CpuMathEngineDnnCtc.cpp:202-403).

The checker is the reference's own CPU engine (oracle/_ref) through the engine shim. On the CPU it is pinned first: its
loss must equal minus the log of the summed probability of every frame-by-frame path that collapses to the labels, found
by enumerating all paths of a small case, and its gradient must equal central differences of that loss. On the GPU the
HIP engine runs the same calls and must agree with it (loss and gradient) within |a - b| <= 1e-5 + 1e-4 |b|.
"""
import ctypes
import itertools

import numpy as np
import pytest

import nhtest
from nhtest import assert_close, fp

needs_ref = pytest.mark.skipif(not nhtest.have_reference(), reason="reference build (oracle/_ref) not present")


def ip(a):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ctypes.c_int))


def ctc_loss(engine, result, labels, blank, skip_blanks, label_lens=None, result_lens=None, weights=None, with_gradient=True):
    """result [T][B][C] (before the softmax), labels [L][B] -> (loss, gradient [T][B][C] or None)"""
    s = nhtest.shim()
    result = np.ascontiguousarray(result, np.float32)
    labels = np.ascontiguousarray(labels, np.int32)
    T, B, C = result.shape
    L = labels.shape[0]
    i32 = lambda a: None if a is None else np.ascontiguousarray(a, np.int32)
    label_lens, result_lens = i32(label_lens), i32(result_lens)
    weights = None if weights is None else np.ascontiguousarray(weights, np.float32)
    loss = np.zeros(1, np.float32)
    grad = np.zeros_like(result) if with_gradient else None
    rc = s.shim_ctc_loss_forward(engine, T, B, C, L, blank, 1 if skip_blanks else 0, fp(result), ip(labels), ip(label_lens),
                                 ip(result_lens), None if weights is None else fp(weights), fp(loss),
                                 None if grad is None else fp(grad))
    assert rc == 0, s.shim_last_error()
    return float(loss[0]), grad


def collapse(path, blank):
    out, previous = [], None
    for k in path:
        if k != previous and k != blank:
            out.append(k)
        previous = k
    return out


def brute_force_loss(result, labels, blank, skip_blanks):
    """- mean over the batch of log( sum over all paths of the product of frame probabilities ). skip_blanks = False is the
    reference's stricter lattice: two different labels must be separated by a blank as well (a path that steps from a label
    straight to the next one does not count)."""
    T, B, C = result.shape
    e = np.exp(result.astype(np.float64) - result.max(axis=2, keepdims=True))
    prob = e / e.sum(axis=2, keepdims=True)
    total = 0.0
    for b in range(B):
        want = [int(v) for v in labels[:, b]]
        p = 0.0
        for path in itertools.product(range(C), repeat=T):
            if collapse(path, blank) != want:
                continue
            if not skip_blanks and any(a != blank and c != blank and a != c for a, c in zip(path, path[1:])):
                continue
            p += float(np.prod([prob[t, b, k] for t, k in enumerate(path)]))
        total += np.log(p)
    return -total / B


@needs_ref
@pytest.mark.parametrize("skip_blanks", [True, False])
def test_reference_ctc_loss_is_the_sum_over_paths(skip_blanks):
    g = np.random.default_rng(5)
    T, B, C, L, blank = 5, 2, 3, 2, 0
    result = g.normal(0, 1, (T, B, C)).astype(np.float32)
    labels = np.array([[1, 2], [2, 2]], np.int32)  # sequence 0: 1 2, sequence 1: 2 2 (a repeated label needs its blank)
    loss, grad = ctc_loss(nhtest.cpu_engine(), result, labels, blank, skip_blanks)
    assert abs(loss - brute_force_loss(result, labels, blank, skip_blanks)) < 1e-4
    # the gradient is the loss's, up to the factor 1 / batch that the loss layer applies
    eps = 1e-2
    for (t, b, k) in [(0, 0, 1), (2, 1, 0), (4, 1, 2), (3, 0, 2)]:
        up, down = result.copy(), result.copy()
        up[t, b, k] += eps
        down[t, b, k] -= eps
        slope = (brute_force_loss(up, labels, blank, skip_blanks) - brute_force_loss(down, labels, blank, skip_blanks)) / (2 * eps)
        assert abs(grad[t, b, k] / B - slope) < 2e-3, (t, b, k, grad[t, b, k] / B, slope)


CASES = [
    # T, B, C, L, blank, skip_blanks, label_lens, result_lens, weights
    (12, 3, 6, 4, 0, True, False, False, False),
    (12, 3, 6, 4, 5, False, False, False, False),
    (20, 5, 11, 6, 10, True, True, False, True),
    (20, 5, 11, 6, 10, False, True, True, False),
    (33, 4, 40, 9, 0, True, True, True, True),
    (128, 8, 101, 20, 100, True, True, True, False),   # the line recogniser's shape at a reduced batch
    (64, 2, 30, 140, 0, True, False, False, False),    # more lattice positions than threads of a workgroup, no labelling fits
]


@pytest.mark.gpu
@needs_ref
@pytest.mark.parametrize("case", CASES)
def test_ctc_loss_on_hip_engine_follows_the_cpu_engine(case):
    T, B, C, L, blank, skip_blanks, with_label_lens, with_result_lens, with_weights = case
    g = np.random.default_rng(sum(case[:5]))
    result = g.normal(0, 2, (T, B, C)).astype(np.float32)
    classes = [k for k in range(C) if k != blank]
    labels = g.choice(classes, size=(L, B)).astype(np.int32) if L > 0 else np.zeros((0, B), np.int32)
    label_lens = g.integers(1, L + 1, B).astype(np.int32) if with_label_lens else None
    result_lens = g.integers(max(1, T - 5), T + 1, B).astype(np.int32) if with_result_lens else None
    weights = g.uniform(0.5, 2.0, B).astype(np.float32) if with_weights else None
    want_loss, want_grad = ctc_loss(nhtest.cpu_engine(), result, labels, blank, skip_blanks, label_lens, result_lens, weights)
    got_loss, got_grad = ctc_loss(nhtest.hip_engine(), result, labels, blank, skip_blanks, label_lens, result_lens, weights)
    assert_close(np.float32(got_loss), np.float32(want_loss), "loss %s" % (case,))
    assert_close(got_grad, want_grad, "gradient %s" % (case,))
    only_loss, none = ctc_loss(nhtest.hip_engine(), result, labels, blank, skip_blanks, label_lens, result_lens, weights,
                               with_gradient=False)
    assert none is None and only_loss == got_loss
