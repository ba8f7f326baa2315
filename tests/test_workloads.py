"""Whole-network parity of the five benchmark configurations, written once as engine-call sequences
(neoml_amd/workloads.py) and executed by three backends: the C oracle, the reference's CPU engine, and the HIP
library through its C ABI.

CPU tests: oracle against the reference engine on small instances (pins the oracle's composition of ops).
GPU tests: HIP path against the reference engine (the oracle when the reference build is absent) on reduced
instances of the same architectures, fp32 within |a-b| <= 1e-5 + 1e-4 |b|, integer labels bit-exact.
"""
import numpy as np
import pytest

import nhtest
from nhtest import assert_close, CpuBackend
from neoml_amd.workloads import ResNet18, MobileNetV2, TransformerEncoder, LineRecognizer

needs_ref = pytest.mark.skipif(not nhtest.have_reference(), reason="reference CPU engine not built (oracle/_ref)")


def checker():
    return CpuBackend("ref" if nhtest.have_reference() else "orc")


SMALL = {
    "resnet": lambda be: ResNet18(be, batch=1, image=32, classes=10, width_scale=0.125),
    "resnet_fused": lambda be: ResNet18(be, batch=1, image=32, classes=10, width_scale=0.125, fused=True),
    "mobilenet": lambda be: MobileNetV2(be, batch=1, image=32, classes=10, head=64),
    "mobilenet_fused": lambda be: MobileNetV2(be, batch=1, image=32, classes=10, head=64, fused=True),
    "transformer": lambda be: TransformerEncoder(be, layers=1, d_model=32, heads=4, ffn=64, seq=8, batch=2),
    "recognizer": lambda be: LineRecognizer(be, batch=2, width=32, hidden=16, classes=10),
}

REDUCED = {
    "resnet": lambda be: ResNet18(be, batch=2, image=96, classes=100, width_scale=0.5),
    "resnet_fused": lambda be: ResNet18(be, batch=2, image=96, classes=100, width_scale=0.5, fused=True),
    "mobilenet": lambda be: MobileNetV2(be, batch=2, image=96, classes=100, head=320),
    "mobilenet_fused": lambda be: MobileNetV2(be, batch=2, image=96, classes=100, head=320, fused=True),
    "transformer": lambda be: TransformerEncoder(be, layers=2, d_model=128, heads=4, ffn=512, seq=64, batch=4),
    "recognizer": lambda be: LineRecognizer(be, batch=4, width=128, hidden=64, classes=100),
}


def run(make, backend):
    net = make(backend)
    out = net.forward(backend.tensor(net.make_input()))
    if isinstance(out, tuple):
        return tuple(np.asarray(backend.to_numpy(o)) for o in out)
    return np.asarray(backend.to_numpy(out))


def labels_agree(labels_a, logp_a, labels_b, logp_b):
    """Arg-max labels must be identical wherever the checker's top two log-probabilities are further apart than the
    fp32 tolerance allows the two paths to differ; a closer pair is a legitimate tie-break difference."""
    top2 = np.sort(logp_b, axis=1)[:, -2:]
    decided = (top2[:, 1] - top2[:, 0]) > 2e-4 * np.maximum(1.0, np.abs(top2[:, 1]))
    a, b = labels_a.ravel(), labels_b.ravel()
    assert decided.mean() > 0.9, "test input has too many near-ties to be meaningful"
    assert np.array_equal(a[decided], b[decided])


@needs_ref
@pytest.mark.parametrize("name", sorted(SMALL))
def test_oracle_matches_reference_engine(name):
    got = run(SMALL[name], CpuBackend("orc"))
    want = run(SMALL[name], CpuBackend("ref"))
    if name == "recognizer":
        assert_close(got[1], want[1], name)
        labels_agree(got[0], got[1], want[0], want[1])
    else:
        assert_close(got, want, name)


def test_recognizer_ctc_collapse_on_oracle_labels():
    labels, _ = run(SMALL["recognizer"], CpuBackend("orc"))
    seqs = nhtest.ctc_greedy_collapse(labels, blank=10)
    for row, seq in zip(labels, seqs):
        expect, prev = [], -1
        for v in row:
            if v != prev and v != 10:
                expect.append(int(v))
            prev = v
        assert seq == expect


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(REDUCED))
def test_hip_matches_cpu_engine(name):
    from neoml_amd.workloads import HipBackend
    got = run(REDUCED[name], HipBackend())
    want = run(REDUCED[name], checker())
    if name == "recognizer":
        assert_close(got[1], want[1], name)
        labels_agree(got[0], got[1], want[0], want[1])
    else:
        assert_close(got, want, name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(REDUCED))
def test_replayed_plan_reproduces_forward(name):
    """The recorded launch list that the benchmark replays computes the same result as the direct pass."""
    from neoml_amd.workloads import HipBackend
    be = HipBackend()
    net = REDUCED[name](be)
    x = be.tensor(net.make_input())
    direct = net.forward(x)
    direct = [be.to_numpy(o).copy() for o in (direct if isinstance(direct, tuple) else (direct,))]
    plan, out = net.record_plan(x)
    for _ in range(3):
        plan.run()
    be.synchronize()
    replay = [be.to_numpy(o) for o in (out if isinstance(out, tuple) else (out,))]
    for a, b in zip(replay, direct):
        if a.dtype == np.int32:
            assert np.array_equal(a, b)
        else:
            # split-K accumulates with float atomics: runs agree to rounding, not bit for bit
            assert_close(a, b, name)
