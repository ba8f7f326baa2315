"""NeoMathEngine's own test suite (NeoMathEngine/test/src/inference and learn, 180 source files, 522 test cases) against
the engines: oracle/_ref/me_tests is those sources compiled where they lie against tests/ref_suite (a small framework
with the Google Test vocabulary they use, and a fixture that can hand them the HIP engine; built by oracle/Makefile).

On the CPU: the suite runs against the reference's own CPU engine, which checks the framework and the build.
On the GPU: the same executable with --MathEngine=hip. Every case must pass, or end in the engine's "is not implemented
by CHipMathEngine" assertion (the four members left out are asserting stubs, the reference GPU engine's own convention;
none of the cases that run here reaches one); the counts of both are printed.
"""
import os
import re
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
BINARY = os.path.join(ROOT, "oracle", "_ref", "me_tests")

# One case of the reference's suite computes its expectation with a quadratic loop over 2.6 M elements (16 minutes on the
# host, whatever the engine).
SLOW = "*GlobalMaxPoolingTest.Random/5"
# The dropout test expects, from an engine whose GetType() is not MET_Cpu, the mask layout of the reference's CUDA engine
# in spatial mode (NeoMathEngine/test/src/inference/DropoutTest.cpp:48-55); the HIP engine reproduces the CPU engine's
# layout there (rows of the mask padded to four values, CpuMathEngineDnnDropout.cpp), which is what parity with the CPU
# engine asks for. Its non-spatial cases are covered by tests/test_hip_parity.py against the CPU engine bit for bit.
ENGINE_TYPE_DEPENDENT = "*CMathEngineDropoutTest*"
# The two factorization tests fail on the reference's own CPU engine as built here (no MKL: its LU/QR need it).
NEEDS_MKL = "CMathEngineLUFactorizationTest*:CMathEngineQRFactorizationTest*"

NOT_IMPLEMENTED = re.compile(r'exception thrown in the test body: !"(\w+) is not implemented by CHipMathEngine"')


def _run(args, timeout):
    res = subprocess.run([BINARY] + args, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout,
                         errors="replace")
    return res.returncode, res.stdout


def _cases(out):
    """name -> (ok, text printed while the case ran)"""
    cases, name, buf = {}, None, []
    for line in out.splitlines():
        m = re.match(r"\[ RUN      \] (\S+)", line)
        if m:
            name, buf = m.group(1), []
        elif name and line.startswith("[       OK ]"):
            cases[name], name = (True, ""), None
        elif name and line.startswith("[  FAILED  ]"):
            cases[name], name = (False, "\n".join(buf)), None
        elif name:
            buf.append(line)
    return cases


needs_binary = pytest.mark.skipif(not os.path.exists(BINARY), reason="oracle/_ref/me_tests is not built (needs the reference sources)")


@needs_binary
def test_reference_suite_lists_its_cases():
    rc, out = _run(["--MathEngine=cpu", "--gtest_list_tests"], 60)
    assert rc == 0
    names = [l for l in out.splitlines() if "." in l and not l.startswith("[")]
    assert len(names) >= 500, len(names)
    # the four operations the suite was asked for first
    for suite in ("CMathEngineBlobConvolutionTest", "CMathEngineBlobChannelwiseConvolutionTest", "CMultiplyMatrixByTransposedMatrixTest",
                  "CMathEngineMaxPoolingTest"):
        assert any(suite in n for n in names), suite


@needs_binary
def test_reference_suite_passes_on_the_reference_cpu_engine():
    rc, out = _run(["--MathEngine=cpu", "--gtest_filter=-%s:%s" % (SLOW, NEEDS_MKL)], 900)
    cases = _cases(out)
    failed = sorted(n for n, (ok, _) in cases.items() if not ok)
    assert not failed, failed[:10]
    assert rc == 0 and len(cases) >= 500, (rc, len(cases))


@needs_binary
@pytest.mark.gpu
def test_reference_suite_on_the_hip_engine(capsys):
    rc, out = _run(["--MathEngine=hip", "--gtest_filter=-%s:%s:%s" % (SLOW, NEEDS_MKL, ENGINE_TYPE_DEPENDENT)], 900)
    cases = _cases(out)
    assert len(cases) >= 500, (rc, len(cases), out[-2000:])
    passed = sorted(n for n, (ok, _) in cases.items() if ok)
    missing, wrong = {}, []
    for name, (ok, text) in cases.items():
        if ok:
            continue
        m = NOT_IMPLEMENTED.search(text)
        # a case that only hit a stub printed nothing else but that exception
        if m and text.count("Failure") == 1:
            missing.setdefault(m.group(1), []).append(name)
        else:
            wrong.append((name, text[:600]))
    with capsys.disabled():
        print("\nreference suite on CHipMathEngine: %d cases passed, %d ended in a not-implemented stub (%d operations: %s)" % (
            len(passed), sum(len(v) for v in missing.values()), len(missing), ", ".join(sorted(missing))))
    assert not wrong, wrong[:5]
    # what the built path covers must stay covered
    assert len(passed) >= 518 and not missing, (len(passed), missing)
    for suite in ("CMathEngineBlobConvolutionTest", "CMathEngineBlobChannelwiseConvolutionTest", "CMultiplyMatrixByTransposedMatrixTest",
                  "CMathEngineMaxPoolingTest", "CMathEngineMeanPoolingTest", "CMathEngineBlobConvolutionBackwardTest",
                  "CMatrixSoftmaxByRowsTest", "CMathEngineFindMaxValueInRowsTest"):
        mine = [n for n in cases if suite in n]
        assert mine and all(cases[n][0] for n in mine), (suite, mine[:3])
