"""nhBlobConvolutionNoAlloc: the convolution entry point that allocates no device memory (its K slices meet in a fixed
array inside the library instead of a block allocated per stream) against nhBlobConvolution on the same inputs.

Runs last in the suite (the file name sorts behind the others): it must pass both alone in a fresh process and after
every other test has used the library."""
import ctypes

import numpy as np
import pytest

import nhtest

pytestmark = pytest.mark.gpu


def _both(hip, x, f, bias, pad, stride):
    """(result of nhBlobConvolutionNoAlloc, result of nhBlobConvolution) on the same device buffers."""
    n, h, w, cin = x.shape
    cout, fh, fw, _ = f.shape
    d = hip.conv_desc(n, h, w, cin, cout, fh, fw, pad, pad, stride, stride)
    xs, fs, bs = hip.up(x), hip.up(f), hip.up(bias)
    out_fixed = hip.empty((n, d.resultHeight, d.resultWidth, cout))
    out_plain = hip.empty((n, d.resultHeight, d.resultWidth, cout))
    out_fixed.fill_(float("nan"))
    out_plain.fill_(float("nan"))
    hip.call("nhBlobConvolutionNoAlloc", ctypes.byref(d), hip.p(xs), hip.p(fs), hip.p(bs), hip.p(out_fixed))
    hip.call("nhBlobConvolution", ctypes.byref(d), hip.p(xs), hip.p(fs), hip.p(bs), hip.p(out_plain))
    return hip.down(out_fixed), hip.down(out_plain)


def _inputs(seed, n, h, w, cin, cout, k):
    g = np.random.default_rng(seed)
    x = g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    f = g.normal(0, 1.0 / np.sqrt(k * k * cin), (cout, k, k, cin)).astype(np.float32)
    bias = g.uniform(-0.5, 0.5, cout).astype(np.float32)
    return x, f, bias


def test_no_alloc_convolution_matches_the_allocating_entry_point_twice_in_a_row():
    hip = nhtest.Hip()
    orc = nhtest.Cpu("orc")
    # first call: 392 tiles x 288 K steps, cut into K slices that meet in the fixed array (the last ResNet-18 stage);
    # second call, right behind it: a smaller input whose slices reuse the front of the same array
    cases = [(0xA110C, 64, 7, 7, 512, 512, 3, 1, 1), (0xA110D, 16, 7, 7, 256, 512, 3, 1, 1)]
    for seed, n, h, w, cin, cout, k, pad, stride in cases:
        x, f, bias = _inputs(seed, n, h, w, cin, cout, k)
        fixed, plain = _both(hip, x, f, bias, pad, stride)
        assert np.isfinite(fixed).all()
        # the same kernels and the same summation order: the bar of the fp32 tolerance, and in fact equal bits
        nhtest.assert_close(fixed, plain, "no-alloc vs allocating convolution, batch %d" % n)
        assert np.array_equal(fixed, plain)
        if n <= 16:
            want = orc.conv(x, f, bias, pad, pad, stride, stride)
            nhtest.assert_close(fixed.reshape(want.shape), want, "no-alloc convolution vs the oracle, batch %d" % n)


def test_no_alloc_convolution_without_slices_and_with_a_tail():
    hip = nhtest.Hip()
    # no K slices at all (many tiles, short reduction), then the tiles behind the last whole round cut into slices
    for seed, n, h, w, cin, cout, k in [(0xA110E, 8, 56, 56, 64, 64, 3), (0xA110F, 64, 28, 28, 128, 128, 3),
                                       (0xA1110, 4, 28, 28, 32, 16, 1)]:
        x, f, bias = _inputs(seed, n, h, w, cin, cout, k)
        fixed, plain = _both(hip, x, f, bias, k // 2, 1)
        nhtest.assert_close(fixed, plain, "no-alloc vs allocating convolution %dx%dx%d" % (h, w, cin))
        assert np.array_equal(fixed, plain)
