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


def test_no_alloc_convolution_leaves_device_memory_as_it_is():
    """The property itself: a warm call allocates nothing on the device. hipMemGetInfo (through torch) reports the same free
    bytes before and after, with torch's caching allocator out of the picture (the buffers exist before the first reading,
    nothing of torch's is allocated or freed in between), and the library's own per-stream scratch does not grow."""
    import torch
    hip = nhtest.Hip()
    x, f, bias = _inputs(0xA1111, 64, 7, 7, 512, 512, 3)
    d = hip.conv_desc(64, 7, 7, 512, 512, 3, 3, 1, 1, 1, 1)
    xs, fs, bs = hip.up(x), hip.up(f), hip.up(bias)
    out = hip.empty((64, d.resultHeight, d.resultWidth, 512))
    call = lambda: hip.call("nhBlobConvolutionNoAlloc", ctypes.byref(d), hip.p(xs), hip.p(fs), hip.p(bs), hip.p(out))
    call()  # the first call on a device looks the array's address up
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    for _ in range(3):
        call()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_reserved() == reserved_before
    assert free_after == free_before, "device memory in use changed by %d bytes across nhBlobConvolutionNoAlloc" % (free_before - free_after)


def test_no_alloc_convolution_refuses_what_does_not_fit_its_array():
    """K slices whose partial tiles exceed the fixed array (sliced tiles x slices x 16 KiB > 64 MiB): NH_ERR_ARGUMENT with a
    message that names the limit, and nothing launched: the result buffer keeps its contents. How many slices a launch
    takes is the launch planner's decision, so a few shapes with many tiles and long reductions are tried."""
    import neoml_amd
    hip = nhtest.Hip()
    g = np.random.default_rng(5)
    refused = 0
    for n, h, w, cin, cout in [(144, 7, 7, 1024, 512), (200, 7, 7, 512, 320), (100, 7, 7, 2048, 640), (250, 5, 5, 1024, 512)]:
        d = hip.conv_desc(n, h, w, cin, cout, 3, 3, 1, 1, 1, 1)
        xs = hip.up(g.uniform(-1, 1, (n, h, w, cin)).astype(np.float32))
        fs = hip.up(g.normal(0, 0.01, (cout, 3, 3, cin)).astype(np.float32))
        out = hip.empty((n, d.resultHeight, d.resultWidth, cout))
        out.fill_(7.0)
        rc = hip.lib.nhBlobConvolutionNoAlloc(hip.stream(), ctypes.byref(d), hip.p(xs), hip.p(fs), None, hip.p(out))
        if rc != 0:
            refused += 1
            assert "fixed scratch" in neoml_amd.last_error()
            assert (hip.down(out) == 7.0).all()
    if refused == 0:
        pytest.skip("none of the shapes tried was cut into more slices than the fixed array holds")
