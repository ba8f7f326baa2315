"""CPU-side checks of the C ABI: the library loads without a GPU, exports every declared symbol, and the host
logic (argument validation, descriptor arithmetic, the caching allocator on host memory) behaves as specified."""
import ctypes
import re
import threading

import pytest

import neoml_amd


def test_library_exports_every_declared_symbol():
    fns = neoml_amd.declared_functions()
    assert len(fns) > 100
    raw = ctypes.CDLL(neoml_amd.LIB_PATH)
    missing = [n for n in fns if not hasattr(raw, n)]
    assert not missing, missing
    # every declaration cites the interface line it replaces or documents itself
    text = open(neoml_amd.HEADER_PATH).read()
    assert len(re.findall(r"NME\.h:\d+", text)) > 90


def test_error_codes_and_messages_without_gpu():
    lib = neoml_amd.load()
    assert lib.nhVectorAdd(None, None, None, None, -5) == 1
    assert "negative" in neoml_amd.last_error()
    d = neoml_amd.ConvDesc(1, 4, 4, 3, 2, 5, 5, 0, 0, 1, 1, 1, 1, 0, 0)
    assert lib.nhInitBlobConvolution(ctypes.byref(d)) == 1
    with pytest.raises(neoml_amd.NeoMLHipError):
        neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
    n = ctypes.c_int(-1)
    assert lib.nhGetDeviceCount(ctypes.byref(n)) == 0 and n.value >= 0


@pytest.mark.parametrize("h,w,fh,fw,ph,pw,sh,sw,dh,dw", [
    (32, 32, 3, 3, 1, 1, 1, 1, 1, 1), (224, 224, 7, 7, 3, 3, 2, 2, 1, 1), (56, 56, 1, 1, 0, 0, 2, 2, 1, 1),
    (12, 10, 3, 3, 2, 2, 1, 1, 2, 3), (5, 5, 3, 1, 2, 10, 2, 2, 1, 1)])
def test_convolution_descriptor_matches_reference_formula(h, w, fh, fw, ph, pw, sh, sw, dh, dw):
    # Hout = 1 + ( H - ( fh - 1 ) * dh + 2 * ph - 1 ) / sh  (src/CPU/CpuMathEngineDnnConv.cpp:59-62)
    lib = neoml_amd.load()
    d = neoml_amd.ConvDesc(2, h, w, 3, 8, fh, fw, ph, pw, sh, sw, dh, dw, 0, 0)
    neoml_amd.check(lib.nhInitBlobConvolution(ctypes.byref(d)))
    assert d.resultHeight == 1 + (h - (fh - 1) * dh + 2 * ph - 1) // sh
    assert d.resultWidth == 1 + (w - (fw - 1) * dw + 2 * pw - 1) // sw


def test_pooling_and_channelwise_descriptors():
    lib = neoml_amd.load()
    p = neoml_amd.PoolingDesc(64, 114, 114, 64, 3, 3, 2, 2, 0, 0)
    neoml_amd.check(lib.nhInitPooling(ctypes.byref(p)))
    assert (p.resultHeight, p.resultWidth) == (56, 56)
    p = neoml_amd.PoolingDesc(1, 2, 2, 1, 3, 3, 1, 1, 0, 0)
    assert lib.nhInitPooling(ctypes.byref(p)) == 1
    c = neoml_amd.ConvDesc(1, 112, 112, 96, 0, 3, 3, 1, 1, 2, 2, 0, 0, 0, 0)
    neoml_amd.check(lib.nhInitBlobChannelwiseConvolution(ctypes.byref(c)))
    assert (c.resultHeight, c.resultWidth, c.filterCount) == (56, 56, 96)
    c = neoml_amd.ConvDesc(1, 8, 8, 4, 0, 3, 3, 3, 1, 1, 1, 0, 0, 0, 0)  # padding must be smaller than the filter
    assert lib.nhInitBlobChannelwiseConvolution(ctypes.byref(c)) == 1


def test_lstm_workspace_size():
    lib = neoml_amd.load()
    size = ctypes.c_size_t(0)
    neoml_amd.check(lib.nhLstmWorkspaceSize(256, 512, 128, 64, ctypes.byref(size)))
    # gates for every step, summed free term, one step of cell state, two sets of two exchange buffers of 64-bit words
    # ( one that every XCD sees, one for readers on the writer's XCD ), the per-XCD role counters, the abort word
    assert size.value == 4 * (128 * 64 * 1024 + 1024 + 64 * 256 + 2 * 2 * 2 * 64 * 256 + 256 + 2)


# ---- caching allocator on host memory (kind 1): same logic as on the device ------------------------------------

class Pool:
    def __init__(self, limit=0):
        self.lib = neoml_amd.load()
        self.h = ctypes.c_void_p()
        neoml_amd.check(self.lib.nhPoolCreate(ctypes.byref(self.h), 1, limit))

    def close(self):
        neoml_amd.check(self.lib.nhPoolDestroy(self.h))

    def alloc(self, size):
        p = ctypes.c_void_p()
        rc = self.lib.nhPoolHeapAlloc(self.h, size, ctypes.byref(p))
        return rc, p.value

    def free(self, p):
        return self.lib.nhPoolHeapFree(self.h, ctypes.c_void_p(p))

    def salloc(self, size):
        p = ctypes.c_void_p()
        rc = self.lib.nhPoolStackAlloc(self.h, size, ctypes.byref(p))
        return rc, p.value

    def sfree(self, p):
        return self.lib.nhPoolStackFree(self.h, ctypes.c_void_p(p))

    def stat(self, name):
        v = ctypes.c_size_t(0)
        neoml_amd.check(getattr(self.lib, "nhPoolGet" + name)(self.h, ctypes.byref(v)))
        return v.value


def test_pool_size_classes_and_reuse():
    pool = Pool()
    rc, p = pool.alloc(1000)
    assert rc == 0 and pool.stat("CurrentMemoryUsage") == 1024  # rounded up to its class
    assert pool.free(p) == 0
    assert pool.stat("MemoryInPools") == 1024 and pool.stat("CurrentMemoryUsage") == 1024  # cached, not released
    rc, q = pool.alloc(600)
    assert q == p and pool.stat("MemoryInPools") == 0
    rc, r = pool.alloc(2049)  # the 1.5x class between 2 KiB and 4 KiB
    assert pool.stat("CurrentMemoryUsage") == 1024 + 3072
    pool.free(q), pool.free(r)
    neoml_amd.check(pool.lib.nhPoolCleanUp(pool.h))
    assert pool.stat("MemoryInPools") == 0 and pool.stat("CurrentMemoryUsage") == 0
    assert pool.stat("PeakMemoryUsage") == 1024 + 3072
    neoml_amd.check(pool.lib.nhPoolResetPeakMemoryUsage(pool.h))
    assert pool.stat("PeakMemoryUsage") == 0
    assert pool.free(12345) == 1  # a pointer the pool does not know
    pool.close()


def test_pool_limit_triggers_cleanup_then_memory_error():
    pool = Pool(limit=1 << 20)
    rc, a = pool.alloc(600 * 1024)  # class 768 KiB
    assert rc == 0
    pool.free(a)
    assert pool.stat("MemoryInPools") == 768 * 1024
    rc, b = pool.alloc(300 * 1024)  # class 384 KiB: over the limit until the cached 768 KiB block is released
    assert rc == 0 and pool.stat("MemoryInPools") == 0 and pool.stat("CurrentMemoryUsage") == 384 * 1024
    rc, c = pool.alloc(900 * 1024)  # class 1 MiB: cannot fit beside b
    assert rc == 3 and "cannot allocate" in neoml_amd.last_error()
    pool.free(b)
    pool.close()


def test_pool_reuse_off_and_threshold():
    pool = Pool()
    neoml_amd.check(pool.lib.nhPoolSetThreadBufferMemoryThreshold(pool.h, 4096))
    t = ctypes.c_size_t(0)
    neoml_amd.check(pool.lib.nhPoolGetThreadBufferMemoryThreshold(pool.h, ctypes.byref(t)))
    assert t.value == 4096
    rc, a = pool.alloc(5000)  # above the threshold: exact size, returned to the raw allocator on free
    assert pool.stat("CurrentMemoryUsage") == 5000
    pool.free(a)
    assert pool.stat("CurrentMemoryUsage") == 0 and pool.stat("MemoryInPools") == 0
    neoml_amd.check(pool.lib.nhPoolSetReuseMemoryMode(pool.h, 0))
    rc, b = pool.alloc(100)
    assert pool.stat("CurrentMemoryUsage") == 100
    pool.free(b)
    assert pool.stat("CurrentMemoryUsage") == 0
    pool.close()


def test_pool_stack_is_lifo_and_regrows_to_high_water_mark():
    pool = Pool()
    rc, a = pool.salloc(1000)
    rc, b = pool.salloc(70000)  # does not fit the first 64 KiB block: a second block
    rc, c = pool.salloc(10)
    assert b != a and c == b + 70144  # sizes are rounded to 256 bytes
    assert pool.sfree(a) == 1  # not in the top block of the stack
    assert pool.sfree(c) == 0 and pool.sfree(b) == 0 and pool.sfree(a) == 0
    # empty stack: the next allocation re-creates one block of the high-water size, so the same sequence now
    # fits a single block
    rc, a2 = pool.salloc(1000)
    rc, b2 = pool.salloc(70000)
    assert b2 == a2 + 1024
    pool.sfree(b2), pool.sfree(a2)
    used = pool.stat("CurrentMemoryUsage")
    neoml_amd.check(pool.lib.nhPoolCleanUp(pool.h))
    assert used > 0 and pool.stat("CurrentMemoryUsage") == 0
    pool.close()


def test_pool_caches_are_per_thread():
    pool = Pool()
    rc, a = pool.alloc(1000)
    pool.free(a)
    seen = {}

    def worker():
        seen["in_pools"] = pool.stat("MemoryInPools")
        rc, b = pool.alloc(1000)
        seen["ptr"] = b
        # hand the block to this thread, free it here, clean up here
        neoml_amd.check(pool.lib.nhPoolTransferToThisThread(pool.h, ctypes.c_void_p(b), 1000))
        pool.free(b)
        seen["after_free"] = pool.stat("MemoryInPools")
        neoml_amd.check(pool.lib.nhPoolCleanUp(pool.h))
        seen["after_cleanup"] = pool.stat("MemoryInPools")

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert seen["in_pools"] == 0 and seen["ptr"] != a  # the other thread does not see this thread's cache
    assert seen["after_free"] == 1024 and seen["after_cleanup"] == 0
    assert pool.stat("MemoryInPools") == 1024  # untouched by the other thread's CleanUp
    pool.close()
