"""neoml_amd: MI355X (gfx950) kernels behind NeoML's IMathEngine interface.

The product is native: `lib/libneoml_hip.so` (HIP kernels + C ABI declared in include/neoml_hip.h) and the C++
engine adapter built on it. This Python package only loads the C ABI through ctypes for tests and benchmarks;
device memory for those comes from torch tensors.
"""
from .capi import (  # noqa: F401
    NeoMLHipError, load, check, last_error, declared_functions,
    ConvDesc, PoolingDesc, BlobDesc, SeparableBlockDesc, LIB_PATH, HEADER_PATH,
)
