"""ctypes binding of include/neoml_hip.h.

Signatures are read from the header itself, so the binding cannot drift from the declared C ABI.
There is no fallback: when the shared library is missing, load() raises.
"""
import ctypes
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))
# NEOML_HIP_LIBRARY names another build of the library (a debug or experimental one)
LIB_PATH = os.environ.get("NEOML_HIP_LIBRARY") or os.path.join(HERE, "lib", "libneoml_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(HERE), "include", "neoml_hip.h")

NH_OK = 0
ERROR_NAMES = {1: "NH_ERR_ARGUMENT", 2: "NH_ERR_HIP", 3: "NH_ERR_MEMORY", 4: "NH_ERR_UNSUPPORTED"}


class NeoMLHipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s: %s" % (ERROR_NAMES.get(code, code), message))
        self.code = code


class ConvDesc(ctypes.Structure):
    """nhConvDesc"""
    _fields_ = [(n, ctypes.c_int) for n in (
        "batch", "height", "width", "channels", "filterCount", "filterHeight", "filterWidth",
        "paddingHeight", "paddingWidth", "strideHeight", "strideWidth", "dilationHeight", "dilationWidth",
        "resultHeight", "resultWidth")]


class PoolingDesc(ctypes.Structure):
    """nhPoolingDesc"""
    _fields_ = [(n, ctypes.c_int) for n in (
        "batch", "height", "width", "channels", "filterHeight", "filterWidth", "strideHeight", "strideWidth",
        "resultHeight", "resultWidth")]


class SeparableBlockDesc(ctypes.Structure):
    """nhSeparableBlockDesc"""
    _fields_ = [(n, ctypes.c_int) for n in (
        "batch", "height", "width", "inputChannels", "expandedChannels", "outputChannels", "stride", "residual")] + [
        ("expandActivation", ctypes.c_int), ("expandParam", ctypes.c_float),
        ("channelwiseActivation", ctypes.c_int), ("channelwiseParam", ctypes.c_float)]


class BlobDesc(ctypes.Structure):
    """nhBlobDesc: BatchLength, BatchWidth, ListSize, Height, Width, Depth, Channels"""
    _fields_ = [("dims", ctypes.c_int * 7)]

    @classmethod
    def of(cls, *dims):
        d = cls()
        assert len(dims) == 7
        for i, v in enumerate(dims):
            d.dims[i] = int(v)
        return d


_DECL = re.compile(r"NH_API\s+(const char\*|int)\s+(nh\w+)\s*\(([^;]*?)\)\s*;", re.S)


def _ctype(arg):
    arg = arg.strip()
    if arg == "void" or not arg:
        return None
    # drop the parameter name
    m = re.match(r"(.*?)(\w+)$", arg)
    typ = m.group(1).strip() if m and m.group(1).strip() else arg
    if "*" in typ or typ in ("nhStream", "nhEvent", "nhPool"):
        return ctypes.c_void_p
    if typ == "int":
        return ctypes.c_int
    if typ == "float":
        return ctypes.c_float
    if typ == "size_t":
        return ctypes.c_size_t
    raise ValueError("unknown C type in header: %r" % arg)


def declared_functions():
    """{name: (restype, [argtypes])} for every NH_API declaration of the header."""
    with open(HEADER_PATH) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for ret, name, args in _DECL.findall(text):
        argtypes = [t for t in (_ctype(a) for a in args.split(",")) if t is not None]
        out[name] = (ctypes.c_char_p if "char" in ret else ctypes.c_int, argtypes)
    return out


_lib = None


def load():
    """Loads libneoml_hip.so and sets the signatures. Raises when the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            "%s is missing: build it with `python -m neoml_amd.build` (no CPU fallback exists)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in declared_functions().items():
        fn = getattr(lib, name)  # AttributeError if the library does not export a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def last_error():
    return load().nhGetLastError().decode()


def check(rc):
    if rc != NH_OK:
        raise NeoMLHipError(rc, last_error())
