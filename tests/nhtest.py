"""Shared helpers of the test-suite: loaders for the checkers (oracle/liboracle.so, oracle/_ref) and thin numpy
front-ends for them, plus the device-side call helpers for the HIP library.

Only tests, the smoke run and the benchmark's cpu_baseline leg import this module; the product never does.
"""
import ctypes
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "liboracle.so")
# NHTEST_SHIM_LIB: another build of the shim + reference engine (the MLAS-backed one of the benchmark's CPU baseline)
SHIM_LIB = os.environ.get("NHTEST_SHIM_LIB") or os.path.join(ORACLE_DIR, "_ref", "libengine_shim.so")

# tolerance of the parity bar: |a - b| <= ATOL + RTOL * |b|
RTOL = 1e-4
ATOL = 1e-5

UNARY = {name: i for i, name in enumerate([
    "relu", "elu", "leaky_relu", "hswish", "abs", "hard_tanh", "hard_sigmoid", "neg", "exp", "log", "erf", "sqrt",
    "inv", "minmax", "sigmoid", "tanh", "add_value", "multiply", "neg_multiply", "copy", "neg_log", "sub_value", "value_sub", "hinge", "squared_hinge", "huber", "huber_derivative"])}
BINARY = {name: i for i, name in enumerate([
    "add", "sub", "eltwise_multiply", "eltwise_neg_multiply", "eltwise_divide", "eltwise_max", "eltwise_min",
    "multiply_and_add", "multiply_and_sub", "eltwise_multiply_add", "relu_diff", "hswish_diff", "sigmoid_diff",
    "sigmoid_diff_op", "tanh_diff", "tanh_diff_op", "elu_diff", "elu_diff_op", "leaky_relu_diff", "hard_tanh_diff",
    "hard_sigmoid_diff", "hard_sigmoid_diff_op", "abs_diff", "hinge_diff", "squared_hinge_diff", "l1_diff_add"])}
BINARY_INT = {"add": 0, "sub": 1, "multiply": 2}

c_float_p = ctypes.POINTER(ctypes.c_float)
c_int_p = ctypes.POINTER(ctypes.c_int)


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def i32(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def fp(a):
    return None if a is None else a.ctypes.data_as(c_float_p)


def ip(a):
    return None if a is None else a.ctypes.data_as(c_int_p)


def build_oracle():
    """Compiles oracle/liboracle.so (and oracle/_ref when the reference sources are present)."""
    import subprocess
    subprocess.run(["make", "-s", "-C", ORACLE_DIR, "-j8", "all"], check=True)


_oracle = None


def oracle():
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_LIB):
            build_oracle()
        _oracle = ctypes.CDLL(ORACLE_LIB)
        _oracle.orc_vector_sum.restype = ctypes.c_float
        _oracle.orc_vector_dot_product.restype = ctypes.c_float
    return _oracle


def have_reference():
    return os.path.exists(SHIM_LIB)


_shim = None
_cpu_engine = None


def shim():
    global _shim
    if _shim is None:
        _shim = ctypes.CDLL(SHIM_LIB)
        _shim.shim_create_cpu_engine.restype = ctypes.c_void_p
        _shim.shim_last_error.restype = ctypes.c_char_p
    return _shim


def cpu_engine():
    """The reference's CCpuMathEngine (one per process)."""
    global _cpu_engine
    if _cpu_engine is None:
        _cpu_engine = ctypes.c_void_p(shim().shim_create_cpu_engine())
        assert _cpu_engine.value, "CreateCpuMathEngine failed"
    return _cpu_engine


ENGINE_LIB = os.path.join(ROOT, "neoml_amd", "lib", "libNeoMathEngineHip.so")
REF_ENGINE_LIB = os.path.join(ORACLE_DIR, "_ref", "libNeoMathEngine.so")
_hip_engine = None


def have_engine_adapter():
    return os.path.exists(ENGINE_LIB) and have_reference()


def hip_engine():
    """The CHipMathEngine adapter, created through its C factory. The host process must already hold NeoML's
    libNeoMathEngine (here: the reference build under oracle/_ref), whose symbols the adapter resolves at load."""
    global _hip_engine
    if _hip_engine is None:
        ctypes.CDLL(REF_ENGINE_LIB, mode=ctypes.RTLD_GLOBAL)
        lib = ctypes.CDLL(ENGINE_LIB, mode=ctypes.RTLD_GLOBAL)
        lib.CreateHipMathEngine.restype = ctypes.c_void_p
        lib.CreateHipMathEngine.argtypes = [ctypes.c_int, ctypes.c_size_t, ctypes.c_int]
        ptr = lib.CreateHipMathEngine(0, 0, 0)
        assert ptr, "CreateHipMathEngine returned null"
        _hip_engine = ctypes.c_void_p(ptr)
    return _hip_engine


def conv_out(h, w, fh, fw, ph, pw, sh, sw, dh=1, dw=1):
    ho = 1 + (h - (fh - 1) * dh + 2 * ph - 1) // sh
    wo = 1 + (w - (fw - 1) * dw + 2 * pw - 1) // sw
    return ho, wo


class Cpu:
    """Numpy front-end shared by the oracle ('orc') and the reference engine through the shim ('ref')."""

    def __init__(self, kind):
        # 'orc': the C oracle; 'ref': the reference CPU engine through the shim; 'hipeng': the HIP engine adapter
        # through the very same shim calls (exercises the IMathEngine boundary; needs a GPU)
        assert kind in ("orc", "ref", "hipeng")
        self.lib = oracle() if kind == "orc" else shim()
        self.pre = "orc_" if kind == "orc" else "shim_"
        if kind == "orc":
            self.eng = ()
        elif kind == "ref":
            self.eng = (cpu_engine(),)
        else:
            self.eng = (hip_engine(),)
        self.kind = "orc" if kind == "orc" else "ref"  # call convention: direct oracle or through the shim
        self.name = kind

    def _call(self, name, *args):
        rc = getattr(self.lib, self.pre + name)(*self.eng, *args)
        if self.kind == "ref" and rc != 0:
            raise RuntimeError("%s engine: %s" % (self.name, self.lib.shim_last_error().decode()))
        return rc

    # ---- element-wise
    def unary(self, op, x, p0=0.0, p1=0.0):
        x = f32(x)
        y = np.empty_like(x)
        self._call("vector_unary", UNARY[op], fp(x), fp(y), x.size, ctypes.c_float(p0), ctypes.c_float(p1))
        return y

    def binary(self, op, a, b, p0=0.0, result=None, p1=0.0):
        a, b = f32(a), f32(b)
        y = np.zeros_like(a) if result is None else f32(result).copy()
        self._call("vector_binary", BINARY[op], fp(a), fp(b), fp(y), a.size, ctypes.c_float(p0), ctypes.c_float(p1))
        return y

    def row_dot(self, a, b):
        a, b = f32(a), f32(b)
        y = np.empty(a.shape[0], np.float32)
        self._call("row_multiply_matrix_by_matrix", fp(a), fp(b), a.shape[0], a.shape[1], fp(y))
        return y

    def softmax_diff_rows(self, y, grad):
        y, grad = f32(y), f32(grad)
        out = np.empty_like(y)
        self._call("matrix_softmax_diff_op_by_rows", fp(y), fp(grad), y.shape[0], y.shape[1], fp(out))
        return out

    def diag_by_matrix_add(self, diag, matrix, result):
        """diag [B][n], matrix [B][n][w], result [n][w] (accumulated into)."""
        diag, matrix = f32(diag), f32(matrix)
        out = f32(result).copy()
        self._call("multiply_diag_matrix_by_matrix_and_add", diag.shape[0], fp(diag), diag.shape[1], fp(matrix), matrix.shape[2], fp(out))
        return out

    def binary_int(self, op, a, b):
        a, b = i32(a), i32(b)
        y = np.empty_like(a)
        self._call("vector_binary_int", BINARY_INT[op], ip(a), ip(b), ip(y), a.size)
        return y

    def float_to_int(self, x):
        x = f32(x)
        y = np.empty(x.shape, np.int32)
        self._call("vector_convert_float_to_int", fp(x), ip(y), x.size)
        return y

    def int_to_float(self, x):
        x = i32(x)
        y = np.empty(x.shape, np.float32)
        self._call("vector_convert_int_to_float", ip(x), fp(y), x.size)
        return y

    def vector_sum(self, x):
        x = f32(x)
        if self.kind == "orc":
            return np.float32(self.lib.orc_vector_sum(fp(x), x.size))
        r = np.zeros(1, np.float32)
        self._call("vector_sum", fp(x), x.size, fp(r))
        return r[0]

    def dot(self, a, b):
        a, b = f32(a), f32(b)
        if self.kind == "orc":
            return np.float32(self.lib.orc_vector_dot_product(fp(a), fp(b), a.size))
        r = np.zeros(1, np.float32)
        self._call("vector_dot_product", fp(a), fp(b), a.size, fp(r))
        return r[0]

    # ---- broadcasts, reductions
    def set_vector_to_matrix_rows(self, h, w, vec):
        vec = f32(vec)
        y = np.empty((h, w), np.float32)
        self._call("set_vector_to_matrix_rows", fp(y), h, w, fp(vec))
        return y

    def add_vector_to_matrix_rows(self, m, vec):
        m, vec = f32(m), f32(vec)  # m [b,h,w], vec [b,w]
        b, h, w = m.shape
        y = np.empty_like(m)
        self._call("add_vector_to_matrix_rows", b, fp(m), fp(y), h, w, fp(vec))
        return y

    def add_vector_to_matrix_columns(self, m, vec, sign=1):
        m, vec = f32(m), f32(vec)
        h, w = m.shape
        y = np.empty_like(m)
        self._call("add_vector_to_matrix_columns", fp(m), fp(y), h, w, fp(vec), sign)
        return y

    def sum_matrix_rows(self, m, add_to=None):
        m = f32(m)
        b, h, w = m.shape
        y = np.zeros((b, w), np.float32) if add_to is None else f32(add_to).copy()
        self._call("sum_matrix_rows", b, fp(y), fp(m), h, w, 0 if add_to is None else 1)
        return y

    def sum_matrix_columns(self, m):
        m = f32(m)
        h, w = m.shape
        y = np.empty(h, np.float32)
        self._call("sum_matrix_columns", fp(y), fp(m), h, w)
        return y

    def multiply_diag_matrix_by_matrix(self, d, m):
        d, m = f32(d), f32(m)
        y = np.empty_like(m)
        self._call("multiply_diag_matrix_by_matrix", fp(d), m.shape[0], fp(m), m.shape[1], fp(y))
        return y

    def batch_multiply_matrix_by_diag_matrix(self, batch, first, h, w, first_off, second, second_off):
        first, second = f32(first), f32(second)
        y = np.empty((batch, h, w), np.float32)
        self._call("batch_multiply_matrix_by_diag_matrix", batch, fp(first), h, w, first_off, fp(second), second_off, fp(y))
        return y

    def softmax_rows(self, m):
        m = f32(m)
        y = np.empty_like(m)
        self._call("matrix_softmax_by_rows", fp(m), m.shape[0], m.shape[1], fp(y))
        return y

    def log_sum_exp_rows(self, m):
        m = f32(m)
        y = np.empty(m.shape[0], np.float32)
        self._call("matrix_log_sum_exp_by_rows", fp(m), m.shape[0], m.shape[1], fp(y))
        return y

    def find_max_in_rows(self, m, with_indices=True):
        m = f32(m)
        v = np.empty(m.shape[0], np.float32)
        idx = np.empty(m.shape[0], np.int32) if with_indices else None
        self._call("find_max_value_in_rows", fp(m), m.shape[0], m.shape[1], fp(v), ip(idx))
        return v, idx

    def find_max_in_columns(self, m):
        m = f32(m)
        b, h, w = m.shape
        v = np.empty((b, w), np.float32)
        idx = np.empty((b, w), np.int32)
        self._call("find_max_value_in_columns", b, fp(m), h, w, fp(v), ip(idx))
        return v, idx

    def transpose(self, x):
        """x [b,h,m,w,c] -> [b,w,m,h,c]"""
        x = f32(x)
        b, h, m, w, c = x.shape
        y = np.empty((b, w, m, h, c), np.float32)
        self._call("transpose_matrix", b, fp(x), h, m, w, c, fp(y))
        return y

    # ---- matrix products (C is M x N, reduction K)
    def matmul(self, kind, a, b, c=None, lda=None, ldb=None, ldc=None, M=None, N=None, K=None, batch=1):
        """kind: 'nt' (strided), 'bnt', 'bnn', 'btn' (batched, dense), 'tn_add' (strided, accumulates into c)."""
        a, b = f32(a), f32(b)
        if self.kind == "orc":
            fn = {"nt": "orc_matmul_nt", "bnt": "orc_matmul_nt", "bnn": "orc_matmul_nn", "btn": "orc_matmul_tn",
                  "tn_add": "orc_matmul_tn"}[kind]
            if kind in ("nt", "tn_add"):
                out = np.zeros(((M - 1) * ldc + N,), np.float32) if c is None else f32(c).copy().ravel()
                getattr(self.lib, fn)(fp(a), lda, fp(b), ldb, fp(out), ldc, M, N, K, 1 if kind == "tn_add" else 0)
                return out
            out = np.empty((batch, M, N), np.float32)
            a_rows, a_cols = (K, M) if kind == "btn" else (M, K)
            b_rows, b_cols = (N, K) if kind == "bnt" else (K, N)
            a3 = a.reshape(batch, a_rows, a_cols)
            b3 = b.reshape(batch, b_rows, b_cols)
            for i in range(batch):
                ai, bi, oi = f32(a3[i]), f32(b3[i]), np.empty((M, N), np.float32)
                getattr(self.lib, fn)(fp(ai), a_cols, fp(bi), b_cols, fp(oi), N, M, N, K, 0)
                out[i] = oi
            return out
        code = {"nt": 0, "bnt": 1, "bnn": 2, "btn": 3, "tn_add": 4}[kind]
        if kind in ("nt", "tn_add"):
            out = np.zeros(((M - 1) * ldc + N,), np.float32) if c is None else f32(c).copy().ravel()
            self._call("matmul", code, 1, fp(a), lda, fp(b), ldb, fp(out), ldc, M, N, K)
            return out
        out = np.empty((batch, M, N), np.float32)
        lda = M if kind == "btn" else K
        ldb = K if kind == "bnt" else N
        self._call("matmul", code, batch, fp(a), lda, fp(b), ldb, fp(out), N, M, N, K)
        return out

    # ---- convolution, pooling
    def conv(self, x, filt, bias, ph, pw, sh, sw, dh=1, dw=1):
        x, filt = f32(x), f32(filt)
        n, h, w, cin = x.shape
        cout, fh, fw, _ = filt.shape
        ho, wo = conv_out(h, w, fh, fw, ph, pw, sh, sw, dh, dw)
        bias = None if bias is None else f32(bias)
        y = np.empty((n, ho, wo, cout), np.float32)
        self._call("blob_convolution", fp(x), n, h, w, cin, fp(filt), cout, fh, fw, ph, pw, sh, sw, dh, dw, fp(bias), fp(y))
        return y

    def channelwise_conv(self, x, filt, bias, ph, pw, sh, sw):
        x, filt = f32(x), f32(filt)
        n, h, w, c = x.shape
        fh, fw, _ = filt.shape
        ho, wo = conv_out(h, w, fh, fw, ph, pw, sh, sw)
        bias = None if bias is None else f32(bias)
        y = np.empty((n, ho, wo, c), np.float32)
        self._call("blob_channelwise_convolution", fp(x), n, h, w, c, fp(filt), fh, fw, ph, pw, sh, sw, fp(bias), fp(y))
        return y

    ACTIVATIONS = {None: 0, "relu": 1, "hswish": 2}

    def separable_block(self, x, expand, channelwise, down, stride=1, residual=False, in_place=False):
        """The fused blocks of depthwise-separable networks. expand = (filter [E][Cin], free term, activation, param)
        or None for the channelwise + 1x1 block; channelwise = (filter [3][3][E], free term, activation, param);
        down = (filter [Cout][E], free term). activation: None, 'relu' (param = upper threshold when > 0), 'hswish'.
        The oracle composes the block from its own convolution, channelwise convolution and activation functions,
        stage by stage as src/CPU/Rowwise/CpuRowwiseMobileNetV2.h:150-300 and CpuRowwiseChConvWith1x1.h do; the
        reference engine runs its MobileNetV2Block / ChannelwiseWith1x1."""
        x = f32(x)
        n, h, w, cin = x.shape
        ch_f, ch_t, ch_act, ch_param = channelwise
        dn_f, dn_t = down
        e = ch_f.shape[2]
        cout = dn_f.shape[0]
        ho, wo = (h + stride - 1) // stride, (w + stride - 1) // stride
        if self.kind == "orc":
            def act(t, name, param):
                if name is None:
                    return t
                return self.unary(name, t, np.float32(param if name == "relu" else 0.0)).reshape(t.shape)
            t = x
            if expand is not None:
                ex_f, ex_t, ex_act, ex_param = expand
                t = act(self.conv(t, f32(ex_f).reshape(e, 1, 1, cin), ex_t, 0, 0, 1, 1), ex_act, ex_param)
            t = act(self.channelwise_conv(t, ch_f, ch_t, 1, 1, stride, stride), ch_act, ch_param)
            y = self.conv(t, f32(dn_f).reshape(cout, 1, 1, e), dn_t, 0, 0, 1, 1)
            return y + x if residual else y
        ex_f, ex_t, ex_act, ex_param = expand if expand is not None else (None, None, None, 0.0)
        y = np.empty((n, ho, wo, cout), np.float32)
        opt = lambda a: None if a is None else f32(a)
        keep = [opt(ex_f), opt(ex_t), f32(ch_f), opt(ch_t), f32(dn_f), opt(dn_t)]
        self._call("separable_block", 1 if expand is not None else 0, fp(x), n, h, w, cin, e, cout, stride,
                   1 if residual else 0, self.ACTIVATIONS[ex_act], ctypes.c_float(ex_param), self.ACTIVATIONS[ch_act],
                   ctypes.c_float(ch_param), fp(keep[0]), fp(keep[1]), fp(keep[2]), fp(keep[3]), fp(keep[4]), fp(keep[5]),
                   1 if in_place else 0, fp(y))
        return y

    def mobilenetv3_pre_se(self, x, expand, channelwise, stride=1):
        """expand = (filter [E][Cin], free term, activation, param); channelwise = (filter [F][F][E], free term,
        activation, param), F = 3 or 5, padding (F - 1) / 2. The oracle composes its own convolution, channelwise
        convolution and activations; the reference engine runs its MobileNetV3PreSEBlock."""
        x = f32(x)
        n, h, w, cin = x.shape
        ex_f, ex_t, ex_act, ex_param = expand
        ch_f, ch_t, ch_act, ch_param = channelwise
        fsize, e = ch_f.shape[0], ch_f.shape[2]
        pad = (fsize - 1) // 2
        if self.kind == "orc":
            def act(t, name, param):
                return t if name is None else self.unary(name, t, np.float32(param if name == "relu" else 0.0)).reshape(t.shape)
            t = act(self.conv(x, f32(ex_f).reshape(e, 1, 1, cin), ex_t, 0, 0, 1, 1), ex_act, ex_param)
            return act(self.channelwise_conv(t, ch_f, ch_t, pad, pad, stride, stride), ch_act, ch_param)
        ho, wo = conv_out(h, w, fsize, fsize, pad, pad, stride, stride)
        y = np.empty((n, ho, wo, e), np.float32)
        opt = lambda a: None if a is None else f32(a)
        keep = [f32(ex_f), opt(ex_t), f32(ch_f), opt(ch_t)]
        self._call("mobilenetv3_pre_se", fp(x), n, h, w, cin, e, fsize, stride, self.ACTIVATIONS[ex_act], ctypes.c_float(ex_param),
                   self.ACTIVATIONS[ch_act], ctypes.c_float(ch_param), fp(keep[0]), fp(keep[1]), fp(keep[2]), fp(keep[3]), fp(y))
        return y

    def mobilenetv3_post_se(self, x, gate, residual, activation, param, down):
        """x [N][H][W][C] (the depthwise stage's output), gate [N][C], residual [N][H][W][Cout] or None,
        down = (filter [Cout][C], free term)."""
        x, gate = f32(x), f32(gate)
        n, h, w, c = x.shape
        dn_f, dn_t = down
        cout = dn_f.shape[0]
        if self.kind == "orc":
            t = x * gate.reshape(n, 1, 1, c)
            if activation is not None:
                t = self.unary(activation, t, np.float32(param if activation == "relu" else 0.0)).reshape(t.shape)
            y = self.conv(t, f32(dn_f).reshape(cout, 1, 1, c), dn_t, 0, 0, 1, 1)
            return y if residual is None else y + f32(residual)
        y = np.empty((n, h, w, cout), np.float32)
        opt = lambda a: None if a is None else f32(a)
        keep = [opt(residual), f32(dn_f), opt(dn_t)]
        self._call("mobilenetv3_post_se", fp(x), n, h, w, c, cout, fp(gate), fp(keep[0]), self.ACTIVATIONS[activation],
                   ctypes.c_float(param), fp(keep[1]), fp(keep[2]), fp(y))
        return y

    # ---- gradients (what the layers' backward and learn passes call)
    def conv_backward(self, out_diff, filt, bias, in_shape, ph, pw, sh, sw, dh=1, dw=1):
        """Gradient by the input; bias [Cin] or None is added to every pixel."""
        out_diff, filt = f32(out_diff), f32(filt)
        n, h, w, cin = in_shape
        cout, fh, fw, _ = filt.shape
        assert out_diff.shape == (n, *conv_out(h, w, fh, fw, ph, pw, sh, sw, dh, dw), cout)
        bias = None if bias is None else f32(bias)
        y = np.empty(in_shape, np.float32)
        self._call("blob_convolution_backward", fp(out_diff), n, h, w, cin, fp(filt), cout, fh, fw, ph, pw, sh, sw, dh, dw,
                   fp(bias), fp(y))
        return y

    def conv_learn_add(self, x, out_diff, filter_diff, ph, pw, sh, sw, dh=1, dw=1, free_term_diff=None):
        """filter_diff [Cout][fh][fw][Cin] += gradient by the filter; free_term_diff [Cout] += column sums of out_diff
        (through the reference interface only: the oracle's form of it is numpy's sum)."""
        x, out_diff = f32(x), f32(out_diff)
        n, h, w, cin = x.shape
        cout, fh, fw, _ = filter_diff.shape
        fd = f32(filter_diff).copy()
        if self.kind == "orc":
            self._call("blob_convolution_learn_add", fp(x), n, h, w, cin, fp(out_diff), cout, fh, fw, ph, pw, sh, sw, dh, dw,
                       fp(fd))
            if free_term_diff is None:
                return fd
            return fd, (f32(free_term_diff) + out_diff.reshape(-1, cout).astype(np.float64).sum(axis=0)).astype(np.float32)
        ftd = None if free_term_diff is None else f32(free_term_diff).copy()
        self._call("blob_convolution_learn_add", fp(x), n, h, w, cin, fp(out_diff), cout, fh, fw, ph, pw, sh, sw, dh, dw,
                   fp(fd), fp(ftd))
        return fd if ftd is None else (fd, ftd)

    def channelwise_conv_backward(self, out_diff, filt, in_shape, ph, pw, sh, sw):
        out_diff, filt = f32(out_diff), f32(filt)
        n, h, w, c = in_shape
        fh, fw, _ = filt.shape
        assert out_diff.shape == (n, *conv_out(h, w, fh, fw, ph, pw, sh, sw), c)
        y = np.empty(in_shape, np.float32)
        self._call("blob_channelwise_convolution_backward", fp(out_diff), n, h, w, c, fp(filt), fh, fw, ph, pw, sh, sw, fp(y))
        return y

    def channelwise_conv_learn_add(self, x, out_diff, filter_diff, ph, pw, sh, sw, free_term_diff=None):
        x, out_diff = f32(x), f32(out_diff)
        n, h, w, c = x.shape
        fh, fw, _ = filter_diff.shape
        fd = f32(filter_diff).copy()
        ftd = None if free_term_diff is None else f32(free_term_diff).copy()
        self._call("blob_channelwise_convolution_learn_add", fp(x), n, h, w, c, fp(out_diff), fh, fw, ph, pw, sh, sw, fp(fd), fp(ftd))
        return fd if ftd is None else (fd, ftd)

    def max_pool_backward(self, x, result_diff, fh, fw, sh, sw):
        """Forward pass over x for the indices, then the gradient by x."""
        x, result_diff = f32(x), f32(result_diff)
        n, h, w, c = x.shape
        y = np.empty_like(x)
        if self.kind == "orc":
            _, idx = self.max_pool(x, fh, fw, sh, sw, with_indices=True)
            self._call("blob_max_pooling_backward", fp(result_diff), ip(idx), n, h * w * c, idx[0].size, fp(y))
        else:
            self._call("blob_pooling_backward", 1, fp(x), fp(result_diff), n, h, w, c, fh, fw, sh, sw, fp(y))
        return y

    def mean_pool_backward(self, in_shape, result_diff, fh, fw, sh, sw):
        result_diff = f32(result_diff)
        n, h, w, c = in_shape
        y = np.empty(in_shape, np.float32)
        if self.kind == "orc":
            self._call("blob_mean_pooling_backward", fp(result_diff), n, h, w, c, fh, fw, sh, sw, fp(y))
        else:
            self._call("blob_pooling_backward", 0, None, fp(result_diff), n, h, w, c, fh, fw, sh, sw, fp(y))
        return y

    def max_pool(self, x, fh, fw, sh, sw, with_indices=False):
        x = f32(x)
        n, h, w, c = x.shape
        ho, wo = (h - fh) // sh + 1, (w - fw) // sw + 1
        y = np.empty((n, ho, wo, c), np.float32)
        idx = np.empty((n, ho, wo, c), np.int32) if with_indices else None
        self._call("blob_max_pooling", fp(x), n, h, w, c, fh, fw, sh, sw, ip(idx), fp(y))
        return (y, idx) if with_indices else y

    def mean_pool(self, x, fh, fw, sh, sw):
        x = f32(x)
        n, h, w, c = x.shape
        ho, wo = (h - fh) // sh + 1, (w - fw) // sw + 1
        y = np.empty((n, ho, wo, c), np.float32)
        self._call("blob_mean_pooling", fp(x), n, h, w, c, fh, fw, sh, sw, fp(y))
        return y

    def resize_image(self, x, dl, dr, dt, db, padding=0, value=0.0):
        x = f32(x)
        n, h, w, c = x.shape
        y = np.empty((n, h + dt + db, w + dl + dr, c), np.float32)
        self._call("blob_resize_image", fp(x), n, h, w, c, dl, dr, dt, db, padding, ctypes.c_float(value), fp(y))
        return y

    def split(self, big, dim, part_dims):
        """big: 7-D array; part_dims: list of 7-tuples. Returns the parts."""
        big = f32(big)
        parts = [np.empty(d, np.float32) for d in part_dims]
        self._split_merge(big, dim, parts, merge=0)
        return parts

    def merge(self, parts, dim, big_dims):
        parts = [f32(p) for p in parts]
        big = np.empty(big_dims, np.float32)
        self._split_merge(big, dim, parts, merge=1)
        return big

    def dropout(self, x, rate, spatial=False, batchwise=False, seed=1):
        """x: 7-D blob."""
        x = f32(x)
        y = np.empty_like(x)
        self._call("dropout", ip(i32(x.shape)), ctypes.c_float(rate), 1 if spatial else 0, 1 if batchwise else 0, seed, fp(x), fp(y))
        return y

    def broadcast_copy(self, x, to_dims, width=1):
        """x: array of shape from_dims (7) + (width,); returns to_dims + (width,)."""
        x = f32(x)
        from_dims = x.shape[:7]
        y = np.empty(tuple(to_dims) + (width,), np.float32)
        self._call("broadcast_copy", ip(i32(to_dims)), ip(i32(from_dims)), width, fp(x), fp(y))
        return y

    def _split_merge(self, big, dim, parts, merge):
        count = len(parts)
        ptrs = (c_float_p * count)(*[fp(p) for p in parts])
        if self.kind == "orc":
            rows = int(np.prod(big.shape[:dim])) if dim > 0 else 1
            sizes = [int(np.prod(p.shape[dim:])) if dim > 0 else p.size for p in parts]
            self.lib.orc_blob_split_merge(fp(big), rows, ptrs, ip(i32(sizes)), count, merge)
        else:
            pd = i32(np.array([p.shape for p in parts]).ravel())
            self._call("blob_split_merge", dim, ip(i32(big.shape)), fp(big), ip(pd), ptrs, count, merge)

    def lstm(self, w_in, b_in, w_rec, b_rec, x, reverse=False, c0=None, h0=None, want_state=True):
        w_in, w_rec, x = f32(w_in), f32(w_rec), f32(x)
        T, B, In = x.shape
        H = w_rec.shape[1]
        b_in = None if b_in is None else f32(b_in)
        b_rec = None if b_rec is None else f32(b_rec)
        c0 = None if c0 is None else f32(c0)
        h0 = None if h0 is None else f32(h0)
        h = np.empty((T, B, H), np.float32)
        c = np.empty((T, B, H), np.float32) if want_state else None
        self._call("lstm", H, In, fp(w_in), fp(b_in), fp(w_rec), fp(b_rec), 1 if reverse else 0, T, B,
                   fp(c0), fp(h0), fp(x), fp(c), fp(h))
        return h, c


def ctc_greedy_collapse(labels, blank, seq_len=None):
    """labels [B][T] int32 -> list of label lists (oracle only: the reference does this on the host in the layer)."""
    labels = i32(labels)
    B, T = labels.shape
    out = np.zeros((B, T), np.int32)
    lengths = np.zeros(B, np.int32)
    sl = None if seq_len is None else i32(seq_len)
    oracle().orc_ctc_greedy_collapse(ip(labels), T, B, blank, ip(sl), ip(out), ip(lengths))
    return [out[b, :lengths[b]].tolist() for b in range(B)]


def assert_close(actual, expected, what="", rtol=RTOL, atol=ATOL):
    actual = np.asarray(actual, dtype=np.float64)
    expected = np.asarray(expected, dtype=np.float64)
    assert actual.shape == expected.shape, "%s: shape %s vs %s" % (what, actual.shape, expected.shape)
    err = np.abs(actual - expected)
    bound = atol + rtol * np.abs(expected)
    bad = ~(err <= bound)
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err - bound, -np.inf)), err.shape)
        raise AssertionError("%s: %d of %d elements outside rtol=%g atol=%g; worst at %s: got %r expected %r" % (
            what, int(bad.sum()), bad.size, rtol, atol, i, actual[i], expected[i]))


# ---------------------------------------------------------------------------------------------------------
# device side: the same front-end, through the C ABI of libneoml_hip.so on torch-owned device memory

class Hip:
    """Calls the HIP library through its C ABI. Inputs are numpy arrays; they are uploaded into torch CUDA
    tensors (plumbing only), the kernel runs on torch's current stream, and the result comes back as numpy."""

    def __init__(self):
        import torch
        import neoml_amd
        self.torch = torch
        self.na = neoml_amd
        self.lib = neoml_amd.load()
        assert torch.cuda.is_available(), "no GPU"
        self.dev = torch.device("cuda:0")

    # -- plumbing
    def stream(self):
        return ctypes.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def up(self, a):
        if a is None:
            return None
        return self.torch.from_numpy(np.ascontiguousarray(a)).to(self.dev)

    def empty(self, shape, dtype=np.float32):
        t = self.torch.float32 if dtype == np.float32 else self.torch.int32
        return self.torch.empty(tuple(int(s) for s in shape), dtype=t, device=self.dev)

    @staticmethod
    def p(t):
        return None if t is None else ctypes.c_void_p(t.data_ptr())

    def scalar(self, v, dtype=np.float32):
        return self.up(np.array([v], dtype=dtype))

    def call(self, name, *args):
        self.na.check(getattr(self.lib, name)(self.stream(), *args))

    @staticmethod
    def down(t):
        return t.cpu().numpy()

    # -- element-wise
    UNARY_FN = {
        "relu": ("nhVectorReLU", 1), "elu": ("nhVectorELU", 1), "leaky_relu": ("nhVectorLeakyReLU", 1),
        "hswish": ("nhVectorHSwish", 0), "abs": ("nhVectorAbs", 0), "hard_tanh": ("nhVectorHardTanh", 0),
        "hard_sigmoid": ("nhVectorHardSigmoid", 2), "neg": ("nhVectorNeg", 0), "exp": ("nhVectorExp", 0),
        "log": ("nhVectorLog", 0), "erf": ("nhVectorErf", 0), "sqrt": ("nhVectorSqrt", 0), "inv": ("nhVectorInv", 0),
        "minmax": ("nhVectorMinMax", 2), "sigmoid": ("nhVectorSigmoid", 0), "tanh": ("nhVectorTanh", 0),
        "add_value": ("nhVectorAddValue", 1), "multiply": ("nhVectorMultiply", 1),
        "neg_multiply": ("nhVectorNegMultiply", 1), "neg_log": ("nhVectorNegLog", 0), "hinge": ("nhVectorHinge", 0),
        "squared_hinge": ("nhVectorSquaredHinge", 0), "huber": ("nhVectorHuber", 0),
        "huber_derivative": ("nhVectorHuberDerivative", 0),
    }


    def unary(self, op, x, p0=0.0, p1=0.0, inplace=False, offset=0):
        """offset > 0 runs on a view that starts `offset` elements into a buffer (unaligned pointers)."""
        x = f32(x).ravel()
        n = x.size
        buf = self.empty((n + offset,))
        buf[offset:] = self.up(x)
        src = buf[offset:]
        if inplace:
            dst = src
        else:
            dbuf = self.empty((n + offset,))
            dst = dbuf[offset:]
        if op == "copy":
            self.call("nhVectorCopy", self.p(dst), self.p(src), n)
            return self.down(dst)
        if op in ("sub_value", "value_sub"):
            self.call("nhVectorSubValue", self.p(src), p0, 1 if op == "value_sub" else 0, self.p(dst), n)
            return self.down(dst)
        fn, nscalars = self.UNARY_FN[op]
        scalars = [self.scalar(p0), self.scalar(p1)][:nscalars]
        self.call(fn, self.p(src), self.p(dst), n, *[self.p(s) for s in scalars])
        return self.down(dst)

    BINARY_FN = {
        "add": "nhVectorAdd", "sub": "nhVectorSub", "eltwise_multiply": "nhVectorEltwiseMultiply",
        "eltwise_neg_multiply": "nhVectorEltwiseNegMultiply", "eltwise_divide": "nhVectorEltwiseDivide",
        "eltwise_max": "nhVectorEltwiseMax", "eltwise_min": "nhVectorEltwiseMin",
        "multiply_and_add": "nhVectorMultiplyAndAdd", "multiply_and_sub": "nhVectorMultiplyAndSub",
        "eltwise_multiply_add": "nhVectorEltwiseMultiplyAdd", "relu_diff": "nhVectorReLUDiff",
        "hswish_diff": "nhVectorHSwishDiff", "sigmoid_diff": "nhVectorSigmoidDiff",
        "sigmoid_diff_op": "nhVectorSigmoidDiffOp", "tanh_diff": "nhVectorTanhDiff", "tanh_diff_op": "nhVectorTanhDiffOp",
        "elu_diff": "nhVectorELUDiff", "elu_diff_op": "nhVectorELUDiffOp", "leaky_relu_diff": "nhVectorLeakyReLUDiff",
        "hard_tanh_diff": "nhVectorHardTanhDiff", "hard_sigmoid_diff": "nhVectorHardSigmoidDiff",
        "hard_sigmoid_diff_op": "nhVectorHardSigmoidDiffOp", "abs_diff": "nhVectorAbsDiff",
        "hinge_diff": "nhVectorHingeDiff", "squared_hinge_diff": "nhVectorSquaredHingeDiff", "l1_diff_add": "nhVectorL1DiffAdd",
    }

    def binary(self, op, a, b, p0=0.0, result=None, inplace_first=False, p1=0.0):
        a, b = self.up(f32(a).ravel()), self.up(f32(b).ravel())
        n = a.numel()
        out = a if inplace_first else (self.empty((n,)) if result is None else self.up(f32(result).ravel()))
        args = [self.p(a), self.p(b), self.p(out), n]
        keep = []
        if op in ("multiply_and_add", "multiply_and_sub", "relu_diff", "elu_diff", "elu_diff_op", "leaky_relu_diff",
                  "hard_sigmoid_diff", "hard_sigmoid_diff_op", "l1_diff_add"):
            s = self.scalar(p0)
            args.append(self.p(s))
        if op in ("hard_sigmoid_diff", "l1_diff_add"):
            keep.append(self.scalar(p1))
            args.append(self.p(keep[0]))
        self.call(self.BINARY_FN[op], *args)
        return self.down(out)

    def row_dot(self, a, b):
        a, b = f32(a), f32(b)
        xa, xb = self.up(a), self.up(b)
        out = self.empty((a.shape[0],))
        self.call("nhRowMultiplyMatrixByMatrix", self.p(xa), self.p(xb), a.shape[0], a.shape[1], self.p(out))
        return self.down(out)

    def softmax_diff_rows(self, y, grad, inplace=False):
        y, grad = f32(y), f32(grad)
        xa, xb = self.up(y), self.up(grad)
        out = xb if inplace else self.empty(y.shape)
        self.call("nhMatrixSoftmaxDiffOpByRows", self.p(xa), self.p(xb), y.shape[0], y.shape[1], self.p(out))
        return self.down(out)

    def diag_by_matrix_add(self, diag, matrix, result):
        diag, matrix = f32(diag), f32(matrix)
        xd, xm, out = self.up(diag), self.up(matrix), self.up(f32(result))
        self.call("nhMultiplyDiagMatrixByMatrixAndAdd", diag.shape[0], self.p(xd), diag.shape[1], self.p(xm), matrix.shape[2], self.p(out))
        return self.down(out)

    def binary_int(self, op, a, b):
        fn = {"add": "nhVectorAddInt", "sub": "nhVectorSubInt", "multiply": "nhVectorEltwiseMultiplyInt"}[op]
        a, b = self.up(i32(a).ravel()), self.up(i32(b).ravel())
        out = self.empty((a.numel(),), np.int32)
        self.call(fn, self.p(a), self.p(b), self.p(out), a.numel())
        return self.down(out)

    def float_to_int(self, x):
        x = self.up(f32(x).ravel())
        out = self.empty((x.numel(),), np.int32)
        self.call("nhVectorConvertFloatToInt", self.p(x), self.p(out), x.numel())
        return self.down(out)

    def int_to_float(self, x):
        x = self.up(i32(x).ravel())
        out = self.empty((x.numel(),))
        self.call("nhVectorConvertIntToFloat", self.p(x), self.p(out), x.numel())
        return self.down(out)

    def fill(self, n, value, from_handle=False, integer=False):
        out = self.empty((n,), np.int32 if integer else np.float32)
        if from_handle:
            s = self.scalar(value, np.int32 if integer else np.float32)
            self.call("nhVectorFillFromHandleInt" if integer else "nhVectorFillFromHandle", self.p(out), n, self.p(s))
        elif integer:
            self.call("nhVectorFillInt", self.p(out), int(value), n)
        else:
            self.call("nhVectorFill", self.p(out), ctypes.c_float(value), n)
        return self.down(out)

    def vector_sum(self, x):
        x = self.up(f32(x).ravel())
        out = self.empty((1,))
        self.call("nhVectorSum", self.p(x), x.numel(), self.p(out))
        return self.down(out)[0]

    def dot(self, a, b):
        a, b = self.up(f32(a).ravel()), self.up(f32(b).ravel())
        out = self.empty((1,))
        self.call("nhVectorDotProduct", self.p(a), self.p(b), a.numel(), self.p(out))
        return self.down(out)[0]

    # -- broadcasts, reductions
    def set_vector_to_matrix_rows(self, h, w, vec):
        v = self.up(f32(vec))
        out = self.empty((h, w))
        self.call("nhSetVectorToMatrixRows", self.p(out), h, w, self.p(v))
        return self.down(out)

    def add_vector_to_matrix_rows(self, m, vec, inplace=False):
        m, v = self.up(f32(m)), self.up(f32(vec))
        b, h, w = m.shape
        out = m if inplace else self.empty(m.shape)
        self.call("nhAddVectorToMatrixRows", b, self.p(m), self.p(out), h, w, self.p(v))
        return self.down(out)

    def add_vector_to_matrix_columns(self, m, vec, sign=1):
        m, v = self.up(f32(m)), self.up(f32(vec))
        h, w = m.shape
        out = self.empty(m.shape)
        self.call("nhAddVectorToMatrixColumns" if sign > 0 else "nhSubVectorFromMatrixColumns",
                  self.p(m), self.p(out), h, w, self.p(v))
        return self.down(out)

    def sum_matrix_rows(self, m, add_to=None):
        m = self.up(f32(m))
        b, h, w = m.shape
        out = self.empty((b, w)) if add_to is None else self.up(f32(add_to))
        self.call("nhSumMatrixRows" if add_to is None else "nhSumMatrixRowsAdd", b, self.p(out), self.p(m), h, w)
        return self.down(out)

    def sum_matrix_columns(self, m):
        m = self.up(f32(m))
        out = self.empty((m.shape[0],))
        self.call("nhSumMatrixColumns", self.p(out), self.p(m), m.shape[0], m.shape[1])
        return self.down(out)

    def multiply_diag_matrix_by_matrix(self, d, m):
        d, m = self.up(f32(d)), self.up(f32(m))
        out = self.empty(m.shape)
        self.call("nhMultiplyDiagMatrixByMatrix", self.p(d), m.shape[0], self.p(m), m.shape[1], self.p(out), m.numel())
        return self.down(out)

    def batch_multiply_matrix_by_diag_matrix(self, batch, first, h, w, first_off, second, second_off):
        a, b = self.up(f32(first).ravel()), self.up(f32(second).ravel())
        out = self.empty((batch, h, w))
        self.call("nhBatchMultiplyMatrixByDiagMatrix", batch, self.p(a), h, w, first_off, self.p(b), second_off,
                  self.p(out), out.numel())
        return self.down(out)

    def softmax_rows(self, m, inplace=False):
        m = self.up(f32(m))
        out = m if inplace else self.empty(m.shape)
        self.call("nhMatrixSoftmaxByRows", self.p(m), m.shape[0], m.shape[1], self.p(out))
        return self.down(out)

    def log_sum_exp_rows(self, m):
        m = self.up(f32(m))
        out = self.empty((m.shape[0],))
        self.call("nhMatrixLogSumExpByRows", self.p(m), m.shape[0], m.shape[1], self.p(out), m.shape[0])
        return self.down(out)

    def find_max_in_rows(self, m, with_indices=True):
        m = self.up(f32(m))
        v = self.empty((m.shape[0],))
        idx = self.empty((m.shape[0],), np.int32) if with_indices else None
        self.call("nhFindMaxValueInRows", self.p(m), m.shape[0], m.shape[1], self.p(v), self.p(idx), m.shape[0])
        return self.down(v), (self.down(idx) if with_indices else None)

    def find_max_in_columns(self, m):
        m = self.up(f32(m))
        b, h, w = m.shape
        v, idx = self.empty((b, w)), self.empty((b, w), np.int32)
        self.call("nhFindMaxValueInColumns", b, self.p(m), h, w, self.p(v), self.p(idx), b * w)
        return self.down(v), self.down(idx)

    def transpose(self, x, integer=False):
        x = self.up(i32(x) if integer else f32(x))
        b, h, m, w, c = x.shape
        out = self.empty((b, w, m, h, c), np.int32 if integer else np.float32)
        self.call("nhTransposeMatrixInt" if integer else "nhTransposeMatrix", b, self.p(x), h, m, w, c, self.p(out), out.numel())
        return self.down(out)

    # -- matrix products
    def matmul(self, kind, a, b, c=None, lda=None, ldb=None, ldc=None, M=None, N=None, K=None, batch=1):
        a, b = self.up(f32(a).ravel()), self.up(f32(b).ravel())
        if kind == "nt":
            out = self.torch.zeros(((M - 1) * ldc + N,), dtype=self.torch.float32, device=self.dev)
            self.call("nhMultiplyMatrixByTransposedMatrix", self.p(a), M, K, lda, self.p(b), N, ldb, self.p(out), ldc, out.numel())
            return self.down(out)
        if kind == "tn_add":
            out = self.up(f32(c).ravel())
            self.call("nhMultiplyTransposedMatrixByMatrixAndAdd", self.p(a), K, M, lda, self.p(b), N, ldb, self.p(out), ldc, out.numel())
            return self.down(out)
        out = self.empty((batch, M, N))
        if kind == "bnt":
            self.call("nhBatchMultiplyMatrixByTransposedMatrix", batch, self.p(a), M, K, self.p(b), N, self.p(out), out.numel())
        elif kind == "bnn":
            self.call("nhBatchMultiplyMatrixByMatrix", batch, self.p(a), M, K, self.p(b), N, self.p(out), out.numel())
        else:
            self.call("nhBatchMultiplyTransposedMatrixByMatrix", batch, self.p(a), K, M, self.p(b), N, self.p(out), out.numel())
        return self.down(out)

    # -- convolution, pooling
    def conv_desc(self, n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh=1, dw=1, channelwise=False):
        d = self.na.ConvDesc(n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw, 0, 0)
        fn = self.lib.nhInitBlobChannelwiseConvolution if channelwise else self.lib.nhInitBlobConvolution
        self.na.check(fn(ctypes.byref(d)))
        return d

    def conv(self, x, filt, bias, ph, pw, sh, sw, dh=1, dw=1, activation=None, param=0.0):
        x, filt = f32(x), f32(filt)
        n, h, w, cin = x.shape
        cout, fh, fw, _ = filt.shape
        d = self.conv_desc(n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw)
        xs, fs, bs = self.up(x), self.up(filt), self.up(None if bias is None else f32(bias))
        out = self.empty((n, d.resultHeight, d.resultWidth, cout))
        if activation is None:
            self.call("nhBlobConvolution", ctypes.byref(d), self.p(xs), self.p(fs), self.p(bs), self.p(out))
        else:
            self.call("nhBlobConvolutionWithActivation", ctypes.byref(d), self.p(xs), self.p(fs), self.p(bs),
                      Cpu.ACTIVATIONS[activation], param, self.p(out))
        return self.down(out)

    def channelwise_conv(self, x, filt, bias, ph, pw, sh, sw):
        x, filt = f32(x), f32(filt)
        n, h, w, c = x.shape
        fh, fw, _ = filt.shape
        d = self.conv_desc(n, h, w, c, c, fh, fw, ph, pw, sh, sw, channelwise=True)
        xs, fs, bs = self.up(x), self.up(filt), self.up(None if bias is None else f32(bias))
        out = self.empty((n, d.resultHeight, d.resultWidth, c))
        self.call("nhBlobChannelwiseConvolution", ctypes.byref(d), self.p(xs), self.p(fs), self.p(bs), self.p(out))
        return self.down(out)

    def separable_block(self, x, expand, channelwise, down, stride=1, residual=False, in_place=False):
        x = f32(x)
        n, h, w, cin = x.shape
        ch_f, ch_t, ch_act, ch_param = channelwise
        dn_f, dn_t = down
        e, cout = ch_f.shape[2], dn_f.shape[0]
        ex_f, ex_t, ex_act, ex_param = expand if expand is not None else (None, None, None, 0.0)
        acts = Cpu.ACTIVATIONS
        d = self.na.SeparableBlockDesc(n, h, w, cin if expand is not None else 0, e, cout, stride, 1 if residual else 0,
                                       acts[ex_act], ex_param, acts[ch_act], ch_param)
        size = ctypes.c_size_t(0)
        which = "nhMobileNetV2Block" if expand is not None else "nhChannelwiseWith1x1"
        self.na.check(getattr(self.lib, which + "WorkspaceSize")(ctypes.byref(d), ctypes.byref(size)))
        work = self.torch.empty((size.value + 15) // 4 + 4, dtype=self.torch.float32, device=self.dev)
        xs = self.up(x)
        ho, wo = (h + stride - 1) // stride, (w + stride - 1) // stride
        out = xs if in_place else self.empty((n, ho, wo, cout))
        up = lambda a: self.up(None if a is None else f32(a))
        ws = [up(ex_f), up(ex_t), up(ch_f), up(ch_t), up(dn_f), up(dn_t)]
        if expand is not None:
            self.call(which, ctypes.byref(d), self.p(xs), self.p(ws[0]), self.p(ws[1]), self.p(ws[2]), self.p(ws[3]),
                      self.p(ws[4]), self.p(ws[5]), self.p(out), self.p(work), size.value)
        else:
            self.call(which, ctypes.byref(d), self.p(xs), self.p(ws[2]), self.p(ws[3]), self.p(ws[4]), self.p(ws[5]),
                      self.p(out), self.p(work), size.value)
        return self.down(out).reshape(n, ho, wo, cout)

    def mobilenetv3_pre_se(self, x, expand, channelwise, stride=1):
        x = f32(x)
        n, h, w, cin = x.shape
        ex_f, ex_t, ex_act, ex_param = expand
        ch_f, ch_t, ch_act, ch_param = channelwise
        fsize, e = ch_f.shape[0], ch_f.shape[2]
        pad = (fsize - 1) // 2
        d = self.conv_desc(n, h, w, e, e, fsize, fsize, pad, pad, stride, stride, channelwise=True)
        size = ctypes.c_size_t(0)
        self.na.check(self.lib.nhMobileNetV3PreSEBlockWorkspaceSize(ctypes.byref(d), ctypes.byref(size)))
        work = self.torch.empty((size.value + 15) // 4 + 4, dtype=self.torch.float32, device=self.dev)
        up = lambda a: self.up(None if a is None else f32(a))
        xs, ws = self.up(x), [up(ex_f), up(ex_t), up(ch_f), up(ch_t)]
        out = self.empty((n, d.resultHeight, d.resultWidth, e))
        acts = Cpu.ACTIVATIONS
        self.call("nhMobileNetV3PreSEBlock", ctypes.byref(d), cin, self.p(xs), self.p(ws[0]), self.p(ws[1]), acts[ex_act],
                  ex_param, self.p(ws[2]), self.p(ws[3]), acts[ch_act], ch_param, self.p(out), self.p(work), size.value)
        return self.down(out)

    def mobilenetv3_post_se(self, x, gate, residual, activation, param, down, in_place_residual=False):
        x, gate = f32(x), f32(gate)
        n, h, w, c = x.shape
        dn_f, dn_t = down
        cout = dn_f.shape[0]
        up = lambda a: self.up(None if a is None else f32(a))
        xs, gs, rs, fs, ts = self.up(x), self.up(gate), up(residual), up(dn_f), up(dn_t)
        work = self.torch.empty(x.size + 4, dtype=self.torch.float32, device=self.dev)
        out = rs if in_place_residual else self.empty((n, h, w, cout))
        self.call("nhMobileNetV3PostSEBlock", n, h * w, c, cout, self.p(xs), self.p(gs), self.p(rs), Cpu.ACTIVATIONS[activation],
                  param, self.p(fs), self.p(ts), self.p(out), self.p(work), x.size * 4)
        return self.down(out).reshape(n, h, w, cout)

    # -- gradients
    def conv_backward(self, out_diff, filt, bias, in_shape, ph, pw, sh, sw, dh=1, dw=1):
        out_diff, filt = f32(out_diff), f32(filt)
        n, h, w, cin = in_shape
        cout, fh, fw, _ = filt.shape
        d = self.conv_desc(n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw)
        size = ctypes.c_size_t(0)
        self.na.check(self.lib.nhBlobConvolutionBackwardWorkspaceSize(ctypes.byref(d), ctypes.byref(size)))
        work = self.torch.empty((size.value + 15) // 4 + 4, dtype=self.torch.float32, device=self.dev)
        gs, fs, bs = self.up(out_diff), self.up(filt), self.up(None if bias is None else f32(bias))
        out = self.empty(in_shape)
        self.call("nhBlobConvolutionBackward", ctypes.byref(d), self.p(gs), self.p(fs), self.p(bs), self.p(out),
                  self.p(work), size.value)
        return self.down(out)

    def conv_learn_add(self, x, out_diff, filter_diff, ph, pw, sh, sw, dh=1, dw=1):
        x, out_diff, filter_diff = f32(x), f32(out_diff), f32(filter_diff)
        n, h, w, cin = x.shape
        cout, fh, fw, _ = filter_diff.shape
        d = self.conv_desc(n, h, w, cin, cout, fh, fw, ph, pw, sh, sw, dh, dw)
        xs, gs, fd = self.up(x), self.up(out_diff), self.up(filter_diff)
        self.call("nhBlobConvolutionLearnAdd", ctypes.byref(d), self.p(xs), self.p(gs), self.p(fd))
        return self.down(fd)

    def channelwise_conv_backward(self, out_diff, filt, in_shape, ph, pw, sh, sw):
        out_diff, filt = f32(out_diff), f32(filt)
        n, h, w, c = in_shape
        fh, fw, _ = filt.shape
        d = self.conv_desc(n, h, w, c, c, fh, fw, ph, pw, sh, sw, channelwise=True)
        gs, fs = self.up(out_diff), self.up(filt)
        out = self.empty(in_shape)
        self.call("nhBlobChannelwiseConvolutionBackward", ctypes.byref(d), self.p(gs), self.p(fs), self.p(out))
        return self.down(out)

    def channelwise_conv_learn_add(self, x, out_diff, filter_diff, ph, pw, sh, sw, free_term_diff=None):
        x, out_diff = f32(x), f32(out_diff)
        n, h, w, c = x.shape
        fh, fw, _ = filter_diff.shape
        d = self.conv_desc(n, h, w, c, c, fh, fw, ph, pw, sh, sw, channelwise=True)
        xs, gs, fd = self.up(x), self.up(out_diff), self.up(f32(filter_diff))
        ftd = self.up(None if free_term_diff is None else f32(free_term_diff))
        self.call("nhBlobChannelwiseConvolutionLearnAdd", ctypes.byref(d), self.p(xs), self.p(gs), self.p(fd), self.p(ftd))
        return self.down(fd) if ftd is None else (self.down(fd), self.down(ftd))

    def max_pool_backward(self, x, result_diff, fh, fw, sh, sw):
        x = f32(x)
        n, h, w, c = x.shape
        d = self.pool_desc(n, h, w, c, fh, fw, sh, sw)
        xs, gs = self.up(x), self.up(f32(result_diff))
        out = self.empty((n, d.resultHeight, d.resultWidth, c))
        idx = self.empty(out.shape, np.int32)
        self.call("nhBlobMaxPooling", ctypes.byref(d), self.p(xs), self.p(idx), self.p(out))
        src_diff = self.empty(x.shape)
        self.call("nhBlobMaxPoolingBackward", ctypes.byref(d), self.p(gs), self.p(idx), self.p(src_diff))
        return self.down(src_diff)

    def mean_pool_backward(self, in_shape, result_diff, fh, fw, sh, sw):
        n, h, w, c = in_shape
        d = self.pool_desc(n, h, w, c, fh, fw, sh, sw)
        gs = self.up(f32(result_diff))
        src_diff = self.empty(in_shape)
        self.call("nhBlobMeanPoolingBackward", ctypes.byref(d), self.p(gs), self.p(src_diff))
        return self.down(src_diff)

    def pool_desc(self, n, h, w, c, fh, fw, sh, sw):
        d = self.na.PoolingDesc(n, h, w, c, fh, fw, sh, sw, 0, 0)
        self.na.check(self.lib.nhInitPooling(ctypes.byref(d)))
        return d

    def max_pool(self, x, fh, fw, sh, sw, with_indices=False):
        x = f32(x)
        n, h, w, c = x.shape
        d = self.pool_desc(n, h, w, c, fh, fw, sh, sw)
        xs = self.up(x)
        out = self.empty((n, d.resultHeight, d.resultWidth, c))
        idx = self.empty(out.shape, np.int32) if with_indices else None
        self.call("nhBlobMaxPooling", ctypes.byref(d), self.p(xs), self.p(idx), self.p(out))
        return (self.down(out), self.down(idx)) if with_indices else self.down(out)

    def mean_pool(self, x, fh, fw, sh, sw):
        x = f32(x)
        n, h, w, c = x.shape
        d = self.pool_desc(n, h, w, c, fh, fw, sh, sw)
        xs = self.up(x)
        out = self.empty((n, d.resultHeight, d.resultWidth, c))
        self.call("nhBlobMeanPooling", ctypes.byref(d), self.p(xs), self.p(out))
        return self.down(out)

    def resize_image(self, x, dl, dr, dt, db, padding=0, value=0.0):
        x = f32(x)
        n, h, w, c = x.shape
        fd = self.na.BlobDesc.of(1, n, 1, h, w, 1, c)
        td = self.na.BlobDesc.of(1, n, 1, h + dt + db, w + dl + dr, 1, c)
        xs = self.up(x)
        out = self.empty((n, h + dt + db, w + dl + dr, c))
        self.call("nhBlobResizeImage", ctypes.byref(fd), self.p(xs), dl, dr, dt, db, padding, ctypes.c_float(value),
                  ctypes.byref(td), self.p(out))
        return self.down(out)

    def dropout(self, x, rate, spatial=False, batchwise=False, seed=1, inplace=False):
        x = f32(x)
        xs = self.up(x)
        out = xs if inplace else self.empty(x.shape)
        self.call("nhDropout", ctypes.byref(self.na.BlobDesc.of(*x.shape)), rate, 1 if spatial else 0, 1 if batchwise else 0, seed,
                  self.p(xs), self.p(out))
        return self.down(out)

    def broadcast_copy(self, x, to_dims, width=1):
        x = f32(x)
        xs = self.up(x)
        out = self.empty(tuple(to_dims) + (width,))
        self.call("nhBroadcastCopy", self.p(out), self.p(xs), ctypes.byref(self.na.BlobDesc.of(*to_dims)),
                  ctypes.byref(self.na.BlobDesc.of(*x.shape[:7])), width)
        return self.down(out)

    def split(self, big, dim, part_dims):
        big = f32(big)
        bs = self.up(big)
        parts = [self.empty(d) for d in part_dims]
        descs = (self.na.BlobDesc * len(parts))(*[self.na.BlobDesc.of(*d) for d in part_dims])
        ptrs = (ctypes.c_void_p * len(parts))(*[p.data_ptr() for p in parts])
        bd = self.na.BlobDesc.of(*big.shape)
        self.call("nhBlobSplitByDim", dim, ctypes.byref(bd), self.p(bs), descs, ptrs, len(parts))
        return [self.down(p) for p in parts]

    def merge(self, parts, dim, big_dims):
        ps = [self.up(f32(p)) for p in parts]
        descs = (self.na.BlobDesc * len(ps))(*[self.na.BlobDesc.of(*p.shape) for p in parts])
        ptrs = (ctypes.c_void_p * len(ps))(*[p.data_ptr() for p in ps])
        out = self.empty(big_dims)
        bd = self.na.BlobDesc.of(*big_dims)
        self.call("nhBlobMergeByDim", dim, descs, ptrs, len(ps), ctypes.byref(bd), self.p(out))
        return self.down(out)

    def lstm(self, w_in, b_in, w_rec, b_rec, x, reverse=False, c0=None, h0=None, want_state=True, return_sync=False):
        x = f32(x)
        T, B, In = x.shape
        H = w_rec.shape[1]
        ws = [self.up(None if a is None else f32(a)) for a in (w_in, b_in, w_rec, b_rec, c0, h0, x)]
        h = self.empty((T, B, H))
        c = self.empty((T, B, H)) if want_state else None
        size = ctypes.c_size_t(0)
        self.na.check(self.lib.nhLstmWorkspaceSize(H, In, T, B, ctypes.byref(size)))
        work = self.torch.empty((size.value + 15) // 4, dtype=self.torch.float32, device=self.dev)
        self.call("nhLstm", H, In, self.p(ws[0]), self.p(ws[1]), self.p(ws[2]), self.p(ws[3]), 1 if reverse else 0, T, B,
                  self.p(ws[4]), self.p(ws[5]), self.p(ws[6]), self.p(c), self.p(h), self.p(work), size.value)
        if return_sync:
            # the last 8 bytes of the workspace hold the abort word of the one-launch path
            word = int(work.view(self.torch.int32)[size.value // 4 - 2].item())
            return self.down(h), (self.down(c) if want_state else None), word
        return self.down(h), (self.down(c) if want_state else None)


class CpuBackend:
    """Host backend for workloads: the same network code on numpy arrays, executed by the oracle
    ('orc') or by the reference's CPU engine ('ref')."""

    def __init__(self, kind):
        self.cpu = Cpu(kind)
        self.name = kind

    def tensor(self, a):
        return f32(a)

    def to_numpy(self, t):
        return t

    def synchronize(self):
        pass

    def conv(self, x, filt, bias, ph, pw, sh, sw, out=None, relu=False):
        y = self.cpu.conv(x, filt, bias, ph, pw, sh, sw)
        return self.cpu.unary("relu", y, 0.0 if relu is True else float(relu)).reshape(y.shape) if relu else y

    def relu_(self, x, threshold=None):
        x[...] = self.cpu.unary("relu", x, 0.0 if threshold is None else threshold).reshape(x.shape)
        return x

    def add_(self, a, b):
        a[...] = self.cpu.binary("add", a, b).reshape(a.shape)
        return a

    def pad(self, x, dl, dr, dt, db, value=0.0, out=None):
        return self.cpu.resize_image(x, dl, dr, dt, db, 0, value)

    def max_pool(self, x, fh, fw, sh, sw, out=None):
        return self.cpu.max_pool(x, fh, fw, sh, sw)

    def global_mean(self, x, out=None):
        n, h, w, c = x.shape
        s = self.cpu.sum_matrix_rows(x.reshape(n, h * w, c))
        return self.cpu.unary("multiply", s, np.float32(1.0 / (h * w))).reshape(n, c)

    def fc(self, x, weight, bias, out=None):
        m, k = x.shape
        n = weight.shape[0]
        y = self.cpu.matmul("nt", x, weight, lda=k, ldb=k, ldc=n, M=m, N=n, K=k).reshape(1, m, n)
        return self.cpu.add_vector_to_matrix_rows(y, bias.reshape(1, n)).reshape(m, n)

    def softmax(self, x, out=None):
        return self.cpu.softmax_rows(x)

    # ---- ops of the depthwise-separable, transformer and line-recogniser configurations
    def relu6_(self, x):
        x[...] = self.cpu.unary("relu", x, 6.0).reshape(x.shape)
        return x

    def channelwise_conv(self, x, filt, bias, ph, pw, sh, sw, out=None):
        return self.cpu.channelwise_conv(x, filt, bias, ph, pw, sh, sw)

    def separable_block(self, x, expand, channelwise, down, stride, residual, out=None):
        ex = None if expand is None else (expand[0].reshape(expand[0].shape[0], -1), expand[1], "relu", 6.0)
        return self.cpu.separable_block(x, ex, (channelwise[0], channelwise[1], "relu", 6.0),
                                        (down[0].reshape(down[0].shape[0], -1), down[1]), stride, residual)

    def pointwise_conv_relu6(self, x, filt, bias, out=None):
        y = self.cpu.conv(x, filt, bias, 0, 0, 1, 1)
        return self.cpu.unary("relu", y, 6.0).reshape(y.shape)

    def add(self, a, b, out=None):
        return self.cpu.binary("add", a, b).reshape(a.shape)

    def mul_scalar_(self, x, value, family=None):
        x[...] = self.cpu.unary("multiply", x, np.float32(value)).reshape(x.shape)
        return x

    def transpose(self, x, out=None):
        return self.cpu.transpose(x)

    def bmm_nn(self, a, b, out=None):
        batch, m, k = a.shape
        return self.cpu.matmul("bnn", a, b, M=m, N=b.shape[2], K=k, batch=batch)

    def layer_norm(self, x, scale, bias, out=None, eps=1e-5):
        c = self.cpu
        rows, width = x.shape
        neg_mean = c.unary("neg_multiply", c.sum_matrix_columns(x), np.float32(1.0 / width))
        sq = c.add_vector_to_matrix_columns(x, neg_mean)
        sq = c.binary("eltwise_multiply", sq, sq)
        var = c.unary("multiply", c.sum_matrix_columns(sq), np.float32(1.0 / width))
        inv_std = c.unary("inv", c.unary("sqrt", c.unary("add_value", var, np.float32(eps))))
        y = c.multiply_diag_matrix_by_matrix(inv_std, c.add_vector_to_matrix_columns(x, neg_mean))
        y = c.batch_multiply_matrix_by_diag_matrix(1, y, rows, width, 0, scale, 0)
        return c.add_vector_to_matrix_rows(y.reshape(1, rows, width), bias.reshape(1, width)).reshape(rows, width)

    def gelu_(self, x):
        c = self.cpu
        t = c.unary("sigmoid", c.unary("multiply", x, np.float32(1.702)))
        x[...] = c.binary("eltwise_multiply", x, t).reshape(x.shape)
        return x

    def lstm(self, x, w_in, b_in, w_rec, b_rec, reverse=False, out=None):
        h, _ = self.cpu.lstm(w_in, b_in, w_rec, b_rec, x, reverse=reverse, want_state=False)
        return h

    def merge_channels(self, parts, out=None):
        rows = parts[0].shape[0]
        total = sum(p.shape[1] for p in parts)
        parts7 = [f32(p).reshape(1, rows, 1, 1, 1, 1, p.shape[1]) for p in parts]
        return self.cpu.merge(parts7, 6, (1, rows, 1, 1, 1, 1, total)).reshape(rows, total)

    def log_(self, x):
        x[...] = self.cpu.unary("log", x).reshape(x.shape)
        return x

    def argmax_rows(self, x):
        return self.cpu.find_max_in_rows(x)[1]
