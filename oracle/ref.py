"""numpy front end of the C oracle (oracle/llc_oracle.c).  TEST INFRASTRUCTURE ONLY.

Each wrapper takes and returns contiguous numpy arrays; fp32 unless the name says otherwise.  bf16
cases are expressed the way the reference's lowering would compute them if it had the type: inputs
already rounded to bf16 values held in fp32, fp32 arithmetic, result rounded to bf16 by the caller
with `round_bf16`.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libllc_oracle.so")

UNARY = {"abs": 0, "sqrt": 1, "exp": 2, "relu": 3, "rsqrt": 4, "neg": 5, "gelu": 6, "tanh": 7,
         "erf": 8, "sigmoid": 9, "log": 10, "recip": 11}
BINARY = {"add": 0, "sub": 1, "mul": 2, "div": 3, "max": 4, "min": 5, "pow": 6}
COMPARE = {"EQ": 1, "GE": 2, "LE": 3, "GT": 4, "LT": 5, "NE": 6}
REDUCE = {"sum": 0, "max": 1, "min": 2}


def build(force=False):
    """Compile the oracle with the committed Makefile (gcc only)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libllc_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.llc_ref_window_out.restype = ctypes.c_int64
        _lib.llc_ref_window_out.argtypes = [ctypes.c_int64] * 6
        _lib.llc_ref_f32_to_bf16.restype = ctypes.c_uint16
        _lib.llc_ref_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.llc_ref_bf16_to_f32.restype = ctypes.c_float
        _lib.llc_ref_bf16_to_f32.argtypes = [ctypes.c_uint16]
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def _i64v(v):
    return (ctypes.c_int64 * len(v))(*[int(x) for x in v])


_c64 = ctypes.c_int64


def round_bf16(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().llc_ref_round_bf16(_p(x), _p(y), _c64(x.size))
    return y


def matmul(a, b, order="mnk"):
    """order: 'mnk' = the reference's loop nest; 'mkn' = same sums, cache friendly; 'f64' = fp64 accumulate."""
    a, b = _f32(a), _f32(b)
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    c = np.empty((M, N), np.float32)
    fn = {"mnk": lib().llc_ref_matmul_f32, "mkn": lib().llc_ref_matmul_f32_mkn,
          "f64": lib().llc_ref_matmul_f64acc}[order]
    fn(_p(a), _p(b), _p(c), _c64(M), _c64(N), _c64(K))
    return c


def batch_matmul(a, b, order="mnk"):
    a, b = _f32(a), _f32(b)
    B, M, K = a.shape
    B2, K2, N = b.shape
    assert B == B2 and K == K2
    c = np.empty((B, M, N), np.float32)
    fn = lib().llc_ref_batch_matmul_f32 if order == "mnk" else lib().llc_ref_batch_matmul_f32_mkn
    fn(_p(a), _p(b), _p(c), _c64(B), _c64(M), _c64(N), _c64(K))
    return c


def window_out(n, pad_lo, pad_hi, dil, k, stride):
    return int(lib().llc_ref_window_out(n, pad_lo, pad_hi, dil, k, stride))


def conv2d(x, w, bias=None, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), group=1):
    """pad = (h_lo, w_lo, h_hi, w_hi), the LLH attribute order."""
    x, w = _f32(x), _f32(w)
    N, C, H, W = x.shape
    F, Cg, KH, KW = w.shape
    assert Cg * group == C and F % group == 0
    OH = window_out(H, pad[0], pad[2], dilation[0], KH, stride[0])
    OW = window_out(W, pad[1], pad[3], dilation[1], KW, stride[1])
    y = np.empty((N, F, OH, OW), np.float32)
    b = None if bias is None else _f32(bias)
    lib().llc_ref_conv2d_f32(_p(x), _p(w), None if b is None else _p(b), _p(y), _c64(N), _c64(C), _c64(H),
                             _c64(W), _c64(F), _c64(KH), _c64(KW), _i64v(pad), _i64v(stride), _i64v(dilation),
                             _c64(group))
    return y


def unary(op, x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().llc_ref_unary_f32(UNARY[op], _p(x), _p(y), _c64(x.size))
    return y


def binary(op, a, b):
    if a.dtype == np.int64:
        a, b = _i64(a), _i64(b)
        assert a.shape == b.shape
        y = np.empty_like(a)
        lib().llc_ref_binary_i64(BINARY[op], _p(a), _p(b), _p(y), _c64(a.size))
        return y
    a, b = _f32(a), _f32(b)
    assert a.shape == b.shape
    y = np.empty_like(a)
    lib().llc_ref_binary_f32(BINARY[op], _p(a), _p(b), _p(y), _c64(a.size))
    return y


def compare(kind, a, b):
    assert a.shape == b.shape
    y = np.empty(a.shape, np.uint8)
    if a.dtype == np.int64:
        a, b = _i64(a), _i64(b)
        lib().llc_ref_compare_i64(COMPARE[kind], _p(a), _p(b), _p(y), _c64(a.size))
    else:
        a, b = _f32(a), _f32(b)
        lib().llc_ref_compare_f32(COMPARE[kind], _p(a), _p(b), _p(y), _c64(a.size))
    return y.astype(bool)


def where(pred, t, f):
    pred = np.ascontiguousarray(pred, dtype=np.uint8)
    t, f = _f32(t), _f32(f)
    y = np.empty_like(t)
    lib().llc_ref_where_f32(_p(pred), _p(t), _p(f), _p(y), _c64(t.size))
    return y


def convert(x, dtype):
    dtype = np.dtype(dtype)
    if x.dtype == np.float32 and dtype == np.int64:
        x = _f32(x)
        y = np.empty(x.shape, np.int64)
        lib().llc_ref_convert_f32_to_i64(_p(x), _p(y), _c64(x.size))
        return y
    if x.dtype == np.int64 and dtype == np.float32:
        x = _i64(x)
        y = np.empty(x.shape, np.float32)
        lib().llc_ref_convert_i64_to_f32(_p(x), _p(y), _c64(x.size))
        return y
    raise TypeError((x.dtype, dtype))


def broadcast_to(x, out_shape):
    x = np.ascontiguousarray(x)
    assert x.ndim == len(out_shape)
    y = np.empty(out_shape, x.dtype)
    lib().llc_ref_broadcast_to(_p(x), _p(y), x.ndim, _i64v(x.shape), _i64v(out_shape), x.itemsize)
    return y


def transpose(x, perms):
    x = np.ascontiguousarray(x)
    y = np.empty([x.shape[p] for p in perms], x.dtype)
    lib().llc_ref_transpose(_p(x), _p(y), x.ndim, _i64v(x.shape), _i64v(perms), x.itemsize)
    return y


def stride_slice(x, start, end, step):
    x = np.ascontiguousarray(x)
    oshape = (ctypes.c_int64 * x.ndim)()
    lib().llc_ref_stride_slice(_p(x), None, x.ndim, _i64v(x.shape), _i64v(start), _i64v(end), _i64v(step),
                               oshape, x.itemsize)
    y = np.empty(list(oshape), x.dtype)
    lib().llc_ref_stride_slice(_p(x), _p(y), x.ndim, _i64v(x.shape), _i64v(start), _i64v(end), _i64v(step),
                               oshape, x.itemsize)
    return y


def extract(x, index):
    x = np.ascontiguousarray(x)
    # (one element of a vector stays a tensor<1>: LLHinfersymbolShape.cpp:513-516)
    y = np.empty(x.shape[1:] if x.ndim > 1 else (1,), x.dtype)
    lib().llc_ref_extract(_p(x), _p(y), x.ndim, _i64v(x.shape), _c64(index), x.itemsize)
    return y


def gather_rows(table, idx):
    table = np.ascontiguousarray(table)
    idx = _i64(idx)
    row = int(np.prod(table.shape[1:])) if table.ndim > 1 else 1
    y = np.empty(idx.shape + table.shape[1:], table.dtype)
    lib().llc_ref_gather_rows(_p(table), _p(idx), _p(y), _c64(idx.size), _c64(row), table.itemsize)
    return y


def reduce(kind, x, axes):
    x = _f32(x)
    axes = [a % x.ndim for a in axes]
    oshape = [s for d, s in enumerate(x.shape) if d not in axes]
    y = np.empty(oshape, np.float32)
    lib().llc_ref_reduce_f32(REDUCE[kind], _p(x), _p(y), x.ndim, _i64v(x.shape), _i64v(axes), len(axes))
    return y


def softmax_lastdim(x):
    x = _f32(x)
    y = np.empty_like(x)
    cols = x.shape[-1]
    lib().llc_ref_softmax_lastdim_f32(_p(x), _p(y), _c64(x.size // cols), _c64(cols))
    return y


def layernorm_lastdim(x, gamma=None, beta=None, eps=1e-5):
    x = _f32(x)
    y = np.empty_like(x)
    cols = x.shape[-1]
    g = None if gamma is None else _f32(gamma)
    b = None if beta is None else _f32(beta)
    lib().llc_ref_layernorm_lastdim_f32(_p(x), None if g is None else _p(g), None if b is None else _p(b),
                                        _p(y), _c64(x.size // cols), _c64(cols), ctypes.c_float(eps))
    return y


def batch_norm_inference(x, scale, bias, mean, var, eps=1e-5):
    x = _f32(x)
    N, C = x.shape[:2]
    HW = x.size // (N * C)
    y = np.empty_like(x)
    s, b, m, v = _f32(scale), _f32(bias), _f32(mean), _f32(var)
    lib().llc_ref_batch_norm_inference_f32(_p(x), _p(s), _p(b), _p(m), _p(v), _p(y), _c64(N), _c64(C), _c64(HW),
                                           ctypes.c_float(eps))
    return y


def fold_bn_into_conv(w, b, scale, bias, mean, var, eps=1e-5):
    w = _f32(w)
    F = w.shape[0]
    per = w.size // F
    w2 = np.empty_like(w)
    b2 = np.empty(F, np.float32)
    bb = None if b is None else _f32(b)
    s, bi, m, v = _f32(scale), _f32(bias), _f32(mean), _f32(var)
    lib().llc_ref_fold_bn_into_conv_f32(_p(w), None if bb is None else _p(bb), _p(s), _p(bi), _p(m), _p(v),
                                        _p(w2), _p(b2), _c64(F), _c64(per), ctypes.c_float(eps))
    return w2, b2


def maxpool2d(x, kernel, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), init_zero=False):
    x = _f32(x)
    N, C, H, W = x.shape
    OH = window_out(H, pad[0], pad[2], dilation[0], kernel[0], stride[0])
    OW = window_out(W, pad[1], pad[3], dilation[1], kernel[1], stride[1])
    y = np.empty((N, C, OH, OW), np.float32)
    lib().llc_ref_maxpool2d_f32(_p(x), _p(y), _c64(N), _c64(C), _c64(H), _c64(W), _c64(kernel[0]),
                                _c64(kernel[1]), _i64v(pad), _i64v(stride), _i64v(dilation), int(init_zero))
    return y


def global_avgpool(x):
    x = _f32(x)
    N, C = x.shape[:2]
    y = np.empty((N, C), np.float32)
    lib().llc_ref_global_avgpool_f32(_p(x), _p(y), _c64(N * C), _c64(x.size // (N * C)))
    return y


def golden_abs():
    y = np.empty(2, np.float32)
    lib().llc_ref_golden_abs(_p(y))
    return y


def golden_i64_mul_to_f32():
    y = np.empty(1, np.float32)
    lib().llc_ref_golden_i64_mul_to_f32(_p(y))
    return y
