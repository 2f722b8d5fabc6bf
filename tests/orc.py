"""numpy front-end of the CPU checker (oracle/libtnn_oracle.so).  Test infrastructure only."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB = os.path.join(ORACLE_DIR, "libtnn_oracle.so")

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.check_call(["make", "-C", ORACLE_DIR, LIB])
        _lib = C.CDLL(LIB)
        _lib.orc_float2int8.restype = C.c_int8
        _lib.orc_float2int8.argtypes = [C.c_float]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ints(v):
    return (C.c_int * max(len(v), 1))(*[int(x) for x in v])


def matmul(a, b):
    """a [..., M, N], b [..., N, K]; batches broadcast by modulo like the reference."""
    a, b = _f32(a), _f32(b)
    M, N = a.shape[-2:]
    K = b.shape[-1]
    assert b.shape[-2] == N
    ba, bb = a.size // (M * N), b.size // (N * K)
    lead = a.shape[:-2] if ba >= bb else b.shape[:-2]
    c = np.empty(lead + (M, K), np.float32)
    lib().orc_matmul_f32(_p(a), _p(b), _p(c), M, N, K, ba, bb, max(ba, bb))
    return c


def inner_product(x, w, bias=None):
    x, w = _f32(x), _f32(w)
    rows, K = x.shape
    N = w.shape[0]
    bias = None if bias is None else _f32(bias)
    y = np.empty((rows, N), np.float32)
    lib().orc_inner_product_f32(_p(x), _p(w), _p(bias), _p(y), rows, K, N)
    return y


def softmax(x, axis=-1):
    x = _f32(x)
    axis = axis % x.ndim
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    y = np.empty_like(x)
    lib().orc_softmax_f32(_p(x), _p(y), outer, x.shape[axis], inner)
    return y


def layernorm(x, gamma, beta, eps):
    x, gamma, beta = _f32(x), _f32(gamma), _f32(beta)
    cols = gamma.size
    y = np.empty_like(x)
    lib().orc_layernorm_f32(_p(x), _p(gamma), _p(beta), _p(y), x.size // cols, cols, C.c_float(eps))
    return y


def gelu(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_gelu_f32(_p(x), _p(y), C.c_size_t(x.size))
    return y


def binary(op, a, b):
    a, b = _f32(a), _f32(b)
    shape = np.broadcast_shapes(a.shape, b.shape)
    out = np.empty(shape, np.float32)
    lib().orc_binary_f32({"add": 0, "sub": 1, "mul": 2, "div": 3}[op], _p(a), _ints(a.shape), a.ndim, _p(b),
                         _ints(b.shape), b.ndim, _p(out), _ints(shape), len(shape))
    return out


def permute(x, order):
    x = np.ascontiguousarray(x)
    out = np.empty([x.shape[o] for o in order], x.dtype)
    lib().orc_permute(_p(x), _p(out), _ints(x.shape), _ints(order), x.ndim, x.itemsize)
    return out


def gather(data, indices, axis=0):
    data = np.ascontiguousarray(data)
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    batch = int(np.prod(data.shape[:axis], dtype=np.int64))
    slice_elems = int(np.prod(data.shape[axis + 1:], dtype=np.int64))
    out = np.zeros(data.shape[:axis] + indices.shape + data.shape[axis + 1:], data.dtype)
    rc = lib().orc_gather(_p(data), _p(indices), _p(out), batch, data.shape[axis],
                          C.c_size_t(slice_elems * data.itemsize), indices.size)
    return out, rc


def float2int8(v):
    v = _f32(v)
    out = np.empty(v.shape, np.int8)
    lib().orc_float2int8_array(_p(v), _p(out), C.c_size_t(v.size))
    return out


def fc_int8_scale(w_scale, o_scale, N):
    w_scale, o_scale = _f32(np.atleast_1d(w_scale)), _f32(np.atleast_1d(o_scale))
    s = np.empty(N, np.float32)
    lib().orc_fc_int8_scale(_p(w_scale), w_scale.size, _p(o_scale), o_scale.size, _p(s), N)
    return s


def fc_int8(x, w, bias, scale):
    x = np.ascontiguousarray(x, np.int8)
    w = np.ascontiguousarray(w, np.int8)
    bias = None if bias is None else np.ascontiguousarray(bias, np.int32)
    scale = _f32(scale)
    rows, K = x.shape
    N = w.shape[0]
    y = np.empty((rows, N), np.int8)
    acc = np.empty((rows, N), np.int32)
    lib().orc_fc_int8(_p(x), _p(w), _p(bias), _p(scale), _p(y), _p(acc), rows, K, N)
    return y, acc


def quantize_x86(x, scale):
    x = _f32(x)
    q = np.empty(x.shape, np.int8)
    lib().orc_quantize_x86(_p(x), C.c_float(scale), _p(q), C.c_size_t(x.size))
    return q


def quantize_naive(x, scale):
    x = _f32(x)
    q = np.empty(x.shape, np.int8)
    lib().orc_quantize_naive(_p(x), C.c_float(scale), _p(q), C.c_size_t(x.size))
    return q


def dequantize(q, scale):
    q = np.ascontiguousarray(q, np.int8)
    x = np.empty(q.shape, np.float32)
    lib().orc_dequantize(_p(q), C.c_float(scale), _p(x), C.c_size_t(q.size))
    return x


def add_int8_x86(a, sa, b, sb, so):
    """a, b: int8 arrays in the blob's own dims (channel axis 1, as the engine counts it)."""
    a = np.ascontiguousarray(a, np.int8)
    b = np.ascontiguousarray(b, np.int8)
    y = np.empty(a.shape, np.int8)
    channels = a.shape[1] if a.ndim >= 2 else 1
    inner = int(np.prod(a.shape[2:], dtype=np.int64)) if a.ndim > 2 else 1
    lib().orc_add_int8_x86(_p(a), C.c_float(sa), _p(b), C.c_float(sb), C.c_float(so), _p(y), C.c_size_t(a.size),
                           channels, C.c_size_t(inner))
    return y


def add_int8_naive(a, sa, b, sb, so):
    a = np.ascontiguousarray(a, np.int8)
    b = np.ascontiguousarray(b, np.int8)
    y = np.empty(a.shape, np.int8)
    lib().orc_add_int8_naive(_p(a), C.c_float(sa), _p(b), C.c_float(sb), C.c_float(so), _p(y), C.c_size_t(a.size))
    return y


def attention_core(q, k, v, scale, mask=None):
    """q,k,v [B,h,S,d]; mask additive [B,S] or None."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, h, S, d = q.shape
    mask = None if mask is None else _f32(mask)
    out = np.empty_like(q)
    lib().orc_attention_core_f32(_p(q), _p(k), _p(v), _p(mask), _p(out), B, h, S, d, C.c_float(scale))
    return out
