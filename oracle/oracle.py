"""ctypes binding of the C oracle declared in llmi_oracle.h.

TEST INFRASTRUCTURE ONLY. The numpy wrappers below add no arithmetic of their
own: they allocate, call the C function and return its result.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libllmi_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_i32 = ctypes.c_int32


def build(force=False):
    """Compile the oracle with the Makefile beside it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "libllmi_oracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.llmi_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.llmi_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.llmi_oracle_bf16_to_f32.restype = ctypes.c_float
        L.llmi_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.llmi_oracle_f32_to_bf16_n.restype = None
        L.llmi_oracle_f32_to_bf16_n.argtypes = [_f32p, _u16p, ctypes.c_size_t]
        L.llmi_oracle_bf16_to_f32_n.restype = None
        L.llmi_oracle_bf16_to_f32_n.argtypes = [_u16p, _f32p, ctypes.c_size_t]
        L.llmi_oracle_dot_scaled.restype = ctypes.c_float
        L.llmi_oracle_dot_scaled.argtypes = [_f32p, _f32p, _i32, ctypes.c_float]
        L.llmi_oracle_softmax_inplace.restype = None
        L.llmi_oracle_softmax_inplace.argtypes = [_f32p, _i32]
        L.llmi_oracle_scale_sum.restype = None
        L.llmi_oracle_scale_sum.argtypes = [_f32p, _f32p, _f32p, _i32, _i32, _i32]
        L.llmi_oracle_mha_cpu.restype = ctypes.c_int
        L.llmi_oracle_mha_cpu.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p] + [_i32] * 7
        L.llmi_oracle_mha_cpu_bf16.restype = ctypes.c_int
        L.llmi_oracle_mha_cpu_bf16.argtypes = [_u16p, _f32p, _u16p, _u16p, _f32p] + [_i32] * 7
        L.llmi_oracle_split_partial.restype = None
        L.llmi_oracle_split_partial.argtypes = [_f32p, _f32p, _f32p, _i32, _i32, _i32, _i32,
                                                ctypes.c_float, _f32p, _f32p, _f32p]
        L.llmi_oracle_combine.restype = None
        L.llmi_oracle_combine.argtypes = [_f32p, _f32p, _f32p, _i32, _i32, _f32p]
        L.llmi_oracle_sincos_table.restype = None
        L.llmi_oracle_sincos_table.argtypes = [_f32p, _f32p, _i32, _i32]
        L.llmi_oracle_qk_norm_rope.restype = None
        L.llmi_oracle_qk_norm_rope.argtypes = [_u16p, _i32, _i32, _u16p, _f32p, _f32p,
                                               ctypes.c_float]
        L.llmi_oracle_gemv_bf16.restype = None
        L.llmi_oracle_gemv_bf16.argtypes = [_u16p, _u16p, _i32, _i32, _f32p]
        _lib = L
    return _lib


def _f(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_f32p)


def _u(a):
    assert a.dtype == np.uint16 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_u16p)


def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.empty(x.shape, dtype=np.uint16)
    lib().llmi_oracle_f32_to_bf16_n(_f(x), _u(y), x.size)
    return y


def bf16_to_f32(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    y = np.empty(x.shape, dtype=np.float32)
    lib().llmi_oracle_bf16_to_f32_n(_u(x), _f(y), x.size)
    return y


def dot_scaled(q, k, scale):
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k, dtype=np.float32)
    return float(lib().llmi_oracle_dot_scaled(_f(q), _f(k), q.size, scale))


def softmax(x):
    y = np.array(x, dtype=np.float32, copy=True, order="C")
    lib().llmi_oracle_softmax_inplace(_f(y), y.size)
    return y


def scale_sum(score, value, pos, head_dim, kv_dim, out=None):
    score = np.ascontiguousarray(score, dtype=np.float32)
    value = np.ascontiguousarray(value, dtype=np.float32)
    if out is None:
        out = np.zeros(head_dim, dtype=np.float32)
    lib().llmi_oracle_scale_sum(_f(score), _f(value), _f(out), pos, head_dim, kv_dim)
    return out


def mha_cpu(query, key_cache, value_cache, layer_id, pos, kv_dim, kv_mul, head_num, head_dim,
            max_seq_len, return_score=False):
    """CPU attention op on position-major caches [layers][max_seq_len][kv_dim].

    fp32 arrays go through llmi_oracle_mha_cpu; uint16 (bf16 bit patterns)
    through llmi_oracle_mha_cpu_bf16. Output is fp32 [head_num*head_dim].
    """
    score = np.zeros((head_num, max_seq_len), dtype=np.float32)
    out = np.zeros(head_num * head_dim, dtype=np.float32)
    args = (layer_id, pos, kv_dim, kv_mul, head_num, head_dim, max_seq_len)
    if query.dtype == np.uint16:
        rc = lib().llmi_oracle_mha_cpu_bf16(_u(query), _f(score), _u(key_cache), _u(value_cache),
                                            _f(out), *args)
    else:
        rc = lib().llmi_oracle_mha_cpu(_f(query), _f(score), _f(key_cache), _f(value_cache),
                                       _f(out), *args)
    if rc != 0:
        raise ValueError("oracle rejected the arguments (the reference would CHECK-fail)")
    return (out, score) if return_score else out


def split_partial(q_head, key_base, value_base, begin, end, head_dim, kv_dim, scale):
    o = np.zeros(head_dim, dtype=np.float32)
    m = ctypes.c_float()
    l = ctypes.c_float()
    lib().llmi_oracle_split_partial(_f(q_head), _f(key_base), _f(value_base), begin, end,
                                    head_dim, kv_dim, scale, _f(o), ctypes.byref(m),
                                    ctypes.byref(l))
    return o, m.value, l.value


def combine(o, m, l):
    o = np.ascontiguousarray(o, dtype=np.float32)
    m = np.ascontiguousarray(m, dtype=np.float32)
    l = np.ascontiguousarray(l, dtype=np.float32)
    out = np.zeros(o.shape[1], dtype=np.float32)
    lib().llmi_oracle_combine(_f(o), _f(m), _f(l), o.shape[0], o.shape[1], _f(out))
    return out


def sincos_table(head_dim, max_seq_len):
    s = np.zeros((max_seq_len, head_dim // 2), dtype=np.float32)
    c = np.zeros((max_seq_len, head_dim // 2), dtype=np.float32)
    lib().llmi_oracle_sincos_table(_f(s), _f(c), head_dim, max_seq_len)
    return s, c


def qk_norm_rope(x, weight, sin_row, cos_row, eps=1e-6):
    """x: uint16 [n_heads, head_dim]; returns the transformed copy."""
    y = np.array(x, dtype=np.uint16, copy=True, order="C")
    weight = np.ascontiguousarray(weight, dtype=np.uint16)
    sin_row = np.ascontiguousarray(sin_row, dtype=np.float32)
    cos_row = np.ascontiguousarray(cos_row, dtype=np.float32)
    lib().llmi_oracle_qk_norm_rope(_u(y), y.shape[0], y.shape[1], _u(weight), _f(sin_row),
                                   _f(cos_row), eps)
    return y


def gemv_bf16(x, w):
    """x: uint16 [k], w: uint16 [n, k]; returns the fp32 sums [n] (before any output rounding)."""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    w = np.ascontiguousarray(w, dtype=np.uint16)
    n, k = w.shape
    assert x.shape == (k,) and k % 8 == 0
    out = np.empty(n, dtype=np.float32)
    lib().llmi_oracle_gemv_bf16(_u(x), _u(w), n, k, _f(out))
    return out
