"""numpy-facing bindings of the CPU oracle (libhom_oracle.so) and of the
single-threaded CPU baseline (libhom_cpu_baseline.so).

TEST INFRASTRUCTURE ONLY.  Importers: tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py -- never the product library.
"""
import ctypes
import os
import subprocess
from ctypes import POINTER, c_double, c_float, c_int, c_int32, c_int64, c_uint16, c_void_p

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_LIB = os.path.join(HERE, "libhom_oracle.so")
BASELINE_LIB = os.path.join(HERE, "libhom_cpu_baseline.so")


def build(force=False):
    cmd = ["make", "-C", HERE]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


def _ptr(a):
    return a.ctypes.data_as(c_void_p) if a is not None else None


_lib = None
_base = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_LIB):
            build()
        L = ctypes.CDLL(ORACLE_LIB)
        L.hom_oracle_half_to_float.restype = c_float
        L.hom_oracle_half_to_float.argtypes = [c_uint16]
        L.hom_oracle_float_to_half.restype = c_uint16
        L.hom_oracle_float_to_half.argtypes = [c_float]
        for n in ("hom_oracle_gelu_erf", "hom_oracle_gelu_tanh", "hom_oracle_gelu_poly"):
            getattr(L, n).restype = c_double
            getattr(L, n).argtypes = [c_double]
        L.hom_oracle_gemm.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int64,
                                      c_int64, c_int64, c_int64, c_int64, c_float,
                                      c_float, c_int, c_int]
        L.hom_oracle_layernorm_f16.argtypes = [c_void_p] * 5 + [c_int64, c_int64, c_float]
        L.hom_oracle_layernorm_f32.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_float]
        L.hom_oracle_row_stats.argtypes = [c_void_p] * 3 + [c_int64, c_int64, c_float]
        L.hom_oracle_attention.argtypes = [c_void_p] * 3 + [c_int64] * 4 + [c_float]
        L.hom_oracle_cu_seqlens_i64.argtypes = [c_void_p, c_void_p, c_int64, c_int64]
        L.hom_oracle_cu_seqlens_i32.argtypes = [c_void_p, c_void_p, c_int64, c_int64]
        ew = [c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p]
        L.hom_oracle_elementwise_f16.argtypes = ew
        L.hom_oracle_elementwise_f32.argtypes = ew
        L.hom_oracle_gather.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int64]
        L.hom_oracle_bert_encoder.argtypes = [c_void_p, c_void_p, c_void_p] + [c_int64] * 6 + \
            [c_float, c_int, c_int]
        _lib = L
    return _lib


def baseline():
    global _base
    if _base is None:
        if not os.path.exists(BASELINE_LIB):
            build()
        L = ctypes.CDLL(BASELINE_LIB)
        L.hom_cpu_matmul_add_f32.argtypes = [c_void_p] * 4 + [c_int64] * 4 + [c_int, c_int]
        L.hom_cpu_gelu_tosa_f32.argtypes = [c_void_p] * 4 + [c_int64]
        L.hom_cpu_layernorm_tosa_f32.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_float]
        L.hom_cpu_add_f32.argtypes = [c_void_p] * 3 + [c_int64]
        L.hom_cpu_attention_f32.argtypes = [c_void_p] * 4 + [c_int64] * 4 + [c_float]
        _base = L
    return _base


def _f16(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


ACT = {"linear": 0, "gelu_erf": 1, "gelu_tanh": 2, "gelu_poly": 3}


def gemm(A, B, C=None, alpha=1.0, beta=0.0, act="linear", b_is_nk=False):
    """A [M,K] f16, B [K,N] (or [N,K] if b_is_nk) f16, C [rowsC,N] f16 broadcast
    with period rowsC over the rows of D.  Returns float32 [M,N]."""
    A, B = _f16(A), _f16(B)
    M, K = A.shape
    N = B.shape[0] if b_is_nk else B.shape[1]
    assert (B.shape[1] if b_is_nk else B.shape[0]) == K
    D = np.empty((M, N), np.float32)
    period, ldc = 1, 0
    if C is not None and beta != 0.0:
        C = _f16(C).reshape(-1, N)
        period, ldc = C.shape[0], N
    lib().hom_oracle_gemm(_ptr(A), _ptr(B), _ptr(C) if (C is not None and beta != 0.0) else None,
                          _ptr(D), M, N, K, ldc, period, alpha, beta, ACT[act], int(b_is_nk))
    return D


def layernorm_f16(x, eps, res=None, gamma=None, beta=None):
    x = _f16(x)
    hidden = x.shape[-1]
    rows = x.size // hidden
    out = np.empty(x.shape, np.float32)
    res = _f16(res) if res is not None else None
    gamma = _f16(gamma) if gamma is not None else None
    beta = _f16(beta) if beta is not None else None
    lib().hom_oracle_layernorm_f16(_ptr(x), _ptr(res), _ptr(gamma), _ptr(beta), _ptr(out),
                                   rows, hidden, eps)
    return out


def layernorm_f32(x, eps):
    x = np.ascontiguousarray(x, np.float32)
    hidden = x.shape[-1]
    out = np.empty_like(x)
    lib().hom_oracle_layernorm_f32(_ptr(x), _ptr(out), x.size // hidden, hidden, eps)
    return out


def row_stats(d, eps):
    d = np.ascontiguousarray(d, np.float32)
    rows, n = d.shape
    var, mean = np.empty(rows, np.float32), np.empty(rows, np.float32)
    lib().hom_oracle_row_stats(_ptr(d), _ptr(var), _ptr(mean), rows, n, eps)
    return var, mean


def attention(qkv, cu, heads, scale):
    qkv = _f16(qkv)
    bs, seq, w = qkv.shape
    d = w // (3 * heads)
    cu = np.ascontiguousarray(cu, np.int32)
    out = np.empty((bs, seq, heads * d), np.float32)
    lib().hom_oracle_attention(_ptr(qkv), _ptr(cu), _ptr(out), bs, seq, heads, d, scale)
    return out


def cu_seqlens(mask):
    mask = np.ascontiguousarray(mask)
    bs, seq = mask.shape
    out = np.empty(bs + 1, np.int32)
    fn = lib().hom_oracle_cu_seqlens_i64 if mask.dtype == np.int64 else lib().hom_oracle_cu_seqlens_i32
    assert mask.dtype in (np.int64, np.int32)
    fn(_ptr(mask), _ptr(out), bs, seq)
    return out


OPS = {"add": 0, "sub": 1, "mul": 2, "div": 3}


def elementwise(op, a, b):
    """a op broadcast(b); b may have size-1 dims and any strides."""
    a = np.ascontiguousarray(a)
    assert a.ndim == b.ndim and a.dtype == b.dtype
    rank = a.ndim
    out = np.empty_like(a)
    ostride = np.array([s // a.itemsize for s in a.strides], np.int64) if a.size else np.ones(rank, np.int64)
    bsize = np.array(b.shape, np.int64)
    bstride = np.array([0 if b.shape[i] == 1 else b.strides[i] // b.itemsize for i in range(rank)], np.int64)
    # address B through its base buffer so that strided views work
    fn = lib().hom_oracle_elementwise_f16 if a.dtype == np.float16 else lib().hom_oracle_elementwise_f32
    assert a.dtype in (np.float16, np.float32)
    fn(OPS[op], _ptr(a), c_void_p(b.ctypes.data), _ptr(out), a.size, rank, _ptr(ostride),
       _ptr(bsize), _ptr(bstride))
    return out


def gather(indices, value):
    indices = np.ascontiguousarray(indices, np.int64)
    value = np.ascontiguousarray(value)
    H = value.shape[-1]
    out = np.empty(indices.shape + (H,), value.dtype)
    lib().hom_oracle_gather(_ptr(indices), _ptr(value), _ptr(out), indices.size, H * value.itemsize)
    return out


def gelu(x, form="erf"):
    fn = getattr(lib(), "hom_oracle_gelu_" + form)
    return np.array([fn(float(v)) for v in np.asarray(x, np.float64).ravel()]).reshape(np.shape(x))


def bert_encoder(h, weights, cu, layers, bs, seq, hidden, heads, ffn, eps=1e-12, gelu_form="erf",
                 round_intermediates=True):
    """h [bs*seq, hidden] f16, weights: flat f16 array of all layers (Wqkv, Wo, W1,
    W2 per layer, each [K, N] row-major).  round_intermediates=True rounds every
    tensor the GPU path stores as fp16 (fp16-boundary-faithful); False keeps
    them unrounded (pure fp32 reference).  Returns the final layer norm as
    float32 [bs, seq, hidden], before its own rounding to fp16."""
    h32 = np.ascontiguousarray(_f16(h).astype(np.float32)).reshape(bs * seq, hidden).copy()
    weights = _f16(weights)
    per_layer = hidden * 3 * hidden + hidden * hidden + 2 * hidden * ffn
    assert weights.size == layers * per_layer
    cu = np.ascontiguousarray(cu, np.int32)
    lib().hom_oracle_bert_encoder(_ptr(h32), _ptr(weights), _ptr(cu), layers, bs, seq, hidden,
                                  heads, ffn, eps, 1 if gelu_form == "erf" else 2,
                                  int(bool(round_intermediates)))
    return h32.reshape(bs, seq, hidden)
