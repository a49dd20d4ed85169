"""ctypes binding of oracle/libkcg_oracle.so for the tests, smoke() and the
benchmark's cpu_baseline leg.  The oracle is the checker, never the product."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_DIR = os.path.join(os.path.dirname(_HERE), "oracle")
_SO = os.path.join(_ORACLE_DIR, "libkcg_oracle.so")

EW_OPS = {"Tanh": 0, "Sqrt": 1, "Log": 2, "Relu": 3, "Gelu": 4}


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _ORACLE_DIR, "-B" if force else "-s"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _declare(_lib)
    return _lib


def _p(a, ty=C.c_void_p):
    return a.ctypes.data_as(ty)


def _declare(L):
    f32p, f64p = C.POINTER(C.c_float), C.POINTER(C.c_double)
    i64, sz, u64 = C.c_int64, C.c_size_t, C.c_uint64
    L.kcg_oracle_fill_uniform.argtypes = [f32p, sz, u64, u64, C.c_float, C.c_float]
    L.kcg_oracle_fill_normal.argtypes = [f32p, sz, u64, u64, C.c_float, C.c_float]
    L.kcg_oracle_f32_to_bf16.argtypes = [C.c_float]
    L.kcg_oracle_f32_to_bf16.restype = C.c_uint16
    L.kcg_oracle_bf16_to_f32.argtypes = [C.c_uint16]
    L.kcg_oracle_bf16_to_f32.restype = C.c_float
    L.kcg_oracle_to_bf16.argtypes = [f32p, C.POINTER(C.c_uint16), sz]
    L.kcg_oracle_from_bf16.argtypes = [C.POINTER(C.c_uint16), f32p, sz]
    L.kcg_oracle_fp8e4m3_to_f32.argtypes = [C.c_uint8]
    L.kcg_oracle_fp8e4m3_to_f32.restype = C.c_float
    L.kcg_oracle_f32_to_fp8e4m3.argtypes = [C.c_float]
    L.kcg_oracle_f32_to_fp8e4m3.restype = C.c_uint8
    L.kcg_oracle_to_fp8e4m3.argtypes = [f32p, C.POINTER(C.c_uint8), sz, C.c_float]
    L.kcg_oracle_from_fp8e4m3.argtypes = [C.POINTER(C.c_uint8), f32p, sz]
    for name in ("kcg_oracle_matmul_f32_nest", "kcg_oracle_matmul_f32"):
        getattr(L, name).argtypes = [f32p, f32p, f32p, i64, i64, i64]
    L.kcg_oracle_matmul_f64acc.argtypes = [f32p, f32p, f64p, i64, i64, i64]
    L.kcg_oracle_matmul_rows_f64acc.argtypes = [f32p, f32p, f64p, i64, i64, i64, i64]
    L.kcg_oracle_batched_matmul_f32.argtypes = [f32p, f32p, f32p, i64, i64, i64, i64, C.c_int, C.c_int]
    L.kcg_oracle_batched_matmul_f64acc.argtypes = [f32p, f32p, f64p, i64, i64, i64, i64, C.c_int, C.c_int]
    L.kcg_oracle_softmax_f32.argtypes = [f32p, i64, i64]
    L.kcg_oracle_softmax_f64.argtypes = [f32p, f64p, i64, i64]
    L.kcg_oracle_layernorm_f32.argtypes = [f32p, f32p, f32p, f32p, i64, i64, i64, i64, C.c_float]
    L.kcg_oracle_layernorm_f64.argtypes = [f32p, f32p, f32p, f64p, i64, i64, i64, i64, C.c_double]
    L.kcg_oracle_gelu_scalar.argtypes = [C.c_float]
    L.kcg_oracle_gelu_scalar.restype = C.c_float
    L.kcg_oracle_elementwise_f32.argtypes = [f32p, f32p, sz, C.c_int]
    L.kcg_oracle_elementwise_f32.restype = C.c_int
    L.kcg_oracle_gelu_f64.argtypes = [f32p, f64p, sz]
    L.kcg_oracle_fmha_f32.argtypes = [f32p, f32p, f32p, f32p, i64, i64, i64, C.c_float, C.c_int]
    L.kcg_oracle_fmha_f64.argtypes = [f32p, f32p, f32p, f64p, i64, i64, i64, C.c_double, C.c_int]
    L.kcg_oracle_fmha_rows_f64.argtypes = [f32p, f32p, f32p, f64p, i64, i64, i64, i64, C.c_double, C.c_int]
    L.kcg_oracle_gather.argtypes = [C.c_void_p, C.POINTER(C.c_int64), C.c_void_p, i64, i64, i64, i64]
    L.kcg_oracle_gather.restype = C.c_int
    L.kcg_oracle_rel_frobenius_f32_f64.argtypes = [f32p, f64p, sz]
    L.kcg_oracle_rel_frobenius_f32_f64.restype = C.c_double


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _dp(a):
    return a.ctypes.data_as(C.POINTER(C.c_double))


SEED = 0x4B4347  # "KCG"


def uniform(shape, stream, lo=-1.0, hi=1.0, seed=SEED):
    out = np.empty(shape, dtype=np.float32)
    lib().kcg_oracle_fill_uniform(_fp(out), out.size, seed, stream, lo, hi)
    return out


def normal(shape, stream, mean=0.0, std=1.0, seed=SEED):
    out = np.empty(shape, dtype=np.float32)
    lib().kcg_oracle_fill_normal(_fp(out), out.size, seed, stream, mean, std)
    return out


def to_bf16_bits(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().kcg_oracle_to_bf16(_fp(x), out.ctypes.data_as(C.POINTER(C.c_uint16)), x.size)
    return out


def from_bf16_bits(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(b.shape, dtype=np.float32)
    lib().kcg_oracle_from_bf16(b.ctypes.data_as(C.POINTER(C.c_uint16)), _fp(out), b.size)
    return out


def round_bf16(x):
    return from_bf16_bits(to_bf16_bits(x))


def to_fp8_bits(x, inv_scale=1.0):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().kcg_oracle_to_fp8e4m3(_fp(x), out.ctypes.data_as(C.POINTER(C.c_uint8)), x.size, inv_scale)
    return out


def from_fp8_bits(b):
    b = np.ascontiguousarray(b, dtype=np.uint8)
    out = np.empty(b.shape, dtype=np.float32)
    lib().kcg_oracle_from_fp8e4m3(b.ctypes.data_as(C.POINTER(C.c_uint8)), _fp(out), b.size)
    return out


def matmul(A, B, nest=False):
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    Cm = np.empty((M, N), dtype=np.float32)
    fn = lib().kcg_oracle_matmul_f32_nest if nest else lib().kcg_oracle_matmul_f32
    fn(_fp(A), _fp(B), _fp(Cm), M, N, K)
    return Cm


def matmul_f64(A, B):
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    N = B.shape[1]
    Cm = np.empty((M, N), dtype=np.float64)
    lib().kcg_oracle_matmul_f64acc(_fp(A), _fp(B), _dp(Cm), M, N, K)
    return Cm


def matmul_rows_f64(A, B, row0, rows):
    A, B = _f32(A), _f32(B)
    K = A.shape[1]
    N = B.shape[1]
    Cm = np.empty((rows, N), dtype=np.float64)
    lib().kcg_oracle_matmul_rows_f64acc(_fp(A), _fp(B), _dp(Cm), row0, rows, N, K)
    return Cm


def _bmm_dims(A, B, transA, transB):
    batch = int(np.prod(A.shape[:-2])) if A.ndim > 2 else 1
    M, K = (A.shape[-1], A.shape[-2]) if transA else (A.shape[-2], A.shape[-1])
    N = B.shape[-2] if transB else B.shape[-1]
    return batch, M, N, K


def batched_matmul(A, B, transA=False, transB=False):
    A, B = _f32(A), _f32(B)
    batch, M, N, K = _bmm_dims(A, B, transA, transB)
    Cm = np.empty(A.shape[:-2] + (M, N), dtype=np.float32)
    lib().kcg_oracle_batched_matmul_f32(_fp(A), _fp(B), _fp(Cm), batch, M, N, K, int(transA), int(transB))
    return Cm


def batched_matmul_f64(A, B, transA=False, transB=False):
    A, B = _f32(A), _f32(B)
    batch, M, N, K = _bmm_dims(A, B, transA, transB)
    Cm = np.empty(A.shape[:-2] + (M, N), dtype=np.float64)
    lib().kcg_oracle_batched_matmul_f64acc(_fp(A), _fp(B), _dp(Cm), batch, M, N, K, int(transA), int(transB))
    return Cm


def softmax(X):
    X = _f32(X).copy()
    cols = X.shape[-1]
    lib().kcg_oracle_softmax_f32(_fp(X), X.size // cols, cols)
    return X


def softmax_f64(X):
    X = _f32(X)
    cols = X.shape[-1]
    Y = np.empty(X.shape, dtype=np.float64)
    lib().kcg_oracle_softmax_f64(_fp(X), _dp(Y), X.size // cols, cols)
    return Y


def layernorm(X, gamma, beta, axis, eps=1e-5):
    X, gamma, beta = _f32(X), _f32(gamma), _f32(beta)
    axis = axis + X.ndim if axis < 0 else axis
    rows = int(np.prod(X.shape[:axis])) if axis > 0 else 1
    n = X.size // rows
    Y = np.empty(X.shape, dtype=np.float32)
    lib().kcg_oracle_layernorm_f32(_fp(X), _fp(gamma), _fp(beta), _fp(Y), rows, n,
                                   gamma.size, beta.size, eps)
    return Y


def layernorm_f64(X, gamma, beta, axis, eps=1e-5):
    X, gamma, beta = _f32(X), _f32(gamma), _f32(beta)
    axis = axis + X.ndim if axis < 0 else axis
    rows = int(np.prod(X.shape[:axis])) if axis > 0 else 1
    n = X.size // rows
    Y = np.empty(X.shape, dtype=np.float64)
    lib().kcg_oracle_layernorm_f64(_fp(X), _fp(gamma), _fp(beta), _dp(Y), rows, n,
                                   gamma.size, beta.size, float(np.float32(eps)))
    return Y


def elementwise(X, op):
    X = _f32(X)
    Y = np.empty(X.shape, dtype=np.float32)
    rc = lib().kcg_oracle_elementwise_f32(_fp(X), _fp(Y), X.size, EW_OPS[op])
    assert rc == 0
    return Y


def gelu_f64(X):
    X = _f32(X)
    Y = np.empty(X.shape, dtype=np.float64)
    lib().kcg_oracle_gelu_f64(_fp(X), _dp(Y), X.size)
    return Y


def fmha(Q, K, V, scale=1.0, causal=False):
    Q, K, V = _f32(Q), _f32(K), _f32(V)
    S, D = Q.shape[-2:]
    bh = Q.size // (S * D)
    O = np.empty(Q.shape, dtype=np.float32)
    lib().kcg_oracle_fmha_f32(_fp(Q), _fp(K), _fp(V), _fp(O), bh, S, D, scale, int(causal))
    return O


def fmha_f64(Q, K, V, scale=1.0, causal=False):
    Q, K, V = _f32(Q), _f32(K), _f32(V)
    S, D = Q.shape[-2:]
    bh = Q.size // (S * D)
    O = np.empty(Q.shape, dtype=np.float64)
    lib().kcg_oracle_fmha_f64(_fp(Q), _fp(K), _fp(V), _dp(O), bh, S, D, scale, int(causal))
    return O


def fmha_rows_f64(Q, K, V, row0, rows, scale=1.0, causal=False):
    """Q, K, V: one [S, D] slab."""
    Q, K, V = _f32(Q), _f32(K), _f32(V)
    S, D = Q.shape
    O = np.empty((rows, D), dtype=np.float64)
    lib().kcg_oracle_fmha_rows_f64(_fp(Q), _fp(K), _fp(V), _dp(O), S, D, row0, rows, scale, int(causal))
    return O


def gather(X, indices, axis=0):
    """out[o.., i.., r..] = X[o.., indices[i..], r..]; a single index (shape (1,)) drops the dimension."""
    X = np.ascontiguousarray(X)
    idx = np.ascontiguousarray(indices, dtype=np.int64)
    axis %= X.ndim
    outer = int(np.prod(X.shape[:axis], dtype=np.int64))
    inner = int(np.prod(X.shape[axis + 1:], dtype=np.int64))
    single = idx.shape == (1,)
    shape = X.shape[:axis] + (() if single else idx.shape) + X.shape[axis + 1:]
    out = np.empty(shape, dtype=X.dtype)
    rc = lib().kcg_oracle_gather(_p(X), idx.ctypes.data_as(C.POINTER(C.c_int64)), _p(out), outer, X.shape[axis], idx.size,
                                 inner * X.itemsize)
    if rc != 0:
        raise IndexError("gather index outside the axis")
    return out


def rel_frobenius(y, ref):
    y = np.asarray(y, dtype=np.float64).ravel()
    ref = np.asarray(ref, dtype=np.float64).ravel()
    den = np.linalg.norm(ref)
    num = np.linalg.norm(y - ref)
    return float(num / den) if den > 0 else float(num)
