"""ctypes/numpy front end of oracle/libaxiom_oracle.so (see axiom_oracle.h).

TEST INFRASTRUCTURE ONLY.  Used by tests/, the smoke check and the benchmark's
cpu_baseline leg as the checker / reported baseline; never by the shipped
library.  Half-precision arrays travel as numpy uint16 bit patterns.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "libaxiom_oracle.so"
REF_PATH = HERE / "_ref" / "libaxiom_ref.so"

F32, F16, BF16 = 0, 1, 2
OP = dict(add=1, sub=2, mul=3, div=4, max=5, min=6,
          relu=16, gelu=17, sqrt=18, exp=19, neg=20, abs=21, sigmoid=22, tanh=23,
          silu=24, log=25, square=26, rsqrt=27, recip=28,
          pow=40, rpow=41, mod=42, rmod=43, atan2=44, ratan2=45, hypot=46, eq=47, ne=48, lt=49, le=50, gt=51, ge=52,
          **{"and": 53, "or": 54, "xor": 55, "not": 77}, leaky_relu=56,
          erf=64, sin=65, cos=66, tan=67, sign=68, floor=69, ceil=70, round=71, trunc=72, cbrt=73,
          isnan=74, isinf=75, isfinite=76)
RED = dict(sum=1, mean=2, max=3, min=4, prod=5)
BK = dict(full=0, rowvec=1, colvec=2, scalar=3)

_lib = None
_ref = None


def build() -> None:
    """Compile the oracle (and oracle/_ref when the reference tree is present)."""
    subprocess.run(["make", "-C", str(HERE), "all"], check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        l = C.CDLL(str(LIB_PATH))
        l.axo_f32_to_bf16.restype = C.c_uint16
        l.axo_f32_to_bf16.argtypes = [C.c_float]
        l.axo_bf16_to_f32.restype = C.c_float
        l.axo_bf16_to_f32.argtypes = [C.c_uint16]
        l.axo_f32_to_f16.restype = C.c_uint16
        l.axo_f32_to_f16.argtypes = [C.c_float]
        l.axo_f16_to_f32.restype = C.c_float
        l.axo_f16_to_f32.argtypes = [C.c_uint16]
        l.axo_convert.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
        l.axo_pcg64_seed.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        l.axo_pcg64_next.restype = C.c_uint64
        l.axo_pcg64_next.argtypes = [C.c_void_p]
        l.axo_fill_normal.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.c_float]
        l.axo_fill_uniform.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.c_float]
        l.axo_sgemm.argtypes = [C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float, C.c_void_p, C.c_size_t,
                                C.c_void_p, C.c_size_t, C.c_float, C.c_void_p, C.c_size_t]
        l.axo_sdpa.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                               C.c_int, C.c_float, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]
        l.axo_softmax.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int]
        l.axo_unary.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]
        l.axo_where.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        l.axo_binary.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int]
        l.axo_argreduce.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t]
        l.axo_reduce_last.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]
        l.axo_layer_norm.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_float]
        l.axo_rms_norm.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_float]
        l.axo_matmul.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_int]
        l.axo_chain_relu_add_mul_softmax_sum.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t]
        _lib = l
    return _lib


def ref():
    """oracle/_ref (the buildable slice of the reference itself) or None."""
    global _ref
    if _ref is None and REF_PATH.exists():
        r = C.CDLL(str(REF_PATH))
        r.axref_sgemm.argtypes = [C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_size_t, C.c_float, C.c_void_p, C.c_size_t,
                                  C.c_void_p, C.c_size_t, C.c_float, C.c_void_p, C.c_size_t]
        r.axref_blas_name.restype = C.c_char_p
        r.axref_pcg64.argtypes = [C.c_uint64, C.c_uint64, C.c_void_p, C.c_size_t]
        r.axref_pcg64_default.argtypes = [C.c_void_p, C.c_size_t]
        _ref = r
    return _ref


def num_threads() -> int:
    return lib().axo_num_threads()


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _np_dtype(dt):
    return np.float32 if dt == F32 else np.uint16


def to_bits(x: np.ndarray, dt: int) -> np.ndarray:
    """float32 array -> storage array of dtype dt (float32, or uint16 bit patterns)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if dt == F32:
        return x.copy()
    out = np.empty(x.shape, np.uint16)
    lib().axo_convert(F32, _p(x), dt, _p(out), x.size)
    return out


def to_f32(x: np.ndarray, dt: int) -> np.ndarray:
    x = np.ascontiguousarray(x)
    if dt == F32:
        return x.astype(np.float32, copy=True)
    out = np.empty(x.shape, np.float32)
    lib().axo_convert(dt, _p(x), F32, _p(out), x.size)
    return out


class PCG64:
    def __init__(self, seed: int = 42, stream: int = 1):
        self._st = (C.c_uint64 * 2)()
        lib().axo_pcg64_seed(self._st, seed, stream)

    def next(self) -> int:
        return lib().axo_pcg64_next(self._st)

    def normal(self, shape, mean=0.0, std=1.0) -> np.ndarray:
        out = np.empty(shape, np.float32)
        lib().axo_fill_normal(self._st, _p(out), out.size, mean, std)
        return out

    def uniform(self, shape, lo=0.0, hi=1.0) -> np.ndarray:
        out = np.empty(shape, np.float32)
        lib().axo_fill_uniform(self._st, _p(out), out.size, lo, hi)
        return out


def sgemm(A, B, transA=False, transB=False, alpha=1.0, beta=0.0, C0=None):
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B, np.float32)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    out = np.zeros((M, N), np.float32) if C0 is None else np.ascontiguousarray(C0, np.float32).copy()
    lib().axo_sgemm(int(transA), int(transB), M, N, K, alpha, _p(A), A.shape[1], _p(B), B.shape[1], beta, _p(out), N)
    return out


def sdpa(q, k, v, dt=F32, scale=-1.0, causal=False, mask=None, slices=None):
    """q,k,v: storage arrays (B,H,S,D) of dtype dt.  Returns storage array of o."""
    B, H, Sq, D = q.shape
    Skv = k.shape[2]
    o = np.zeros((B, H, Sq, D), _np_dtype(dt))
    mnd, mb, mh = 0, 1, 1
    if mask is not None:
        mask = np.ascontiguousarray(mask, np.uint8)
        mnd = mask.ndim
        if mnd == 4:
            mb, mh = mask.shape[0], mask.shape[1]
    lo, hi = slices if slices else (0, B * H)
    rc = lib().axo_sdpa(dt, _p(q), _p(k), _p(v), _p(o), B, H, Sq, Skv, D, scale, int(causal), _p(mask), mnd, mb, mh, lo, hi)
    assert rc == 0, rc
    return o


def softmax(x, dt=F32, axis=-1, log=False):
    x = np.ascontiguousarray(x)
    ax = axis % x.ndim
    outer = int(np.prod(x.shape[:ax], dtype=np.int64))
    inner = int(np.prod(x.shape[ax + 1:], dtype=np.int64))
    out = np.empty_like(x)
    assert lib().axo_softmax(dt, _p(x), _p(out), outer, x.shape[ax], inner, int(log)) == 0
    return out


def unary(op, x, dt=F32):
    x = np.ascontiguousarray(x)
    out = np.empty_like(x)
    assert lib().axo_unary(OP[op], dt, _p(x), _p(out), x.size) == 0
    return out


def binary(op, a, b, dt=F32, kind="full"):
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    rows = int(np.prod(a.shape[:-1], dtype=np.int64))
    cols = a.shape[-1]
    out = np.empty_like(a)
    assert lib().axo_binary(OP[op], dt, _p(a), _p(b), _p(out), rows, cols, BK[kind]) == 0
    return out


def where(cond, a, b, dt=F32):
    """cond: uint8 / bool array of a's shape."""
    cond = np.ascontiguousarray(cond).astype(np.uint8)
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    out = np.empty_like(a)
    assert lib().axo_where(dt, _p(cond), _p(a), _p(b), _p(out), a.size) == 0
    return out


def reduce_last(red, x, dt=F32):
    x = np.ascontiguousarray(x)
    rows = int(np.prod(x.shape[:-1], dtype=np.int64))
    out = np.empty(x.shape[:-1], x.dtype)
    assert lib().axo_reduce_last(RED[red], dt, _p(x), _p(out), rows, x.shape[-1]) == 0
    return out


def argreduce(x, axis=-1, want_min=False, dt=F32):
    """argmax / argmin along one axis (int64 indices, first occurrence wins)."""
    x = np.ascontiguousarray(x)
    axis %= x.ndim
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    out = np.empty(x.shape[:axis] + x.shape[axis + 1:], np.int64)
    assert lib().axo_argreduce(int(want_min), dt, _p(x), _p(out), outer, x.shape[axis], inner) == 0
    return out


def layer_norm(x, w=None, b=None, dt=F32, eps=1e-5):
    x = np.ascontiguousarray(x)
    rows = int(np.prod(x.shape[:-1], dtype=np.int64))
    out = np.empty(x.shape, np.float32)
    assert lib().axo_layer_norm(dt, _p(x), _p(w), _p(b), _p(out), rows, x.shape[-1], eps) == 0
    return out


def rms_norm(x, w=None, dt=F32, eps=1e-5):
    x = np.ascontiguousarray(x)
    rows = int(np.prod(x.shape[:-1], dtype=np.int64))
    out = np.empty(x.shape, np.float32)
    assert lib().axo_rms_norm(dt, _p(x), _p(w), _p(out), rows, x.shape[-1], eps) == 0
    return out


def matmul(A, B, dt=F32, transA=False, transB=False):
    A = np.ascontiguousarray(A)
    B = np.ascontiguousarray(B)
    M, K = (A.shape[1], A.shape[0]) if transA else A.shape
    N = B.shape[0] if transB else B.shape[1]
    out = np.empty((M, N), A.dtype)
    assert lib().axo_matmul(dt, _p(A), _p(B), _p(out), M, N, K, int(transA), int(transB)) == 0
    return out


def chain_relu_add_mul_softmax_sum(a, b, want_softmax=False):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    rows, cols = a.shape
    out = np.empty(rows, np.float32)
    sm = np.empty((rows, cols), np.float32) if want_softmax else None
    assert lib().axo_chain_relu_add_mul_softmax_sum(_p(a), _p(b), _p(out), _p(sm), rows, cols) == 0
    return (out, sm) if want_softmax else out
