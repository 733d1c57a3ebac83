"""ctypes view of the C ABI declared in include/axhip.h.

Loads the in-tree axiom_amd/lib/libaxhip.so.  There is no fallback of any
kind: if the library is missing, or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libaxhip.so"

DTYPE_F32, DTYPE_F16, DTYPE_BF16, DTYPE_U8 = 0, 1, 2, 3

OP = dict(add=1, sub=2, mul=3, div=4, max=5, min=6, rsub=7, rdiv=8,
          relu=16, gelu=17, sqrt=18, exp=19, neg=20, abs=21, sigmoid=22, tanh=23,
          silu=24, log=25, square=26, rsqrt=27, recip=28,
          pow=40, rpow=41, mod=42, rmod=43, atan2=44, ratan2=45, hypot=46, eq=47, ne=48, lt=49, le=50, gt=51, ge=52,
          **{"and": 53, "or": 54, "xor": 55, "not": 77}, leaky_relu=56,
          erf=64, sin=65, cos=66, tan=67, sign=68, floor=69, ceil=70, round=71, trunc=72, cbrt=73,
          isnan=74, isinf=75, isfinite=76)
ROWOP = dict(none=0, softmax=1, logsoftmax=2, layernorm=3, rmsnorm=4)
RED = dict(none=0, sum=1, mean=2, max=3, min=4, prod=5)
BK = dict(full=0, rowvec=1, colvec=2, scalar=3, imm=4)
PAD = dict(constant=0, reflect=1, replicate=2, circular=3)

MAX_CHAIN, MAX_OPERANDS = 16, 8
ERR_INVALID_ARG, ERR_UNSUPPORTED, ERR_NO_DEVICE, ERR_WORKSPACE = -1, -2, -3, -4


class AxhipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"axhip error {code}: {message}")
        self.code = code


class SdpaParams(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32),
        ("batch", C.c_int32), ("heads", C.c_int32), ("seq_q", C.c_int32), ("seq_kv", C.c_int32), ("head_dim", C.c_int32),
        ("scale", C.c_float),
        ("is_causal", C.c_int32),
        ("q_strides", C.c_int64 * 3), ("k_strides", C.c_int64 * 3), ("v_strides", C.c_int64 * 3), ("o_strides", C.c_int64 * 3),
        ("mask_strides", C.c_int64 * 2),
    ]


class Operand(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("dtype", C.c_int32), ("kind", C.c_int32)]


class ChainOp(C.Structure):
    _fields_ = [("op", C.c_int32), ("operand", C.c_int32), ("imm", C.c_float), ("imm_kind", C.c_int32)]


class RowsProgram(C.Structure):
    _fields_ = [
        ("rows", C.c_int64), ("cols", C.c_int64),
        ("input", C.c_void_p), ("input_dtype", C.c_int32), ("n_operands", C.c_int32),
        ("operands", Operand * MAX_OPERANDS),
        ("n_pre", C.c_int32), ("pre", ChainOp * MAX_CHAIN),
        ("row_op", C.c_int32), ("eps", C.c_float), ("norm_weight", C.c_int32), ("norm_bias", C.c_int32),
        ("n_post", C.c_int32), ("post", ChainOp * MAX_CHAIN),
        ("reduce", C.c_int32),
        ("output", C.c_void_p), ("output_dtype", C.c_int32),
    ]


class GemmParams(C.Structure):
    _fields_ = [
        ("dtype", C.c_int32), ("trans_a", C.c_int32), ("trans_b", C.c_int32),
        ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
        ("lda", C.c_int64), ("ldb", C.c_int64), ("ldc", C.c_int64),
        ("batch", C.c_int64), ("stride_a", C.c_int64), ("stride_b", C.c_int64), ("stride_c", C.c_int64),
        ("bias", C.c_void_p), ("residual", C.c_void_p), ("epilogue_op", C.c_int32),
    ]


_lib = None


def lib() -> C.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise FileNotFoundError(
                f"{LIB_PATH} is missing: build it with `python -m axiom_amd.build` (there is no CPU fallback)")
        l = C.CDLL(str(LIB_PATH))
        l.axhip_last_error.restype = C.c_char_p
        l.axhip_version.restype = C.c_char_p
        l.axhip_default_stream.restype = C.c_void_p
        l.axhip_sdpa_kernel_name.restype = C.c_char_p
        l.axhip_sdpa_kernel_name.argtypes = [C.POINTER(SdpaParams)]
        l.axhip_sdpa_last_schedule.restype = C.c_char_p
        l.axhip_fused_rows_kernel_name.restype = C.c_char_p
        l.axhip_fused_rows_kernel_name.argtypes = [C.POINTER(RowsProgram)]
        l.axhip_full_reduce_workspace_bytes.restype = C.c_size_t
        l.axhip_sizeof.restype = C.c_size_t
        l.axhip_sizeof.argtypes = [C.c_int]
        l.axhip_device_count.argtypes = [C.POINTER(C.c_int)]
        l.axhip_init.argtypes = [C.c_int]
        l.axhip_malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        l.axhip_free.argtypes = [C.c_void_p]
        for name in ("axhip_memcpy_h2d_async", "axhip_memcpy_d2h_async", "axhip_memcpy_d2d_async"):
            getattr(l, name).argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        l.axhip_stream_sync.argtypes = [C.c_void_p]
        l.axhip_sdpa_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(SdpaParams), C.c_void_p]
        l.axhip_sdpa_workspace_bytes.restype = C.c_size_t
        l.axhip_sdpa_workspace_bytes.argtypes = [C.POINTER(SdpaParams), C.c_int]
        l.axhip_sdpa_fwd_ws.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(SdpaParams), C.c_void_p, C.c_size_t, C.c_void_p]
        l.axhip_fused_rows.argtypes = [C.POINTER(RowsProgram), C.c_void_p]
        l.axhip_fused_rows_jit_counters.restype = None
        l.axhip_fused_rows_jit_counters.argtypes = [C.POINTER(C.c_int), C.POINTER(C.c_int)]
        l.axhip_fused_rows_prepare.argtypes = [C.POINTER(RowsProgram)]
        l.axhip_fused_full_reduce.argtypes = [C.POINTER(RowsProgram), C.c_void_p, C.c_size_t, C.c_void_p]
        l.axhip_fused_full_reduce_noalloc.argtypes = [C.POINTER(RowsProgram), C.c_void_p]
        l.axhip_full_reduce_noalloc_max_elements.restype = C.c_int64
        l.axhip_strided_copy.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_int32,
                                         C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.c_void_p]
        l.axhip_fill.argtypes = [C.c_void_p, C.c_int32, C.c_double, C.c_int64, C.c_void_p]
        l.axhip_gemm.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(GemmParams), C.c_void_p]
        l.axhip_gemm_workspace_bytes.restype = C.c_size_t
        l.axhip_gemm_workspace_bytes.argtypes = [C.POINTER(GemmParams)]
        l.axhip_gemm_ws.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(GemmParams), C.c_void_p, C.c_size_t, C.c_void_p]
        i64p = C.POINTER(C.c_int64)
        l.axhip_pad.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, i64p, i64p, i64p, i64p, C.c_double, C.c_void_p]
        l.axhip_pad_mode.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, i64p, i64p, i64p, i64p, C.c_int32, C.c_double, C.c_void_p]
        l.axhip_masked_fill.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, i64p, i64p, i64p, C.c_double, C.c_void_p]
        l.axhip_where.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_int32, C.c_int32,
                                  i64p, i64p, i64p, i64p, C.c_void_p]
        l.axhip_argreduce.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]
        l.axhip_reduce_axis.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p]
        l.axhip_argreduce_workspace_bytes.restype = C.c_size_t
        l.axhip_argreduce_workspace_bytes.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64]
        l.axhip_argreduce_ws.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        l.axhip_reduce_axis_workspace_bytes.restype = C.c_size_t
        l.axhip_reduce_axis_workspace_bytes.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64]
        l.axhip_reduce_axis_ws.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_int32, C.c_void_p, C.c_size_t, C.c_void_p]
        l.axhip_softmax_axis.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]
        l.axhip_gather_rows.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p, C.c_int32, C.c_int64, C.c_void_p, C.c_void_p]
        _lib = l
    return _lib


def check(code: int) -> None:
    if code != 0:
        raise AxhipError(code, lib().axhip_last_error().decode(errors="replace"))


def device_count() -> int:
    n = C.c_int(0)
    check(lib().axhip_device_count(C.byref(n)))
    return n.value
