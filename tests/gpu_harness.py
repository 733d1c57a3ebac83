"""Helpers for the GPU parity tests: device buffers come from torch (plumbing
only), every compute call goes through the C ABI in include/axhip.h."""
from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from axiom_amd import capi

F32, F16, BF16, U8 = capi.DTYPE_F32, capi.DTYPE_F16, capi.DTYPE_BF16, capi.DTYPE_U8


def to_dev(a: np.ndarray) -> torch.Tensor:
    """numpy (float32 / uint16 bit patterns / uint8) -> device tensor with the same bytes."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    return torch.from_numpy(a).cuda()


def to_host(t: torch.Tensor, like_dtype) -> np.ndarray:
    a = t.cpu().numpy()
    return a.view(np.uint16) if like_dtype == np.uint16 else a


def np_store_dtype(dt):
    return np.float32 if dt == F32 else np.uint8 if dt == U8 else np.uint16


def empty_dev(shape, dt) -> torch.Tensor:
    return torch.empty(shape, dtype=torch.float32 if dt == F32 else torch.uint8 if dt == U8 else torch.int16, device="cuda")


def sync():
    torch.cuda.synchronize()
    capi.check(capi.lib().axhip_stream_sync(None))


def contiguous_strides(H, S, D):
    return (H * S * D, S * D, D)


def sdpa(q, k, v, dt, scale=-1.0, causal=False, mask=None, q_strides=None, k_strides=None, v_strides=None,
         shape=None, poison=True, o_strides=None, out_init=None):
    """q/k/v: numpy storage arrays.  With `shape`=(B,H,Sq,Skv,D) and explicit strides the
    arrays are raw buffers viewed through those strides; otherwise (B,H,S,D) contiguous.
    `out_init` (with `o_strides`): the raw output buffer's initial content; it is returned whole."""
    if shape is None:
        B, H, Sq, D = q.shape
        Skv = k.shape[2]
    else:
        B, H, Sq, Skv, D = shape
    dq, dk, dv = to_dev(q), to_dev(k), to_dev(v)
    if out_init is not None:
        o = to_dev(out_init)
    else:
        o = empty_dev((B, H, Sq, D), dt)
        if poison:
            o.fill_(float("nan") if dt == F32 else 0x7FC1)
    p = capi.SdpaParams()
    p.dtype, p.batch, p.heads, p.seq_q, p.seq_kv, p.head_dim = dt, B, H, Sq, Skv, D
    p.scale, p.is_causal = scale, int(causal)
    p.q_strides[:] = q_strides or contiguous_strides(H, Sq, D)
    p.k_strides[:] = k_strides or contiguous_strides(H, Skv, D)
    p.v_strides[:] = v_strides or contiguous_strides(H, Skv, D)
    p.o_strides[:] = o_strides or contiguous_strides(H, Sq, D)
    dm = None
    if mask is not None:
        mask = np.ascontiguousarray(mask, np.uint8)
        dm = to_dev(mask)
        if mask.ndim == 4:
            mb, mh = mask.shape[:2]
            p.mask_strides[:] = (0 if mb == 1 else mh * Sq * Skv if mh != 1 else Sq * Skv, 0 if mh == 1 else Sq * Skv)
        else:
            p.mask_strides[:] = (0, 0)
    sync()
    capi.check(capi.lib().axhip_sdpa_fwd(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), o.data_ptr(),
                                         dm.data_ptr() if dm is not None else None, C.byref(p), None))
    sync()
    return to_host(o, np_store_dtype(dt)), capi.lib().axhip_sdpa_kernel_name(C.byref(p)).decode()


class Rows:
    """Builder for an AxhipRowsProgram over device copies of numpy arrays."""

    def __init__(self, x: np.ndarray, dt: int, out_dt: int | None = None):
        self.x = np.ascontiguousarray(x)
        self.dt = dt
        self.out_dt = dt if out_dt is None else out_dt
        self.keep = [to_dev(self.x)]
        self.p = capi.RowsProgram()
        self.p.rows = int(np.prod(self.x.shape[:-1], dtype=np.int64))
        self.p.cols = self.x.shape[-1]
        self.p.input = self.keep[0].data_ptr()
        self.p.input_dtype = dt
        self.p.norm_weight = self.p.norm_bias = -1
        self.stage = "pre"

    def _operand(self, arr, dt, kind) -> int:
        t = to_dev(arr)
        self.keep.append(t)
        i = self.p.n_operands
        self.p.operands[i].ptr = t.data_ptr()
        self.p.operands[i].dtype = dt
        self.p.operands[i].kind = capi.BK[kind]
        self.p.n_operands = i + 1
        return i

    def _push(self, op, operand=-1, imm=0.0, imm_kind=0):
        if self.stage == "pre":
            c = self.p.pre[self.p.n_pre]
            self.p.n_pre += 1
        else:
            c = self.p.post[self.p.n_post]
            self.p.n_post += 1
        c.op, c.operand, c.imm, c.imm_kind = capi.OP[op], operand, imm, imm_kind
        return self

    def unary(self, op):
        return self._push(op)

    def binary(self, op, arr, kind="full", dt=None):
        return self._push(op, self._operand(arr, self.dt if dt is None else dt, kind))

    def imm(self, op, value):
        return self._push(op, -1, float(value), capi.BK["imm"])

    def row_op(self, name, eps=1e-5, w=None, b=None, wdt=None):
        self.p.row_op = capi.ROWOP[name]
        self.p.eps = eps
        if w is not None:
            self.p.norm_weight = self._operand(w, self.dt if wdt is None else wdt, "rowvec")
        if b is not None:
            self.p.norm_bias = self._operand(b, self.dt if wdt is None else wdt, "rowvec")
        self.stage = "post"
        return self

    def post(self):
        self.stage = "post"
        return self

    def kernel_name(self):
        return capi.lib().axhip_fused_rows_kernel_name(C.byref(self.p)).decode()

    def run(self, reduce="none"):
        self.p.reduce = capi.RED[reduce]
        shape = self.x.shape[:-1] if reduce != "none" else self.x.shape
        out = empty_dev(shape if len(shape) else (1,), self.out_dt)
        out.fill_(float("nan") if self.out_dt == F32 else 0xCC if self.out_dt == U8 else 0x7FC1)
        self.p.output = out.data_ptr()
        self.p.output_dtype = self.out_dt
        sync()
        capi.check(capi.lib().axhip_fused_rows(C.byref(self.p), None))
        sync()
        return to_host(out, np_store_dtype(self.out_dt)).reshape(shape if len(shape) else (1,))

    def run_full_reduce(self, reduce):
        self.p.reduce = capi.RED[reduce]
        out = empty_dev((1,), self.out_dt)
        self.p.output = out.data_ptr()
        self.p.output_dtype = self.out_dt
        nbytes = capi.lib().axhip_full_reduce_workspace_bytes()
        ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        sync()
        capi.check(capi.lib().axhip_fused_full_reduce(C.byref(self.p), ws.data_ptr(), nbytes, None))
        sync()
        return to_host(out, np_store_dtype(self.out_dt))


def gemm(a, b, dt, trans_a=False, trans_b=False, bias=None, residual=None, epilogue=None, batch=1):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    if a.ndim == 2:
        a, b = a[None], b[None] if b.ndim == 2 else b
    nb = a.shape[0]
    M, K = (a.shape[2], a.shape[1]) if trans_a else a.shape[1:]
    bb = b if b.ndim == 3 else b[None]
    N = bb.shape[1] if trans_b else bb.shape[2]
    da, db = to_dev(a), to_dev(bb)
    c = empty_dev((nb, M, N), dt)
    p = capi.GemmParams()
    p.dtype, p.trans_a, p.trans_b = dt, int(trans_a), int(trans_b)
    p.m, p.n, p.k = M, N, K
    p.lda, p.ldb, p.ldc = a.shape[2], bb.shape[2], N
    p.batch = nb
    p.stride_a = a.shape[1] * a.shape[2]
    p.stride_b = 0 if bb.shape[0] == 1 else bb.shape[1] * bb.shape[2]
    p.stride_c = M * N
    keep = []
    if bias is not None:
        keep.append(to_dev(bias))
        p.bias = keep[-1].data_ptr()
    if residual is not None:
        keep.append(to_dev(residual))
        p.residual = keep[-1].data_ptr()
    p.epilogue_op = capi.OP[epilogue] if epilogue else 0
    sync()
    capi.check(capi.lib().axhip_gemm(da.data_ptr(), db.data_ptr(), c.data_ptr(), C.byref(p), None))
    sync()
    return to_host(c, np_store_dtype(dt))
