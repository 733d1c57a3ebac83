"""The *_ws entry points: the four calls that need temporary device memory take it from a caller's workspace and
allocate nothing.  Each is compared bit for bit with its allocating form on the same inputs, is refused with
AXHIP_ERR_WORKSPACE when the workspace is too small, and asks for no memory where the plain call takes none."""
import ctypes as C

import numpy as np
import pytest
import torch

from axiom_amd import capi
from oracle import axo
from tests import gpu_harness as gh

pytestmark = pytest.mark.gpu
F32, F16, BF16 = axo.F32, axo.F16, axo.BF16


def workspace(nbytes, fill=0x5A):
    """A 256-byte aligned device buffer of nbytes plus a guard behind it that the call must leave alone."""
    t = torch.full((nbytes + 512,), fill, dtype=torch.uint8, device="cuda")
    gh.sync()  # (torch fills on its own stream, the library works on another: the fill has to be over first)
    off = (-t.data_ptr()) % 256
    return t, t.data_ptr() + off, off


def guard_intact(t, off, nbytes, fill=0x5A):
    return bool((t[off + nbytes:] == fill).all().item())


def test_decoding_attention_with_a_caller_workspace():
    lib = capi.lib()
    B, H, Sq, Skv, D = 1, 32, 1, 4096, 128
    g = axo.PCG64(3)
    q, k, v = (gh.to_dev(axo.to_bits(g.normal(s), BF16)) for s in ((B, H, Sq, D), (B, H, Skv, D), (B, H, Skv, D)))
    p = capi.SdpaParams()
    p.dtype, p.batch, p.heads, p.seq_q, p.seq_kv, p.head_dim, p.scale, p.is_causal = BF16, B, H, Sq, Skv, D, -1.0, 0
    p.q_strides[:] = gh.contiguous_strides(H, Sq, D)
    p.o_strides[:] = gh.contiguous_strides(H, Sq, D)
    p.k_strides[:] = gh.contiguous_strides(H, Skv, D)
    p.v_strides[:] = gh.contiguous_strides(H, Skv, D)
    need = lib.axhip_sdpa_workspace_bytes(C.byref(p), 0)
    assert need > 0 and need % 256 == 0
    assert lib.axhip_sdpa_workspace_bytes(C.byref(p), 1) == 0  # with a mask the keys are not split
    o1, o2 = gh.empty_dev((B, H, Sq, D), BF16), gh.empty_dev((B, H, Sq, D), BF16)
    capi.check(lib.axhip_sdpa_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o1.data_ptr(), None, C.byref(p), None))
    assert lib.axhip_sdpa_last_schedule() == b"decode_split"
    t, ws, off = workspace(need)
    capi.check(lib.axhip_sdpa_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), o2.data_ptr(), None, C.byref(p), ws, need, None))
    gh.sync()
    assert torch.equal(o1, o2)
    assert guard_intact(t, off, need)
    assert lib.axhip_sdpa_fwd_ws(q.data_ptr(), k.data_ptr(), v.data_ptr(), o2.data_ptr(), None, C.byref(p), ws, need - 256, None) == capi.ERR_WORKSPACE
    assert b"workspace" in lib.axhip_last_error()
    # a problem that takes no temporary memory asks for none, and runs with a NULL workspace
    p.seq_q = 512
    p.q_strides[:] = gh.contiguous_strides(H, 512, D)
    assert lib.axhip_sdpa_workspace_bytes(C.byref(p), 0) == 0


@pytest.mark.parametrize("dt,k", [(BF16, 1024), (BF16, 1001), (F32, 1001)], ids=["bf16-transposed-b", "bf16-k1001", "f32-k1001"])
def test_repacked_products_with_a_caller_workspace(dt, k):
    lib = capi.lib()
    M, N = 1024, 1024
    g = axo.PCG64(4)
    a = g.normal((M, k)).astype(np.float32)
    b = (g.normal((k, N)) * 0.05).astype(np.float32)  # stored [K, N]: trans_b = 0
    da, db = (gh.to_dev(t if dt == F32 else axo.to_bits(t, dt)) for t in (a, b))
    p = capi.GemmParams()
    p.dtype, p.trans_a, p.trans_b, p.m, p.n, p.k = dt, 0, 0, M, N, k
    p.lda, p.ldb, p.ldc, p.batch = k, N, N, 1
    need = lib.axhip_gemm_workspace_bytes(C.byref(p))
    assert need > 0
    c1, c2 = gh.empty_dev((M, N), dt), gh.empty_dev((M, N), dt)
    capi.check(lib.axhip_gemm(da.data_ptr(), db.data_ptr(), c1.data_ptr(), C.byref(p), None))
    t, ws, off = workspace(need)
    capi.check(lib.axhip_gemm_ws(da.data_ptr(), db.data_ptr(), c2.data_ptr(), C.byref(p), ws, need, None))
    gh.sync()
    assert torch.equal(c1, c2)
    assert guard_intact(t, off, need)
    assert lib.axhip_gemm_ws(da.data_ptr(), db.data_ptr(), c2.data_ptr(), C.byref(p), ws, need // 2, None) == capi.ERR_WORKSPACE
    # x W^T with an aligned k is not repacked
    p.trans_b, p.k, p.ldb = 1, 1024, 1024
    assert lib.axhip_gemm_workspace_bytes(C.byref(p)) == 0


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
def test_long_axis_reductions_with_a_caller_workspace(dt):
    """Few results over a long axis: argmax / sum over axis 0 of a tall matrix cut the axis into segments."""
    lib = capi.lib()
    outer, axis, inner = 1, 8192, 2048
    g = axo.PCG64(6)
    x = g.normal((outer, axis, inner)).astype(np.float32)
    dx = gh.to_dev(x if dt == F32 else axo.to_bits(x, dt))
    # argmax
    need = lib.axhip_argreduce_workspace_bytes(dx.data_ptr(), dt, outer, axis, inner)
    assert need > 0
    i1 = torch.empty((outer * inner,), dtype=torch.int64, device="cuda")
    i2 = torch.empty_like(i1)
    capi.check(lib.axhip_argreduce(dx.data_ptr(), dt, outer, axis, inner, 0, i1.data_ptr(), None))
    t, ws, off = workspace(need)
    capi.check(lib.axhip_argreduce_ws(dx.data_ptr(), dt, outer, axis, inner, 0, i2.data_ptr(), ws, need, None))
    gh.sync()
    assert torch.equal(i1, i2) and guard_intact(t, off, need)
    xf = x if dt == F32 else axo.to_f32(axo.to_bits(x, dt), dt)
    assert np.array_equal(i2.cpu().numpy().reshape(outer, inner), xf.argmax(1))
    assert lib.axhip_argreduce_ws(dx.data_ptr(), dt, outer, axis, inner, 0, i2.data_ptr(), ws, 256, None) == capi.ERR_WORKSPACE
    # sum
    need = lib.axhip_reduce_axis_workspace_bytes(dx.data_ptr(), dt, outer, axis, inner)
    assert need > 0
    s1, s2 = gh.empty_dev((outer, inner), F32), gh.empty_dev((outer, inner), F32)
    capi.check(lib.axhip_reduce_axis(dx.data_ptr(), dt, outer, axis, inner, capi.RED["sum"], s1.data_ptr(), F32, None))
    t, ws, off = workspace(need)
    capi.check(lib.axhip_reduce_axis_ws(dx.data_ptr(), dt, outer, axis, inner, capi.RED["sum"], s2.data_ptr(), F32, ws, need, None))
    gh.sync()
    assert torch.equal(s1, s2) and guard_intact(t, off, need)
    assert np.allclose(s2.cpu().numpy(), xf.astype(np.float64).sum(1), rtol=1e-4, atol=1e-2)
    assert lib.axhip_reduce_axis_ws(dx.data_ptr(), dt, outer, axis, inner, capi.RED["sum"], s2.data_ptr(), F32, ws, 256, None) == capi.ERR_WORKSPACE
    # many results over a short axis: one pass, no temporary memory
    assert lib.axhip_reduce_axis_workspace_bytes(dx.data_ptr(), dt, 4096, 4, 1024) == 0
    assert lib.axhip_argreduce_workspace_bytes(dx.data_ptr(), dt, 4096, 4, 1024) == 0
