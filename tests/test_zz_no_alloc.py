"""axhip_fused_full_reduce_noalloc (partials in the library's own device array, no allocation) against
axhip_fused_full_reduce (caller's workspace): same kernels, so the results must agree bit for bit.  Two calls in a
row, the second on a smaller input, so that stale partials of the first would show."""
import ctypes as C

import numpy as np
import pytest
import torch

from axiom_amd import capi
from oracle import axo
from tests import gpu_harness as gh

pytestmark = pytest.mark.gpu

F32, BF16 = gh.F32, gh.BF16


def both_ways(rows: gh.Rows, reduce: str):
    """(workspace entry point, no-allocation entry point) results of the same program, as raw storage."""
    want = rows.run_full_reduce(reduce)
    out = gh.empty_dev((1,), rows.out_dt)
    out.fill_(float("nan") if rows.out_dt == F32 else 0x7FC1)
    rows.p.output = out.data_ptr()
    gh.sync()
    capi.check(capi.lib().axhip_fused_full_reduce_noalloc(C.byref(rows.p), None))
    gh.sync()
    return want, gh.to_host(out, gh.np_store_dtype(rows.out_dt))


def test_noalloc_full_reduce_matches_workspace_entry_point_on_two_calls_in_a_row():
    g = axo.PCG64(20240607)
    big = g.normal((4096, 1024))     # 16 MiB: 512 rows of 2048 chunks on the row-reduction kernel, a partial each
    small = g.normal((3, 40))        # one block of the generic kernel: the other slots keep the first call's partials
    for x, reduce in ((big, "sum"), (small, "sum"), (big, "max"), (small, "min"), (small, "mean")):
        want, got = both_ways(gh.Rows(x, F32).unary("square") if reduce in ("sum", "mean") else gh.Rows(x, F32), reduce)
        assert got.view(np.uint32)[0] == want.view(np.uint32)[0], (x.shape, reduce, got, want)
    # and against the CPU oracle's double-precision sum (the bar of the workspace entry point's own test)
    _, got = both_ways(gh.Rows(small, F32).unary("square"), "sum")
    assert np.isclose(got[0], np.sum(small.astype(np.float64) ** 2), rtol=1e-4, atol=1e-4)
    # 16-bit input with a binary operand
    xb, yb = (axo.to_bits(g.normal((257, 64)), axo.BF16) for _ in range(2))
    want, got = both_ways(gh.Rows(xb, BF16, F32).binary("mul", yb), "sum")
    assert got.view(np.uint32)[0] == want.view(np.uint32)[0]


def test_noalloc_full_reduce_rejects_oversized_and_malformed_programs():
    lib = capi.lib()
    limit = lib.axhip_full_reduce_noalloc_max_elements()
    assert limit == 1 << 40
    x = torch.zeros(16, dtype=torch.float32, device="cuda")
    p = capi.RowsProgram()
    p.rows, p.cols = (1 << 20) + 1, 1 << 20   # one row beyond the limit; rejected before any launch
    p.input = p.output = x.data_ptr()
    p.reduce = capi.RED["sum"]
    p.norm_weight = p.norm_bias = -1
    with pytest.raises(capi.AxhipError) as e:
        capi.check(lib.axhip_fused_full_reduce_noalloc(C.byref(p), None))
    assert e.value.code == capi.ERR_UNSUPPORTED and "exceed the maximum" in str(e.value)
    p.rows, p.cols, p.reduce = 4, 4, capi.RED["none"]
    with pytest.raises(capi.AxhipError):
        capi.check(lib.axhip_fused_full_reduce_noalloc(C.byref(p), None))
