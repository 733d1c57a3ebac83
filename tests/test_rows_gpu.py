"""GPU parity of axhip_fused_rows / axhip_fused_full_reduce against the CPU
oracle (Axiom's op-by-op CPU path restated) and float64 closed forms.

Tolerances: fp32 1e-4 abs + 1e-4 rel (relu/add/mul chains bit-exact); bf16 / f16
2e-2 abs against an fp32-or-better evaluation of the same half inputs."""
import math

import numpy as np
import pytest

from oracle import axo
from tests import gpu_harness as gh

pytestmark = pytest.mark.gpu
F32, F16, BF16 = axo.F32, axo.F16, axo.BF16
ONE = np.array([1.0], np.float32)


def close32(a, b):
    return np.allclose(a, b, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("shape", [(4, 5), (1, 1), (3, 37), (64, 256), (7, 1000), (33, 4096), (5, 8200), (2, 70000), (1024, 64)])
def test_relu_add_mul_chain_is_bit_exact(shape):
    g = axo.PCG64(1)
    a, b = g.normal(shape), g.normal(shape)
    prog = gh.Rows(a, F32).unary("relu").binary("add", ONE, "scalar").binary("mul", b)
    got = prog.run()
    want = axo.binary("mul", axo.binary("add", axo.unary("relu", a), ONE, kind="scalar"), b)
    assert np.array_equal(got, want), prog.kernel_name()


def test_fused_pattern_known_answers_on_gpu():
    # tests/test_fusion_extended.cpp:114-220
    a, b, c = (np.full((4, 4), x, np.float32) for x in (3.0, 2.0, 4.0))
    assert np.all(gh.Rows(a, F32).binary("add", b).unary("relu").run() == 5.0)
    assert np.all(gh.Rows(b, F32).binary("sub", a).unary("relu").run() == 0.0)
    assert np.all(gh.Rows(a, F32).binary("add", b).unary("square").run() == 25.0)
    assert np.all(gh.Rows(b, F32).binary("sub", a).unary("abs").run() == 1.0)
    assert np.all(gh.Rows(a, F32).binary("mul", b).binary("add", c).run() == 10.0)
    assert np.all(gh.Rows(a, F32).binary("add", b).binary("mul", c).run() == 20.0)
    assert np.all(gh.Rows(a, F32).binary("rsub", b).run() == -1.0)  # b - a
    assert np.allclose(gh.Rows(a, F32).binary("add", b).unary("sigmoid").run(), 1 / (1 + math.exp(-5)), atol=1e-6)
    x = np.ones((8,), np.float32)
    p = gh.Rows(x.reshape(1, 8), F32)
    for _ in range(10):
        p.imm("add", 1.0)
    assert np.all(p.run() == 11.0)  # long chain, tests/test_fusion_extended.cpp:561-572


@pytest.mark.parametrize("op", ["relu", "gelu", "sqrt", "exp", "neg", "abs", "sigmoid", "tanh", "silu", "log", "square", "rsqrt", "recip"])
def test_unary_ops_match_oracle(op):
    x = axo.PCG64(2).normal((17, 96))
    if op in ("sqrt", "log", "rsqrt"):
        x = np.abs(x) + 0.1
    got = gh.Rows(x, F32).unary(op).run()
    assert close32(got, axo.unary(op, x)), op


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "max", "min"])
@pytest.mark.parametrize("kind", ["full", "rowvec", "colvec", "scalar"])
def test_binary_ops_and_broadcast_kinds(op, kind):
    g = axo.PCG64(3)
    a = g.normal((9, 40))
    b = {"full": g.normal((9, 40)), "rowvec": g.normal((40,)), "colvec": g.normal((9,)), "scalar": g.normal((1,))}[kind] + 3.0
    got = gh.Rows(a, F32).binary(op, b, kind).run()
    assert np.array_equal(got, axo.binary(op, a, b, kind=kind))


@pytest.mark.parametrize("shape", [(4, 5), (2, 3, 33), (16, 256), (8, 1024), (3, 8192), (2, 20000), (1, 70001)])
@pytest.mark.parametrize("log", [False, True])
def test_softmax_matches_oracle(shape, log):
    x = axo.PCG64(4).normal(shape) * 3
    p = gh.Rows(x, F32).row_op("logsoftmax" if log else "softmax")
    got = p.run()
    want = axo.softmax(x, log=log)
    assert close32(got, want), p.kernel_name()
    if not log:
        assert np.allclose(got.sum(-1), 1.0, atol=1e-4)


@pytest.mark.parametrize("dt,tol", [(BF16, 4e-3), (F16, 5e-4)])
def test_softmax_half(dt, tol):
    x = axo.to_bits(axo.PCG64(5).normal((33, 1000)) * 2, dt)
    got = axo.to_f32(gh.Rows(x, dt).row_op("softmax").run(), dt)
    assert np.max(np.abs(got - axo.to_f32(axo.softmax(x, dt), dt))) <= tol


@pytest.mark.parametrize("red", ["sum", "mean", "max", "min"])
@pytest.mark.parametrize("shape", [(4, 5), (64, 64), (5, 4096), (3, 50000)])
def test_row_reductions(red, shape):
    x = axo.PCG64(6).normal(shape)
    got = gh.Rows(x, F32).run(reduce=red)
    want = axo.reduce_last(red, x)
    assert close32(got, want)
    if red in ("max", "min"):
        assert np.array_equal(got, want)


def test_reduce_known_answers_on_gpu():
    a, b = np.full((1, 16), 3.0, np.float32), np.full((1, 16), 2.0, np.float32)
    assert gh.Rows(a, F32).binary("add", b).run(reduce="sum")[0] == 80.0  # tests/test_fusion_extended.cpp:346-352
    big = np.ones((1, 1 << 20), np.float32)
    assert gh.Rows(big, F32).imm("mul", 2.0).run(reduce="sum")[0] == 2097152.0  # :436-443
    assert gh.Rows(big.reshape(1024, 1024), F32).imm("mul", 2.0).run_full_reduce("sum")[0] == 2097152.0
    x = axo.PCG64(8).normal((300, 777))
    got = gh.Rows(x, F32).unary("square").run_full_reduce("mean")[0]
    assert abs(got - float((x.astype(np.float64) ** 2).mean())) < 1e-4
    assert gh.Rows(x, F32).run_full_reduce("max")[0] == x.max()
    assert gh.Rows(x, F32).run_full_reduce("min")[0] == x.min()


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_short_rows_that_share_a_wavefront(dt):
    """Aligned rows of up to 32 chunks run 4, 8, 16 or 32 lanes per row, several rows to a wavefront: every group size,
    rows that fill their group and rows that leave lanes idle, row counts that leave a wavefront's (and a block's)
    last set of rows partial, per-row and per-column operands, a reduction; guard words behind the output."""
    g = axo.PCG64(900 + dt)
    e = 4 if dt == F32 else 8
    tag = {F32: "f32", BF16: "bf16", F16: "f16"}[dt]
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    tol = 1e-5 if dt == F32 else (2.0 ** -8 if dt == BF16 else 2.0 ** -10)
    sentinel = np.float32(-77.0) if dt == F32 else np.uint16(0x7FC1)
    for chunks, group in ((1, 4), (3, 4), (4, 4), (5, 8), (8, 8), (11, 16), (16, 16), (25, 32), (32, 32)):
        cols = chunks * e
        for rows in (1, 5, 64 // group * 4 + 1, 1000):
            x = store(g.normal((rows, cols)) * 2)
            xf = wide(x)
            cv, rv = store(g.uniform((rows,), 0.5, 1.5)), store(g.uniform((cols,), 0.5, 1.5))
            dst = gh.to_dev(np.full(rows * cols + 64, sentinel, x.dtype))
            p = gh.Rows(x, dt).row_op("softmax")
            p.keep.append(dst)
            p.p.output, p.p.output_dtype = dst.data_ptr(), dt
            assert p.kernel_name() == f"rows_{'jit' if dt == F16 else 'static'}_softmax_{tag}_g{group}_it1", (cols, p.kernel_name())
            gh.sync()
            gh.capi.check(gh.capi.lib().axhip_fused_rows(gh.C.byref(p.p), None))
            gh.sync()
            out = gh.to_host(dst, x.dtype)
            assert np.all(out[rows * cols:] == sentinel), (rows, cols)
            got = wide(out[:rows * cols].reshape(rows, cols))
            ex = np.exp(xf - xf.max(-1, keepdims=True))
            want = ex / ex.sum(-1, keepdims=True)
            assert np.all(np.abs(got - want) <= tol * want + (2.0 ** -24 if dt == F16 else 1e-9)), (rows, cols)
            # a per-row scale, a per-column weight, layer norm, then the row maximum
            w, b = store(g.uniform((cols,), 0.5, 1.5)), store(g.uniform((cols,), -0.5, 0.5))
            p = gh.Rows(x, dt, F32).binary("mul", cv, "colvec").binary("add", rv, "rowvec").row_op("layernorm", 1e-5, w=w, b=b)
            got = p.run(reduce="max").astype(np.float64).reshape(-1)
            assert p.kernel_name().endswith(f"_g{group}_it1"), p.kernel_name()
            t = xf * wide(cv)[:, None] + wide(rv)
            n = (t - t.mean(-1, keepdims=True)) / np.sqrt(t.var(-1, keepdims=True) + 1e-5) * wide(w) + wide(b)
            assert np.max(np.abs(got - n.max(-1))) < (1e-4 if dt == F32 else 1e-3), (rows, cols)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_short_rows_of_odd_length_share_a_wavefront_on_the_16_byte_grid(dt):
    """Short rows whose length no vector divides (10 class logits, 77 or 197 tokens): the rows of a wavefront are
    consecutive in memory, each on the 16-byte grid with a shift of its own, a masked partial chunk at either end
    (two rows may share a 16-byte word: each stores its own elements only).  Lengths from one element to 32 grid
    chunks, row counts that leave the last wavefront partial, from a base 3 elements past a boundary, with guard words
    on both sides of the output; softmax against float64, a norm with weight, bias and per-row operand, a reduction."""
    g = axo.PCG64(1300 + dt)
    e, es = (4, 4) if dt == F32 else (8, 2)
    tag = {F32: "f32", BF16: "bf16", F16: "f16"}[dt]
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    tol = 1e-5 if dt == F32 else (2.0 ** -8 if dt == BF16 else 2.0 ** -10)
    sentinel = np.float32(-77.0) if dt == F32 else np.uint16(0x7FC1)
    off, pad = 3, 64
    for cols in (1, 3, e - 1, e + 1, 10, 3 * e + 1, 77, 15 * e - 1, 197 if dt != F32 else 101, 31 * e - 6):
        chunks = (cols + 2 * e - 2) // e
        group = 4 if chunks <= 4 else 8 if chunks <= 8 else 16 if chunks <= 16 else 32
        for rows in (1, 7, 64 // group * 4 + 3, 501):
            x = store(g.normal((rows, cols)) * 2)
            xf = wide(x)
            src = gh.to_dev(np.concatenate([np.full(off, sentinel, x.dtype), x.ravel()]))
            dst = gh.to_dev(np.full(pad + off + rows * cols + pad, sentinel, x.dtype))
            p = gh.Rows(x[:1], dt).row_op("softmax")
            p.keep += [src, dst]
            p.p.rows, p.p.input = rows, src.data_ptr() + off * es
            p.p.output, p.p.output_dtype = dst.data_ptr() + (pad + off) * es, dt
            assert p.kernel_name() == f"rows_{'jit' if dt == F16 else 'static'}_softmax_{tag}_g{group}_it1_grid", (cols, p.kernel_name())
            gh.sync()
            gh.capi.check(gh.capi.lib().axhip_fused_rows(gh.C.byref(p.p), None))
            gh.sync()
            out = gh.to_host(dst, x.dtype)
            assert np.all(out[:pad + off] == sentinel) and np.all(out[pad + off + rows * cols:] == sentinel), (rows, cols)
            got = wide(out[pad + off:pad + off + rows * cols].reshape(rows, cols))
            ex = np.exp(xf - xf.max(-1, keepdims=True))
            want = ex / ex.sum(-1, keepdims=True)
            assert np.all(np.abs(got - want) <= tol * want + (2.0 ** -24 if dt == F16 else 1e-9)), (rows, cols)
            if cols < 2:
                continue
            w, b, cv = store(g.uniform((cols,), 0.5, 1.5)), store(g.uniform((cols,), -0.5, 0.5)), store(g.uniform((rows,), 0.5, 1.5))
            p = gh.Rows(x, dt).binary("mul", cv, "colvec").row_op("layernorm", 1e-5, w=w, b=b)
            got = wide(p.run())
            assert p.kernel_name().endswith(f"_g{group}_it1_grid"), p.kernel_name()
            t = xf * wide(cv)[:, None]
            n = (t - t.mean(-1, keepdims=True)) / np.sqrt(t.var(-1, keepdims=True) + 1e-5) * wide(w) + wide(b)
            assert np.max(np.abs(got - n)) < (2e-4 if dt == F32 else 4e-2), (rows, cols, np.max(np.abs(got - n)))
            p = gh.Rows(x, dt, F32).unary("abs")
            got = p.run(reduce="max").astype(np.float64).reshape(-1)
            assert np.array_equal(got, np.abs(xf).max(-1)), (rows, cols)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_many_short_rows_of_odd_length_are_staged_in_lds_a_row_per_lane(dt):
    """From 32768 rows on, rows whose length no vector divides go through LDS: a wavefront copies the contiguous span of
    its 64 / L rows with whole 16-byte accesses, L = 1, 2, 4 or 8 lanes walk each row there, and the results leave the
    same way (the last bytes of the array, where they do not fill a vector, element by element).  Lengths from one
    element to more than 64 chunks, row counts that leave the last wavefront partial and the array's end inside a
    vector, guard words on both sides of the output; softmax and log-softmax against float64, a norm with weight, bias
    and per-row operand, a norm behind a two-operand pre chain with a post chain, a row reduction."""
    g = axo.PCG64(4300 + dt)
    e, es = (4, 4) if dt == F32 else (8, 2)
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    step = 1e-5 if dt == F32 else (2.0 ** -8 if dt == BF16 else 2.0 ** -10)
    sentinel = np.float32(-77.0) if dt == F32 else np.uint16(0x7FC1)
    pad = 64
    for cols, rows in ((1, 32768 + 37), (3, 33023), (e + 1, 32768), (10, 32805), (77, 32768 + 37), (101, 33023), (197 if dt != F32 else 125, 32805),
                       (513 if dt != F32 else 259, 32768 + 5)):
        x = store(g.normal((rows, cols)) * 2)
        xf = wide(x)
        dst = gh.to_dev(np.full(pad + rows * cols + pad, sentinel, x.dtype))
        p = gh.Rows(x, dt).row_op("softmax")
        p.keep += [dst]
        p.p.output, p.p.output_dtype = dst.data_ptr() + pad * es, dt
        assert "_lane" in p.kernel_name(), (cols, p.kernel_name())
        gh.sync()
        gh.capi.check(gh.capi.lib().axhip_fused_rows(gh.C.byref(p.p), None))
        gh.sync()
        out = gh.to_host(dst, x.dtype)
        assert np.all(out[:pad] == sentinel) and np.all(out[pad + rows * cols:] == sentinel), (rows, cols)
        got = wide(out[pad:pad + rows * cols].reshape(rows, cols))
        ex = np.exp(xf - xf.max(-1, keepdims=True))
        want = ex / ex.sum(-1, keepdims=True)
        assert np.all(np.abs(got - want) <= step * want + (2.0 ** -24 if dt == F16 else 1e-9)), (rows, cols)
        got = wide(gh.Rows(x, dt).row_op("logsoftmax").run())
        want = (xf - xf.max(-1, keepdims=True)) - np.log(ex.sum(-1, keepdims=True))
        assert np.all(np.abs(got - want) <= step * np.abs(want) + 1e-4), (rows, cols)
        if cols < 2:
            continue
        w, b, cv = store(g.uniform((cols,), 0.5, 1.5)), store(g.uniform((cols,), -0.5, 0.5)), store(g.uniform((rows,), 0.5, 1.5))
        p = gh.Rows(x, dt).binary("mul", cv, "colvec").row_op("layernorm", 1e-5, w=w, b=b)
        got = wide(p.run())
        assert "_lane" in p.kernel_name(), p.kernel_name()
        t = xf * wide(cv)[:, None]
        n = (t - t.mean(-1, keepdims=True)) / np.sqrt(t.var(-1, keepdims=True) + 1e-5) * wide(w) + wide(b)
        assert np.max(np.abs(got - n)) < (2e-4 if dt == F32 else 4e-2), (rows, cols, np.max(np.abs(got - n)))
        y = store(g.normal((rows, cols)))
        p = gh.Rows(x, dt).binary("add", y).binary("mul", w, "rowvec").row_op("rmsnorm", 1e-5, w=b).post().unary("relu")
        got = wide(p.run())
        assert "_lane" in p.kernel_name(), p.kernel_name()
        t = (xf + wide(y)) * wide(w)
        n = np.maximum(t / np.sqrt((t * t).mean(-1, keepdims=True) + 1e-5) * wide(b), 0)
        assert np.max(np.abs(got - n)) < (2e-4 if dt == F32 else 4e-2), (rows, cols, np.max(np.abs(got - n)))
        p = gh.Rows(x, dt, F32).unary("abs")
        got = p.run(reduce="max").astype(np.float64).reshape(-1)
        assert "_lane" in p.kernel_name(), p.kernel_name()
        assert np.array_equal(got, np.abs(xf).max(-1)), (rows, cols)


def test_short_odd_rows_in_lds_take_streams_of_different_element_sizes():
    """The row-per-lane plan gives every stream its own geometry in LDS: a 16-bit input with an fp32 full-size operand
    and an fp32 result (three spans of two sizes), and an fp32 input with a 16-bit result."""
    g = axo.PCG64(4400)
    rows, cols = 32768 + 21, 45
    x = axo.to_bits(g.normal((rows, cols)), BF16)
    y = g.normal((rows, cols)).astype(np.float32)
    w = g.uniform((cols,), 0.5, 1.5).astype(np.float32)
    p = gh.Rows(x, BF16, F32).binary("add", y, dt=F32).row_op("rmsnorm", 1e-5, w=w, wdt=F32)
    got = p.run().astype(np.float64)
    assert "_to_f32_lane" in p.kernel_name(), p.kernel_name()
    t = axo.to_f32(x, BF16).astype(np.float64) + y
    want = t / np.sqrt((t * t).mean(-1, keepdims=True) + 1e-5) * w
    assert np.max(np.abs(got - want)) < 2e-4, np.max(np.abs(got - want))
    xf = g.normal((rows, cols)).astype(np.float32) * 2
    p = gh.Rows(xf, F32, F16).row_op("softmax")
    got = axo.to_f32(p.run(), F16).astype(np.float64)
    assert "_to_f16_lane" in p.kernel_name(), p.kernel_name()
    ex = np.exp(xf.astype(np.float64) - xf.max(-1, keepdims=True))
    want = ex / ex.sum(-1, keepdims=True)
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * want + 2.0 ** -24)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_large_elementwise_chains_take_compiled_row_kernels(dt):
    """From 8 MiB on an elementwise chain runs as a compiled row program without a row operation: an array whose
    operands are full-size, one-element or immediate is seen as rows of 512 chunks whatever its shape (a vector, short
    rows, a shape that is no multiple of 4096 columns), one with a per-column or per-row operand keeps its rows.
    relu / add / mul chains are exact against the oracle's fp32 evaluation of the same inputs; activations to a
    16-bit step; an fp32 result from 16-bit inputs; comparisons that leave one-byte truth values; guard words around
    the output."""
    g = axo.PCG64(5100 + dt)
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_f32(t, dt))
    es = 4 if dt == F32 else 2
    sentinel = np.float32(-77.0) if dt == F32 else np.uint16(0x7FC1)
    for shape in ((1, 1 << 22), (3 << 16, 24), (2048, 2304)):
        rows, cols = shape
        a, b = store(g.normal(shape)), store(g.normal(shape))
        one = store(np.array([1.25]))
        pad = 64
        dst = gh.to_dev(np.full(pad + rows * cols + pad, sentinel, a.dtype))
        p = gh.Rows(a, dt).unary("relu").binary("add", one, "scalar").binary("mul", b).imm("mul", 0.5)
        p.keep.append(dst)
        p.p.output, p.p.output_dtype = dst.data_ptr() + pad * es, dt
        assert "_map_" in p.kernel_name() and "_g64_it8" in p.kernel_name(), p.kernel_name()
        gh.sync()
        gh.capi.check(gh.capi.lib().axhip_fused_rows(gh.C.byref(p.p), None))
        gh.sync()
        out = gh.to_host(dst, a.dtype)
        assert np.all(out[:pad] == sentinel) and np.all(out[pad + rows * cols:] == sentinel), shape
        want = store((np.maximum(wide(a), 0) + wide(one)) * wide(b) * np.float32(0.5))
        assert np.array_equal(out[pad:pad + rows * cols].reshape(shape), want), shape
    # per-column and per-row operands: the array keeps its rows
    rows, cols = 8192, 1024
    a = store(g.normal((rows, cols)))
    bias, gate = store(g.normal((cols,))), store(g.uniform((rows,), 0.5, 1.5))
    p = gh.Rows(a, dt).binary("add", bias, "rowvec").binary("mul", gate, "colvec").unary("relu")
    got = p.run()
    assert "_map_" in p.kernel_name(), p.kernel_name()
    assert np.array_equal(got, store(np.maximum((wide(a) + wide(bias)) * wide(gate)[:, None], 0)))
    # activations, and an fp32 result
    x = store(g.normal((4096, 4096)) * 2)
    xf = wide(x).astype(np.float64)
    tol = 2e-6 if dt == F32 else (2.0 ** -8 if dt == BF16 else 2.0 ** -10)
    for op, ref in (("gelu", lambda t: 0.5 * t * (1 + __import__("scipy.special").special.erf(t / np.sqrt(2.0)))), ("silu", lambda t: t / (1 + np.exp(-t))),
                    ("tanh", np.tanh)):
        p = gh.Rows(x, dt).unary(op)
        got = wide(p.run()).astype(np.float64)
        assert "_map_" in p.kernel_name(), p.kernel_name()
        want = ref(xf)
        assert np.all(np.abs(got - want) <= tol * np.abs(want) + (1e-6 if dt == F32 else 3e-4)), (op, float(np.max(np.abs(got - want))))
    if dt != F32:
        p = gh.Rows(x, dt, F32).unary("square").imm("add", 1.0)
        got = p.run()
        assert "_to_f32_" in p.kernel_name() and "_map_" in p.kernel_name(), p.kernel_name()
        assert np.array_equal(got, wide(x) * wide(x) + np.float32(1.0))
    # truth values: one byte per element, four or eight of them per store
    y = store(g.normal((4096, 4096)) * 2)
    p = gh.Rows(x, dt, gh.U8).binary("gt", y)
    got = p.run()
    assert "_to_u8_" in p.kernel_name() and "_map_" in p.kernel_name(), p.kernel_name()
    assert np.array_equal(got, (wide(x) > wide(y)).astype(np.uint8))
    p = gh.Rows(x, dt, gh.U8).unary("abs").imm("lt", 0.5)
    got = p.run()
    assert "_to_u8_" in p.kernel_name(), p.kernel_name()
    assert np.array_equal(got, (np.abs(wide(x)) < np.float32(0.5)).astype(np.uint8))


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_elementwise_chains_over_rows_no_vector_divides(dt):
    """Flat chains (no row operation, no reduction) over row lengths that no 16-byte vector divides walk the arrays as
    one run of chunks: a chunk may straddle two rows, so per-column and per-row operands are picked by position.
    Exact where the arithmetic is (relu, add, mul in fp32 from the same inputs), to a 16-bit step otherwise; rows
    shorter than a chunk and arrays that start inside a 16-byte block keep the element-wise kernel."""
    g = axo.PCG64(700 + dt)
    e = 4 if dt == F32 else 8
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_f32(t, dt))
    rnd = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_f32(axo.to_bits(t, dt), dt))  # the result's rounding
    for rows, cols in ((9, 1001), (300, 4097), (4, e + 1), (1, 2 * e + 3), (5, e - 1), (33, 50257)):
        x, y = store(g.normal((rows, cols))), store(g.normal((rows, cols)))
        rv, cv, sc = store(g.uniform((cols,), 0.5, 1.5)), store(g.uniform((rows,), 0.5, 1.5)), store(g.uniform((1,), 0.5, 1.5))
        xf, yf, rf, cf, sf = wide(x), wide(y), wide(rv), wide(cv)[:, None], wide(sc)
        name = f"elementwise_flat_e{e}" if cols >= e else "elementwise_e1"
        p = gh.Rows(x, dt).unary("relu").binary("mul", rv, "rowvec").binary("add", y)
        got = wide(p.run())
        assert p.kernel_name() == name, p.kernel_name()
        assert np.array_equal(got, rnd(np.maximum(xf, 0) * rf + yf)), (rows, cols)
        p = gh.Rows(x, dt).binary("add", cv, "colvec").binary("sub", sc, "scalar").imm("mul", 0.5)
        got = wide(p.run())
        assert np.array_equal(got, rnd(((xf + cf) - sf) * np.float32(0.5))), (rows, cols)
        p = gh.Rows(x, dt).unary("silu").binary("mul", y)
        got = wide(p.run()).astype(np.float64)
        want = xf.astype(np.float64) / (1 + np.exp(-xf.astype(np.float64))) * yf
        step = 1e-6 if dt == F32 else (2.0 ** -8 if dt == BF16 else 2.0 ** -11)  # half a unit in the last place of the result, relative
        assert np.all(np.abs(got - want) <= step * np.maximum(np.abs(want), 1e-2) + 1e-6), (rows, cols)
        if dt != F32:  # widening cast: fp32 result, 4-element chunks
            p = gh.Rows(x, dt, F32).binary("mul", rv, "rowvec")
            got = p.run()
            assert p.kernel_name() == ("elementwise_flat_e4" if cols >= 4 else "elementwise_e1"), p.kernel_name()
            assert np.array_equal(got, xf * rf), (rows, cols)
    # an input that starts one element into its buffer: element by element as before
    x = store(g.normal((6, 1001)))
    p = gh.Rows(x, dt).unary("relu")
    pad = gh.to_dev(np.concatenate([np.zeros(1, x.dtype), x.ravel()]))
    p.keep.append(pad)
    p.p.input = pad.data_ptr() + (4 if dt == F32 else 2)
    got = wide(p.run())
    assert p.kernel_name() == "elementwise_e1", p.kernel_name()
    assert np.array_equal(got, np.maximum(wide(x), 0))


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_full_reductions_over_flat_and_row_dependent_chains(dt):
    """A reduction over every element.  Chains of full-size, one-element and immediate operands over aligned arrays
    are reduced as one flat array (16-byte chunks whatever the row length, the elements behind the last whole chunk
    one by one); a per-column or per-row operand, or an array that starts inside a 16-byte block, keeps the
    row-and-column form.  Sum, mean, maximum and minimum against float64."""
    g = axo.PCG64(500 + dt)
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    for rows, cols in ((1, 5), (7, 3), (1, 13), (9, 1001), (300, 4097), (64, 2048), (2048, 4096), (3, 1 << 20)):
        x, y = store(g.normal((rows, cols))), store(g.uniform((rows, cols), 0.5, 1.5))
        xf, yf = wide(x), wide(y)
        yw = g.uniform((rows, cols), 0.5, 1.5).astype(np.float32)  # an fp32 operand beside 16-bit data: 4-element chunks
        rv, cv, sc = store(g.uniform((cols,), 0.5, 1.5)), store(g.uniform((rows,), 0.5, 1.5)), store(g.uniform((1,), 0.5, 1.5))
        n = rows * cols
        cases = [
            (lambda p: p, "sum", xf.sum()), (lambda p: p, "mean", xf.mean()), (lambda p: p, "max", xf.max()), (lambda p: p, "min", xf.min()),
            (lambda p: p.unary("abs"), "max", np.abs(xf).max()),
            (lambda p: p.binary("mul", y), "sum", (xf * yf).sum()),
            (lambda p: p.imm("mul", 0.5).binary("add", yw, "full", F32).unary("square"), "mean", ((xf * 0.5 + yw) ** 2).mean()),
            (lambda p: p.binary("sub", sc, "scalar").unary("relu"), "sum", np.maximum(xf - wide(sc), 0).sum()),
            (lambda p: p.binary("mul", rv, "rowvec"), "sum", (xf * wide(rv)).sum()),
            (lambda p: p.binary("add", cv, "colvec").unary("abs"), "min", np.abs(xf + wide(cv)[:, None]).min()),
        ]
        for build, red, want in cases:
            got = float(build(gh.Rows(x, dt, F32)).run_full_reduce(red)[0])
            if red in ("max", "min"):
                assert abs(got - want) <= 1e-6 * abs(want), (rows, cols, red, got, want)
            else:
                scale = np.abs(xf).sum() * 3 if red == "sum" else np.abs(xf).mean() * 3
                assert abs(got - want) <= 2e-6 * max(scale, 1.0) * (1 if red == "sum" else 4), (rows, cols, red, got, want)
        # the same array from one element into a larger buffer: not 16-byte aligned
        if n >= 2:
            p = gh.Rows(x.reshape(-1)[1:].reshape(1, n - 1), dt, F32)
            pad = gh.to_dev(x.reshape(-1))
            p.keep.append(pad)
            p.p.input = pad.data_ptr() + (4 if dt == F32 else 2)
            got = float(p.run_full_reduce("sum")[0])
            assert abs(got - xf.reshape(-1)[1:].sum()) <= 2e-6 * max(np.abs(xf).sum() * 3, 1.0), (rows, cols)


@pytest.mark.parametrize("rows,cols", [(256, 512), (16, 8192), (3, 100)])
def test_c2_chain_softmax_then_row_sum(rows, cols):
    """softmax((relu(a)+1)*b, -1).sum(1) in ONE launch; plus the intermediate softmax."""
    g = axo.PCG64(42)
    a, b = g.normal((rows, cols)), g.normal((rows, cols))
    want_sum, want_sm = axo.chain_relu_add_mul_softmax_sum(a, b, want_softmax=True)
    got_sm = gh.Rows(a, F32).unary("relu").binary("add", ONE, "scalar").binary("mul", b).row_op("softmax").run()
    assert close32(got_sm, want_sm)
    got_sum = gh.Rows(a, F32).unary("relu").binary("add", ONE, "scalar").binary("mul", b).row_op("softmax").run(reduce="sum")
    assert close32(got_sum, want_sum) and np.allclose(got_sum, 1.0, atol=1e-4)


def ln64(xf, w=None, b=None, eps=1e-5, gelu=False, rms=False):
    x = xf.astype(np.float64)
    if rms:
        y = x / np.sqrt((x**2).mean(-1, keepdims=True) + eps)
    else:
        y = (x - x.mean(-1, keepdims=True)) / np.sqrt(x.var(-1, keepdims=True) + eps)
    if w is not None:
        y = y * w
    if b is not None:
        y = y + b
    if gelu:
        y = 0.5 * y * (1 + np.vectorize(math.erf)(y / math.sqrt(2)))
    return y


@pytest.mark.parametrize("shape", [(4, 5), (16, 96), (32, 4096), (4, 20000), (2, 3, 1280)])
def test_layer_norm_f32(shape):
    g = axo.PCG64(10)
    x = g.normal(shape) * 2 + 0.5
    w, b = g.uniform((shape[-1],), 0.5, 1.5), g.uniform((shape[-1],), -0.1, 0.1)
    got = gh.Rows(x, F32).row_op("layernorm", 1e-5, w, b).run()
    assert close32(got, axo.layer_norm(x, w, b))
    plain = gh.Rows(x, F32).row_op("layernorm", 1e-5).run()
    assert np.allclose(plain.mean(-1), 0, atol=1e-4) and np.allclose(plain.var(-1), 1, atol=1e-2)


def test_rms_norm_f32_known_answers():
    x = np.array([[3.0, 4.0]], np.float32)
    got = gh.Rows(x, F32).row_op("rmsnorm", 0.0, np.ones(2, np.float32)).run()
    assert np.allclose(got, x / math.sqrt(12.5), atol=1e-6)  # tests/test_tensor_normalization.cpp:80-141
    x4 = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    assert abs(gh.Rows(x4, F32).row_op("rmsnorm", 1e-5, np.ones(4, np.float32)).run()[0, 0] - 1 / math.sqrt(7.5)) < 1e-4
    g = axo.PCG64(11)
    x, w = g.normal((9, 200)), g.uniform((200,), 0.5, 1.5)
    assert close32(gh.Rows(x, F32).row_op("rmsnorm", 1e-5, w).run(), axo.rms_norm(x, w))


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("rms", [False, True], ids=["layernorm", "rmsnorm"])
@pytest.mark.parametrize("shape", [(64, 4096), (7, 1280), (3, 100)])
def test_c3_norm_gelu_chain_half(dt, rms, shape):
    """gelu(layer_norm(x)*gamma+beta) and the RMSNorm variant, half in / half out, one launch."""
    g = axo.PCG64(42)
    x = axo.to_bits(g.normal(shape), dt)
    w = axo.to_bits(g.uniform((shape[-1],), 0.5, 1.5), dt)
    b = axo.to_bits(g.uniform((shape[-1],), -0.1, 0.1), dt)
    p = gh.Rows(x, dt).row_op("rmsnorm" if rms else "layernorm", 1e-5, w, None if rms else b).unary("gelu")
    got = axo.to_f32(p.run(), dt)
    xf, wf, bf = (axo.to_f32(t, dt) for t in (x, w, b))
    want = ln64(xf, wf, None if rms else bf, gelu=True, rms=rms)
    err = np.abs(got - want)
    # one rounding of the result to the half type: half an ulp of |y| (bf16: 2^-8 relative)
    ulp = np.maximum(np.abs(want), 1e-3) * (2.0**-8 if dt == BF16 else 2.0**-11)
    assert np.all(err <= np.maximum(2e-2, ulp * 1.01)) and np.max(err[np.abs(want) < 4]) < 2e-2
    # distance to the literal CPU path (float32 output, half-rounded first mean): reported bound
    lit = axo.rms_norm(x, w, dt) if rms else axo.layer_norm(x, w, b, dt)
    lit = axo.unary("gelu", lit)
    assert np.max(np.abs(got - lit)) < 6e-2


def test_mixed_dtype_operands_and_output_dtype():
    g = axo.PCG64(12)
    x = axo.to_bits(g.normal((8, 256)), BF16)
    w = g.uniform((256,), 0.5, 1.5)  # fp32 weights on a bf16 activation
    got = gh.Rows(x, BF16, out_dt=F32).row_op("layernorm", 1e-5, w, None, wdt=F32).run()
    assert got.dtype == np.float32
    assert np.allclose(got, ln64(axo.to_f32(x, BF16), w), atol=1e-4)


def test_full_size_c2_and_c3_properties():
    """BASELINE shapes: C2 fp32 [8192,8192] chain -> every row sums to 1; C3 bf16 [16384,4096]
    layer norm: per-row mean ~ 0 and variance ~ 1; a 256-row slice of each against the oracle."""
    g = axo.PCG64(42)
    a, b = g.normal((8192, 8192)), g.normal((8192, 8192))
    p = gh.Rows(a, F32).unary("relu").binary("add", ONE, "scalar").binary("mul", b).row_op("softmax")
    s = p.run(reduce="sum")
    assert p.kernel_name() == "rows_static_relu_adds_mulf_softmax_sum_f32_g256_it8"  # one specialised launch
    assert np.allclose(s, 1.0, atol=1e-4)
    sm = gh.Rows(a[:256], F32).unary("relu").binary("add", ONE, "scalar").binary("mul", b[:256]).row_op("softmax").run()
    _, want_sm = axo.chain_relu_add_mul_softmax_sum(a[:256], b[:256], want_softmax=True)
    assert close32(sm, want_sm)
    del a, b
    x = axo.to_bits(g.normal((16384, 4096)), BF16)
    y = axo.to_f32(gh.Rows(x, BF16).row_op("layernorm", 1e-5).run(), BF16)
    assert np.allclose(y.mean(-1), 0, atol=2e-3) and np.allclose(y.var(-1), 1, atol=2e-2)
    want = ln64(axo.to_f32(x[:256], BF16))
    assert np.max(np.abs(y[:256] - want)) < 2e-2 + 2.0**-8 * np.max(np.abs(want))


@pytest.fixture
def no_jit(monkeypatch):
    """Run-time compilation off: programs without a built-in kernel run on the interpreter."""
    monkeypatch.setenv("AXHIP_JIT", "0")


def test_empty_inputs_are_no_ops():
    x = np.zeros((0, 16), np.float32)
    assert gh.Rows(x, F32).unary("relu").run().shape == (0, 16)


def test_mixed_chains_around_row_ops_match_oracle():
    """Chains that the specialised kernels do not cover (scalar and unary ops before the row op,
    a reversed subtraction, two full-size operands, a row dot product) run on the interpreter;
    results match the oracle composed op by op."""
    g = axo.PCG64(77)
    x, f = g.normal((48, 2048)), g.normal((48, 2048))
    half = np.array([0.5], np.float32)
    # softmax(exp(x * 0.5) - f) * 3 -> row sum
    p = gh.Rows(x, F32).binary("mul", half, "scalar").unary("exp").binary("sub", f).row_op("softmax").imm("mul", 3.0)
    got = p.run(reduce="sum")
    t = axo.binary("sub", axo.unary("exp", axo.binary("mul", x, half, kind="scalar")), f)
    want = (axo.softmax(t) * np.float32(3.0)).sum(-1)
    assert close32(got, want)
    # f - x (chain on the right-hand side), then rms norm, then sigmoid; bf16
    xb, fb = axo.to_bits(x, BF16), axo.to_bits(f, BF16)
    w = axo.to_bits(g.uniform((2048,), 0.5, 1.5), BF16)
    p = gh.Rows(xb, BF16).binary("rsub", fb).row_op("rmsnorm", 1e-5, w=w).unary("sigmoid")
    got = axo.to_f32(p.run(), BF16)
    d = (axo.to_f32(fb, BF16) - axo.to_f32(xb, BF16)).astype(np.float64)
    r = d / np.sqrt((d * d).mean(-1, keepdims=True) + 1e-5) * axo.to_f32(w, BF16)
    assert np.max(np.abs(got - 1 / (1 + np.exp(-r)))) < 2e-2
    # two different full-size operands: no built-in kernel has that shape, the library compiles one when it is first launched
    f2 = g.normal((48, 2048))
    p = gh.Rows(x, F32).binary("add", f).binary("mul", f2).row_op("softmax")
    got = p.run()
    assert p.kernel_name() == "rows_jit_addf_mulf_softmax_f32_g64_it8", p.kernel_name()
    assert close32(got, axo.softmax((x + f) * f2))
    # row dot product: sum(x * f) per row
    p = gh.Rows(x, F32).binary("mul", f)
    got = p.run(reduce="sum")
    assert np.allclose(got, (x.astype(np.float64) * f).sum(-1), rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_scaled_and_biased_softmax_on_the_specialised_kernels(dt):
    """softmax(x * s), softmax(x + y) and softmax(x * s + y) -- the forms a decomposed attention or a masked
    classifier head produces -- are specialised kernels; s as an immediate and as a one-element device operand."""
    g = axo.PCG64(91)
    tol = 1e-4 if dt == F32 else 2e-2
    for rows, cols in ((33, 512), (7, 4096), (5, 8200 if dt != F32 else 8192)):
        x, y = g.normal((rows, cols)) * 3, g.normal((rows, cols))
        xs, ys = (x.astype(np.float32), y.astype(np.float32)) if dt == F32 else (axo.to_bits(x, dt), axo.to_bits(y, dt))
        xf, yf = (xs, ys) if dt == F32 else (axo.to_f32(xs, dt), axo.to_f32(ys, dt))
        sc = np.array([0.125], np.float32) if dt == F32 else axo.to_bits(np.array([0.125]), dt)
        cases = [(gh.Rows(xs, dt).imm("mul", 0.125).row_op("softmax"), "muls_softmax", xf.astype(np.float64) * 0.125),
                 (gh.Rows(xs, dt).binary("mul", sc, "scalar").row_op("softmax"), "muls_softmax", xf.astype(np.float64) * 0.125),
                 (gh.Rows(xs, dt).binary("add", ys).row_op("softmax"), "addf_softmax", xf.astype(np.float64) + yf),
                 (gh.Rows(xs, dt).imm("mul", 0.125).binary("add", ys).row_op("softmax"), "muls_addf_softmax", xf.astype(np.float64) * 0.125 + yf)]
        for prog, tag, logits in cases:
            got = prog.run()
            # a built-in kernel, or for a row length between the built-in plans (8200 columns) one compiled for it
            assert prog.kernel_name().startswith(("rows_static_" + tag, "rows_jit_" + tag)), prog.kernel_name()
            # (built in: softmax(x * s) and softmax(x + y) for fp32 and bf16 at the stock row lengths; the rest is compiled when first launched)
            assert not (cols % 1024 == 0 and dt != F16 and tag != "muls_addf_softmax" and prog.p.n_operands == (0 if tag == "muls_softmax" else 1)) \
                or prog.kernel_name().startswith("rows_static_"), prog.kernel_name()
            got = got.astype(np.float64) if dt == F32 else axo.to_f32(got, dt).astype(np.float64)
            e = np.exp(logits - logits.max(-1, keepdims=True))
            want = e / e.sum(-1, keepdims=True)
            assert np.max(np.abs(got - want)) < tol, (tag, rows, cols)
    # fp32: the same roundings as the chain evaluated op by op (product, then sum)
    x, y = g.normal((9, 1024)).astype(np.float32), g.normal((9, 1024)).astype(np.float32)
    got = gh.Rows(x, F32).imm("mul", 0.3).binary("add", y).row_op("softmax").run()
    assert close32(got, axo.softmax(axo.binary("add", axo.binary("mul", x, np.array([0.3], np.float32), kind="scalar"), y)))


def test_two_stream_rows_just_past_512_chunks_take_nine_or_ten_chunks_per_lane():
    """Rows of 513 to 640 chunks with a second full-size stream: a wavefront with 9 or 10 chunks per lane (the registers
    of 2 waves per SIMD) instead of a 256-thread block with a third of it idle; values against float64."""
    g = axo.PCG64(123)
    for cols, ragged in ((4099, True), (4104, False), (5000, False)):
        x, y = axo.to_bits(g.normal((37, cols)) * 2, BF16), axo.to_bits(g.normal((37, cols)), BF16)
        w, b = axo.to_bits(g.uniform((cols,), 0.5, 1.5), BF16), axo.to_bits(g.uniform((cols,), -0.5, 0.5), BF16)
        t = axo.to_f32(x, BF16).astype(np.float64) + axo.to_f32(y, BF16)
        it = 9 if cols < 4609 else 10
        prog = gh.Rows(x, BF16).binary("add", y).row_op("layernorm", 1e-5, w=w, b=b)
        got = axo.to_f32(prog.run(), BF16).astype(np.float64)
        assert prog.kernel_name() == f"rows_jit_addf_layernorm_wb_bf16_g64_it{it}" + ("_ragged" if ragged else ""), prog.kernel_name()
        mu, var = t.mean(-1, keepdims=True), t.var(-1, keepdims=True)
        want = (t - mu) / np.sqrt(var + 1e-5) * axo.to_f32(w, BF16) + axo.to_f32(b, BF16)
        assert np.max(np.abs(got - want)) < 3e-2, cols
        prog = gh.Rows(x, BF16).binary("add", y).row_op("softmax")
        got = axo.to_f32(prog.run(), BF16).astype(np.float64)
        assert f"_g64_it{it}" in prog.kernel_name(), prog.kernel_name()
        e = np.exp(t - t.max(-1, keepdims=True))
        assert np.max(np.abs(got - e / e.sum(-1, keepdims=True))) < 2e-2, cols


@pytest.mark.parametrize("post", ["silu", "sigmoid", "tanh"])
def test_fast_activations_after_a_norm_in_16_bit(post):
    g = axo.PCG64(17)
    x = axo.to_bits(g.normal((19, 1024)) * 2, BF16)
    w, b = axo.to_bits(g.uniform((1024,), 0.5, 1.5), BF16), axo.to_bits(g.uniform((1024,), -0.5, 0.5), BF16)
    prog = gh.Rows(x, BF16).row_op("layernorm", 1e-5, w=w, b=b).unary(post)
    got = axo.to_f32(prog.run(), BF16).astype(np.float64)
    assert prog.kernel_name() == f"rows_jit_layernorm_{post}_wb_bf16_g64_it2", prog.kernel_name()  # (of the activations only gelu is built in)
    xf = axo.to_f32(x, BF16).astype(np.float64)
    n = (xf - xf.mean(-1, keepdims=True)) / np.sqrt(xf.var(-1, keepdims=True) + 1e-5) * axo.to_f32(w, BF16) + axo.to_f32(b, BF16)
    want = {"silu": n / (1 + np.exp(-n)), "sigmoid": 1 / (1 + np.exp(-n)), "tanh": np.tanh(n)}[post]
    assert np.max(np.abs(got - want)) < 2e-2


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_vocabulary_sized_rows_stay_in_registers_as_raw_words(dt):
    """Rows of 8193 to 16384 chunks (a language model's vocabulary: 50 304 fp32 or 128 256 16-bit logits) are read once:
    the 1024 threads of a block keep the raw words and every pass -- maximum, sum of exponentials, output -- unpacks
    them and applies the pre chain again.  Aligned and odd lengths, softmax / log-softmax behind a pre chain, both
    norms, a row reduction."""
    g = axo.PCG64(2024)
    tol = 1e-4 if dt == F32 else 2e-2
    to_dev = (lambda a: a.astype(np.float32)) if dt == F32 else (lambda a: axo.to_bits(a, dt))
    to_f64 = (lambda a: a.astype(np.float64)) if dt == F32 else (lambda a: axo.to_f32(a, dt).astype(np.float64))
    tag = {F32: "f32", BF16: "bf16", F16: "f16"}[dt]
    for cols in ((50304, 50257) if dt == F32 else (128256, 100001)):
        ragged = "_grid" if cols % 2 else ""  # odd lengths: chunks on memory's 16-byte grid
        it = (cols + (4 if dt == F32 else 8) * 1024 - 1) // ((4 if dt == F32 else 8) * 1024)
        x = to_dev(g.normal((3, cols)) * 3)
        xf = to_f64(x)
        # softmax(x * 0.5): scaled logits
        p = gh.Rows(x, dt).imm("mul", 0.5).row_op("softmax")
        got = to_f64(p.run())
        assert p.kernel_name() == f"rows_jit_muls_softmax_{tag}_g1024_it{it}{ragged}", p.kernel_name()
        e = np.exp(xf * 0.5 - (xf * 0.5).max(-1, keepdims=True))
        assert np.max(np.abs(got - e / e.sum(-1, keepdims=True))) < tol
        assert np.max(np.abs(got.sum(-1) - 1.0)) < (1e-4 if dt == F32 else 2e-2)
        # log-softmax
        p = gh.Rows(x, dt).row_op("logsoftmax")
        got = to_f64(p.run())
        assert p.kernel_name() == f"rows_jit_logsoftmax_{tag}_g1024_it{it}{ragged}", p.kernel_name()
        want = xf - xf.max(-1, keepdims=True) - np.log(np.exp(xf - xf.max(-1, keepdims=True)).sum(-1, keepdims=True))
        assert np.max(np.abs(got - want)) < (1e-4 if dt == F32 else 2e-2 * 8)  # |log-softmax| reaches 20 here: 16-bit steps of 2^-3
        # layer norm with weight and bias (off-centre rows: mean 3), RMS norm
        w, b = to_dev(g.uniform((cols,), 0.5, 1.5)), to_dev(g.uniform((cols,), -0.5, 0.5))
        x3 = to_dev(g.normal((2, cols)) + 3.0)
        x3f = to_f64(x3)
        p = gh.Rows(x3, dt).row_op("layernorm", 1e-5, w=w, b=b)
        got = to_f64(p.run())
        assert p.kernel_name() == f"rows_jit_layernorm_wb_{tag}_g1024_it{it}{ragged}", p.kernel_name()
        want = (x3f - x3f.mean(-1, keepdims=True)) / np.sqrt(x3f.var(-1, keepdims=True) + 1e-5) * to_f64(w) + to_f64(b)
        assert np.max(np.abs(got - want)) < tol * (1 if dt == F32 else 2)
        p = gh.Rows(x3, dt).row_op("rmsnorm", 1e-5, w=w)
        got = to_f64(p.run())
        want = x3f / np.sqrt((x3f * x3f).mean(-1, keepdims=True) + 1e-5) * to_f64(w)
        assert np.max(np.abs(got - want)) < tol * (1 if dt == F32 else 2)
        # max |x| per row
        p = gh.Rows(x, dt, F32).unary("abs")
        got = p.run(reduce="max")
        assert p.kernel_name() == f"rows_jit_abs_reduce_max_{tag}_g1024_it{it}{ragged}", p.kernel_name()
        assert np.allclose(got.reshape(-1), np.abs(xf).max(-1), rtol=1e-6)
    # two streams: softmax(x + y) over 70 000 16-bit columns is 9 chunks of each per thread
    if dt != F32:
        x, y = to_dev(g.normal((2, 70000)) * 2), to_dev(g.normal((2, 70000)))
        p = gh.Rows(x, dt).binary("add", y).row_op("softmax")
        got = to_f64(p.run())
        assert p.kernel_name() == f"rows_jit_addf_softmax_{tag}_g1024_it9", p.kernel_name()
        lg = to_f64(x) + to_f64(y)
        e = np.exp(lg - lg.max(-1, keepdims=True))
        assert np.max(np.abs(got - e / e.sum(-1, keepdims=True))) < tol


def test_long_rows_on_the_1024_thread_resident_plan_and_the_streamed_one():
    """Rows beyond the 32 KiB the built-in kernels hold: up to 8192 16-byte chunks stay in the registers of a
    512- or 1024-thread block as fp32, up to 16384 as the raw words they were loaded as (one read either way; kernels
    compiled at first launch); longer aligned ones are walked in passes by a compiled kernel, longer odd ones by the
    interpreter."""
    g = axo.PCG64(123)
    for cols, plan in ((12000, "rows_jit_softmax_f32_g512_it6"), (16384, "rows_jit_softmax_f32_g512_it8"), (20000, "rows_jit_softmax_f32_g1024_it5"),
                       (40000, "rows_jit_softmax_f32_g1024_it10"), (70000, "rows_jit_softmax_f32_g1024_it4_loop"), (70001, "rows_streamed_e1")):
        x = (g.normal((3, cols)) * 2).astype(np.float32)
        p = gh.Rows(x, F32).row_op("softmax")
        got = p.run()
        assert p.kernel_name() == plan, p.kernel_name()
        assert close32(got, axo.softmax(x))
    xb = axo.to_bits(g.normal((2, 30000)), BF16)
    w, b = axo.to_bits(g.uniform((30000,), 0.5, 1.5), BF16), axo.to_bits(g.uniform((30000,), -0.5, 0.5), BF16)
    p = gh.Rows(xb, BF16).row_op("layernorm", 1e-5, w=w, b=b).unary("gelu")
    got = axo.to_f32(p.run(), BF16).astype(np.float64)
    assert p.kernel_name() == "rows_jit_layernorm_gelu_wb_bf16_g512_it8", p.kernel_name()
    xf = axo.to_f32(xb, BF16).astype(np.float64)
    n = (xf - xf.mean(-1, keepdims=True)) / np.sqrt(xf.var(-1, keepdims=True) + 1e-5) * axo.to_f32(w, BF16) + axo.to_f32(b, BF16)
    import math
    want = 0.5 * n * (1 + np.vectorize(math.erf)(n / math.sqrt(2)))
    assert np.max(np.abs(got - want)) < 2e-2
    got = gh.Rows(x, F32).unary("square").run(reduce="mean")
    assert np.allclose(got, (x.astype(np.float64) ** 2).mean(-1), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_rows_beyond_the_registers_of_a_block_are_walked_in_passes(dt):
    """Aligned rows of more than 16384 chunks (fp32 logits over a vocabulary of 128 256; two 16-bit streams of that
    length): a 1024-thread block walks the row in steps of four chunks per thread, once for the statistics (online
    softmax reference and sum per thread, merged across the block; sum and sum of squares for the norms, with a centred
    second pass for rows far from zero) and once for the output.  Row lengths that end inside a step and on one."""
    g = axo.PCG64(31 + dt)
    tag = {F32: "f32", BF16: "bf16", F16: "f16"}[dt]
    e = 4 if dt == F32 else 8
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    tol = 1e-5 if dt == F32 else (2.0 ** -8 if dt == BF16 else 2.0 ** -10)
    for cols in (16385 * e, 4096 * e * 5, 128256 * (1 if dt == F32 else 2)):
        x = store(g.normal((3, cols)) * 2)
        xf = wide(x)
        p = gh.Rows(x, dt).row_op("softmax")
        got = wide(p.run())
        assert p.kernel_name() == f"rows_jit_softmax_{tag}_g1024_it4_loop", p.kernel_name()
        ex = np.exp(xf - xf.max(-1, keepdims=True))
        want = ex / ex.sum(-1, keepdims=True)
        assert np.all(np.abs(got - want) <= tol * want + (2.0 ** -24 if dt == F16 else 1e-9)), cols  # (f16: subnormal results step by 2^-24)
        assert np.max(np.abs(got.sum(-1) - 1.0)) < (1e-4 if dt == F32 else 5e-3)
    cols = 20000 * e
    x, y = store(g.normal((2, cols)) * 2), store(g.normal((2, cols)))
    xf, yf = wide(x), wide(y)
    # log-softmax of scaled logits plus a full-size bias, exponentiated again and summed per row: 1
    p = gh.Rows(x, dt, F32).imm("mul", 0.5).binary("add", y).row_op("logsoftmax").unary("exp")
    got = p.run(reduce="sum")
    assert p.kernel_name() == f"rows_jit_muls_addf_logsoftmax_exp_sum_{tag}_g1024_it4_loop", p.kernel_name()
    assert np.max(np.abs(got.astype(np.float64) - 1.0)) < 1e-4
    p = gh.Rows(x, dt).imm("mul", 0.5).binary("add", y).row_op("logsoftmax")
    got = wide(p.run())
    z = xf * 0.5 + yf
    want = z - z.max(-1, keepdims=True) - np.log(np.exp(z - z.max(-1, keepdims=True)).sum(-1, keepdims=True))
    assert np.all(np.abs(got - want) <= tol * np.abs(want) + 1e-5), np.max(np.abs(got - want))
    # layer norm with weight and bias, rows near zero and far from it (mean 40 at sigma 1: the centred second pass)
    w, b = store(g.uniform((cols,), 0.5, 1.5)), store(g.uniform((cols,), -0.5, 0.5))
    for shift in (0.0, 40.0):
        x3 = store(g.normal((2, cols)) + shift)
        x3f = wide(x3)
        p = gh.Rows(x3, dt).row_op("layernorm", 1e-5, w=w, b=b)
        got = wide(p.run())
        assert p.kernel_name() == f"rows_jit_layernorm_wb_{tag}_g1024_it4_loop", p.kernel_name()
        want = (x3f - x3f.mean(-1, keepdims=True)) / np.sqrt(x3f.var(-1, keepdims=True) + 1e-5) * wide(w) + wide(b)
        assert np.max(np.abs(got - want)) < (1e-4 if dt == F32 else 2e-2 * 2), (shift, np.max(np.abs(got - want)))
    p = gh.Rows(x, dt).row_op("rmsnorm", 1e-5, w=w).unary("silu")
    got = wide(p.run())
    n = xf / np.sqrt((xf * xf).mean(-1, keepdims=True) + 1e-5) * wide(w)
    assert np.max(np.abs(got - n / (1 + np.exp(-n)))) < (1e-4 if dt == F32 else 2e-2)
    # reductions without a row operation: one pass
    p = gh.Rows(x, dt, F32).unary("abs")
    got = p.run(reduce="max")
    assert p.kernel_name() == f"rows_jit_abs_reduce_max_{tag}_g1024_it4_loop", p.kernel_name()
    assert np.array_equal(got.reshape(-1).astype(np.float64), np.abs(xf).max(-1))
    p = gh.Rows(x, dt, F32).binary("mul", y)
    got = p.run(reduce="mean")
    assert np.allclose(got.reshape(-1), (xf * yf).mean(-1), rtol=1e-4, atol=1e-5)


def test_unary_then_row_reduction_runs_on_the_specialised_reduce_kernels():
    g = axo.PCG64(321)
    x = (g.normal((37, 4096)) * 2).astype(np.float32)
    xb = axo.to_bits(x, BF16)
    xbf = axo.to_f32(xb, BF16).astype(np.float64)
    p = gh.Rows(x, F32).unary("relu")
    got = p.run(reduce="sum")
    assert p.kernel_name().startswith("rows_jit_relu_reduce_sum_f32"), p.kernel_name()  # (square and abs are built in, relu is compiled on first use)
    assert np.allclose(got, np.maximum(x.astype(np.float64), 0).sum(-1), rtol=1e-4, atol=1e-3)
    p = gh.Rows(xb, BF16, F32).unary("square")
    got = p.run(reduce="mean")
    assert p.kernel_name().startswith("rows_static_square_reduce_sum_bf16"), p.kernel_name()
    assert np.allclose(got, (xbf * xbf).mean(-1), rtol=1e-4, atol=1e-5)
    p = gh.Rows(xb, BF16).unary("abs")
    got = axo.to_f32(p.run(reduce="max"), BF16)
    assert p.kernel_name().startswith("rows_static_abs_reduce_max_bf16"), p.kernel_name()
    assert np.array_equal(got.reshape(-1), np.abs(xbf).max(-1).astype(np.float32))
    # an fp32 result keeps the exact activation (no polynomial GELU under a sum)
    import math
    p = gh.Rows(xb, BF16, F32).unary("gelu")
    got = p.run(reduce="sum")
    want = (0.5 * xbf * (1 + np.vectorize(math.erf)(xbf / math.sqrt(2)))).sum(-1)
    assert np.allclose(got.reshape(-1), want, rtol=1e-4, atol=2e-3)


def test_sum_of_a_sum_and_row_dot_product_on_the_specialised_kernels():
    # tests/test_fusion_extended.cpp:346-352: sum(a + b) over 1s and 3s
    a, b = np.full((4, 2048), 1.0, np.float32), np.full((4, 2048), 3.0, np.float32)
    p = gh.Rows(a, F32).binary("add", b)
    got = p.run(reduce="sum")
    assert p.kernel_name().startswith("rows_static_addf_reduce_sum_f32"), p.kernel_name()
    assert np.all(got == 4.0 * 2048)
    g = axo.PCG64(55)
    x, y = g.normal((21, 4096)).astype(np.float32), g.normal((21, 4096)).astype(np.float32)
    p = gh.Rows(x, F32).binary("mul", y)
    got = p.run(reduce="sum")
    assert p.kernel_name().startswith("rows_static_mulf_reduce_sum_f32"), p.kernel_name()
    assert np.allclose(got.reshape(-1), (x.astype(np.float64) * y).sum(-1), rtol=1e-4, atol=1e-3)
    xb, yb = axo.to_bits(x, BF16), axo.to_bits(y, BF16)
    p = gh.Rows(xb, BF16, F32).binary("mul", yb)
    got = p.run(reduce="mean")
    assert p.kernel_name().startswith("rows_static_mulf_reduce_sum_bf16"), p.kernel_name()
    assert np.allclose(got.reshape(-1), (axo.to_f32(xb, BF16).astype(np.float64) * axo.to_f32(yb, BF16)).mean(-1), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_rows_of_odd_length_on_the_ragged_plans(dt):
    """Column counts that no aligned vector divides (4097, 1001, 77): full-width unaligned accesses plus a partial
    last chunk, on the specialised kernels (softmax of a sum, layer norm with weight and bias, a row reduction) and
    on the interpreter (a chain the specialised set does not hold)."""
    g = axo.PCG64(808)
    for cols in (77, 1001, 4097):
        x, y = g.normal((11, cols)) * 2, g.normal((11, cols))
        w, b = g.uniform((cols,), 0.5, 1.5), g.uniform((cols,), -0.5, 0.5)
        if dt == F32:
            xs, ys, ws, bs = (t.astype(np.float32) for t in (x, y, w, b))
            f = lambda t: t.astype(np.float64)
            out = lambda t: t.astype(np.float64)
        else:
            xs, ys, ws, bs = (axo.to_bits(t, dt) for t in (x, y, w, b))
            f = lambda t: axo.to_f32(t, dt).astype(np.float64)
            out = lambda t: axo.to_f32(t, dt).astype(np.float64)
        tol = 1e-4 if dt == F32 else 2e-2
        p = gh.Rows(xs, dt).binary("add", ys).row_op("softmax")
        got = out(p.run())
        ce = 4 if dt == F32 else 8
        short = (cols + 2 * ce - 2) // ce <= 32  # rows that share a wavefront
        on_grid = short or cols // ce > 128     # ... or 3 chunks per lane and more
        assert p.kernel_name().endswith("_grid" if on_grid else "_ragged"), p.kernel_name()
        lg = f(xs) + f(ys)
        e = np.exp(lg - lg.max(-1, keepdims=True))
        assert np.max(np.abs(got - e / e.sum(-1, keepdims=True))) < tol
        p = gh.Rows(xs, dt).row_op("layernorm", 1e-5, w=ws, b=bs).unary("relu")
        got = out(p.run())
        assert p.kernel_name().endswith("_grid" if short else "_ragged"), p.kernel_name()  # (per-column weights: on the grid only where rows share a wavefront)
        xf = f(xs)
        n = (xf - xf.mean(-1, keepdims=True)) / np.sqrt(xf.var(-1, keepdims=True) + 1e-5) * f(ws) + f(bs)
        assert np.max(np.abs(got - np.maximum(n, 0))) < tol * (1 if dt == F32 else 2)
        p = gh.Rows(xs, dt, F32).unary("square")
        got = p.run(reduce="sum")
        assert np.allclose(got.reshape(-1), (xf * xf).sum(-1), rtol=1e-4, atol=1e-3)
        if cols >= 8:
            assert p.kernel_name().startswith(("rows_static_square_reduce_sum", "rows_jit_square_reduce_sum")) and p.kernel_name().endswith(("_ragged", "_grid")), p.kernel_name()
        p = gh.Rows(xs, dt).row_op("logsoftmax")
        got = out(p.run())
        assert p.kernel_name().endswith(("_ragged", "_grid")), p.kernel_name()
        ref = xf - xf.max(-1, keepdims=True)
        ref = ref - np.log(np.exp(ref).sum(-1, keepdims=True))
        assert np.max(np.abs(got - ref)) < (1e-4 if dt == F32 else 8e-2)  # |log p| reaches 16: half an ulp of a 16-bit result
        for red, fn in (("max", np.max), ("min", np.min)):
            p = gh.Rows(xs, dt, F32)
            got = p.run(reduce=red)
            assert np.array_equal(got.reshape(-1).astype(np.float64), fn(xf, axis=-1)), red  # exact: a selection
        p = gh.Rows(xs, dt).unary("abs").binary("mul", ys).row_op("softmax")
        got = out(p.run())
        assert p.kernel_name().startswith("rows_jit_abs_mulf_softmax_") and p.kernel_name().endswith(("_ragged", "_grid")), p.kernel_name()
        lg = np.abs(f(xs)) * f(ys)
        e = np.exp(lg - lg.max(-1, keepdims=True))
        assert np.max(np.abs(got - e / e.sum(-1, keepdims=True))) < tol


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_bases_that_are_only_element_aligned(dt):
    """Input, residual, weight and bias start a few elements into their buffers (views into larger tensors): the
    specialised kernels take them on their ragged variant, with a column count the vector does divide."""
    g = axo.PCG64(909)
    rows, cols = 9, 1024
    es = 4 if dt == F32 else 2
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    f = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    x, y = store(g.normal((rows, cols)) * 2), store(g.normal((rows, cols)))
    w, b = store(g.uniform((cols,), 0.5, 1.5)), store(g.uniform((cols,), -0.5, 0.5))

    def shifted(p, arr, off):
        pad = gh.to_dev(np.concatenate([np.zeros(off, arr.dtype), arr.ravel()]))
        p.keep.append(pad)
        return pad.data_ptr() + off * es

    p = gh.Rows(x, dt).binary("add", y).row_op("layernorm", 1e-5, w=w, b=b)
    p.p.input = shifted(p, x, 3)
    p.p.operands[0].ptr = shifted(p, y, 1)
    p.p.operands[1].ptr = shifted(p, w, 5)
    p.p.operands[2].ptr = shifted(p, b, 2)
    got = f(p.run())
    assert p.kernel_name().startswith(("rows_static_addf_layernorm", "rows_jit_addf_layernorm")) and p.kernel_name().endswith("_ragged"), p.kernel_name()
    t = f(x) + f(y)
    ref = (t - t.mean(-1, keepdims=True)) / np.sqrt(t.var(-1, keepdims=True) + 1e-5) * f(w) + f(b)
    assert np.max(np.abs(got - ref)) < (1e-4 if dt == F32 else 4e-2)

    p = gh.Rows(x, dt).row_op("softmax")
    p.p.input = shifted(p, x, 1)
    got = f(p.run())
    assert p.kernel_name().endswith("_ragged"), p.kernel_name()  # the output is aligned, the input is not
    e = np.exp(f(x) - f(x).max(-1, keepdims=True))
    assert np.max(np.abs(got - e / e.sum(-1, keepdims=True))) < (1e-4 if dt == F32 else 2e-2)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_ragged_rows_on_the_16_byte_grid_at_the_ends_of_a_plan(dt):
    """Rows addressed on memory's 16-byte grid: the shortest and the longest row each plan takes (the row's last chunk
    in a thread's second-to-last slot for some shifts and in its last slot for others; every slot of the plan used),
    from a base 3 elements past a boundary and with odd lengths, so that consecutive rows meet every shift.  A masked
    store that went wrong would write outside the row: the words around the output keep their pattern, and every
    row is checked against the oracle.  Wavefront, 256- and 1024-thread plans, built in and compiled here, rows held
    as fp32 and as raw words."""
    e, es = (4, 4) if dt == F32 else (8, 2)
    tag = {F32: "f32", BF16: "bf16", F16: "f16"}[dt]
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    f = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    g = axo.PCG64(1616)
    rows, off, pad = 19, 3, 64
    sentinel = np.float32(-77.0) if dt == F32 else np.uint16(0x7FC1)
    for group, it in ((64, 4), (64, 9), (256, 5), (1024, 9)):
        shortest = e * ((it - 1) * group + 1) - (2 * e - 2)
        longest = e * it * group - e + 1
        for cols in (shortest, shortest + 1, longest - 1, longest):
            x = store(g.normal((rows, cols)) * 2)
            xf = f(x)
            src = gh.to_dev(np.concatenate([np.full(off, sentinel, x.dtype), x.ravel()]))
            dst = gh.to_dev(np.full(pad + off + rows * cols + pad, sentinel, x.dtype))
            p = gh.Rows(x[:1], dt).row_op("softmax")
            p.keep += [src, dst]
            p.p.rows, p.p.input = rows, src.data_ptr() + off * es
            p.p.output, p.p.output_dtype = dst.data_ptr() + (pad + off) * es, dt  # pad * es is a multiple of 16: input and output shifted alike
            assert p.kernel_name().endswith(f"softmax_{tag}_g{group}_it{it}_grid"), (cols, p.kernel_name())
            gh.sync()
            gh.capi.check(gh.capi.lib().axhip_fused_rows(gh.C.byref(p.p), None))
            gh.sync()
            out = gh.to_host(dst, x.dtype)
            assert np.all(out[:pad + off] == sentinel) and np.all(out[pad + off + rows * cols:] == sentinel), cols
            got = f(out[pad + off:pad + off + rows * cols].reshape(rows, cols))
            ex = np.exp(xf - xf.max(-1, keepdims=True))
            assert np.max(np.abs(got - ex / ex.sum(-1, keepdims=True))) < (1e-5 if dt == F32 else 2e-3), cols
            # a reduction to [rows] values: exact (a selection), whatever the alignment of its output
            p = gh.Rows(x[:1], dt, F32).unary("abs")
            p.keep.append(src)
            p.p.rows, p.p.input = rows, src.data_ptr() + off * es
            res = gh.empty_dev((rows,), F32)
            p.keep.append(res)
            p.p.output, p.p.output_dtype, p.p.reduce = res.data_ptr(), F32, gh.capi.RED["max"]
            assert p.kernel_name().endswith(f"abs_reduce_max_{tag}_g{group}_it{it}_grid"), (cols, p.kernel_name())
            gh.capi.check(gh.capi.lib().axhip_fused_rows(gh.C.byref(p.p), None))
            gh.sync()
            assert np.array_equal(gh.to_host(res, np.float32).astype(np.float64), np.abs(xf).max(-1)), cols


def test_interpreter_serves_programs_without_a_built_in_kernel_when_run_time_compilation_is_off(no_jit):
    """AXHIP_JIT=0: the shapes the library would compile on first use run on the generic interpreter instead
    (resident plans, their ragged variant, the 1024-thread plan), with the same results."""
    g = axo.PCG64(4242)
    x, f, f2 = g.normal((48, 2048)), g.normal((48, 2048)), g.normal((48, 2048))
    p = gh.Rows(x, F32).binary("add", f).binary("mul", f2).row_op("softmax")
    got = p.run()
    assert p.kernel_name() == "rows_resident_g256_it2_e4", p.kernel_name()
    assert close32(got, axo.softmax((x + f) * f2))
    xs, ys = axo.to_bits(g.normal((11, 1001)) * 2, BF16), axo.to_bits(g.normal((11, 1001)), BF16)
    p = gh.Rows(xs, BF16).unary("abs").binary("mul", ys).row_op("softmax")
    got = axo.to_f32(p.run(), BF16).astype(np.float64)
    assert p.kernel_name().startswith("rows_resident_") and p.kernel_name().endswith("_ragged"), p.kernel_name()
    lg = np.abs(axo.to_f32(xs, BF16).astype(np.float64)) * axo.to_f32(ys, BF16)
    e = np.exp(lg - lg.max(-1, keepdims=True))
    assert np.max(np.abs(got - e / e.sum(-1, keepdims=True))) < 2e-2
    xl = (g.normal((3, 12000)) * 2).astype(np.float32)
    p = gh.Rows(xl, F32).row_op("softmax")
    got = p.run()
    assert p.kernel_name() == "rows_resident_g1024_it4_e4", p.kernel_name()
    assert close32(got, axo.softmax(xl))
    # a built-in shape is not affected by the switch
    p = gh.Rows(x, F32).row_op("softmax")
    p.run()
    assert p.kernel_name() == "rows_static_softmax_f32_g64_it8", p.kernel_name()


@pytest.mark.parametrize("rms", [False, True], ids=["layernorm", "rmsnorm"])
def test_full_size_c3_chain_with_weights_and_gelu(rms):
    """BASELINE configs[2] as it is benchmarked: gelu(layer_norm(x) * gamma + beta) and the RMSNorm variant on bf16
    [16384, 4096].  Every row is checked through statistics that do not depend on its position (the pre-activation
    is recovered where gelu is injective), and slices from the start, the middle and the END of the tensor go against
    the float64 evaluation element by element."""
    g = axo.PCG64(4242)
    R, Cc = 16384, 4096
    x = axo.to_bits(g.normal((R, Cc)), BF16)
    w = axo.to_bits(g.uniform((Cc,), 0.5, 1.5), BF16)
    b = axo.to_bits(g.uniform((Cc,), -0.1, 0.1), BF16)
    p = gh.Rows(x, BF16).row_op("rmsnorm" if rms else "layernorm", 1e-5, w, None if rms else b).unary("gelu")
    got = axo.to_f32(p.run(), BF16)
    assert p.kernel_name() == ("rows_static_rmsnorm_gelu_w_bf16_g64_it8" if rms else "rows_static_layernorm_gelu_wb_bf16_g64_it8")
    assert np.isfinite(got).all()
    wf, bf = axo.to_f32(w, BF16), axo.to_f32(b, BF16)
    for lo, hi in ((0, 96), (R // 2 - 48, R // 2 + 48), (R - 96, R)):
        want = ln64(axo.to_f32(x[lo:hi], BF16), wf, None if rms else bf, gelu=True, rms=rms)
        err = np.abs(got[lo:hi] - want)
        ulp = np.maximum(np.abs(want), 1e-3) * 2.0**-8
        assert np.all(err <= np.maximum(2e-2, ulp * 1.01)) and np.max(err[np.abs(want) < 4]) < 2e-2, (lo, hi)
    # all 16384 rows: where y > 1 gelu is increasing and y ~ n to within 0.16, so n = (y solved back) has the row's
    # normalised statistics; cheaper and as telling: the mean of gelu(n) over a row of N(0,1)-like n * w + b is stable.
    # Compare per-row means and mean squares with the float64 evaluation of a strided sample of rows.
    rows = np.arange(0, R, 61)
    want = ln64(axo.to_f32(x[rows], BF16), wf, None if rms else bf, gelu=True, rms=rms)
    assert np.allclose(got[rows].mean(-1), want.mean(-1), atol=2e-3)
    assert np.allclose((got[rows].astype(np.float64) ** 2).mean(-1), (want**2).mean(-1), rtol=5e-3)
    # and every row against its neighbours' scale: no row left unwritten or written twice with another row's statistics
    ms = (got.astype(np.float64) ** 2).mean(-1)
    assert ms.min() > 0.2 and ms.max() < 1.5, (ms.min(), ms.max())


@pytest.mark.parametrize("dt,offset,spread", [(BF16, 8.0, 0.5), (F16, 64.0, 0.25), (BF16, 300.0, 3.0), (F16, -1000.0, 2.0)],
                         ids=["bf16_ratio16", "f16_ratio256", "bf16_ratio100", "f16_ratio500"])
@pytest.mark.parametrize("cols", [4096, 1000, 16384])
def test_layer_norm_of_16_bit_rows_far_from_zero(dt, offset, spread, cols):
    """Rows whose mean dwarfs their spread (|mean| / sigma from 16 to 500): the one-sweep variance E[x^2] - mean^2
    loses its digits there, and the kernels re-sweep such rows with the mean taken out (the reference's CPU path is
    two-pass, src/tensor/operations.cpp:1803-1817).  Checked against float64 on the rounded inputs, plain and behind a
    residual sum (statistics of fp32 sums instead of the packed input)."""
    g = axo.PCG64(777)
    x = axo.to_bits(offset + spread * g.normal((9, cols)), dt)
    xf = axo.to_f32(x, dt).astype(np.float64)
    w = axo.to_bits(g.uniform((cols,), 0.5, 1.5), dt)
    b = axo.to_bits(g.uniform((cols,), -0.5, 0.5), dt)
    wf, bf = axo.to_f32(w, dt).astype(np.float64), axo.to_f32(b, dt).astype(np.float64)

    def ln(t):
        return (t - t.mean(-1, keepdims=True)) / np.sqrt(t.var(-1, keepdims=True) + 1e-5) * wf + bf

    tol = lambda want: np.maximum(2e-2, np.abs(want) * (2.0**-8 if dt == BF16 else 2.0**-11) * 1.01)
    got = axo.to_f32(gh.Rows(x, dt).row_op("layernorm", 1e-5, w, b).run(), dt)
    want = ln(xf)
    assert np.all(np.abs(got - want) <= tol(want)), float(np.max(np.abs(got - want)))
    y = axo.to_bits(spread * g.normal((9, cols)), dt)
    got = axo.to_f32(gh.Rows(x, dt).binary("add", y).row_op("layernorm", 1e-5, w, b).run(), dt)
    want = ln(xf + axo.to_f32(y, dt))
    assert np.all(np.abs(got - want) <= tol(want)), float(np.max(np.abs(got - want)))


def _random_row_program(r, g, dt, many_short_rows=False):
    """A seeded random program and its float64 evaluation on the values the device reads (16-bit inputs widened)."""
    store = (lambda t: t.astype(np.float32)) if dt == F32 else (lambda t: axo.to_bits(t, dt))
    wide = (lambda t: t.astype(np.float64)) if dt == F32 else (lambda t: axo.to_f32(t, dt).astype(np.float64))
    if many_short_rows:
        rows = int(r.integers(32768, 33100))
        cols = int(r.choice([3, 10, 45, 77, 101, 197, 250, 333]))
    else:
        rows = int(r.integers(1, 24))
        cols = int(r.choice([5, 64, 100, 777, 1001, 1024, 1500, 2048, 3000, 4097, 5000, 9000, 12288, 20000, 40001, 140000]))
    x = store(g.normal((rows, cols)) * 1.5)
    row_op = str(r.choice(["none", "softmax", "logsoftmax", "layernorm", "rmsnorm", "softmax", "layernorm"]))
    reduce = str(r.choice(["sum", "max", "mean"])) if row_op == "none" else str(r.choice(["none", "none", "none", "sum", "max"]))
    out_dt = F32 if (reduce != "none" or r.integers(0, 5) == 0) else dt
    p = gh.Rows(x, dt, out_dt)
    ref = wide(x)
    desc = []

    def operand(kind):
        shape = {"full": (rows, cols), "rowvec": (cols,), "colvec": (rows,), "scalar": (1,)}[kind]
        v = store(g.uniform(shape, 0.5, 1.5) * (1 if r.integers(0, 2) else -1))
        w = wide(v)
        return v, (w[:, None] if kind == "colvec" else w)

    def chain(n_ops, choices):
        nonlocal ref
        for _ in range(n_ops):
            op = str(r.choice(choices))
            desc.append(op)
            if op in ("relu", "abs", "neg", "tanh", "sigmoid", "silu", "gelu", "square"):
                p.unary(op)
                ref = {"relu": lambda t: np.maximum(t, 0), "abs": np.abs, "neg": lambda t: -t, "tanh": np.tanh,
                       "sigmoid": lambda t: 1 / (1 + np.exp(-t)), "silu": lambda t: t / (1 + np.exp(-t)),
                       "gelu": lambda t: 0.5 * t * (1 + __import__("scipy.special").special.erf(t / np.sqrt(2.0))), "square": lambda t: t * t}[op](ref)
            elif op in ("mul_imm", "add_imm"):
                c = float(np.float32(r.uniform(0.25, 2.0)))
                p.imm(op[:3], c)
                ref = ref * c if op == "mul_imm" else ref + c
            else:  # add / mul / sub / max with an operand of some broadcast kind
                name, kind = op.split("_")
                v, w = operand(kind)
                p.binary(name, v, kind)
                ref = {"add": ref + w, "mul": ref * w, "sub": ref - w, "max": np.maximum(ref, w)}[name]

    binary = [f"{o}_{k}" for o in ("add", "mul", "sub", "max") for k in ("full", "rowvec", "colvec", "scalar")]
    chain(int(r.integers(0, 4)), ["relu", "abs", "neg", "tanh", "mul_imm", "add_imm"] + binary)
    if row_op != "none":
        desc.append(row_op)
        if row_op in ("softmax", "logsoftmax"):
            p.row_op(row_op)
            z = ref - ref.max(-1, keepdims=True)
            lse = np.log(np.exp(z).sum(-1, keepdims=True))
            ref = np.exp(z - lse) if row_op == "softmax" else z - lse
        else:
            affine = int(r.integers(0, 3)) if row_op == "layernorm" else int(r.integers(0, 2))
            w = store(g.uniform((cols,), 0.5, 1.5)) if affine >= 1 else None
            b = store(g.uniform((cols,), -0.5, 0.5)) if affine >= 2 else None
            p.row_op(row_op, 1e-5, w=w, b=b)
            if row_op == "layernorm":
                ref = (ref - ref.mean(-1, keepdims=True)) / np.sqrt(ref.var(-1, keepdims=True) + 1e-5)
            else:
                ref = ref / np.sqrt((ref * ref).mean(-1, keepdims=True) + 1e-5)
            if w is not None:
                ref = ref * wide(w)
            if b is not None:
                ref = ref + wide(b)
        chain(int(r.integers(0, 3)), ["relu", "gelu", "silu", "sigmoid", "tanh", "mul_imm", "add_imm", "mul_full", "add_rowvec", "mul_colvec"])
    mag = np.abs(ref)  # what the result's rounding errors scale with: for a sum, the sum of the magnitudes
    if reduce != "none":
        desc.append("reduce_" + reduce)
        mag = {"sum": mag.sum(-1), "max": np.abs(ref.max(-1)), "mean": mag.mean(-1)}[reduce]
        ref = {"sum": ref.sum(-1), "max": ref.max(-1), "mean": ref.mean(-1)}[reduce]
    return p, reduce, ref, mag, out_dt, f"{rows}x{cols} " + " ".join(desc)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_seeded_random_row_programs_match_fp64(dt):
    """Forty seeded random programs per element type: up to three pre operations (unary, immediate, operands of all four
    broadcast kinds), a row operation with or without affine part, up to two post operations, an optional row
    reduction, fp32 or same-type results, over row lengths from 5 to 140 000 (aligned, odd, one to 1024 threads per
    row, rows walked in passes) -- whatever kernel the library picks (built in, compiled here, interpreter), against float64."""
    r = np.random.default_rng(4242 + dt)
    g = axo.PCG64(99 + dt)
    kinds = set()
    for case in range(40):
        p, reduce, ref, mag, out_dt, desc = _random_row_program(r, g, dt)
        got = p.run(reduce=reduce)
        name = p.kernel_name()
        kinds.add(name.split("_")[1])
        got = got.astype(np.float64) if out_dt == F32 else axo.to_f32(got, out_dt).astype(np.float64)
        # the device computes in fp32 from the same inputs; a 16-bit result adds half an ulp of its own
        ulp = {F32: 0.0, BF16: 2.0 ** -8, F16: 2.0 ** -11}[out_dt]
        tol = 4e-5 * np.maximum(1.0, mag) + ulp * np.abs(ref) + (0.0 if out_dt == F32 else 1e-7)
        if dt != F32 and out_dt != F32:
            tol = tol + 2e-4  # the polynomial activations behind a 16-bit result
        err = np.abs(got.reshape(ref.shape) - ref)
        assert np.all(err <= tol), (case, desc, name, float(np.max(err / tol)))
    assert ({"jit"} if dt == F16 else {"static", "jit"}) <= kinds, kinds  # (no f16 shape is built in)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_seeded_random_row_programs_over_many_short_odd_rows_match_fp64(dt):
    """Twelve of the same random programs per element type over 32768 to 33100 rows of 3 to 333 columns: the rows of
    a wavefront staged in LDS, one to eight lanes per row, full-size operands as further spans, per-column operands as
    tables, results of the input's type or fp32, row reductions -- against float64."""
    r = np.random.default_rng(777 + dt)
    g = axo.PCG64(55 + dt)
    staged = 0
    for case in range(12):
        p, reduce, ref, mag, out_dt, desc = _random_row_program(r, g, dt, many_short_rows=True)
        got = p.run(reduce=reduce)
        name = p.kernel_name()
        staged += "_lane" in name
        got = got.astype(np.float64) if out_dt == F32 else axo.to_f32(got, out_dt).astype(np.float64)
        ulp = {F32: 0.0, BF16: 2.0 ** -8, F16: 2.0 ** -11}[out_dt]
        tol = 4e-5 * np.maximum(1.0, mag) + ulp * np.abs(ref) + (0.0 if out_dt == F32 else 1e-7)
        if dt != F32 and out_dt != F32:
            tol = tol + 2e-4
        err = np.abs(got.reshape(ref.shape) - ref)
        assert np.all(err <= tol), (case, desc, name, float(np.max(err / tol)))
    assert staged >= 8, staged


def test_run_time_compiled_kernels_come_back_from_the_on_disk_cache(tmp_path):
    """A process that finds the code object of a "rows_jit_" kernel in AXHIP_CACHE_DIR loads it instead of compiling
    it again; the result is the same bits.  Two fresh processes, the second after the first."""
    import os
    import subprocess
    import sys

    script = r'''
import ctypes as C, sys, numpy as np
from oracle import axo
from tests import gpu_harness as gh
g = axo.PCG64(77)
x = axo.to_bits(g.normal((33, 1536)), axo.BF16)
w, b = axo.to_bits(g.uniform((1536,), 0.5, 1.5), axo.BF16), axo.to_bits(g.uniform((1536,), -0.1, 0.1), axo.BF16)
prog = gh.Rows(x, axo.BF16).row_op("layernorm", 1e-5, w=w, b=b).unary("sigmoid")
y = prog.run()
assert prog.kernel_name().startswith("rows_jit_"), prog.kernel_name()
d, c = C.c_int(0), C.c_int(0)
gh.capi.lib().axhip_fused_rows_jit_counters(C.byref(d), C.byref(c))
print("COUNTERS", d.value, c.value, int(np.asarray(y, np.uint16).astype(np.uint64).sum()))
'''
    env = dict(os.environ, AXHIP_CACHE_DIR=str(tmp_path / "axhip-cache"), PYTHONPATH=os.pathsep.join([os.getcwd(), os.environ.get("PYTHONPATH", "")]))
    outs = []
    for _ in range(2):
        r = subprocess.run([sys.executable, "-c", script], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
        assert r.returncode == 0, r.stdout[-2000:]
        outs.append([ln for ln in r.stdout.splitlines() if ln.startswith("COUNTERS")][-1].split()[1:])
    (d1, c1, sum1), (d2, c2, sum2) = outs
    assert (int(d1), int(c1)) == (0, 1), outs  # compiled, stored
    assert (int(d2), int(c2)) == (1, 0), outs  # loaded
    assert sum1 == sum2
    assert any(f.suffix == ".hsaco" for f in (tmp_path / "axhip-cache").iterdir())
