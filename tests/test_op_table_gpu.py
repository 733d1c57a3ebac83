"""GPU parity of the wider operator table (power, modulo, comparisons, logical operations, the trigonometric and
rounding functions, the is* tests, leaky ReLU, where, Bool casts, prod / any / all) against the CPU oracle and
the reference tests' own expectations, through the C ABI.

Tolerances: comparisons, logical operations, rounding functions, sign, where and casts are bit-exact; the
library routines (pow, fmod, sin ...) 1e-5 relative + 1e-6 absolute in fp32; 16-bit results within one rounding
step of the fp32 evaluation of the same inputs (2e-2 absolute at the magnitudes used here)."""
import ctypes as C
import math

import numpy as np
import pytest
import torch

from axiom_amd import capi
from oracle import axo
from tests import gpu_harness as gh

pytestmark = pytest.mark.gpu
F32, F16, BF16, U8 = gh.F32, gh.F16, gh.BF16, gh.U8

TRUTH_UNARY = ["isnan", "isinf", "isfinite", "not"]
EXACT_UNARY = ["sign", "floor", "ceil", "round", "trunc"]
LIB_UNARY = ["erf", "sin", "cos", "tan", "cbrt"]
TRUTH_BINARY = ["eq", "ne", "lt", "le", "gt", "ge", "and", "or", "xor"]
LIB_BINARY = ["pow", "rpow", "mod", "rmod", "atan2", "ratan2", "hypot"]


def i64(values):
    return (C.c_int64 * len(values))(*values)


def special(shape, seed):
    """N(0, 2) values salted with zeros, halves, infinities and NaN."""
    x = axo.PCG64(seed).normal(shape, 0.0, 2.0)
    flat = x.reshape(-1)
    flat[::7] = 0.0
    flat[1::11] = np.float32(2.5)
    flat[2::13] = np.float32(-0.5)
    flat[3::17] = np.inf
    flat[4::19] = -np.inf
    flat[5::23] = np.nan
    return x


def same(got, want):
    return np.array_equal(got, want, equal_nan=True)


def close(got, want, rtol=1e-5, atol=1e-6):
    return np.allclose(got, want, rtol=rtol, atol=atol, equal_nan=True)


@pytest.mark.parametrize("shape", [(17, 96), (5, 37), (3, 1000)], ids=["vec", "scalar", "flat"])
@pytest.mark.parametrize("op", TRUTH_UNARY + EXACT_UNARY + LIB_UNARY)
def test_unary_operators_elementwise(op, shape):
    x = special(shape, 31)
    if op in LIB_UNARY:
        x = np.nan_to_num(x, nan=0.25, posinf=3.0, neginf=-3.0)
    want = axo.unary(op, x)
    if op in TRUTH_UNARY:
        got = gh.Rows(x, F32, out_dt=U8).unary(op).run()
        assert got.dtype == np.uint8 and same(got, (want != 0).astype(np.uint8)), op
        assert same(gh.Rows(x, F32).unary(op).run(), want), op  # the same as 1.0 / 0.0 in a float result
    elif op in EXACT_UNARY:
        assert same(gh.Rows(x, F32).unary(op).run(), want), op
    else:
        assert close(gh.Rows(x, F32).unary(op).run(), want), op


@pytest.mark.parametrize("kind", ["full", "rowvec", "colvec", "scalar", "imm"])
@pytest.mark.parametrize("op", TRUTH_BINARY + LIB_BINARY + ["leaky_relu"])
def test_binary_operators_and_broadcast_kinds(op, kind):
    g = axo.PCG64(32)
    a = special((9, 40), 33)
    b = {"full": g.normal((9, 40)), "rowvec": g.normal((40,)), "colvec": g.normal((9,)), "scalar": g.normal((1,)), "imm": np.array([0.75], np.float32)}[kind]
    b = b.copy()
    b.reshape(-1)[::3] = 2.5  # ties with the 2.5 entries of a
    if op in LIB_BINARY:
        a = np.nan_to_num(a, nan=0.25, posinf=3.0, neginf=-3.0)
        if op in ("pow", "rpow"):
            a, b = np.abs(a) + 0.25, np.abs(b) + 0.25
        if op in ("mod", "rmod"):
            a, b = a + np.float32(0.125) * (a == 0), np.abs(b) + 0.5
    want = axo.binary(op, a, b, kind="scalar" if kind == "imm" else kind)
    prog = (lambda dt: gh.Rows(a, F32, out_dt=dt).imm(op, b[0]) if kind == "imm" else gh.Rows(a, F32, out_dt=dt).binary(op, b, kind))
    if op in TRUTH_BINARY:
        assert same(prog(U8).run(), (want != 0).astype(np.uint8)), (op, kind)
    elif op == "leaky_relu":
        assert same(prog(F32).run(), want), (op, kind)
    else:
        assert close(prog(F32).run(), want), (op, kind)


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
def test_comparisons_of_16_bit_values_and_truth_inputs(dt):
    a, b = axo.to_bits(special((12, 64), 34), dt), axo.to_bits(special((12, 64), 35), dt)
    for op in TRUTH_BINARY:
        want = axo.to_f32(axo.binary(op, a, b, dt), dt)
        assert same(gh.Rows(a, dt, out_dt=U8).binary(op, b).run(), (want != 0).astype(np.uint8)), op
    # Bool inputs and operands: logical operations over byte arrays (tests/test_tensor_logical_bitwise.cpp:11-58)
    la = np.array([[1, 1, 0, 0]], np.uint8)
    lb = np.array([[1, 0, 1, 0]], np.uint8)
    assert gh.Rows(la, U8, out_dt=U8).binary("and", lb, dt=U8).run().tolist() == [[1, 0, 0, 0]]
    assert gh.Rows(la, U8, out_dt=U8).binary("or", lb, dt=U8).run().tolist() == [[1, 1, 1, 0]]
    assert gh.Rows(la, U8, out_dt=U8).binary("xor", lb, dt=U8).run().tolist() == [[0, 1, 1, 0]]
    assert gh.Rows(np.array([[1, 0, 1, 0]], np.uint8), U8, out_dt=U8).unary("not").run().tolist() == [[0, 1, 0, 1]]
    # any nonzero byte is true, and a truth value read into a float chain is 1.0
    big = (np.arange(24 * 64).reshape(24, 64) % 5).astype(np.uint8) * 51
    other = (np.arange(24 * 64).reshape(24, 64) % 3).astype(np.uint8)
    assert same(gh.Rows(big, U8, out_dt=U8).binary("and", other, dt=U8).run(), ((big != 0) & (other != 0)).astype(np.uint8))
    assert same(gh.Rows(big, U8, out_dt=F32).imm("mul", 3.0).run(), (big != 0).astype(np.float32) * 3)


def test_reference_known_answers_on_gpu():
    f = lambda *v: np.array([v], np.float32)
    a5, two5 = f(0, 1, 2, 3, 4), f(2, 2, 2, 2, 2)
    cmp = lambda op: gh.Rows(a5, F32, out_dt=U8).binary(op, two5).run()[0].astype(bool).tolist()
    # tests/test_tensor_comparisons.cpp:24-113 (and their GPU twins :141-219)
    assert cmp("lt") == [True, True, False, False, False]
    assert cmp("le") == [True, True, True, False, False]
    assert cmp("gt") == [False, False, False, True, True]
    assert cmp("ge") == [False, False, True, True, True]
    assert cmp("ne") == [True, True, False, True, True]
    # tests/test_tensor_numpy_ops.cpp:13-79 (GPU twins :487-560)
    assert same(gh.Rows(f(-3, -1, 0, 1, 3), F32).unary("sign").run(), f(-1, -1, 0, 1, 1))
    x = f(-2.7, -0.5, 0.5, 2.7)
    assert same(gh.Rows(x, F32).unary("floor").run(), f(-3, -1, 0, 2))
    assert same(gh.Rows(x, F32).unary("ceil").run(), f(-2, 0, 1, 3))
    assert same(gh.Rows(x, F32).unary("trunc").run(), f(-2, 0, 0, 2))
    assert close(gh.Rows(f(8, 27, 64), F32).unary("cbrt").run(), f(2, 3, 4), atol=1e-5)
    t = f(1.0, np.nan, np.inf, -np.inf, 0.0)
    assert gh.Rows(t, F32, out_dt=U8).unary("isnan").run()[0].tolist() == [0, 1, 0, 0, 0]
    assert gh.Rows(t, F32, out_dt=U8).unary("isinf").run()[0].tolist() == [0, 0, 1, 1, 0]
    assert gh.Rows(t, F32, out_dt=U8).unary("isfinite").run()[0].tolist() == [1, 0, 0, 0, 1]
    assert same(gh.Rows(f(-5, -1, 0, 1, 5), F32).imm("min", 2.0).imm("max", -2.0).run(), f(-2, -1, 0, 1, 2))  # clip
    # tests/test_tensor_operations.cpp:107-121; tests/test_tensor_logical_bitwise.cpp:245-292
    assert np.allclose(gh.Rows(np.full((2, 2), 3.0, np.float32), F32).binary("pow", np.full((2, 2), 4.0, np.float32)).run(), 81.0, atol=1e-4)
    assert close(gh.Rows(f(1, 1, 0), F32).binary("atan2", f(1, 0, 1)).run(), f(math.pi / 4, math.pi / 2, 0), atol=1e-6)
    assert close(gh.Rows(f(3, 0, 5), F32).binary("hypot", f(4, 5, 12)).run(), f(5, 5, 13), atol=1e-5)
    # tests/test_tensor_activations.cpp:356-375
    e = gh.Rows(f(0, 1, -1), F32).unary("erf").run()[0]
    assert abs(e[0]) < 1e-6 and abs(e[1] - 0.8427) < 1e-4 and abs(e[1] + e[2]) < 1e-6
    # tests/test_tensor_numpy_ops.cpp:91-104, tests/test_fusion_extended.cpp:376-385, tests/test_tensor_activations.cpp:446-478
    assert gh.Rows(f(1, 2, 3, 4), F32).run("prod")[0] == 24.0
    assert abs(gh.Rows(f(4, 9, 16), F32).unary("sqrt").run_full_reduce("prod")[0] - 24.0) < 1e-4
    assert gh.Rows(f(0, 0, 1, 0), F32, out_dt=U8).imm("ne", 0.0).run_full_reduce("max")[0] == 1  # any
    assert gh.Rows(f(1, 1, 1, 1), F32, out_dt=U8).imm("ne", 0.0).run_full_reduce("min")[0] == 1  # all
    assert gh.Rows(f(1, 0, 1, 1), F32, out_dt=U8).imm("ne", 0.0).run_full_reduce("min")[0] == 0
    # fmod keeps the dividend's sign, halves round away from zero, the slope of leaky ReLU
    assert same(gh.Rows(f(5.5, -5.5, 5.5, -5.5), F32).binary("mod", f(2, 2, -2, -2)).run(), f(1.5, -1.5, 1.5, -1.5))
    assert same(gh.Rows(f(0.5, 1.5, 2.5, -0.5, -1.5, 2.4), F32).unary("round").run(), f(1, 2, 3, -1, -2, 2))
    assert close(gh.Rows(f(-2, 3, 0), F32).imm("leaky_relu", 0.01).run(), f(-0.02, 3.0, 0.0), atol=1e-9)


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("cols", [256, 1000, 4096], ids=["c256", "c1000", "c4096"])
def test_operators_inside_compiled_row_programs(dt, cols):
    """The same operators in front of and behind a softmax and under a row reduction: the kernels the library
    compiles for the program (or has built in), not the interpreter."""
    g = axo.PCG64(36)
    xf = g.normal((24, cols))
    bf = g.normal((24, cols))
    x, b = (xf, bf) if dt == F32 else (axo.to_bits(xf, dt), axo.to_bits(bf, dt))
    x64 = (xf if dt == F32 else axo.to_f32(x, dt)).astype(np.float64)
    b64 = (bf if dt == F32 else axo.to_f32(b, dt)).astype(np.float64)
    tol = 1e-4 if dt == F32 else 2e-2
    val = lambda r: r if dt == F32 else axo.to_f32(r, dt)

    # sum(sin(x) * (x > b)) per row
    p = gh.Rows(x, dt).binary("gt", b).binary("mul", x).unary("sin")
    got = val(p.run("sum"))
    want = np.sin((x64 > b64) * x64).sum(-1)
    assert p.kernel_name().startswith(("rows_jit_", "rows_static_")), p.kernel_name()
    assert np.allclose(got, want, rtol=tol, atol=tol * math.sqrt(cols)), p.kernel_name()

    # softmax(leaky_relu(x, 0.1) - floor(b)) then sign(.. - 1/cols)
    p = gh.Rows(x, dt).imm("leaky_relu", 0.1).row_op("softmax").imm("sub", 1.0 / cols).unary("sign")
    got = val(p.run())
    z = np.where(x64 > 0, x64, np.float64(np.float32(0.1)) * x64)
    sm = np.exp(z - z.max(-1, keepdims=True))
    sm /= sm.sum(-1, keepdims=True)
    clear = np.abs(sm - 1.0 / cols) > (1e-6 if dt == F32 else 1e-3) / cols  # away from the sign's jump
    assert p.kernel_name().startswith(("rows_jit_", "rows_static_")), p.kernel_name()
    assert np.array_equal(got[clear], np.sign(sm - 1.0 / cols)[clear]), p.kernel_name()

    # any / all per row: a one-byte result from a compiled reduction kernel
    xz = xf.copy()
    xz[::2] = np.abs(xz[::2]) + 1.0  # rows without a zero
    xz[1::4, cols // 2] = 0.0
    xin = xz if dt == F32 else axo.to_bits(xz, dt)
    nz = (xz if dt == F32 else axo.to_f32(xin, dt)) != 0
    p_any = gh.Rows(xin, dt, out_dt=U8).imm("ne", 0.0)
    assert same(p_any.run("max"), nz.any(-1).astype(np.uint8)), p_any.kernel_name()
    p_all = gh.Rows(xin, dt, out_dt=U8).imm("ne", 0.0)
    assert same(p_all.run("min"), nz.all(-1).astype(np.uint8)), p_all.kernel_name()
    assert p_all.kernel_name().startswith(("rows_jit_", "rows_static_")), p_all.kernel_name()


@pytest.mark.parametrize("shape", [(4, 5), (64, 64), (5, 4096), (3, 50000)])
def test_row_and_full_products(shape):
    x = (1.0 + 0.01 * axo.PCG64(37).normal(shape)).astype(np.float32)
    x[0, 0] = -1.0
    want = x.astype(np.float64).prod(-1)
    got = gh.Rows(x, F32).run("prod")
    assert np.allclose(got, want, rtol=1e-4), shape
    full = gh.Rows(x, F32).run_full_reduce("prod")[0]
    assert math.isclose(full, x.astype(np.float64).prod(), rel_tol=2e-4), shape
    xb = axo.to_bits(x, BF16)
    gotb = axo.to_f32(gh.Rows(xb, BF16).run("prod"), BF16)
    assert np.allclose(gotb, axo.to_f32(xb, BF16).astype(np.float64).prod(-1), rtol=1e-2), shape
    # a chain in front: prod(|x| * 0.9999) over everything
    p = gh.Rows(x, F32).unary("abs").imm("mul", 0.9999)
    assert math.isclose(p.run_full_reduce("prod")[0], (np.abs(x.astype(np.float64)) * np.float64(np.float32(0.9999))).prod(), rel_tol=5e-4)


def _reduce_axis(dev, dt, outer, axis, inner, red, out_dt):
    out = gh.empty_dev((outer * inner,), out_dt)
    gh.sync()
    capi.check(capi.lib().axhip_reduce_axis(dev.data_ptr(), dt, outer, axis, inner, capi.RED[red], out.data_ptr(), out_dt, None))
    gh.sync()
    return gh.to_host(out, gh.np_store_dtype(out_dt))


def test_products_and_truth_reductions_along_inner_axes():
    x = (1.0 + 0.02 * axo.PCG64(38).normal((6, 33, 40))).astype(np.float32)
    got = _reduce_axis(gh.to_dev(x), F32, 6, 33, 40, "prod", F32).reshape(6, 40)
    assert np.allclose(got, x.astype(np.float64).prod(1), rtol=1e-4)
    xb = axo.to_bits(x, BF16)
    gotb = axo.to_f32(_reduce_axis(gh.to_dev(xb), BF16, 6, 33, 40, "prod", BF16), BF16).reshape(6, 40)
    assert np.allclose(gotb, axo.to_f32(xb, BF16).astype(np.float64).prod(1), rtol=1e-2)
    # any / all: the largest / smallest truth value along the axis, bytes in, bytes out
    t = (axo.PCG64(39).uniform((5, 17, 24)) > 0.1).astype(np.uint8)
    t[0, :, 3] = 0
    t[1, :, 5] = 1
    assert same(_reduce_axis(gh.to_dev(t), U8, 5, 17, 24, "max", U8).reshape(5, 24), t.any(1).astype(np.uint8))
    assert same(_reduce_axis(gh.to_dev(t), U8, 5, 17, 24, "min", U8).reshape(5, 24), t.all(1).astype(np.uint8))
    # float input, truth output
    f = t.astype(np.float32) * np.float32(-2.5)
    assert same(_reduce_axis(gh.to_dev(f), F32, 5, 17, 24, "min", U8).reshape(5, 24), (f.min(1) != 0).astype(np.uint8))


def _where(cond, a, b, a_dt, b_dt, out_dt, shape, cond_strides, a_strides, b_strides):
    dc, da, db = gh.to_dev(cond), gh.to_dev(a), gh.to_dev(b)
    out = gh.empty_dev(tuple(shape), out_dt)
    out.fill_(float("nan") if out_dt == F32 else 0xC1 if out_dt == U8 else 0x7FC1)
    gh.sync()
    capi.check(capi.lib().axhip_where(dc.data_ptr(), U8, da.data_ptr(), a_dt, db.data_ptr(), b_dt, out.data_ptr(), out_dt, len(shape), i64(list(shape)),
                                      i64(list(cond_strides)), i64(list(a_strides)), i64(list(b_strides)), None))
    gh.sync()
    return gh.to_host(out, gh.np_store_dtype(out_dt))


def elem_strides(shape, full):
    """element strides of a contiguous array of `shape` broadcast against `full` (0 on broadcast dims)."""
    st, run = [], 1
    for d in reversed(shape):
        st.append(0 if d == 1 else run)
        run *= d
    st = [0] * (len(full) - len(shape)) + st[::-1]
    return st


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_where_contiguous_broadcast_and_scalar_branches(dt):
    g = axo.PCG64(40)
    shape = (6, 10, 64)
    cond = (g.uniform(shape) > 0.5).astype(np.uint8) * 7  # any nonzero byte selects a
    af, bf = special(shape, 41), g.normal(shape)
    if dt != F32:
        af = np.nan_to_num(af, nan=0.5, posinf=np.inf, neginf=-np.inf)  # (NaN payloads of 16-bit types differ between converters)
    a, b = (af, bf) if dt == F32 else (axo.to_bits(af, dt), axo.to_bits(bf, dt))
    want = axo.where(cond, a, b, dt)
    full = elem_strides(shape, shape)
    assert same(_where(cond, a, b, dt, dt, dt, shape, full, full, full), want)
    # one broadcast element on either branch (where(mask, x, 0), where(mask, -inf, x))
    zero = np.zeros(1, a.dtype)
    assert same(_where(cond, a, zero, dt, dt, dt, shape, full, full, [0, 0, 0]), axo.where(cond, a, np.broadcast_to(zero, shape).copy(), dt))
    assert same(_where(cond, zero, b, dt, dt, dt, shape, full, [0, 0, 0], full), axo.where(cond, np.broadcast_to(zero, shape).copy(), b, dt))
    # a (10, 1) condition and a (64,) branch against the full shape
    c2 = (g.uniform((10, 1)) > 0.5).astype(np.uint8)
    row = a.reshape(-1)[:64].copy()
    got = _where(c2, row, b, dt, dt, dt, shape, elem_strides((10, 1), shape), elem_strides((64,), shape), full)
    assert same(got, axo.where(np.broadcast_to(c2, shape).copy(), np.broadcast_to(row, shape).copy(), b, dt))
    # a (10, 64) mask over the batch (attention scores under a [queries, keys] mask), one branch a scalar; the same with
    # the other branch a (6, 1, 1) column of per-batch values and an fp32 result
    c4 = (g.uniform((10, 64)) > 0.5).astype(np.uint8) * 3
    got = _where(c4, zero, b, dt, dt, dt, shape, elem_strides((10, 64), shape), [0, 0, 0], full)
    assert same(got, axo.where(np.broadcast_to(c4, shape).copy(), np.broadcast_to(zero, shape).copy(), b, dt))
    col = g.normal((6, 1, 1))
    got = _where(c4, a, col, dt, F32, F32, shape, elem_strides((10, 64), shape), full, elem_strides((6, 1, 1), shape))
    assert same(got, np.where(np.broadcast_to(c4, shape) != 0, a if dt == F32 else axo.to_f32(a, dt), np.broadcast_to(col, shape)))
    # rows of a wider array (pitch 64, 48 taken) and a truth-valued result
    s3 = (6, 10, 48)
    pitched = [640, 64, 1]
    c5 = (g.uniform(s3) > 0.5).astype(np.uint8)
    got = _where(c5, a, b, dt, dt, dt, s3, elem_strides(s3, s3), pitched, pitched)
    assert same(got, axo.where(c5, np.ascontiguousarray(a[..., :48]), np.ascontiguousarray(b[..., :48]), dt))
    bf32 = b if dt == F32 else axo.to_f32(b, dt)
    got = _where(c5, a, b, dt, dt, U8, s3, elem_strides(s3, s3), [0, 0, 0], pitched)
    a0 = (a if dt == F32 else axo.to_f32(a, dt)).reshape(-1)[0]
    assert same(got, np.where(c5 != 0, a0 != 0, bf32[..., :48] != 0).astype(np.uint8))
    # odd sizes (the element-wise kernel) and mixed branch types with an fp32 result
    s2 = (5, 37)
    c3 = (g.uniform(s2) > 0.3).astype(np.uint8)
    a3 = a.reshape(-1)[: 5 * 37].reshape(s2).copy()
    b3 = g.normal(s2)
    got = _where(c3, a3, b3, dt, F32, F32, s2, elem_strides(s2, s2), elem_strides(s2, s2), elem_strides(s2, s2))
    a3f = a3 if dt == F32 else axo.to_f32(a3, dt)
    assert same(got, np.where(c3 != 0, a3f, b3))


def test_where_reference_expectations():
    f = lambda *v: np.array(v, np.float32)
    st = [1]
    # tests/test_tensor_where.cpp:113-125, 160-175, 176-205
    assert _where(np.array([1, 0, 1, 0], np.uint8), np.ones(4, np.float32), np.zeros(4, np.float32), F32, F32, F32, (4,), st, st, st).tolist() == [1, 0, 1, 0]
    x = f(1, -2, 3, -4, 0)
    cond = gh.Rows(x.reshape(1, 5), F32, out_dt=U8).imm("gt", 0.0).run()[0]
    assert cond.tolist() == [1, 0, 1, 0, 0]
    assert _where(cond, x, np.zeros(5, np.float32), F32, F32, F32, (5,), st, st, st).tolist() == [1, 0, 3, 0, 0]
    assert _where(cond[:4], np.ones(4, np.float32), -np.ones(4, np.float32), F32, F32, F32, (4,), st, st, st).tolist() == [1, -1, 1, -1]
    scores = f(0.5, 0.3, 0.2, 0.1)
    mask = np.array([1, 0, 0, 1], np.uint8)  # attention-style masking: where(mask, -1e9, scores)
    assert same(_where(mask, np.full(4, -1e9, np.float32), scores, F32, F32, F32, (4,), st, st, st), f(-1e9, 0.3, 0.2, -1e9))


def _copy(src, sdt, ddt, shape, strides):
    d = gh.to_dev(src)
    out = gh.empty_dev(tuple(shape), ddt)
    gh.sync()
    capi.check(capi.lib().axhip_strided_copy(d.data_ptr(), sdt, out.data_ptr(), ddt, len(shape), i64(list(shape)), i64(list(strides)), None))
    gh.sync()
    return gh.to_host(out, gh.np_store_dtype(ddt))


def test_casts_to_and_from_truth_values():
    x = special((7, 24), 42)
    assert same(_copy(x, F32, U8, (7, 24), (24, 1)), (x != 0).astype(np.uint8))  # NaN is true, like static_cast<bool>
    xb = axo.to_bits(x, BF16)
    assert same(_copy(xb, BF16, U8, (7, 24), (24, 1)), (axo.to_f32(xb, BF16) != 0).astype(np.uint8))
    t = (np.arange(7 * 24).reshape(7, 24) % 3).astype(np.uint8)
    assert same(_copy(t, U8, F32, (7, 24), (24, 1)), (t != 0).astype(np.float32))
    assert same(axo.to_f32(_copy(t, U8, F16, (7, 24), (24, 1)), F16), (t != 0).astype(np.float32))
    assert same(_copy(t, U8, U8, (24, 7), (1, 24)), (t.T != 0).astype(np.uint8))  # a transposed view of bytes
    # the same casts inside a chain kernel: a program without arithmetic converts on load and on store
    assert same(gh.Rows(x, F32, out_dt=U8).imm("ne", 0.0).run(), (x != 0).astype(np.uint8))
    assert same(gh.Rows(t, U8, out_dt=F32).run(), (t != 0).astype(np.float32))


def test_bad_arguments_are_refused():
    l = capi.lib()
    x = gh.to_dev(np.zeros((4, 4), np.float32))
    p = gh.Rows(np.zeros((4, 4), np.float32), F32)
    p.p.pre[0].op, p.p.pre[0].operand, p.p.n_pre = 39, -1, 1  # between the two tables
    p.p.output, p.p.output_dtype = x.data_ptr(), F32
    assert l.axhip_fused_rows(C.byref(p.p), None) == capi.ERR_INVALID_ARG
    p.p.pre[0].op = 78  # past the unary table
    assert l.axhip_fused_rows(C.byref(p.p), None) == capi.ERR_INVALID_ARG
    p.p.pre[0].op = capi.OP["sin"]
    p.p.output_dtype = 4
    assert l.axhip_fused_rows(C.byref(p.p), None) == capi.ERR_INVALID_ARG
    st = i64([4, 1])
    assert l.axhip_where(x.data_ptr(), 5, x.data_ptr(), F32, x.data_ptr(), F32, x.data_ptr(), F32, 2, i64([4, 4]), st, st, st, None) == capi.ERR_INVALID_ARG
    assert l.axhip_where(None, U8, x.data_ptr(), F32, x.data_ptr(), F32, x.data_ptr(), F32, 2, i64([4, 4]), st, st, st, None) == capi.ERR_INVALID_ARG
    assert l.axhip_where(x.data_ptr(), U8, x.data_ptr(), F32, x.data_ptr(), F32, x.data_ptr(), F32, 2, i64([4, 4]), i64([-4, 1]), st, st, None) == capi.ERR_UNSUPPORTED
    # attention and GEMM keep to the floating-point types
    sp = capi.SdpaParams()
    sp.dtype, sp.batch, sp.heads, sp.seq_q, sp.seq_kv, sp.head_dim = U8, 1, 1, 4, 4, 8
    assert l.axhip_sdpa_fwd(x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), None, C.byref(sp), None) == capi.ERR_INVALID_ARG
    torch.cuda.synchronize()
