"""GPU parity of axhip_gemm (the nn::Linear / ops::matmul path) against float64
and against the CPU oracle's matmul."""
import math

import numpy as np
import pytest

from oracle import axo
from tests import gpu_harness as gh

pytestmark = pytest.mark.gpu
F32, F16, BF16 = axo.F32, axo.F16, axo.BF16


def test_linear_known_answers():
    # tests/test_nn_layers.cpp:12-73
    x, W = np.ones((1, 3), np.float32), np.ones((2, 3), np.float32)
    assert np.all(gh.gemm(x, W, F32, trans_b=True) == 3.0)
    assert np.all(gh.gemm(x, W, F32, trans_b=True, bias=np.ones(2, np.float32)) == 4.0)
    assert np.all(gh.gemm(np.ones((2, 4), np.float32), np.full((3, 4), 0.5, np.float32), F32, trans_b=True) == 2.0)
    assert np.all(gh.gemm(np.ones((5, 8), np.float32), np.ones((8, 8), np.float32), F32) == 8.0)


@pytest.mark.parametrize("M,N,K,ta,tb", [(7, 5, 9, False, False), (64, 64, 64, False, True), (70, 130, 300, True, False),
                                          (33, 129, 65, True, True), (1500, 1280, 1280, False, True)])
def test_f32_matches_oracle(M, N, K, ta, tb):
    g = axo.PCG64(M + N)
    A = g.normal((K, M) if ta else (M, K))
    B = g.normal((N, K) if tb else (K, N)) * (0.02 if K > 1000 else 1.0)
    got = gh.gemm(A, B, F32, ta, tb)[0]
    want = axo.matmul(A, B, F32, ta, tb)
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("M,N,K,extras,batch", [(1500, 1280, 1280, False, 1), (300, 250, 36, True, 1), (260, 257, 100, True, 1),
                                                (1500, 3840, 384, False, 1), (2000, 330, 240, True, 1), (256, 256, 32, False, 1),
                                                (200, 136, 520, True, 3)])
def test_f32_mfma_path_matches_fp64(M, N, K, extras, batch):
    """fp32 x W^T on the fp32 matrix instruction: ragged tiles, k extents that are not a multiple of the 32-float
    k-tile (36, 100, 240, 520), fewer k-tiles than ring stages, every tile shape, batches against a shared weight,
    and the bias / residual / GELU epilogue.  fp32 products and sums: held to the fp32 bar against float64."""
    import math

    g = axo.PCG64(M * 3 + K)
    x = g.normal((batch, M, K)).astype(np.float32)
    W = (g.normal((N, K)) / np.sqrt(K)).astype(np.float32)
    bias = (g.normal((N,)) * 0.1).astype(np.float32) if extras else None
    res = g.normal((batch, M, N)).astype(np.float32) if extras else None
    got = gh.gemm(x, W, F32, trans_b=True, bias=bias, residual=res, epilogue="gelu" if extras else None)
    want = x.astype(np.float64) @ W.astype(np.float64).T
    if extras:
        y = want + bias + res
        want = 0.5 * y * (1 + np.vectorize(math.erf)(y / math.sqrt(2)))
    assert got.shape == (batch, M, N)
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4), np.max(np.abs(got - want))


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("M,N,K", [(1, 3, 8), (128, 128, 64), (130, 70, 200), (1500, 1280, 1280)])
def test_half_linear_matches_fp32_reference(dt, M, N, K):
    g = axo.PCG64(K)
    x, W = axo.to_bits(g.normal((M, K)), dt), axo.to_bits(g.normal((N, K)) * 0.02, dt)
    bias = axo.to_bits(g.normal((N,)) * 0.1, dt)
    res = axo.to_bits(g.normal((M, N)), dt)
    got = axo.to_f32(gh.gemm(x, W, dt, trans_b=True, bias=bias, residual=res)[0], dt)
    xf, Wf = axo.to_f32(x, dt).astype(np.float64), axo.to_f32(W, dt).astype(np.float64)
    want = xf @ Wf.T + axo.to_f32(bias, dt) + axo.to_f32(res, dt)
    assert np.max(np.abs(got - want)) < 2e-2 + 2.0**-8 * np.max(np.abs(want))


def test_batched_shared_weight_and_gelu_epilogue():
    g = axo.PCG64(5)
    x, W = axo.to_bits(g.normal((3, 40, 64)), BF16), axo.to_bits(g.normal((48, 64)) * 0.1, BF16)
    got = axo.to_f32(gh.gemm(x, W, BF16, trans_b=True, epilogue="gelu"), BF16)
    y = axo.to_f32(x, BF16).astype(np.float64) @ axo.to_f32(W, BF16).astype(np.float64).T
    import math

    want = 0.5 * y * (1 + np.vectorize(math.erf)(y / math.sqrt(2)))
    assert np.max(np.abs(got - want)) < 2e-2


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("M,N,K,extras", [(2300, 3800, 192, True), (2304, 3840, 64, False), (4096, 2048, 320, False)])
def test_half_large_tile_path_matches_fp64(dt, M, N, K, extras):
    """Shapes that take the 256 x 256 work-group tiles, with ragged last tiles in both
    directions, a k extent of one and of several tiles, and the full epilogue."""
    g = axo.PCG64(M + K)
    x, W = axo.to_bits(g.normal((M, K)), dt), axo.to_bits(g.normal((N, K)) * 0.05, dt)
    bias = axo.to_bits(g.normal((N,)) * 0.1, dt) if extras else None
    res = axo.to_bits(g.normal((M, N)), dt) if extras else None
    got = axo.to_f32(gh.gemm(x, W, dt, trans_b=True, bias=bias, residual=res, epilogue="relu" if extras else None)[0], dt)
    want = axo.to_f32(x, dt).astype(np.float64) @ axo.to_f32(W, dt).astype(np.float64).T
    if extras:
        want = np.maximum(want + axo.to_f32(bias, dt) + axo.to_f32(res, dt), 0.0)
    assert np.max(np.abs(got - want)) < 2e-2 + 2.0**-8 * np.max(np.abs(want))
    # and the CPU oracle's matmul (accumulates in the 16-bit type as the reference's CPU path
    # does, cpu_operations.cpp:1840-1872) stays within its own, wider, band on a corner block
    if not extras and K <= 64:
        o = axo.to_f32(axo.matmul(x[:64], W[:64], dt, False, True), dt)
        assert np.max(np.abs(o - got[:64, :64])) < 0.25


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("M,N,K,epilogue,with_bias,with_res", [
    (2050, 3803, 128, "gelu", True, True),    # odd row pitch of C: two-byte stores everywhere
    (2049, 3802, 256, None, False, True),     # a last column group of two: masked tail beside 8-byte stores
    (2304, 3801, 64, "silu", True, False),    # one k-tile
    (2100, 2310, 448, "tanh", False, False),
    (4096, 2048, 512, "sigmoid", True, True)])
def test_half_large_tile_epilogues_and_column_tails(dt, M, N, K, epilogue, with_bias, with_res):
    """The 256 x 256 kernel's epilogue: a lane owns four consecutive columns of a row, stored as 8 bytes where the
    row pitch and the origin allow it and as masked 2-byte stores otherwise; every activation, with and without bias
    and residual, against float64."""
    g = axo.PCG64(3 * M + N + K)
    x, W = axo.to_bits(g.normal((M, K)), dt), axo.to_bits(g.normal((N, K)) * 0.05, dt)
    bias = axo.to_bits(g.normal((N,)) * 0.1, dt) if with_bias else None
    res = axo.to_bits(g.normal((M, N)), dt) if with_res else None
    got = axo.to_f32(gh.gemm(x, W, dt, trans_b=True, bias=bias, residual=res, epilogue=epilogue)[0], dt)
    want = axo.to_f32(x, dt).astype(np.float64) @ axo.to_f32(W, dt).astype(np.float64).T
    if with_bias:
        want = want + axo.to_f32(bias, dt)
    if with_res:
        want = want + axo.to_f32(res, dt)
    if epilogue == "gelu":
        from scipy.special import erf
        want = 0.5 * want * (1.0 + erf(want / np.sqrt(2.0)))
    elif epilogue == "silu":
        want = want / (1.0 + np.exp(-want))
    elif epilogue == "tanh":
        want = np.tanh(want)
    elif epilogue == "sigmoid":
        want = 1.0 / (1.0 + np.exp(-want))
    assert got.shape == want.shape
    assert np.max(np.abs(got - want)) < 2e-2 + 2.0**-8 * np.max(np.abs(want))


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("M,N,K,extras", [(1500, 5120, 1280, False), (1500, 1280, 5120, True), (200, 330, 256, True), (129, 257, 320, False),
                                          (1000, 2000, 448, True), (64, 128, 4096, False),
                                          (1500, 3840, 1280, False), (1500, 3700, 320, True)])
def test_half_ring_path_matches_fp64(dt, M, N, K, extras):
    """Mid-size products: the multi-stage LDS ring kernels (128 x 128, 64 x 128 and, for the last two shapes,
    128 x 192 tiles), with k extents of exactly, fewer and more k-tiles than the ring has stages, ragged tiles,
    and the full epilogue."""
    g = axo.PCG64(M * 7 + K)
    x, W = axo.to_bits(g.normal((M, K)), dt), axo.to_bits(g.normal((N, K)) * (2.0 / np.sqrt(K)), dt)
    bias = axo.to_bits(g.normal((N,)) * 0.1, dt) if extras else None
    res = axo.to_bits(g.normal((M, N)), dt) if extras else None
    got = axo.to_f32(gh.gemm(x, W, dt, trans_b=True, bias=bias, residual=res, epilogue="gelu" if extras else None)[0], dt)
    want = axo.to_f32(x, dt).astype(np.float64) @ axo.to_f32(W, dt).astype(np.float64).T
    if extras:
        import math

        y = want + axo.to_f32(bias, dt) + axo.to_f32(res, dt)
        want = 0.5 * y * (1 + np.vectorize(math.erf)(y / math.sqrt(2)))
    assert np.max(np.abs(got - want)) < 2e-2 + 2.0**-8 * np.max(np.abs(want))


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("ta,tb,K", [(False, False, 264), (True, False, 264), (True, True, 264), (False, True, 263), (True, False, 301)],
                         ids=["nn", "tn", "tt", "nt_k263", "tn_k301"])
def test_large_products_with_operands_not_along_k(dt, ta, tb, K):
    """Large products whose A is stored [k, m] and / or whose B is stored [k, n], or whose k is not a whole number of
    16-byte vectors: the library repacks such operands into temporary memory (transposed, k zero-padded) and runs the
    k-contiguous kernels; same bar as those.  Batched, with a shared B."""
    M, N, nb = 1040, 784, 3  # (above the size from which the library repacks)
    g = axo.PCG64(M + N + int(ta) + 2 * int(tb))
    A = axo.to_bits(g.normal((nb, K, M) if ta else (nb, M, K)), dt)
    B = axo.to_bits(g.normal((N, K) if tb else (K, N)) * 0.05, dt)
    bias = axo.to_bits(g.normal((N,)) * 0.1, dt)
    got = axo.to_f32(gh.gemm(A, B, dt, trans_a=ta, trans_b=tb, bias=bias, epilogue="relu"), dt)
    a64, b64 = axo.to_f32(A, dt).astype(np.float64), axo.to_f32(B, dt).astype(np.float64)
    want = np.maximum((a64.transpose(0, 2, 1) if ta else a64) @ (b64.T if tb else b64) + axo.to_f32(bias, dt), 0.0)
    tol = 1e-4 + 1e-4 * np.abs(want) if dt == F32 else 2e-2 + 2.0**-8 * np.abs(want)
    assert np.all(np.abs(got - want) <= tol)
    # per-batch B as well
    Bb = axo.to_bits(g.normal((nb, N, K) if tb else (nb, K, N)) * 0.05, dt)
    got = axo.to_f32(gh.gemm(A, Bb, dt, trans_a=ta, trans_b=tb), dt)
    bb64 = axo.to_f32(Bb, dt).astype(np.float64)
    want = (a64.transpose(0, 2, 1) if ta else a64) @ (bb64.transpose(0, 2, 1) if tb else bb64)
    tol = 1e-4 + 1e-4 * np.abs(want) if dt == F32 else 2e-2 + 2.0**-8 * np.abs(want)
    assert np.all(np.abs(got - want) <= tol)


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("M,N,K,extras", [(1, 1280, 1280, False), (1, 4096, 4096, True), (5, 100, 5120, True), (32, 1283, 264, False), (8, 51865, 384, False),
                                          (3, 2048, 4104, True), (1, 32, 256, False), (2, 4099, 776, True), (7, 16390, 520, False), (4, 1, 264, True)])
def test_skinny_products_of_a_decoding_step_match_fp64(dt, M, N, K, extras):
    """A few rows against a weight matrix (x W^T): up to 8 rows take the kernel that walks W's rows with whole
    wavefronts (1, 2 or 4 rows of W each, by N), ragged N and k tails, bias + residual + GELU; 32 rows stay on the
    tiled kernels; same bar for both."""
    g = axo.PCG64(M * 7 + N + K)
    x, W = axo.to_bits(g.normal((M, K)), dt), axo.to_bits(g.normal((N, K)) * 0.05, dt)
    bias = axo.to_bits(g.normal((N,)) * 0.1, dt) if extras else None
    res = axo.to_bits(g.normal((M, N)), dt) if extras else None
    got = axo.to_f32(gh.gemm(x, W, dt, trans_b=True, bias=bias, residual=res, epilogue="gelu" if extras else None)[0], dt)
    want = axo.to_f32(x, dt).astype(np.float64) @ axo.to_f32(W, dt).astype(np.float64).T
    if extras:
        want = want + axo.to_f32(bias, dt) + axo.to_f32(res, dt)
        want = 0.5 * want * (1.0 + np.vectorize(math.erf)(want / math.sqrt(2.0)))
    if dt == F32:
        assert np.max(np.abs(got - want)) < 1e-4 + 1e-5 * np.max(np.abs(want))
    else:
        assert np.max(np.abs(got - want)) < 2e-2 + 2.0**-8 * np.max(np.abs(want))


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_seeded_random_shapes_match_fp64(dt):
    """Forty seeded random products per dtype, shaped to land on every kernel and tile shape (matrix-core ring tiles,
    the 256 x 256 kernel, the register-staged and FMA fallbacks): ragged m and n, k with and without the alignment the
    matrix-core paths need, batches against a shared or a per-batch right operand, random epilogues."""
    import math

    r = np.random.default_rng(1234 + dt)
    erf = np.vectorize(math.erf)
    for case in range(40):
        big = case % 8 == 0
        M = int(r.integers(1, 2200 if big else 700))
        N = int(r.integers(1, 2200 if big else 700))
        K = int(r.choice([r.integers(1, 600), 8 * r.integers(1, 80), 64 * r.integers(1, 12)]))
        batch = int(r.choice([1, 1, 2, 3])) if not big else 1
        shared_w = bool(r.integers(0, 2))
        extras = bool(r.integers(0, 2))
        epi = [None, "relu", "gelu"][int(r.integers(0, 3))] if extras else None
        g = axo.PCG64(case * 7 + 1)
        x = g.normal((batch, M, K))
        W = g.normal((N, K) if shared_w else (batch, N, K)) / np.sqrt(K)
        bias = g.normal((N,)) * 0.1 if extras else None
        res = g.normal((batch, M, N)) if extras else None
        if dt == F32:
            xs, Ws = x.astype(np.float32), W.astype(np.float32)
            bs, rs = (bias.astype(np.float32), res.astype(np.float32)) if extras else (None, None)
            xf, Wf, bf, rf = xs, Ws, bs, rs
        else:
            xs, Ws = axo.to_bits(x, dt), axo.to_bits(W, dt)
            bs, rs = (axo.to_bits(bias, dt), axo.to_bits(res, dt)) if extras else (None, None)
            xf, Wf = axo.to_f32(xs, dt), axo.to_f32(Ws, dt)
            bf, rf = (axo.to_f32(bs, dt), axo.to_f32(rs, dt)) if extras else (None, None)
        got = gh.gemm(xs, Ws, dt, trans_b=True, bias=bs, residual=rs, epilogue=epi)
        got = got.astype(np.float64) if dt == F32 else axo.to_f32(got, dt).astype(np.float64)
        want = xf.astype(np.float64) @ np.swapaxes(Wf.astype(np.float64), -1, -2)
        if extras:
            want = want + bf + rf
            if epi == "relu":
                want = np.maximum(want, 0.0)
            elif epi == "gelu":
                want = 0.5 * want * (1 + erf(want / math.sqrt(2)))
        tol = 1e-4 * (1 + np.abs(want)) if dt == F32 else 2e-2 + 2.0**-8 * np.abs(want)
        assert got.shape == (batch, M, N)
        assert np.all(np.abs(got - want) <= tol), (case, M, N, K, batch, shared_w, epi, float(np.max(np.abs(got - want))))
