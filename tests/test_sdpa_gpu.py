"""GPU parity of axhip_sdpa_fwd against the CPU oracle (Axiom's tiled flash
attention restated) and the float64 textbook formula.  Shape cases follow the
reference's tests/test_flash_attention.cpp and tests/test_nn_attention.cpp.

Tolerances: fp32 1e-4 abs + 1e-4 rel; bf16 / f16 2e-2 abs against an fp32-or-better
evaluation of the SAME half-precision inputs."""
import math

import numpy as np
import pytest

from oracle import axo
from tests import gpu_harness as gh
from tests.test_oracle import SDPA_CASES, make_mask, naive_attention64

pytestmark = pytest.mark.gpu
F32, F16, BF16 = axo.F32, axo.F16, axo.BF16


def inputs(B, H, Sq, Skv, D, dt, seed=42):
    g = axo.PCG64(seed)
    return tuple(axo.to_bits(g.normal(s), dt) for s in ((B, H, Sq, D), (B, H, Skv, D), (B, H, Skv, D)))


@pytest.mark.parametrize("case", SDPA_CASES, ids=lambda c: "x".join(str(x) for x in c))
def test_f32_matches_cpu_oracle(case):
    B, H, Sq, Skv, D, scale, causal, mk = case
    q, k, v = inputs(B, H, Sq, Skv, D, F32)
    mask = make_mask(mk, Sq, Skv)
    sc = -1.0 if scale is None else scale
    got, kern = gh.sdpa(q, k, v, F32, sc, causal, mask)
    assert kern == (f"mfma_f32_d{D}" if D <= 128 and D % 4 == 0 else "generic")
    want = axo.sdpa(q, k, v, F32, sc, causal, mask)
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4), np.max(np.abs(got - want))


HALF_CASES = [  # (B,H,Sq,Skv,D, causal, mask)
    (1, 2, 16, 16, 64, False, None),       # tests/test_flash_attention.cpp:233-249 (Float16 GPU case)
    (1, 2, 8, 8, 32, False, None), (1, 2, 8, 8, 128, False, None), (1, 2, 16, 32, 32, False, None),
    (1, 2, 16, 16, 32, True, None), (1, 1, 8, 8, 32, False, "mod3"), (1, 1, 37, 37, 32, False, None),
    (1, 1, 256, 256, 64, False, None), (4, 8, 16, 16, 32, False, None), (1, 1, 1, 1, 32, False, None),
    (2, 3, 130, 70, 64, True, None), (2, 3, 70, 130, 64, True, None), (1, 2, 300, 300, 128, True, None),
    (1, 3, 257, 511, 128, False, "mod3"), (1, 20, 1500, 1500, 64, False, None),  # Whisper encoder shape
    (2, 8, 1024, 1024, 128, True, None), (1, 1, 8, 8, 48, False, None), (1, 1, 64, 64, 96, True, None),
    # head_dim 64 with enough (batch, head, block) units for the 8-wave work-groups: causal pairs, ragged blocks, a mask
    (2, 64, 600, 600, 64, True, None), (1, 128, 300, 520, 64, False, "mod3"),
    # head_dim 256 (16-bit: the register-staged matrix-core kernel with its tiles in dynamic LDS)
    (1, 2, 8, 8, 256, False, None), (2, 3, 130, 200, 256, True, None), (1, 2, 300, 300, 256, False, "mod3"), (1, 4, 257, 129, 256, False, "mod3"), (1, 2, 200, 333, 256, True, None),
    # head sizes between 128 and 256 on the head_dim-256 kernel, zeros in the missing dims
    (1, 2, 130, 130, 192, True, None), (2, 2, 100, 257, 136, False, "mod3"), (1, 3, 64, 64, 248, False, None)]


@pytest.mark.parametrize("case", HALF_CASES, ids=lambda c: "x".join(str(x) for x in c))
def test_f32_on_the_larger_shapes(case):
    """fp32 through the fp32-MFMA kernel (head_dim 32 / 64 / 128; 48 and 96 take the FMA kernel) on the multi-tile,
    ragged, causal, cross-attention and masked shapes, held to the fp32 bar."""
    B, H, Sq, Skv, D, causal, mk = case
    q, k, v = inputs(B, H, Sq, Skv, D, F32, seed=11)
    mask = make_mask(mk, Sq, Skv)
    got, kern = gh.sdpa(q, k, v, F32, -1.0, causal, mask)
    assert kern == (f"mfma_f32_d{D}" if D <= 128 and D % 4 == 0 else "generic")
    if B * H * Sq * Skv <= 1 << 24:
        want = naive_attention64(q, k, v, 1 / math.sqrt(D), causal, mask)
    else:
        want = axo.sdpa(q, k, v, F32, -1.0, causal, mask)
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4), np.max(np.abs(got - want))


@pytest.mark.parametrize("split", ["1", "2", "4"])
def test_f32_with_each_key_split_forced(split):
    """The fp32 kernel lets 1, 2 or 4 waves share a query block and merges their partial softmax states; the library
    picks by problem size.  Here every mode runs every fp32 shape: the choice is an environment setting read when
    the library loads, so each mode gets a process of its own."""
    import os
    import subprocess
    import sys

    if os.environ.get("AXHIP_SDPA_F32_SPLIT"):
        pytest.skip("already inside a forced-split run")
    env = dict(os.environ, AXHIP_SDPA_F32_SPLIT=split)
    r = subprocess.run([sys.executable, "-m", "pytest", "-x", "-q", "-p", "no:cacheprovider", __file__, "-k",
                        "test_f32_on_the_larger_shapes or test_f32_matches_cpu_oracle or test_fully_masked"],
                       env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:]


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", HALF_CASES, ids=lambda c: "x".join(str(x) for x in c))
def test_half_matches_fp32_reference_of_same_inputs(case, dt):
    B, H, Sq, Skv, D, causal, mk = case
    q, k, v = inputs(B, H, Sq, Skv, D, dt, seed=7)
    mask = make_mask(mk, Sq, Skv)
    got, kern = gh.sdpa(q, k, v, dt, -1.0, causal, mask)
    assert kern == f"mfma_{'bf16' if dt == BF16 else 'f16'}_d{D}"  # (48 and 96: on the 64 and 128 kernels, zeros in the missing dims)
    qf, kf, vf = (axo.to_f32(t, dt) for t in (q, k, v))
    if B * H * Sq * Skv <= 1 << 24:
        want = naive_attention64(qf, kf, vf, 1 / math.sqrt(D), causal, mask)
    else:  # large cases: the CPU oracle's fp32 tiled algorithm on the widened inputs
        want = axo.sdpa(qf, kf, vf, F32, -1.0, causal, mask)
    gotf = axo.to_f32(got, dt)
    assert np.isfinite(gotf).all()
    err = np.max(np.abs(gotf - want))
    assert err < 2e-2, err
    # and the distance to the literal CPU path (half output of the tiled algorithm)
    lit = axo.to_f32(axo.sdpa(q, k, v, dt, -1.0, causal, mask), dt)
    assert np.max(np.abs(gotf - lit)) < 4e-2


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
def test_small_head_dim_64_problems_split_their_keys_between_the_halves_of_a_work_group(dt):
    """Unmasked head_dim-64 problems with 128-row work-groups for at most half of the compute units run with
    work-groups of 64 query rows whose two halves take half of the key tiles each and merge their softmax states at
    the end.  Key counts around the tile size (two tiles with one key in the second, an odd number of tiles, a ragged
    last tile), a single query row, cross attention, and the Whisper shape (which stays unsplit: 240 work-groups);
    against float64, and with V = 1 (every output is then the merged normalisation itself: exactly 1)."""
    for B, H, Sq, Skv in ((2, 3, 64, 65), (1, 2, 1, 1000), (1, 4, 200, 130), (1, 1, 70, 128), (2, 2, 130, 129), (1, 3, 300, 77),
                          (1, 5, 33, 192), (1, 20, 1500, 1500)):
        q, k, v = inputs(B, H, Sq, Skv, 64, dt, seed=100 + Skv)
        got, kern = gh.sdpa(q, k, v, dt, -1.0, False, None)
        assert kern == f"mfma_{'bf16' if dt == BF16 else 'f16'}_d64"
        qf, kf, vf = (axo.to_f32(t, dt) for t in (q, k, v))
        if B * H * Sq * Skv <= 1 << 24:
            want = naive_attention64(qf, kf, vf, 0.125, False, None)
        else:
            want = axo.sdpa(qf, kf, vf, F32, -1.0, False, None)
        err = np.max(np.abs(axo.to_f32(got, dt) - want))
        assert err < 2e-2, (B, H, Sq, Skv, err)
        ones = axo.to_bits(np.ones(v.shape, np.float32), dt)
        got, _ = gh.sdpa(q, k, ones, dt, -1.0, False, None)
        assert np.max(np.abs(axo.to_f32(got, dt) - 1.0)) <= (2.0 ** -8 if dt == BF16 else 2.0 ** -10), (B, H, Sq, Skv)


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
def test_head_sizes_between_the_compiled_ones(dt):
    """Multiples of 8 between 32 and 128 run on the next compiled head size: Q fragments beyond the head size stay
    zero, the K/V chunks beyond it are loaded as zeros, the output keeps its own width (guard values behind every
    output row: the rows sit in a wider buffer).  Self and cross attention, causal, a mask, the 8- and 4-wave and the
    key-split work-groups, packed (batch, seq, heads*dim) strides."""
    tag = "bf16" if dt == BF16 else "f16"
    for D, (B, H, Sq, Skv), causal, mk in ((40, (1, 2, 70, 70), False, None), (48, (2, 3, 130, 70), True, None), (56, (1, 4, 64, 200), False, "mod3"),
                                           (72, (1, 2, 100, 100), True, None), (80, (2, 2, 257, 300), False, None), (96, (1, 3, 300, 300), True, "mod3"),
                                           (104, (1, 1, 33, 129), False, None), (120, (1, 2, 64, 64), False, None), (96, (2, 70, 520, 520), True, None),
                                           (80, (1, 130, 600, 600), False, None)):
        q, k, v = inputs(B, H, Sq, Skv, D, dt, seed=300 + D)
        mask = make_mask(mk, Sq, Skv)
        got, kern = gh.sdpa(q, k, v, dt, -1.0, causal, mask)
        assert kern == f"mfma_{tag}_d{D}", kern
        qf, kf, vf = (axo.to_f32(t, dt) for t in (q, k, v))
        if B * H * Sq * Skv <= 1 << 24:
            want = naive_attention64(qf, kf, vf, 1 / math.sqrt(D), causal, mask)
        else:
            want = axo.sdpa(qf, kf, vf, F32, -1.0, causal, mask)
        err = np.max(np.abs(axo.to_f32(got, dt) - want))
        assert err < 2e-2, (D, B, H, Sq, Skv, err)
    # rows of 80 inside rows of 128: what lies behind a row's 80 values must survive
    B, S, H, D, W = 1, 150, 3, 80, 128
    g = axo.PCG64(17)
    packed = [axo.to_bits(g.normal((B, S, H, W)), dt) for _ in range(3)]
    st = (S * H * W, W, H * W)
    out_init = axo.to_bits(np.full((B, S, H, W), 7.0, np.float32), dt)
    got, kern = gh.sdpa(*packed, dt, -1.0, False, None, q_strides=st, k_strides=st, v_strides=st, o_strides=st, shape=(B, H, S, S, D), out_init=out_init)
    assert kern == f"mfma_{tag}_d80"
    gf = axo.to_f32(got, dt).reshape(B, S, H, W)
    assert np.all(gf[..., D:] == 7.0)
    qf, kf, vf = (axo.to_f32(t, dt)[..., :D].transpose(0, 2, 1, 3) for t in packed)
    want = naive_attention64(qf, kf, vf, 1 / math.sqrt(D), False)
    assert np.max(np.abs(gf[..., :D].transpose(0, 2, 1, 3) - want)) < 2e-2
    # and rows of 192 inside rows of 256 (the head_dim-256 kernel)
    B, S, H, D, W = 1, 90, 2, 192, 256
    packed = [axo.to_bits(g.normal((B, S, H, W)), dt) for _ in range(3)]
    st = (S * H * W, W, H * W)
    out_init = axo.to_bits(np.full((B, S, H, W), 7.0, np.float32), dt)
    got, kern = gh.sdpa(*packed, dt, -1.0, True, None, q_strides=st, k_strides=st, v_strides=st, o_strides=st, shape=(B, H, S, S, D), out_init=out_init)
    assert kern == f"mfma_{tag}_d192"
    gf = axo.to_f32(got, dt).reshape(B, S, H, W)
    assert np.all(gf[..., D:] == 7.0)
    qf, kf, vf = (axo.to_f32(t, dt)[..., :D].transpose(0, 2, 1, 3) for t in packed)
    want = naive_attention64(qf, kf, vf, 1 / math.sqrt(D), True)
    assert np.max(np.abs(gf[..., :D].transpose(0, 2, 1, 3) - want)) < 2e-2


def test_fp32_multiples_of_four_and_small_16_bit_head_sizes_run_on_the_matrix_cores():
    """fp32 head sizes that are multiples of 4 (4 .. 124) run on the fp32 matrix-core kernel of the next of 32 / 64 / 128,
    16-bit head sizes 8 / 16 / 24 on the head_dim-32 kernel: zeros in the missing dims, the output keeps its width
    (guard values behind every row of a wider buffer), every key split of the fp32 kernel, causal and masked."""
    for D, (B, H, Sq, Skv), causal, mk in ((4, (1, 2, 70, 70), False, None), (20, (2, 3, 130, 70), True, None), (36, (1, 4, 64, 200), False, "mod3"),
                                           (100, (1, 2, 100, 100), True, None), (124, (2, 2, 257, 300), False, None), (52, (1, 40, 300, 300), True, None)):
        q, k, v = inputs(B, H, Sq, Skv, D, F32, seed=500 + D)
        mask = make_mask(mk, Sq, Skv)
        got, kern = gh.sdpa(q, k, v, F32, -1.0, causal, mask)
        assert kern == f"mfma_f32_d{D}", kern
        want = naive_attention64(q, k, v, 1 / math.sqrt(D), causal, mask)
        assert np.max(np.abs(got - want)) < 1e-4, D
    for dt, tag in ((BF16, "bf16"), (F16, "f16")):
        for D in (8, 16, 24):
            q, k, v = inputs(2, 3, 90, 150, D, dt, seed=600 + D)
            got, kern = gh.sdpa(q, k, v, dt, -1.0, D == 16, None)
            assert kern == f"mfma_{tag}_d{D}", kern
            want = naive_attention64(*(axo.to_f32(t, dt) for t in (q, k, v)), 1 / math.sqrt(D), D == 16, None)
            assert np.max(np.abs(axo.to_f32(got, dt) - want)) < 2e-2, (tag, D)
    # fp32 rows of 40 inside rows of 64: what lies behind a row's 40 values must survive
    B, S, H, D, W = 1, 150, 3, 40, 64
    g = axo.PCG64(18)
    packed = [g.normal((B, S, H, W)).astype(np.float32) for _ in range(3)]
    st = (S * H * W, W, H * W)
    out_init = np.full((B, S, H, W), 7.0, np.float32)
    got, kern = gh.sdpa(*packed, F32, -1.0, False, None, q_strides=st, k_strides=st, v_strides=st, o_strides=st, shape=(B, H, S, S, D), out_init=out_init)
    assert kern == "mfma_f32_d40"
    gf = got.reshape(B, S, H, W)
    assert np.all(gf[..., D:] == 7.0)
    qf, kf, vf = (t[..., :D].transpose(0, 2, 1, 3) for t in packed)
    assert np.max(np.abs(gf[..., :D].transpose(0, 2, 1, 3) - naive_attention64(qf, kf, vf, 1 / math.sqrt(D), False))) < 1e-4


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
def test_decoding_steps_split_their_keys_between_work_groups(dt):
    """Few query rows, few (batch, head) slices, a long key sequence: the keys are split between work-groups and the
    partial results merged (head sizes 64, 128 and in between, ragged last chunks, one to 128 query rows, a key
    sequence with one dominant key in the last chunk); against float64."""
    tag = "bf16" if dt == BF16 else "f16"
    for B, H, Sq, Skv, D in ((1, 8, 1, 8192, 128), (2, 8, 5, 9001, 64), (1, 30, 128, 3030, 96), (1, 32, 1, 4096, 128), (1, 64, 33, 3072, 48), (3, 32, 2, 1500, 64),
                               # up to 384 (batch, head) slices are split (enough work-groups for four per CU)
                               (4, 32, 1, 2100, 128), (2, 160, 3, 1100, 64)):
        q, k, v = inputs(B, H, Sq, Skv, D, dt, seed=700 + Sq + D)
        kf = axo.to_f32(k, dt)
        kf[..., Skv - 3, :] = 4.0 * axo.to_f32(q, dt)[..., 0, :]  # a key far above the rest, in the last chunk
        k = axo.to_bits(kf, dt)
        got, kern = gh.sdpa(q, k, v, dt, -1.0, False, None)
        assert kern == f"mfma_{tag}_d{D}"
        want = naive_attention64(*(axo.to_f32(t, dt) for t in (q, k, v)), 1 / math.sqrt(D), False, None)
        err = np.max(np.abs(axo.to_f32(got, dt) - want))
        assert err < 2e-2, (B, H, Sq, Skv, D, float(err))


def test_fully_masked_rows_give_zeros_everywhere_else_matches():
    q, k, v = inputs(1, 2, 70, 70, 64, BF16, seed=3)
    m = np.zeros((70, 70), np.uint8)
    m[5, :] = 1
    m[9, :64] = 1  # first 64-key tile fully masked, the tail visible
    for dt, (qq, kk, vv) in ((BF16, (q, k, v)), (F32, tuple(axo.to_f32(t, BF16) for t in (q, k, v)))):
        got, _ = gh.sdpa(qq, kk, vv, dt, -1.0, False, m)
        gf = axo.to_f32(got, dt)
        assert np.all(gf[:, :, 5, :] == 0.0)
        want = naive_attention64(*(axo.to_f32(t, dt) for t in (qq, kk, vv)), 0.125, False, m)
        assert np.max(np.abs(gf - want)) < (2e-2 if dt == BF16 else 1e-4)


@pytest.mark.parametrize("dt,S", [(BF16, 96), (BF16, 256), (F32, 96), (F32, 256), (F16, 192)], ids=["bf16-96", "bf16-256", "f32-96", "f32-256", "f16-192"])
def test_per_batch_head_mask_and_broadcast_masks(dt, S):
    """Random masks of every supported shape; S = 96 ends in a ragged tile (mask bytes read one by one), the other
    lengths are whole tiles with 4-byte aligned rows (mask words applied through the accumulators' initial value)."""
    B, H, D = 2, 3, 64
    q, k, v = inputs(B, H, S, S, D, dt, seed=5)
    r = np.random.default_rng(0)
    for shape in ((B, H, S, S), (1, 1, S, S), (B, 1, S, S), (1, H, S, S)):
        m = (r.random(shape) < 0.3).astype(np.uint8) * r.choice(np.array([1, 2, 128, 255], np.uint8), shape)  # any nonzero byte masks
        m[..., 0] = 0
        got, _ = gh.sdpa(q, k, v, dt, -1.0, False, m)
        want = naive_attention64(*(axo.to_f32(t, dt) for t in (q, k, v)), 0.125, False, m)
        assert np.max(np.abs(axo.to_f32(got, dt) - want)) < (1e-4 if dt == F32 else 2e-2)


def test_head_split_view_strides_need_no_copy():
    # nn::MultiHeadAttention hands (B,S,H*D) projections viewed as (B,H,S,D): strides (S*H*D, D, H*D)
    B, S, H, D = 2, 200, 4, 64
    g = axo.PCG64(9)
    packed = [axo.to_bits(g.normal((B, S, H, D)), BF16) for _ in range(3)]
    st = (S * H * D, D, H * D)
    got, kern = gh.sdpa(*packed, BF16, -1.0, True, None, q_strides=st, k_strides=st, v_strides=st, shape=(B, H, S, S, D))
    assert kern == "mfma_bf16_d64"
    qf, kf, vf = (axo.to_f32(t, BF16).transpose(0, 2, 1, 3) for t in packed)
    want = naive_attention64(qf, kf, vf, 0.125, True)
    assert np.max(np.abs(axo.to_f32(got, BF16) - want)) < 2e-2


def test_scale_parameter_and_auto_scale():
    q, k, v = inputs(1, 1, 64, 64, 64, BF16, seed=1)
    f = [axo.to_f32(t, BF16) for t in (q, k, v)]
    a, _ = gh.sdpa(q, k, v, BF16, 0.5)
    assert np.max(np.abs(axo.to_f32(a, BF16) - naive_attention64(*f, 0.5))) < 2e-2
    b, _ = gh.sdpa(q, k, v, BF16, -1.0)
    c, _ = gh.sdpa(q, k, v, BF16, 0.125)
    assert np.array_equal(b, c)  # scale <= 0 -> 1/sqrt(D)


def test_uniform_input_gives_ones():
    ones = axo.to_bits(np.ones((1, 1, 4, 32), np.float32), BF16)
    got, _ = gh.sdpa(ones, ones, ones, BF16, -1.0, True)
    assert np.allclose(axo.to_f32(got, BF16), 1.0, atol=1e-2)


def test_full_size_causal_bf16_properties():
    """B4 H32 S4096 D128 causal bf16: size-independent checks on the whole tensor plus the
    oracle on a deterministic subset of (batch, head) slices."""
    B, H, S, D = 4, 32, 4096, 128
    g = axo.PCG64(42)
    q, k, v = (axo.to_bits(g.normal((B, H, S, D)), BF16) for _ in range(3))
    got, kern = gh.sdpa(q, k, v, BF16, -1.0, True)
    assert kern == "mfma_bf16_d128"
    from axiom_amd import capi

    assert capi.lib().axhip_sdpa_last_schedule() == b"pingpong"
    gf = axo.to_f32(got, BF16)
    assert np.isfinite(gf).all()
    vf = axo.to_f32(v, BF16)
    # causal row 0 attends to key 0 only: O[...,0,:] == V[...,0,:] exactly
    assert np.array_equal(gf[:, :, 0, :], vf[:, :, 0, :])
    # every output is a convex combination of the visible values
    run_max = np.maximum.accumulate(vf, axis=2)
    run_min = np.minimum.accumulate(vf, axis=2)
    assert np.all(gf <= run_max + 2e-2) and np.all(gf >= run_min - 2e-2)
    # oracle on slices 0, 37, 127 (fp32 tiled algorithm on the widened bf16 inputs)
    for sl in (0, 37, 127):
        b, h = divmod(sl, H)
        qs, ks, vs = (axo.to_f32(t[b:b + 1, h:h + 1], BF16) for t in (q, k, v))
        want = axo.sdpa(qs, ks, vs, F32, -1.0, True)
        err = np.max(np.abs(gf[b:b + 1, h:h + 1] - want))
        assert err < 2e-2, (sl, err)


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
def test_head_dim_256_seeded_random_problems_match_fp64(dt):
    """Twelve seeded random head_dim-256 problems per 16-bit type (ragged lengths, causal, shared and per-(batch, head)
    masks of either alignment, explicit scales) on the matrix-core kernel, against float64."""
    r = np.random.default_rng(256 + dt)
    for case in range(12):
        B, H = int(r.integers(1, 3)), int(r.integers(1, 5))
        Sq = int(r.integers(1, 400))
        Skv = Sq if r.integers(0, 2) else int(r.integers(1, 400))
        if r.integers(0, 3) == 0:
            Skv = 4 * max(1, Skv // 4)
        causal = bool(r.integers(0, 2))
        mkind = int(r.integers(0, 3))
        scale = float(r.choice([-1.0, 2.0 / math.sqrt(256), 0.03]))
        q, k, v = inputs(B, H, Sq, Skv, 256, dt, seed=300 + case)
        mask = None
        if mkind:
            shape = (Sq, Skv) if mkind == 1 else (B, H, Sq, Skv)
            mask = (r.random(shape) < 0.25).astype(np.uint8) * r.choice(np.array([1, 7, 255], np.uint8), shape)
        got, kern = gh.sdpa(q, k, v, dt, scale, causal, mask)
        assert kern == f"mfma_{'bf16' if dt == BF16 else 'f16'}_d256"
        sc = 1 / math.sqrt(256) if scale < 0 else scale
        want = naive_attention64(*(axo.to_f32(t, dt) for t in (q, k, v)), sc, causal, mask)
        err = np.max(np.abs(axo.to_f32(got, dt).astype(np.float64) - want))
        assert err < 2e-2, (case, B, H, Sq, Skv, causal, mkind, scale, float(err))


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
def test_seeded_random_problems_match_fp64(dt):
    """Thirty seeded random problems per dtype: head sizes on and off the matrix-core kernels, self and cross
    attention with ragged lengths, causal, shared and per-(batch, head) masks with rows of either alignment, explicit
    scales; each against the float64 textbook evaluation of the same inputs."""
    r = np.random.default_rng(77 + dt)
    for case in range(30):
        D = int(r.choice([32, 64, 128, 64, 128, 48]))
        B, H = int(r.integers(1, 4)), int(r.integers(1, 6))
        Sq = int(r.integers(1, 420))
        Skv = Sq if r.integers(0, 2) else int(r.integers(1, 420))
        if r.integers(0, 3) == 0:
            Skv = 4 * max(1, Skv // 4)  # 4-byte aligned mask rows
        causal = bool(r.integers(0, 2))
        mkind = int(r.integers(0, 3))  # none, shared, per (batch, head)
        # explicit scales up to twice the default: the 16-bit kernels fold the scale into Q (one more 16-bit rounding of
        # the logits' inputs), so the 2e-2 bar is stated for logits of ordinary size, as in the reference's own cases
        scale = float(r.choice([-1.0, 2.0 / math.sqrt(D), 0.05]))
        q, k, v = inputs(B, H, Sq, Skv, D, dt, seed=100 + case)
        mask = None
        if mkind:
            shape = (Sq, Skv) if mkind == 1 else (B, H, Sq, Skv)
            mask = (r.random(shape) < 0.25).astype(np.uint8) * r.choice(np.array([1, 7, 255], np.uint8), shape)
        got, _ = gh.sdpa(q, k, v, dt, scale, causal, mask)
        sc = 1 / math.sqrt(D) if scale < 0 else scale
        want = naive_attention64(*(axo.to_f32(t, dt) for t in (q, k, v)), sc, causal, mask)
        err = np.max(np.abs(axo.to_f32(got, dt).astype(np.float64) - want))
        assert err < (1e-4 if dt == F32 else 2e-2), (case, B, H, Sq, Skv, D, causal, mkind, scale, float(err))


# (B, H, Sq, Skv, causal): unmasked head_dim-128 problems with a 256-row work-group for every CU -- the ping-pong
# schedule with persistent work-groups.  Ragged query blocks and key tails, one and two passes per causal pair, even
# and odd tile counts (only an even count requests the next segment's first tiles ahead), more units than
# work-groups, a (batch, head) count that 8 does not divide, cross attention.
PINGPONG_CASES = [
    (8, 32, 256, 256, False), (8, 32, 256, 256, True), (8, 32, 300, 333, False), (4, 32, 1000, 1000, True),
    (8, 32, 700, 150, False), (8, 32, 260, 64, False), (8, 32, 257, 70, True), (4, 65, 256, 192, False),
    (2, 64, 1030, 1030, True), (8, 32, 512, 1000, True), (16, 32, 129, 640, False),
]


@pytest.mark.parametrize("dt", [BF16, F16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", PINGPONG_CASES, ids=lambda c: "x".join(str(int(x)) for x in c))
def test_chip_filling_head_dim_128_problems_on_the_ping_pong_schedule(case, dt):
    from axiom_amd import capi

    B, H, Sq, Skv, causal = case
    D = 128
    q, k, v = inputs(B, H, Sq, Skv, D, dt, seed=11)
    got, kern = gh.sdpa(q, k, v, dt, -1.0, causal)
    assert kern == f"mfma_{'bf16' if dt == BF16 else 'f16'}_d128"
    assert capi.lib().axhip_sdpa_last_schedule() == b"pingpong"
    gotf = axo.to_f32(got, dt)
    assert np.isfinite(gotf).all()
    # float64 textbook attention on slices spread over the units: first, last, and every 19th in between
    slices = sorted(set([0, B * H - 1] + list(range(3, B * H, 19))))
    for sl in slices:
        b, h = divmod(sl, H)
        qs, ks, vs = (axo.to_f32(t[b:b + 1, h:h + 1], dt) for t in (q, k, v))
        want = naive_attention64(qs, ks, vs, 1 / math.sqrt(D), causal, None)
        err = np.max(np.abs(gotf[b:b + 1, h:h + 1] - want))
        assert err < 2e-2, (sl, err)


def test_ping_pong_schedule_on_head_split_views_and_a_row_dominated_by_a_late_key():
    """Strided (B,S,H,D) -> (B,H,S,D) views as nn::MultiHeadAttention hands them over, and a key far down the
    sequence whose logit dwarfs the running maximum (the accumulators are rescaled late)."""
    from axiom_amd import capi

    B, H, S, D = 4, 64, 512, 128
    g = axo.PCG64(5)
    raw = [g.normal((B, S, H, D)) for _ in range(3)]
    raw[1][:, 450, :, :] *= 6.0  # one key with large logits for many queries
    raw[2] *= 0.5  # (outputs stay below 2: a bf16 step of 2^-7, well inside the 2e-2 bar)
    q, k, v = (axo.to_bits(t, BF16) for t in raw)
    st = (S * H * D, D, H * D)
    got, _ = gh.sdpa(q, k, v, BF16, -1.0, False, None, q_strides=st, k_strides=st, v_strides=st, shape=(B, H, S, S, D))
    assert capi.lib().axhip_sdpa_last_schedule() == b"pingpong"
    gotf = axo.to_f32(got, BF16)
    for b, h in ((0, 0), (1, 17), (3, 63)):
        qs, ks, vs = (axo.to_f32(t[b:b + 1, :, h:h + 1], BF16).transpose(0, 2, 1, 3) for t in (q, k, v))
        want = naive_attention64(qs, ks, vs, 1 / math.sqrt(D), False, None)
        err = np.max(np.abs(gotf[b:b + 1, h:h + 1] - want))
        assert err < 2e-2, ((b, h), err)
