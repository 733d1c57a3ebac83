"""GPU parity of the data movers behind gpu_make_contiguous / Cast / Pad / MaskedFill /
Embedding: pure data movement, so every comparison is bit-exact against numpy."""
import ctypes as C

import numpy as np
import pytest
import torch

from axiom_amd import capi
from oracle import axo
from tests import gpu_harness as gh

pytestmark = pytest.mark.gpu
F32, F16, BF16 = axo.F32, axo.F16, axo.BF16


def i64(values):
    return (C.c_int64 * len(values))(*[int(v) for v in values])


def sample(shape, dt, seed):
    x = axo.PCG64(seed).normal(shape)
    return x if dt == F32 else axo.to_bits(x, dt)


def elem_strides(a):
    return [s // a.itemsize for s in a.strides]


@pytest.mark.parametrize("dt", [F32, F16, BF16], ids=["f32", "f16", "bf16"])
def test_strided_copy_of_transposed_and_broadcast_views(dt):
    base = sample((6, 5, 7), dt, 3)
    d = gh.to_dev(base)
    for view in (base.transpose(2, 0, 1), base[:, ::2, 1:6], np.broadcast_to(base[:, :1, :], (6, 4, 7))):
        out = gh.empty_dev(view.shape, dt)
        off = (view.__array_interface__["data"][0] - base.__array_interface__["data"][0])
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(d.data_ptr() + off, dt, out.data_ptr(), dt, view.ndim, i64(view.shape), i64(elem_strides(view)), None))
        gh.sync()
        assert np.array_equal(gh.to_host(out, base.dtype), np.ascontiguousarray(view))


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
def test_strided_copy_fast_paths_are_bit_exact(dt):
    """Views big enough for the 16-byte path (innermost dimension contiguous: head splits, row and column slices,
    broadcast rows) and for the tiled transpose (innermost dimension strided, another one contiguous), ragged
    against the 64 x 64 tile and with further dimensions around the transposed pair."""
    base = sample((3, 40, 70, 48), dt, 5)
    d = gh.to_dev(base)
    views = [base.transpose(0, 2, 1, 3), base[:, 3:35, ::2, 8:40], np.broadcast_to(base[:, :1], base.shape),  # vector path
             base.transpose(0, 1, 3, 2), base.transpose(3, 2, 1, 0), base.transpose(1, 3, 0, 2), base.transpose(2, 0, 3, 1),
             base[1].transpose(2, 1, 0), base[0, 5].T, base[:, :, 1:66, 3:41].transpose(0, 3, 2, 1)]
    for view in views:
        out = gh.empty_dev(view.shape, dt)
        off = (view.__array_interface__["data"][0] - base.__array_interface__["data"][0])
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(d.data_ptr() + off, dt, out.data_ptr(), dt, view.ndim, i64(view.shape), i64(elem_strides(view)), None))
        gh.sync()
        assert np.array_equal(gh.to_host(out, base.dtype), np.ascontiguousarray(view)), view.shape


@pytest.mark.parametrize("dt", [F32, F16, BF16], ids=["f32", "f16", "bf16"])
def test_transposes_in_vector_tiles_are_bit_exact(dt):
    """Transposed views whose two sides move whole 16-byte vectors, or 8-byte pieces (rows of 1500 16-bit elements): tiles
    of 16 x 16 vectors through LDS.  Several tiles each way with ragged last tiles, extents that are multiples of a
    vector on one side and of half a vector on the other, further dimensions before, between and behind the
    transposed pair, a view at an offset inside its array, and extents that fall back to the element-wise tiles."""
    vec = 4 if dt == F32 else 8
    cases = [((300, 264), (1, 0)), ((3, 136, 200), (0, 2, 1)), ((2, 3, 72, 40 * vec), (0, 1, 3, 2)), ((2, 24 * vec, 5, 136), (0, 3, 2, 1)),
             ((130, vec * 33 + vec // 2), (1, 0)), ((vec * 17 + vec // 2, 520), (1, 0)), ((2, 100, vec * 9 + vec // 2), (0, 2, 1)),
             ((5, 129, 257), (0, 2, 1))]  # (the last: odd extents, the element-wise tiles)
    g = axo.PCG64(600 + dt)
    for shape, perm in cases:
        base = sample(shape, dt, int(g.uniform((1,), 1, 100)[0]))
        d = gh.to_dev(base)
        view = base.transpose(perm)
        out = gh.empty_dev(view.shape, dt)
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(d.data_ptr(), dt, out.data_ptr(), dt, view.ndim, i64(view.shape), i64(elem_strides(view)), None))
        gh.sync()
        assert np.array_equal(gh.to_host(out, base.dtype), np.ascontiguousarray(view)), (shape, perm)
    # a window of a larger array, transposed (its rows start every 264 elements, its first element at a vector boundary)
    base = sample((4, 200, 264), dt, 7)
    d = gh.to_dev(base)
    view = base[1:3, 8:168, 2 * vec:2 * vec + 128].transpose(0, 2, 1)
    off = view.__array_interface__["data"][0] - base.__array_interface__["data"][0]
    out = gh.empty_dev(view.shape, dt)
    gh.sync()
    capi.check(capi.lib().axhip_strided_copy(d.data_ptr() + off, dt, out.data_ptr(), dt, view.ndim, i64(view.shape), i64(elem_strides(view)), None))
    gh.sync()
    assert np.array_equal(gh.to_host(out, base.dtype), np.ascontiguousarray(view))


def test_strided_copy_casts_on_the_fast_paths():
    x = axo.PCG64(10).normal((96, 200))
    d = gh.to_dev(x)
    for dt in (F16, BF16):
        for view, strides in ((x, [200, 1]), (x.T, [1, 200])):
            out = gh.empty_dev(view.shape, dt)
            gh.sync()
            capi.check(capi.lib().axhip_strided_copy(d.data_ptr(), F32, out.data_ptr(), dt, 2, i64(view.shape), i64(strides), None))
            gh.sync()
            assert np.array_equal(gh.to_host(out, np.uint16), axo.to_bits(np.ascontiguousarray(view), dt))
        # and back: 16-bit source, fp32 destination
        bits = axo.to_bits(x, dt)
        db = gh.to_dev(bits)
        out = gh.empty_dev(x.shape, F32)
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(db.data_ptr(), dt, out.data_ptr(), F32, 2, i64(x.shape), i64([200, 1]), None))
        gh.sync()
        assert np.array_equal(gh.to_host(out, np.float32), axo.to_f32(bits, dt))


@pytest.mark.parametrize("dt", [F32, F16, BF16], ids=["f32", "f16", "bf16"])
def test_gathers_from_unaligned_and_every_other_positions_are_bit_exact(dt):
    """Views whose innermost dimension is contiguous in the source but starts anywhere (a column slice from an odd
    column, the windows of a convolution) move as unaligned 16-byte loads and aligned stores; views that take every
    other element (x[:, ::2], the windows of a stride-2 convolution) pick a group out of two such loads, the second of
    which ends with the group's last element -- the array's very last element included.  With a cast on the way for
    the contiguous kind."""
    vec = 4 if dt == F32 else 8
    base = sample((3, 5, 40, 12 * vec + 3), dt, 21)
    d = gh.to_dev(base)
    w = 8 * vec
    views = [base[:, :, :, 1:1 + w], base[:, :, 3:, 3:3 + w], base[1, :, ::3, 2:2 + w],
             np.lib.stride_tricks.as_strided(base, (3, 5, 3, 38, w), base.strides[:2] + (base.strides[2], base.strides[2], base.strides[3])),  # windows of 3 rows
             base[:, :, :, ::2][..., :5 * vec], base[:, :, :, 1::2][..., :6 * vec], base[2, 4, 39:, 3::2][..., :6 * vec],
             np.lib.stride_tricks.as_strided(base[0, 0, 0], (3, 4 * vec), (base.strides[3], 2 * base.strides[3]))]  # windows of a stride-2 convolution
    flat = base.reshape(-1)
    views.append(flat[flat.size - 2 * (2 * vec) + 1::2])  # ends with the array's last element
    views.append(flat[flat.size - 2 * (vec + vec // 2) + 1::2])  # the same with a half group at its end
    views.append(base[:, :, :, ::2][..., :5 * vec + vec // 2])  # rows of whole half groups (8-byte loads and stores)
    for view in views:
        out = gh.empty_dev(view.shape, dt)
        off = view.__array_interface__["data"][0] - base.__array_interface__["data"][0]
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(d.data_ptr() + off, dt, out.data_ptr(), dt, view.ndim, i64(view.shape), i64(elem_strides(view)), None))
        gh.sync()
        assert np.array_equal(gh.to_host(out, base.dtype), np.ascontiguousarray(view)), view.shape
    if dt != F32:
        view = base[:, :, :, 1:1 + w]
        out = gh.empty_dev(view.shape, F32)
        off = view.__array_interface__["data"][0] - base.__array_interface__["data"][0]
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(d.data_ptr() + off, dt, out.data_ptr(), F32, view.ndim, i64(view.shape), i64(elem_strides(view)), None))
        gh.sync()
        assert np.array_equal(gh.to_host(out, np.float32), axo.to_f32(np.ascontiguousarray(view), dt))


def test_large_contiguous_casts_are_bit_exact():
    """A cast of a contiguous array of 8 MiB or more runs as a compiled elementwise chain with no operation; the bits
    are those of the oracle's conversions (round to nearest even into the 16-bit types, exact widening)."""
    x = axo.PCG64(12).normal((1 << 22,)) * 3
    d = gh.to_dev(x)
    for dt in (F16, BF16):
        out = gh.empty_dev(x.shape, dt)
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(d.data_ptr(), F32, out.data_ptr(), dt, 1, i64(x.shape), i64([1]), None))
        gh.sync()
        bits = gh.to_host(out, np.uint16)
        assert np.array_equal(bits, axo.to_bits(x, dt))
        db = gh.to_dev(bits)
        back = gh.empty_dev((1 << 11, 1 << 11), F32)  # (the same array as a matrix: contiguous all the same)
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(db.data_ptr(), dt, back.data_ptr(), F32, 2, i64((1 << 11, 1 << 11)), i64([1 << 11, 1]), None))
        gh.sync()
        assert np.array_equal(gh.to_host(back, np.float32).ravel(), axo.to_f32(bits, dt))


def test_strided_copy_casts_like_the_oracle():
    x = axo.PCG64(9).normal((33, 17))
    d = gh.to_dev(x)
    for dt in (F16, BF16):
        out = gh.empty_dev(x.shape, dt)
        gh.sync()
        capi.check(capi.lib().axhip_strided_copy(d.data_ptr(), F32, out.data_ptr(), dt, 2, i64(x.shape), i64([17, 1]), None))
        gh.sync()
        assert np.array_equal(gh.to_host(out, np.uint16), axo.to_bits(x, dt))


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
def test_fill(dt):
    out = gh.empty_dev((1000,), dt)
    gh.sync()
    capi.check(capi.lib().axhip_fill(out.data_ptr(), dt, 1.5, 1000, None))
    gh.sync()
    got = gh.to_host(out, gh.np_store_dtype(dt))
    want = np.full(1000, 1.5, np.float32)
    assert np.array_equal(got, want if dt == F32 else axo.to_bits(want, dt))


@pytest.mark.parametrize("dt", [F32, F16, BF16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("shape,before,after", [((5,), (2,), (3,)), ((3, 4), (0, 1), (2, 0)), ((2, 3, 50), (0, 0, 1), (0, 0, 1)),
                                                ((2, 1, 3, 4), (1, 0, 2, 0), (0, 3, 0, 5)),
                                                # innermost output extents of whole 16-byte vectors: one store per vector
                                                ((3, 5, 27), (1, 0, 2), (0, 2, 3)), ((2, 2, 30, 48), (0, 0, 0, 0), (0, 0, 0, 16)), ((7, 1001), (0, 0), (0, 23)),
                                                ((64,), (0,), (0,)), ((4, 300), (0, 40), (1, 37)), ((2, 3, 256), (0, 0, 64), (0, 1, 64)),
                                                # odd rows in an aligned output: groups cut from the whole output, some across two rows
                                                ((3, 7, 301), (0, 1, 1), (1, 0, 1)), ((5, 9), (1, 0), (0, 0))])
def test_pad_matches_numpy(dt, shape, before, after):
    x = sample(shape, dt, 11)
    value = -2.5
    fill = np.float32(value) if dt == F32 else axo.to_bits(np.array([value], np.float32), dt)[0]
    want = np.pad(x, list(zip(before, after)), constant_values=fill)
    d = gh.to_dev(x)
    out = gh.empty_dev(want.shape, dt)
    gh.sync()
    capi.check(capi.lib().axhip_pad(d.data_ptr(), out.data_ptr(), dt, x.ndim, i64(shape), i64(elem_strides(x)), i64(before), i64(after), value, None))
    gh.sync()
    assert np.array_equal(gh.to_host(out, x.dtype), want)


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("mode,np_mode", [("reflect", "reflect"), ("replicate", "edge"), ("circular", "wrap")])
@pytest.mark.parametrize("shape,before,after", [((5,), (2,), (3,)), ((3, 4), (0, 1), (2, 0)), ((3, 5, 27), (1, 0, 2), (0, 2, 3)),
                                                ((2, 2, 30, 48), (0, 1, 0, 7), (1, 0, 0, 9)), ((7, 1001), (3, 0), (0, 23)),
                                                # pads longer than a 16-byte group along the innermost extent: whole groups are mirror images
                                                # (read backwards) or wrapped-around runs; odd and whole-vector output rows
                                                ((4, 300), (0, 40), (0, 37)), ((2, 3, 256), (0, 0, 64), (0, 1, 64)), ((3, 100), (1, 99), (0, 99)),
                                                ((3, 7, 301), (0, 1, 1), (1, 0, 1)), ((5, 9), (1, 0), (0, 0))])
def test_pad_modes_match_numpy(dt, mode, np_mode, shape, before, after):
    """reflect / replicate / circular as the reference indexes them (src/tensor/operations.cpp:2216-2246), which is
    what numpy's 'reflect' / 'edge' / 'wrap' do."""
    x = sample(shape, dt, 13)
    want = np.pad(x, list(zip(before, after)), mode=np_mode)
    d = gh.to_dev(x)
    out = gh.empty_dev(want.shape, dt)
    gh.sync()
    capi.check(capi.lib().axhip_pad_mode(d.data_ptr(), out.data_ptr(), dt, x.ndim, i64(shape), i64(elem_strides(x)), i64(before), i64(after),
                                         capi.PAD[mode], 0.0, None))
    gh.sync()
    assert np.array_equal(gh.to_host(out, x.dtype), want)


def test_pad_mode_errors():
    x = gh.to_dev(np.zeros((4,), np.float32))
    out = gh.empty_dev((12,), F32)
    l = capi.lib()
    assert l.axhip_pad_mode(x.data_ptr(), out.data_ptr(), F32, 1, i64([4]), i64([1]), i64([4]), i64([4]), capi.PAD["reflect"], 0.0, None) == capi.ERR_INVALID_ARG
    assert l.axhip_pad_mode(x.data_ptr(), out.data_ptr(), F32, 1, i64([4]), i64([1]), i64([4]), i64([4]), 4, 0.0, None) == capi.ERR_INVALID_ARG
    assert l.axhip_pad_mode(x.data_ptr(), out.data_ptr(), F32, 1, i64([0]), i64([1]), i64([1]), i64([1]), capi.PAD["replicate"], 0.0, None) == capi.ERR_INVALID_ARG
    assert l.axhip_pad_mode(x.data_ptr(), out.data_ptr(), F32, 1, i64([4]), i64([1]), i64([4]), i64([4]), capi.PAD["circular"], 0.0, None) == 0
    gh.sync()


def test_pad_of_a_transposed_view():
    base = sample((4, 6), F32, 12)
    view = base.T
    want = np.pad(view, [(1, 1), (0, 2)])
    d = gh.to_dev(base)
    out = gh.empty_dev(want.shape, F32)
    gh.sync()
    capi.check(capi.lib().axhip_pad(d.data_ptr(), out.data_ptr(), F32, 2, i64(view.shape), i64(elem_strides(view)), i64([1, 0]), i64([1, 2]), 0.0, None))
    gh.sync()
    assert np.array_equal(gh.to_host(out, np.float32), want)


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
def test_pad_of_a_transposed_operand_to_an_aligned_reduction_length(dt):
    """What the matrix product's repacking asks for: a [k, n] operand read as its (batch, n, k) transpose, k padded
    with zeros to the next multiple of 64."""
    base = sample((2, 301, 40), dt, 21)
    view = base.transpose(0, 2, 1)
    want = np.pad(view, [(0, 0), (0, 0), (0, 19)])
    d = gh.to_dev(base)
    out = gh.empty_dev(want.shape, dt)
    gh.sync()
    capi.check(capi.lib().axhip_pad(d.data_ptr(), out.data_ptr(), dt, 3, i64(view.shape), i64(elem_strides(view)), i64([0, 0, 0]), i64([0, 0, 19]), 0.0, None))
    gh.sync()
    assert np.array_equal(gh.to_host(out, base.dtype), want)


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
def test_masked_fill_with_broadcast_masks(dt):
    x = sample((2, 3, 8, 8), dt, 13)
    d = gh.to_dev(x)
    i, j = np.meshgrid(np.arange(8), np.arange(8), indexing="ij")
    causal = (j > i).astype(np.uint8)  # the attention use: mask (Sq, Skv) over (B, H, Sq, Skv)
    full = (axo.PCG64(14).normal(x.shape) > 0.5).astype(np.uint8)
    fill = np.float32(-1e9) if dt == F32 else axo.to_bits(np.array([-1e9], np.float32), dt)[0]
    for mask, mstr in ((causal, [0, 0, 8, 1]), (full, [192, 64, 8, 1]), (full[:, :1, :, :1].copy(), [8, 0, 1, 0])):
        m = torch.from_numpy(mask).cuda()
        out = gh.empty_dev(x.shape, dt)
        gh.sync()
        capi.check(capi.lib().axhip_masked_fill(d.data_ptr(), dt, m.data_ptr(), out.data_ptr(), 4, i64(x.shape), i64(elem_strides(x)), i64(mstr), -1e9, None))
        gh.sync()
        bm = np.broadcast_to(mask.reshape([x.shape[k] if mstr[k] else 1 for k in range(4)]) if mask.ndim == 4 else mask, x.shape)
        assert np.array_equal(gh.to_host(out, x.dtype), np.where(bm != 0, fill, x))


@pytest.mark.parametrize("dt", [F32, BF16, F16], ids=["f32", "bf16", "f16"])
@pytest.mark.parametrize("cols,pitch", [(64, 64), (48, 72), (12, 12), (40, 44)], ids=["64", "48of72", "12", "40of44"])
def test_masked_fill_of_row_views_sixteen_bytes_at_a_time(dt, cols, pitch):
    """Rows that are contiguous in the source take the vector kernel when their length, pitch and the mask's pitches
    are whole 16-byte groups (64, 48 of 72) and the element kernel otherwise (12; 40 of 44 for the 16-bit types); the
    mask's bytes are any non-zero value; a mask over [queries, keys], one over everything, and one that repeats along
    the keys."""
    base = sample((3, 5, 33, pitch), dt, 31)
    x = base[..., :cols]
    d = gh.to_dev(base)
    rng = axo.PCG64(32)
    any_byte = lambda shape: ((rng.normal(shape) > 0.3) * (1 + (np.abs(rng.normal(shape)) * 100).astype(np.int64) % 255)).astype(np.uint8)
    fill = np.float32(-3.5)
    for mshape, mstr in (((33, cols), [0, 0, cols, 1]), (x.shape, [5 * 33 * cols, 33 * cols, cols, 1]), ((3, 1, 33, 1), [33, 0, 1, 0]), ((3, 1, 1, cols), [cols, 0, 0, 1])):
        mask = any_byte(mshape)
        m = torch.from_numpy(mask).cuda()
        out = gh.empty_dev(x.shape, dt)
        gh.sync()
        capi.check(capi.lib().axhip_masked_fill(d.data_ptr(), dt, m.data_ptr(), out.data_ptr(), 4, i64(x.shape), i64(elem_strides(x)), i64(mstr), float(fill), None))
        gh.sync()
        want = np.where(np.broadcast_to(mask, x.shape) != 0, fill if dt == F32 else axo.to_bits(np.array([fill], np.float32), dt)[0], x)
        assert np.array_equal(gh.to_host(out, x.dtype), want), (mshape, mstr)


@pytest.mark.parametrize("dt,cols", [(F32, 8), (BF16, 64), (F16, 7), (F32, 3)], ids=["f32x8", "bf16x64", "f16x7", "f32x3"])
@pytest.mark.parametrize("itype", [np.int64, np.int32], ids=["i64", "i32"])
def test_gather_rows_is_an_embedding_lookup(dt, cols, itype):
    table = sample((50, cols), dt, 15)
    idx = np.array([0, 49, 7, 7, 23, -1, 50, 3], itype)  # two out-of-range entries -> zero rows
    d, di = gh.to_dev(table), torch.from_numpy(idx).cuda()
    out = gh.empty_dev((idx.size, cols), dt)
    gh.sync()
    capi.check(capi.lib().axhip_gather_rows(d.data_ptr(), dt, 50, cols, di.data_ptr(), idx.itemsize, idx.size, out.data_ptr(), None))
    gh.sync()
    want = np.where(((idx >= 0) & (idx < 50))[:, None], table[np.clip(idx, 0, 49)], np.zeros((), table.dtype))
    assert np.array_equal(gh.to_host(out, table.dtype), want)


def _argreduce(dev, dt, outer, axis, inner, want_min):
    out = torch.full((outer * inner,), -7, dtype=torch.int64, device="cuda")
    gh.sync()
    capi.check(capi.lib().axhip_argreduce(dev.data_ptr(), dt, outer, axis, inner, int(want_min), out.data_ptr(), None))
    gh.sync()
    return out.cpu().numpy()


@pytest.mark.parametrize("dt", [F32, F16, BF16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("rows,cols", [(37, 1), (513, 10), (300, 77), (64, 1001), (33, 4096), (9, 8192), (5, 50257), (3, 128256), (2, 200003)],
                         ids=lambda v: str(v))
def test_argmax_argmin_over_rows_match_the_cpu_scan(dt, rows, cols):
    """Row form (inner == 1) against the oracle's scan, bit-exact indices; values drawn from a small set so that every row
    has ties (the first occurrence must win), with NaN and infinities sprinkled in; odd row lengths start rows at
    every alignment."""
    rng = np.random.default_rng(rows * 1000 + cols)
    x = rng.integers(-6, 7, (rows, cols)).astype(np.float32) * 0.5
    x[rng.random((rows, cols)) < 0.01] = np.nan
    x[rng.random((rows, cols)) < 0.002] = np.inf
    x[rng.random((rows, cols)) < 0.002] = -np.inf
    if rows > 2:
        x[1, :] = np.nan  # nothing beats the start value: index 0
        x[2, :] = -np.inf
    bits = x if dt == F32 else axo.to_bits(x, dt)
    d = gh.to_dev(bits)
    for want_min in (False, True):
        got = _argreduce(d, dt, rows, cols, 1, want_min)
        assert np.array_equal(got, axo.argreduce(bits, -1, want_min, dt)), (want_min, rows, cols)
    if rows > 2:
        assert _argreduce(d, dt, rows, cols, 1, False)[1] == 0 and _argreduce(d, dt, rows, cols, 1, False)[2] == 0


@pytest.mark.parametrize("dt", [F32, BF16], ids=["f32", "bf16"])
def test_argmax_argmin_along_inner_axes_and_on_unaligned_bases(dt):
    rng = np.random.default_rng(11)
    x = rng.integers(-9, 10, (6, 130, 70)).astype(np.float32)
    bits = x if dt == F32 else axo.to_bits(x, dt)
    d = gh.to_dev(bits)
    for axis, (outer, n, inner) in ((0, (1, 6, 130 * 70)), (1, (6, 130, 70)), (2, (6 * 130, 70, 1))):
        for want_min in (False, True):
            got = _argreduce(d, dt, outer, n, inner, want_min).reshape(axo.argreduce(bits, axis, want_min, dt).shape)
            assert np.array_equal(got, axo.argreduce(bits, axis, want_min, dt)), (axis, want_min)
    # few results over a long axis: the axis is cut into segments and the candidates merged (ties across segments, NaN)
    y = rng.integers(-3, 4, (1, 8192, 64)).astype(np.float32)
    y[0, rng.integers(0, 8192, 40), rng.integers(0, 64, 40)] = np.nan
    y[0, :, 5] = np.nan
    yb = y if dt == F32 else axo.to_bits(y, dt)
    dy = gh.to_dev(yb)
    for want_min in (False, True):
        assert np.array_equal(_argreduce(dy, dt, 1, 8192, 64, want_min), axo.argreduce(yb, 1, want_min, dt).reshape(-1)), want_min
    # a view that starts one element into the buffer: rows of 4099 elements at every alignment
    flat = rng.normal(size=1 + 12 * 4099).astype(np.float32)
    fb = flat if dt == F32 else axo.to_bits(flat, dt)
    df = gh.to_dev(fb)
    out = torch.empty(12, dtype=torch.int64, device="cuda")
    gh.sync()
    capi.check(capi.lib().axhip_argreduce(df.data_ptr() + fb.itemsize, dt, 12, 4099, 1, 0, out.data_ptr(), None))
    gh.sync()
    assert np.array_equal(out.cpu().numpy(), axo.argreduce(fb[1:].reshape(12, 4099), -1, False, dt))


def test_argreduce_known_answers_and_errors():
    """tests/test_tensor_argmax_argmin.cpp:4-58 on the device; argument checks."""
    L = capi.lib()
    d = gh.to_dev(np.array([1, 5, 3, 9, 2], np.float32))
    assert _argreduce(d, F32, 1, 5, 1, False).tolist() == [3]
    m = gh.to_dev(np.array([[1, 5], [3, 2]], np.float32))
    assert _argreduce(m, F32, 1, 2, 2, False).tolist() == [1, 0] and _argreduce(m, F32, 2, 2, 1, False).tolist() == [1, 0]
    assert _argreduce(m, F32, 1, 2, 2, True).tolist() == [0, 1]
    assert L.axhip_argreduce(None, F32, 0, 5, 1, 0, None, None) == 0  # nothing to do
    assert L.axhip_argreduce(d.data_ptr(), F32, 1, 0, 1, 0, d.data_ptr(), None) == capi.ERR_INVALID_ARG  # empty axis
    assert L.axhip_argreduce(d.data_ptr(), 9, 1, 5, 1, 0, d.data_ptr(), None) == capi.ERR_INVALID_ARG
    assert L.axhip_argreduce(None, F32, 1, 5, 1, 0, None, None) == capi.ERR_INVALID_ARG
    assert L.axhip_argreduce(d.data_ptr(), F32, 1, 1 << 31, 1, 0, d.data_ptr(), None) == capi.ERR_UNSUPPORTED


@pytest.mark.parametrize("dt", [F32, F16, BF16], ids=["f32", "f16", "bf16"])
def test_reductions_along_inner_axes_match_the_oracle(dt):
    """Sum / mean / max / min along the middle extent of (outer, axis, inner) views: vector-aligned and odd inner
    extents, few and many outputs, an axis of one element; against the oracle's reduction of the same axis moved last
    (sums: fp32 accumulation in another order, 1e-4 relative to the sum of magnitudes; max / min bit-exact)."""
    rng = np.random.default_rng(5 + dt)
    for outer, axis, inner in ((1, 37, 4096), (6, 130, 72), (3, 1, 64), (64, 300, 8), (5, 77, 9), (2, 1000, 33), (300, 5, 256), (1, 4100, 24),
                               (1, 8192, 512), (2, 6000, 64),  # few results over a long axis: two passes
                               (1200, 7, 1024), (5000, 2, 264)):  # a short axis with many results: a thread per vector
        x = (rng.normal(size=(outer, axis, inner)) * 3).astype(np.float32)
        bits = x if dt == F32 else axo.to_bits(x, dt)
        xf = axo.to_f32(bits, dt)
        d = gh.to_dev(bits)
        for red in ("sum", "mean", "max", "min"):
            odt = F32 if red == "mean" else dt
            out = gh.empty_dev((outer, inner), odt)
            gh.sync()
            capi.check(capi.lib().axhip_reduce_axis(d.data_ptr(), dt, outer, axis, inner, capi.RED[red], out.data_ptr(), odt, None))
            gh.sync()
            got = axo.to_f32(gh.to_host(out, gh.np_store_dtype(odt)), odt)
            if red in ("max", "min"):
                want = axo.to_f32(axo.reduce_last(red, np.ascontiguousarray(np.moveaxis(bits, 1, -1)), dt), dt)
                assert np.array_equal(got, want), (red, outer, axis, inner)
            else:
                want = xf.astype(np.float64).sum(1) / (axis if red == "mean" else 1)
                mag = np.abs(xf).astype(np.float64).sum(1) / (axis if red == "mean" else 1)
                tol = 1e-4 * mag + (0 if odt == F32 else 2.0 ** (-8 if odt == BF16 else -11) * np.abs(want)) + 1e-6
                assert np.all(np.abs(got - want) <= tol), (red, outer, axis, inner, float(np.max(np.abs(got - want) - tol)))
    # inner == 1 goes to the row kernels
    x = rng.normal(size=(50, 333)).astype(np.float32)
    bits = x if dt == F32 else axo.to_bits(x, dt)
    d, out = gh.to_dev(bits), gh.empty_dev((50,), dt)
    gh.sync()
    capi.check(capi.lib().axhip_reduce_axis(d.data_ptr(), dt, 50, 333, 1, capi.RED["max"], out.data_ptr(), dt, None))
    gh.sync()
    assert np.array_equal(gh.to_host(out, gh.np_store_dtype(dt)), axo.reduce_last("max", bits, dt))
    L = capi.lib()
    assert L.axhip_reduce_axis(d.data_ptr(), dt, 1, 0, 4, capi.RED["sum"], out.data_ptr(), dt, None) == capi.ERR_INVALID_ARG
    assert L.axhip_reduce_axis(d.data_ptr(), dt, 1, 4, 4, 9, out.data_ptr(), dt, None) == capi.ERR_INVALID_ARG
    assert L.axhip_reduce_axis(None, dt, 0, 4, 4, capi.RED["sum"], None, dt, None) == 0


@pytest.mark.parametrize("dt", [F32, F16, BF16], ids=["f32", "f16", "bf16"])
def test_softmax_along_inner_axes_matches_the_oracle(dt):
    """softmax / log-softmax along the middle extent of (outer, axis, inner) views against the oracle's softmax over
    that axis: vector-aligned and odd inner extents, an axis of one element, long axes, large logits; fp32 1e-5
    (log: 1e-4), 16-bit one rounding step of the result."""
    rng = np.random.default_rng(9 + dt)
    for outer, axis, inner, scale in ((1, 37, 4096, 1.0), (6, 130, 72, 3.0), (3, 1, 64, 1.0), (64, 300, 8, 10.0), (5, 77, 9, 2.0), (2, 1000, 33, 1.0),
                                      (1, 5000, 24, 4.0), (1200, 7, 1024, 2.0),
                                      # short axes with many results: the axis stays in a thread's registers (up to 16 elements)
                                      (1100, 16, 512, 3.0), (1030, 13, 2048, 1.0), (1100, 17, 512, 2.0), (1500, 1, 512, 1.0), (1040, 4, 520, 5.0),
                                      # long axes that a block holds in registers (fp32: 512 to 2048 elements, 16-bit: 1024 to 4096; tiles of 16, 8 or 4 vectors,
                                      # column tiles that are not whole, one element past a tile size)
                                      (2, 1024, 136, 3.0), (3, 1025, 72, 1.0), (2, 2048, 40, 8.0), (1, 2049, 24, 2.0), (2, 4096, 24, 1.0), (5, 600, 264, 2.0),
                                      (3, 256, 4096, 1.0), (1, 4097, 16, 1.0)):
        x = (rng.normal(size=(outer, axis, inner)) * scale).astype(np.float32)
        bits = x if dt == F32 else axo.to_bits(x, dt)
        d = gh.to_dev(bits)
        for log in (False, True):
            out = gh.empty_dev((outer, axis, inner), dt)
            gh.sync()
            capi.check(capi.lib().axhip_softmax_axis(d.data_ptr(), dt, outer, axis, inner, int(log), out.data_ptr(), None))
            gh.sync()
            got = axo.to_f32(gh.to_host(out, gh.np_store_dtype(dt)), dt)
            xf = axo.to_f32(bits, dt).astype(np.float64)
            z = xf - xf.max(1, keepdims=True)
            want = z - np.log(np.exp(z).sum(1, keepdims=True)) if log else np.exp(z) / np.exp(z).sum(1, keepdims=True)
            step = 0.0 if dt == F32 else 2.0 ** (-8 if dt == BF16 else -11)
            tol = (1e-4 if log else 1e-5) + step * np.abs(want) + (1e-5 * np.abs(want) if log else 0)
            assert np.all(np.abs(got - want) <= tol), (log, outer, axis, inner, float(np.max(np.abs(got - want) - tol)))
            if not log:
                assert np.allclose(got.astype(np.float64).sum(1), 1.0, atol=1e-5 if dt == F32 else 2e-2)
            # and the oracle's own evaluation of the same axis (cpu path restated), to its 16-bit rounding
            lit = axo.to_f32(axo.softmax(bits, dt, 1, log), dt)
            assert np.all(np.abs(got - lit) <= 2 * tol + 1e-6)


def test_mover_argument_errors():
    L = capi.lib()
    assert L.axhip_pad(None, None, 7, 1, i64([1]), i64([1]), i64([0]), i64([0]), 0.0, None) == capi.ERR_INVALID_ARG
    assert L.axhip_pad(None, None, F32, 9, i64([1]), i64([1]), i64([0]), i64([0]), 0.0, None) == capi.ERR_INVALID_ARG
    assert L.axhip_gather_rows(None, F32, 4, 4, None, 2, 1, None, None) == capi.ERR_INVALID_ARG
    assert L.axhip_masked_fill(None, F32, None, None, 1, i64([4]), i64([-1]), i64([1]), 0.0, None) == capi.ERR_UNSUPPORTED
