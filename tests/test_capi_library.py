"""CPU-side checks of the C-ABI library: it loads, exports every symbol the
header declares, and rejects bad arguments before touching a device."""
import ctypes as C
import re
from pathlib import Path

import pytest

from axiom_amd import capi

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "axhip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(axhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.lib()
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/axhip.h but not exported"


def test_struct_layouts_match_the_compiled_library():
    lib = capi.lib()
    lib.axhip_sizeof.restype = C.c_size_t
    for which, cls in enumerate((capi.SdpaParams, capi.RowsProgram, capi.GemmParams, capi.Operand, capi.ChainOp)):
        assert lib.axhip_sizeof(which) == C.sizeof(cls), cls.__name__
    assert lib.axhip_sizeof(99) == 0


def test_version_and_kernel_selection_without_device():
    lib = capi.lib()
    assert b"gfx950" in lib.axhip_version()
    p = capi.SdpaParams()
    p.dtype, p.batch, p.heads, p.seq_q, p.seq_kv, p.head_dim = capi.DTYPE_BF16, 4, 32, 4096, 4096, 128
    for i, s in enumerate((32 * 4096 * 128, 4096 * 128, 128)):
        p.q_strides[i] = p.k_strides[i] = p.v_strides[i] = p.o_strides[i] = s
    assert lib.axhip_sdpa_kernel_name(C.byref(p)) == b"mfma_bf16_d128"
    p.head_dim = 48  # multiples of 8 between the compiled head sizes run on the next one, zeros in the missing dims
    assert lib.axhip_sdpa_kernel_name(C.byref(p)) == b"mfma_bf16_d48"
    p.head_dim = 20
    assert lib.axhip_sdpa_kernel_name(C.byref(p)) == b"generic"  # the fallback of the reference's unsupported head sizes
    p.dtype, p.head_dim = capi.DTYPE_F32, 64
    assert lib.axhip_sdpa_kernel_name(C.byref(p)) == b"mfma_f32_d64"
    p.head_dim = 96  # fp32: multiples of 4 up to 128 run as the next of 32 / 64 / 128
    assert lib.axhip_sdpa_kernel_name(C.byref(p)) == b"mfma_f32_d96"
    p.head_dim = 98
    assert lib.axhip_sdpa_kernel_name(C.byref(p)) == b"generic"
    r = capi.RowsProgram()
    r.rows, r.cols, r.input_dtype, r.output_dtype = 8192, 8192, capi.DTYPE_F32, capi.DTYPE_F32
    r.row_op = capi.ROWOP["softmax"]
    assert lib.axhip_fused_rows_kernel_name(C.byref(r)) == b"rows_resident_g256_it8_e4"
    r.cols, r.input_dtype = 4096, capi.DTYPE_BF16
    # a 16-bit input with an fp32 output moves in chunks of 4 elements (16 bytes of the wider stream) ...
    assert lib.axhip_fused_rows_kernel_name(C.byref(r)) == b"rows_resident_g256_it4_e4"
    r.output_dtype = capi.DTYPE_BF16  # ... and of 8 when every full-size stream is 16-bit
    assert lib.axhip_fused_rows_kernel_name(C.byref(r)) == b"rows_resident_g256_it2_e8"
    r.cols = 1 << 20
    assert lib.axhip_fused_rows_kernel_name(C.byref(r)) == b"rows_streamed_e8"
    r.cols, r.row_op = 37, 0  # no vector divides 37: the aligned array is walked as one flat run of 8-element chunks
    assert lib.axhip_fused_rows_kernel_name(C.byref(r)) == b"elementwise_flat_e8"
    r.cols = 5  # rows shorter than a chunk: element by element
    assert lib.axhip_fused_rows_kernel_name(C.byref(r)) == b"elementwise_e1"


def test_argument_errors_are_reported_before_any_launch():
    lib = capi.lib()
    with pytest.raises(capi.AxhipError) as e:
        capi.check(lib.axhip_sdpa_fwd(None, None, None, None, None, None, None))
    assert e.value.code == -1 and "params" in str(e.value)
    p = capi.SdpaParams()
    p.dtype = 9
    with pytest.raises(capi.AxhipError):
        capi.check(lib.axhip_sdpa_fwd(None, None, None, None, None, C.byref(p), None))
    r = capi.RowsProgram()
    r.rows, r.cols = 4, 4
    r.n_pre = 1
    r.pre[0].op = 999
    with pytest.raises(capi.AxhipError) as e:
        capi.check(lib.axhip_fused_rows(C.byref(r), None))
    assert "unknown op" in str(e.value)
    r.pre[0].op = capi.OP["add"]
    r.pre[0].operand = 3  # no such operand
    with pytest.raises(capi.AxhipError):
        capi.check(lib.axhip_fused_rows(C.byref(r), None))
    g = capi.GemmParams()
    g.dtype, g.m, g.n, g.k, g.ldc = 0, 4, 4, 4, 2  # ldc < n
    with pytest.raises(capi.AxhipError):
        capi.check(lib.axhip_gemm(None, None, None, C.byref(g), None))


def test_no_device_is_an_error_not_a_fallback():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a device is present")
    lib = capi.lib()
    assert capi.device_count() == 0
    with pytest.raises(capi.AxhipError) as e:
        capi.check(lib.axhip_init(0))
    assert e.value.code == -3
    ptr = C.c_void_p()
    with pytest.raises(capi.AxhipError):  # make_storage(GPU) without a device -> DeviceError in the reference
        capi.check(lib.axhip_malloc(C.byref(ptr), 1024))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(capi, "_lib", None)
    monkeypatch.setattr(capi, "LIB_PATH", tmp_path / "libaxhip.so")
    with pytest.raises(FileNotFoundError):
        capi.lib()
