"""The C-ABI library loads and exports every symbol the public header declares; the
validation mirrors answer without a device.  No compute calls: these run without a GPU."""
import ctypes as C
import os
import re

import pytest

from nuvec_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "nuvec_hip.h")).read()
    return sorted(set(re.findall(r"NVQ_API[^;(]*?\b(nvq_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    names = declared_symbols()
    assert len(names) >= 14
    assert sorted(_lib.SIGNATURES) == names


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_symbols():
        assert getattr(lib, name) is not None
    assert lib.nvq_version().startswith(b"nuvec-hip")


def test_quant_check_messages():
    """Quant::checked's refusals, word for word (reference: quantized.rs:133-168)."""
    lib = _lib.load()
    cases = [
        ((0, 48, 4), "quantize: group size 48 is not supported (32, 64 or 128)"),
        ((0, 64, 7), "quantize: 7 bits are not supported (1, 2, 3, 4, 5, 6 or 8)"),
        ((1, 64, 4), "quantize: mxfp4 quantization requires group size 32 but got 64"),
        ((2, 32, 4), "quantize: mxfp8 quantization requires bits to be 8 but got 4"),
        ((3, 32, 4), "quantize: nvfp4 quantization requires group size 16 but got 32"),
    ]
    for (mode, group, bits), msg in cases:
        q = _lib.QuantC(mode, group, bits)
        assert lib.nvq_quant_check(C.byref(q), b"quantize") == _lib.INVALID_ARGUMENT
        assert _lib.last_error() == msg
    for ok in [(0, 32, 1), (0, 64, 4), (0, 128, 8), (1, 32, 4), (2, 32, 8), (3, 16, 4)]:
        assert lib.nvq_quant_check(C.byref(_lib.QuantC(*ok)), b"quantize") == _lib.OK


def test_grouped_rule():
    """quantized.rs:724-735: at least 16 rows and 4 per expert; row-exact, more than 64 rows."""
    lib = _lib.load()
    assert lib.nvq_gather_grouped(16, 4, 0) == 1
    assert lib.nvq_gather_grouped(15, 1, 0) == 0
    assert lib.nvq_gather_grouped(100, 32, 0) == 0   # 3 per expert
    assert lib.nvq_gather_grouped(1024, 32, 0) == 1
    assert lib.nvq_gather_grouped(64, 4, 1) == 0
    assert lib.nvq_gather_grouped(65, 4, 1) == 1
    assert lib.nvq_gather_grouped(20, 0, 0) == 1     # no experts counts as one


def test_argument_errors_come_before_the_device():
    """Bad arguments are refused on the host, device or not (primitive.rs:1223-1320)."""
    lib = _lib.load()
    q = _lib.QuantC(0, 64, 4)
    assert lib.nvq_quantize(C.byref(q), _lib.F32, None, 2, 100, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert "divisible by the group size 64" in _lib.last_error()
    assert lib.nvq_quantize(C.byref(q), _lib.I32, None, 2, 128, None, None, None, None) == _lib.INVALID_ARGUMENT
    assert lib.nvq_dequantize(C.byref(q), _lib.F32, None, None, None, 2, 128, None, None) == _lib.INVALID_ARGUMENT
    assert _lib.last_error() == "dequantize: biases must be provided for affine quantization"
    one = C.c_void_p(16)
    assert lib.nvq_dequantize_rows(C.byref(q), _lib.F32, one, one, one, 4, 100, one, 2, one, None) == _lib.INVALID_ARGUMENT
    assert "dequantize_rows: packed weights [4, 12]" in _lib.last_error()
    assert lib.nvq_dequantize_rows(C.byref(q), _lib.F32, one, one, one, 4, 128, None, 2, one, None) == _lib.INVALID_ARGUMENT
    assert _lib.last_error() == "dequantize_rows: null ids"
    assert lib.nvq_dequantize_rows(C.byref(q), _lib.F32, one, one, one, 0, 128, one, 2, one, None) == _lib.INVALID_ARGUMENT
    assert lib.nvq_dequantize_rows(C.byref(q), _lib.F32, one, one, one, 4, 128, None, 0, one, None) == _lib.OK
    d = _lib.QmmDescC()
    d.quant, d.dtype, d.transpose, d.m, d.n, d.k = q, _lib.F32, 1, 1, 8, 100
    assert lib.nvq_quantized_matmul_supported(C.byref(d)) == 0
    d.k = 128
    assert lib.nvq_quantized_matmul_supported(C.byref(d)) == 1
    d.transpose = 0
    assert lib.nvq_quantized_matmul_supported(C.byref(d)) == 0


def test_compute_without_a_device_fails_loudly():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    lib = _lib.load()
    assert lib.nvq_init(0) == _lib.NO_DEVICE
    q = _lib.QuantC(0, 64, 4)
    one = C.c_void_p(16)
    assert lib.nvq_quantize(C.byref(q), _lib.F32, one, 1, 64, one, one, one, None) == _lib.NO_DEVICE
    import nuvec_amd as nv
    with pytest.raises(_lib.NoDevice):
        nv.quantize(torch.zeros(2, 64))
