"""Op-level rejections of the public ops and of the C ABI, without a device.

Mirrors the reference's tests of the same contract: `invalid_arguments_are_rejected` and
`fp_invalid_params_error` (crates/nuvec-core/tests/quantized.rs:127-166, 943-1001) over `nuvec_amd.ops`, and
`quantization_parameters_are_validated` plus the random primitives of
crates/nuvec-core/tests/primitive_fuzz.rs:97-131, 396-445 over the C entry points: bad parameters are answered with a
status and a message, never with a crash, and before any device is touched.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import nuvec_amd as nv
from nuvec_amd import _lib


def aq(w, group, bits):
    return nv.quantize(w, nv.Quant.affine(group, bits))


def qw(wq, s, b, group, bits):
    return nv.Quantized(wq, s, b, nv.Quant.affine(group, bits))


WQ, S, B = torch.zeros(2, 8, dtype=torch.uint32), torch.ones(2, 1), torch.zeros(2, 1)
W8, S8 = torch.zeros(2, 16, dtype=torch.uint32), torch.zeros(2, 2, dtype=torch.uint8)
MXFP8 = nv.Quant.new(nv.QuantMode.MXFP8)


def test_invalid_arguments_are_rejected():
    """tests/quantized.rs:127-166, case by case."""
    w = torch.ones(2, 64)
    for what, call in [
        ("group size", lambda: aq(w, 48, 4)),
        ("bits", lambda: aq(w, 64, 7)),
        ("1-D", lambda: aq(torch.ones(64), 64, 4)),
        ("divisibility", lambda: aq(torch.ones(2, 96), 64, 4)),
        ("dtype", lambda: aq(w.to(torch.int32), 64, 4)),
        ("group mismatch", lambda: nv.dequantize(qw(WQ, S, B, 32, 4))),
        ("packed dtype", lambda: nv.dequantize(qw(S, S, B, 64, 4))),
        ("inner size", lambda: nv.quantized_matmul(torch.ones(3, 63), qw(WQ, S, B, 64, 4))),
        ("float64 activations", lambda: nv.quantized_matmul(torch.ones(3, 64, dtype=torch.float64), qw(WQ, S, B, 64, 4))),
    ]:
        with pytest.raises(nv.InvalidArgument):
            call()
            pytest.fail(f"{what} was accepted")


def test_fp_invalid_params_error():
    """tests/quantized.rs:943-1001: MLX's wording for the floating-point modes."""
    w = torch.ones(2, 64)
    with pytest.raises(nv.InvalidArgument, match="mxfp4 quantization requires group size 32 but got 64"):
        nv.quantize(w, nv.Quant(nv.QuantMode.MXFP4, 64, 4))
    with pytest.raises(nv.InvalidArgument, match="nvfp4 quantization requires bits to be 4 but got 8"):
        nv.quantize(w, nv.Quant(nv.QuantMode.NVFP4, 16, 8))
    with pytest.raises(nv.InvalidArgument, match="biases must be null"):
        nv.dequantize(nv.Quantized(W8, S8, torch.zeros(2, 2), MXFP8))
    with pytest.raises(nv.InvalidArgument, match="biases must be provided"):
        nv.dequantize(nv.Quantized(W8, S8, None, nv.Quant.affine(32, 8)))
    with pytest.raises(nv.InvalidArgument, match="scale type must be uint8"):
        nv.dequantize(nv.Quantized(W8, S8.float(), None, MXFP8))
    with pytest.raises(nv.InvalidArgument):  # integer output
        nv.dequantize(nv.Quantized(W8, S8, None, MXFP8), torch.int32)
    with pytest.raises(nv.InvalidArgument):  # float64
        nv.quantize(w.to(torch.float64), nv.QuantMode.MXFP4)
    with pytest.raises(nv.InvalidArgument):  # float64 activations
        nv.quantized_matmul(torch.ones(3, 64, dtype=torch.float64), nv.Quantized(W8, S8, None, MXFP8))
    with pytest.raises(nv.InvalidArgument):  # inner size
        nv.quantized_matmul(torch.ones(3, 63), nv.Quantized(W8, S8, None, MXFP8))
    assert nv.QuantMode["NVFP4"] == nv.QuantMode.NVFP4


def test_gather_rejections():
    """quantized.rs:589-673: indices must be integers, shapes must match, a global scale is NVFP4's."""
    q = nv.Quantized(W8.reshape(1, 2, 16), S8.reshape(1, 2, 2), None, MXFP8)
    with pytest.raises(nv.InvalidArgument, match="indices must be integers"):
        nv.gather_qmm(torch.ones(3, 1, 64), q, None, torch.tensor([0.5]))
    with pytest.raises(nv.InvalidArgument, match="do not match"):
        nv.gather_qmm(torch.ones(3, 1, 63), q, None, torch.tensor([0]))
    scaled = nv.Quantized(W8.reshape(1, 2, 16), S8.reshape(1, 2, 2), None, MXFP8, torch.ones(1))
    with pytest.raises(nv.InvalidArgument, match="global scale"):
        nv.gather_qmm(torch.ones(3, 1, 64), scaled, None, torch.tensor([0]))


def _quant(mode, group, bits):
    return _lib.QuantC(mode, group, bits)


def test_gather_with_an_empty_operand_is_refused():
    """The device clamps indices into [0, x_batches) and [0, experts): pairs against an empty x or no experts have
    nothing to clamp to and are refused on the host, before the device is asked for."""
    lib = _lib.load()
    one = C.c_void_p(16)
    for x_batches, experts in ((0, 2), (2, 0), (0, 0)):
        g = _lib.GatherDescC(_quant(0, 64, 4), _lib.BF16, 1, 0, 0, 1, 8, 64, 3, x_batches, experts)
        assert lib.nvq_gather_qmm(C.byref(g), one, one, one, one, one, one, None, one, None, None) == _lib.INVALID_ARGUMENT
        assert "experts" in _lib.last_error()
        assert lib.nvq_gather_qmm_glu(C.byref(g), 0, 1.0, 7.0, one, one, one, one, one, one, None, one, None, None) == _lib.INVALID_ARGUMENT
    empty = _lib.GatherDescC(_quant(0, 64, 4), _lib.BF16, 1, 0, 0, 1, 8, 64, 0, 0, 0)  # no pairs: nothing to do
    assert lib.nvq_gather_qmm(C.byref(empty), one, one, one, one, one, one, None, one, None, None) == _lib.OK


def test_gated_gather_counts_rows_and_ids_without_offsets():
    """The unsorted route (no offsets) answers a row / id count mismatch with InvalidArgument, like the sorted one."""
    q = nv.Quantized(torch.zeros(2, 128, 8, dtype=torch.uint32), torch.ones(2, 128, 1), torch.zeros(2, 128, 1), nv.Quant.affine(64, 4))
    with pytest.raises(nv.InvalidArgument, match="no offsets"):
        nv.gather_qmm_glu(torch.ones(3, 64), q, torch.tensor([0, 1, 2], dtype=torch.int32), torch.tensor([0, 1], dtype=torch.int32), None)


def test_quantization_parameters_are_validated_by_the_library():
    """primitive_fuzz.rs:97-131 at the C boundary: each bad `Quant` is refused by every entry point that takes one,
    with NVQ_INVALID_ARGUMENT and before the device is asked for (none is bound in this process)."""
    lib = _lib.load()
    bad = [_quant(0, 0, 4), _quant(0, 64, 7), _quant(0, 64, 0), _quant(1, 64, 4), _quant(3, 16, 8), _quant(9, 32, 4)]
    one = C.c_void_p(16)  # never dereferenced: validation comes first
    for q in bad:
        assert lib.nvq_quantize(C.byref(q), _lib.F32, one, 4, 64, one, one, one, None) == _lib.INVALID_ARGUMENT
        assert lib.nvq_dequantize(C.byref(q), _lib.F32, one, one, one, 4, 64, one, None) == _lib.INVALID_ARGUMENT
        d = _lib.QmmDescC()
        d.quant, d.dtype, d.transpose, d.m, d.n, d.k = q, _lib.F32, 1, 4, 4, 64
        assert lib.nvq_quantized_matmul(C.byref(d), one, one, one, one, one, None, None) == _lib.INVALID_ARGUMENT
        assert lib.nvq_quantized_matmul_supported(C.byref(d)) == 0
        assert lib.nvq_quantized_matmul_workspace_bytes(C.byref(d)) == 0
        g = _lib.GatherDescC(q, _lib.F32, 1, 0, 0, 1, 4, 64, 2, 2, 2)
        assert lib.nvq_gather_qmm(C.byref(g), one, one, one, one, one, one, None, one, None, None) == _lib.INVALID_ARGUMENT
        assert _lib.last_error()
    # floating-point modes take no biases, affine needs them (quantized.rs:363-379)
    mx = _quant(1, 32, 4)
    assert lib.nvq_dequantize(C.byref(mx), _lib.F32, one, one, one, 4, 64, one, None) == _lib.INVALID_ARGUMENT
    assert "biases must be null" in _lib.last_error()
    af = _quant(0, 64, 4)
    assert lib.nvq_dequantize(C.byref(af), _lib.F32, one, one, None, 4, 64, one, None) == _lib.INVALID_ARGUMENT
    assert "biases must be provided" in _lib.last_error()


def test_random_descriptors_never_crash():
    """primitive_fuzz.rs:396-445: random modes, group sizes, bit counts, element types, orientations and sizes.  Without a
    device every call must come back with a status: a bad descriptor NVQ_INVALID_ARGUMENT, a good one NVQ_NO_DEVICE (or
    NVQ_OK for an empty product), and the queries must answer 0."""
    lib = _lib.load()
    rng = np.random.default_rng(0xF022)
    one = C.c_void_p(16)
    seen = set()
    for _ in range(3000):
        q = _quant(int(rng.integers(0, 5)), int(rng.choice([0, 1, 16, 32, 64, 128])), int(rng.integers(0, 10)))
        dtype = int(rng.choice([_lib.F32, _lib.BF16, _lib.F16, _lib.U8, _lib.I32, 0]))
        d = _lib.QmmDescC()
        d.quant, d.dtype, d.transpose = q, dtype, int(rng.integers(0, 2))
        d.row_exact, d.rows = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        d.m, d.n, d.k = (int(rng.choice([-1, 0, 1, 3, 16, 63, 64, 96, 128, 4096, 1 << 33])) for _ in range(3))
        d.batch_ndim = int(rng.choice([-1, 0, 0, 0, 1, 2, 7]))
        for i in range(_lib.MAX_BATCH_DIMS):
            d.batch_shape[i] = int(rng.choice([-1, 0, 1, 2, 5]))
            d.x_strides[i], d.w_strides[i], d.s_strides[i] = (int(rng.choice([-3, 0, 1, 64])) for _ in range(3))
        biases = one if rng.integers(0, 2) else None
        rc = lib.nvq_quantized_matmul(C.byref(d), one, one, one, biases, one, None, None)
        assert rc in (_lib.OK, _lib.INVALID_ARGUMENT, _lib.UNSUPPORTED, _lib.NO_DEVICE), rc
        assert rc == _lib.OK or _lib.last_error()
        assert lib.nvq_quantized_matmul_workspace_bytes(C.byref(d)) == 0  # no device: nothing to size
        lib.nvq_quantized_matmul_supported(C.byref(d))
        rc2 = lib.nvq_quantize(C.byref(q), dtype, one, d.m, d.k, one, one, biases, None)
        rc3 = lib.nvq_dequantize(C.byref(q), dtype, one, one, biases, d.n, d.k, one, None)
        g = _lib.GatherDescC(q, dtype, d.transpose, d.row_exact, 0, d.m, d.n, d.k, int(rng.choice([-1, 0, 3])), 2, 2)
        rc4 = lib.nvq_gather_qmm(C.byref(g), one, one, one, biases, one, one, None, one, None, None)
        for r in (rc2, rc3, rc4):
            assert r in (_lib.OK, _lib.INVALID_ARGUMENT, _lib.UNSUPPORTED, _lib.NO_DEVICE), r
        seen.update((rc, rc2, rc3, rc4))
    assert {_lib.INVALID_ARGUMENT, _lib.NO_DEVICE} <= seen  # both kinds of answers were exercised
