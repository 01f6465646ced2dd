"""ctypes binding of `libnuvec_hip.so` — the same C ABI a Rust `extern "C"` block would bind.

There is no fallback: if the library is missing it is built with hipcc, and if that fails
the import error says so.  Nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libnuvec_hip.so")

OK, INVALID_ARGUMENT, UNSUPPORTED, OUT_OF_MEMORY, BACKEND, NO_DEVICE = range(6)
U8, U32, I32, F16, BF16, F32 = 1, 3, 7, 9, 10, 11
AFFINE, MXFP4, MXFP8, NVFP4 = 0, 1, 2, 3
MAX_BATCH_DIMS = 6
STATIC_SCRATCH_BYTES = 64 * 1024 * 1024


class InvalidArgument(ValueError):
    """nuvec's Error::InvalidArgument / shape / dtype mismatch."""


class Unsupported(NotImplementedError):
    """No gfx950 kernel: nuvec's `supports()` is false and its CPU path would run."""


class BackendError(RuntimeError):
    """nuvec's Error::Backend."""


class NoDevice(RuntimeError):
    """nuvec's Error::UnsupportedDevice."""


class QuantC(C.Structure):
    _fields_ = [("mode", C.c_int32), ("group_size", C.c_int32), ("bits", C.c_int32)]


class DeviceInfoC(C.Structure):
    _fields_ = [("device", C.c_int32), ("compute_units", C.c_int32), ("wavefront_size", C.c_int32),
                ("lds_bytes_per_block", C.c_int32), ("global_memory_bytes", C.c_int64),
                ("arch", C.c_char * 64), ("name", C.c_char * 128)]


_DIMS = C.c_int64 * MAX_BATCH_DIMS


class QmmDescC(C.Structure):
    _fields_ = [("quant", QuantC), ("dtype", C.c_int32), ("transpose", C.c_int32), ("row_exact", C.c_int32),
                ("rows", C.c_int32), ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64),
                ("item_rows", C.c_int64), ("batch_ndim", C.c_int32), ("batch_shape", _DIMS),
                ("x_strides", _DIMS), ("w_strides", _DIMS), ("s_strides", _DIMS)]


class AttentionDescC(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("bits", C.c_int32), ("group_size", C.c_int32), ("head_dim", C.c_int32),
                ("batch", C.c_int64), ("query_heads", C.c_int64), ("key_heads", C.c_int64), ("positions", C.c_int64),
                ("scale", C.c_float)]


class GluDescC(C.Structure):
    _fields_ = [("dtype", C.c_int32), ("activation", C.c_int32), ("alpha", C.c_float), ("limit", C.c_float),
                ("rows", C.c_int64), ("hidden", C.c_int64), ("gate_stride", C.c_int64), ("up_stride", C.c_int64),
                ("experts", C.c_int64)]


class GatherDescC(C.Structure):
    _fields_ = [("quant", QuantC), ("dtype", C.c_int32), ("transpose", C.c_int32), ("row_exact", C.c_int32),
                ("reserved", C.c_int32), ("m", C.c_int64), ("n", C.c_int64), ("k", C.c_int64), ("pairs", C.c_int64),
                ("x_batches", C.c_int64), ("experts", C.c_int64)]


# name -> (restype, argtypes): every symbol include/nuvec_hip.h declares.
SIGNATURES = {
    "nvq_init": (C.c_int32, [C.c_int32]),
    "nvq_get_device_info": (C.c_int32, [C.POINTER(DeviceInfoC)]),
    "nvq_last_error": (C.c_char_p, []),
    "nvq_version": (C.c_char_p, []),
    "nvq_calibrate": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.POINTER(C.c_int64), C.c_void_p]),
    "nvq_quant_check": (C.c_int32, [C.POINTER(QuantC), C.c_char_p]),
    "nvq_gather_grouped": (C.c_int32, [C.c_int64, C.c_int64, C.c_int32]),
    "nvq_quantized_matmul_supported": (C.c_int32, [C.POINTER(QmmDescC)]),
    "nvq_quantize": (C.c_int32, [C.POINTER(QuantC), C.c_int32, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p,
                                 C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_dequantize": (C.c_int32, [C.POINTER(QuantC), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                   C.c_int64, C.c_void_p, C.c_void_p]),
    "nvq_dequantize_rows": (C.c_int32, [C.POINTER(QuantC), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                        C.c_int64, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p]),
    "nvq_quantized_matmul_workspace_bytes": (C.c_size_t, [C.POINTER(QmmDescC)]),
    "nvq_quantized_matmul": (C.c_int32, [C.POINTER(QmmDescC), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                         C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_quantized_linear": (C.c_int32, [C.POINTER(QmmDescC)] + [C.c_void_p] * 8),
    "nvq_quantized_matmul_static": (C.c_int32, [C.POINTER(QmmDescC), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                                C.c_void_p, C.c_void_p]),
    "nvq_quantized_matmul_route": (C.c_char_p, [C.POINTER(QmmDescC)]),
    "nvq_quantized_attention_workspace_bytes": (C.c_size_t, [C.POINTER(AttentionDescC)]),
    "nvq_quantized_attention": (C.c_int32, [C.POINTER(AttentionDescC)] + [C.c_void_p] * 11),
    "nvq_sorted_offsets": (C.c_int32, [C.c_void_p, C.c_int64, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p]),
    "nvq_quantize_scaled": (C.c_int32, [C.c_void_p, C.c_int32, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_dequantize_scaled": (C.c_int32, [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]),
    "nvq_quantized_matmul_scaled": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_gather_qmm_scaled": (C.c_int32, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                          C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_gather_qmm_scatter": (C.c_int32, [C.c_void_p] * 13),
    "nvq_gather_qmm_expert_bias": (C.c_int32, [C.c_void_p] * 14),
    "nvq_quantize_dequantize": (C.c_int32, [C.c_void_p, C.c_int32, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_moe_route": (C.c_int32, [C.c_int32, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_quantized_matmul_glu": (C.c_int32, [C.POINTER(QmmDescC), C.c_int32, C.c_float, C.c_float] + [C.c_void_p] * 7),
    "nvq_gather_qmm_glu": (C.c_int32, [C.POINTER(GatherDescC), C.c_int32, C.c_float, C.c_float] + [C.c_void_p] * 10),
    "nvq_glu": (C.c_int32, [C.POINTER(GluDescC), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_weighted_sum": (C.c_int32, [C.c_int32, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int64, C.c_void_p, C.c_void_p]),
    "nvq_moe_order": (C.c_int32, [C.c_void_p, C.c_int64, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                  C.c_void_p, C.c_void_p]),
    "nvq_moe_order_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int32]),
    "nvq_convert_packed": (C.c_int32, [C.c_int32, C.POINTER(QuantC), C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                       C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "nvq_gather_qmm_workspace_bytes": (C.c_size_t, [C.POINTER(GatherDescC)]),
    "nvq_gather_qmm": (C.c_int32, [C.POINTER(GatherDescC), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                   C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
}

_lib = None


def load() -> C.CDLL:
    """Loads the library (building it first only if it was never built)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        from . import build
        build.build()
    try:
        # torch ships its own HIP runtime with the same soname; loading torch first makes both
        # share one runtime in processes that use torch for device memory.
        import torch  # noqa: F401
    except Exception:  # pragma: no cover - torch is optional for the binding itself
        pass
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export the symbol
        fn.restype, fn.argtypes = restype, argtypes
    _lib = lib
    return lib


def last_error() -> str:
    return load().nvq_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
    """Raises the exception nuvec would surface for a non-zero status."""
    if status == OK:
        return
    msg = last_error()
    if status == INVALID_ARGUMENT:
        raise InvalidArgument(msg)
    if status == UNSUPPORTED:
        raise Unsupported(msg)
    if status == OUT_OF_MEMORY:
        raise MemoryError(msg)
    if status == NO_DEVICE:
        raise NoDevice(msg)
    raise BackendError(msg)
