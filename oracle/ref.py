"""ctypes/numpy front end of `libnvq_ref.so` (see nvq_ref.c for what each call restates).

TEST INFRASTRUCTURE: the checker, never the thing shipped or measured (except as
the labelled CPU baseline).  Arrays are numpy; float16 is `np.float16`, bfloat16
travels as `np.uint16` bit patterns, so every call names its dtype code.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

F16, BF16, F32 = 9, 10, 11
AFFINE, MXFP4, MXFP8, NVFP4 = 0, 1, 2, 3
MODES = {"affine": AFFINE, "mxfp4": MXFP4, "mxfp8": MXFP8, "nvfp4": NVFP4}
FP_PARAMS = {MXFP4: (32, 4), MXFP8: (32, 8), NVFP4: (16, 4)}
DTYPE_CODE = {"f16": F16, "bf16": BF16, "f32": F32}
NP_OF = {F16: np.float16, BF16: np.uint16, F32: np.float32}

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libnvq_ref.so")
_lib = None


def build() -> str:
    """Compiles the oracle with its Makefile and returns the library path."""
    subprocess.run(["make", "-s", "-C", _HERE, "-B"], check=True)
    return _LIB


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            build()
        _lib = C.CDLL(_LIB)
        _lib.nvq_ref_code.restype = C.c_uint32
        for name in ("nvq_ref_ftz", "nvq_ref_canonical", "nvq_ref_e4m3_to_f32", "nvq_ref_e2m1_to_f32",
                     "nvq_ref_e8m0_to_f32", "nvq_ref_mx_scale_round_up", "nvq_ref_dot_few_rows"):
            getattr(_lib, name).restype = C.c_float
        for name in ("nvq_ref_ftz", "nvq_ref_canonical", "nvq_ref_mx_scale_round_up",
                     "nvq_ref_e4m3_from_f32", "nvq_ref_e2m1_from_f32", "nvq_ref_e8m0_from_f32"):
            getattr(_lib, name).argtypes = [C.c_float]
        for name in ("nvq_ref_e4m3_from_f32", "nvq_ref_e2m1_from_f32", "nvq_ref_e8m0_from_f32"):
            getattr(_lib, name).restype = C.c_uint8
        for name in ("nvq_ref_e4m3_to_f32", "nvq_ref_e2m1_to_f32", "nvq_ref_e8m0_to_f32"):
            getattr(_lib, name).argtypes = [C.c_uint8]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a)
    return a if dtype is None else a.astype(dtype, copy=False)


def _check(rc, what):
    if rc:
        raise ValueError(f"oracle {what}: status {rc}")


def max_threads() -> int:
    return int(lib().nvq_ref_max_threads())


# ── bf16 helpers (numpy has no bfloat16) ───────────────────────────────────────────

def bf16_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16(x: np.ndarray) -> np.ndarray:
    """Round to nearest even, NaN quieted (the `half` crate's bf16::from_f32)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    up = ((u & 0x8000) != 0) & ((u & 0x17FFF) != 0)
    out = ((u >> 16) + up).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), out)


def to_f32(a: np.ndarray, dtype: int) -> np.ndarray:
    return bf16_to_f32(a) if dtype == BF16 else a.astype(np.float32)


def from_f32(a: np.ndarray, dtype: int) -> np.ndarray:
    if dtype == BF16:
        return f32_to_bf16(a)
    return a.astype(NP_OF[dtype])


# ── the path ────────────────────────────────────────────────────────────────────────

def affine_quantize(w: np.ndarray, dtype: int, group: int, bits: int):
    w = _c(w)
    n, last = w.size, w.shape[-1]
    if last % group != 0 or (last * bits) % 32 != 0:
        raise ValueError(f"affine_quantize: last dimension {last} is not whole groups of {group} and whole words")
    packed = np.zeros(w.shape[:-1] + (last * bits // 32,), np.uint32)
    scales = np.zeros(w.shape[:-1] + (last // group,), NP_OF[dtype])
    biases = np.zeros_like(scales)
    _check(lib().nvq_ref_affine_quantize(_p(w), dtype, C.c_int64(n), group, bits, _p(packed), _p(scales),
                                         _p(biases)), "affine_quantize")
    return packed, scales, biases


def affine_dequantize(packed, scales, biases, dtype: int, group: int, bits: int, fma: bool = False):
    packed, scales, biases = _c(packed, np.uint32), _c(scales), _c(biases)
    last = packed.shape[-1] * 32 // bits
    out = np.zeros(packed.shape[:-1] + (last,), NP_OF[dtype])
    fn = lib().nvq_ref_affine_dequantize_fma if fma else lib().nvq_ref_affine_dequantize
    _check(fn(_p(packed), _p(scales), _p(biases), dtype, C.c_int64(out.size), group, bits, _p(out)),
           "affine_dequantize")
    return out


def fp_quantize(w: np.ndarray, dtype: int, mode: int, global_scale=None):
    """kernels.rs:914-971; `global_scale`: NVFP4's one float32 value (scales relative to g / (448 * 6))."""
    w = _c(w)
    group, bits = FP_PARAMS[mode]
    last = w.shape[-1]
    packed = np.zeros(w.shape[:-1] + (last * bits // 32,), np.uint32)
    scales = np.zeros(w.shape[:-1] + (last // group,), np.uint8)
    if global_scale is None:
        rc = lib().nvq_ref_fp_quantize(_p(w), dtype, C.c_int64(w.size), mode, _p(packed), _p(scales))
    else:
        rc = lib().nvq_ref_fp_quantize_scaled(_p(w), dtype, C.c_int64(w.size), mode, C.c_float(float(global_scale)),
                                              _p(packed), _p(scales))
    _check(rc, "fp_quantize")
    return packed, scales


def fp_dequantize(packed, scales, mode: int, out_dtype: int, global_scale=None):
    """kernels.rs:976-1009; `global_scale`: NVFP4's one float32 value."""
    packed, scales = _c(packed, np.uint32), _c(scales, np.uint8)
    _, bits = FP_PARAMS[mode]
    last = packed.shape[-1] * 32 // bits
    out = np.zeros(packed.shape[:-1] + (last,), NP_OF[out_dtype])
    if global_scale is None:
        rc = lib().nvq_ref_fp_dequantize(_p(packed), _p(scales), C.c_int64(out.size), mode, out_dtype, _p(out))
    else:
        rc = lib().nvq_ref_fp_dequantize_scaled(_p(packed), _p(scales), C.c_int64(out.size), mode, out_dtype,
                                                C.c_float(float(global_scale)), _p(out))
    _check(rc, "fp_dequantize")
    return out


def fp_quantize_dequantize(x, dtype: int, mode: int, global_scale=None):
    """kernels.rs:1011-1065: the values the quantization of `x` represents, in x's dtype (`qqmm`'s activations)."""
    x = _c(x)
    out = np.zeros(x.shape, NP_OF[dtype])
    if global_scale is None:
        rc = lib().nvq_ref_fp_quantize_dequantize(_p(x), dtype, C.c_int64(x.size), mode, _p(out))
    else:
        rc = lib().nvq_ref_fp_quantize_dequantize_scaled(_p(x), dtype, C.c_int64(x.size), mode, C.c_float(float(global_scale)), _p(out))
    _check(rc, "fp_quantize_dequantize")
    return out


def qqmm(x, w, dtype: int, mode: int, gx=None, gw=None):
    """products.rs:333-345, 354-367 (`qqmm` of a 2-D activation, forward): x through its quantization times the
    quantized weight, transposed.  `w` is the dense weight [N, K]; `gx`, `gw` NVFP4's global scales (both or neither)."""
    packed, scales = fp_quantize(w, dtype, mode, gw)
    xq = fp_quantize_dequantize(x, dtype, mode, gx)
    group, bits = FP_PARAMS[mode]
    if gw is None:
        return quantized_matmul(xq, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype)
    return fp_quantized_matmul_scaled(xq, packed, scales, mode, dtype, gw)


def gather_qqmm(x, w, rhs, dtype: int, mode: int, gx=None, gw=None):
    """products.rs:431-470: `gather_qmm` of the quantized activations x [B, M, K] with the quantized experts w [E, N, K],
    pair i against expert rhs[i]; the weight's one global scale serves every expert."""
    xq = fp_quantize_dequantize(x, dtype, mode, gx)
    return np.stack([qqmm_pair(xq[i], w[int(r)], dtype, mode, gw) for i, r in enumerate(np.asarray(rhs).reshape(-1))])


def qqmm_pair(xq, w, dtype: int, mode: int, gw=None):
    packed, scales = fp_quantize(w, dtype, mode, gw)
    group, bits = FP_PARAMS[mode]
    if gw is None:
        return quantized_matmul(xq, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype)
    return fp_quantized_matmul_scaled(xq, packed, scales, mode, dtype, gw)


def dense_matmul(x, dense, dtype: int, transpose: bool = True, threads: int = 1):
    """x [M, K] times an already dequantized float32 matrix ([N, K] if transpose else [K, N]), rounded once to
    `dtype`: the product step of kernels.rs:1112-1142 (weights dequantized with a global scale go this way)."""
    x, dense = _c(x), _c(dense, np.float32)
    M, K = x.shape
    N = dense.shape[0] if transpose else dense.shape[1]
    y = np.zeros((M, N), NP_OF[dtype])
    _check(lib().nvq_ref_dense_matmul(dtype, int(transpose), C.c_int64(M), C.c_int64(N), C.c_int64(K), _p(x), _p(dense),
                                      _p(y), threads), "dense_matmul")
    return y


def fp_quantized_matmul_scaled(x, packed, scales, mode: int, dtype: int, global_scale, transpose: bool = True):
    """quantized.rs:469-491 with a global scale: x . dequantize(w, float32, g)^T (or x . dequantize(w)), one rounding."""
    dense = fp_dequantize(packed, scales, mode, F32, global_scale)
    return dense_matmul(x, dense, dtype, transpose)


def sorted_offsets(indices: np.ndarray, groups: int) -> np.ndarray:
    indices = _c(indices, np.uint32)
    m = indices.shape[-1]
    rows = indices.size // max(m, 1)
    out = np.zeros(indices.shape[:-1] + (groups,), np.int32)
    _check(lib().nvq_ref_sorted_offsets(_p(indices), C.c_int64(rows), C.c_int64(m), groups, _p(out)),
           "sorted_offsets")
    return out


def quantized_matmul(x, w, scales, biases, *, mode=AFFINE, group=64, bits=4, dtype=F32, transpose=True,
                     threads=1):
    """x [batch..., M, K] (or [M, K]); w [N, Kp] shared or [batch..., N, Kp] matching x's batch."""
    x, w, scales = _c(x), _c(w, np.uint32), _c(scales)
    biases = None if biases is None else _c(biases)
    M, K = x.shape[-2], x.shape[-1]
    batch = int(np.prod(x.shape[:-2], dtype=np.int64))
    w_batch = int(np.prod(w.shape[:-2], dtype=np.int64)) if w.ndim > 2 else 1
    packed_cols = w.shape[-1] * 32 // bits
    N = w.shape[-2] if transpose else packed_cols
    y = np.zeros(x.shape[:-1] + (N,), NP_OF[dtype])
    _check(lib().nvq_ref_quantized_matmul(mode, group, bits, dtype, int(transpose), C.c_int64(batch),
                                          C.c_int64(M), C.c_int64(N), C.c_int64(K), C.c_int64(w_batch),
                                          _p(x), _p(w), _p(scales), _p(biases), _p(y), threads),
           "quantized_matmul")
    return y


def quantized_matmul_device(x, w, scales, biases, *, group=64, bits=4, dtype=F32, rounded_weights=True):
    """The affine product in the arithmetic of the reference's device kernels, which comes in two forms.
    rounded_weights=True, the tiled kernels: the weights are dequantized in the element type with ONE
    rounding of fma(code, scale, bias) (crates/nuvec-kernels/src/metal/quantized.h:583-817; the same
    values as `affine_dequantize(fma=True)`, which the reference's device fixtures pin bit for bit).
    rounded_weights=False, the vector kernels: scale * sum(x * code) + bias * sum(x) per group, the
    weights never rounded (quantized.h:1358-1485).  Either way the products accumulate wider than the
    element type (float64 here) and the sum is rounded once.  The CPU path differs in rounding the
    weights twice (crates/nuvec-core/src/kernels.rs:835-859).  x [M, K], w [N, Kp]."""
    x, w = _c(x), _c(w, np.uint32)
    if rounded_weights:
        wd = to_f32(affine_dequantize(w, scales, biases, dtype, group, bits, fma=True), dtype).astype(np.float64)
    else:
        codes = to_f32(affine_dequantize(w, np.ones_like(_c(scales), np.float32), np.zeros_like(_c(scales), np.float32),
                                         F32, group, bits), F32).astype(np.float64)
        s64 = np.repeat(to_f32(_c(scales), dtype).astype(np.float64), group, axis=-1)
        b64 = np.repeat(to_f32(_c(biases), dtype).astype(np.float64), group, axis=-1)
        wd = codes * s64 + b64
    y = to_f32(x, dtype).astype(np.float64) @ wd.T
    return from_f32(y.astype(np.float32), dtype)


def gather_qmm(x, w, scales, biases, lhs, rhs, *, mode=AFFINE, group=64, bits=4, dtype=F32, transpose=True,
               threads=1):
    """x [xb..., M, K]; w [e..., N, Kp]; lhs/rhs broadcast-equal integer arrays of one shape."""
    x, w, scales = _c(x), _c(w, np.uint32), _c(scales)
    biases = None if biases is None else _c(biases)
    lhs, rhs = _c(lhs, np.uint32), _c(rhs, np.uint32)
    M, K = x.shape[-2], x.shape[-1]
    xb = int(np.prod(x.shape[:-2], dtype=np.int64))
    experts = int(np.prod(w.shape[:-2], dtype=np.int64))
    packed_cols = w.shape[-1] * 32 // bits
    N = w.shape[-2] if transpose else packed_cols
    y = np.zeros(rhs.shape + (M, N), NP_OF[dtype])
    _check(lib().nvq_ref_gather_qmm(mode, group, bits, dtype, int(transpose), C.c_int64(rhs.size),
                                    C.c_int64(M), C.c_int64(N), C.c_int64(K), C.c_int64(xb),
                                    C.c_int64(experts), _p(x), _p(w), _p(scales), _p(biases), _p(lhs),
                                    _p(rhs), _p(y), threads), "gather_qmm")
    return y


def quantized_matmul_sample(x, w, scales, biases, rows, cols, *, mode=AFFINE, group=64, bits=4, dtype=F32):
    x, w, scales = _c(x), _c(w, np.uint32), _c(scales)
    biases = None if biases is None else _c(biases)
    rows, cols = _c(rows, np.int64), _c(cols, np.int64)
    M, K = x.shape
    N = w.shape[0]
    y = np.zeros(rows.shape, NP_OF[dtype])
    _check(lib().nvq_ref_quantized_matmul_sample(mode, group, bits, dtype, C.c_int64(M), C.c_int64(N),
                                                 C.c_int64(K), _p(x), _p(w), _p(scales), _p(biases),
                                                 C.c_int64(rows.size), _p(rows), _p(cols), _p(y)),
           "quantized_matmul_sample")
    return y
