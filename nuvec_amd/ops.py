"""The public quantization ops with nuvec's (MLX-compatible) signatures, on torch device tensors.

This is the host-side mirror of crates/nuvec-core/src/quantized.rs and ops.rs:965-1074:
same names, argument meaning and refusals.  torch supplies device memory and the stream;
every computation runs in libnuvec_hip.so through the C ABI.

    q = quantize(w, Quant.affine(64, 4))          # Quantized(weight u32, scales, biases)
    w2 = dequantize(q)                            # or q.dequantize(dtype)
    y = quantized_matmul(x, q, transpose=True)    # x . dequantize(w)^T
    y = gather_qmm(x, q, None, rhs, GatherQmm(sorted_indices=True))
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, replace
from enum import IntEnum
from typing import Optional

import torch

from . import _lib
from ._lib import InvalidArgument, Unsupported  # noqa: F401  (re-exported)


class QuantMode(IntEnum):
    """quantized.rs:22-35; `name` strings are MLX's."""
    AFFINE = _lib.AFFINE
    MXFP4 = _lib.MXFP4
    MXFP8 = _lib.MXFP8
    NVFP4 = _lib.NVFP4

    @property
    def mlx_name(self) -> str:
        return self.name.lower()

    @staticmethod
    def parse(s: str) -> "QuantMode":
        try:
            return {"affine": QuantMode.AFFINE, "mxfp4": QuantMode.MXFP4, "mxfp8": QuantMode.MXFP8,
                    "nvfp4": QuantMode.NVFP4}[s]
        except KeyError:
            raise InvalidArgument(f"invalid quantization mode '{s}' (affine, mxfp4, mxfp8 or nvfp4)") from None


_DEFAULTS = {QuantMode.AFFINE: (64, 4), QuantMode.MXFP4: (32, 4), QuantMode.MXFP8: (32, 8), QuantMode.NVFP4: (16, 4)}


_VALID: set = set()     # quantizations the library has accepted
_QUANT_C: dict = {}     # their C descriptors (read-only: descriptors that embed one copy it)
_READY: set = set()     # devices nvq_init has answered for


@dataclass(frozen=True)
class Quant:
    """quantized.rs:93-168: a mode, a group size and a bit width."""
    mode: QuantMode = QuantMode.AFFINE
    group_size: int = 64
    bits: int = 4

    @staticmethod
    def new(mode: QuantMode) -> "Quant":
        g, b = _DEFAULTS[QuantMode(mode)]
        return Quant(QuantMode(mode), g, b)

    @staticmethod
    def affine(group_size: int, bits: int) -> "Quant":
        return Quant(QuantMode.AFFINE, group_size, bits)

    def checked(self, op: str):
        """Quant::checked: raises InvalidArgument with the reference's message.  (A quantization that has passed is not
        asked about again: the library's answer depends on its three numbers alone.)"""
        if self not in _VALID:
            _lib.check(_lib.load().nvq_quant_check(C.byref(self._c()), op.encode()))
            _VALID.add(self)
        return self.group_size, self.bits

    def _c(self) -> _lib.QuantC:
        c = _QUANT_C.get(self)
        if c is None:
            c = _QUANT_C[self] = _lib.QuantC(int(self.mode), int(self.group_size), int(self.bits))
        return c


@dataclass
class Quantized:
    """quantized.rs:194-278: packed codes, scales, (affine) biases and how they were quantized."""
    weight: torch.Tensor
    scales: torch.Tensor
    biases: Optional[torch.Tensor]
    quant: Quant
    global_scale: Optional[torch.Tensor] = None  # NVFP4: one float32 value, or one per expert (`[E]`) of stacked experts

    def with_global_scale(self, global_scale: torch.Tensor) -> "Quantized":
        """quantized.rs:248-253."""
        return Quantized(self.weight, self.scales, self.biases, self.quant, global_scale)

    @staticmethod
    def affine(weight, scales, biases, group_size, bits) -> "Quantized":
        return Quantized(weight, scales, biases, Quant.affine(group_size, bits))

    @staticmethod
    def fp(weight, scales, mode) -> "Quantized":
        return Quantized(weight, scales, None, Quant.new(mode))

    def dequantize(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return dequantize(self, dtype)


@dataclass(frozen=True)
class GatherQmm:
    """quantized.rs:314-359."""
    transpose: bool = True
    sorted_indices: bool = False

    @staticmethod
    def groups(rows: int, experts: int, row_exact: bool = False) -> bool:
        return bool(_lib.load().nvq_gather_grouped(rows, experts, int(row_exact)))


_CODE = {torch.float16: _lib.F16, torch.bfloat16: _lib.BF16, torch.float32: _lib.F32}
_FLOATS = tuple(_CODE)


def _init(t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise _lib.NoDevice("operands must live on the GPU: this backend has no CPU path")
    index = t.device.index or 0
    if index not in _READY:
        _lib.check(_lib.load().nvq_init(index))
        _READY.add(index)


def _stream() -> C.c_void_p:
    """torch's current stream on the current device (the raw handle: `torch.cuda.current_stream()` builds a Python stream
    object per call, 8 of the 19 us a one-row product spent on the host)."""
    return C.c_void_p(torch._C._cuda_getCurrentRawStream(torch.cuda.current_device()))


def _ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    """The tensor's device address; NULL means "operand absent" in the C ABI, so an empty
    tensor (torch gives it address 0) is passed as a never-dereferenced aligned non-null value."""
    if t is None:
        return C.c_void_p(None)
    return C.c_void_p(t.data_ptr() or 16)


def _u32(t: torch.Tensor) -> torch.Tensor:
    return t.view(torch.uint32) if t.dtype == torch.int32 else t


def _name(dtype) -> str:
    return str(dtype).replace("torch.", "")


def _check_groups(op: str, mode: QuantMode, scales: torch.Tensor, biases) -> None:
    """quantized.rs:363-379."""
    if mode == QuantMode.AFFINE:
        if biases is None:
            raise InvalidArgument(f"{op}: biases must be provided for affine quantization")
    elif biases is not None:
        raise InvalidArgument(f"{op}: biases must be null for quantization mode '{mode.mlx_name}'")
    elif scales.dtype != torch.uint8:
        raise InvalidArgument(f"{op}: scale type must be uint8 but received type {_name(scales.dtype)}")


def _quantized_columns(op: str, w, scales, biases, quant: Quant) -> int:
    """primitive.rs:1412-1460: values per packed row, after MLX's validate_quantized_input."""
    group, bits = quant.checked(op)
    w = _u32(w)
    if w.dtype != torch.uint32:
        raise InvalidArgument(f"{op}: packed weights must be uint32, got {_name(w.dtype)}")
    if quant.mode == QuantMode.AFFINE:
        if scales.dtype not in _FLOATS or biases.dtype != scales.dtype or biases.shape != scales.shape:
            raise InvalidArgument(
                f"{op}: scales and biases must share a float dtype and shape, got {_name(scales.dtype)} "
                f"{list(scales.shape)} and {_name(biases.dtype)} {list(biases.shape)}")
    elif scales.dtype != torch.uint8:
        raise InvalidArgument(f"{op}: scale type must be uint8 but received type {_name(scales.dtype)}")
    packed = (w.shape[-1] if w.ndim else 0) * 32
    groups = (scales.shape[-1] if scales.ndim else 0) * group
    if w.ndim < 2 or scales.ndim != w.ndim or w.shape[:-1] != scales.shape[:-1] or packed != groups * bits:
        raise InvalidArgument(f"{op}: packed weights {list(w.shape)} and scales {list(scales.shape)} do not match "
                              f"group size {group} and {bits} bits")
    return groups


def _global_scale(op: str, quant: Quant, g: Optional[torch.Tensor], device) -> Optional[torch.Tensor]:
    """primitive.rs:1378-1395 (MLX's `validate_global_scale`): NVFP4 only, one float32 value."""
    if g is None:
        return None
    if quant.mode != QuantMode.NVFP4:
        raise InvalidArgument(f"{op}: a global scale is only supported for nvfp4, got {quant.mode.mlx_name}")
    if g.numel() != 1 or g.dtype != torch.float32:
        raise InvalidArgument(f"{op}: the global scale must be one float32 value, got {_name(g.dtype)} {list(g.shape)}")
    return g.to(device).contiguous()


def quantize(w: torch.Tensor, quant: Quant | QuantMode = Quant(), global_scale: Optional[torch.Tensor] = None) -> Quantized:
    """ops.rs:965-1008 (`quantize`, `quantize_scaled`), primitive.rs:1223-1259: quantizes the last axis of `w`; with
    NVFP4's `global_scale` the group scales are relative to it, g / (448 * 6), and the result carries it."""
    quant = Quant.new(quant) if isinstance(quant, QuantMode) else quant
    group, bits = quant.checked("quantize")
    if w.dtype not in _FLOATS:
        raise InvalidArgument(f"quantize: unsupported dtype {_name(w.dtype)}")
    if w.ndim < 2 or w.shape[-1] % group != 0:
        raise InvalidArgument(f"quantize: needs at least 2 dimensions with the last divisible by the group size "
                              f"{group}, got shape {list(w.shape)}")
    _init(w)
    w = w.contiguous()
    last = w.shape[-1]
    rows = w.numel() // last if last else 0
    packed = torch.empty(w.shape[:-1] + (last * bits // 32,), dtype=torch.uint32, device=w.device)
    affine = quant.mode == QuantMode.AFFINE
    scales = torch.empty(w.shape[:-1] + (last // group,), dtype=w.dtype if affine else torch.uint8, device=w.device)
    biases = torch.empty_like(scales) if affine else None
    g = _global_scale("quantize", quant, global_scale, w.device)
    if g is not None:
        _lib.check(_lib.load().nvq_quantize_scaled(C.byref(quant._c()), _CODE[w.dtype], _ptr(w), rows, last, _ptr(g), _ptr(packed),
                                                   _ptr(scales), _stream()))
        return Quantized(packed, scales, None, quant, global_scale)
    _lib.check(_lib.load().nvq_quantize(C.byref(quant._c()), _CODE[w.dtype], _ptr(w), rows, last, _ptr(packed),
                                        _ptr(scales), _ptr(biases), _stream()))
    return Quantized(packed, scales, biases, quant)


def dequantize(q: Quantized, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """ops.rs:1014-1027, quantized.rs:401-444: affine computes in the scales' dtype, then casts;
    the floating-point modes default to bfloat16."""
    quant = q.quant
    quant.checked("dequantize")
    _check_groups("dequantize", quant.mode, q.scales, q.biases)
    if dtype is not None and not dtype.is_floating_point:
        raise InvalidArgument(f"dequantize: only real floating types are supported but the output dtype is {_name(dtype)}")
    affine = quant.mode == QuantMode.AFFINE
    cols = _quantized_columns("dequantize", q.weight, q.scales, q.biases, quant)
    compute = q.scales.dtype if affine else (dtype or torch.bfloat16)
    if compute not in _FLOATS:
        raise InvalidArgument(f"dequantize: unsupported dtype {_name(compute)}")
    _init(q.weight)
    w, s = _u32(q.weight).contiguous(), q.scales.contiguous()
    b = q.biases.contiguous() if affine else None
    out = torch.empty(w.shape[:-1] + (cols,), dtype=compute, device=w.device)
    rows = out.numel() // cols if cols else 0
    g = _global_scale("dequantize", quant, q.global_scale, w.device)
    if g is not None:
        _lib.check(_lib.load().nvq_dequantize_scaled(C.byref(quant._c()), _CODE[compute], _ptr(w), _ptr(s), _ptr(g), rows, cols,
                                                     _ptr(out), _stream()))
        return out
    _lib.check(_lib.load().nvq_dequantize(C.byref(quant._c()), _CODE[compute], _ptr(w), _ptr(s), _ptr(b), rows, cols,
                                          _ptr(out), _stream()))
    if affine and dtype is not None and dtype != out.dtype:
        out = out.to(dtype)
    return out


def quantize_dequantize(x: torch.Tensor, quant: Quant | QuantMode, global_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """products.rs:307-315 (`fake_quant`, MLX's `fp_quantize_dequantize`): `x` through its quantization in a
    floating-point mode, in x's dtype."""
    quant = Quant.new(quant) if isinstance(quant, QuantMode) else quant
    group, _ = quant.checked("quantize_dequantize")
    if quant.mode == QuantMode.AFFINE:
        raise InvalidArgument("quantize_dequantize: mode affine is not a floating-point block format")
    if x.dtype not in _FLOATS:
        raise InvalidArgument(f"quantize_dequantize: unsupported dtype {_name(x.dtype)}")
    if x.ndim < 1 or x.shape[-1] % group != 0:
        raise InvalidArgument(f"quantize_dequantize: the last dimension of {list(x.shape)} is not whole groups of {group}")
    _init(x)
    x = x.contiguous()
    g = _global_scale("quantize_dequantize", quant, global_scale, x.device)
    out = torch.empty_like(x)
    last = x.shape[-1]
    _lib.check(_lib.load().nvq_quantize_dequantize(C.byref(quant._c()), _CODE[x.dtype], _ptr(x), x.numel() // last if last else 0, last,
                                                   _ptr(g), _ptr(out), _stream()))
    return out


def _qq_weight(op: str, w, quant, global_scale_x):
    """products.rs:317-330, 431-462: the weight of `qqmm` / `gather_qqmm` as a `Quantized` in a floating-point mode (a
    dense weight is quantized for the product), and MLX's rule: NVFP4 global scales for both operands or neither."""
    if isinstance(w, Quantized):
        q = w
    else:
        quant = Quant.new(quant) if isinstance(quant, QuantMode) else quant
        if quant is None:
            raise InvalidArgument(f"{op}: a dense weight needs the mode to quantize it in")
        q = quantize(w, quant)
    if q.quant.mode == QuantMode.AFFINE:
        raise InvalidArgument(f"{op}: both operands are quantized in a floating-point mode, got affine")
    if (global_scale_x is None) != (q.global_scale is None):
        raise InvalidArgument(f"{op}: for nvfp4, give global scales for both the activations and the weight, or neither")
    return q


def qqmm(x: torch.Tensor, w, quant=None, global_scale_x: Optional[torch.Tensor] = None) -> torch.Tensor:
    """products.rs:333-429 (MLX's `qqmm`, forward): `x` (`[..., K]`) times `w^T` (`[N, K]`) with both quantized in a
    floating-point mode.  `w` is a `Quantized` or a dense weight (quantized here in `quant`; with NVFP4 global scales
    pass `quantize(w, NVFP4, gw)`)."""
    q = _qq_weight("qqmm", w, quant, global_scale_x)
    if x.ndim == 0:
        raise InvalidArgument("qqmm: the activation needs at least one dimension")
    x2 = x.reshape(-1, x.shape[-1])
    y = quantized_matmul(quantize_dequantize(x2, q.quant, global_scale_x), q, True)
    return y.reshape(x.shape[:-1] + (y.shape[-1],))


def gather_qqmm(x: torch.Tensor, w, lhs_indices=None, rhs_indices=None, sorted_indices: bool = False, quant=None,
                global_scale_x: Optional[torch.Tensor] = None) -> torch.Tensor:
    """products.rs:431-470 (MLX's `gather_qqmm`): `gather_qmm` of the quantized activations with quantized experts
    (`w [E, N, K]`), transposed; the weight's one global scale serves every expert."""
    q = _qq_weight("gather_qqmm", w, quant, global_scale_x)
    if q.global_scale is not None and q.global_scale.numel() == 1:
        q = q.with_global_scale(q.global_scale.reshape(()).expand(q.weight.shape[:-2]).contiguous())
    xq = quantize_dequantize(x, q.quant, global_scale_x)
    return gather_qmm(xq, q, lhs_indices, rhs_indices, GatherQmm(True, sorted_indices))


def embedding(q: Quantized, ids: torch.Tensor, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """nuvec-nn layers.rs:245-255 (`QuantizedEmbedding::forward`): the rows `ids` of a quantized table,
    dequantized; shape `ids.shape + [cols]`.  Equals `dequantize` of the taken rows bit for bit."""
    op = "dequantize_rows"
    quant = q.quant
    quant.checked(op)
    _check_groups(op, quant.mode, q.scales, q.biases)
    if q.weight.ndim != 2:
        raise InvalidArgument(f"{op}: the table must be two-dimensional, got {list(q.weight.shape)}")
    if ids.dtype.is_floating_point or ids.dtype == torch.bool:
        raise InvalidArgument(f"{op}: ids must be integers, got {_name(ids.dtype)}")
    affine = quant.mode == QuantMode.AFFINE
    cols = _quantized_columns(op, q.weight, q.scales, q.biases, quant)
    compute = q.scales.dtype if affine else (dtype or torch.bfloat16)
    if compute not in _FLOATS:
        raise InvalidArgument(f"{op}: unsupported dtype {_name(compute)}")
    _init(q.weight)
    w, s = _u32(q.weight).contiguous(), q.scales.contiguous()
    b = q.biases.contiguous() if affine else None
    flat = ids.reshape(-1) if ids.dtype == torch.uint32 else ids.reshape(-1).to(torch.int32).view(torch.uint32)
    flat = flat.contiguous()
    out = torch.empty(tuple(ids.shape) + (cols,), dtype=compute, device=w.device)
    _lib.check(_lib.load().nvq_dequantize_rows(C.byref(quant._c()), _CODE[compute], _ptr(w), _ptr(s), _ptr(b), w.shape[0], cols,
                                               _ptr(flat), flat.numel(), _ptr(out), _stream()))
    if affine and dtype is not None and dtype != out.dtype:
        out = out.to(dtype)
    return out


def _promoted(op: str, x, scales, biases) -> torch.dtype:
    """quantized.rs:491-497: affine promotes x, scales and biases; fp modes keep x's dtype."""
    dtype = x.dtype
    if biases is not None:
        dtype = torch.promote_types(torch.promote_types(x.dtype, scales.dtype), biases.dtype)
    if dtype not in _FLOATS:
        raise InvalidArgument(f"{op}: unsupported dtype {_name(dtype)}")
    return dtype


def _strides(t: torch.Tensor, nbatch: int):
    return [int(t.stride(i)) for i in range(nbatch)]


def quantized_matmul(x: torch.Tensor, q: Quantized, transpose: bool = True, *, row_exact: bool = False, rows: bool = False,
                     scratch: bool = True, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ops.rs:1031-1045, quantized.rs:446-537, primitive.rs:1279-1320.  `row_exact` and `rows` are the primitive's
    routing flags (primitive.rs:489-493; `with_row_exact`, lib.rs:159-193).  `scratch=False` hands the library no
    workspace (a transposed product then runs without splitting K).  `bias` ([N], the product's dtype) is added in the
    kernels' epilogues as `QuantizedLinear::forward` adds it (layers.rs:155-162)."""
    op = "quantized_matmul"
    quant = q.quant
    group, bits = quant.checked(op)
    _check_groups(op, quant.mode, q.scales, q.biases)
    g = _global_scale(op, quant, q.global_scale, x.device)
    if g is not None and (q.weight.ndim > 2 or x.ndim > 2 or not transpose):
        # quantized.rs:481-491: only x [M, K] times transposed w [N, K'] reaches a kernel with a global scale; the
        # reference dequantizes in x's type and multiplies densely otherwise.
        dense = dequantize(q, x.dtype)
        return x.matmul(dense.transpose(-1, -2) if transpose else dense)
    affine = quant.mode == QuantMode.AFFINE
    dtype = _promoted(op, x, q.scales, q.biases)
    x = x.to(dtype)
    w = _u32(q.weight)
    scales = q.scales.to(dtype) if affine else q.scales
    biases = q.biases.to(dtype) if affine else None
    vector = x.ndim == 1
    if vector:
        x = x.unsqueeze(0)
    columns = _quantized_columns(op, w, scales, biases, quant)
    w_rows = w.shape[-2]
    inner, outer = (columns, w_rows) if transpose else (w_rows, columns)
    # Dense last two dimensions for every operand; batch dimensions broadcast by stride 0.
    x, w, scales = x.contiguous(), w.contiguous(), scales.contiguous()
    biases = biases.contiguous() if affine else None
    if w.ndim > 2 and x.ndim >= 2:
        try:
            batch = torch.broadcast_shapes(x.shape[:-2], w.shape[:-2])
        except RuntimeError:
            raise InvalidArgument(f"{op}: shapes {list(x.shape)} and {list(w.shape)} do not broadcast") from None
        full = lambda a: a.expand(batch + a.shape[-2:])
        x, w, scales = full(x), full(w), full(scales)
        biases = full(biases) if affine else None
    xn, wn = x.ndim, w.ndim
    batch_ok = wn == 2 or (xn == wn and x.shape[:-2] == w.shape[:-2])
    if xn == 0 or x.shape[-1] != inner or not batch_ok:
        raise InvalidArgument(f"{op}: shapes {list(x.shape)} and {list(w.shape)} do not match")
    _init(x)
    out = torch.empty(x.shape[:-1] + (outer,), dtype=dtype, device=x.device)
    d = _lib.QmmDescC()
    d.quant, d.dtype, d.transpose, d.row_exact, d.rows = quant._c(), _CODE[dtype], int(transpose), int(row_exact), int(rows)
    d.n, d.k = outer, inner
    if wn == 2:  # the reference's "flat" rule: every leading row of x is a row of one product
        d.m = 1
        for dim in x.shape[:-1]:
            d.m *= dim
        d.item_rows = x.shape[-2]
        d.batch_ndim = 0
    else:
        d.m = d.item_rows = x.shape[-2]
        nb = xn - 2
        if nb > _lib.MAX_BATCH_DIMS:
            raise Unsupported(f"{op}: {nb} batch dimensions")
        d.batch_ndim = nb
        for i in range(nb):
            d.batch_shape[i] = x.shape[i]
            d.x_strides[i], d.w_strides[i], d.s_strides[i] = x.stride(i), w.stride(i), scales.stride(i)
    lib = _lib.load()
    need = lib.nvq_quantized_matmul_workspace_bytes(C.byref(d))
    workspace = torch.empty(need, dtype=torch.uint8, device=x.device) if need and scratch else None
    if bias is not None:
        if g is not None or bias.dtype != dtype or bias.ndim != 1 or bias.shape[0] != outer:
            raise InvalidArgument(f"{op}: the fused bias must be [{outer}] of {_name(dtype)} and the mode without a global scale")
        bias = bias.contiguous()
        _lib.check(lib.nvq_quantized_linear(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(bias), _ptr(out),
                                            _ptr(workspace), _stream()))
    elif g is not None:
        _lib.check(lib.nvq_quantized_matmul_scaled(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(g), _ptr(out),
                                                   _ptr(workspace), _stream()))
    else:
        _lib.check(lib.nvq_quantized_matmul(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(out),
                                            _ptr(workspace), _stream()))
    return out.squeeze(-2) if vector else out


def quantized_matmul_route(m: int, n: int, k: int, quant: Quant, dtype: torch.dtype, *, batch=1, transpose: bool = True,
                           row_exact: bool = False, rows: bool = False, device: int = 0) -> str:
    """The kernel a product of `m` rows of x per item ([.., m, k] times `batch` weight matrices [n, k] — a count or a
    tuple of batch dimensions —, or one matrix when `batch` is 1) runs on, from the library's own routing code: what the reference's tests read from the kernel
    names (tests/quantized.rs:843-861)."""
    _lib.check(_lib.load().nvq_init(device))
    d = _lib.QmmDescC()
    d.quant, d.dtype, d.transpose, d.row_exact, d.rows = quant._c(), _CODE[dtype], int(transpose), int(row_exact), int(rows)
    d.m = d.item_rows = m
    d.n, d.k = n, k
    dims = () if batch == 1 else tuple(batch) if isinstance(batch, (tuple, list)) else (batch,)
    d.batch_ndim = len(dims)
    items = 1
    for i in reversed(range(len(dims))):  # dense operands
        d.batch_shape[i] = dims[i]
        d.x_strides[i], d.w_strides[i], d.s_strides[i] = items * m * k, items * n * k * quant.bits // 32, items * n * k // quant.group_size
        items *= dims[i]
    name = _lib.load().nvq_quantized_matmul_route(C.byref(d))
    if name is None:
        raise Unsupported(_lib.last_error())
    return name.decode()


def quantized_attention_fits(q: torch.Tensor, k: Quantized, v: Quantized, sinks: Optional[torch.Tensor] = None) -> bool:
    """fast/imp.rs:3944-3992: whether the fused kernel takes these operands (else the composition)."""
    if q.ndim != 4 or k.weight.ndim != 4 or v.weight.ndim != 4 or k.quant != v.quant or k.quant.mode != QuantMode.AFFINE:
        return False
    b, hq, l, d = q.shape
    group, bits = k.quant.group_size, k.quant.bits
    if q.dtype not in _FLOATS or l != 1 or d not in (64, 128) or bits not in (3, 4, 8) or group not in (32, 64, 128) or d % group:
        return False
    hkv, n = k.weight.shape[1], k.weight.shape[2]
    for t in (k, v):
        if t.biases is None or t.weight.dtype != torch.uint32 or tuple(t.weight.shape) != (b, hkv, n, d * bits // 32):
            return False
        if tuple(t.scales.shape) != (b, hkv, n, d // group) or t.biases.shape != t.scales.shape:
            return False
        if t.scales.dtype != q.dtype or t.biases.dtype != q.dtype:
            return False
    if hkv == 0 or n < 1 or hq % hkv or hq // hkv not in (1, 2, 4, 8):
        return False
    if b > 65535 or b * hkv * n * d >= 1 << 31:  # the kernel's grid and 32-bit cache offsets
        return False
    return sinks is None or (sinks.ndim == 1 and sinks.numel() == hq and sinks.dtype == q.dtype)


def quantized_attention(q: torch.Tensor, k: Quantized, v: Quantized, scale: float,
                        sinks: Optional[torch.Tensor] = None, scratch: bool = True) -> torch.Tensor:
    """fast.rs:694-718 where the kernel fits (`quantized_attention_fits`): one query row per head over the quantized
    cache in one launch."""
    if not quantized_attention_fits(q, k, v, sinks):
        raise Unsupported("quantized_attention: the operands do not fit the kernel")
    _init(q)
    b, hq, _, d = q.shape
    q = q.contiguous()
    kw, ks, kb = _u32(k.weight).contiguous(), k.scales.contiguous(), k.biases.contiguous()
    vw, vs, vb = _u32(v.weight).contiguous(), v.scales.contiguous(), v.biases.contiguous()
    sinks = None if sinks is None else sinks.contiguous()
    out = torch.empty_like(q)
    desc = _lib.AttentionDescC(_CODE[q.dtype], k.quant.bits, k.quant.group_size, d, b, hq, kw.shape[1], kw.shape[2], float(scale))
    lib = _lib.load()
    need = lib.nvq_quantized_attention_workspace_bytes(C.byref(desc)) if scratch else 0
    workspace = torch.empty(need, dtype=torch.uint8, device=q.device) if need else None
    _lib.check(lib.nvq_quantized_attention(C.byref(desc), _ptr(q), _ptr(kw), _ptr(ks), _ptr(kb), _ptr(vw), _ptr(vs), _ptr(vb),
                                           _ptr(sinks), _ptr(out), _ptr(workspace), _stream()))
    return out


def sorted_offsets(rhs: torch.Tensor, groups: int) -> torch.Tensor:
    """kernels.rs:873-892: per row of the last axis, where each group's indices start."""
    _init(rhs)
    rhs = rhs.contiguous()
    m = rhs.shape[-1]
    rows = rhs.numel() // m if m else 0
    out = torch.empty(rhs.shape[:-1] + (groups,), dtype=torch.int32, device=rhs.device)
    _lib.check(_lib.load().nvq_sorted_offsets(_ptr(rhs), rows, m, groups, _ptr(out), _stream()))
    return out


def moe_order(expert_ids: torch.Tensor, experts: int):
    """nuvec-lm model.rs:2193-2210 (`SwitchGlu::forward`): the flattened pairs (token, choice) ordered by expert.
    Returns `(order, restore, sorted_ids, offsets)`: `order = argsort(ids)` (stable), `restore = argsort(order)`,
    `sorted_ids = ids[order]` and `offsets = sorted_offsets(sorted_ids, experts)`, from one kernel."""
    if expert_ids.dtype.is_floating_point or expert_ids.dtype == torch.bool:
        raise InvalidArgument("moe_order: expert ids must be integers")
    _init(expert_ids)
    ids = expert_ids.reshape(-1)
    ids = (ids if ids.dtype == torch.uint32 else ids.to(torch.int32)).contiguous()
    pairs = ids.numel()
    order = torch.empty(pairs, dtype=torch.int32, device=ids.device)
    restore, sorted_ids = torch.empty_like(order), torch.empty_like(order)
    offsets = torch.empty(experts, dtype=torch.int32, device=ids.device)
    lib = _lib.load()
    need = lib.nvq_moe_order_workspace_bytes(pairs, experts)
    workspace = torch.empty(need, dtype=torch.uint8, device=ids.device) if need else None
    _lib.check(lib.nvq_moe_order(_ptr(ids), pairs, experts, _ptr(order), _ptr(restore), _ptr(sorted_ids), _ptr(offsets),
                                 _ptr(workspace), _stream()))
    return order, restore, sorted_ids, offsets


def moe_route(probs: torch.Tensor, k: int, normalize: bool):
    """fast.rs:740-746 (`fast::moe_route`): per row of router probabilities `[..., E]` the `k` largest in the stable
    ascending order of the sort (the last `k` of `argsort`; NaN last for float32 and half), as int32 `[..., k]`, and
    their values (divided by their sum in the probabilities' type, in order, with `normalize`) `[..., k]`."""
    if probs.dtype not in _CODE:
        raise InvalidArgument(f"moe_route: probabilities must be floating point, got {probs.dtype}")
    e = probs.shape[-1] if probs.ndim else 0
    if not isinstance(k, int) or not 1 <= k <= e:
        raise InvalidArgument(f"moe_route: k must be in 1..={e} for probabilities of shape {list(probs.shape)}")
    _init(probs)
    p = probs.contiguous()
    rows = p.numel() // e
    top = torch.empty(p.shape[:-1] + (k,), dtype=torch.int32, device=p.device)
    scores = torch.empty(p.shape[:-1] + (k,), dtype=p.dtype, device=p.device)
    _lib.check(_lib.load().nvq_moe_route(_CODE[p.dtype], _ptr(p), rows, e, k, int(bool(normalize)), _ptr(top), _ptr(scores), _stream()))
    return top, scores


def weighted_sum(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """fast.rs (`fast::weighted_sum`, fast/imp.rs:2731-2747): `sum(x * w[..., None], -2)` over `x [..., k, D]` and
    `w [..., k]` of one floating-point type, every product and addition rounded to that type in the kernel's order."""
    if x.ndim < 2 or tuple(w.shape) != tuple(x.shape[:-1]):
        raise InvalidArgument(f"weighted_sum: x must be [..., k, D] and w [..., k], got {list(x.shape)} and {list(w.shape)}")
    if x.dtype not in _CODE or w.dtype != x.dtype:
        raise Unsupported(f"weighted_sum: x and w must share a floating-point type, got {x.dtype} and {w.dtype}")
    _init(x)
    x, w = x.contiguous(), w.contiguous()
    k, d = x.shape[-2], x.shape[-1]
    rows = w.numel() // k if k else 0
    out = torch.empty(x.shape[:-2] + (d,), dtype=x.dtype, device=x.device)
    _lib.check(_lib.load().nvq_weighted_sum(_CODE[x.dtype], _ptr(x), _ptr(w), rows, k, d, _ptr(out), _stream()))
    return out


GLU_ACTIVATIONS = {"swiglu": 0, "swiglu_oai": 1, "geglu": 2}


def glu(gate: torch.Tensor, up: torch.Tensor, activation: str = "swiglu", *, alpha: float = 1.702, limit: float = 7.0,
        gate_bias: Optional[torch.Tensor] = None, up_bias: Optional[torch.Tensor] = None,
        ids: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The experts' gated activation (`SwitchGlu::through`, model.rs:2157-2170): `swiglu` is nuvec-nn's
    `silu(gate) * up` (lib.rs:513-519), `swiglu_oai` gpt-oss's clamped form (lib.rs:564-570), every operation rounded
    to the activations' type in the reference's order.  `gate` and `up` are `[..., hidden]` with unit stride along
    the last axis and one stride between rows (views of the two halves of one fused product serve); with `gate_bias`
    and `up_bias` (`[experts, hidden]`) and `ids` (one expert per row) each row's expert's biases are added first
    (model.rs:2139-2143)."""
    if activation not in GLU_ACTIVATIONS:
        raise InvalidArgument(f"glu: unknown activation {activation!r}")
    if gate.dtype not in _CODE or up.dtype != gate.dtype or gate.shape != up.shape or gate.ndim < 1:
        raise InvalidArgument(f"glu: gate and up must share a floating-point type and a shape, got {gate.dtype} {list(gate.shape)} "
                              f"and {up.dtype} {list(up.shape)}")
    _init(gate)
    hidden = gate.shape[-1]
    rows = gate.numel() // hidden if hidden else 0

    def as_rows(t):  # [rows, hidden] with unit stride along the columns and one stride between the rows; a copy only if needed
        t2 = t.reshape(rows, hidden)
        ok = hidden <= 1 or t2.stride(1) == 1
        if rows > 1 and hidden > 0:
            ok = ok and t2.stride(0) >= hidden
        return t2 if ok else t2.contiguous()
    g2, u2 = as_rows(gate), as_rows(up)
    d = _lib.GluDescC(_CODE[gate.dtype], GLU_ACTIVATIONS[activation], float(alpha), float(limit), rows, hidden,
                      g2.stride(0) if rows > 1 else hidden, u2.stride(0) if rows > 1 else hidden, 0)
    gb = ub = idp = None
    if (gate_bias is None) != (up_bias is None):
        raise InvalidArgument("glu: one bias without the other")
    if gate_bias is not None:
        if ids is None or ids.numel() != rows or ids.dtype.is_floating_point:
            raise InvalidArgument("glu: biases need one integer expert id per row")
        if gate_bias.dtype != gate.dtype or up_bias.dtype != gate.dtype or gate_bias.ndim != 2 or gate_bias.shape != up_bias.shape \
                or gate_bias.shape[1] != hidden:
            raise InvalidArgument(f"glu: biases must be [experts, {hidden}] of {gate.dtype}")
        gb, ub = gate_bias.contiguous(), up_bias.contiguous()
        idp = ids.reshape(-1).to(torch.int32).contiguous()
        d.experts = gb.shape[0]
    out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    _lib.check(_lib.load().nvq_glu(C.byref(d), _ptr(g2), _ptr(u2), _ptr(gb), _ptr(ub), _ptr(idp), _ptr(out), _stream()))
    return out


def _out_rows(op: str, given: Optional[torch.Tensor], pairs: int, device) -> Optional[torch.Tensor]:
    """Where each pair's result goes (`nvq_gather_qmm_scatter`): one integer per pair, a permutation of the pairs."""
    if given is None:
        return None
    if given.dtype.is_floating_point or given.dtype == torch.bool:
        raise InvalidArgument(f"{op}: output rows must be integers")
    if given.numel() != pairs:
        raise InvalidArgument(f"{op}: {given.numel()} output rows for {pairs} pairs")
    given = given.to(device).reshape(-1)
    return (given.to(torch.int32) if given.dtype != torch.uint32 else given.view(torch.int32)).contiguous()


def gather_qmm_grouped(x: torch.Tensor, q: Quantized, rows: torch.Tensor, sorted_ids: torch.Tensor,
                       offsets: torch.Tensor, out_rows: Optional[torch.Tensor] = None,
                       expert_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The grouped route of `gather_qmm` (quantized.rs:646-651, 772-782) with the rows of x taken inside the kernel:
    output row i = x[rows[i]] . dequantize(w)[sorted_ids[i]]^T for ids sorted by expert (`offsets` from `moe_order`
    or `sorted_offsets`).  Equal to `gather_qmm(x[rows], q, None, sorted_ids, sorted)`; the gathered copy of x is
    never written.  x is `[T, K]`, the result `[len(rows), N]`.  With `out_rows` (a permutation, e.g. the `order` of
    `moe_order`) result row i is written at row `out_rows[i]`: the ordered product lands in pair order and
    model.rs:2205-2210's `take(out, inverse)` is not needed.  `expert_bias` `[E, N]` adds each row's expert's bias
    (model.rs:2139-2143) in the kernel's epilogue (`Unsupported` where the grouped kernel does not take the product).
    NVFP4 experts carry their global scales (`q.global_scale`, one per expert)."""
    op = "gather_qmm"
    quant = q.quant
    quant.checked(op)
    _check_groups(op, quant.mode, q.scales, q.biases)
    affine = quant.mode == QuantMode.AFFINE
    dtype = _promoted(op, x, q.scales, q.biases)
    w = _u32(q.weight).contiguous()
    if x.ndim != 2 or w.ndim != 3:
        raise InvalidArgument(f"{op}: x must be [T, K] and w [E, N, K'], got {list(x.shape)} and {list(w.shape)}")
    x = x.to(dtype).contiguous()
    scales = (q.scales.to(dtype) if affine else q.scales).contiguous()
    biases = q.biases.to(dtype).contiguous() if affine else None
    columns = _quantized_columns(op, w, scales, biases, quant)
    if x.shape[-1] != columns:
        raise InvalidArgument(f"{op}: shapes {list(x.shape)} and {list(w.shape)} do not match")
    _init(x)
    lhs, rhs = _indices(op, x, rows.reshape(-1)).contiguous(), _indices(op, w, sorted_ids.reshape(-1)).contiguous()
    if lhs.numel() != rhs.numel() or offsets.numel() != w.shape[0] or offsets.dtype != torch.int32:
        raise InvalidArgument(f"{op}: {lhs.numel()} rows, {rhs.numel()} expert ids, {offsets.numel()} offsets for {w.shape[0]} experts")
    out = torch.empty((rhs.numel(), w.shape[-2]), dtype=dtype, device=x.device)
    d = _lib.GatherDescC(quant._c(), _CODE[dtype], 1, 0, 0, 1, w.shape[-2], columns, rhs.numel(), x.shape[0], w.shape[0])
    scatter = _out_rows(op, out_rows, rhs.numel(), x.device)
    gs = q.global_scale
    if gs is not None:  # quantized.rs:620-636
        if quant.mode != QuantMode.NVFP4:
            raise InvalidArgument(f"{op}: global scale is only supported for 'nvfp4' quantization mode")
        if gs.dtype != torch.float32 or gs.numel() != w.shape[0]:
            raise InvalidArgument(f"{op}: global scale must be float32 with one entry per expert, got {_name(gs.dtype)} {list(gs.shape)}")
        gs = gs.to(x.device).contiguous()
    if expert_bias is not None and (expert_bias.dtype != dtype or tuple(expert_bias.shape) != (w.shape[0], w.shape[-2])):
        raise InvalidArgument(f"{op}: the experts' bias must be [{w.shape[0]}, {w.shape[-2]}] of {_name(dtype)}")
    if expert_bias is not None or gs is not None:  # the entry point with every optional operand
        eb = expert_bias.contiguous() if expert_bias is not None else None
        _lib.check(_lib.load().nvq_gather_qmm_expert_bias(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(gs),
                                                          _ptr(lhs), _ptr(rhs), _ptr(offsets.contiguous()), _ptr(scatter),
                                                          _ptr(eb), _ptr(out), _ptr(None), _stream()))
        return out
    if scatter is not None:
        _lib.check(_lib.load().nvq_gather_qmm_scatter(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(gs),
                                                      _ptr(lhs), _ptr(rhs), _ptr(offsets.contiguous()), _ptr(scatter),
                                                      _ptr(out), _ptr(None), _stream()))
        return out
    _lib.check(_lib.load().nvq_gather_qmm(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(lhs), _ptr(rhs),
                                          _ptr(offsets.contiguous()), _ptr(out), _ptr(None), _stream()))
    return out


def gather_qmm_glu(x: torch.Tensor, q: Quantized, rows: torch.Tensor, sorted_ids: torch.Tensor, offsets: Optional[torch.Tensor],
                   activation: str = "swiglu", *, alpha: float = 1.702, limit: float = 7.0,
                   expert_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`gather_qmm_grouped` of the experts' gate and up projections with `glu` as the kernel's epilogue
    (`SwitchGlu::through` up to the down projection, model.rs:2157-2169): `q` (and `expert_bias` `[E, N]`) hold both
    projections in alternating runs of 64 rows (`pair_rows`), the result is `[len(rows), N / 2]`, bit for bit
    `glu(gate, up, ...)` of the two products.  `offsets` None: the ids are in any order (the few pairs of decoded
    tokens) and every pair runs on the decode kernel, with the same epilogue.  Raises `Unsupported` where the grouped
    kernel (the decode kernel) does not take the product."""
    op = "gather_qmm"
    if activation not in GLU_ACTIVATIONS:
        raise InvalidArgument(f"{op}: unknown activation {activation!r}")
    quant = q.quant
    quant.checked(op)
    _check_groups(op, quant.mode, q.scales, q.biases)
    affine = quant.mode == QuantMode.AFFINE
    dtype = _promoted(op, x, q.scales, q.biases)
    w = _u32(q.weight).contiguous()
    if x.ndim != 2 or w.ndim != 3:
        raise InvalidArgument(f"{op}: x must be [T, K] and w [E, N, K'], got {list(x.shape)} and {list(w.shape)}")
    x = x.to(dtype).contiguous()
    scales = (q.scales.to(dtype) if affine else q.scales).contiguous()
    biases = q.biases.to(dtype).contiguous() if affine else None
    columns = _quantized_columns(op, w, scales, biases, quant)
    if x.shape[-1] != columns:
        raise InvalidArgument(f"{op}: shapes {list(x.shape)} and {list(w.shape)} do not match")
    n = w.shape[-2]
    if expert_bias is not None and (tuple(expert_bias.shape) != (w.shape[0], n) or expert_bias.dtype != dtype):
        raise InvalidArgument(f"{op}: the experts' bias must be [{w.shape[0]}, {n}] of {dtype}")
    lhs, rhs = _indices(op, x, rows.reshape(-1)).contiguous(), _indices(op, w, sorted_ids.reshape(-1)).contiguous()
    if lhs.numel() != rhs.numel() or (offsets is not None and (offsets.numel() != w.shape[0] or offsets.dtype != torch.int32)):
        raise InvalidArgument(f"{op}: {lhs.numel()} rows, {rhs.numel()} expert ids, "
                              f"{'no' if offsets is None else offsets.numel()} offsets for {w.shape[0]} experts")
    _init(x)
    out = torch.empty((rhs.numel(), n // 2), dtype=dtype, device=x.device)
    d = _lib.GatherDescC(quant._c(), _CODE[dtype], 1, 0, 0, 1, n, columns, rhs.numel(), x.shape[0], w.shape[0])
    eb = None if expert_bias is None else expert_bias.contiguous()
    _lib.check(_lib.load().nvq_gather_qmm_glu(C.byref(d), GLU_ACTIVATIONS[activation], float(alpha), float(limit), _ptr(x), _ptr(w),
                                              _ptr(scales), _ptr(biases), _ptr(lhs), _ptr(rhs),
                                              _ptr(None if offsets is None else offsets.contiguous()), _ptr(eb), _ptr(out), _stream()))
    return out


def quantized_matmul_glu(x: torch.Tensor, q: Quantized, activation: str = "swiglu", *, alpha: float = 1.702, limit: float = 7.0,
                         bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """`Mlp::forward` up to the down projection (model.rs:2066-2074) for a few rows of x in one kernel: `q` (and `bias`
    `[N]`) hold the gate and up projections in alternating runs of 64 rows (`pair_rows`); the result is `[..., N / 2]`, bit
    for bit `glu(gate(x), up(x))` of the two rounded products.  Raises `Unsupported` beyond four rows of x and where the
    decode kernel does not take the product (the caller then composes the products and `glu`)."""
    op = "quantized_matmul"
    if activation not in GLU_ACTIVATIONS:
        raise InvalidArgument(f"{op}: unknown activation {activation!r}")
    quant = q.quant
    quant.checked(op)
    _check_groups(op, quant.mode, q.scales, q.biases)
    if q.global_scale is not None:
        raise Unsupported(f"{op}: the gated epilogue takes no global scale")
    affine = quant.mode == QuantMode.AFFINE
    dtype = _promoted(op, x, q.scales, q.biases)
    w = _u32(q.weight)
    if x.ndim < 1 or w.ndim != 2:
        raise Unsupported(f"{op}: the gated epilogue takes x [..., K] and one weight matrix, got {list(x.shape)} and {list(w.shape)}")
    x = x.to(dtype).contiguous()
    w = w.contiguous()
    scales = (q.scales.to(dtype) if affine else q.scales).contiguous()
    biases = q.biases.to(dtype).contiguous() if affine else None
    columns = _quantized_columns(op, w, scales, biases, quant)
    n = w.shape[0]
    if x.shape[-1] != columns:
        raise InvalidArgument(f"{op}: shapes {list(x.shape)} and {list(w.shape)} do not match")
    if bias is not None and (bias.dtype != dtype or tuple(bias.shape) != (n,)):
        raise InvalidArgument(f"{op}: the fused bias must be [{n}] of {_name(dtype)}")
    _init(x)
    rows = x.numel() // columns if columns else 0
    out = torch.empty(x.shape[:-1] + (n // 2,), dtype=dtype, device=x.device)
    d = _lib.QmmDescC()
    d.quant, d.dtype, d.transpose = quant._c(), _CODE[dtype], 1
    d.m = d.item_rows = rows
    d.n, d.k, d.batch_ndim = n, columns, 0
    _lib.check(_lib.load().nvq_quantized_matmul_glu(C.byref(d), GLU_ACTIVATIONS[activation], float(alpha), float(limit), _ptr(x), _ptr(w),
                                                    _ptr(scales), _ptr(biases), _ptr(None if bias is None else bias.contiguous()),
                                                    _ptr(out), _stream()))
    return out


def pair_rows(gate: torch.Tensor, up: torch.Tensor, dim: int) -> torch.Tensor:
    """The gate and up projections' rows (along `dim`, a multiple of 64 long) in alternating runs of 64: the layout
    `gather_qmm_glu` reads.  A copy, made once at load time."""
    n = gate.shape[dim]
    if up.shape != gate.shape or n % 64 != 0:
        raise InvalidArgument(f"pair_rows: two tensors of one shape with a multiple of 64 rows, got {list(gate.shape)} and {list(up.shape)}")
    dim = dim % gate.ndim
    shape = gate.shape[:dim] + (n // 64, 64) + gate.shape[dim + 1:]
    both = torch.stack([gate.reshape(shape), up.reshape(shape)], dim=dim + 1)  # [.., n / 64, 2, 64, ..]
    return both.reshape(gate.shape[:dim] + (2 * n,) + gate.shape[dim + 1:]).contiguous()


_IDENTITY: dict = {}


def _identity(n: int, device: torch.device) -> torch.Tensor:
    """0 .. n - 1 as int32 on the device, kept between calls (an `arange` is a kernel launch per call otherwise); callers
    only read it."""
    key = (n, device)
    t = _IDENTITY.get(key)
    if t is None:
        if len(_IDENTITY) >= 64:
            _IDENTITY.clear()
        t = _IDENTITY[key] = torch.arange(n, dtype=torch.int32, device=device)
    return t


def _pair_tokens(tokens: int, k: int, device: torch.device) -> torch.Tensor:
    """The token of each of `tokens * k` pairs (pair t * k + j belongs to token t) as int32, kept between calls."""
    key = ("pairs", tokens, k, device)
    t = _IDENTITY.get(key)
    if t is None:
        if len(_IDENTITY) >= 64:
            _IDENTITY.clear()
        t = _IDENTITY[key] = torch.arange(tokens, dtype=torch.int32, device=device).repeat_interleave(k)
    return t


def _indices(op: str, a: torch.Tensor, given: Optional[torch.Tensor]) -> torch.Tensor:
    """quantized.rs:739-767: integer indices as uint32 (carried as int32 bit patterns)."""
    batch = a.shape[:-2]
    if given is None:
        n = 1
        for s in batch:
            n *= s
        return _identity(n, a.device).reshape(batch)
    if given.dtype.is_floating_point or given.dtype == torch.bool:
        raise InvalidArgument(f"{op}: indices must be integers")
    return given.to(device=a.device).to(torch.int32) if given.dtype != torch.uint32 else given.view(torch.int32)


def gather_qmm(x: torch.Tensor, q: Quantized, lhs_indices: Optional[torch.Tensor] = None,
               rhs_indices: Optional[torch.Tensor] = None, options: GatherQmm = GatherQmm(), *,
               row_exact: bool = False, out_rows: Optional[torch.Tensor] = None,
               expert_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """ops.rs:1050-1074, quantized.rs:589-673: output batch i = x[lhs[i]] . dequantize(w)[rhs[i]]^T.  `out_rows` (not in
    the reference; one integer per pair, a permutation) writes batch i at position `out_rows[i]` of the flattened
    batches instead.  `expert_bias` `[E, N]` adds `bias[rhs[i]]` to every row of batch i in the kernels' epilogues
    (`SwitchProjection::forward`, model.rs:2139-2143; weights stored [N, K] only)."""
    op = "gather_qmm"
    quant = q.quant
    quant.checked(op)
    if lhs_indices is None and rhs_indices is None:
        return quantized_matmul(x, q, options.transpose, row_exact=row_exact)
    _check_groups(op, quant.mode, q.scales, q.biases)
    affine = quant.mode == QuantMode.AFFINE
    dtype = _promoted(op, x, q.scales, q.biases)
    w = _u32(q.weight)
    if x.ndim < 2 or w.ndim < 2 or (q.biases is not None and q.scales.shape != q.biases.shape):
        raise InvalidArgument(f"{op}: x must be [..., M, K] and w [..., N, K'], got {list(x.shape)} and {list(w.shape)}")
    x = x.to(dtype).contiguous()
    scales = (q.scales.to(dtype) if affine else q.scales).contiguous()
    biases = q.biases.to(dtype).contiguous() if affine else None
    w = w.contiguous()
    columns = _quantized_columns(op, w, scales, biases, quant)
    rows = w.shape[-2]
    inner, outer = (columns, rows) if options.transpose else (rows, columns)
    if x.shape[-1] != inner:
        raise InvalidArgument(f"{op}: shapes {list(x.shape)} and {list(w.shape)} do not match")
    lhs, rhs = _indices(op, x, lhs_indices), _indices(op, w, rhs_indices)
    try:
        lhs, rhs = torch.broadcast_tensors(lhs, rhs)
    except RuntimeError:
        raise InvalidArgument(f"{op}: index shapes {list(lhs.shape)} and {list(rhs.shape)} do not broadcast") from None
    lhs, rhs = lhs.contiguous(), rhs.contiguous()
    gs = q.global_scale
    if gs is not None:  # quantized.rs:620-636: one float32 value per expert
        if quant.mode != QuantMode.NVFP4:
            raise InvalidArgument(f"{op}: global scale is only supported for 'nvfp4' quantization mode")
        if gs.dtype != torch.float32:
            raise InvalidArgument(f"{op}: global scale must have dtype float32 but got {_name(gs.dtype)}")
        if tuple(gs.shape) != tuple(w.shape[:-2]):
            raise InvalidArgument(f"{op}: global scale must have one entry per expert with shape {list(w.shape[:-2])} but got {list(gs.shape)}")
        gs = gs.to(x.device).contiguous()
    _init(x)
    m = x.shape[-2]
    x_batches = x.numel() // (m * inner) if m * inner else 0
    experts = 1
    for s in w.shape[:-2]:
        experts *= s
    is_sorted = lhs_indices is None and options.sorted_indices and GatherQmm.groups(rhs.numel(), experts, row_exact)
    offsets = None
    if is_sorted and m == 1 and x.ndim == 3 and rhs.ndim == 1:  # quantized.rs:772-782
        offsets = sorted_offsets(rhs, experts)
    out = torch.empty(tuple(rhs.shape) + (m, outer), dtype=dtype, device=x.device)
    d = _lib.GatherDescC(quant._c(), _CODE[dtype], int(options.transpose), int(row_exact), 0, m, outer, inner, rhs.numel(), x_batches, experts)
    lib = _lib.load()
    need = lib.nvq_gather_qmm_workspace_bytes(C.byref(d))
    workspace = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
    scatter = _out_rows(op, out_rows, rhs.numel(), x.device)
    if scatter is not None and lhs_indices is None and rhs_indices is None:
        raise InvalidArgument(f"{op}: output rows need indices")
    if expert_bias is not None:
        if expert_bias.dtype != dtype or tuple(expert_bias.shape) != (experts, outer):
            raise InvalidArgument(f"{op}: the experts' bias must be [{experts}, {outer}] of {_name(dtype)}")
        _lib.check(lib.nvq_gather_qmm_expert_bias(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(gs), _ptr(lhs),
                                                  _ptr(rhs), _ptr(offsets), _ptr(scatter), _ptr(expert_bias.contiguous()), _ptr(out),
                                                  _ptr(workspace), _stream()))
        return out
    if scatter is not None:
        _lib.check(lib.nvq_gather_qmm_scatter(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(gs), _ptr(lhs),
                                              _ptr(rhs), _ptr(offsets), _ptr(scatter), _ptr(out), _ptr(workspace), _stream()))
        return out
    if gs is not None:
        _lib.check(lib.nvq_gather_qmm_scaled(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(gs), _ptr(lhs), _ptr(rhs),
                                             _ptr(offsets), _ptr(out), _ptr(workspace), _stream()))
        return out
    _lib.check(lib.nvq_gather_qmm(C.byref(d), _ptr(x), _ptr(w), _ptr(scales), _ptr(biases), _ptr(lhs), _ptr(rhs),
                                  _ptr(offsets), _ptr(out), _ptr(workspace), _stream()))
    return out
