"""Quantized checkpoint tensors in Hugging Face layouts as nuvec's `Quantized` operands
(crates/nuvec-lm/src/quant.rs).  The repacking runs in the HIP library; this is the host mirror of the
reference's two functions (same names, argument meaning and errors)."""
from __future__ import annotations

import ctypes as C
from typing import Dict

import torch

from . import _lib
from .ops import _CODE, _FLOATS, InvalidArgument, Quant, QuantMode, _init, _name, _ptr, _stream

AWQ, GPTQ_V1, GPTQ_V2 = "awq", "gptq", "gptq_v2"  # config.rs:30-48 (`PackedFormat::Awq`, `Gptq { v1 }`)
_FORMAT = {AWQ: 0, GPTQ_V1: 1, GPTQ_V2: 2}


def mxfp4_from_hf_blocks(blocks: torch.Tensor) -> torch.Tensor:
    """quant.rs:9-33: gpt-oss's MXFP4 experts (`*_blocks`, uint8 `[..., K / 32, 16]`) as packed codes
    (uint32 `[..., K / 8]`); the bytes are reinterpreted, not copied, when the blocks are contiguous."""
    codes = blocks.contiguous().view(torch.uint32)
    if codes.ndim < 2:
        return codes
    return codes.reshape(codes.shape[:-2] + (codes.shape[-2] * codes.shape[-1],))


def convert_packed(weights: Dict[str, torch.Tensor], fmt: str, quant: Quant) -> Dict[str, torch.Tensor]:
    """quant.rs:66-196: every `{prefix}.qweight / .qzeros / .scales (/ .g_idx)` of an AWQ or GPTQ checkpoint as
    `{prefix}.weight / .scales / .biases` in the affine layout, and every other float tensor in the scales'
    dtype; other tensors pass through."""
    if fmt not in _FORMAT:
        raise InvalidArgument(f"convert_packed: unknown format {fmt!r}")
    if quant.mode != QuantMode.AFFINE:
        raise InvalidArgument("convert_packed: the packed formats are affine")
    bits, group = quant.bits, quant.group_size
    per_word = 32 // bits
    out = dict(weights)
    dtype = None
    for prefix in [k[: -len(".qweight")] for k in weights if k.endswith(".qweight")]:
        qweight = out.pop(f"{prefix}.qweight")
        scales = out.pop(f"{prefix}.scales", None)
        if scales is None:
            raise InvalidArgument(f"{prefix}: qweight without scales")
        qzeros = out.pop(f"{prefix}.qzeros", None)
        g_idx = out.pop(f"{prefix}.g_idx", None)
        if qweight.ndim != 2:
            raise InvalidArgument(f"{prefix}: a 2-D packed tensor, got {list(qweight.shape)}")
        rows, cols = qweight.shape
        inputs, outputs = (rows, cols * per_word) if fmt == AWQ else (rows * per_word, cols)
        groups = -(-inputs // group)
        if inputs % group != 0 or tuple(scales.shape) != (groups, outputs):
            raise InvalidArgument(f"{prefix}: {inputs} inputs and scales {list(scales.shape)} do not match groups of {group}")
        if g_idx is not None:
            want = torch.arange(inputs, device=g_idx.device) // group
            if g_idx.numel() != inputs or not torch.equal(g_idx.reshape(-1).to(torch.int64), want):
                raise InvalidArgument(f"{prefix}: g_idx reorders the inputs (activation reordering), which MLX's grouping "
                                      "cannot express")
        if qzeros is not None and tuple(qzeros.shape) != (groups, -(-outputs // per_word)):
            raise InvalidArgument(f"{prefix}: qzeros {list(qzeros.shape)} for {groups} groups of {outputs} outputs")
        if scales.dtype not in _FLOATS:
            raise InvalidArgument(f"{prefix}: unsupported scale dtype {_name(scales.dtype)}")
        _init(qweight)
        dev = qweight.device
        qw = qweight.to(torch.int32).contiguous()
        qz = qzeros.to(device=dev, dtype=torch.int32).contiguous() if qzeros is not None else None
        sc = scales.to(dev).contiguous()
        weight = torch.empty((outputs, inputs // per_word), dtype=torch.uint32, device=dev)
        scales_out = torch.empty((outputs, groups), dtype=sc.dtype, device=dev)
        biases_out = torch.empty_like(scales_out)
        _lib.check(_lib.load().nvq_convert_packed(_FORMAT[fmt], C.byref(quant._c()), _CODE[sc.dtype], _ptr(qw), _ptr(qz), _ptr(sc),
                                                  rows, cols, _ptr(weight), _ptr(scales_out), _ptr(biases_out), _stream()))
        dtype = dtype or sc.dtype
        out[f"{prefix}.weight"], out[f"{prefix}.scales"], out[f"{prefix}.biases"] = weight, scales_out, biases_out
    if dtype is not None:
        for name, w in out.items():
            quantized = name.endswith(".scales") or name.endswith(".biases")
            if not quantized and w.dtype.is_floating_point and w.dtype != dtype:
                out[name] = w.to(dtype)
    return out
