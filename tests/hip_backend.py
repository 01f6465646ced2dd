"""Adapter that runs replayed cases and seeded parity inputs on the HIP backend.

numpy in, numpy out (bfloat16 as uint16 bit patterns), through `nuvec_amd.ops` and therefore
through the C ABI of libnuvec_hip.so.  There is no CPU path behind it.
"""
from __future__ import annotations

import numpy as np
import torch

import nuvec_amd as nv
from oracle import ref

TORCH = {ref.F16: torch.float16, ref.BF16: torch.bfloat16, ref.F32: torch.float32}


def to_dev(a, dtype_code=None):
    """numpy -> cuda tensor; `dtype_code` says how to read uint16 data."""
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:  # bfloat16 bit patterns
        return torch.from_numpy(a.view(np.int16)).cuda().view(torch.bfloat16)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda().view(torch.uint32)
    return torch.from_numpy(a).cuda()


def to_host(t):
    if t.dtype == torch.bfloat16:
        return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    if t.dtype == torch.uint32:
        return t.contiguous().view(torch.int32).cpu().numpy().view(np.uint32)
    return t.contiguous().cpu().numpy()


def quant(mode, group, bits):
    return nv.Quant(nv.QuantMode(mode), group, bits)


class HipBackend:
    name = "hip"

    def quantize(self, w, dtype, mode, group, bits, global_scale=None):
        q = nv.quantize(to_dev(w), quant(mode, group, bits), None if global_scale is None else to_dev(np.asarray(global_scale)))
        return to_host(q.weight), to_host(q.scales), None if q.biases is None else to_host(q.biases)

    def dequantize(self, w, scales, biases, mode, group, bits, scales_dtype, out_dtype=None, global_scale=None):
        q = nv.Quantized(to_dev(w), to_dev(scales), to_dev(biases), quant(mode, group, bits),
                         None if global_scale is None else to_dev(np.asarray(global_scale)))
        out = nv.dequantize(q, None if out_dtype is None else TORCH[out_dtype])
        code = {torch.float16: ref.F16, torch.bfloat16: ref.BF16, torch.float32: ref.F32}[out.dtype]
        return to_host(out), code

    def quantized_matmul(self, x, w, scales, biases, mode, group, bits, dtype, transpose):
        q = nv.Quantized(to_dev(w), to_dev(scales), to_dev(biases), quant(mode, group, bits))
        return to_host(nv.quantized_matmul(to_dev(x), q, transpose))

    def gather_qmm(self, x, w, scales, biases, lhs, rhs, mode, group, bits, dtype, transpose, sorted_indices,
                   global_scales=None):
        q = nv.Quantized(to_dev(w), to_dev(scales), to_dev(biases), quant(mode, group, bits), to_dev(global_scales))
        idx = lambda i: None if i is None else torch.from_numpy(np.ascontiguousarray(i).astype(np.int64)).cuda()
        y = nv.gather_qmm(to_dev(x), q, idx(lhs), idx(rhs), nv.GatherQmm(transpose, sorted_indices))
        return to_host(y)

    def _qq_weight(self, w, mode, gw, prequantized):
        qm = nv.Quant.new(nv.QuantMode(mode))
        if prequantized or gw is not None:  # a dense weight with a global scale is quantized with it for the product
            return nv.quantize(to_dev(w), qm, None if gw is None else to_dev(np.asarray(gw))), None
        return to_dev(w), qm

    def qqmm(self, x, w, dtype, mode, gx, gw, prequantized):
        weight, qm = self._qq_weight(w, mode, gw, prequantized)
        return to_host(nv.qqmm(to_dev(x), weight, qm, None if gx is None else to_dev(np.asarray(gx))))

    def gather_qqmm(self, x, w, rhs, dtype, mode, gx, gw, prequantized):
        weight, qm = self._qq_weight(w, mode, gw, prequantized)
        idx = torch.from_numpy(np.ascontiguousarray(rhs).astype(np.int64)).cuda()
        return to_host(nv.gather_qqmm(to_dev(x), weight, None, idx, False, qm, None if gx is None else to_dev(np.asarray(gx))))
