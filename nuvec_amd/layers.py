"""The two callers of the quantized path in nuvec-nn (crates/nuvec-nn/src/layers.rs:89-162 and
207-262): a linear layer and an embedding whose weights are stored packed.  Thin host glue over
`ops`; every product, lookup and quantization runs in the HIP library.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from . import ops
from .ops import Quant, QuantMode, Quantized


def _quant(quant) -> Quant:
    return Quant.new(quant) if isinstance(quant, QuantMode) else quant


@dataclass
class QuantizedLinear:
    """layers.rs:89-162: `x W^T + b` by `quantized_matmul` from the packed weight
    `[output_dims, input_dims * bits / 32]`, its scales and (affine) biases; `bias` is `[output_dims]`."""
    weight: torch.Tensor
    scales: torch.Tensor
    biases: Optional[torch.Tensor]
    bias: Optional[torch.Tensor] = None
    quant: Quant = Quant()

    @staticmethod
    def from_linear(weight: torch.Tensor, bias: Optional[torch.Tensor] = None, quant=Quant()) -> "QuantizedLinear":
        """layers.rs:121-139: quantizes a dense `[output_dims, input_dims]` weight; the bias is kept."""
        q = ops.quantize(weight, _quant(quant))
        return QuantizedLinear(q.weight, q.scales, q.biases, bias, q.quant)

    def quantized(self) -> Quantized:
        return Quantized(self.weight, self.scales, self.biases, self.quant)

    def dequantized_weight(self, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return ops.dequantize(self.quantized(), dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """layers.rs:155-162: the product, then the bias added as a separate rounded addition."""
        y = ops.quantized_matmul(x, self.quantized(), transpose=True)
        return y if self.bias is None else y + self.bias

    __call__ = forward


@dataclass
class QuantizedEmbedding:
    """layers.rs:207-262: a lookup table stored packed, `[num_embeddings, dims * bits / 32]`."""
    weight: torch.Tensor
    scales: torch.Tensor
    biases: Optional[torch.Tensor]
    quant: Quant = Quant()

    @staticmethod
    def from_embedding(table: torch.Tensor, quant=Quant()) -> "QuantizedEmbedding":
        """layers.rs:221-235."""
        q = ops.quantize(table, _quant(quant))
        return QuantizedEmbedding(q.weight, q.scales, q.biases, q.quant)

    def quantized(self) -> Quantized:
        return Quantized(self.weight, self.scales, self.biases, self.quant)

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        """layers.rs:245-255: the rows for `ids`, dequantized (scales' dtype for affine, bfloat16 for the
        floating-point modes): shape `ids.shape + [dims]`.  One fused kernel; the taken packed rows are
        never written out."""
        return ops.embedding(self.quantized(), ids)

    def as_linear(self, x: torch.Tensor) -> torch.Tensor:
        """layers.rs:258-261: `x W^T` with the quantized table (tied embeddings)."""
        return ops.quantized_matmul(x, self.quantized(), transpose=True)

    __call__ = forward
