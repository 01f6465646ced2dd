"""The callers of the quantized path: nuvec-nn's linear layer and embedding with packed weights
(crates/nuvec-nn/src/layers.rs:89-162 and 207-262) and nuvec-lm's expert projections of a mixture-of-experts
block (crates/nuvec-lm/src/model.rs:2103-2211).  Thin host glue over `ops`; every product, lookup, ordering
and quantization runs in the HIP library.
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
        """layers.rs:155-162: the product, then the bias added as a separate rounded addition: here in the product
        kernels' epilogues (same two roundings, one launch) when the bias has the product's dtype and the mode no global
        scale; otherwise the addition stays separate, as in the reference, and promotes."""
        q = self.quantized()
        if self.bias is None:
            return ops.quantized_matmul(x, q, transpose=True)
        affine = self.quant.mode == QuantMode.AFFINE
        dtype = torch.promote_types(torch.promote_types(x.dtype, self.scales.dtype), self.biases.dtype) if affine else x.dtype
        if self.bias.dtype == dtype and self.bias.ndim == 1 and x.shape[-1] > 0 and getattr(q, "global_scale", None) is None:
            return ops.quantized_matmul(x, q, transpose=True, bias=self.bias)
        return ops.quantized_matmul(x, q, transpose=True) + self.bias

    __call__ = forward


@dataclass
class Mlp:
    """model.rs:2044-2075 (`Mlp`): `down(act(gate(x), up(x)))` with SwiGLU, or Gemma's GeGLU (`geglu`)."""
    gate_proj: QuantizedLinear
    up_proj: QuantizedLinear
    down_proj: QuantizedLinear
    geglu: bool = False
    gate_up_proj: Optional[QuantizedLinear] = None  # `fuse_gate_up`: both projections' rows in alternating runs of 64

    def fuse_gate_up(self) -> "Mlp":
        """Stores the gate and up projections as one weight whose rows alternate in runs of 64 (a copy made once, at load
        time), so that a few rows of x (decoding) take both products and the activation in one kernel
        (`ops.quantized_matmul_glu`).  Left apart: projections that differ in shape or quantization, hidden sizes off
        whole runs, affine projections of fewer than 1024 rows (they take the kernels with the CPU's weights at every row count)."""
        g, u = self.gate_proj, self.up_proj
        hidden = g.weight.shape[0]
        if g.quant != u.quant or g.weight.shape != u.weight.shape or (g.bias is None) != (u.bias is None) or hidden % 64 != 0:
            return self
        if g.quant.mode == QuantMode.AFFINE and hidden < 1024:
            return self
        cat = lambda a, b: None if a is None else ops.pair_rows(a, b, 0)
        self.gate_up_proj = QuantizedLinear(cat(g.weight, u.weight), cat(g.scales, u.scales), cat(g.biases, u.biases), cat(g.bias, u.bias), g.quant)
        return self

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """model.rs:2066-2074."""
        activation = "geglu" if self.geglu else "swiglu"
        rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
        # (measured at 4096 -> 14336 -> 4096, device time: one row 29.1 -> 23.6 us with 4-bit weights, 25.9 -> 21.1 us with
        # MXFP4; four rows 36.7 -> 34.0 us with MXFP4 but 33.6 -> 39.3 us with 4-bit weights, whose three and four rows have
        # a matrix-core decode kernel of their own)
        most = 2 if self.gate_proj.quant.mode == QuantMode.AFFINE else 4
        if self.gate_up_proj is not None and 1 <= rows <= most:
            p = self.gate_up_proj
            try:
                return self.down_proj(ops.quantized_matmul_glu(x, p.quantized(), activation, bias=p.bias))
            except ops.Unsupported:  # (a product the decode kernel does not take: the composition below)
                pass
        return self.down_proj(ops.glu(self.gate_proj(x), self.up_proj(x), activation))

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


@dataclass
class SwitchProjection:
    """model.rs:2103-2146 (`SwitchProjection::Quantized`, mlx-lm's `SwitchLinear`): one packed weight
    `[experts, output_dims, input_dims * bits / 32]` per expert, an optional bias `[experts, output_dims]`."""
    weight: torch.Tensor
    scales: torch.Tensor
    biases: Optional[torch.Tensor]
    bias: Optional[torch.Tensor] = None
    quant: Quant = Quant()
    global_scale: Optional[torch.Tensor] = None  # NVFP4: one float32 value per expert (model.rs:2095, quantized.rs:620-636)

    def quantized(self) -> Quantized:
        return Quantized(self.weight, self.scales, self.biases, self.quant, self.global_scale)

    def forward(self, x: torch.Tensor, indices: torch.Tensor, sorted_indices: bool = False, add_bias: bool = True) -> torch.Tensor:
        """model.rs:2113-2146: `x` (`[..., 1, input_dims]` batches) through the experts `indices`."""
        if self.bias is None or not add_bias:
            return ops.gather_qmm(x, self.quantized(), None, indices, ops.GatherQmm(sorted_indices=sorted_indices))
        return ops.gather_qmm(x, self.quantized(), None, indices, ops.GatherQmm(sorted_indices=sorted_indices), expert_bias=self.bias)

    def forward_sorted_rows(self, x: torch.Tensor, rows, sorted_ids: torch.Tensor, offsets: torch.Tensor,
                            out_rows: Optional[torch.Tensor] = None, add_bias: bool = True) -> torch.Tensor:
        """Rows `rows` of `x` (`[T, input_dims]`; None: its rows in order) through experts sorted by id.  With
        `out_rows` (a permutation) result row i is written at row `out_rows[i]`.  `add_bias` False leaves the experts'
        bias to the caller (the gated activation adds it in its own pass)."""
        if rows is None:
            rows = ops._identity(x.shape[0], x.device)
        if self.bias is None or not add_bias:
            return ops.gather_qmm_grouped(x, self.quantized(), rows, sorted_ids, offsets, out_rows)
        try:  # the bias in the grouped kernel's epilogue
            return ops.gather_qmm_grouped(x, self.quantized(), rows, sorted_ids, offsets, out_rows, expert_bias=self.bias)
        except ops.Unsupported:  # (a product the grouped matrix-core kernel does not take: the addition on its own)
            y = ops.gather_qmm_grouped(x, self.quantized(), rows, sorted_ids, offsets, out_rows)
        if out_rows is None:
            return y + self.bias[sorted_ids.long()]
        ids = torch.empty_like(sorted_ids)
        ids[out_rows.long()] = sorted_ids  # the expert of each output row
        return y + self.bias[ids.long()]


@dataclass
class SwitchGlu:
    """model.rs:2149-2211 (mlx-lm's `SwitchGLU`): the experts' gated MLPs."""
    gate_proj: SwitchProjection
    up_proj: SwitchProjection
    down_proj: SwitchProjection
    gate_up_proj: Optional[SwitchProjection] = None  # `fuse_gate_up`: both projections' rows, gate first
    gate_up_paired: bool = False  # `gate_up_proj` alternates the two projections' rows in runs of 64
    activation: str = "swiglu"  # or "swiglu_oai" with `alpha` and `limit` (model.rs:2161-2166; gpt-oss: 1.702 and 7), or "geglu" (model.rs:2167)
    alpha: float = 1.702
    limit: float = 7.0

    def gated(self, gate: torch.Tensor, up: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """model.rs:2157-2169 between the products: the experts' biases (model.rs:2139-2143) and the activation in one
        pass over the two products, which arrive without their biases."""
        gb, ub = self.gate_proj.bias, self.up_proj.bias
        if (gb is None) != (ub is None):  # one projection with a bias: added on its own, as SwitchProjection does
            rows = ids.reshape(-1).long()
            if gb is not None:
                gate = (gate.reshape(rows.numel(), -1) + gb[rows]).reshape(gate.shape)
            else:
                up = (up.reshape(rows.numel(), -1) + ub[rows]).reshape(up.shape)
            gb = ub = None
        return ops.glu(gate, up, self.activation, alpha=self.alpha, limit=self.limit, gate_bias=gb, up_bias=ub, ids=ids)

    def fuse_gate_up(self) -> "SwitchGlu":
        """Stores the gate and up projections as one weight `[experts, 2 * hidden, ...]` (a copy made once, at load
        time), so that the ordered pairs take one product that reads x and walks the experts once instead of two.  Where
        `hidden` is a multiple of 64 the rows alternate in runs of 64 (`ops.pair_rows`) and the product applies the
        activation itself (`ops.gather_qmm_glu`); otherwise the gate's rows come first, then the up projection's, and
        the activation is a pass of its own.  Every output is computed as before: the results are bit-identical."""
        g, u = self.gate_proj, self.up_proj
        if g.quant != u.quant or g.weight.shape != u.weight.shape or (g.bias is None) != (u.bias is None):
            raise ops.InvalidArgument("fuse_gate_up: the gate and up projections differ in shape or quantization")
        if g.global_scale is not None or u.global_scale is not None:
            return self  # (NVFP4 with global scales: each projection has its own per expert)
        hidden = g.weight.shape[1]
        if g.quant.mode == ops.QuantMode.AFFINE and 512 <= hidden < 1024:
            # Affine products of fewer than 1024 outputs per row materialise the CPU's doubly rounded weights: one product
            # of 2 * hidden rows would not, the two of `hidden` rows do.  Such projections stay apart.
            return self
        self.gate_up_paired = hidden % 64 == 0
        if self.gate_up_paired:
            cat = lambda a, b: None if a is None else ops.pair_rows(a, b, 1)
        else:
            cat = lambda a, b: None if a is None else torch.cat([a, b], dim=1).contiguous()
        self.gate_up_proj = SwitchProjection(cat(g.weight, u.weight), cat(g.scales, u.scales), cat(g.biases, u.biases),
                                             cat(g.bias, u.bias), g.quant)
        return self

    def forward(self, x: torch.Tensor, indices: torch.Tensor) -> torch.Tensor:
        """`x` `[B, L, D]` through each token's experts `indices` `[B, L, k]`: `[B, L, k, D]`.  With 64 pairs or
        more they are ordered by expert (model.rs:2193-2210) so that each expert's weights are read once; here one
        kernel orders the pairs, the products take the token rows of `x` themselves, and the last product writes
        each row at its pair's place (`out_rows`), so the inverse permutation of model.rs:2210 is never run."""
        b, l, d = x.shape
        k = indices.shape[2]
        if indices.numel() < 64:  # model.rs:2189-2192
            xe = x.reshape(b, l, 1, 1, d)
            hidden = None
            if self.gate_up_proj is not None and self.gate_up_paired:
                try:  # one kernel: both products of every pair on the decode kernel, the activation as its epilogue
                    tokens = ops._pair_tokens(b * l, k, x.device)
                    hidden = ops.gather_qmm_glu(x.reshape(b * l, d), self.gate_up_proj.quantized(), tokens, indices.reshape(-1), None,
                                                self.activation, alpha=self.alpha, limit=self.limit, expert_bias=self.gate_up_proj.bias)
                    hidden = hidden.reshape(b, l, k, 1, -1)
                except ops.Unsupported:
                    hidden = None
            if hidden is not None:
                return self.down_proj.forward(hidden, indices).squeeze(-2)
            if self.gate_up_proj is not None:  # one gather for both projections (a decoded token's few pairs are launch-bound)
                both = self.gate_up_proj.forward(xe, indices, add_bias=False)
                if self.gate_up_paired:
                    runs = both.reshape(both.shape[:-1] + (-1, 2, 64))
                    gate, up = runs[..., 0, :].reshape(both.shape[:-1] + (-1,)), runs[..., 1, :].reshape(both.shape[:-1] + (-1,))
                else:
                    half = both.shape[-1] // 2
                    gate, up = both[..., :half], both[..., half:]
            else:
                up, gate = self.up_proj.forward(xe, indices, add_bias=False), self.gate_proj.forward(xe, indices, add_bias=False)
            return self.down_proj.forward(self.gated(gate, up, indices), indices).squeeze(-2)
        experts = self.up_proj.weight.shape[0]
        order, restore, sorted_ids, offsets = ops.moe_order(indices, experts)
        tokens = torch.div(order, k, rounding_mode="floor").to(torch.int32)  # pair t*k + j belongs to token t
        xt = x.reshape(b * l, d)
        hidden = None
        if self.gate_up_proj is not None and self.gate_up_paired:
            try:  # one kernel: both products and the activation
                hidden = ops.gather_qmm_glu(xt, self.gate_up_proj.quantized(), tokens, sorted_ids, offsets, self.activation,
                                            alpha=self.alpha, limit=self.limit, expert_bias=self.gate_up_proj.bias)
            except ops.Unsupported:  # (a product the grouped matrix-core kernel does not take)
                both = self.gate_up_proj.forward_sorted_rows(xt, tokens, sorted_ids, offsets, add_bias=False)
                runs = both.reshape(both.shape[0], -1, 2, 64)
                hidden = self.gated(runs[:, :, 0].reshape(both.shape[0], -1), runs[:, :, 1].reshape(both.shape[0], -1), sorted_ids)
        elif self.gate_up_proj is not None:
            both = self.gate_up_proj.forward_sorted_rows(xt, tokens, sorted_ids, offsets, add_bias=False)
            half = both.shape[-1] // 2
            hidden = self.gated(both[:, :half], both[:, half:], sorted_ids)  # (read in place: the activation takes a row stride)
        else:
            up = self.up_proj.forward_sorted_rows(xt, tokens, sorted_ids, offsets, add_bias=False)
            gate = self.gate_proj.forward_sorted_rows(xt, tokens, sorted_ids, offsets, add_bias=False)
            hidden = self.gated(gate, up, sorted_ids)
        out = self.down_proj.forward_sorted_rows(hidden, None, sorted_ids, offsets, out_rows=order)
        return out.reshape(b, l, k, -1)

    __call__ = forward


@dataclass
class MoeMlp:
    """model.rs:2218-2272 (`MoeMlp`, mlx-lm's sparse MoE blocks): the router's probabilities (a softmax in the
    activations' type), each token's best `k` experts (`moe_route`), the experts' gated MLPs (`SwitchGlu`) and their
    outputs weighted by the (renormalised) scores and summed (`weighted_sum`).  `gate` is the router's dense weight
    `[experts, D]`; the shared expert of some models is a dense MLP outside this path and is left to the caller."""
    gate: torch.Tensor
    switch_mlp: SwitchGlu
    experts_per_token: int
    norm_topk_prob: bool = True

    def route(self, x: torch.Tensor):
        """The router: `(top, scores)` of `moe_route` over `softmax(x gate^T)`."""
        logits = torch.nn.functional.linear(x, self.gate.to(x.dtype))
        probs = torch.softmax(logits.float(), dim=-1).to(x.dtype)  # softmax_precise: float32 inside, one rounding
        return ops.moe_route(probs, self.experts_per_token, self.norm_topk_prob)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """`x` `[B, L, D]` -> `[B, L, D]`."""
        top, scores = self.route(x)
        experts = self.switch_mlp.forward(x, top)  # [B, L, k, D]
        return ops.weighted_sum(experts, scores)

    __call__ = forward


def quantized_attention(q: torch.Tensor, k: ops.Quantized, v: ops.Quantized, scale: float,
                        sinks: Optional[torch.Tensor] = None, causal: bool = False, fused: bool = True) -> torch.Tensor:
    """fast.rs:694-718, fast/imp.rs:3992-4035 (`quantized_attention`, mlx-lm's quantized KV cache): attention of the
    queries `q [B, Hq, L, D]` over affine-quantized keys and values (codes `[B, Hkv, S, D * bits / 32]`, scales and
    biases `[B, Hkv, S, D / group]`), grouped query heads, optional per-head `sinks [Hq]`, optionally causal (query i
    of L sees keys up to S - L + i, nuvec-lm's `quantized_attention`, model.rs:3646-3700):
    `softmax(scale * q k^T [, sinks]) v`.  One query row per head that fits the kernel (head size 64 or 128, 3, 4 or 8 bits)
    takes the library's fused kernel; the rest is the reference's composition (the one it runs wherever its fused
    kernel does not fit): both products are the library's quantized products, transposed for the keys and
    untransposed for the values; the softmax (float32 inside, one rounding) is an elementwise step outside the path."""
    if k.quant != v.quant or k.quant.mode != ops.QuantMode.AFFINE:
        raise ops.InvalidArgument("quantized_attention: keys and values need one affine quantization")
    if k.biases is None or v.biases is None:
        raise ops.InvalidArgument("quantized_attention: affine biases missing")
    # (a single causal query row sees every key: the mask is empty)
    if fused and (not causal or q.shape[-2] == 1) and q.is_cuda and ops.quantized_attention_fits(q, k, v, sinks):
        return ops.quantized_attention(q, k, v, scale, sinks)  # one kernel (the reference's FastOp::QuantizedAttention)
    b, hq, l, d = q.shape
    hkv = k.weight.shape[1]
    if hq % hkv != 0:
        raise ops.InvalidArgument(f"quantized_attention: {hq} query heads over {hkv} key heads")
    rep = hq // hkv
    qs = (q * scale).reshape(b, hkv, rep, l, d)
    expand = lambda t: ops.Quantized(t.weight.unsqueeze(-3), t.scales.unsqueeze(-3), t.biases.unsqueeze(-3), t.quant)
    scores = ops.quantized_matmul(qs, expand(k), True)  # [B, Hkv, rep, L, S]
    s = scores.shape[-1]
    if causal and l > 1:
        hidden = torch.arange(s, device=q.device)[None, :] > (s - l + torch.arange(l, device=q.device))[:, None]
        scores = scores.masked_fill(hidden, float("-inf"))
    if sinks is not None:
        column = sinks.to(scores.dtype).reshape(1, hkv, rep, 1, 1).expand(b, hkv, rep, l, 1)
        probs = torch.softmax(torch.cat([scores, column], dim=-1).float(), dim=-1).to(scores.dtype)[..., :s]
    else:
        probs = torch.softmax(scores.float(), dim=-1).to(scores.dtype)
    out = ops.quantized_matmul(probs.contiguous(), expand(v), False)  # [B, Hkv, rep, L, D]
    return out.reshape(b, hq, l, d)
