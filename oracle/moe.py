"""TEST INFRASTRUCTURE ONLY: a CPU restatement of nuvec's mixture-of-experts glue kernels, for the parity tests.

`moe_route` and `weighted_sum` follow crates/nuvec-kernels/src/metal/moe.metal line by line (33-88 and 90-118): the
reference defines both by that kernel's arithmetic, in the element type, in that order.  What pins them beyond the
source: the indices are the last k of a stable ascending sort with NaN last (numpy's stable argsort, a library routine,
in tests/test_oracle_math.py), the documented example of crates/nuvec-core/src/fast.rs:733-737 and the NaN case of
crates/nuvec-core/tests/fast.rs:900-911; the scores and sums are checked against float64 within the rounding of the
element type.  `glu` restates the gated activations of crates/nuvec-nn/src/lib.rs (343-345, 513-519, 564-570) one
operation at a time, each result rounded to the element type as the reference's element-wise graphs evaluate
(crates/nuvec-core/src/fused.rs:190-215), with the experts' biases of crates/nuvec-lm/src/model.rs:2139-2143 added
first; pinned by the documented example of lib.rs:555-560 and by the closed forms in float64 within the rounding of
the element type.  Its last bit is PARITY UNPINNED: it depends on the host's `exp` (numpy's here, Rust's libm there).
Nothing here is imported by the product.
"""
from __future__ import annotations

import numpy as np

from . import ref


def _round(a: np.ndarray, dtype: int) -> np.ndarray:
    """float32 values rounded to the element type and widened again."""
    return ref.to_f32(ref.from_f32(np.asarray(a, np.float32), dtype), dtype)


def _less(a: float, b: float, dtype: int) -> bool:
    """moe.metal:19-31: NaN sorts last where the sort compares NaN (float32 and half, not bfloat16)."""
    if dtype != ref.BF16:
        an, bn = np.isnan(a), np.isnan(b)
        if an or bn:
            return (not an) and bn
    return bool(a < b)


def moe_route(probs: np.ndarray, dtype: int, k: int, normalize: bool):
    """probs: element-type array [rows, E] (as stored).  Returns (indices u32 [rows, k], scores as stored [rows, k])."""
    p = ref.to_f32(probs, dtype)
    rows, n = p.shape
    indices = np.zeros((rows, k), np.uint32)
    top = np.zeros((rows, k), np.float32)
    for r in range(rows):
        for e in range(n):
            v = p[r, e]
            rank = 0
            for j in range(n):
                u = p[r, j]
                rank += 1 if (_less(u, v, dtype) or (not _less(v, u, dtype) and j < e)) else 0
            slot = rank - (n - k)
            if slot >= 0:
                indices[r, slot] = e
                top[r, slot] = v
    if normalize:
        scores = np.zeros_like(top)
        for r in range(rows):
            total = np.float32(0)
            for j in range(k):
                total = _round(top[r, j] + total, dtype)
            with np.errstate(divide="ignore", invalid="ignore"):
                scores[r] = _round(top[r] / total, dtype)
    else:
        scores = top
    return indices, ref.from_f32(scores, dtype)


def weighted_sum(x: np.ndarray, w: np.ndarray, dtype: int) -> np.ndarray:
    """x [rows, k, D], w [rows, k] as stored; returns [rows, D] as stored."""
    xf, wf = ref.to_f32(x, dtype), ref.to_f32(w, dtype)
    rows, k, d = xf.shape
    lanes = 1 if d == 1 else min(k, 8)
    total = None
    for y in range(lanes):
        t = np.zeros((rows, d), np.float32)
        for j in range(y, k, lanes):
            product = _round(xf[:, j, :] * wf[:, j, None], dtype)
            t = _round(product + t, dtype)
        total = t if y == 0 else _round(t + total, dtype)
    return ref.from_f32(total, dtype)


SWIGLU, SWIGLU_OAI, GEGLU = 0, 1, 2


def _sigmoid(x: np.ndarray) -> np.ndarray:
    """kernels.rs:1539-1543, in float32."""
    x = np.asarray(x, np.float32)
    with np.errstate(over="ignore"):
        y = (np.float32(1.0) / (np.float32(1.0) + np.exp(np.abs(x), dtype=np.float32))).astype(np.float32)
    return np.where(x < 0, y, np.float32(1.0) - y).astype(np.float32)


def _nan_min(a, b):
    """kernels.rs:1367-1368: NaN if either operand is NaN (numpy's minimum does the same)."""
    return np.minimum(a, b).astype(np.float32)


def glu(gate: np.ndarray, up: np.ndarray, dtype: int, activation: int = SWIGLU, alpha: float = 1.702, limit: float = 7.0,
        gate_bias=None, up_bias=None, ids=None) -> np.ndarray:
    """gate, up [rows, hidden] as stored (and biases [experts, hidden] with ids [rows]); returns [rows, hidden] as stored."""
    with np.errstate(invalid="ignore", over="ignore"):  # inf * 0 and inf - inf are NaN, as in the reference
        g, x = ref.to_f32(gate, dtype), ref.to_f32(up, dtype)
        if gate_bias is not None:  # model.rs:2139-2143
            ids = np.asarray(ids).astype(np.int64)
            g = _round(g + ref.to_f32(gate_bias, dtype)[ids], dtype)
            x = _round(x + ref.to_f32(up_bias, dtype)[ids], dtype)
        if activation == SWIGLU:
            s = _round(_sigmoid(g), dtype)              # lib.rs:344
            y = _round(_round(g * s, dtype) * x, dtype)  # lib.rs:344, 517
        elif activation == GEGLU:
            # lib.rs:350-357, 583-590: x^3 is one power (kernels.rs:1375, 1594), the constants weak scalars of the dtype
            k1, k2 = _round(np.float32(0.044715), dtype), _round(np.float32(np.sqrt(2.0 / np.pi)), dtype)
            cube = _round(np.power(g.astype(np.float64), 3.0).astype(np.float32), dtype)
            inner = _round(_round(g + _round(cube * k1, dtype), dtype) * k2, dtype)
            t = _round(np.tanh(inner.astype(np.float64)).astype(np.float32), dtype)
            y = _round(_round(_round(g * np.float32(0.5), dtype) * _round(t + np.float32(1.0), dtype), dtype) * x, dtype)
        else:
            a, l = _round(np.float32(alpha), dtype), _round(np.float32(limit), dtype)  # lib.rs:505-507
            g = _nan_min(g, l)                           # lib.rs:566
            x = _nan_min(np.maximum(x, -l), l)           # lib.rs:567
            s = _round(_sigmoid(_round(a * g, dtype)), dtype)
            y = _round(_round(x + np.float32(1.0), dtype) * _round(g * s, dtype), dtype)  # lib.rs:568-569
    return ref.from_f32(y, dtype)
