"""CPU restatement of nuvec-lm's checkpoint conversions (test infrastructure only: nothing outside
tests/ may import this).

* `mxfp4_from_hf_blocks`: crates/nuvec-lm/src/quant.rs:9-33.
* `convert_packed`: crates/nuvec-lm/src/quant.rs:35-196 (one layer's tensors).

Pinned by the reference's own documented vectors (quant.rs:16-21 and 50-64, in tests/test_formats.py) and by
round trips through the packers AutoAWQ and AutoGPTQ publish (pack integers their way, convert, unpack MLX's
layout: the integers, zeros and scales come back).
"""
import numpy as np

from . import ref

AWQ_ORDER = (0, 4, 1, 5, 2, 6, 3, 7)  # quant.rs:37


def mxfp4_from_hf_blocks(blocks: np.ndarray) -> np.ndarray:
    """uint8 [..., K/32, 16] -> uint32 [..., K/8]: the bytes reinterpreted (quant.rs:22-33)."""
    codes = np.ascontiguousarray(blocks).view(np.uint32)
    if codes.ndim < 2:
        return codes
    return codes.reshape(codes.shape[:-2] + (codes.shape[-2] * codes.shape[-1],))


def convert_packed(qweight, qzeros, scales, dtype, fmt, bits, group):
    """One layer (quant.rs:86-196).  `fmt`: "awq", "gptq" (v1: zeros stored minus one) or "gptq_v2".
    qweight int32 [in, out/8] (AWQ) or [in*bits/32, out] (GPTQ); qzeros likewise along the outputs, or None;
    scales [groups, out] in `dtype` (ref.F16 / ref.BF16 / ref.F32 bit patterns).
    Returns (weight u32 [out, in*bits/32], scales [out, groups], biases [out, groups])."""
    per_word = 32 // bits
    mask = (1 << bits) - 1
    words = np.asarray(qweight).astype(np.int32).view(np.uint32)
    rows, cols = words.shape
    inputs, outputs = (rows, cols * per_word) if fmt == "awq" else (rows * per_word, cols)
    groups = -(-inputs // group)
    if inputs % group != 0 or tuple(scales.shape) != (groups, outputs):
        raise ValueError(f"{inputs} inputs and scales {scales.shape} do not match groups of {group}")
    if fmt == "awq":
        shifts = np.array([4 * AWQ_ORDER[o % per_word] for o in range(outputs)], dtype=np.uint32)
        codes = (words[:, np.arange(outputs) // per_word] >> shifts[None, :]) & mask          # [in, out]
    else:
        i = np.arange(inputs)
        codes = (words[i // per_word, :] >> (bits * (i % per_word)).astype(np.uint32)[:, None]) & mask
    packed = np.zeros((outputs, inputs // per_word), dtype=np.uint32)
    for j in range(per_word):
        packed |= codes[j::per_word, :].T.astype(np.uint32) << np.uint32(bits * j)
    if qzeros is None:
        zeros = np.full((groups, outputs), float(1 << (bits - 1)), dtype=np.float32)
    else:
        zw = np.asarray(qzeros).astype(np.int32).view(np.uint32)
        if zw.shape != (groups, -(-outputs // per_word)):
            raise ValueError(f"qzeros {zw.shape} for {groups} groups of {outputs} outputs")
        o = np.arange(outputs)
        shift = np.array([4 * AWQ_ORDER[k % per_word] for k in o], dtype=np.uint32) if fmt == "awq" else (bits * (o % per_word)).astype(np.uint32)
        offset = 1 if fmt == "gptq" else 0
        zeros = (((zw[:, o // per_word] >> shift[None, :]) & mask) + offset).astype(np.float32)
    # -zero in float32 times the scales in float32, then the scales' dtype; both [out, groups] (quant.rs:171-180)
    product = (-zeros) * ref.to_f32(scales, dtype)
    biases = ref.from_f32(np.ascontiguousarray(product.T.astype(np.float32)), dtype)
    return packed, np.ascontiguousarray(scales.T), biases
