"""Checkpoint conversions (nuvec-lm quant.rs): the oracle against the reference's documented vectors and against
round trips through the packers AutoAWQ / AutoGPTQ publish (no GPU), then the HIP library against the oracle."""
import numpy as np
import pytest

from oracle import formats as fmt_ref
from oracle import ref


def test_hf_blocks_documented_vector():
    """quant.rs:16-21."""
    blocks = np.array([[[[1, 0, 0, 0, 2, 0, 0, 0, 3, 0, 0, 0, 4, 0, 0, 0]]]], dtype=np.uint8)
    codes = fmt_ref.mxfp4_from_hf_blocks(blocks)
    assert codes.shape == (1, 1, 4) and codes.tolist() == [[[1, 2, 3, 4]]]


def test_gptq_documented_vector():
    """quant.rs:50-64: GPTQ v2, 4-bit, 32 inputs (one group), one output: codes 0..16, 0..16 down the inputs,
    zero 8, scale 0.5; the affine layout dequantizes to (code - 8) / 2."""
    words = np.array([[sum((((r * 8 + k) % 16) << (4 * k)) for k in range(8))] for r in range(4)], dtype=np.uint32).view(np.int32)
    zeros = np.array([[8]], dtype=np.int32)
    scales = np.array([[0.5]], dtype=np.float16)
    w, s, b = fmt_ref.convert_packed(words, zeros, scales, ref.F16, "gptq_v2", 4, 32)
    dense = ref.affine_dequantize(w, s, b, ref.F16, 32, 4).astype(np.float32)
    assert dense.reshape(-1).tolist() == [((i % 16) - 8.0) * 0.5 for i in range(32)]


def pack_awq(ints):
    """AutoAWQ's GEMM packing (awq/utils/packing_utils.py, order_map [0, 2, 4, 6, 1, 3, 5, 7]): word c of a row
    takes values 8 c + order_map[i] at nibble i."""
    order_map = [0, 2, 4, 6, 1, 3, 5, 7]
    rows, n = ints.shape
    out = np.zeros((rows, n // 8), dtype=np.uint32)
    for i in range(8):
        out |= ints[:, order_map[i]::8].astype(np.uint32) << np.uint32(4 * i)
    return out.view(np.int32)


def pack_gptq_rows(ints, bits):
    """AutoGPTQ's qweight: values of consecutive inputs fill a word from the low bits (along axis 0)."""
    per = 32 // bits
    out = np.zeros((ints.shape[0] // per, ints.shape[1]), dtype=np.uint32)
    for j in range(per):
        out |= ints[j::per, :].astype(np.uint32) << np.uint32(bits * j)
    return out.view(np.int32)


def pack_gptq_cols(ints, bits):
    """AutoGPTQ's qzeros: values of consecutive outputs fill a word from the low bits (along axis 1)."""
    per = 32 // bits
    out = np.zeros((ints.shape[0], ints.shape[1] // per), dtype=np.uint32)
    for j in range(per):
        out |= ints[:, j::per].astype(np.uint32) << np.uint32(bits * j)
    return out.view(np.int32)


def unpack_mlx(packed, bits):
    per = 32 // bits
    return np.stack([(packed >> np.uint32(bits * j)) & np.uint32((1 << bits) - 1) for j in range(per)], axis=-1).reshape(packed.shape[0], -1)


def make_layer(rng, fmt, bits, group, inputs, outputs, dtype, zeros=True):
    ints = rng.integers(0, 1 << bits, size=(inputs, outputs))
    z = rng.integers(1 if fmt == "gptq" else 0, 1 << bits, size=(inputs // group, outputs))
    scales = ref.from_f32((rng.random((inputs // group, outputs), dtype=np.float32) * 0.1 + 0.001), dtype)
    if fmt == "awq":
        return ints, z, scales, pack_awq(ints), (pack_awq(z) if zeros else None)
    stored = z - 1 if fmt == "gptq" else z
    return ints, z, scales, pack_gptq_rows(ints, bits), (pack_gptq_cols(stored, bits) if zeros else None)


CASES = [("awq", 4, 64, 256, 64), ("gptq", 4, 32, 128, 24), ("gptq_v2", 4, 128, 256, 40), ("gptq", 8, 32, 64, 16), ("gptq_v2", 8, 64, 128, 12)]


@pytest.mark.parametrize("fmt,bits,group,inputs,outputs", CASES)
@pytest.mark.parametrize("dtype", [ref.F16, ref.BF16])
def test_oracle_round_trips_the_published_packers(fmt, bits, group, inputs, outputs, dtype):
    rng = np.random.default_rng(3000 + bits + group + inputs + dtype)
    ints, z, scales, qweight, qzeros = make_layer(rng, fmt, bits, group, inputs, outputs, dtype)
    w, s, b = fmt_ref.convert_packed(qweight, qzeros, scales, dtype, fmt, bits, group)
    assert w.shape == (outputs, inputs * bits // 32) and np.array_equal(unpack_mlx(w, bits), ints.T)
    assert np.array_equal(s.view(np.uint16), scales.T.view(np.uint16))
    # bias = -zero * scale: an integer times the scale, one float32 product rounded to the scales' type
    want = ref.from_f32((-z.T.astype(np.float32)) * ref.to_f32(np.ascontiguousarray(scales.T), dtype), dtype)
    assert np.array_equal(b.view(np.uint16), want.view(np.uint16))
    w2, _, b2 = fmt_ref.convert_packed(qweight, None, scales, dtype, fmt, bits, group)  # symmetric: zero = 2^(bits-1)
    assert np.array_equal(w2, w)
    assert np.array_equal(ref.to_f32(b2, dtype), ref.to_f32(ref.from_f32(-float(1 << (bits - 1)) * ref.to_f32(np.ascontiguousarray(scales.T), dtype), dtype), dtype))


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,bits,group,inputs,outputs", CASES + [("awq", 4, 128, 1024, 512), ("gptq", 4, 128, 2048, 384)])
@pytest.mark.parametrize("dtype", [ref.F16, ref.BF16, ref.F32])
def test_hip_conversion_matches_the_oracle(fmt, bits, group, inputs, outputs, dtype):
    import torch

    import nuvec_amd as nv
    from nuvec_amd import formats
    from tests.hip_backend import to_dev, to_host
    rng = np.random.default_rng(3100 + bits + group + inputs + dtype)
    for zeros in (True, False):
        ints, z, scales, qweight, qzeros = make_layer(rng, fmt, bits, group, inputs, outputs, dtype, zeros)
        want_w, want_s, want_b = fmt_ref.convert_packed(qweight, qzeros, scales, dtype, fmt, bits, group)
        tensors = {"l.qweight": torch.from_numpy(qweight).cuda(), "l.scales": to_dev(scales), "norm.weight": torch.ones(4, device="cuda"),
                   "l.g_idx": torch.arange(inputs, device="cuda") // group}
        if zeros:
            tensors["l.qzeros"] = torch.from_numpy(qzeros).cuda()
        got = formats.convert_packed(tensors, fmt, nv.Quant.affine(group, bits))
        assert sorted(got) == ["l.biases", "l.scales", "l.weight", "norm.weight"]
        assert np.array_equal(to_host(got["l.weight"]), want_w)
        assert np.array_equal(to_host(got["l.scales"]).view(np.uint8), want_s.view(np.uint8))
        assert np.array_equal(to_host(got["l.biases"]).view(np.uint8), want_b.view(np.uint8))
        assert got["norm.weight"].dtype == got["l.scales"].dtype
    # the converted layer is a product operand like any other
    q = nv.Quantized(got["l.weight"], got["l.scales"], got["l.biases"], nv.Quant.affine(group, bits))
    x = ref.from_f32(rng.standard_normal((3, inputs), dtype=np.float32), dtype)
    y = to_host(nv.quantized_matmul(to_dev(x), q))
    want = ref.quantized_matmul(x, want_w, want_s, want_b, group=group, bits=bits, dtype=dtype)
    from tests.test_gpu_parity import assert_rows_close
    assert_rows_close(y, want, dtype, f"converted {fmt} layer b{bits} g{group} {inputs}x{outputs}")
    with pytest.raises(nv.InvalidArgument, match="reorders the inputs"):
        bad = dict(tensors)
        bad["l.g_idx"] = torch.flip(tensors["l.g_idx"], dims=[0])
        formats.convert_packed(bad, fmt, nv.Quant.affine(group, bits))


@pytest.mark.gpu
def test_hf_blocks_view_on_device():
    import torch

    from nuvec_amd import formats
    blocks = torch.arange(2 * 3 * 4 * 16, dtype=torch.int32).to(torch.uint8).reshape(2, 3, 4, 16).cuda()
    codes = formats.mxfp4_from_hf_blocks(blocks)
    assert tuple(codes.shape) == (2, 3, 16)
    assert np.array_equal(codes.cpu().view(torch.int32).numpy().view(np.uint32), fmt_ref.mxfp4_from_hf_blocks(blocks.cpu().numpy()))
