"""Pins of the CPU oracle that do not come from recorded vectors: the known answers the
reference's unit tests hold, closed forms, invariants and brute force on small inputs."""
import ctypes as C
from fractions import Fraction

import numpy as np
import pytest

from oracle import ref

L = ref.lib()


def test_e2m1_known_answers():
    """fp8.rs:185-214: round trips, values, tie thresholds, signed zero, NaN."""
    values = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    for code, v in enumerate(values):
        assert L.nvq_ref_e2m1_to_f32(code) == v and L.nvq_ref_e2m1_to_f32(code | 8) == -v
    for code in range(16):
        assert L.nvq_ref_e2m1_from_f32(L.nvq_ref_e2m1_to_f32(code)) == code
    for x, code in [(0.25, 0), (0.75, 2), (1.25, 2), (1.75, 4), (2.5, 4), (3.5, 6), (5.0, 6), (7.0, 7)]:
        assert L.nvq_ref_e2m1_from_f32(x) == code
    assert L.nvq_ref_e2m1_from_f32(-0.0) == 8
    assert L.nvq_ref_e2m1_from_f32(float("nan")) == 7


def test_e8m0_known_answers():
    """fp8.rs:216-233."""
    tiny = np.array([0x400000], np.uint32).view(np.float32)[0]
    assert L.nvq_ref_e8m0_from_f32(1.0) == 127 and L.nvq_ref_e8m0_from_f32(0.25) == 125
    assert L.nvq_ref_e8m0_from_f32(0.0) == 0 and L.nvq_ref_e8m0_from_f32(-1.0) == 0
    assert L.nvq_ref_e8m0_from_f32(float("inf")) == 0xFF and L.nvq_ref_e8m0_from_f32(float("nan")) == 0xFF
    assert L.nvq_ref_e8m0_to_f32(0) == tiny and L.nvq_ref_e8m0_to_f32(0xFF) == float("inf")
    assert L.nvq_ref_mx_scale_round_up(1.0 / 6.0) == 0.25
    assert L.nvq_ref_mx_scale_round_up(0.0) == tiny
    assert L.nvq_ref_mx_scale_round_up(0.5) == 0.5


def test_e4m3_known_answers():
    """fp8.rs:137-183: MLX's probes and every code's round trip."""
    nan, inf = float("nan"), float("inf")
    values = [0.1, 1.0, 448.0, 500.0, -3.3, 1e-4, 0.0, -0.0, inf, -inf, nan, 2.0 ** -9, 2.0 ** -10, 0.0029296875, 464.0,
              465.0, 1.0625, 1.1875]
    expected = [29, 56, 126, 126, 197, 0, 0, 128, 126, 254, 126, 1, 0, 2, 126, 126, 56, 58]
    assert [L.nvq_ref_e4m3_from_f32(v) for v in values] == expected
    for code, v in [(0, 0.0), (1, 0.001953125), (7, 0.013671875), (8, 0.015625), (56, 1.0), (126, 448.0), (254, -448.0)]:
        assert L.nvq_ref_e4m3_to_f32(code) == v
    for code in range(256):
        if code & 0x7F != 0x7F:
            assert L.nvq_ref_e4m3_from_f32(L.nvq_ref_e4m3_to_f32(code)) == code


def test_mx_scale_is_the_smallest_power_of_two_not_below():
    """Closed form of mx_scale_round_up on normal inputs: exponent + (mantissa != 0)."""
    rng = np.random.default_rng(3)
    xs = np.concatenate([np.exp2(rng.uniform(-100, 100, 2000)).astype(np.float32), np.exp2(np.arange(-100, 100)).astype(np.float32)])
    for x in xs:
        u = int(np.array([x], np.float32).view(np.uint32)[0])
        want = min((u >> 23) + ((u & 0x7FFFFF) != 0), 254)
        assert L.nvq_ref_e8m0_from_f32(L.nvq_ref_mx_scale_round_up(float(x))) == want


def test_code_is_a_little_endian_bit_stream():
    """kernels.rs:749-756 against brute force over an integer made of the bytes."""
    rng = np.random.default_rng(4)
    data = rng.integers(0, 256, 64, dtype=np.uint8)
    big = int.from_bytes(data.tobytes(), "little")
    for bits in (1, 2, 3, 4, 5, 6, 8):
        for i in range(64 * 8 // bits - 1):
            got = L.nvq_ref_code(data.ctypes.data_as(C.POINTER(C.c_uint8)), C.c_int64(i), bits)
            assert got == (big >> (i * bits)) & ((1 << bits) - 1)


@pytest.mark.parametrize("dtype", [ref.F32, ref.BF16, ref.F16])
@pytest.mark.parametrize("bits", [2, 3, 4, 5, 6, 8])
@pytest.mark.parametrize("group", [32, 64, 128])
def test_round_trip_within_one_step(dtype, bits, group):
    """crates/nuvec-core/tests/quantized.rs:69-96: error at most one step, mean at most half a step."""
    rng = np.random.default_rng(bits * 131 + group)
    w = ref.from_f32(rng.standard_normal((8, 4 * group)).astype(np.float32), dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
    back = ref.to_f32(ref.affine_dequantize(packed, scales, biases, dtype, group, bits), dtype)
    step = np.repeat(np.abs(ref.to_f32(scales, dtype)), group, axis=-1)
    err = np.abs(back - ref.to_f32(w, dtype))
    eps = {ref.F32: 1e-6, ref.BF16: 2.0 ** -7, ref.F16: 2.0 ** -10}[dtype]
    slack = eps * (np.abs(back) + step * ((1 << bits) - 1))
    assert np.all(err <= step + slack)
    assert float(np.mean(err / step)) <= 0.5 + 0.05


def test_constant_and_zero_groups():
    """quantized.rs:98-125: a constant group and an exact zero are representable."""
    w = np.full((2, 64), 0.375, np.float32)
    p, s, b = ref.affine_quantize(w, ref.F32, 64, 4)
    assert np.array_equal(ref.affine_dequantize(p, s, b, ref.F32, 64, 4), w)
    w = np.linspace(-1, 2, 128, dtype=np.float32).reshape(2, 64)
    w[0, 5] = 0.0
    p, s, b = ref.affine_quantize(w, ref.F32, 64, 4)
    assert ref.affine_dequantize(p, s, b, ref.F32, 64, 4)[0, 5] == 0.0


def exact_dot(x, w):
    return float(sum(Fraction(float(a)) * Fraction(float(b)) for a, b in zip(x, w)))


def test_few_rows_order_invariants():
    """few_rows.rs:336-395: close to the exact dot product (1e-5 sqrt K), independent of the weight
    layout (stride), and unchanged by zero padding of the reduction."""
    rng = np.random.default_rng(9)
    for k in (1, 7, 8, 9, 64, 100, 1000):
        x = rng.standard_normal(k).astype(np.float32)
        w = rng.standard_normal(k).astype(np.float32)
        fp = lambda a: a.ctypes.data_as(C.POINTER(C.c_float))
        got = L.nvq_ref_dot_few_rows(fp(x), fp(w), C.c_int64(1), C.c_int64(k))
        assert abs(got - exact_dot(x, w)) <= 1e-5 * np.sqrt(k) * max(1.0, float(np.max(np.abs(x)) * np.max(np.abs(w))))
        strided = np.zeros(3 * k, np.float32)
        strided[::3] = w
        assert L.nvq_ref_dot_few_rows(fp(x), fp(strided), C.c_int64(3), C.c_int64(k)) == got
        xp, wp = np.concatenate([x, np.zeros(13, np.float32)]), np.concatenate([w, np.ones(13, np.float32)])
        assert L.nvq_ref_dot_few_rows(fp(xp), fp(wp), C.c_int64(1), C.c_int64(k + 13)) == got
    # the fixed tree: partial p mod 8, combined ((s0+s4)+(s2+s6))+((s1+s5)+(s3+s7))
    x = np.array([1e8, 1, -1e8, 1, 1, 1, 1, 1], np.float32)
    w = np.ones(8, np.float32)
    f = np.float32
    want = ((f(1e8) + f(1)) + (f(-1e8) + f(1))) + ((f(1) + f(1)) + (f(1) + f(1)))
    assert L.nvq_ref_dot_few_rows(x.ctypes.data_as(C.POINTER(C.c_float)), w.ctypes.data_as(C.POINTER(C.c_float)), C.c_int64(1), C.c_int64(8)) == want


def test_product_equals_x_times_dequantized_weights():
    """quantized.rs:168-215: quantized_matmul == x . dequantize(w)^T, here against an exact rational product."""
    rng = np.random.default_rng(12)
    for bits, group, dtype in [(4, 64, ref.F32), (3, 32, ref.BF16), (8, 128, ref.F16), (2, 64, ref.BF16)]:
        n, k, m = 5, 2 * group, 3
        w = ref.from_f32((rng.standard_normal((n, k)) * 0.1).astype(np.float32), dtype)
        x = ref.from_f32(rng.standard_normal((m, k)).astype(np.float32), dtype)
        p, s, b = ref.affine_quantize(w, dtype, group, bits)
        dense = ref.to_f32(ref.affine_dequantize(p, s, b, dtype, group, bits), dtype)
        y = ref.to_f32(ref.quantized_matmul(x, p, s, b, group=group, bits=bits, dtype=dtype), dtype)
        x32 = ref.to_f32(x, dtype)
        for i in range(m):
            for j in range(n):
                want = exact_dot(x32[i], dense[j])
                tol = {ref.F32: 1e-6, ref.BF16: 2.0 ** -8, ref.F16: 2.0 ** -11}[dtype] * max(1.0, abs(want)) + 1e-5
                assert abs(float(y[i, j]) - want) <= tol
    # transpose=False reads the same dense matrix the other way
    w = (rng.standard_normal((64, 64)) * 0.1).astype(np.float32)
    x = rng.standard_normal((2, 64)).astype(np.float32)
    p, s, b = ref.affine_quantize(w, ref.F32, 64, 4)
    dense = ref.affine_dequantize(p, s, b, ref.F32, 64, 4)
    y = ref.quantized_matmul(x, p, s, b, group=64, bits=4, dtype=ref.F32, transpose=False)
    assert np.allclose(y, x.astype(np.float64) @ dense.astype(np.float64), rtol=1e-5, atol=1e-5)


def test_sorted_offsets_is_a_lower_bound():
    rng = np.random.default_rng(5)
    for rows, groups in [(0, 4), (1, 1), (40, 8), (1024, 32)]:
        rhs = np.sort(rng.integers(0, groups, rows)).astype(np.uint32)
        got = ref.sorted_offsets(rhs, groups)
        assert np.array_equal(got, np.searchsorted(rhs, np.arange(groups), side="left").astype(np.int32))
        assert np.array_equal(got, np.array([int(np.sum(rhs < g)) for g in range(groups)], np.int32))


def test_gather_equals_per_pair_products():
    """quantized.rs:506-527."""
    rng = np.random.default_rng(6)
    e, n, k, m = 4, 6, 64, 2
    w = (rng.standard_normal((e, n, k)) * 0.1).astype(np.float32)
    x = rng.standard_normal((3, m, k)).astype(np.float32)
    p, s = ref.fp_quantize(w, ref.F32, ref.MXFP4)
    lhs, rhs = np.array([2, 0, 1, 1], np.uint32), np.array([3, 3, 0, 2], np.uint32)
    y = ref.gather_qmm(x, p, s, None, lhs, rhs, mode=ref.MXFP4, group=32, bits=4, dtype=ref.F32)
    for i in range(4):
        one = ref.quantized_matmul(x[lhs[i]], p[rhs[i]], s[rhs[i]], None, mode=ref.MXFP4, group=32, bits=4, dtype=ref.F32)
        assert np.array_equal(y[i], one)


# ── the mixture-of-experts glue (oracle/moe.py) ─────────────────────────────────────────

def test_moe_route_documented_examples():
    """crates/nuvec-core/src/fast.rs:733-737 and crates/nuvec-core/tests/fast.rs:900-911."""
    from oracle import moe
    top, scores = moe.moe_route(np.array([[0.1, 0.4, 0.2, 0.3]], np.float32), ref.F32, 2, True)
    assert top.tolist() == [[3, 1]]
    assert abs(scores[0, 0] - 0.3 / 0.7) < 1e-6 and abs(scores[0, 1] - 0.4 / 0.7) < 1e-6
    nan_row = np.array([[0.1, np.nan, 0.3, 0.2]], np.float32)
    assert moe.moe_route(nan_row, ref.F32, 2, False)[0].tolist() == [[2, 1]]
    assert moe.moe_route(ref.from_f32(nan_row, ref.F16), ref.F16, 2, False)[0].tolist() == [[2, 1]]


@pytest.mark.parametrize("dtype", [ref.F32, ref.F16, ref.BF16])
def test_moe_route_is_the_tail_of_a_stable_sort(dtype):
    """The indices are the last k of numpy's stable ascending argsort (ties in index order), the scores the taken
    values, normalized ones within a rounding of the float64 quotient (crates/nuvec-core/tests/fast.rs:831-839)."""
    from oracle import moe
    rng = np.random.default_rng(72)
    for rows, e, ks in [(3, 8, (1, 2, 8)), (5, 60, (4, 8)), (2, 128, (1, 10, 128))]:
        logits = rng.standard_normal((rows, e)).astype(np.float32)
        p = np.exp(logits) / np.exp(logits).sum(-1, keepdims=True)
        ties = (np.floor(p * 4 * e) + 1) / (4 * e)  # a few values repeated across experts
        for probs in (p, ties):
            stored = ref.from_f32(probs.astype(np.float32), dtype)
            wide = ref.to_f32(stored, dtype).astype(np.float64)
            for k in ks:
                want = np.argsort(wide, axis=-1, kind="stable")[:, -k:]
                top, scores = moe.moe_route(stored, dtype, k, False)
                assert np.array_equal(top, want)
                assert np.array_equal(ref.to_f32(scores, dtype), np.take_along_axis(wide, want, -1).astype(np.float32))
                _, normalized = moe.moe_route(stored, dtype, k, True)
                taken = np.take_along_axis(wide, want, -1)
                exact = taken / taken.sum(-1, keepdims=True)
                eps = {ref.F32: 2.0 ** -23, ref.F16: 2.0 ** -10, ref.BF16: 2.0 ** -7}[dtype]
                assert np.all(np.abs(ref.to_f32(normalized, dtype) - exact) <= (k + 2) * eps * np.abs(exact) + 1e-30)


@pytest.mark.parametrize("dtype", [ref.F32, ref.F16, ref.BF16])
def test_weighted_sum_equals_multiply_and_sum(dtype):
    """crates/nuvec-core/tests/fast.rs:955-987: sum(x * w[..., None], -2) within the rounding of k products and sums."""
    from oracle import moe
    rng = np.random.default_rng(73)
    eps = {ref.F32: 2.0 ** -23, ref.F16: 2.0 ** -10, ref.BF16: 2.0 ** -7}[dtype]
    for rows, k, d in [(3, 1, 64), (2, 4, 7), (3, 10, 64), (2, 16, 1), (1, 31, 96)]:
        x = ref.from_f32(rng.standard_normal((rows, k, d)).astype(np.float32), dtype)
        w = ref.from_f32(rng.standard_normal((rows, k)).astype(np.float32), dtype)
        got = ref.to_f32(moe.weighted_sum(x, w, dtype), dtype).astype(np.float64)
        xf, wf = ref.to_f32(x, dtype).astype(np.float64), ref.to_f32(w, dtype).astype(np.float64)
        exact = (xf * wf[..., None]).sum(-2)
        bound = (k + 1) * eps * (np.abs(xf) * np.abs(wf[..., None])).sum(-2)
        assert np.all(np.abs(got - exact) <= bound + 1e-30)
    # one weighted row is the rounded product itself
    x = ref.from_f32(rng.standard_normal((2, 1, 5)).astype(np.float32), dtype)
    w = ref.from_f32(rng.standard_normal((2, 1)).astype(np.float32), dtype)
    want = ref.from_f32((ref.to_f32(x, dtype)[:, 0] * ref.to_f32(w, dtype)).astype(np.float32), dtype)
    assert np.array_equal(moe.weighted_sum(x, w, dtype).view(np.uint8), want.view(np.uint8))


def test_glu_documented_example_and_clamps():
    """crates/nuvec-nn/src/lib.rs:555-560: swiglu_oai([10, -1], [9, 0.5], 1.702, 7)[0] = 8 * 7 / (1 + exp(-1.702 * 7));
    the gate is clamped from above only, the other operand on both sides; NaN stays NaN."""
    from oracle import moe
    y = moe.glu(np.array([[10.0, -1.0]], np.float32), np.array([[9.0, 0.5]], np.float32), ref.F32, moe.SWIGLU_OAI, 1.702, 7.0)
    assert abs(float(y[0, 0]) - 8.0 * 7.0 / (1.0 + np.exp(-1.702 * 7.0))) < 1e-4
    assert abs(float(y[0, 1]) - 1.5 * -1.0 / (1.0 + np.exp(1.702))) < 1e-6
    low = moe.glu(np.array([[-20.0, 3.0]], np.float32), np.array([[-50.0, 50.0]], np.float32), ref.F32, moe.SWIGLU_OAI, 1.702, 7.0)
    assert abs(float(low[0, 0]) - (-7.0 + 1.0) * -20.0 / (1.0 + np.exp(1.702 * 20.0))) < 1e-6  # gate below -limit is kept
    assert abs(float(low[0, 1]) - 8.0 * 3.0 / (1.0 + np.exp(-1.702 * 3.0))) < 1e-5
    nan = moe.glu(np.array([[np.nan, 1.0]], np.float32), np.array([[1.0, np.nan]], np.float32), ref.F32, moe.SWIGLU_OAI)
    assert np.isnan(nan).all()
    assert np.isnan(moe.glu(np.array([[np.nan]], np.float32), np.array([[1.0]], np.float32), ref.F32, moe.SWIGLU)).all()


@pytest.mark.parametrize("dtype", [ref.F32, ref.F16, ref.BF16])
def test_glu_equals_the_closed_forms(dtype):
    """silu(g) * x and the clamped form in float64, within the roundings of the element type (three and five
    operations); each row's expert's bias is added to both operands first."""
    from oracle import moe
    rng = np.random.default_rng(40 + dtype)
    eps = {ref.F32: 2.0 ** -23, ref.F16: 2.0 ** -10, ref.BF16: 2.0 ** -7}[dtype]
    rows, hidden, experts = 37, 50, 5
    g = ref.from_f32((rng.standard_normal((rows, hidden)) * 4).astype(np.float32), dtype)
    x = ref.from_f32((rng.standard_normal((rows, hidden)) * 4).astype(np.float32), dtype)
    gb = ref.from_f32(rng.standard_normal((experts, hidden)).astype(np.float32), dtype)
    xb = ref.from_f32(rng.standard_normal((experts, hidden)).astype(np.float32), dtype)
    ids = rng.integers(0, experts, rows)
    for biased in (False, True):
        g64, x64 = ref.to_f32(g, dtype).astype(np.float64), ref.to_f32(x, dtype).astype(np.float64)
        if biased:  # the sums as the element type rounds them
            g64 = ref.to_f32(ref.from_f32((g64 + ref.to_f32(gb, dtype)[ids]).astype(np.float32), dtype), dtype).astype(np.float64)
            x64 = ref.to_f32(ref.from_f32((x64 + ref.to_f32(xb, dtype)[ids]).astype(np.float32), dtype), dtype).astype(np.float64)
        kw = dict(gate_bias=gb, up_bias=xb, ids=ids) if biased else {}
        got = ref.to_f32(moe.glu(g, x, dtype, moe.SWIGLU, **kw), dtype).astype(np.float64)
        want = g64 / (1.0 + np.exp(-g64)) * x64
        # (float16 rounds a sigmoid or a product below 2^-14 to a multiple of 2^-24)
        tiny = 2.0 ** -24 if dtype == ref.F16 else 0.0
        assert np.all(np.abs(got - want) <= 4 * eps * np.abs(want) + tiny * (np.abs(g64 * x64) + np.abs(x64) + 1.0) + 1e-30)
        alpha = float(ref.to_f32(ref.from_f32(np.array([1.702], np.float32), dtype), dtype)[0])
        got = ref.to_f32(moe.glu(g, x, dtype, moe.SWIGLU_OAI, 1.702, 7.0, **kw), dtype).astype(np.float64)
        gc, xc = np.minimum(g64, 7.0), np.clip(x64, -7.0, 7.0)
        want = (xc + 1.0) * gc / (1.0 + np.exp(-alpha * gc))
        # (x + 1 may cancel: its rounding error is relative to |x| + 1, not to the sum)
        slack = 6 * eps * np.abs(want) + 2 * eps * np.abs(gc / (1.0 + np.exp(-alpha * gc))) * (np.abs(xc) + 1.0)
        # the rounded product alpha * g moves the sigmoid by up to |alpha g| eps / 4 (its slope is at most 1 / 4)
        slack += np.abs(xc + 1.0) * np.abs(gc) * np.abs(alpha * gc) * eps / 4
        slack += tiny * (np.abs((xc + 1.0) * gc) + np.abs(xc + 1.0) + 1.0)
        assert np.all(np.abs(got - want) <= slack + 1e-30)


def test_glu_equals_the_activations_mlx_lm_recorded():
    """The reference's own test of its gated activations (crates/nuvec-nn/tests/rope_scaling.rs:150-172) holds what
    mlx-lm computed for `swiglu_oai(gate, x, 1.702, 7)` and `geglu(gate, x)` in float32 and bfloat16 and asks for 1e-6
    and 1e-2 of max(|value|, 1) for every element (its `close`).  The oracle meets those bounds; how many outputs agree bit for bit is
    printed (MLX's GPU kernels evaluate the fused graph in float32 and round once, the reference's CPU path and the
    oracle round after every operation)."""
    import os

    import torch
    from safetensors.torch import load_file as load_torch

    from oracle import moe
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mlx_lm_activations.safetensors")
    recorded = load_torch(path)
    for label, dtype, tol in (("f32", ref.F32, 1e-6), ("bf16", ref.BF16, 1e-2)):
        def stored(name):
            t = recorded[f"act_{label}.{name}"]
            return t.numpy() if dtype == ref.F32 else t.view(torch.int16).numpy().view(np.uint16)
        gate, x = stored("gate"), stored("x")
        assert gate.shape == (4, 33)
        for name, activation in (("swiglu_oai", moe.SWIGLU_OAI), ("geglu", moe.GEGLU)):
            got = ref.to_f32(moe.glu(gate, x, dtype, activation, 1.702, 7.0), dtype).astype(np.float64)
            want = ref.to_f32(stored(name), dtype).astype(np.float64)
            ratio = np.abs(got - want) / (tol * np.maximum(np.abs(want), 1.0))  # the rule of the reference's `close` (rope_scaling.rs:37-43)
            print(f"{label} {name}: worst difference {float(ratio.max()):.3f} x the bound, {int(np.count_nonzero(got == want))} of {want.size} equal")
            assert float(ratio.max()) <= 1.0, (label, name)


@pytest.mark.parametrize("dtype", [ref.F32, ref.F16, ref.BF16])
def test_geglu_equals_the_closed_form(dtype):
    """0.5 g (1 + tanh(sqrt(2 / pi) (g + 0.044715 g^3))) x in float64 with the constants as the element type holds them,
    within the roundings of the eight operations; the cube of a 16-bit element is the correctly rounded one."""
    from oracle import moe
    rng = np.random.default_rng(60 + dtype)
    eps = {ref.F32: 2.0 ** -23, ref.F16: 2.0 ** -10, ref.BF16: 2.0 ** -7}[dtype]
    g = ref.from_f32((rng.standard_normal((29, 64)) * 3).astype(np.float32), dtype)
    x = ref.from_f32((rng.standard_normal((29, 64)) * 3).astype(np.float32), dtype)
    g64, x64 = ref.to_f32(g, dtype).astype(np.float64), ref.to_f32(x, dtype).astype(np.float64)
    k1 = float(ref.to_f32(ref.from_f32(np.array([0.044715], np.float32), dtype), dtype)[0])
    k2 = float(ref.to_f32(ref.from_f32(np.array([np.sqrt(2.0 / np.pi)], np.float32), dtype), dtype)[0])
    inner = k2 * (g64 + k1 * g64 ** 3)
    want = 0.5 * g64 * (1.0 + np.tanh(inner)) * x64
    got = ref.to_f32(moe.glu(g, x, dtype, moe.GEGLU), dtype).astype(np.float64)
    # the argument of tanh carries about four roundings (slope of tanh at most 1); 1 + tanh cancels for negative gates:
    # its error is relative to 1, not to the sum
    slack = 4 * eps * np.abs(want) + np.abs(0.5 * g64 * x64) * (4 * eps * np.abs(inner) * (1.0 - np.tanh(inner) ** 2) + 2 * eps)
    tiny = 2.0 ** -24 if dtype == ref.F16 else 0.0
    assert np.all(np.abs(got - want) <= slack + tiny * (np.abs(x64) + 1.0) + 1e-30)
    if dtype != ref.F32:  # the cube: exact product, one rounding
        cube = ref.to_f32(ref.from_f32((g64 ** 3).astype(np.float32), dtype), dtype)
        again = ref.to_f32(ref.from_f32(np.power(ref.to_f32(g, dtype), np.float32(3.0)), dtype), dtype)
        assert np.array_equal(cube, again)
    assert np.isnan(ref.to_f32(moe.glu(ref.from_f32(np.array([[np.nan]], np.float32), dtype), x[:1, :1], dtype, moe.GEGLU), dtype)).all()
