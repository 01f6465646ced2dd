"""HIP path against the CPU oracle on the same seeded inputs (the BASELINE configurations).

Bars: packed words, scales and biases bit-exact; dequantize bit-exact; product outputs within
1e-2 * max|row| for bfloat16 and 1e-4 * max|row| for float32 (float32 accumulation), `row` being
the oracle's output row.  float16 has no stated bar: it gets the bfloat16 bar scaled by the ratio
of the formats' unit roundoffs (2.56 output ulps at the row maximum in both), 1.25e-3 * max|row|
times two because the float16 dequantized weights are themselves rounded once here and twice on
the CPU: 2.5e-3 * max|row|.

How the half-precision bar is applied.  EVERY output of every product is held to the bar against the
CPU oracle (`assert_rows_close`), and the worst ratio error / bar of each case is printed and appended to
a `parity_ratios.txt` in the run's output folder so that a run's record holds the margin.  The kernels compute in the
arithmetic of the reference's device kernels (weights dequantized with one rounding of
fma(code, scale, bias), or not rounded at all in the decode kernels) while the reference's CPU path rounds
the dequantized weights twice in the element type; a second check (`assert_device_arithmetic`) holds every
output to HALF the bar against an oracle in that device arithmetic.
"""
import os

import numpy as np
import pytest
import torch

import nuvec_amd as nv
from oracle import ref
from tests.hip_backend import TORCH, to_dev, to_host

pytestmark = pytest.mark.gpu

TOL = {ref.BF16: 1e-2, ref.F16: 2.5e-3, ref.F32: 1e-4}


def make_w(rng, n, k, dtype):
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    return ref.from_f32(w, dtype)


def make_x(rng, m, k, dtype):
    return ref.from_f32(rng.standard_normal((m, k)).astype(np.float32), dtype)


def _excess(got, want, dtype):
    """|got - want| over the bar of each output's row."""
    g, w = ref.to_f32(got, dtype).astype(np.float64), ref.to_f32(want, dtype).astype(np.float64)
    g, w = g.reshape(-1, g.shape[-1]), w.reshape(-1, w.shape[-1])
    bound = TOL[dtype] * np.max(np.abs(w), axis=1, keepdims=True)
    return np.abs(g - w) / np.maximum(bound, 1e-30)


RATIOS = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out", "parity_ratios.txt")


def record_ratio(what, worst, count):
    """The worst error of a case as a fraction of its bar: printed (pytest -rA shows it) and kept on file."""
    line = f"{what}: worst error {worst:.3f} x the bar over {count} outputs"
    print(line, flush=True)
    try:
        os.makedirs(os.path.dirname(RATIOS), exist_ok=True)
        with open(RATIOS, "a") as f:
            f.write(line + "\n")
    except OSError:
        pass


def assert_rows_close(got, want, dtype, what, exact_weights=False):
    """Against the CPU oracle: every output within the bar of its row (1e-2 * max|row| for bfloat16), whatever the
    length of the row.  (Half-precision affine products of fewer than 1024 outputs per row, whose bar is tightest, run
    on kernels that materialise the CPU's doubly rounded weights; `exact_weights` marks the block formats, whose weights
    both sides hold exactly.)"""
    ratio = _excess(got, want, dtype)
    worst = float(np.max(ratio)) if ratio.size else 0.0
    record_ratio(what, worst, ratio.size)
    beyond = int(np.count_nonzero(ratio > 1.0))
    assert worst <= 1.0, f"{what}: max error is {worst:.3f} x the bound, {beyond} of {ratio.size} outputs beyond it"


def assert_device_arithmetic(got, x, packed, scales, biases, group, bits, dtype, what, limit=0.5):
    """Against the arithmetic of the kernel that ran: every output within half the bar.  The reference's device
    kernels come in two forms (weights rounded once in the tiled kernels, never in the vector kernels); which one a
    product takes here is a routing matter, so either is accepted; rows of fewer than 1024 outputs, and bfloat16
    products of more than 16 rows up to 8192 outputs, take the CPU's own weights (two roundings), i.e. the CPU oracle
    itself."""
    forms = [ref.quantized_matmul_device(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, rounded_weights=r) for r in (True, False)]
    rows, outputs = np.asarray(got).shape[-2:]
    if outputs < 1024 or (dtype == ref.BF16 and rows > 16 and outputs < 8192):  # the products that take the CPU's own weights
        forms = [ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, threads=8)]
    worst = min(float(np.max(_excess(got, form, dtype))) for form in forms)
    assert worst <= limit, f"{what}: max error against the device arithmetic is {worst:.3f} x the bound"


@pytest.mark.parametrize("dtype", [ref.F32, ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(64, 4), (64, 3), (32, 8), (128, 2), (32, 6), (64, 5), (128, 1)])
def test_affine_quantize_dequantize_bit_exact(dtype, group, bits):
    rng = np.random.default_rng(1000 + bits * 7 + group)
    w = make_w(rng, 96, 1024, dtype)
    w.reshape(-1)[::97] = ref.from_f32(np.zeros(1, np.float32), dtype)[0]  # exact zeros among the values
    packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
    q = nv.quantize(to_dev(w), nv.Quant.affine(group, bits))
    assert np.array_equal(to_host(q.weight), packed)
    assert np.array_equal(to_host(q.scales).view(np.uint8), scales.view(np.uint8))
    assert np.array_equal(to_host(q.biases).view(np.uint8), biases.view(np.uint8))
    want = ref.affine_dequantize(packed, scales, biases, dtype, group, bits)
    got = to_host(nv.dequantize(q))
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("dtype", [ref.F32, ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(32, 4), (64, 4), (128, 4), (64, 3), (32, 8), (64, 2), (128, 6), (32, 5), (64, 1)])
def test_affine_quantize_ties_specials_and_tails(dtype, group, bits):
    """Groups whose quotients are exact halves or one unit in the last place from a half (the rounding the kernel
    must take from the true division), zeros of both signs, NaN (quiet and signalling), infinities, a constant
    group and tiny ranges; a number of rows that fills neither a wavefront nor a group of lanes."""
    rng = np.random.default_rng(31 * bits + group)
    n_bins, groups = (1 << bits) - 1, 37
    w = np.zeros((groups, group), np.float32)
    for g in range(groups):
        top = float(2.0 ** int(rng.integers(-3, 4))) * n_bins
        codes = rng.integers(0, n_bins + 1, group).astype(np.float32)
        half = rng.integers(0, 2, group).astype(np.float32) * 0.5
        v = np.minimum(codes + half, n_bins) * (top / n_bins)
        v[:2] = (0.0, top)
        w[g] = v if g % 2 else -v
    w = ref.to_f32(ref.from_f32(w, dtype), dtype)
    near = w.view(np.uint32).copy()
    if dtype == ref.F32:
        near[5::3, 7::5] += 1  # one unit in the last place beside the ties
        near[6::3, 9::5] -= 1
    w = near.view(np.float32)
    w[3, :] = 0.0
    w[3, ::3] = -0.0
    w[4, :] = -0.0
    w[7, :] = 1.25
    w[8, 3] = np.nan
    w[9, 5] = np.inf
    w[10, 6] = -np.inf
    w[11, :] = np.float32(1.0) + np.arange(group, dtype=np.float32) * np.float32(2.0 ** -20 if dtype == ref.F32 else 2.0 ** -7)
    bits_w = w.view(np.uint32)
    bits_w[12, 4] = 0x7F810000  # a signalling NaN in every element type's range
    bits_w[13, :] = 0x00010000 * (1 + np.arange(group, dtype=np.uint32) % 5)  # float32 subnormals
    stored = ref.from_f32(w, dtype)
    if dtype != ref.F32:  # the conversion above quiets the signalling NaN: put its bits back
        raw = stored.view(np.uint16)
        raw[12, 4] = 0x7F81 if dtype == ref.BF16 else 0x7D01
    packed, scales, biases = ref.affine_quantize(stored, dtype, group, bits)
    q = nv.quantize(to_dev(stored), nv.Quant.affine(group, bits))
    assert np.array_equal(to_host(q.weight), packed)
    assert np.array_equal(to_host(q.scales).view(np.uint8), scales.view(np.uint8))
    assert np.array_equal(to_host(q.biases).view(np.uint8), biases.view(np.uint8))


def test_config1_fp32_4bit_g64():
    """BASELINE config 1: W f32 [4096,4096] ~ N(0,0.02), x f32 [1,4096], 4-bit g64."""
    rng = np.random.default_rng(20260101)
    w, x = make_w(rng, 4096, 4096, ref.F32), make_x(rng, 1, 4096, ref.F32)
    packed, scales, biases = ref.affine_quantize(w, ref.F32, 64, 4)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    assert np.array_equal(to_host(q.weight), packed)
    assert np.array_equal(to_host(q.scales), scales) and np.array_equal(to_host(q.biases), biases)
    want_dense = ref.affine_dequantize(packed, scales, biases, ref.F32, 64, 4)
    assert np.array_equal(to_host(nv.dequantize(q)), want_dense)
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.F32, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert got.shape == (1, 4096)
    assert_rows_close(got, want, ref.F32, "config 1")


@pytest.mark.parametrize("m", [1, 4, 8])
def test_config2_decode_bf16_4bit_g64(m):
    """BASELINE config 2: W [14336,4096] bf16 scales/biases, x bf16 [M,4096]."""
    rng = np.random.default_rng(20260102)
    w, x = make_w(rng, 14336, 4096, ref.BF16), make_x(rng, m, 4096, ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 4)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    assert np.array_equal(to_host(q.weight), packed)
    assert np.array_equal(to_host(q.scales), scales) and np.array_equal(to_host(q.biases), biases)
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.BF16, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, ref.BF16, f"config 2, M={m}")
    assert_device_arithmetic(got, x, packed, scales, biases, 64, 4, ref.BF16, f"config 2, M={m}")


@pytest.mark.parametrize("group,bits", [(64, 3), (32, 8)])
@pytest.mark.parametrize("m", [1, 16])
def test_config4_odd_bit_widths(group, bits, m):
    """BASELINE config 4: 3-bit g64 (codes cross word boundaries) and 8-bit g32, W [4096,4096]."""
    rng = np.random.default_rng(20260104 + bits)
    w, x = make_w(rng, 4096, 4096, ref.BF16), make_x(rng, m, 4096, ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, group, bits)
    q = nv.quantize(to_dev(w), nv.Quant.affine(group, bits))
    assert np.array_equal(to_host(q.weight), packed)
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=ref.BF16, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, ref.BF16, f"config 4 b{bits} g{group} M={m}")
    assert_device_arithmetic(got, x, packed, scales, biases, group, bits, ref.BF16, f"config 4 b{bits} g{group} M={m}")


@pytest.mark.parametrize("group,bits", [(64, 3), (32, 8)])
def test_config4_odd_bit_widths_512_rows(group, bits):
    """BASELINE config 4 at M = 512: the tiled kernel with K split over the grid and the partial sums added from the
    caller's workspace, and the same product handed no workspace (K not split).  The whole product against the oracle."""
    import ctypes as C

    from nuvec_amd import _lib
    rng = np.random.default_rng(20260104 + bits)
    m, n, k = 512, 4096, 4096
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, group, bits)
    q = nv.quantize(to_dev(w), nv.Quant.affine(group, bits))
    assert np.array_equal(to_host(q.weight), packed)
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=ref.BF16, threads=8)
    d = _lib.QmmDescC()
    d.quant, d.dtype, d.transpose = nv.Quant.affine(group, bits)._c(), _lib.BF16, 1
    d.m, d.n, d.k, d.item_rows = m, n, k, m
    need = _lib.load().nvq_quantized_matmul_workspace_bytes(C.byref(d))
    assert need > 0, "this product is expected to split K through a workspace"
    xd = to_dev(x)
    split = to_host(nv.quantized_matmul(xd, q))
    assert_rows_close(split, want, ref.BF16, f"config 4 b{bits} g{group} M=512, K split through the workspace")
    some = np.sort(rng.choice(m, 48, replace=False))
    assert_device_arithmetic(split[some], x[some], packed, scales, biases, group, bits, ref.BF16, f"config 4 b{bits} g{group} M=512")
    unsplit = to_host(nv.quantized_matmul(xd, q, scratch=False))
    assert_rows_close(unsplit, want, ref.BF16, f"config 4 b{bits} g{group} M=512, no workspace")


def test_untransposed_product_needs_its_workspace():
    """Weights stored [K, N] split K through the caller's workspace: handed none, the call is refused, not run."""
    rng = np.random.default_rng(3)
    k, n, m = 480, 256, 3  # (K is no multiple of 64: the vector kernel, which cannot run unsplit)
    w, x = make_w(rng, k, n, ref.BF16), make_x(rng, m, k, ref.BF16)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    assert nv.quantized_matmul_route(m, n, k, q.quant, torch.bfloat16, transpose=False) == "qvm_kernel"
    y = nv.quantized_matmul(to_dev(x), q, transpose=False)
    assert y.shape == (m, n)
    with pytest.raises((nv.InvalidArgument, nv.Unsupported)):
        nv.quantized_matmul(to_dev(x), q, transpose=False, scratch=False)


@pytest.mark.parametrize("dtype", [ref.F32, ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(64, 4), (32, 2), (128, 6), (64, 5), (128, 1), (32, 3), (64, 8)])
def test_ragged_shapes_every_width(dtype, group, bits):
    """N not a multiple of the rows per block, K not a multiple of the wavefront step, M = 3."""
    rng = np.random.default_rng(7 + bits)
    n, k, m = 77, 2 * 2048 + 3 * group, 3
    w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, dtype, f"ragged b{bits} g{group}")


def test_mxfp4_quantize_and_products():
    rng = np.random.default_rng(5)
    n, k = 360, 2880
    w = make_w(rng, n, k, ref.BF16)
    packed, scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
    q = nv.quantize(to_dev(w), nv.QuantMode.MXFP4)
    assert np.array_equal(to_host(q.weight), packed) and np.array_equal(to_host(q.scales), scales)
    for out in (ref.BF16, ref.F32, ref.F16):
        want = ref.fp_dequantize(packed, scales, ref.MXFP4, out)
        assert np.array_equal(to_host(nv.dequantize(q, TORCH[out])).view(np.uint8), want.view(np.uint8))
    for m in (1, 5):
        x = make_x(rng, m, k, ref.BF16)
        want = ref.quantized_matmul(x, packed, scales, None, mode=ref.MXFP4, group=32, bits=4, dtype=ref.BF16)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, ref.BF16, f"mxfp4 M={m}", exact_weights=True)


def test_empty_and_degenerate_products():
    dev = torch.device("cuda")
    q = nv.Quantized(torch.zeros((8, 16), dtype=torch.uint32, device=dev), torch.ones((8, 2), device=dev),
                     torch.zeros((8, 2), device=dev), nv.Quant.affine(64, 4))
    y = nv.quantized_matmul(torch.zeros((0, 128), device=dev), q)
    assert y.shape == (0, 8)
    q0 = nv.Quantized(torch.zeros((8, 0), dtype=torch.uint32, device=dev), torch.ones((8, 0), device=dev),
                      torch.zeros((8, 0), device=dev), nv.Quant.affine(64, 4))
    y = nv.quantized_matmul(torch.ones((3, 0), device=dev), q0)
    assert y.shape == (3, 8) and float(y.abs().sum()) == 0.0


def test_sorted_offsets_and_gather_pairs():
    rng = np.random.default_rng(11)
    experts, n, k, rows = 8, 64, 512, 40
    w = make_w(rng, experts * n, k, ref.BF16).reshape(experts, n, k)
    packed, scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
    rhs = np.sort(rng.integers(0, experts, rows)).astype(np.uint32)
    x = make_x(rng, rows, k, ref.BF16).reshape(rows, 1, k)
    off = to_host(nv.sorted_offsets(torch.from_numpy(rhs.astype(np.int32)).cuda(), experts))
    assert np.array_equal(off, ref.sorted_offsets(rhs, experts))
    assert np.array_equal(off, np.searchsorted(rhs, np.arange(experts), side="left").astype(np.int32))
    q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(nv.QuantMode.MXFP4))
    got = to_host(nv.gather_qmm(to_dev(x), q, None, torch.from_numpy(rhs.astype(np.int64)).cuda(),
                                nv.GatherQmm(sorted_indices=True)))
    want = ref.gather_qmm(x, packed, scales, None, np.arange(rows, dtype=np.uint32), rhs, mode=ref.MXFP4, group=32,
                          bits=4, dtype=ref.BF16)
    assert got.shape == (rows, 1, n)
    assert_rows_close(got, want, ref.BF16, "sorted gather", exact_weights=True)


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_rows_of_few_outputs_take_the_cpu_weights(dtype):
    """Half-precision affine products of fewer than 1024 outputs per row, on every kernel that serves them (few rows and
    tiles on the matrix cores, the general vector kernel, both kernels of the [K, N] storage, gathered pairs): the
    weights are the CPU's doubly rounded ones (kernels.rs:835-859), so the outputs differ from the CPU product only by
    the order of the float32 sums: nearly all agree bit for bit, none is off by more than one rounding step (which is up to
    0.78 x the bar for a row's largest output)."""
    rng = np.random.default_rng(8800 + dtype)
    tdtype = TORCH[dtype]
    cases = [(24, 200, 1024, 4, 64, True, "qmf_kernel"), (5, 200, 1024, 4, 64, True, "qmv_lds_kernel"), (1, 100, 4096, 4, 64, True, "qmv_lds_kernel"), (3, 64, 480, 8, 32, True, "qmv_lds_kernel"),
             (2048, 768, 512, 4, 64, True, "qmm_kernel"), (300, 640, 1024, 4, 64, True, None), (260, 257, 192, 3, 64, True, None), (16, 48, 6400, 8, 128, True, "qmf_kernel"),
             (16, 48, 1536, 8, 128, True, "qmv_lds_kernel"),
             (40, 384, 256, 4, 64, False, "qmn_kernel"), (130, 992, 192, 8, 32, False, "qmn_kernel"), (7, 256, 200, 4, 64, False, "qvm_kernel"),
             (9, 128, 320, 6, 64, False, "qmn_kernel")]
    for m, n, k, bits, group, transpose, kernel in cases:
        w = make_w(rng, n, k, dtype) if transpose else make_w(rng, k, n, dtype)
        x = make_x(rng, m, k, dtype)
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
        if kernel is not None:
            assert nv.quantized_matmul_route(m, n, k, q.quant, tdtype, transpose=transpose) == kernel
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, transpose=transpose, threads=8)
        for rows_flag in (False, True):
            got = to_host(nv.quantized_matmul(to_dev(x), q, transpose=transpose, rows=rows_flag))
            what = f"CPU weights b{bits} g{group} M={m} N={n} K={k} transpose={transpose} rows={rows_flag}"
            worst = float(np.max(_excess(got, want, dtype)))
            record_ratio(what, worst, got.size)
            differ = np.count_nonzero(got.view(np.uint16) != want.view(np.uint16))
            assert worst <= 0.8 and differ <= max(2, got.size // 50), f"{what}: {worst:.3f} x the bar, {differ} of {got.size} outputs differ"
    # gathered pairs: one product per pair
    experts, n, k, m, pairs = 4, 96, 512, 3, 6
    w = make_w(rng, experts * n, k, dtype).reshape(experts, n, k)
    packed, scales, biases = ref.affine_quantize(w, dtype, 64, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(64, 4))
    x = make_x(rng, pairs * m, k, dtype).reshape(pairs, m, k)
    rhs = rng.integers(0, experts, pairs)
    got = to_host(nv.gather_qmm(to_dev(x), q, None, torch.from_numpy(rhs).cuda()))
    want = ref.gather_qmm(x, packed, scales, biases, np.arange(pairs, dtype=np.uint32), rhs.astype(np.uint32), group=64, bits=4, dtype=dtype)
    assert float(np.max(_excess(got.reshape(pairs * m, n), want.reshape(pairs * m, n), dtype))) <= 0.8


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("m,n,k,group", [(17, 40, 64, 64), (100, 300, 1024 + 64, 64), (260, 257, 96, 32), (64, 512, 2048, 128)])
def test_tiled_products_ragged(dtype, m, n, k, group):
    """The matrix-core kernel on shapes that are not multiples of its 256 x 256 x 64 tile."""
    rng = np.random.default_rng(31 + m)
    w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, 4))
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=4, dtype=dtype, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, dtype, f"tiled {m}x{n}x{k} g{group}")
    assert_device_arithmetic(got, x, packed, scales, biases, group, 4, dtype, f"tiled {m}x{n}x{k} g{group}")


@pytest.mark.parametrize("m", [40, 200])
def test_tiled_products_batched(m):
    """x [B, M, K] against w [B, N, K/8]: one product per batch (few-row kernel and tiled kernel)."""
    rng = np.random.default_rng(77)
    b, n, k = 3, 96, 256
    w = make_w(rng, b * n, k, ref.BF16).reshape(b, n, k)
    x = make_x(rng, b * m, k, ref.BF16).reshape(b, m, k)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(64, 4))
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.BF16)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert got.shape == (b, m, n)
    assert_rows_close(got, want, ref.BF16, "batched tiled")


def test_config3_prefill_bf16_4bit_g64():
    """BASELINE config 3 at full size: x bf16 [2048,4096], W [14336,4096].  The oracle computes a
    sample of outputs (whole product: 240 GFLOP); every row is also compared, within the same
    tolerance, against the decode kernel's product of that row alone."""
    rng = np.random.default_rng(20260103)
    m, n, k = 2048, 14336, 4096
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    packed, scales, biases = to_host(q.weight), to_host(q.scales), to_host(q.biases)
    xd = to_dev(x)
    y = nv.quantized_matmul(xd, q)
    assert y.shape == (m, n)
    got = to_host(y)
    samples = 6000
    rows, cols = rng.integers(0, m, samples), rng.integers(0, n, samples)
    rows[:4], cols[:4] = [0, m - 1, 0, m - 1], [0, 0, n - 1, n - 1]
    want = ref.to_f32(ref.quantized_matmul_sample(x, packed, scales, biases, rows, cols, group=64, bits=4, dtype=ref.BF16), ref.BF16)
    g32 = ref.to_f32(got, ref.BF16)
    row_max = np.max(np.abs(g32), axis=1)
    ratio = np.abs(g32[rows, cols].astype(np.float64) - want.astype(np.float64)) / (1e-2 * row_max[rows])
    record_ratio("config 3, 6000 sampled outputs", float(np.max(ratio)), ratio.size)
    assert float(np.max(ratio)) <= 1.0, f"max sample error {float(np.max(ratio)):.3f} x the bound"
    some = np.sort(rng.choice(m, 256, replace=False))  # whole rows against the CPU oracle (3.7 million outputs) ...
    want_rows = ref.quantized_matmul(x[some], packed, scales, biases, group=64, bits=4, dtype=ref.BF16, threads=16)
    assert_rows_close(got[some], want_rows, ref.BF16, "config 3, 256 whole rows")
    some = some[::4]  # ... and against the device arithmetic
    assert_device_arithmetic(got[some], x[some], packed, scales, biases, 64, 4, ref.BF16, "config 3, 64 whole rows")
    for i in (0, 777, m - 1):
        one = ref.to_f32(to_host(nv.quantized_matmul(xd[i:i + 1], q)), ref.BF16)[0]
        assert np.all(np.abs(one - g32[i]) <= 1e-2 * row_max[i])


def moe_inputs(rng, experts, n, k, tokens, top):
    w = make_w(rng, experts * n, k, ref.BF16).reshape(experts, n, k)
    packed, scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
    x_tok = make_x(rng, tokens, k, ref.BF16)
    choice = np.stack([rng.permutation(experts)[:top] for _ in range(tokens)])  # distinct experts per token
    pair_expert, pair_token = choice.reshape(-1), np.repeat(np.arange(tokens), top)
    order = np.argsort(pair_expert, kind="stable")  # the caller's sort by expert (model.rs:2195-2210)
    rhs = pair_expert[order].astype(np.uint32)
    x = np.ascontiguousarray(x_tok[pair_token[order]]).reshape(-1, 1, k)
    return packed, scales, x, rhs


def test_config5_moe_gather_mxfp4():
    """BASELINE config 5: 32 experts [2880,2880] MXFP4, 256 tokens x top-4 sorted by expert -> x [1024,1,2880].
    Every output row against the oracle's per-pair product; grouped route == per-pair route within the bar."""
    rng = np.random.default_rng(20260105)
    experts, n, k = 32, 2880, 2880
    packed, scales, x, rhs = moe_inputs(rng, experts, n, k, 256, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(nv.QuantMode.MXFP4))
    rhs_dev = torch.from_numpy(rhs.astype(np.int64)).cuda()
    assert nv.GatherQmm.groups(rhs.size, experts)
    got = to_host(nv.gather_qmm(to_dev(x), q, None, rhs_dev, nv.GatherQmm(sorted_indices=True)))
    assert got.shape == (1024, 1, n)
    want = ref.gather_qmm(x, packed, scales, None, np.arange(1024, dtype=np.uint32), rhs, mode=ref.MXFP4, group=32, bits=4,
                          dtype=ref.BF16, threads=8)
    assert_rows_close(got, want, ref.BF16, "config 5 grouped", exact_weights=True)
    unsorted = to_host(nv.gather_qmm(to_dev(x[:40]), q, None, rhs_dev[:40], nv.GatherQmm(sorted_indices=False)))
    assert_rows_close(unsorted, want[:40], ref.BF16, "config 5 per pair", exact_weights=True)


def test_grouped_gather_edge_cases():
    """Experts without rows, an expert with more than 32 rows (two passes), affine 4-bit weights."""
    rng = np.random.default_rng(8)
    experts, n, k = 6, 72, 256
    w = make_w(rng, experts * n, k, ref.BF16).reshape(experts, n, k)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 4)
    rhs = np.sort(np.array([0] * 3 + [2] * 45 + [5] * 20, np.uint32))
    x = make_x(rng, rhs.size, k, ref.BF16).reshape(-1, 1, k)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(64, 4))
    got = to_host(nv.gather_qmm(to_dev(x), q, None, torch.from_numpy(rhs.astype(np.int64)).cuda(), nv.GatherQmm(sorted_indices=True)))
    want = ref.gather_qmm(x, packed, scales, biases, np.arange(rhs.size, dtype=np.uint32), rhs, group=64, bits=4, dtype=ref.BF16)
    assert_rows_close(got, want, ref.BF16, "grouped affine")
    # Uneven loads over many experts (the kernel's blocks find their pass of 64 rows in the offsets, every lane walking a
    # run of experts: more than 256 experts is more than four a lane): one expert with several passes, the last expert
    # with two, singletons, most experts empty.
    experts, n, k = 300, 136, 128
    w = make_w(rng, experts * n, k, ref.BF16).reshape(experts, n, k)
    packed, scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
    counts = np.zeros(experts, np.int64)
    counts[[7, 299, 0, 64, 128, 255, 256, 257, 298]] = [200, 70, 1, 1, 65, 1, 3, 64, 1]
    rhs = np.repeat(np.arange(experts), counts).astype(np.uint32)
    x = make_x(rng, rhs.size, k, ref.BF16).reshape(-1, 1, k)
    q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(nv.QuantMode.MXFP4))
    ids = torch.from_numpy(rhs.astype(np.int32)).cuda()
    rows = torch.arange(rhs.size, dtype=torch.int32, device="cuda")
    got = to_host(nv.gather_qmm_grouped(to_dev(x).reshape(-1, k), q, rows, ids, nv.sorted_offsets(ids, experts)))  # (the grouped kernel whatever the rows per expert)
    want = ref.gather_qmm(x, packed, scales, None, np.arange(rhs.size, dtype=np.uint32), rhs, mode=ref.MXFP4, group=32, bits=4, dtype=ref.BF16)
    assert_rows_close(got, want.reshape(rhs.size, n), ref.BF16, "grouped MXFP4, 300 experts with uneven loads", exact_weights=True)


@pytest.mark.parametrize("quant", ["MXFP4", "affine4", "NVFP4-gs"])
def test_grouped_gather_with_the_experts_bias(quant):
    """`SwitchProjection::forward` on ordered pairs (model.rs:2113-2146): the product, then each row's expert's bias.  The
    grouped kernel adds it in its epilogue (`nvq_gather_qmm_expert_bias`): bit for bit the product followed by the
    separate rounded addition, with the rows in sorted order and scattered to their pairs' places; NVFP4 experts with a
    global scale each take the same route.  Unsorted pairs (and products the grouped kernel does not take) run pair by
    pair with the bias in those kernels' epilogues."""
    from nuvec_amd.layers import SwitchProjection
    rng = np.random.default_rng(8100 + len(quant))
    experts, n, k, pairs = 6, 1160, 512, 300
    w = (torch.randn(experts, n, k, device="cuda") * 0.05).to(torch.bfloat16)
    gs = None
    if quant == "NVFP4-gs":
        gs = to_dev(np.array([0.5, 2.0, 7.5, 1.0, 3.25, 0.75], np.float32))
        parts = [nv.quantize(w[e], nv.QuantMode.NVFP4, gs[e]) for e in range(experts)]
        q = nv.Quantized(torch.stack([p.weight for p in parts]), torch.stack([p.scales for p in parts]), None, parts[0].quant, gs)
    else:
        q = nv.quantize(w, nv.Quant.new(nv.QuantMode.MXFP4) if quant == "MXFP4" else nv.Quant.affine(64, 4))
    bias = to_dev(make_x(rng, experts, n, ref.BF16))
    x = to_dev(make_x(rng, 40, k, ref.BF16))
    ids = torch.from_numpy(rng.integers(0, experts - 1, pairs).astype(np.int32)).cuda()  # (the last expert has no rows)
    order, restore, sorted_ids, offsets = nv.moe_order(ids.reshape(1, pairs, 1), experts)
    rows = torch.from_numpy(rng.integers(0, 40, pairs).astype(np.int32)).cuda()
    plain = nv.gather_qmm_grouped(x, q, rows, sorted_ids, offsets)
    if gs is not None:  # the grouped route with the experts' global scales equals the sorted gather of ops.gather_qmm
        same = nv.gather_qmm(x[rows.long()].unsqueeze(1), q, None, sorted_ids, nv.GatherQmm(sorted_indices=True)).squeeze(1)
        assert torch.equal(plain, same)
        assert not torch.equal(plain, nv.gather_qmm_grouped(x, nv.Quantized(q.weight, q.scales, None, q.quant), rows, sorted_ids, offsets))
    want = plain + bias[sorted_ids.long()]
    got = nv.gather_qmm_grouped(x, q, rows, sorted_ids, offsets, expert_bias=bias)
    assert torch.equal(got, want), f"{quant}: the bias in the epilogue"
    scattered = nv.gather_qmm_grouped(x, q, rows, sorted_ids, offsets, out_rows=order, expert_bias=bias)
    assert torch.equal(scattered[order.long()], want), f"{quant}: scattered rows"
    proj = SwitchProjection(q.weight, q.scales, q.biases, bias, q.quant, gs)
    assert torch.equal(proj.forward_sorted_rows(x, rows, sorted_ids, offsets), want)
    assert torch.equal(proj.forward_sorted_rows(x, rows, sorted_ids, offsets, out_rows=order)[order.long()], want)
    # the unsorted pairs of the same projection (the route of fewer than 64 pairs) against the ordered ones
    xf, idf = x[rows.long()[:20]].reshape(20, 1, 1, k), sorted_ids[:20].reshape(20, 1)
    few = proj.forward(xf, idf)
    assert torch.equal(few, nv.gather_qmm(xf, q, None, idf) + bias[idf.long()].unsqueeze(-2)), f"{quant}: the bias in the per-pair kernels"
    scale = float(want[:20].float().abs().max())
    assert float((few.reshape(20, n).float() - want[:20].float()).abs().max()) <= 2e-2 * scale
    for m in (3, 12, 40):  # several rows per pair: the few-row matrix-core kernels' epilogues
        xm = to_dev(make_x(rng, 5 * m, k, ref.BF16)).reshape(5, m, k)
        lhs, rhs = torch.tensor([4, 0, 2, 2], device="cuda"), torch.tensor([1, 3, 0, 3], device="cuda")
        got_m = nv.gather_qmm(xm, q, lhs, rhs, expert_bias=bias)
        assert torch.equal(got_m, nv.gather_qmm(xm, q, lhs, rhs) + bias[rhs].unsqueeze(-2)), f"{quant}: {m} rows per pair"
    # a product the grouped kernel does not take (K off its steps of 64) runs pair by pair, the bias in those epilogues
    if quant == "MXFP4":
        q2 = nv.quantize(w[:, :, :96].contiguous(), nv.Quant.new(nv.QuantMode.MXFP4))
        proj2 = SwitchProjection(q2.weight, q2.scales, None, bias, q2.quant)
        y2 = proj2.forward_sorted_rows(x[:, :96].contiguous(), rows, sorted_ids, offsets)
        assert torch.equal(y2, nv.gather_qmm_grouped(x[:, :96].contiguous(), q2, rows, sorted_ids, offsets) + bias[sorted_ids.long()])
        with pytest.raises(nv.Unsupported):  # weights stored [K, N]
            nv.gather_qmm(torch.randn(4, 1, n, device="cuda").to(torch.bfloat16), q, None, torch.tensor([0, 1, 2, 3], device="cuda"),
                          nv.GatherQmm(transpose=False), expert_bias=bias[:, :k].contiguous())
    with pytest.raises(nv.InvalidArgument):
        nv.gather_qmm_grouped(x, q, rows, sorted_ids, offsets, expert_bias=bias[:, :-1])


@pytest.mark.parametrize("m", [3, 16, 33, 100])
def test_few_rows_on_matrix_cores(m):
    """3 <= M < 128 of BASELINE's decode weights: one weight decode shared by all rows."""
    rng = np.random.default_rng(40 + m)
    n, k = 1000, 4096
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(64, 4))
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.BF16, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, ref.BF16, f"few rows M={m}")
    assert_device_arithmetic(got, x, packed, scales, biases, 64, 4, ref.BF16, f"few rows M={m}")


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(32, 2), (64, 3), (128, 3), (64, 6), (32, 8), (128, 8), (32, 4), (64, 5), (32, 5), (128, 1), (32, 1)])
def test_few_rows_every_width(dtype, group, bits):
    """The few-row matrix-core kernel at every code width it takes: K of whole and of half windows
    (128 and 64 values), N off the rows per block, passes of 8, 16 and 32 rows of x."""
    rng = np.random.default_rng(900 + 10 * bits + group)
    for m, n, k in [(1, 200, 256), (5, 77, 1152), (16, 130, 2048 + 128), (14, 77, 7168), (33, 64, 128), (2, 96, 576 if group < 128 else 640)]:
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, dtype, f"few rows b{bits} g{group} M={m} N={n} K={k}")
        assert_device_arithmetic(got, x, packed, scales, biases, group, bits, dtype, f"few rows b{bits} g{group} M={m} N={n} K={k}")
        if m >= 5 and k % 128 == 0:  # (a single row of some widths stays on the vector kernels; odd widths need whole windows)
            # (up to 16 rows against rows of fewer than 1024 outputs: the vector kernel with the CPU's weights while m K <= 12 x 8192)
            few = ("qmv_lds_kernel",) if m <= 16 and m * k <= 12 * 8192 else ("qmf_kernel", "qmd_kernel", "qmm_kernel")
            assert nv.quantized_matmul_route(m, n, k, q.quant, TORCH[dtype]) in few


@pytest.mark.parametrize("bits,group", [(3, 64), (8, 32)])
def test_few_rows_batched_widths(bits, group):
    """A batch of weight matrices with one stride per operand, 3- and 8-bit codes."""
    rng = np.random.default_rng(77 + bits)
    b, m, n, k = 3, 4, 96, 512
    w, x = make_w(rng, b * n, k, ref.BF16), make_x(rng, b * m, k, ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, group, bits)
    q = nv.Quantized(to_dev(packed.reshape(b, n, -1)), to_dev(scales.reshape(b, n, -1)), to_dev(biases.reshape(b, n, -1)),
                     nv.Quant.affine(group, bits))
    got = to_host(nv.quantized_matmul(to_dev(x.reshape(b, m, k)), q))
    for i in range(b):
        want = ref.quantized_matmul(x[i * m:(i + 1) * m], packed[i * n:(i + 1) * n], scales[i * n:(i + 1) * n],
                                    biases[i * n:(i + 1) * n], group=group, bits=bits, dtype=ref.BF16)
        assert_rows_close(got[i], want, ref.BF16, f"batched b{bits} item {i}")


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(32, 2), (64, 3), (128, 6), (32, 8), (64, 8), (64, 5), (128, 5), (64, 1), (32, 1)])
def test_tiled_every_width(dtype, group, bits):
    """The tiled matrix-core kernel (M >= 193) at the other code widths, on shapes off its 256 x 256 x 64 tile."""
    rng = np.random.default_rng(1200 + 10 * bits + group)
    for m, n, k in [(260, 300, 1152), (193, 64, 128)]:
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, threads=8)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, dtype, f"tiled b{bits} g{group} {m}x{n}x{k}")
        assert_device_arithmetic(got, x, packed, scales, biases, group, bits, dtype, f"tiled b{bits} g{group} {m}x{n}x{k}")
        assert nv.quantized_matmul_route(m, n, k, q.quant, TORCH[dtype]) in ("qmm_kernel", "qmf_kernel", "qmd_kernel")


def test_tiled_mxfp4():
    """The tiled kernel on MXFP4 weights (dense prefill of an MXFP4 layer)."""
    rng = np.random.default_rng(99)
    m, n, k = 300, 200, 2880
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
    packed, scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.mxfp4()) if hasattr(nv.Quant, "mxfp4") else nv.quantize(to_dev(w), nv.QuantMode.MXFP4)
    want = ref.quantized_matmul(x, packed, scales, None, mode=ref.MXFP4, group=32, bits=4, dtype=ref.BF16, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, ref.BF16, "tiled mxfp4", exact_weights=True)


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
@pytest.mark.parametrize("dtype", [ref.BF16, ref.F32, ref.F16])
def test_mxfp8_nvfp4_quantize_and_products(mode, qmode, dtype):
    """The other two floating-point block formats (no global scale): quantize and dequantize bit for bit,
    products (on the general kernel) within the bar.  The CPU path keeps these weights in float32, so the
    bar holds for every output."""
    rng = np.random.default_rng(300 + mode + dtype)
    n, k = 200, 1152
    w = make_w(rng, n, k, dtype)
    packed, scales = ref.fp_quantize(w, dtype, mode)
    q = nv.quantize(to_dev(w), getattr(nv.QuantMode, qmode))
    assert np.array_equal(to_host(q.weight), packed) and np.array_equal(to_host(q.scales), scales)
    for out in (ref.BF16, ref.F32, ref.F16):
        want = ref.fp_dequantize(packed, scales, mode, out)
        assert np.array_equal(to_host(nv.dequantize(q, TORCH[out])).view(np.uint8), want.view(np.uint8))
    group, bits = ref.FP_PARAMS[mode]
    for m in (1, 5, 40):
        x = make_x(rng, m, k, dtype)
        want = ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        ratio = _excess(got, want, dtype)
        assert float(np.max(ratio)) <= 1.0, f"{qmode} M={m}: max error is {float(np.max(ratio)):.3f} x the bound"


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_block_formats_on_the_matrix_cores(mode, qmode, dtype):
    """MXFP4, MXFP8 and NVFP4 (no global scale) through the few-row, the tiled and the grouped matrix-core kernels: few rows,
    passes of 32 rows, tiles off the 256 x 256 shape with K split and unsplit, a batch, sorted experts.  Their weights are
    exact in the element type (a few significant bits times a scale of few bits), so the bar holds for every output."""
    rng = np.random.default_rng(4100 + 10 * mode + dtype)
    group, bits = ref.FP_PARAMS[mode]
    for m, n, k in [(1, 200, 1152), (5, 77, 2880), (33, 130, 640), (100, 96, 1024), (300, 260, 1152), (520, 64, 4096)]:
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        packed, scales = ref.fp_quantize(w, dtype, mode)
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(getattr(nv.QuantMode, qmode)))
        want = ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype, threads=8)
        for scratch in (True, False):
            got = to_host(nv.quantized_matmul(to_dev(x), q, scratch=scratch))
            assert_rows_close(got, want, dtype, f"{qmode} M={m} N={n} K={k} scratch={scratch}", exact_weights=True)
    # a batch with one stride per operand
    b, m, n, k = 3, 40, 96, 512
    w, x = make_w(rng, b * n, k, dtype), make_x(rng, b * m, k, dtype)
    packed, scales = ref.fp_quantize(w, dtype, mode)
    q = nv.Quantized(to_dev(packed.reshape(b, n, -1)), to_dev(scales.reshape(b, n, -1)), None, nv.Quant.new(getattr(nv.QuantMode, qmode)))
    got = to_host(nv.quantized_matmul(to_dev(x.reshape(b, m, k)), q))
    for i in range(b):
        want = ref.quantized_matmul(x[i * m:(i + 1) * m], packed[i * n:(i + 1) * n], scales[i * n:(i + 1) * n], None, mode=mode,
                                    group=group, bits=bits, dtype=dtype)
        assert_rows_close(got[i], want, dtype, f"{qmode} batch item {i}", exact_weights=True)
    # experts: rows sorted by expert (the grouped kernel), an expert without rows, one with more than 64
    experts, n, k = 5, 136, 768
    w = make_w(rng, experts * n, k, dtype).reshape(experts, n, k)
    packed, scales = ref.fp_quantize(w, dtype, mode)
    rhs = np.sort(np.array([0] * 7 + [1] * 70 + [3] * 33 + [4] * 18, np.uint32))
    x = make_x(rng, rhs.size, k, dtype).reshape(-1, 1, k)
    q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(getattr(nv.QuantMode, qmode)))
    got = to_host(nv.gather_qmm(to_dev(x), q, None, torch.from_numpy(rhs.astype(np.int64)).cuda(), nv.GatherQmm(sorted_indices=True)))
    want = ref.gather_qmm(x, packed, scales, None, np.arange(rhs.size, dtype=np.uint32), rhs, mode=mode, group=group, bits=bits, dtype=dtype)
    assert_rows_close(got, want, dtype, f"{qmode} grouped gather", exact_weights=True)
    some = rng.permutation(rhs.size)[:20]
    got = to_host(nv.gather_qmm(to_dev(x), q, torch.from_numpy(some.astype(np.int64)).cuda(),
                                torch.from_numpy(rhs[some].astype(np.int64)).cuda(), nv.GatherQmm()))
    assert_rows_close(got, want[some], dtype, f"{qmode} gather per pair", exact_weights=True)


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_block_formats_on_the_decode_kernel(mode, qmode, dtype):
    """One to four rows of x against MXFP4, MXFP8 and NVFP4 weights on the decode kernel of the vector units (the conversion
    instructions give the code values, a group's float32 scale multiplies the group's sum): K of one slice, off the
    kernel's steps and over several, weight rows off the block's eight, a batch, the pairs of an unsorted gather (the
    experts of a decoded token).  The weights are exact in the element type, so the bar holds for every output."""
    rng = np.random.default_rng(4700 + 10 * mode + dtype)
    group, bits = ref.FP_PARAMS[mode]
    quant = nv.Quant.new(getattr(nv.QuantMode, qmode))
    for m, n, k in [(1, 203, 32), (1, 1000, 2880), (2, 77, 4096 + 96), (3, 130, 1024), (4, 61, 2880), (1, 48, 14336), (2, 1030, 8192), (4, 96, 224)]:
        # (rows of at most 512 values take the short-row form of the same arithmetic: several weight rows a wavefront)
        assert nv.quantized_matmul_route(m, n, k, quant, TORCH[dtype]) == ("qmv4_short_kernel" if k <= 512 else "qmv4_lds_kernel"), (qmode, m, n, k)
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        packed, scales = ref.fp_quantize(w, dtype, mode)
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, quant)
        want = ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype, threads=8)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, dtype, f"decode kernel {qmode} M={m} N={n} K={k}", exact_weights=True)
    b, m, n, k = 3, 2, 90, 1056
    w, x = make_w(rng, b * n, k, dtype), make_x(rng, b * m, k, dtype)
    packed, scales = ref.fp_quantize(w, dtype, mode)
    q = nv.Quantized(to_dev(packed.reshape(b, n, -1)), to_dev(scales.reshape(b, n, -1)), None, quant)
    assert nv.quantized_matmul_route(m, n, k, quant, TORCH[dtype], batch=b) == "qmv4_lds_kernel"
    got = to_host(nv.quantized_matmul(to_dev(x.reshape(b, m, k)), q))
    for i in range(b):
        want = ref.quantized_matmul(x[i * m:(i + 1) * m], packed[i * n:(i + 1) * n], scales[i * n:(i + 1) * n], None, mode=mode,
                                    group=group, bits=bits, dtype=dtype)
        assert_rows_close(got[i], want, dtype, f"decode kernel {qmode} batch item {i}", exact_weights=True)
    # four experts of one token, unsorted: a product of one row per pair
    lhs, rhs = np.zeros(4, np.int64), np.array([2, 0, 1, 2], np.int64)
    xt = make_x(rng, 1, k, dtype)
    got = to_host(nv.gather_qmm(to_dev(xt.reshape(1, 1, k)), q, torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), nv.GatherQmm()))
    for z in range(4):
        e = int(rhs[z])
        want = ref.quantized_matmul(xt, packed[e * n:(e + 1) * n], scales[e * n:(e + 1) * n], None, mode=mode, group=group, bits=bits, dtype=dtype)
        assert_rows_close(got[z], want, dtype, f"decode kernel {qmode} pair {z}", exact_weights=True)


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("bits,group", [(2, 32), (2, 64), (2, 128), (3, 32), (3, 64), (3, 128), (5, 32), (5, 64), (5, 128), (6, 32), (6, 64), (6, 128), (8, 32), (8, 64), (8, 128)])
def test_decode_kernel_other_affine_widths(dtype, bits, group):
    """The decode kernel's 2-, 3-, 5-, 6- and 8-bit variants (a lane's 32 codes: two dwords split 16 bits, three dwords
    split 24 bits at a time into two halves of four codes; five or six dwords split 20 or 24 bits at a time into two halves
    of two codes; eight dwords converted in memory order): one row at any K, up to two (2 and 3 bits), three or four (8
    bits), four (5 and 6 bits) where K
    is beyond 2048; K off the kernel's steps, weight rows off the block's eight; a batch and the pairs of a gather.
    Against the CPU oracle within the bar and the device arithmetic within half of it."""
    rng = np.random.default_rng(5200 + 10 * bits + group + dtype)
    most = 2 if bits in (2, 3) else 4 if group == 32 or bits in (5, 6) else 3
    quant = nv.Quant.affine(group, bits)
    for m, n, k in [(1, 1030, 4096), (1, 1100, 2944), (1, 2053, 128), (1, 1025, 1024), (2, 1061, 4096 + 128), (most, 1030, 2944), (most, 1024, 8192)]:
        route = nv.quantized_matmul_route(m, n, k, quant, TORCH[dtype])
        # (a single row of 3-bit codes in groups of 128 with K a multiple of 512 up to 2048 stays on the direct kernel)
        assert route == "qmv4_lds_kernel" or (bits == 3 and group == 128 and k <= 2048 and k % 512 == 0 and route == "qmd_kernel"), (bits, group, m, n, k, route)
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), quant)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, threads=8)
        assert_rows_close(got, want, dtype, f"decode kernel b{bits} g{group} M={m} N={n} K={k}")
        assert_device_arithmetic(got, x, packed, scales, biases, group, bits, dtype, f"decode kernel b{bits} g{group} M={m} N={n} K={k}")
    assert nv.quantized_matmul_route(most + 1, 1030, 4096, quant, TORCH[dtype]) != "qmv4_lds_kernel"
    # the pairs of a gather, one row each
    experts, n, k = 3, 1040, 2304
    w = make_w(rng, experts * n, k, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
    q = nv.Quantized(to_dev(packed.reshape(experts, n, -1)), to_dev(scales.reshape(experts, n, -1)), to_dev(biases.reshape(experts, n, -1)), quant)
    x = make_x(rng, 4, k, dtype)
    rhs = np.array([2, 0, 2, 1], np.int64)
    got = to_host(nv.gather_qmm(to_dev(x.reshape(4, 1, k)), q, None, torch.from_numpy(rhs).cuda()))
    for z in range(4):
        e = int(rhs[z])
        want = ref.quantized_matmul(x[z:z + 1], packed[e * n:(e + 1) * n], scales[e * n:(e + 1) * n], biases[e * n:(e + 1) * n], group=group, bits=bits, dtype=dtype)
        assert_rows_close(got[z], want, dtype, f"decode kernel b{bits} g{group} pair {z}")


@pytest.mark.parametrize("quant", ["affine4-g32", "affine4-g64", "affine4-g128", "MXFP4", "MXFP8", "NVFP4"])
@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_short_rows_of_gathered_pairs(quant, dtype):
    """Unsorted pairs of one to four rows against weight rows of up to 2048 values (the down projections of a decoded
    token's experts): the short-row decode kernel, a weight row on 16, 32 or 64 lanes.  K on and off the lanes' powers
    of two, weight rows off the block's count, every pair against the oracle's product; the experts' bias in the
    epilogue bit for bit the separate addition."""
    rng = np.random.default_rng(4900 + len(quant) + dtype)
    affine = quant.startswith("affine")
    group = int(quant.split("g")[1]) if affine else None
    mode = ref.AFFINE if affine else getattr(ref, quant)
    q_of = nv.Quant.affine(group, 4) if affine else nv.Quant.new(getattr(nv.QuantMode, quant))
    fgroup, bits = (group, 4) if affine else ref.FP_PARAMS[mode]
    experts = 5
    for m, n, k in [(1, 1030, 768), (2, 1061, 384), (3, 1024, 1408), (4, 1100, 2048), (1, 1025, 128), (1, 1040, 1152)]:
        w = make_w(rng, experts * n, k, dtype)
        if affine:
            packed, scales, biases = ref.affine_quantize(w, dtype, group, 4)
        else:
            (packed, scales), biases = ref.fp_quantize(w, dtype, mode), None
        q = nv.Quantized(to_dev(packed.reshape(experts, n, -1)), to_dev(scales.reshape(experts, n, -1)),
                         None if biases is None else to_dev(biases.reshape(experts, n, -1)), q_of)
        x = make_x(rng, 3 * m, k, dtype)
        lhs, rhs = np.array([2, 0, 1, 1, 0, 2, 2], np.int64), np.array([4, 0, 3, 3, 1, 0, 2], np.int64)
        got = nv.gather_qmm(to_dev(x.reshape(3, m, k)), q, torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda())
        for z in range(lhs.size):
            e, i = int(rhs[z]), int(lhs[z])
            want = ref.quantized_matmul(x[i * m:(i + 1) * m], packed[e * n:(e + 1) * n], scales[e * n:(e + 1) * n],
                                        None if biases is None else biases[e * n:(e + 1) * n], mode=mode, group=fgroup, bits=bits, dtype=dtype)
            assert_rows_close(to_host(got[z]), want, dtype, f"short rows {quant} M={m} N={n} K={k} pair {z}", exact_weights=not affine)
        bias = to_dev(make_x(rng, experts, n, dtype))
        with_bias = nv.gather_qmm(to_dev(x.reshape(3, m, k)), q, torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), expert_bias=bias)
        assert torch.equal(with_bias, got + bias[torch.from_numpy(rhs).cuda()].unsqueeze(-2))


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
def test_block_formats_at_every_scale_code(mode, qmode, dtype):
    """Every scale code on every product route, weights stored [N, K] and [K, N]: output column n carries scale code n in all
    its groups (E8M0: 2^(n - 127), zero flushed at code 0; E4M3: both signs, subnormals, 448, NaN at 0x7F and 0xFF), so a
    conversion that mistook one code fails its column of the output.  Outputs are compared after division by their
    column's scale, each against the bar of its row.  x is small enough for the large scales to stay finite; the E8M0
    codes whose weights overflow float32 (from 246; 255 is infinity in the reference, fp8.rs:95-102, and only an infinite
    weight quantizes to it) or whose products would be float32 subnormals (below 30) are left out; code 0, which
    flushes to zero (fp8.rs:95-112), stays, and its columns are zero on every route.  float16 keeps the E8M0 codes whose
    outputs are normal float16 values, and code 0."""
    rng = np.random.default_rng(4800 + mode + 10 * dtype)
    group, bits = ref.FP_PARAMS[mode]
    quant = nv.Quant.new(getattr(nv.QuantMode, qmode))
    n, k = 256, 512
    codes = np.arange(256, dtype=np.uint8)
    if mode != ref.NVFP4:
        keep = (codes == 0) | ((codes >= 120) & (codes <= 134) if dtype == ref.F16 else (codes >= 30) & (codes <= 245))
        codes = np.where(keep, codes, 127).astype(np.uint8)
    x_scale = 2.0 ** -6 if dtype == ref.F16 else 2.0 ** -14
    one = np.full((n, k * bits // 32), 0x38383838 if mode == ref.MXFP8 else 0x22222222, np.uint32)  # every code 1.0
    value = ref.fp_dequantize(one, np.repeat(codes[:, None], k // group, axis=1), mode, ref.F32)[:, 0].astype(np.float64)  # the scales as the oracle decodes them
    nan, zero = np.isnan(value), value == 0.0
    assert (nan[[0x7F, 0xFF]].all() if mode == ref.NVFP4 else zero[0] and not nan.any())
    assert np.count_nonzero(~nan & ~zero) >= (15 if dtype == ref.F16 and mode != ref.NVFP4 else 200)
    live = ~nan & ~zero
    routes = set()

    def compare(got, want, what):
        assert np.isnan(want[:, nan]).all() and np.isnan(got[:, nan]).all(), f"{what}: NaN scales"
        assert not want[:, zero].any() and not got[:, zero].any(), f"{what}: scales that flush to zero"
        g, r = got[:, live].astype(np.float64) / value[live], want[:, live].astype(np.float64) / value[live]
        ratio = np.abs(g - r) / (TOL[dtype] * np.max(np.abs(r), axis=1, keepdims=True))
        worst = np.unravel_index(np.argmax(ratio), ratio.shape)
        assert ratio[worst] <= 1.0, f"{what} scale code {codes[live][worst[1]]}: {ratio[worst]:.3f} x the bound"

    # weights stored [N, K]: row n of the weight carries code n (rows of 512 values: the short-row decode kernel at one
    # and three rows of x; rows of 1024: the decode kernel)
    for k in (512, 1024):
        w = make_w(rng, n, k, dtype)
        packed, _ = ref.fp_quantize(w, dtype, mode)
        scales = np.repeat(codes[:, None], k // group, axis=1)
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, quant)
        for m in ((1, 3, 8, 40, 300) if k == 512 else (1, 2)):
            x = ref.from_f32(rng.standard_normal((m, k)).astype(np.float32) * x_scale, dtype)
            want = ref.to_f32(ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype, threads=8), dtype)
            got = ref.to_f32(to_host(nv.quantized_matmul(to_dev(x), q)), dtype)
            routes.add(nv.quantized_matmul_route(m, n, k, quant, TORCH[dtype]))
            compare(got, want, f"{qmode} M={m} K={k}")
    assert {"qmv4_lds_kernel", "qmv4_short_kernel", "qmd_kernel"} <= routes and len(routes) >= 4, routes

    # weights stored [K, N]: the groups run along N, so every column of group n carries code n; the matrix-core kernel
    # and the kernel of few rows
    k2, n2 = 256, 256 * group
    w = make_w(rng, k2, n2, dtype)
    packed, _ = ref.fp_quantize(w, dtype, mode)
    scales = np.repeat(codes[None, :], k2, axis=0)
    q = nv.Quantized(to_dev(packed), to_dev(scales), None, quant)
    nan, zero, live, value, codes = (np.repeat(v, group) for v in (nan, zero, live, value, codes))
    routes = set()
    for m in (1, 40, 300):
        x = ref.from_f32(rng.standard_normal((m, k2)).astype(np.float32) * x_scale, dtype)
        want = ref.to_f32(ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype, transpose=False, threads=8), dtype)
        got = ref.to_f32(to_host(nv.quantized_matmul(to_dev(x), q, transpose=False)), dtype)
        routes.add(nv.quantized_matmul_route(m, n2, k2, quant, TORCH[dtype], transpose=False))
        compare(got, want, f"{qmode} stored [K, N] M={m}")
    assert "qmn_kernel" in routes, routes


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F32, ref.F16])
def test_nvfp4_global_scale(dtype):
    """NVFP4 with a global scale (MLX's `quantize(..., global_scale=)`): codes, scales and dequantized values bit for
    bit; the product of two matrices on the kernel and the shapes the reference multiplies densely, within the bar;
    a gather with one scale per expert; the mode check."""
    rng = np.random.default_rng(3300 + dtype)
    n, k, g = 160, 1152, 3.25
    w = make_w(rng, n, k, dtype)
    gs = torch.tensor(g, dtype=torch.float32, device="cuda")
    packed, scales = ref.fp_quantize(w, dtype, ref.NVFP4, g)
    q = nv.quantize(to_dev(w), nv.QuantMode.NVFP4, gs)
    assert q.global_scale is gs and q.biases is None
    assert np.array_equal(to_host(q.weight), packed) and np.array_equal(to_host(q.scales), scales)
    assert not np.array_equal(scales, ref.fp_quantize(w, dtype, ref.NVFP4)[1])  # the scale does change the codes
    for out in (ref.BF16, ref.F32, ref.F16):
        want = ref.fp_dequantize(packed, scales, ref.NVFP4, out, g)
        assert np.array_equal(to_host(nv.dequantize(q, TORCH[out])).view(np.uint8), want.view(np.uint8))
    for m in (1, 5, 40, 300):
        x = make_x(rng, m, k, dtype)
        want = ref.fp_quantized_matmul_scaled(x, packed, scales, ref.NVFP4, dtype, g)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, dtype, f"NVFP4 with a global scale M={m} K={k} N={n}")
    if dtype != ref.F32:  # the matrix-core kernels fold the global scale into the group scales (kernels.rs:992-998)
        n2, k2 = 640, 1024
        w2 = make_w(rng, n2, k2, dtype)
        p2, s2 = ref.fp_quantize(w2, dtype, ref.NVFP4, g)
        q2 = nv.quantize(to_dev(w2), nv.QuantMode.NVFP4, gs)
        for m, kernels in ((1, ("qmv4_lds_kernel",)), (2, ("qmv4_lds_kernel",)), (16, ("qmd_kernel",)), (40, ("qmf_kernel", "qmd_kernel")), (600, ("qmm_kernel", "qmf_kernel"))):
            x = make_x(rng, m, k2, dtype)
            want = ref.fp_quantized_matmul_scaled(x, p2, s2, ref.NVFP4, dtype, g)
            got = to_host(nv.quantized_matmul(to_dev(x), q2))
            assert_rows_close(got, want, dtype, f"NVFP4 with a global scale on the matrix cores M={m} K={k2} N={n2}")
            assert nv.quantized_matmul_route(m, n2, k2, q2.quant, TORCH[dtype]) in kernels  # (the scale does not change the route)
    # a batch of x: the reference dequantizes in x's type and multiplies densely (quantized.rs:481-491); so does the mirror
    xb = make_x(rng, 6, k, dtype).reshape(2, 3, k)
    got = to_host(nv.quantized_matmul(to_dev(xb), q)).reshape(6, n)
    want = ref.fp_quantized_matmul_scaled(xb.reshape(6, k), packed, scales, ref.NVFP4, dtype, g)
    assert float(np.max(_excess(got, want, dtype))) <= 2.0
    # stacked experts, one scale each
    experts, pairs = 3, 7
    we = make_w(rng, experts * 64, 256, dtype).reshape(experts, 64, 256)
    ge = np.array([0.5, 2.0, 7.5], np.float32)
    pe, se = zip(*(ref.fp_quantize(we[e], dtype, ref.NVFP4, float(ge[e])) for e in range(experts)))
    qe = nv.Quantized(to_dev(np.stack(pe)), to_dev(np.stack(se)), None, nv.Quant.new(nv.QuantMode.NVFP4), to_dev(ge))
    xe = make_x(rng, pairs, 256, dtype).reshape(pairs, 1, 256)
    rhs = rng.integers(0, experts, pairs)
    got = to_host(nv.gather_qmm(to_dev(xe), qe, None, torch.from_numpy(rhs).cuda()))
    for i in range(pairs):
        want = ref.fp_quantized_matmul_scaled(xe[i], pe[rhs[i]], se[rhs[i]], ref.NVFP4, dtype, float(ge[rhs[i]]))
        assert float(np.max(_excess(got[i], want, dtype))) <= 1.0, f"pair {i}"
    # many pairs sorted by expert: the grouped route, one scale per expert there too
    many = 90
    xm = make_x(rng, many, 256, dtype).reshape(many, 1, 256)
    ids = np.sort(rng.integers(0, experts, many))
    got = to_host(nv.gather_qmm(to_dev(xm), qe, None, torch.from_numpy(ids).cuda(), nv.GatherQmm(sorted_indices=True)))
    want = np.stack([ref.fp_quantized_matmul_scaled(xm[i], pe[ids[i]], se[ids[i]], ref.NVFP4, dtype, float(ge[ids[i]])) for i in range(many)])
    assert_rows_close(got.reshape(many, 64), want.reshape(many, 64), dtype, "NVFP4 experts with a global scale each, sorted pairs")
    with pytest.raises(nv.Unsupported):  # untransposed weights with a global scale: no kernel, and nothing else answers
        nv.gather_qmm(to_dev(xe[:, :, :64]), qe, None, torch.from_numpy(rhs).cuda(), nv.GatherQmm(transpose=False))
    with pytest.raises(nv.InvalidArgument):
        nv.quantize(to_dev(w), nv.QuantMode.MXFP4, gs)
    with pytest.raises(nv.InvalidArgument):
        nv.quantize(to_dev(w), nv.QuantMode.NVFP4, torch.ones(2, device="cuda"))


@pytest.mark.parametrize("dtype", [ref.F32, ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(64, 4), (32, 2), (128, 6), (64, 5), (128, 1), (32, 3), (64, 8)])
def test_untransposed_products_every_width(dtype, group, bits):
    """Weights stored [K, N] (transpose=False): one row and a few rows of x, K split over the grid or not,
    N beyond and below one wavefront's 2048 outputs."""
    rng = np.random.default_rng(1700 + 10 * bits + group + dtype)
    for m, k, n in [(1, 300, 2 * 128), (5, 64, 2048 + 3 * 128), (1, 2500, 128)]:
        w = make_w(rng, k, n, dtype)  # quantized along N
        x = make_x(rng, m, k, dtype)
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, transpose=False)
        got = to_host(nv.quantized_matmul(to_dev(x), q, transpose=False))
        assert got.shape == (m, n)
        assert_rows_close(got, want, dtype, f"x.w b{bits} g{group} M={m} K={k} N={n}")


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
def test_untransposed_products_block_formats(mode, qmode):
    rng = np.random.default_rng(1800 + mode)
    group, bits = ref.FP_PARAMS[mode]
    for m, k, n in [(1, 200, 256), (7, 96, 2048 + 64)]:
        w, x = make_w(rng, k, n, ref.BF16), make_x(rng, m, k, ref.BF16)
        packed, scales = ref.fp_quantize(w, ref.BF16, mode)
        q = nv.quantize(to_dev(w), getattr(nv.QuantMode, qmode))
        assert np.array_equal(to_host(q.weight), packed)
        want = ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=ref.BF16, transpose=False)
        got = to_host(nv.quantized_matmul(to_dev(x), q, transpose=False))
        ratio = _excess(got, want, ref.BF16)
        assert float(np.max(ratio)) <= 1.0, f"x.w {qmode} M={m}: max error is {float(np.max(ratio)):.3f} x the bound"


def test_untransposed_products_batched():
    """x [B, M, K] against w [B, K, N/8]: one product per batch item."""
    rng = np.random.default_rng(1900)
    b, m, k, n = 3, 2, 160, 256
    w = make_w(rng, b * k, n, ref.F32).reshape(b, k, n)
    x = make_x(rng, b * m, k, ref.F32).reshape(b, m, k)
    packed, scales, biases = ref.affine_quantize(w, ref.F32, 64, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(64, 4))
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.F32, transpose=False)
    got = to_host(nv.quantized_matmul(to_dev(x), q, transpose=False))
    assert got.shape == (b, m, n)
    assert_rows_close(got, want, ref.F32, "batched x.w")


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(64, 4), (32, 4), (128, 8), (32, 8), (64, 2), (128, 2), (64, 3), (32, 5), (64, 6), (128, 1), (128, 3), (32, 6)])
def test_untransposed_products_on_the_matrix_cores(dtype, group, bits):
    """Weights stored [K, N] with K in whole steps of 64 and codes in runs of eight columns: the tiled matrix-core
    kernel, for one row of x and for several tiles of rows, ragged M and N, K split over the grid (through the
    workspace) and not (without one)."""
    rng = np.random.default_rng(2100 + 10 * bits + group + dtype)
    tdtype = torch.bfloat16 if dtype == ref.BF16 else torch.float16
    for m, k, n in [(1, 64, 128), (5, 128, 2048 + 3 * 128), (130, 192, 384), (300, 2048, 640), (33, 4096, 128)]:
        w = make_w(rng, k, n, dtype)  # quantized along N
        x = make_x(rng, m, k, dtype)
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
        assert nv.quantized_matmul_route(m, n, k, q.quant, tdtype, transpose=False) == "qmn_kernel"
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, transpose=False)
        got = to_host(nv.quantized_matmul(to_dev(x), q, transpose=False))
        assert got.shape == (m, n)
        assert_rows_close(got, want, dtype, f"x.w tiled b{bits} g{group} M={m} K={k} N={n}")
        unsplit = to_host(nv.quantized_matmul(to_dev(x), q, transpose=False, scratch=False))
        assert_rows_close(unsplit, want, dtype, f"x.w tiled b{bits} g{group} M={m} K={k} N={n}, no workspace")


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
def test_untransposed_block_formats_on_the_matrix_cores(mode, qmode):
    """The block formats of the same kernel (NVFP4: also a last group of 16 columns); their weights are exact in the
    element type, so the bar has no exception for short rows."""
    rng = np.random.default_rng(2200 + mode)
    group, bits = ref.FP_PARAMS[mode]
    for dtype, tdtype in ((ref.BF16, torch.bfloat16), (ref.F16, torch.float16)):
        for m, k, n in [(1, 128, 256), (70, 320, 2048 + 64), (260, 1024, 96 + (16 if mode == ref.NVFP4 else 0))]:
            w, x = make_w(rng, k, n, dtype), make_x(rng, m, k, dtype)
            packed, scales = ref.fp_quantize(w, dtype, mode)
            q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(getattr(nv.QuantMode, qmode)))
            assert nv.quantized_matmul_route(m, n, k, q.quant, tdtype, transpose=False) == "qmn_kernel"
            want = ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype, transpose=False)
            got = to_host(nv.quantized_matmul(to_dev(x), q, transpose=False))
            assert_rows_close(got, want, dtype, f"x.w tiled {qmode} M={m} K={k} N={n}", exact_weights=True)


def test_untransposed_products_on_the_matrix_cores_batched_with_bias():
    """x [B, M, K] against w [B, K, N / 8] on the tiled kernel, with and without the layer's bias (the separate rounded
    addition, bit for bit) and with one weight for every batch item."""
    rng = np.random.default_rng(2300)
    b, m, k, n = 3, 40, 256, 384
    w = make_w(rng, b * k, n, ref.BF16).reshape(b, k, n)
    x = make_x(rng, b * m, k, ref.BF16).reshape(b, m, k)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(64, 4))
    assert nv.quantized_matmul_route(m, n, k, q.quant, torch.bfloat16, batch=b, transpose=False) == "qmn_kernel"
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.BF16, transpose=False)
    plain = nv.quantized_matmul(to_dev(x), q, transpose=False)
    assert plain.shape == (b, m, n)
    assert_rows_close(to_host(plain), want, ref.BF16, "batched x.w tiled")
    bias = to_dev(make_x(rng, 1, n, ref.BF16).reshape(n))
    fused = nv.quantized_matmul(to_dev(x), q, transpose=False, bias=bias)
    assert np.array_equal(to_host(fused).view(np.uint8), to_host(plain + bias).view(np.uint8))
    shared = nv.Quantized(q.weight[1], q.scales[1], q.biases[1], q.quant)  # broadcast over the batch
    got = to_host(nv.quantized_matmul(to_dev(x), shared, transpose=False))
    want1 = ref.quantized_matmul(x, packed[1], scales[1], biases[1], group=64, bits=4, dtype=ref.BF16, transpose=False)
    assert_rows_close(got, want1, ref.BF16, "batched x against one w, tiled")


@pytest.mark.parametrize("dtype", [ref.F32, ref.BF16, ref.F16])
@pytest.mark.parametrize("group,bits", [(64, 4), (32, 3), (128, 8), (64, 6), (32, 2)])
def test_embedding_rows_bit_exact(dtype, group, bits):
    """The lookup of a quantized embedding (nuvec-nn layers.rs:245-255: take of weight, scales and biases, then
    dequantize): equal to the oracle's dequantize of the taken rows bit for bit; repeated, first and last ids."""
    rng = np.random.default_rng(2100 + bits + group + dtype)
    vocab, dim = 777, 384
    w = make_w(rng, vocab, dim, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
    ids = rng.integers(0, vocab, size=(3, 41))
    ids[0, :4] = [0, vocab - 1, 5, 5]
    want = ref.affine_dequantize(packed[ids.reshape(-1)], scales[ids.reshape(-1)], biases[ids.reshape(-1)], dtype, group, bits)
    for torch_ids in (torch.tensor(ids, dtype=torch.int64), torch.tensor(ids, dtype=torch.int32)):
        got = nv.embedding(q, torch_ids.cuda())
        assert tuple(got.shape) == (3, 41, dim)
        assert np.array_equal(to_host(got).reshape(-1, dim).view(np.uint8), want.view(np.uint8))
    assert nv.embedding(q, torch.zeros((0,), dtype=torch.int64).cuda()).shape == (0, dim)
    with pytest.raises(nv.InvalidArgument):
        nv.embedding(q, torch.zeros(3).cuda())


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
def test_embedding_rows_block_formats(mode, qmode):
    rng = np.random.default_rng(2200 + mode)
    vocab, dim = 300, 256
    w = make_w(rng, vocab, dim, ref.BF16)
    packed, scales = ref.fp_quantize(w, ref.BF16, mode)
    q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(getattr(nv.QuantMode, qmode)))
    ids = rng.integers(0, vocab, size=97)
    for out in (ref.BF16, ref.F32, ref.F16):
        want = ref.fp_dequantize(packed[ids], scales[ids], mode, out)
        got = to_host(nv.embedding(q, torch.tensor(ids).cuda(), TORCH[out]))
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))


def test_layers_mirror_the_reference_callers():
    """QuantizedLinear (layers.rs:121-162) and QuantizedEmbedding (layers.rs:221-262) over the library:
    from_linear quantizes as the oracle, forward is product + bias, the tied embedding serves both ways."""
    from nuvec_amd.layers import QuantizedEmbedding, QuantizedLinear
    rng = np.random.default_rng(2300)
    n, k, m = 320, 512, 6
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
    bias = make_x(rng, 1, n, ref.BF16).reshape(n)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 4)
    layer = QuantizedLinear.from_linear(to_dev(w), to_dev(bias))
    assert np.array_equal(to_host(layer.weight), packed)
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.BF16)
    plain = to_host(QuantizedLinear.from_linear(to_dev(w))(to_dev(x)))
    assert_rows_close(plain, want, ref.BF16, "QuantizedLinear without bias")
    # The bias is one more rounded addition on the product this library returned.
    with_bias = to_host(layer(to_dev(x)))
    expect = ref.from_f32(ref.to_f32(plain, ref.BF16) + ref.to_f32(bias, ref.BF16), ref.BF16)
    assert np.array_equal(with_bias.view(np.uint8), expect.view(np.uint8))
    assert np.array_equal(to_host(layer.dequantized_weight()).view(np.uint8),
                          ref.affine_dequantize(packed, scales, biases, ref.BF16, 64, 4).view(np.uint8))
    emb = QuantizedEmbedding.from_embedding(to_dev(w), nv.QuantMode.MXFP4)
    fp_packed, fp_scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
    ids = rng.integers(0, n, size=(2, 9))
    assert np.array_equal(to_host(emb(torch.tensor(ids).cuda())).reshape(-1, k).view(np.uint8),
                          ref.fp_dequantize(fp_packed[ids.reshape(-1)], fp_scales[ids.reshape(-1)], ref.MXFP4, ref.BF16).view(np.uint8))
    tied = to_host(emb.as_linear(to_dev(x)))
    want = ref.quantized_matmul(x, fp_packed, fp_scales, None, mode=ref.MXFP4, group=32, bits=4, dtype=ref.BF16)
    assert_rows_close(tied, want, ref.BF16, "tied embedding")


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16, ref.F32])
def test_linear_bias_in_the_product_epilogues(dtype):
    """nvq_quantized_linear on every product route (decode kernels, both matrix-core few-row kernels, the tiled kernel with
    and without a split of K, the general kernel's widths and block formats, weights stored [K, N]): bit for bit the
    product this library returns followed by the separate rounded addition of the reference (layers.rs:155-162)."""
    rng = np.random.default_rng(5200 + dtype)
    cases = [(nv.Quant.affine(64, 4), 4096, 1024, (1, 2, 3, 4, 8, 16, 40, 300)), (nv.Quant.affine(64, 4), 4096, 4096, (512,)),
             (nv.Quant.affine(64, 3), 1024, 200, (1, 5, 33, 260)), (nv.Quant.affine(32, 8), 512, 96, (1, 7, 200)),
             (nv.Quant.affine(128, 5), 1024, 77, (1, 9)), (nv.Quant.new(nv.QuantMode.MXFP4), 2880, 360, (1, 6, 70, 300)),
             (nv.Quant.new(nv.QuantMode.MXFP8), 1024, 130, (1, 12)), (nv.Quant.new(nv.QuantMode.NVFP4), 1024, 130, (1, 12, 300))]
    for quant, k, n, ms in cases:
        q = nv.quantize(to_dev(make_w(rng, n, k, dtype)), quant)
        bias = to_dev(make_x(rng, 1, n, dtype).reshape(n))
        for m in ms:
            x = to_dev(make_x(rng, m, k, dtype))
            plain = nv.quantized_matmul(x, q)
            fused = nv.quantized_matmul(x, q, bias=bias)
            assert np.array_equal(to_host(fused).view(np.uint8), to_host(plain + bias).view(np.uint8)), f"{quant} M={m} N={n} K={k}"
    # weights stored [K, N]
    k, n = 512, 256
    q = nv.quantize(to_dev(make_w(rng, k, n, dtype)), nv.Quant.affine(64, 4))
    bias = to_dev(make_x(rng, 1, n, dtype).reshape(n))
    for m in (1, 6):
        x = to_dev(make_x(rng, m, k, dtype))
        fused = nv.quantized_matmul(x, q, transpose=False, bias=bias)
        assert np.array_equal(to_host(fused).view(np.uint8), to_host(nv.quantized_matmul(x, q, transpose=False) + bias).view(np.uint8))
    with pytest.raises(nv.InvalidArgument):
        nv.quantized_matmul(x, q, transpose=False, bias=bias[:-1])


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("group,k,n", [(64, 2048, 1124), (128, 4096, 1120), (64, 6144, 1057), (128, 10240, 1088)])
def test_four_row_decode_on_matrix_cores(dtype, group, k, n):
    """Four rows of x at 4 bits, K a multiple of 2048 (the matrix-core decode kernel): N not a multiple of its 32
    weight rows, K beyond one staging round, both group sizes it takes, and a batch of products."""
    rng = np.random.default_rng(2400 + group + k + n + dtype)
    w, x = make_w(rng, n, k, dtype), make_x(rng, 4, k, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, 4))
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=4, dtype=dtype)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, dtype, f"four rows g{group} K={k} N={n}")
    assert_device_arithmetic(got, x, packed, scales, biases, group, 4, dtype, f"four rows g{group} K={k} N={n}")
    if k == 2048:  # x [3, 4, K] against one weight matrix and against a matrix per item
        xb = make_x(rng, 12, k, dtype).reshape(3, 4, k)
        want = ref.quantized_matmul(xb, packed, scales, biases, group=group, bits=4, dtype=dtype)
        got = to_host(nv.quantized_matmul(to_dev(xb), q))
        assert_rows_close(got.reshape(12, n), want.reshape(12, n), dtype, "four rows, shared weights")
        wb = make_w(rng, 3 * n, k, dtype).reshape(3, n, k)
        pb, sb, bb = ref.affine_quantize(wb, dtype, group, 4)
        qb = nv.Quantized(to_dev(pb), to_dev(sb), to_dev(bb), nv.Quant.affine(group, 4))
        want = ref.quantized_matmul(xb, pb, sb, bb, group=group, bits=4, dtype=dtype)
        got = to_host(nv.quantized_matmul(to_dev(xb), qb))
        assert_rows_close(got.reshape(12, n), want.reshape(12, n), dtype, "four rows, a matrix per item")


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("m,n,k", [(2, 1124, 4096), (3, 1057, 4096), (4, 1088, 4096), (5, 1071, 4096), (8, 1154, 4096), (2, 1064, 1024), (7, 1057, 1536),
                                   (4, 1074, 8192), (8, 1044, 8192), (6, 1060, 3584), (1, 1094, 1024), (1, 1057, 2048), (1, 1048, 5120), (4, 1064, 14336), (8, 1041, 12288), (3, 1044, 28672)])
def test_decode_rows_on_16x16x32(dtype, m, n, k):
    """One to eight rows of x at 4 bits, groups of 64, K a multiple of 512 up to 8192 (the 16x16x32 matrix-core decode
    kernel, a wavefront per 512 values, chunks of K beyond 8192): every tile-row layout (rows of x times groups), the smallest and the largest
    block, N not a multiple of a block's weight rows, and a matrix per item."""
    group = 64
    rng = np.random.default_rng(5200 + 16 * m + n + k + dtype)
    w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, 4))
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=4, dtype=dtype)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    assert_rows_close(got, want, dtype, f"{m} rows N={n}")
    assert_device_arithmetic(got, x, packed, scales, biases, group, 4, dtype, f"{m} rows N={n}")
    if n == 33:  # x [2, m, K] against a matrix per item
        xb = make_x(rng, 2 * m, k, dtype).reshape(2, m, k)
        wb = make_w(rng, 2 * n, k, dtype).reshape(2, n, k)
        pb, sb, bb = ref.affine_quantize(wb, dtype, group, 4)
        qb = nv.Quantized(to_dev(pb), to_dev(sb), to_dev(bb), nv.Quant.affine(group, 4))
        want = ref.quantized_matmul(xb, pb, sb, bb, group=group, bits=4, dtype=dtype)
        got = to_host(nv.quantized_matmul(to_dev(xb), qb))
        assert_rows_close(got.reshape(2 * m, n), want.reshape(2 * m, n), dtype, f"{m} rows, a matrix per item")


@pytest.mark.parametrize("pairs,experts", [(0, 4), (5, 3), (1024, 32), (3000, 7), (5000, 130), (2049, 32), (5000, 8), (65536, 32), (100001, 200)])
def test_moe_order_is_the_stable_argsort(pairs, experts):
    """The ordering of a mixture-of-experts layer's pairs (nuvec-lm model.rs:2193-2210): argsort of the expert
    ids with ties in pair order, its inverse, the sorted ids and where each expert starts: integers, exact."""
    rng = np.random.default_rng(2500 + pairs + experts)
    ids = rng.integers(0, experts, size=pairs).astype(np.int32)
    if pairs > 100:
        ids[ids == 1] = 0  # an expert without pairs
    order, restore, sorted_ids, offsets = nv.moe_order(torch.from_numpy(ids).cuda(), experts)
    want = np.argsort(ids, kind="stable")
    assert np.array_equal(order.cpu().numpy(), want)
    assert np.array_equal(sorted_ids.cpu().numpy(), ids[want])
    inverse = np.empty(pairs, dtype=np.int64)
    inverse[want] = np.arange(pairs)
    assert np.array_equal(restore.cpu().numpy(), inverse)
    assert np.array_equal(offsets.cpu().numpy(), np.searchsorted(ids[want], np.arange(experts), side="left"))
    if pairs:
        assert np.array_equal(offsets.cpu().numpy(), nv.sorted_offsets(sorted_ids, experts).cpu().numpy())


def test_switch_glu_sorts_gathers_and_restores():
    """SwitchGlu::forward (nuvec-lm model.rs:2177-2211) over the library: pairs ordered by expert, token rows taken
    inside the grouped products, results put back in pair order.  Each projection against the oracle's per-pair
    product; the few-pairs route (no sorting) against the same."""
    from nuvec_amd.layers import SwitchGlu, SwitchProjection
    rng = np.random.default_rng(2600)
    experts, d, inner, b, l, k = 6, 256, 320, 2, 24, 2
    def projection(n, kk):
        w = make_w(rng, experts * n, kk, ref.BF16).reshape(experts, n, kk)
        packed, scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
        return (packed, scales), SwitchProjection(to_dev(packed), to_dev(scales), None, None, nv.Quant.new(nv.QuantMode.MXFP4))
    (gp, gate), (up_, up), (dp, down) = projection(inner, d), projection(inner, d), projection(d, inner)
    glu = SwitchGlu(gate, up, down)
    x = make_x(rng, b * l, d, ref.BF16).reshape(b, l, d)
    idx = np.stack([rng.permutation(experts)[:k] for _ in range(b * l)]).reshape(b, l, k).astype(np.int32)
    # the ordered products, one projection at a time, against the oracle on the pairs in their own order
    order, restore, sorted_ids, offsets = nv.moe_order(torch.from_numpy(idx).cuda(), experts)
    tokens = torch.div(order, k, rounding_mode="floor").to(torch.int32)
    got_up = to_host(up.forward_sorted_rows(to_dev(x).reshape(b * l, d), tokens, sorted_ids, offsets)[restore.long()])
    flat = idx.reshape(-1)
    xrows = np.repeat(x.reshape(b * l, d), k, axis=0)
    want_up = np.stack([ref.quantized_matmul(xrows[p:p + 1], up_[0][flat[p]], up_[1][flat[p]], None, mode=ref.MXFP4, group=32, bits=4,
                                             dtype=ref.BF16)[0] for p in range(flat.size)])
    assert_rows_close(got_up, want_up, ref.BF16, "up projection, ordered")
    # the whole block both ways: ordered (96 pairs) and pair by pair (the same pairs, a few at a time)
    whole = glu(to_dev(x), torch.from_numpy(idx).cuda())
    assert tuple(whole.shape) == (b, l, k, d)
    few = torch.cat([glu(to_dev(x)[:, t:t + 8], torch.from_numpy(idx).cuda()[:, t:t + 8]) for t in range(0, l, 8)], dim=1)
    scale = float(few.float().abs().max())
    assert float((whole.float() - few.float()).abs().max()) <= 2e-2 * scale
    # the fused gate + up weight on the few-pairs route: one gather for both projections, the same rows of the same weights
    for fused in (SwitchGlu(gate, up, down).fuse_gate_up(),
                  SwitchGlu(gate, up, down, SwitchProjection(torch.cat([gate.weight, up.weight], 1), torch.cat([gate.scales, up.scales], 1), None,
                                                             None, gate.quant))):
        assert fused.gate_up_proj is not None
        again = torch.cat([fused(to_dev(x)[:, t:t + 8], torch.from_numpy(idx).cuda()[:, t:t + 8]) for t in range(0, l, 8)], dim=1)
        assert torch.equal(again, few), "paired" if fused.gate_up_paired else "gate rows first"


@pytest.mark.parametrize("dtype", [ref.F32, ref.F16, ref.BF16])
def test_moe_route_and_weighted_sum_bit_exact(dtype):
    """fast::moe_route and fast::weighted_sum over the shapes of the reference's tests
    (crates/nuvec-core/tests/fast.rs:841-987), bit for bit the restated kernels."""
    from oracle import moe
    rng = np.random.default_rng(7200 + dtype)
    for rows, e, ks in [(3, 8, (1, 2, 8)), (5, 60, (4, 8)), (4, 128, (1, 8, 10, 128)), (2, 512, (8, 22))]:
        logits = rng.standard_normal((rows, e)).astype(np.float32)
        p = np.exp(logits) / np.exp(logits).sum(-1, keepdims=True)
        ties = (np.floor(p * 4 * e) + 1) / (4 * e)
        for name, probs in (("probs", p), ("ties", ties)):
            stored = ref.from_f32(probs.astype(np.float32), dtype)
            for k in ks:
                for normalize in (False, True):
                    if normalize and k > 64:  # beyond 64 summed scores the reference composes sum and divide itself
                        with pytest.raises(nv.Unsupported):
                            nv.moe_route(to_dev(stored), k, normalize)
                        continue
                    want_top, want_scores = moe.moe_route(stored, dtype, k, normalize)
                    top, scores = nv.moe_route(to_dev(stored), k, normalize)
                    case = f"{name} rows {rows} E {e} k {k} norm {normalize}"
                    assert np.array_equal(to_host(top).astype(np.uint32), want_top), case
                    assert np.array_equal(to_host(scores).view(np.uint8), want_scores.view(np.uint8)), case
    if dtype != ref.BF16:  # NaN sorts last where the sort compares it
        nan_row = ref.from_f32(np.array([[0.1, np.nan, 0.3, 0.2]], np.float32), dtype)
        assert to_host(nv.moe_route(to_dev(nan_row), 2, False)[0]).tolist() == [[2, 1]]
    batched = ref.from_f32(rng.random((2, 3, 16)).astype(np.float32), dtype)
    top, scores = nv.moe_route(to_dev(batched), 4, True)
    want_top, want_scores = moe.moe_route(batched.reshape(6, 16), dtype, 4, True)
    assert tuple(top.shape) == (2, 3, 4) and np.array_equal(to_host(top).reshape(6, 4).astype(np.uint32), want_top)
    assert np.array_equal(to_host(scores).reshape(6, 4).view(np.uint8), want_scores.view(np.uint8))
    for k in (0, 17, -1):
        with pytest.raises(nv.InvalidArgument):
            nv.moe_route(to_dev(batched), k, False)
    with pytest.raises(nv.InvalidArgument):
        nv.moe_route(torch.ones(2, 8, dtype=torch.int32, device="cuda"), 2, False)
    for rows, k, d in [(3, 1, 64), (2, 4, 7), (4, 8, 2048), (3, 10, 64), (2, 16, 1), (1, 31, 96)]:
        x = ref.from_f32(rng.standard_normal((rows, k, d)).astype(np.float32), dtype)
        w = ref.from_f32(rng.standard_normal((rows, k)).astype(np.float32), dtype)
        got = to_host(nv.weighted_sum(to_dev(x), to_dev(w)))
        assert np.array_equal(got.view(np.uint8), moe.weighted_sum(x, w, dtype).view(np.uint8)), (rows, k, d)
    with pytest.raises(nv.Unsupported):  # 32 weighted rows and more: the reference composes multiply and sum itself
        nv.weighted_sum(torch.ones(2, 32, 8, device="cuda"), torch.ones(2, 32, device="cuda"))
    with pytest.raises(nv.InvalidArgument):
        nv.weighted_sum(torch.ones(2, 4, 8, device="cuda"), torch.ones(2, 5, device="cuda"))


def test_moe_block_routes_multiplies_and_sums():
    """MoeMlp::forward (nuvec-lm model.rs:2251-2272) over the library: router, moe_route, the experts' gated MLPs on
    the ordered pairs, weighted_sum; against the same steps restated on the host from the library's own routing."""
    from oracle import moe
    from nuvec_amd.layers import MoeMlp, SwitchGlu, SwitchProjection
    rng = np.random.default_rng(2700)
    experts, d, inner, b, l, k = 8, 256, 320, 2, 40, 2
    def projection(n, kk):
        w = make_w(rng, experts * n, kk, ref.BF16).reshape(experts, n, kk)
        packed, scales = ref.fp_quantize(w, ref.BF16, ref.MXFP4)
        return SwitchProjection(to_dev(packed), to_dev(scales), None, None, nv.Quant.new(nv.QuantMode.MXFP4))
    glu = SwitchGlu(projection(inner, d), projection(inner, d), projection(d, inner))
    gate = torch.randn(experts, d, device="cuda", dtype=torch.bfloat16)
    block = MoeMlp(gate, glu, k, True)
    x = to_dev(make_x(rng, b * l, d, ref.BF16).reshape(b, l, d))
    top, scores = block.route(x)
    probs = torch.softmax(torch.nn.functional.linear(x, gate).float(), -1).to(torch.bfloat16)
    want_top, want_scores = moe.moe_route(to_host(probs).reshape(b * l, experts), ref.BF16, k, True)
    assert np.array_equal(to_host(top).reshape(b * l, k).astype(np.uint32), want_top)
    assert np.array_equal(to_host(scores).reshape(b * l, k).view(np.uint8), want_scores.view(np.uint8))
    y = block(x)
    assert tuple(y.shape) == (b, l, d) and y.dtype == torch.bfloat16
    outputs = glu(x, top)  # [B, L, k, D]
    want = moe.weighted_sum(to_host(outputs).reshape(b * l, k, d), to_host(scores).reshape(b * l, k), ref.BF16)
    assert np.array_equal(to_host(y).reshape(b * l, d).view(np.uint8), want.view(np.uint8))
    # gate and up projections stored as one weight: one product instead of two, the same bits
    glu.fuse_gate_up()
    assert glu.gate_up_proj.weight.shape == (experts, 2 * inner, d // 8)
    assert torch.equal(glu(x, top).view(torch.int16), outputs.view(torch.int16))


@pytest.mark.parametrize("dtype", [ref.F32, ref.F16, ref.BF16])
@pytest.mark.parametrize("activation", ["swiglu", "swiglu_oai", "geglu"])
def test_gated_activation_against_the_oracle(dtype, activation):
    """`nvq_glu` (SwitchGlu::through between the products, model.rs:2157-2170; the experts' biases of model.rs:2139-2143)
    against the oracle's operation-by-operation restatement.  The two differ only through `exp` or `tanh` (the device's and
    the host's, either within a few ulps of float32), which the rounding of the sigmoid or the tanh to a half type hides
    except at a tie: there all but a few outputs in ten thousand agree bit for bit and none is off by more than one step of
    the type; float32 outputs agree within four steps.  (geglu: a step of the tanh is a step of 1 + tanh, which cancels
    for negative gates, so there the step is taken of |gate up / 2| as well as of the output.)"""
    from oracle import moe
    rng = np.random.default_rng(7600 + dtype + len(activation))
    tdtype = {ref.F32: torch.float32, ref.F16: torch.float16, ref.BF16: torch.bfloat16}[dtype]
    act = {"swiglu": moe.SWIGLU, "swiglu_oai": moe.SWIGLU_OAI, "geglu": moe.GEGLU}[activation]
    rows, hidden, experts = 300, 360, 6
    specials = np.array([0.0, -0.0, 7.0, -7.0, 7.5, -9.0, 60.0, -60.0, 100.0, -100.0, np.inf, -np.inf, np.nan, 1e-30, -1e-30], np.float32)
    g = (rng.standard_normal((rows, 2 * hidden)) * 3).astype(np.float32)
    g[0, :specials.size], g[0, hidden:hidden + specials.size] = specials, specials[::-1]
    g[1, :specials.size], g[1, hidden:hidden + specials.size] = specials, 1.0
    both = ref.from_f32(g, dtype)  # one product of fused gate / up weights: the gate's columns, then the up's
    gate, up = both[:, :hidden], both[:, hidden:]
    gb = ref.from_f32(rng.standard_normal((experts, hidden)).astype(np.float32), dtype)
    ub = ref.from_f32(rng.standard_normal((experts, hidden)).astype(np.float32), dtype)
    ids = np.sort(rng.integers(0, experts, rows)).astype(np.int32)

    def check(got, want, what, biased=False):
        got, want = np.asarray(got), np.asarray(want)
        gf, wf = ref.to_f32(got, dtype), ref.to_f32(want, dtype)
        same = (got.view(np.uint8).reshape(got.shape + (-1,)) == want.view(np.uint8).reshape(want.shape + (-1,))).all(-1) | (np.isnan(gf) & np.isnan(wf))
        if dtype != ref.F32:  # (float32 shows the last bits of exp itself: within four steps below)
            assert np.count_nonzero(~same) <= max(1, same.size // 2000), f"{what}: {np.count_nonzero(~same)} of {same.size} outputs differ"
        step = {ref.F32: 4 * 2.0 ** -23, ref.F16: 2.0 ** -10, ref.BF16: 2.0 ** -7}[dtype]
        size = np.abs(wf).astype(np.float64)
        if activation == "geglu":
            with np.errstate(invalid="ignore", over="ignore"):
                gv = ref.to_f32(gate, dtype).astype(np.float64) + (ref.to_f32(gb, dtype)[ids] if biased else 0.0)
                uv = ref.to_f32(up, dtype).astype(np.float64) + (ref.to_f32(ub, dtype)[ids] if biased else 0.0)
                size = size + np.nan_to_num(np.abs(0.5 * gv * uv), nan=0.0, posinf=0.0)
        off = np.abs(gf[~same].astype(np.float64) - wf[~same].astype(np.float64))
        assert np.all(off <= step * size[~same] + 2.0 ** -24), f"{what}: an output off by more than a step"

    dboth = to_dev(both)
    dgate, dup = dboth[:, :hidden], dboth[:, hidden:]  # strided views: read in place
    check(to_host(nv.glu(dgate, dup, activation)), moe.glu(gate, up, dtype, act), f"{activation} {dtype}")
    check(to_host(nv.glu(dgate.contiguous(), dup.contiguous(), activation, alpha=1.5, limit=5.0)),
          moe.glu(gate, up, dtype, act, 1.5, 5.0), f"{activation} {dtype} alpha 1.5 limit 5")
    got = nv.glu(dgate, dup, activation, gate_bias=to_dev(gb), up_bias=to_dev(ub), ids=torch.from_numpy(ids).cuda())
    check(to_host(got), moe.glu(gate, up, dtype, act, gate_bias=gb, up_bias=ub, ids=ids), f"{activation} {dtype} with biases", biased=True)
    # batched shapes and the composition this library's SwitchGlu replaces: bias added by a separate rounded addition
    lead = nv.glu(dgate.reshape(3, 100, hidden), dup.reshape(3, 100, hidden), activation)
    assert tuple(lead.shape) == (3, 100, hidden) and lead.dtype == tdtype
    assert torch.equal(lead.reshape(rows, hidden).view(torch.uint8), nv.glu(dgate, dup, activation).view(torch.uint8))
    idl = torch.from_numpy(ids).cuda().long()
    separate = nv.glu(dgate + to_dev(gb)[idl], dup + to_dev(ub)[idl], activation)
    assert torch.equal(got.view(torch.uint8), separate.view(torch.uint8))
    # empty, and what the op refuses
    assert tuple(nv.glu(dgate[:0], dup[:0], activation).shape) == (0, hidden)
    with pytest.raises(nv.InvalidArgument):
        nv.glu(dgate, dup[:, :-1], activation)
    with pytest.raises(nv.InvalidArgument):
        nv.glu(dgate, dup, "reglu")
    with pytest.raises(nv.InvalidArgument):
        nv.glu(dgate, dup, activation, gate_bias=to_dev(gb))
    with pytest.raises(nv.InvalidArgument):
        nv.glu(dgate, dup, activation, gate_bias=to_dev(gb), up_bias=to_dev(ub))
    with pytest.raises(nv.InvalidArgument):
        nv.glu(dgate, dup.to(torch.float64), activation)


def test_gated_activations_equal_what_mlx_lm_recorded():
    """The vectors of the reference's own test (crates/nuvec-nn/tests/rope_scaling.rs:150-172: mlx-lm's `swiglu_oai` and
    `geglu` in float32 and bfloat16) under its own rule (rope_scaling.rs:37-43: 1e-6 and 1e-2 of max(|value|, 1))."""
    import os

    from safetensors.torch import load_file
    recorded = load_file(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "mlx_lm_activations.safetensors"))
    for label, tol in (("f32", 1e-6), ("bf16", 1e-2)):
        gate, x = recorded[f"act_{label}.gate"].cuda(), recorded[f"act_{label}.x"].cuda()
        for name in ("swiglu_oai", "geglu"):
            got = nv.glu(gate, x, name, alpha=1.702, limit=7.0).double().cpu()
            want = recorded[f"act_{label}.{name}"].double()
            ratio = (got - want).abs() / (tol * want.abs().clamp(min=1.0))
            record_ratio(f"mlx-lm {label} {name}", float(ratio.max()), ratio.numel())
            assert float(ratio.max()) <= 1.0, (label, name)


@pytest.mark.parametrize("quant", ["MXFP4", "NVFP4", "affine4-g64", "affine4-g128"])
@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_dense_mlp_with_the_gated_epilogue(quant, dtype):
    """`Mlp::forward` (model.rs:2044-2075) over the library: the composition (two products with their biases, the
    activation, the down projection) against the oracle's products and activation, and — with the gate and up
    projections stored as one weight — up to four rows of x through `nvq_quantized_matmul_glu`: bit for bit the
    composition where its products run on the same decode kernel (K = 2880), within a step of the type elsewhere."""
    from nuvec_amd.layers import Mlp, QuantizedLinear
    from oracle import moe
    rng = np.random.default_rng(7900 + len(quant) + dtype)
    affine = quant.startswith("affine")
    q_of = nv.Quant.affine(int(quant.split("g")[1]), 4) if affine else nv.Quant.new(getattr(nv.QuantMode, quant))
    hidden = 1152
    for k, geglu, biased in ((2880, False, True), (2880, True, False), (4096, False, False)):
        def linear(n, kk, with_bias):
            q = nv.quantize(to_dev(make_w(rng, n, kk, dtype)), q_of)
            return QuantizedLinear(q.weight, q.scales, q.biases, to_dev(make_x(rng, 1, n, dtype)[0]) if with_bias else None, q.quant)
        if quant == "affine4-g128" and k % 128:
            k = 2944
        gate, up, down = linear(hidden, k, biased), linear(hidden, k, biased), linear(1024, hidden, biased)
        apart = Mlp(gate, up, down, geglu)
        fused = Mlp(gate, up, down, geglu).fuse_gate_up()
        assert fused.gate_up_proj is not None
        for rows in (1, 2, 3, 4, 5):
            x = to_dev(make_x(rng, rows, k, dtype))
            want = apart(x)
            got = fused(x)
            assert tuple(got.shape) == (rows, 1024)
            if k % 512:  # (both ways on the decode kernel)
                assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{quant} K={k} rows={rows}"
            else:
                assert float((got.float() - want.float()).abs().max()) <= 2e-2 * float(want.float().abs().max())
        # the hidden activations against the oracle: products, biases, activation
        x = to_dev(make_x(rng, 2, k, dtype))
        p = fused.gate_up_proj
        hid = to_host(nv.quantized_matmul_glu(x, p.quantized(), "geglu" if geglu else "swiglu", bias=p.bias))
        def product(lin):
            args = (to_host(lin.weight), to_host(lin.scales), None if lin.biases is None else to_host(lin.biases))
            if affine:
                y = ref.quantized_matmul(to_host(x), *args, group=q_of.group_size, bits=4, dtype=dtype)
            else:
                mode = getattr(ref, quant)
                group, bits = ref.FP_PARAMS[mode]
                y = ref.quantized_matmul(to_host(x), args[0], args[1], None, mode=mode, group=group, bits=bits, dtype=dtype)
            if lin.bias is not None:
                y = ref.from_f32(ref.to_f32(ref.from_f32(ref.to_f32(y, dtype), dtype), dtype) + ref.to_f32(to_host(lin.bias), dtype), dtype)
            return y
        want_hid = moe.glu(product(gate), product(up), dtype, moe.GEGLU if geglu else moe.SWIGLU)
        wf, gf = ref.to_f32(want_hid, dtype), ref.to_f32(hid, dtype)
        bound = (4e-2 if dtype == ref.BF16 else 1e-2) * np.abs(wf).max()  # (the activation of two outputs that each carry the product's bar)
        assert float(np.abs(gf - wf).max()) <= bound, f"{quant} K={k}: hidden activations against the oracle"
    with pytest.raises(nv.Unsupported):
        nv.quantized_matmul_glu(to_dev(make_x(rng, 5, k, dtype)), fused.gate_up_proj.quantized())
    with pytest.raises(nv.InvalidArgument):
        nv.quantized_matmul_glu(x, fused.gate_up_proj.quantized(), "reglu")


@pytest.mark.parametrize("quant", ["MXFP4", "MXFP8", "NVFP4", "affine4-g64", "affine4-g32"])
@pytest.mark.parametrize("activation", ["swiglu", "swiglu_oai", "geglu"])
def test_unsorted_pairs_with_the_gated_epilogue(quant, activation):
    """`nvq_gather_qmm_glu` without offsets: the experts of decoded tokens, pairs in any order, on the decode kernel with
    the gated activation as its epilogue (a wavefront takes a gate row and its up row).  Bit for bit the per-pair
    product of the paired weights followed by `nvq_glu` where that product runs on the same decode kernel (K beyond
    2048 off the 16x16x32 kernel's shapes), and within a step of the type elsewhere; with the experts' biases; through
    `SwitchGlu`'s route of fewer than 64 pairs."""
    from nuvec_amd.layers import SwitchGlu, SwitchProjection
    rng = np.random.default_rng(7800 + len(quant) + len(activation))
    q_of = {"MXFP4": nv.Quant.new(nv.QuantMode.MXFP4), "MXFP8": nv.Quant.new(nv.QuantMode.MXFP8), "NVFP4": nv.Quant.new(nv.QuantMode.NVFP4),
            "affine4-g64": nv.Quant.affine(64, 4), "affine4-g32": nv.Quant.affine(32, 4)}[quant]
    experts, hidden = 5, 1088  # (affine projections below 1024 rows stay apart)
    for dtype, k in ((ref.BF16, 2880), (ref.F16, 2304), (ref.BF16, 768)):
        gate = nv.quantize(to_dev(make_w(rng, experts * hidden, k, dtype).reshape(experts, hidden, k)), q_of)
        up = nv.quantize(to_dev(make_w(rng, experts * hidden, k, dtype).reshape(experts, hidden, k)), q_of)
        down = nv.quantize(to_dev(make_w(rng, experts * 1024, hidden, dtype).reshape(experts, 1024, hidden)), q_of)
        pair = lambda a, b: None if a is None else nv.pair_rows(a, b, 1)
        both = nv.Quantized(pair(gate.weight, up.weight), pair(gate.scales, up.scales), pair(gate.biases, up.biases), q_of)
        tokens, top = 3, 4
        x = to_dev(make_x(rng, tokens, k, dtype))
        ids = torch.from_numpy(np.stack([rng.permutation(experts)[:top] for _ in range(tokens)]).astype(np.int32)).cuda()
        rows = torch.arange(tokens, dtype=torch.int32, device="cuda").repeat_interleave(top)
        gb, ub = to_dev(make_x(rng, experts, hidden, dtype)), to_dev(make_x(rng, experts, hidden, dtype))
        xe = x[rows.long()].unsqueeze(1)
        g = nv.gather_qmm(xe, gate, None, ids.reshape(-1)).squeeze(1)
        u = nv.gather_qmm(xe, up, None, ids.reshape(-1)).squeeze(1)
        for biased in (False, True):
            kw = dict(gate_bias=gb, up_bias=ub, ids=ids.reshape(-1)) if biased else {}
            want = nv.glu(g, u, activation, alpha=1.702, limit=7.0, **kw)
            got = nv.gather_qmm_glu(x, both, rows, ids.reshape(-1), None, activation, alpha=1.702, limit=7.0,
                                    expert_bias=nv.pair_rows(gb, ub, 1) if biased else None)
            assert tuple(got.shape) == (tokens * top, hidden)
            if k > 2048 and not (quant == "affine4-g64" and k % 512 == 0):  # the same kernel both ways
                assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{quant} {activation} K={k} biased {biased}"
            else:
                scale = float(want.float().abs().max())
                assert float((got.float() - want.float()).abs().max()) <= 2e-2 * scale, f"{quant} {activation} K={k} biased {biased}"
        block = SwitchGlu(SwitchProjection(gate.weight, gate.scales, gate.biases, gb, q_of), SwitchProjection(up.weight, up.scales, up.biases, ub, q_of),
                          SwitchProjection(down.weight, down.scales, down.biases, None, q_of), activation=activation)
        apart = block(x.reshape(1, tokens, k), ids.reshape(1, tokens, top))
        fused = block.fuse_gate_up()
        assert fused.gate_up_paired
        together = fused(x.reshape(1, tokens, k), ids.reshape(1, tokens, top))
        scale = float(apart.float().abs().max())
        assert tuple(together.shape) == (1, tokens, top, 1024) and float((together.float() - apart.float()).abs().max()) <= 2e-2 * scale
    with pytest.raises(nv.Unsupported):  # five rows of x per pair are beyond the decode kernel
        from nuvec_amd import _lib
        import ctypes as C
        d = _lib.GatherDescC(q_of._c(), _lib.BF16, 1, 0, 0, 5, 2 * hidden, k, 2, 2, experts)
        p = lambda t: C.c_void_p(None if t is None else t.data_ptr())
        _lib.check(_lib.load().nvq_gather_qmm_glu(C.byref(d), 0, 1.702, 7.0, p(x), p(both.weight), p(both.scales), p(both.biases), p(rows), p(rows),
                                                  None, None, p(x), None))


@pytest.mark.parametrize("quant", ["MXFP4", "affine4", "affine8", "NVFP4"])
@pytest.mark.parametrize("activation", ["swiglu", "swiglu_oai", "geglu"])
def test_grouped_gather_with_the_gated_epilogue(quant, activation):
    """`nvq_gather_qmm_glu`: the gate and up products of the ordered pairs and the activation in one kernel, bit for bit
    the two grouped products (`nvq_gather_qmm`) followed by `nvq_glu`; experts without rows, with one pass of one tile
    (up to 32 rows), of two tiles (up to 64) and with several passes; with and without the experts' biases."""
    rng = np.random.default_rng(7700 + len(quant) + len(activation))
    experts, k, hidden = 7, 320, (1024 if quant.startswith("affine") else 192)  # (affine projections below 1024 rows stay apart)
    q_of = {"MXFP4": nv.Quant.new(nv.QuantMode.MXFP4), "NVFP4": nv.Quant.new(nv.QuantMode.NVFP4), "affine4": nv.Quant.affine(64, 4),
            "affine8": nv.Quant.affine(32, 8)}[quant]
    for dtype in (ref.BF16, ref.F16):
        gate = nv.quantize(to_dev(make_w(rng, experts * hidden, k, dtype).reshape(experts, hidden, k)), q_of)
        up = nv.quantize(to_dev(make_w(rng, experts * hidden, k, dtype).reshape(experts, hidden, k)), q_of)
        pair = lambda a, b: None if a is None else nv.pair_rows(a, b, 1)
        both = nv.Quantized(pair(gate.weight, up.weight), pair(gate.scales, up.scales), pair(gate.biases, up.biases), q_of)
        counts = [0, 5, 32, 33, 64, 150, 0]  # rows per expert
        ids = np.repeat(np.arange(experts), counts).astype(np.int32)
        pairs = ids.size
        tokens = 40
        x = to_dev(make_x(rng, tokens, k, dtype))
        rows = torch.from_numpy(rng.integers(0, tokens, pairs).astype(np.int32)).cuda()
        sorted_ids = torch.from_numpy(ids).cuda()
        offsets = nv.sorted_offsets(sorted_ids, experts)
        gb, ub = to_dev(make_x(rng, experts, hidden, dtype)), to_dev(make_x(rng, experts, hidden, dtype))
        g = nv.gather_qmm_grouped(x, gate, rows, sorted_ids, offsets)
        u = nv.gather_qmm_grouped(x, up, rows, sorted_ids, offsets)
        for biased in (False, True):
            kw = dict(gate_bias=gb, up_bias=ub, ids=sorted_ids) if biased else {}
            want = nv.glu(g, u, activation, alpha=1.702, limit=7.0, **kw)
            got = nv.gather_qmm_glu(x, both, rows, sorted_ids, offsets, activation, alpha=1.702, limit=7.0,
                                    expert_bias=nv.pair_rows(gb, ub, 1) if biased else None)
            assert tuple(got.shape) == (pairs, hidden)
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"{quant} {activation} dtype {dtype} biased {biased}"
    with pytest.raises(nv.Unsupported):  # rows not in whole runs of 64 (affine: also fewer than 1024 rows each)
        nv.gather_qmm_glu(x, nv.Quantized(both.weight[:, :320], both.scales[:, :320], None if both.biases is None else both.biases[:, :320], q_of),
                          rows, sorted_ids, offsets, activation)
    with pytest.raises(nv.InvalidArgument):
        nv.gather_qmm_glu(x, both, rows, sorted_ids, offsets, "reglu")


@pytest.mark.parametrize("mode,qmode", [(ref.AFFINE, None), (ref.MXFP4, "MXFP4"), (ref.NVFP4, "NVFP4")])
def test_untransposed_gathers(mode, qmode):
    """gather_qmm with the weights stored [K, N] (transpose=False): one product per pair, K split over the grid or not,
    one row and a few rows of x per pair, against the oracle's per-pair products."""
    rng = np.random.default_rng(5100 + mode)
    dtype = ref.BF16
    experts, pairs = 4, 9
    for m, k, n in [(1, 320, 256), (3, 2048, 384)]:
        w = make_w(rng, experts * k, n, dtype).reshape(experts, k, n)  # quantized along N
        if mode == ref.AFFINE:
            group, bits = 64, 4
            packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
            q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
        else:
            group, bits = ref.FP_PARAMS[mode]
            packed, scales = ref.fp_quantize(w, dtype, mode)
            biases = None
            q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(getattr(nv.QuantMode, qmode)))
        x = make_x(rng, pairs * m, k, dtype).reshape(pairs, m, k)
        lhs, rhs = rng.permutation(pairs), rng.integers(0, experts, pairs)
        got = to_host(nv.gather_qmm(to_dev(x), q, torch.from_numpy(lhs).cuda(), torch.from_numpy(rhs).cuda(), nv.GatherQmm(transpose=False)))
        assert got.shape == (pairs, m, n)
        want = ref.gather_qmm(x, packed, scales, biases, lhs.astype(np.uint32), rhs.astype(np.uint32), mode=mode, group=group, bits=bits,
                              dtype=dtype, transpose=False)
        assert_rows_close(got.reshape(pairs * m, n), want.reshape(pairs * m, n), dtype, f"untransposed gather mode {mode} M={m} K={k} N={n}")
    # Rows sorted by expert (the grouped route: the reference's `_nn` kernel of the block formats, gpu.rs:6786-6812; here for
    # affine weights too): each expert's weights read once per tile of its rows.  An expert without rows, one with more
    # rows than a tile of 32 and, with 700 pairs, than a tile of 128; every row against the oracle and close to the
    # per-pair route's (whose split of K orders the sums differently).
    experts, k, n = 5, 1088, 1280
    w = make_w(rng, experts * k, n, dtype).reshape(experts, k, n)
    if mode == ref.AFFINE:
        packed, scales, biases = ref.affine_quantize(w, dtype, 64, 4)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(64, 4))
        group, bits = 64, 4
    else:
        group, bits = ref.FP_PARAMS[mode]
        (packed, scales), biases = ref.fp_quantize(w, dtype, mode), None
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(getattr(nv.QuantMode, qmode)))
    for counts in ([3, 0, 45, 33, 20], [100, 0, 300, 129, 171]):
        rhs = np.repeat(np.arange(experts), counts).astype(np.int64)
        x = make_x(rng, rhs.size, k, dtype).reshape(rhs.size, 1, k)
        assert nv.GatherQmm.groups(rhs.size, experts)
        got = nv.gather_qmm(to_dev(x), q, None, torch.from_numpy(rhs).cuda(), nv.GatherQmm(transpose=False, sorted_indices=True))
        want = ref.gather_qmm(x, packed, scales, biases, np.arange(rhs.size, dtype=np.uint32), rhs.astype(np.uint32), mode=mode,
                              group=group, bits=bits, dtype=dtype, transpose=False)
        assert_rows_close(to_host(got).reshape(rhs.size, n), want.reshape(rhs.size, n), dtype,
                          f"untransposed grouped gather mode {mode}, {rhs.size} rows", exact_weights=mode != ref.AFFINE)
        pairwise = nv.gather_qmm(to_dev(x), q, None, torch.from_numpy(rhs).cuda(), nv.GatherQmm(transpose=False))
        assert float((got.float() - pairwise.float()).abs().max()) <= 2e-2 * float(pairwise.float().abs().max())


@pytest.mark.parametrize("route", ["grouped-mxfp4", "grouped-affine4", "pairs-affine4-decode", "pairs-affine8-few", "pairs-mxfp8-general",
                                   "pairs-affine3-rows"])
def test_gather_scatter_rows(route):
    """`nvq_gather_qmm_scatter`: every transposed route of the gathered product writes pair i at `out_rows[i]`; the
    result is the plain gathered product permuted, bit for bit.  The untransposed route refuses it."""
    rng = np.random.default_rng(7300 + len(route))
    dtype = ref.BF16
    experts, k, n = 6, 512, 192
    mode = {"mxfp4": ref.MXFP4, "mxfp8": ref.MXFP8}.get(route.split("-")[1], ref.AFFINE)
    w = make_w(rng, experts * n, k, dtype).reshape(experts, n, k)
    if mode == ref.AFFINE:
        bits = int(route.split("-")[1][len("affine"):])
        group = 64
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
    else:
        packed, scales = ref.fp_quantize(w, dtype, mode)
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(nv.QuantMode.MXFP4 if mode == ref.MXFP4 else nv.QuantMode.MXFP8))
    if route.startswith("grouped"):
        pairs, tokens = 300, 75
        ids = torch.from_numpy(rng.integers(0, experts, pairs).astype(np.int32)).cuda()
        order, restore, sorted_ids, offsets = nv.moe_order(ids, experts)
        x = to_dev(make_x(rng, tokens, k, dtype))
        rows = torch.div(order, pairs // tokens, rounding_mode="floor").to(torch.int32)
        plain = nv.ops.gather_qmm_grouped(x, q, rows, sorted_ids, offsets)
        got = nv.ops.gather_qmm_grouped(x, q, rows, sorted_ids, offsets, out_rows=order)
        assert torch.equal(got.view(torch.int16), plain[restore.long()].view(torch.int16)), route
        with pytest.raises(nv.InvalidArgument):
            nv.ops.gather_qmm_grouped(x, q, rows, sorted_ids, offsets, out_rows=order[:-1])
        return
    m = 3 if route.endswith("rows") else 1
    pairs = 11
    x = to_dev(make_x(rng, pairs * m, k, dtype).reshape(pairs, m, k))
    lhs = torch.from_numpy(rng.permutation(pairs).astype(np.int32)).cuda()
    rhs = torch.from_numpy(rng.integers(0, experts, pairs).astype(np.int32)).cuda()
    perm = torch.from_numpy(rng.permutation(pairs).astype(np.int32)).cuda()
    plain = nv.gather_qmm(x, q, lhs, rhs)
    got = nv.gather_qmm(x, q, lhs, rhs, out_rows=perm)
    want = torch.empty_like(plain)
    want[perm.long()] = plain
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), route
    if route == "pairs-affine4-decode":  # the untransposed route has no scattered form
        wt = make_w(rng, experts * k, n, dtype).reshape(experts, k, n)
        pt, st, bt = ref.affine_quantize(wt, dtype, 64, 4)
        qt = nv.Quantized(to_dev(pt), to_dev(st), to_dev(bt), nv.Quant.affine(64, 4))
        with pytest.raises(nv.Unsupported):
            nv.gather_qmm(x, qt, lhs, rhs, nv.GatherQmm(transpose=False), out_rows=perm)


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
@pytest.mark.parametrize("dtype", [ref.BF16, ref.F32, ref.F16])
def test_quantize_dequantize_bit_exact(mode, qmode, dtype):
    """`fp_quantize_dequantize` (kernels.rs:1011-1065), qqmm's activations: bit for bit the oracle, special values
    included, with and without NVFP4's global scale; it equals dequantize(quantize(x)) in x's type where no global scale
    is involved."""
    rng = np.random.default_rng(6100 + mode + dtype)
    x = make_x(rng, 37, 320, dtype)
    wide = ref.to_f32(x, dtype)
    wide[3, :] = 0.0
    wide[4, 5], wide[5, 6], wide[6, 7] = np.nan, np.inf, -np.inf
    wide[7, :] = wide[7, :] * 1e-30
    x = ref.from_f32(wide, dtype)
    qm = getattr(nv.QuantMode, qmode)
    want = ref.fp_quantize_dequantize(x, dtype, mode)
    got = to_host(nv.quantize_dequantize(to_dev(x), qm))
    nan = lambda a: np.isnan(ref.to_f32(a, dtype))
    same = (got.view(np.uint8).reshape(got.shape + (-1,)) == want.view(np.uint8).reshape(want.shape + (-1,))).all(-1)
    assert np.all(same | (nan(got) & nan(want)))
    packed, scales = ref.fp_quantize(x, dtype, mode)
    round_trip = ref.fp_dequantize(packed, scales, mode, dtype)
    assert np.array_equal(ref.to_f32(want, dtype)[:3], ref.to_f32(round_trip, dtype)[:3])
    if mode == ref.NVFP4:
        g = torch.tensor(2.75, dtype=torch.float32, device="cuda")
        want = ref.fp_quantize_dequantize(x[:3], dtype, mode, 2.75)
        got = to_host(nv.quantize_dequantize(to_dev(x[:3]), qm, g))
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    else:
        with pytest.raises(nv.InvalidArgument):
            nv.quantize_dequantize(to_dev(x), qm, torch.tensor(1.0, device="cuda"))
    with pytest.raises(nv.InvalidArgument):
        nv.quantize_dequantize(to_dev(x), nv.Quant.affine(64, 4))


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F32, ref.F16])
@pytest.mark.parametrize("group,bits,d", [(64, 4, 128), (32, 8, 64), (64, 3, 128)])
def test_quantized_attention_composition(dtype, group, bits, d):
    """`quantized_attention` (fast.rs:694-718) as the reference composes it over the library's products: one query row
    per head over quantized keys and values, grouped heads, with and without sinks, against attention over the
    oracle's dequantized cache in float64 (the bound the reference states for it: that of the dequantized attention)."""
    from nuvec_amd.layers import quantized_attention
    rng = np.random.default_rng(8100 + bits + dtype)
    b, hkv, rep, s = 2, 2, 4, 203  # positions that fill no tile of keys
    hq = hkv * rep
    kd, vd = make_x(rng, b * hkv * s, d, dtype).reshape(b, hkv, s, d), make_x(rng, b * hkv * s, d, dtype).reshape(b, hkv, s, d)
    kq, vq = ref.affine_quantize(kd, dtype, group, bits), ref.affine_quantize(vd, dtype, group, bits)
    q = make_x(rng, b * hq, d, dtype).reshape(b, hq, 1, d)
    sinks = ref.from_f32(rng.standard_normal(hq).astype(np.float32), dtype)
    quant = nv.Quant.affine(group, bits)
    K = nv.Quantized(to_dev(kq[0]), to_dev(kq[1]), to_dev(kq[2]), quant)
    V = nv.Quantized(to_dev(vq[0]), to_dev(vq[1]), to_dev(vq[2]), quant)
    scale = 1.0 / np.sqrt(d)
    kf = ref.to_f32(ref.affine_dequantize(*kq, dtype, group, bits), dtype).astype(np.float64)
    vf = ref.to_f32(ref.affine_dequantize(*vq, dtype, group, bits), dtype).astype(np.float64)
    qf = ref.to_f32(q, dtype).astype(np.float64).reshape(b, hkv, rep, d)
    logits = scale * np.einsum("bhrd,bhsd->bhrs", qf, kf)
    tol = {ref.BF16: 2e-2, ref.F32: 2e-5, ref.F16: 2.5e-3}[dtype]
    from nuvec_amd import ops as nv_ops
    fits = nv_ops.quantized_attention_fits(to_dev(q), K, V)
    assert fits == (bits in (3, 4, 8) and d in (64, 128))  # the fused kernel's rule (fast/imp.rs:3944-3992)
    for use_sinks in (False, True):
        full = logits
        if use_sinks:
            full = np.concatenate([logits, np.broadcast_to(ref.to_f32(sinks, dtype).astype(np.float64).reshape(1, hkv, rep, 1), (b, hkv, rep, 1))], -1)
        p = np.exp(full - full.max(-1, keepdims=True))
        p = (p / p.sum(-1, keepdims=True))[..., :s]
        want = np.einsum("bhrs,bhsd->bhrd", p, vf).reshape(b, hq, 1, d)
        for fused in (True, False):  # the kernel where it fits, and the composition
            got = quantized_attention(to_dev(q), K, V, scale, to_dev(sinks) if use_sinks else None, fused=fused)
            assert tuple(got.shape) == (b, hq, 1, d)
            err = np.abs(ref.to_f32(to_host(got), dtype).astype(np.float64) - want).max()
            assert err <= tol * max(1.0, np.abs(want).max()), f"sinks={use_sinks} fused={fused}: {err}"
    with pytest.raises(nv.InvalidArgument):
        quantized_attention(to_dev(q), K, nv.Quantized(V.weight, V.scales, V.biases, nv.Quant.affine(group, 2 if bits != 2 else 4)), scale)
