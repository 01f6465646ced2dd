"""A seeded sweep of shapes over every product route of the HIP library against the CPU oracle: modes, widths, groups,
element types, row counts on both sides of every routing threshold, K and N with tails, both weight orientations,
batched and gathered products.  The bars are those of tests/test_gpu_parity.py."""
import numpy as np
import pytest
import torch

import nuvec_amd as nv
from oracle import ref
from tests.hip_backend import to_dev, to_host
from tests.test_gpu_parity import assert_rows_close, make_w, make_x

pytestmark = pytest.mark.gpu

AFFINE_FORMS = [(g, b) for g in (32, 64, 128) for b in (1, 2, 3, 4, 5, 6, 8)]
ROWS = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 33, 64, 100, 192, 193, 257]


def draw(rng):
    mode = int(rng.choice([ref.AFFINE, ref.AFFINE, ref.AFFINE, ref.MXFP4, ref.MXFP8, ref.NVFP4]))
    dtype = int(rng.choice([ref.BF16, ref.BF16, ref.F16, ref.F32]))
    if mode == ref.AFFINE:
        group, bits = AFFINE_FORMS[int(rng.integers(len(AFFINE_FORMS)))]
    else:
        group, bits = ref.FP_PARAMS[mode]
    return mode, dtype, group, bits


def quantized(rng, mode, dtype, group, bits, lead, rows, cols):
    """Weights `lead + [rows, cols]` quantized along `cols` by the oracle; the operands on the host and the device."""
    w = make_w(rng, int(np.prod(lead, dtype=np.int64)) * rows, cols, dtype).reshape(tuple(lead) + (rows, cols))
    if mode == ref.AFFINE:
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), nv.Quant.affine(group, bits))
    else:
        packed, scales = ref.fp_quantize(w, dtype, mode)
        biases = None
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, nv.Quant.new(nv.QuantMode(mode)))
    return (packed, scales, biases), q


def unit(group, bits):
    """The last dimension comes in whole groups and whole words."""
    step = group
    while (step * bits) % 32:
        step += group
    return step


@pytest.mark.parametrize("seed", range(48))
def test_products_sweep(seed):
    rng = np.random.default_rng(9000 + seed)
    mode, dtype, group, bits = draw(rng)
    transpose = bool(rng.random() < 0.75)
    m = int(rng.choice(ROWS))
    step = unit(group, bits)
    inner = step * int(rng.integers(1, 2048 // step + 2))      # the quantized axis: K (transposed) or N
    other = int(rng.choice([32, 96, 200, 256, 513, 1000])) if transpose else 32 * int(rng.integers(1, 17))
    k, n = (inner, other) if transpose else (other, inner)
    batch = () if rng.random() < 0.7 else (int(rng.integers(1, 4)),)
    shared = bool(rng.random() < 0.5)
    (packed, scales, biases), q = quantized(rng, mode, dtype, group, bits, () if shared else batch, n if transpose else k, inner)
    x = make_x(rng, int(np.prod(batch, dtype=np.int64)) * m, k, dtype).reshape(batch + (m, k))
    got = to_host(nv.quantized_matmul(to_dev(x), q, transpose))
    want = ref.quantized_matmul(x, packed, scales, biases, mode=mode, group=group, bits=bits, dtype=dtype, transpose=transpose,
                                threads=ref.max_threads())
    what = f"seed {seed}: mode {mode} g{group} b{bits} dtype {dtype} M={m} K={k} N={n} batch={batch} shared={shared} transpose={transpose}"
    assert got.shape == want.shape, what
    assert_rows_close(got.reshape(-1, n), want.reshape(-1, n), dtype, what)


@pytest.mark.parametrize("seed", range(32))
def test_gathers_sweep(seed):
    rng = np.random.default_rng(9500 + seed)
    mode, dtype, group, bits = draw(rng)
    transpose = bool(rng.random() < 0.8)
    step = unit(group, bits)
    inner = step * int(rng.integers(1, 1024 // step + 2))
    other = int(rng.choice([32, 96, 200, 256])) if transpose else 32 * int(rng.integers(1, 9))
    k, n = (inner, other) if transpose else (other, inner)
    experts = int(rng.integers(1, 9))
    (packed, scales, biases), q = quantized(rng, mode, dtype, group, bits, (experts,), n if transpose else k, inner)
    form = int(rng.integers(3))
    if form == 0 and transpose:  # sorted rows of one token each: the grouped route when the rule takes it
        pairs = int(rng.choice([16, 40, 130, 300]))
        rhs = np.sort(rng.integers(0, experts, pairs)).astype(np.uint32)
        x = make_x(rng, pairs, k, dtype).reshape(pairs, 1, k)
        got = nv.gather_qmm(to_dev(x), q, None, torch.from_numpy(rhs.astype(np.int32)).cuda(), nv.GatherQmm(sorted_indices=True))
        lhs = np.arange(pairs, dtype=np.uint32)
        m = 1
    else:
        pairs, m = int(rng.integers(1, 20)), int(rng.choice([1, 1, 2, 5]))
        xb = int(rng.integers(1, 6))
        x = make_x(rng, xb * m, k, dtype).reshape(xb, m, k)
        lhs, rhs = rng.integers(0, xb, pairs).astype(np.uint32), rng.integers(0, experts, pairs).astype(np.uint32)
        got = nv.gather_qmm(to_dev(x), q, torch.from_numpy(lhs.astype(np.int32)).cuda(), torch.from_numpy(rhs.astype(np.int32)).cuda(),
                            nv.GatherQmm(transpose=transpose))
    want = ref.gather_qmm(x, packed, scales, biases, lhs, rhs, mode=mode, group=group, bits=bits, dtype=dtype, transpose=transpose,
                          threads=ref.max_threads())
    what = f"seed {seed}: mode {mode} g{group} b{bits} dtype {dtype} M={m} K={k} N={n} experts={experts} pairs={pairs} form={form} transpose={transpose}"
    got = to_host(got)
    assert got.shape == want.shape, what
    assert_rows_close(got.reshape(-1, n), want.reshape(-1, n), dtype, what)


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F32])
def test_nvfp4_rows_ending_in_half_a_slice(dtype):
    """NVFP4 groups hold 16 values, so a packed row may end in half of a lane's slice of 32 (K % 32 == 16 with the
    weights stored [N, K], N % 32 == 16 with [K, N]): row strides, the absent group's codes and scale, the stores."""
    rng = np.random.default_rng(9900 + dtype)
    for transpose, m, k, n in [(True, 1, 16, 40), (True, 3, 112, 33), (True, 15, 1232, 96), (False, 1, 64, 16), (False, 5, 96, 48),
                               (False, 2, 160, 2064)]:
        inner = k if transpose else n
        (packed, scales, _), q = quantized(rng, ref.NVFP4, dtype, 16, 4, (), n if transpose else k, inner)
        x = make_x(rng, m, k, dtype)
        got = to_host(nv.quantized_matmul(to_dev(x), q, transpose))
        want = ref.quantized_matmul(x, packed, scales, None, mode=ref.NVFP4, group=16, bits=4, dtype=dtype, transpose=transpose)
        assert got.shape == want.shape == (m, n)
        # few outputs per row: the bar is taken against the largest output of the product, not of the row
        g, w = ref.to_f32(got, dtype).astype(np.float64), ref.to_f32(want, dtype).astype(np.float64)
        assert np.abs(g - w).max() <= {ref.BF16: 1e-2, ref.F32: 1e-4}[dtype] * np.abs(w).max(), (transpose, m, k, n)
