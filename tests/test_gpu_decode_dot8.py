"""The integer dot-product decode kernel (`qmv4_dot8_kernel`): one row of x against 4-bit affine weights with K in whole
chunks of 2048 up to 14336, the reference's `qmv_fast` shape (crates/nuvec-kernels/src/metal/quantized.h:876-988, routed at
crates/nuvec-core/src/gpu.rs:7025-7060).  x enters as 16-bit fixed point per slice of 32 values, so the tests hold the
values to the CPU's product like every other kernel's (every output within the bar of its row, and within half of it
against the device arithmetic) and then press on what fixed point could break: slices whose values span many binades,
zeros, tiny and huge magnitudes, NaN and infinities, rows off the block size, every group size, both element types, the
bias epilogue, and row-exact rows against their one-row products."""
import numpy as np
import pytest
import torch

import nuvec_amd as nv
from nuvec_amd import ops
from oracle import ref
from tests.hip_backend import TORCH, to_dev, to_host
from tests.test_gpu_parity import assert_device_arithmetic, assert_rows_close, make_w, make_x

pytestmark = pytest.mark.gpu


def product(x, w, dtype, group, **kw):
    q = nv.quantize(to_dev(w), nv.Quant.affine(group, 4))
    got = to_host(nv.quantized_matmul(to_dev(x), q, **kw))
    return got, (to_host(q.weight), to_host(q.scales), to_host(q.biases))


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("n,k,group", [(14336, 4096, 64), (4096, 4096, 64), (4096, 2048, 64), (1024, 4096, 32), (11008, 4096, 128),
                                       (2049, 2048, 128), (1031, 4096, 64), (5000, 2048, 32), (28672, 4096, 64), (16400, 2048, 64),
                                       (4096, 14336, 64), (4096, 8192, 64), (1032, 6144, 128), (5120, 12288, 32), (2048, 10240, 64)])
def test_values_against_the_cpu_product(dtype, n, k, group):
    """Rows that fill the blocks and rows that do not (N off 8 R for every R the host picks), both K, the three groups."""
    rng = np.random.default_rng(n + k + group)
    w, x = make_w(rng, n, k, dtype), make_x(rng, 1, k, dtype)
    assert ops.quantized_matmul_route(1, n, k, nv.Quant.affine(group, 4), TORCH[dtype]) == "qmv4_dot8_kernel"
    got, (packed, scales, biases) = product(x, w, dtype, group)
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=4, dtype=dtype, threads=8)
    what = f"integer decode g{group} N={n} K={k}"
    assert_rows_close(got, want, dtype, what)
    assert_device_arithmetic(got, x, packed, scales, biases, group, 4, dtype, what)


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_slices_that_span_many_binades(dtype):
    """Fixed point is relative to a slice's largest value: slices with one large value among small ones, values that
    shrink by a factor of two from one to the next, exact zeros, whole slices of zeros, and magnitudes near the ends of
    the element type's range.  The bar is the row's, so what the large values dominate must still be within it."""
    rng = np.random.default_rng(77)
    n, k, group = 2048, 4096, 64
    w = make_w(rng, n, k, dtype)
    big, small = (3.0e4, 1.0e-4) if dtype == ref.F16 else (1.0e30, 1.0e-30)
    rows = []
    base = rng.standard_normal(k).astype(np.float32)
    a = base.copy(); a[::32] *= 4096.0; rows.append(a)                                   # one large value per slice
    a = base.copy(); a *= np.exp2(-(np.arange(k) % 32)).astype(np.float32); rows.append(a)  # 31 binades inside a slice
    a = base.copy(); a[::3] = 0.0; a[64:128] = 0.0; rows.append(a)                       # zeros, a group of zeros
    rows.append(base * np.float32(big / 8))                                              # near the top of the range
    rows.append(base * np.float32(small))                                                # tiny (subnormal halves in f16)
    a = np.zeros(k, np.float32); a[5] = 1.0; rows.append(a)                              # a single value
    rows.append(np.zeros(k, np.float32))                                                 # nothing at all
    q = nv.quantize(to_dev(w), nv.Quant.affine(group, 4))
    packed, scales, biases = to_host(q.weight), to_host(q.scales), to_host(q.biases)
    for i, r in enumerate(rows):
        x = ref.from_f32(r.reshape(1, k), dtype)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=4, dtype=dtype, threads=8)
        if i == len(rows) - 1:
            assert not ref.to_f32(got, dtype).any()  # an all-zero x gives exact zeros
            continue
        assert_rows_close(got, want, dtype, f"integer decode, x case {i}")


def test_nan_and_infinity_reach_every_output():
    """A NaN in x is a NaN in every output (the CPU's product multiplies it with every row); an infinity gives a
    non-finite output everywhere (infinity or NaN on the CPU, NaN here: the slice's scale is NaN)."""
    rng = np.random.default_rng(3)
    n, k = 1024, 2048
    w = make_w(rng, n, k, ref.BF16)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    for bad in (np.nan, np.inf, -np.inf):
        x = rng.standard_normal((1, k)).astype(np.float32)
        x[0, 777] = bad
        got = ref.to_f32(to_host(nv.quantized_matmul(to_dev(ref.from_f32(x, ref.BF16)), q)), ref.BF16)
        assert not np.isfinite(got).any()


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_row_exact_rows_have_the_bits_of_the_one_row_product(dtype):
    """crates/nuvec-core/tests/quantized.rs:794-831 on this kernel: a plain one-row product, a row-exact one and the rows of
    a row-exact or `rows` product all run the same arithmetic."""
    rng = np.random.default_rng(11)
    n, k, m = 3000, 4096, 5
    w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    xd = to_dev(x)
    both = to_host(nv.quantized_matmul(xd, q, row_exact=True)).view(np.uint8)
    wide = to_host(nv.quantized_matmul(to_dev(np.concatenate([x, x, x])), q, rows=True)).view(np.uint8)
    for r in range(m):
        one = to_host(nv.quantized_matmul(xd[r:r + 1], q)).view(np.uint8)
        assert np.array_equal(one[0], both[r]) and np.array_equal(one[0], wide[r]) and np.array_equal(one[0], wide[2 * m + r])


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_two_rows_in_one_pass(dtype):
    """Two rows of x against 8192 weight rows and more share one pass over the weights (the limbs of both rows in
    registers, the codes fetched once); each row keeps the bits of its one-row product, so the pair is row-exact as it is."""
    rng = np.random.default_rng(23)
    n, k = 8200, 4096
    quant = nv.Quant.affine(64, 4)
    assert ops.quantized_matmul_route(2, n, k, quant, TORCH[dtype]) == "qmv4_dot8_kernel"
    assert ops.quantized_matmul_route(2, 4096, k, quant, TORCH[dtype]) != "qmv4_dot8_kernel"  # (small matrices: the other decode kernels)
    assert ops.quantized_matmul_route(3, n, k, quant, TORCH[dtype]) != "qmv4_dot8_kernel"
    w, x = make_w(rng, n, k, dtype), make_x(rng, 2, k, dtype)
    got, (packed, scales, biases) = product(x, w, dtype, 64)
    want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=dtype, threads=8)
    assert_rows_close(got, want, dtype, "integer decode, two rows")
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), quant)
    for r in range(2):
        one = to_host(nv.quantized_matmul(to_dev(x[r:r + 1]), q))
        assert np.array_equal(one.view(np.uint8)[0], got.view(np.uint8)[r])


def test_bias_epilogue_and_repeatability():
    """QuantizedLinear's bias (crates/nuvec-nn/src/layers.rs:155-162): the rounded product plus the bias, rounded again, bit
    for bit; and two launches give the same bits."""
    rng = np.random.default_rng(19)
    n, k = 4096, 4096
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, 1, k, ref.BF16)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    bias = torch.randn(n, device="cuda").to(torch.bfloat16)
    xd = to_dev(x)
    plain = nv.quantized_matmul(xd, q)
    assert torch.equal(plain, nv.quantized_matmul(xd, q))
    from nuvec_amd.layers import QuantizedLinear
    layer = QuantizedLinear(q.weight, q.scales, q.biases, bias, q.quant)
    assert torch.equal(layer(xd), plain + bias)


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("k,group", [(64, 64), (128, 32), (128, 128), (256, 64), (512, 64), (96, 32)])
def test_short_rows_of_single_products(dtype, k, group):
    """Rows of at most 512 values (the reference's `qmv_quad` shapes K = 64 and 128,
    crates/nuvec-kernels/src/metal/quantized.h:819-874, and up to sixteen lanes a row): single products take the short-row
    decode kernel, 2 to 16 lanes a weight row, one to four rows of x; rows off the block size."""
    rng = np.random.default_rng(600 + k + group)
    quant = nv.Quant.affine(group, 4)
    for m, n in ((1, 32768), (4, 5000), (3, 1031), (2, 2048)):
        assert ops.quantized_matmul_route(m, n, k, quant, TORCH[dtype]) == "qmv4_short_kernel", (m, n, k)
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        got, (packed, scales, biases) = product(x, w, dtype, group)
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=4, dtype=dtype, threads=8)
        what = f"short rows g{group} M={m} N={n} K={k}"
        assert_rows_close(got, want, dtype, what)
        assert_device_arithmetic(got, x, packed, scales, biases, group, 4, dtype, what, limit=0.8)
    assert ops.quantized_matmul_route(1, 32768, 1024, quant, TORCH[dtype]) != "qmv4_short_kernel" or group != 64  # (longer rows: the other decode kernels)
