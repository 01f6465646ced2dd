"""Batched decode (`qmr_kernel`): 17 to 64 rows of x (up to 128 against few weight rows) against 4- and 8-bit affine weights
stored [N, K] with 8192 rows or more - and fewer rows where the direct few-row kernel's slices of K do not fit -, every
weight fetched and dequantized once per pass.  The reference takes these row counts on its tiled kernel
(crates/nuvec-core/src/gpu.rs:6975-7060, crates/nuvec-kernels/src/metal/quantized.h:1358-1485); the values are held to the
CPU product (crates/nuvec-core/src/kernels.rs:1091-1142) at the bar of the element type (1e-2 of a row's largest output
in bfloat16, 1e-3 in float16) and to the device arithmetic of a once-rounded weight at half of it."""
import numpy as np
import pytest
import torch

import nuvec_amd as nv
from nuvec_amd import ops
from oracle import ref
from tests.hip_backend import to_dev, to_host
from tests.test_gpu_parity import _excess, assert_device_arithmetic, assert_rows_close, make_w, make_x

pytestmark = pytest.mark.gpu

TORCH = {ref.BF16: torch.bfloat16, ref.F16: torch.float16}


# Whole tiles and tails: rows of x off the pass of 64, weight rows off the block of 64 and off the 16-byte stores of y,
# K whose chunks of 512 do not divide among the four wavefronts (9 and 10 chunks), every group size, both element types.
@pytest.mark.parametrize("dtype,group,m,n,k", [
    (ref.BF16, 64, 64, 11008, 4096),
    (ref.BF16, 64, 33, 11017, 4096),
    (ref.F16, 32, 50, 11040, 4608),
    (ref.BF16, 128, 47, 11072, 5120),
    (ref.F16, 128, 64, 12288, 4096),
    # more than 16384 weight rows: blocks of 128 of them; weight rows off the block and off the 16-byte stores
    (ref.BF16, 64, 64, 16512, 4096),
    (ref.F16, 32, 37, 16501, 4096),
    (ref.BF16, 128, 50, 16648, 4608),
    # passes of 32 rows; K of one chunk (three of the block's wavefronts have none), of three and of five; two passes of 64
    # rows, the second short; the 128-row blocks with passes of 32 rows, with the table of scales and (groups of 32) without
    (ref.BF16, 64, 17, 8192, 512),
    (ref.F16, 32, 32, 8200, 1024),
    (ref.BF16, 128, 24, 11008, 4096),
    (ref.BF16, 64, 100, 8192, 2048),
    (ref.F16, 64, 128, 9001, 1536),
    (ref.BF16, 64, 29, 16448, 2560),
    (ref.BF16, 32, 20, 16500, 1024),
    # passes of 16 rows: a short K, the 128-row blocks, groups of 32 and of 128, five and seven rows
    (ref.BF16, 64, 9, 11008, 512),
    (ref.F16, 64, 16, 16500, 8192),
    (ref.BF16, 32, 5, 11050, 4096),
    (ref.BF16, 128, 13, 11008, 8192),
    (ref.BF16, 64, 7, 14350, 512),
    (ref.BF16, 32, 11, 28700, 4096),
])
def test_against_the_cpu_product(dtype, group, m, n, k):
    rng = np.random.default_rng(6100 + group + m + k)
    quant = nv.Quant.affine(group, 4)
    assert ops.quantized_matmul_route(m, n, k, quant, TORCH[dtype]) == "qmr_kernel"
    w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, 4)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), quant)
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=4, dtype=dtype, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    what = f"batched decode g{group} M={m} N={n} K={k}"
    assert_rows_close(got, want, dtype, what)
    assert_device_arithmetic(got, x, packed, scales, biases, group, 4, dtype, what)


# 8-bit codes: blocks of 64 weight rows, the codes of a window one window ahead; passes of 16, 32 and 64 rows, two passes,
# every group size, tails of rows and of weight rows, K of three chunks.
@pytest.mark.parametrize("dtype,group,m,n,k", [
    (ref.BF16, 64, 64, 11008, 4096),
    (ref.F16, 32, 33, 11017, 2048),
    (ref.BF16, 128, 24, 8192, 1536),
    (ref.BF16, 64, 12, 14336, 1024),
    (ref.F16, 64, 100, 8200, 2048),
    (ref.BF16, 32, 50, 16648, 4608),
])
def test_eight_bit_codes_against_the_cpu_product(dtype, group, m, n, k):
    rng = np.random.default_rng(6500 + group + m + k)
    quant = nv.Quant.affine(group, 8)
    assert ops.quantized_matmul_route(m, n, k, quant, TORCH[dtype]) == "qmr_kernel"
    w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
    packed, scales, biases = ref.affine_quantize(w, dtype, group, 8)
    q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), quant)
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=8, dtype=dtype, threads=8)
    got = to_host(nv.quantized_matmul(to_dev(x), q))
    what = f"batched decode b8 g{group} M={m} N={n} K={k}"
    assert_rows_close(got, want, dtype, what)
    assert_device_arithmetic(got, x, packed, scales, biases, group, 8, dtype, what)


def test_routes():
    """The rule is measured: 17 to 64 rows against 8192 weight rows or more (11008 from K = 3072 and for groups of 128,
    which also need K from 4096; short K only up to a number of weight rows), up to 128 rows against fewer than 11008
    weight rows; 4 bits, K in chunks of 512, one product; everything else stays where it was."""
    q4 = nv.Quant.affine(64, 4)
    route = lambda m, n, k, quant=q4, dtype=torch.bfloat16, **kw: ops.quantized_matmul_route(m, n, k, quant, dtype, **kw)
    assert route(33, 14336, 4096) == "qmr_kernel" and route(64, 14336, 4096) == "qmr_kernel"
    assert route(64, 14336, 4096, dtype=torch.float16) == "qmr_kernel" and route(48, 28672, 8192) == "qmr_kernel"
    assert route(17, 14336, 4096) == "qmr_kernel" and route(32, 14336, 4096) == "qmr_kernel"
    assert route(16, 14336, 4096) != "qmr_kernel" and route(65, 14336, 4096) != "qmr_kernel"
    # up to 16 rows: where the direct few-row kernel's slices of K do not fit
    assert route(16, 14336, 512) == "qmr_kernel" and route(9, 14336, 8192) == "qmr_kernel" and route(9, 14336, 2048) == "qmr_kernel"
    assert route(8, 14336, 8192) != "qmr_kernel" and route(8, 14336, 512) == "qmr_kernel" and route(4, 14336, 512) != "qmr_kernel"
    assert route(12, 32768, 2048) != "qmr_kernel" and route(12, 8192, 512) != "qmr_kernel"
    assert route(8, 14336, 4096, nv.Quant.affine(32, 4)) == "qmr_kernel" and route(8, 32768, 4096, nv.Quant.affine(32, 4)) == "qmr_kernel" and route(8, 20480, 4096, nv.Quant.affine(32, 4)) != "qmr_kernel"
    assert route(64, 8192, 4096) != "qmr_kernel" and route(64, 8192, 2048) == "qmr_kernel" and route(128, 8192, 4096) == "qmr_kernel"
    assert route(129, 8192, 4096) != "qmr_kernel" and route(128, 8192, 8192) != "qmr_kernel"
    assert route(64, 14336, 2048) == "qmr_kernel" and route(64, 151936, 4096) == "qmr_kernel"
    assert route(32, 16384, 512) == "qmr_kernel" and route(32, 20480, 512) != "qmr_kernel"
    assert route(32, 32768, 1024) == "qmr_kernel" and route(32, 65536, 1024) != "qmr_kernel" and route(33, 65536, 1024) == "qmr_kernel"
    q128 = nv.Quant.affine(128, 4)
    assert route(64, 14336, 4096, q128) == "qmr_kernel" and route(64, 14336, 2048, q128) != "qmr_kernel"
    assert route(64, 4096, 4096, dtype=torch.float16) != "qmr_kernel"
    assert route(64, 14336, 4096 + 256) != "qmr_kernel"  # K off the chunks of 512
    q8 = nv.Quant.affine(64, 8)
    assert route(64, 14336, 4096, q8) == "qmr_kernel" and route(17, 8192, 2048, q8) == "qmr_kernel" and route(16, 14336, 4096, q8) == "qmr_kernel"
    assert route(7, 14336, 4096, q8) != "qmr_kernel" and route(16, 8192, 4096, q8) != "qmr_kernel" and route(16, 32768, 4096, q8) != "qmr_kernel"
    assert route(128, 8192, 4096, q8) == "qmr_kernel" and route(128, 14336, 4096, q8) != "qmr_kernel" and route(64, 32768, 1024, q8) != "qmr_kernel"
    assert route(32, 14336, 512, q8) != "qmr_kernel" and route(64, 14336, 4096, nv.Quant.affine(64, 6)) != "qmr_kernel"
    assert route(64, 14336, 4096, nv.Quant.new(nv.QuantMode.MXFP4)) != "qmr_kernel"
    assert route(64, 14336, 4096, dtype=torch.float32) != "qmr_kernel"
    assert route(64, 14336, 4096, batch=2) != "qmr_kernel"
    assert route(64, 14336, 4096, rows=True) != "qmr_kernel"


def test_bias_epilogue_and_determinism():
    """QuantizedLinear's bias in the epilogue is the separate addition bit for bit (crates/nuvec-nn/src/layers.rs:155-162),
    and two launches give the same bits (the wavefronts' partial tiles are added in a fixed order)."""
    rng = np.random.default_rng(6200)
    m, n, k = 40, 11008, 4096
    quant = nv.Quant.affine(64, 4)
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
    q = nv.quantize(to_dev(w), quant)
    xd = to_dev(x)
    bias = (torch.randn(n, device="cuda") * 0.5).to(torch.bfloat16)
    plain = nv.quantized_matmul(xd, q)
    again = nv.quantized_matmul(xd, q)
    assert torch.equal(plain.view(torch.int16), again.view(torch.int16))
    fused = nv.quantized_matmul(xd, q, bias=bias)
    assert torch.equal(fused.view(torch.int16), (plain + bias).view(torch.int16))


@pytest.mark.parametrize("m,n,k,limit", [(64, 11008, 4096, 0.95), (32, 8192, 512, 1.0)])
def test_margin_over_seeds(m, n, k, limit):
    """The weights are rounded once, as the tiled and the few-row kernels': the worst output of a product stays under the
    bar for every seed tried - with room at K = 4096 (0.68 to 0.72 of it), with little at the fewest weight rows and the
    shortest K the route sends here (0.70 to 0.93: the same outputs, to the digit, as on the kernel that took the product
    before; the CPU's first rounding of code * scale is a noise of the same fraction of an output as of a weight, and
    a short K leaves the largest output of a row less far above the others)."""
    quant = nv.Quant.affine(64, 4)
    assert ops.quantized_matmul_route(m, n, k, quant, torch.bfloat16) == "qmr_kernel"
    worst = []
    for seed in range(10):
        rng = np.random.default_rng(6300 + seed)
        w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
        packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 4)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), quant)
        want = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.BF16, threads=8)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        worst.append(float(np.max(_excess(got, want, ref.BF16))))
    print(f"batched decode M={m} N={n} K={k}, worst output over 10 seeds, x the bar:", " ".join(f"{v:.3f}" for v in worst))
    assert max(worst) <= limit, worst
