"""The few-row kernel on the 16x16x32 matrix instruction with directly loaded weight operands (`qmd_kernel`: the
counterpart of the reference's `affine_qmv_mma`, crates/nuvec-kernels/src/metal/quantized.h:1722-1905, routed at
crates/nuvec-core/src/gpu.rs:6978-7024), and the routing of the BASELINE configurations.

Like the reference's `few_row_mma_products_match_the_dequantized_product` (crates/nuvec-core/tests/quantized.rs:881-935)
the tests name the kernel a product must run on and hold its values to the CPU's product: every output within the
bar of its row against the CPU oracle, and within half of it against the device arithmetic."""
import numpy as np
import pytest
import torch

import nuvec_amd as nv
from nuvec_amd import ops
from oracle import ref
from tests.hip_backend import TORCH, to_dev, to_host
from tests.test_gpu_parity import assert_device_arithmetic, assert_rows_close, make_w, make_x

pytestmark = pytest.mark.gpu

WIDTHS = [(2, 64), (2, 128), (3, 64), (3, 128), (4, 32), (4, 64), (4, 128), (5, 64), (5, 128), (6, 32), (6, 64), (6, 128), (8, 32), (8, 64), (8, 128)]


def test_routes_of_the_baseline_configurations():
    """Which kernel each BASELINE configuration runs on (the routing code answers, not a table of the test)."""
    bf16 = torch.bfloat16
    c2 = lambda m, **kw: ops.quantized_matmul_route(m, 14336, 4096, nv.Quant.affine(64, 4), bf16, **kw)
    assert ops.quantized_matmul_route(1, 4096, 4096, nv.Quant.affine(64, 4), torch.float32) == "qmv_lds_kernel"
    assert c2(1) == "qmv4_dot8_kernel"  # (one row, K = 4096: the integer dot-product decode kernel)
    assert c2(2) == "qmv4_dot8_kernel"  # (two rows share a pass over a matrix this large)
    assert c2(3) == "qmv4_mm16_kernel" and c2(4) == "qmv4_mm16_kernel" and c2(8) == "qmv4_mm16_kernel"
    assert c2(12) == "qmd_kernel" and c2(16) == "qmd_kernel"
    assert c2(2048) == "qmm_kernel"
    # row-exact rows take the kernel of the one-row product, each row as its own pass
    assert c2(8, row_exact=True) == "qmv4_dot8_kernel" and c2(300, rows=True) == "qmv4_dot8_kernel"
    assert ops.quantized_matmul_route(1, 14336, 8192, nv.Quant.affine(64, 4), bf16) == "qmv4_dot8_kernel"  # (K in chunks of 2048 up to 14336)
    assert ops.quantized_matmul_route(1, 14336, 16384, nv.Quant.affine(64, 4), bf16) == "qmv4_lds_kernel"
    assert ops.quantized_matmul_route(2, 14336, 8192, nv.Quant.affine(64, 4), bf16) != "qmv4_dot8_kernel"  # (one row of x only beyond 4096)
    for group, bits in ((64, 3), (32, 8)):
        c4 = lambda m, **kw: ops.quantized_matmul_route(m, 4096, 4096, nv.Quant.affine(group, bits), bf16, **kw)
        assert c4(1) == "qmv4_lds_kernel"  # (the decode kernel takes a row of 3- and of 8-bit codes too)
        assert c4(16) == "qmd_kernel" and c4(5) == "qmd_kernel" and c4(2) == "qmv4_lds_kernel"  # (K = 4096: two rows stay on the decode kernel)
        assert c4(512) == "qmm_kernel"
        assert c4(16, transpose=False) == "qmn_kernel" and c4(1, transpose=False) == "qmn_kernel"  # runs of eight codes: every width
        assert ops.quantized_matmul_route(1, 14336, 4096, nv.Quant.affine(group, bits), bf16, transpose=False) == ("qmn_kernel" if bits == 8 else "qvm_kernel")
        assert c4(16, row_exact=False, rows=True) == "qmv_lds_kernel"
    assert ops.quantized_matmul_route(24, 1000, 1024, nv.Quant.affine(64, 6), bf16) == "qmf_kernel"
    assert ops.quantized_matmul_route(96, 4096, 14336, nv.Quant.affine(64, 4), bf16) == "qmm_kernel"  # (a long K: the tiles split it: 41 us against 75; at 24 rows the few-row kernel's one round is ahead, 32 against 38)
    assert ops.quantized_matmul_route(16, 1100, 4096 + 128, nv.Quant.affine(64, 3), bf16) == "qmf_kernel"  # K off the kernel's slices
    # (rows of fewer than 1024 outputs, up to 16 rows of x: the vector kernel with the CPU's weights, ahead on matrices this small)
    assert ops.quantized_matmul_route(16, 1000, 4096 + 128, nv.Quant.affine(64, 3), bf16) == "qmv_lds_kernel"
    assert ops.quantized_matmul_route(64, 2880, 2880, nv.Quant.new(nv.QuantMode.MXFP4), bf16) in ("qmf_kernel", "qmm_kernel")
    # passes of 16 rows where the matrix is small enough to be read again from the caches; the tiles beyond
    # (bfloat16 products of more than 16 rows and fewer than 8192 outputs per row take the kernels that hold the CPU's weights)
    small = lambda m, t=torch.float16: ops.quantized_matmul_route(m, 1024, 4096, nv.Quant.affine(64, 4), t)
    assert small(64) == "qmd_kernel" and small(192) == "qmd_kernel" and small(512) in ("qmf_kernel", "qmm_kernel")
    assert small(16, bf16) == "qmd_kernel" and small(64, bf16) in ("qmf_kernel", "qmm_kernel") and small(192, bf16) in ("qmf_kernel", "qmm_kernel")
    assert ops.quantized_matmul_route(64, 8192, 4096, nv.Quant.affine(64, 4), bf16) == "qmd_kernel"
    assert c2(17) == "qmr_kernel" and c2(32) == "qmr_kernel" and c2(96) == "qmm_kernel"
    assert c2(33) == "qmr_kernel" and c2(64) == "qmr_kernel"  # (one pass over this many weight rows: the batched-decode kernel)
    # the few-row kernel of the 32x32x16 instruction keeps what the direct kernel does not take
    for m, n, k, group, bits in ((5, 1077, 1152, 64, 3), (16, 1130, 2176, 32, 8), (20, 1000, 1024, 64, 6)):
        assert ops.quantized_matmul_route(m, n, k, nv.Quant.affine(group, bits), bf16) == "qmf_kernel", (m, n, k, group, bits)
    # (a tiny product of more than 16 rows: the two kernels are within a microsecond of each other, W[4096,128] at 32 rows 6.5 against 7.1 us)
    assert ops.quantized_matmul_route(30, 64, 128, nv.Quant.affine(64, 4), bf16) in ("qmf_kernel", "qmm_kernel")


# (rows of 1024 outputs or more: affine products of shorter rows take the kernels that materialise the CPU's weights)
SHAPES = [(2, 1224, 512), (9, 2024, 1024), (16, 1154, 4096), (13, 1120, 8192), (11, 1072, 14336), (23, 1088, 1536), (16, 5000, 512),
          (12, 1064, 7168), (77, 1324, 2048), (130, 1072, 512), (23, 8200, 512)]


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
@pytest.mark.parametrize("bits,group", WIDTHS)
def test_direct_few_row_kernel_every_width(dtype, bits, group):
    """One to nine passes of rows, K of one chunk, of several (8192: 2 chunks of 8 slices; 14336: 4 of 7; 7168: 2 of 7),
    N off the tile and with several tiles per block, tails of rows."""
    rng = np.random.default_rng(4000 + 10 * bits + group)
    quant = nv.Quant.affine(group, bits)
    for m, n, k in SHAPES:
        route = ops.quantized_matmul_route(m, n, k, quant, TORCH[dtype])
        if bits == 4 and m <= 8:
            continue  # the 4-bit decode kernels' rows
        if bits in (5, 6) and m > 16:
            continue  # passes of rows of 5- and 6-bit codes stay on the kernels that round a weight once
        if dtype == ref.BF16 and m > 16 and n < 8192:  # the CPU's weights: not this kernel's, which never materialises one
            assert route in ("qmf_kernel", "qmm_kernel"), f"b{bits} g{group} M={m} N={n} K={k} runs on {route}"
            continue
        # (more than 16 rows against 8192 weight rows or more of 4-bit codes: one pass of the batched-decode kernel, but
        # for groups of 128 at a short K)
        expect = "qmr_kernel" if bits == 4 and group != 128 and m > 16 and n >= 8192 else "qmd_kernel"
        assert route == expect, f"b{bits} g{group} M={m} N={n} K={k} runs on {route}"
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        packed, scales, biases = ref.affine_quantize(w, dtype, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), quant)
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype, threads=8)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        what = f"direct few rows b{bits} g{group} M={m} N={n} K={k}"
        assert_rows_close(got, want, dtype, what)
        if m <= 32:  # (one rounding step of a row's largest output is up to 0.78 x the bar: the float32 sums differ in order)
            assert_device_arithmetic(got, x, packed, scales, biases, group, bits, dtype, what, limit=0.8)


@pytest.mark.parametrize("bits,group", [(3, 64), (8, 32), (4, 128)])
def test_direct_few_row_kernel_batched_with_bias(bits, group):
    """A batch of weight matrices (one stride per operand) and the layer's bias in the epilogue."""
    rng = np.random.default_rng(4100 + bits)
    b, m, n, k = 3, 10, 1120, 1024
    quant = nv.Quant.affine(group, bits)
    assert ops.quantized_matmul_route(m, n, k, quant, torch.bfloat16, batch=b) == "qmd_kernel"
    w, x = make_w(rng, b * n, k, ref.BF16), make_x(rng, b * m, k, ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, group, bits)
    q = nv.Quantized(to_dev(packed.reshape(b, n, -1)), to_dev(scales.reshape(b, n, -1)), to_dev(biases.reshape(b, n, -1)), quant)
    got = to_host(nv.quantized_matmul(to_dev(x.reshape(b, m, k)), q))
    for i in range(b):
        want = ref.quantized_matmul(x[i * m:(i + 1) * m], packed[i * n:(i + 1) * n], scales[i * n:(i + 1) * n],
                                    biases[i * n:(i + 1) * n], group=group, bits=bits, dtype=ref.BF16)
        assert_rows_close(got[i], want, ref.BF16, f"direct few rows batched b{bits} item {i}")
    # two batch dimensions of dense operands are one to the kernels (not the vector kernels' business)
    assert ops.quantized_matmul_route(m, n, k, quant, torch.bfloat16, batch=(3, 1)) == "qmd_kernel"
    assert ops.quantized_matmul_route(40, n, k, nv.Quant.affine(32, 5), torch.bfloat16, batch=(2, 3)) in ("qmf_kernel", "qmm_kernel")  # (5 bits in groups of 32: not the direct kernel's)
    w2, x2 = make_w(rng, 6 * n, k, ref.BF16), make_x(rng, 6 * m, k, ref.BF16)
    p2, s2, b2 = ref.affine_quantize(w2, ref.BF16, group, bits)
    q2 = nv.Quantized(to_dev(p2.reshape(2, 3, n, -1)), to_dev(s2.reshape(2, 3, n, -1)), to_dev(b2.reshape(2, 3, n, -1)), quant)
    got2 = to_host(nv.quantized_matmul(to_dev(x2.reshape(2, 3, m, k)), q2)).reshape(6, m, n)
    for i in range(6):
        want = ref.quantized_matmul(x2[i * m:(i + 1) * m], p2[i * n:(i + 1) * n], s2[i * n:(i + 1) * n], b2[i * n:(i + 1) * n],
                                    group=group, bits=bits, dtype=ref.BF16)
        assert_rows_close(got2[i], want, ref.BF16, f"direct few rows, batch [2,3] b{bits} item {i}")
    # bias: the rounded product plus the bias, rounded (layers.rs:155-162), bit for bit the separate addition
    q0 = nv.Quantized(q.weight[0].contiguous(), q.scales[0].contiguous(), q.biases[0].contiguous(), quant)
    bias = to_dev(make_x(rng, 1, n, ref.BF16)[0])
    xd = to_dev(x[:m])
    fused = nv.quantized_matmul(xd, q0, bias=bias)
    assert np.array_equal(to_host(fused).view(np.uint8), to_host(nv.quantized_matmul(xd, q0) + bias).view(np.uint8))


def test_direct_few_row_kernel_per_pair_gather():
    """gather_qmm without offsets: one product per pair on the same kernel (pairs over grid z)."""
    rng = np.random.default_rng(4200)
    experts, n, k, m, pairs = 5, 1104, 1024, 6, 7
    w = make_w(rng, experts * n, k, ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, 64, 3)
    q = nv.Quantized(to_dev(packed.reshape(experts, n, -1)), to_dev(scales.reshape(experts, n, -1)),
                     to_dev(biases.reshape(experts, n, -1)), nv.Quant.affine(64, 3))
    x = make_x(rng, 4 * m, k, ref.BF16)
    lhs = rng.integers(0, 4, pairs).astype(np.uint32)
    rhs = rng.integers(0, experts, pairs).astype(np.uint32)
    got = to_host(nv.gather_qmm(to_dev(x.reshape(4, m, k)), q, torch.from_numpy(lhs.astype(np.int64)).cuda(),
                                torch.from_numpy(rhs.astype(np.int64)).cuda(), nv.GatherQmm()))
    for z in range(pairs):
        e = int(rhs[z])
        want = ref.quantized_matmul(x[lhs[z] * m:(lhs[z] + 1) * m], packed[e * n:(e + 1) * n], scales[e * n:(e + 1) * n],
                                    biases[e * n:(e + 1) * n], group=64, bits=3, dtype=ref.BF16)
        assert_rows_close(got[z], want, ref.BF16, f"direct few rows, pair {z}")


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16])
def test_direct_few_row_kernel_block_formats(mode, qmode, dtype):
    """MXFP4, MXFP8 and NVFP4 (no global scale) on the same kernel: the scaled conversions give the dequantized elements
    themselves, exact in the element type, so the bar holds for every output; a batch; pairs of a gather."""
    rng = np.random.default_rng(4300 + 10 * mode + dtype)
    group, bits = ref.FP_PARAMS[mode]
    quant = nv.Quant.new(getattr(nv.QuantMode, qmode))
    for m, n, k in [(5, 200, 512), (7, 1000, 1024), (16, 130, 4096), (13, 96, 8192), (3, 48, 14336), (23, 64, 1536), (8, 5000, 512),
                    (50, 300, 2048)]:
        assert ops.quantized_matmul_route(m, n, k, quant, TORCH[dtype]) == "qmd_kernel", (qmode, m, n, k)
        w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
        packed, scales = ref.fp_quantize(w, dtype, mode)
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, quant)
        want = ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=dtype, threads=8)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, dtype, f"direct few rows {qmode} M={m} N={n} K={k}", exact_weights=True)
    b, m, n, k = 3, 6, 96, 512
    assert ops.quantized_matmul_route(m, n, k, quant, TORCH[dtype], batch=b) == "qmd_kernel"
    w, x = make_w(rng, b * n, k, dtype), make_x(rng, b * m, k, dtype)
    packed, scales = ref.fp_quantize(w, dtype, mode)
    q = nv.Quantized(to_dev(packed.reshape(b, n, -1)), to_dev(scales.reshape(b, n, -1)), None, quant)
    got = to_host(nv.quantized_matmul(to_dev(x.reshape(b, m, k)), q))
    for i in range(b):
        want = ref.quantized_matmul(x[i * m:(i + 1) * m], packed[i * n:(i + 1) * n], scales[i * n:(i + 1) * n], None, mode=mode,
                                    group=group, bits=bits, dtype=dtype)
        assert_rows_close(got[i], want, dtype, f"direct few rows {qmode} batch item {i}", exact_weights=True)
    pairs = rng.integers(0, b, 5)
    got = to_host(nv.gather_qmm(to_dev(x.reshape(b, m, k)), q, torch.from_numpy(pairs.astype(np.int64)).cuda(),
                                torch.from_numpy(pairs[::-1].copy().astype(np.int64)).cuda(), nv.GatherQmm()))
    for z in range(5):
        i, e = int(pairs[z]), int(pairs[::-1][z])
        want = ref.quantized_matmul(x[i * m:(i + 1) * m], packed[e * n:(e + 1) * n], scales[e * n:(e + 1) * n], None, mode=mode,
                                    group=group, bits=bits, dtype=dtype)
        assert_rows_close(got[z], want, dtype, f"direct few rows {qmode} pair {z}", exact_weights=True)
