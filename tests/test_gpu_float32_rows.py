"""float32 products of many rows on the float32 matrix instruction (`qmm_f32_kernel`): the reference instantiates its
tiled kernels for float at every affine width (crates/nuvec-kernels/src/metal/quantized.metal:40-70); the CPU product
(crates/nuvec-core/src/kernels.rs:1091-1142) dequantizes in float32 with two roundings and accumulates in float32.  The
bar is the float32 one, 1e-4 of a row's largest output."""
import numpy as np
import pytest
import torch

import nuvec_amd as nv
from nuvec_amd import ops
from oracle import ref
from tests.hip_backend import to_dev, to_host
from tests.test_gpu_parity import assert_rows_close, make_w, make_x

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bits,group", [(4, 64), (4, 32), (8, 32), (8, 128), (3, 64), (6, 64), (5, 32), (2, 128), (1, 128)])
def test_every_width_against_the_cpu_product(bits, group):
    """Whole tiles and tails of rows and of weight rows, one step of K and many."""
    rng = np.random.default_rng(5200 + 10 * bits + group)
    quant = nv.Quant.affine(group, bits)
    for m, n, k in ((300, 1000, 1024), (64, 4096, 512), (129, 2055, 128), (2048, 320, 256)):
        assert ops.quantized_matmul_route(m, n, k, quant, torch.float32) == "qmm_f32_kernel", (m, n, k)
        w, x = make_w(rng, n, k, ref.F32), make_x(rng, m, k, ref.F32)
        packed, scales, biases = ref.affine_quantize(w, ref.F32, group, bits)
        q = nv.Quantized(to_dev(packed), to_dev(scales), to_dev(biases), quant)
        want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=ref.F32, threads=8)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, ref.F32, f"float32 rows b{bits} g{group} M={m} N={n} K={k}")


@pytest.mark.parametrize("mode,qmode", [(ref.MXFP4, "MXFP4"), (ref.MXFP8, "MXFP8"), (ref.NVFP4, "NVFP4")])
def test_block_formats_against_the_cpu_product(mode, qmode):
    """The block formats (the reference instantiates them for float32 as well, crates/nuvec-kernels/src/metal/fp_quantized.metal:105-107):
    decoded code times decoded scale in float32; NVFP4 also with a global scale (kernels.rs:992-998)."""
    rng = np.random.default_rng(5400 + mode)
    group, bits = ref.FP_PARAMS[mode]
    quant = nv.Quant.new(getattr(nv.QuantMode, qmode))
    for m, n, k in ((300, 1000, 1024), (70, 4100, 512), (2048, 320, 256)):
        assert ops.quantized_matmul_route(m, n, k, quant, torch.float32) == "qmm_f32_kernel", (m, n, k)
        w, x = make_w(rng, n, k, ref.F32), make_x(rng, m, k, ref.F32)
        packed, scales = ref.fp_quantize(w, ref.F32, mode)
        q = nv.Quantized(to_dev(packed), to_dev(scales), None, quant)
        want = ref.quantized_matmul(x, packed, scales, None, mode=mode, group=group, bits=bits, dtype=ref.F32, threads=8)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, ref.F32, f"float32 rows {qmode} M={m} N={n} K={k}", exact_weights=True)
    if mode == ref.NVFP4:
        m, n, k, g = 300, 1000, 1024, 3.25
        w, x = make_w(rng, n, k, ref.F32), make_x(rng, m, k, ref.F32)
        gs = torch.tensor(g, dtype=torch.float32, device="cuda")
        q = nv.quantize(to_dev(w), nv.QuantMode.NVFP4, gs)
        packed, scales = ref.fp_quantize(w, ref.F32, ref.NVFP4, g)
        assert np.array_equal(to_host(q.weight), packed) and np.array_equal(to_host(q.scales), scales)
        want = ref.fp_quantized_matmul_scaled(x, packed, scales, ref.NVFP4, ref.F32, g)
        got = to_host(nv.quantized_matmul(to_dev(x), q))
        assert_rows_close(got, want, ref.F32, "float32 rows NVFP4 with a global scale", exact_weights=True)


def test_routes_and_what_stays_on_the_vector_kernel():
    """The rule is an estimate of both kernels: few rows, row-exact products, K off whole steps of 64 and batches stay
    where they were."""
    q4 = nv.Quant.affine(64, 4)
    route = lambda m, n, k, **kw: ops.quantized_matmul_route(m, n, k, q4, torch.float32, **kw)
    assert route(1, 4096, 4096) == "qmv_lds_kernel" and route(8, 4096, 4096) == "qmv_lds_kernel" and route(32, 4096, 4096) == "qmv_lds_kernel"
    assert route(64, 4096, 4096) == "qmm_f32_kernel" and route(512, 4096, 4096) == "qmm_f32_kernel"
    assert route(32, 14336, 4096) == "qmm_f32_kernel" and route(8, 14336, 4096) == "qmv_lds_kernel"
    assert route(512, 4096, 4096, rows=True) == "qmv_lds_kernel"
    assert ops.quantized_matmul_route(512, 4096, 4096 + 32, nv.Quant.affine(32, 4), torch.float32) == "qmv_lds_kernel"
    assert route(512, 4096, 4096, batch=2) == "qmv_lds_kernel"
    assert ops.quantized_matmul_route(512, 4096, 4096, nv.Quant.new(nv.QuantMode.MXFP4), torch.float32) == "qmm_f32_kernel"
    assert ops.quantized_matmul_route(4, 4096, 4096, nv.Quant.new(nv.QuantMode.MXFP4), torch.float32) == "qmv_lds_kernel"


def test_bias_epilogue_determinism_and_the_vector_kernel():
    """QuantizedLinear's bias in the epilogue is the separate addition bit for bit (crates/nuvec-nn/src/layers.rs:155-162);
    two launches give the same bits; and the rows agree with the vector kernel's (the row-exact product of the same
    operands) within the float32 bar."""
    rng = np.random.default_rng(5300)
    m, n, k = 200, 1536, 1024
    w, x = make_w(rng, n, k, ref.F32), make_x(rng, m, k, ref.F32)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, 4))
    xd = to_dev(x)
    plain = nv.quantized_matmul(xd, q)
    assert torch.equal(plain, nv.quantized_matmul(xd, q))
    bias = torch.randn(n, device="cuda")
    from nuvec_amd.layers import QuantizedLinear
    layer = QuantizedLinear(q.weight, q.scales, q.biases, bias, q.quant)
    assert torch.equal(layer(xd), plain + bias)
    by_rows = nv.quantized_matmul(xd, q, rows=True)
    assert_rows_close(to_host(plain), to_host(by_rows), ref.F32, "float32 rows against the vector kernel")
