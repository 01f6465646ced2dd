"""Replays the reference's golden vectors on the MI355X through the C ABI.

Criteria as the reference applies them to its own device backend (tests/mlx.rs:55-147):
quantize and the MXFP4 codecs bit for bit; affine dequantize exact against MLX's CPU vectors
(the backend keeps the CPU's two roundings); products and gathers within FR-008's bound
against MLX's device outputs and within the CPU-fixture bound against MLX's CPU outputs.
"""
import numpy as np
import pytest

from oracle import ref
from tests import replay

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    from tests.hip_backend import HipBackend
    return HipBackend()


def _supported(c):
    """Every recorded case of the path has a kernel (gathers with the weights stored [K, N] included)."""
    return True


def _failures(cases, check):
    out = []
    for c in cases:
        msg = check(c)
        if msg:
            out.append(f"{c.name}: {msg}")
    return out


def test_affine_quantize_bits(hip, golden_cpu):
    cases = [c for c in golden_cpu[1] if c.op == "quantize"]
    assert len(cases) == 70
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, hip), c.outputs))


def test_affine_dequantize_bits(hip, golden_cpu):
    cases = [c for c in golden_cpu[1] if c.op == "dequantize"]
    assert len(cases) == 21
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, hip), c.outputs))


def test_affine_dequantize_equals_oracle_on_device_vectors(hip, golden_gpu):
    """The 54 device-recorded inputs: the backend equals the CPU oracle bit for bit."""
    cases = [c for c in golden_gpu[1] if c.name.startswith("affine-dequantize-")]
    oracle = replay.OracleBackend()

    def check(c):
        want = replay.run_case(c, oracle)
        got = replay.run_case(c, hip)
        same = np.array_equal(got[0][0].view(np.uint8), want[0][0].view(np.uint8))
        return None if same and got[0][1] == want[0][1] else "differs from the CPU oracle"

    assert len(cases) == 54
    assert not _failures(cases, check)


@pytest.mark.parametrize("mode", ["mxfp4", "mxfp8", "nvfp4"])
def test_fp_quantize_bits(hip, golden_gpu, mode):
    cases = [c for c in golden_gpu[1] if c.op == "quantize" and c.params.get("mode") == mode and c.params.get("gs") != "1"]
    assert len(cases) == 18
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, hip), c.outputs))


@pytest.mark.parametrize("mode", ["mxfp4", "mxfp8", "nvfp4"])
def test_fp_dequantize_bits(hip, golden_gpu, mode):
    cases = [c for c in golden_gpu[1] if c.op == "dequantize" and c.params.get("mode") == mode and c.params.get("gs") != "1"]
    assert len(cases) == 15
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, hip), c.outputs))


def test_nvfp4_global_scale(hip, golden_gpu):
    """NVFP4 with a global scale: quantize and dequantize bit for bit, the gathers (one scale per expert) within FR-008."""
    scaled = [c for c in golden_gpu[1] if c.params.get("gs") == "1"]
    exact = [c for c in scaled if c.op in ("quantize", "dequantize")]
    gathers = [c for c in scaled if c.op == "gather_qmm"]
    assert len(exact) == 12 and len(gathers) >= 10
    assert not _failures(exact, lambda c: replay.exact_bits(replay.run_case(c, hip), c.outputs))
    assert not _failures(gathers, lambda c: replay.within_fr008(replay.run_case(c, hip), c.outputs))


def test_qqmm_against_mlx_gpu(hip, golden_gpu):
    """`qqmm` and `gather_qqmm`: the activations through nvq_quantize_dequantize, then the quantized products."""
    cases = [c for c in golden_gpu[1] if c.op in ("qqmm", "gather_qqmm")]
    assert len(cases) == 64
    assert not _failures(cases, lambda c: replay.within_fr008(replay.run_case(c, hip), c.outputs))


def test_products_against_mlx_cpu(hip, golden_cpu):
    cases = [c for c in golden_cpu[1] if c.op == "quantized_matmul" and _supported(c)]
    assert len(cases) >= 20
    assert not _failures(cases, lambda c: replay.by_value(replay.run_case(c, hip), c.outputs, replay.product_bound(c)))


def test_products_against_mlx_gpu(hip, golden_gpu):
    cases = [c for c in golden_gpu[1] if c.op == "quantized_matmul" and _supported(c)]
    assert len(cases) >= 40
    assert not _failures(cases, lambda c: replay.within_fr008(replay.run_case(c, hip), c.outputs))


def test_gathers_against_mlx_gpu(hip, golden_gpu):
    cases = [c for c in golden_gpu[1] if c.op == "gather_qmm" and _supported(c)]
    assert len(cases) >= 12
    assert not _failures(cases, lambda c: replay.within_fr008(replay.run_case(c, hip), c.outputs))
