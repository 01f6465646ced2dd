"""Pins the CPU oracle against every golden vector the reference's tests hold for the path.

These run without a GPU.  Criteria are the reference's own (tests/mlx.rs:55-147,
tests/common/fixture.rs:1297-1316,1331-1394).
"""
import numpy as np
import pytest

from oracle import ref
from tests import replay

ORACLE = replay.OracleBackend()


def _failures(cases, check):
    out = []
    for c in cases:
        msg = check(c)
        if msg:
            out.append(f"{c.name}: {msg}")
    return out


def test_fixture_meta(golden_cpu, golden_gpu):
    meta, cases = golden_cpu
    assert "mlx=0.32.4" in meta and "device=cpu" in meta
    assert len(cases) == 135
    meta, cases = golden_gpu
    assert "mlx=0.32.4" in meta and "device=gpu" in meta
    assert len(cases) == 367


def test_affine_quantize_bits(golden_cpu):
    """70 cases: packed words, scales and biases equal to MLX's CPU."""
    cases = [c for c in golden_cpu[1] if c.op == "quantize"]
    assert len(cases) == 70
    # The reference compares by value (a zero bias of either sign passes); bits are checked too.
    assert not _failures(cases, lambda c: replay.by_value(replay.run_case(c, ORACLE), c.outputs))
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, ORACLE), c.outputs))


def test_affine_dequantize_cpu_semantics(golden_cpu):
    """21 cases: two roundings in the scales' dtype, exact."""
    cases = [c for c in golden_cpu[1] if c.op == "dequantize"]
    assert len(cases) == 21
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, ORACLE), c.outputs))


def test_affine_dequantize_device_vectors(golden_gpu):
    """54 device-recorded cases: the one-rounding variant equals them bit for bit (pins the code
    extraction for every bit width and group size); the CPU semantics stay within the
    reference's bound 2 eps (max|s| (2^bits - 1) + max|b|) (fixture.rs:1297-1307)."""
    cases = [c for c in golden_gpu[1] if c.name.startswith("affine-dequantize-")]
    assert len(cases) == 54

    def fma(c):
        xs = [t.array() for t in c.inputs]
        _, group, bits = replay.quant_of(c)
        dt = replay.DT[c.inputs[1].dtype]
        out = ref.affine_dequantize(xs[0], xs[1], xs[2], dt, group, bits, fma=True)
        return replay.exact_bits([(out, c.inputs[1].dtype)], c.outputs)

    def cpu(c):
        bits = int(c.params["bits"])
        m = lambda t: float(np.max(np.abs(replay.as_f64(t.array(), t.dtype))))
        tol = 2.0 * replay.EPS[replay.DT[c.outputs[0].dtype]] * (m(c.inputs[1]) * ((1 << bits) - 1) + m(c.inputs[2]))
        return replay.by_value(replay.run_case(c, ORACLE), c.outputs, tol)

    assert not _failures(cases, fma)
    assert not _failures(cases, cpu)


@pytest.mark.parametrize("mode", ["mxfp4", "mxfp8", "nvfp4"])
def test_fp_quantize_bits(golden_gpu, mode):
    """18 cases per format incl. NaN/Inf/subnormal/signed-zero edges, transposed and reversed inputs."""
    cases = [c for c in golden_gpu[1] if c.op == "quantize" and c.params.get("mode") == mode and c.params.get("gs") != "1"]
    assert len(cases) == 18
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, ORACLE), c.outputs))


@pytest.mark.parametrize("mode", ["mxfp4", "mxfp8", "nvfp4"])
def test_fp_dequantize_bits(golden_gpu, mode):
    cases = [c for c in golden_gpu[1] if c.op == "dequantize" and c.params.get("mode") == mode and c.params.get("gs") != "1"]
    assert len(cases) == 15
    assert not _failures(cases, lambda c: replay.exact_bits(replay.run_case(c, ORACLE), c.outputs))


def test_nvfp4_global_scale(golden_gpu):
    """NVFP4 with a global scale (kernels.rs:914-1009 with `g`): 6 quantize and 6 dequantize cases bit for bit, the
    gathers with one scale per expert within FR-008."""
    scaled = [c for c in golden_gpu[1] if c.params.get("gs") == "1"]
    exact = [c for c in scaled if c.op in ("quantize", "dequantize")]
    gathers = [c for c in scaled if c.op == "gather_qmm"]
    assert len(exact) == 12 and len(gathers) >= 10
    assert not _failures(exact, lambda c: replay.exact_bits(replay.run_case(c, ORACLE), c.outputs))
    assert not _failures(gathers, lambda c: replay.within_fr008(replay.run_case(c, ORACLE), c.outputs))


def test_qqmm_against_mlx_gpu(golden_gpu):
    """`qqmm` and `gather_qqmm` (activations through their quantization, products.rs:307-470) in the three
    floating-point modes, dense and quantized weights, with and without NVFP4 global scales: FR-008's bound."""
    cases = [c for c in golden_gpu[1] if c.op in ("qqmm", "gather_qqmm")]
    assert len(cases) == 64
    assert not _failures(cases, lambda c: replay.within_fr008(replay.run_case(c, ORACLE), c.outputs))


def test_products_against_mlx_cpu(golden_cpu):
    """44 cases, every bit width, both orientations, batched and shared weights: within the
    reference's bound against MLX's CPU (fixture.rs:1309-1316)."""
    cases = [c for c in golden_cpu[1] if c.op == "quantized_matmul"]
    assert len(cases) == 44
    assert not _failures(cases, lambda c: replay.by_value(replay.run_case(c, ORACLE), c.outputs,
                                                          replay.product_bound(c)))


def test_products_against_mlx_gpu(golden_gpu):
    """Affine and MXFP4 products recorded on the device: FR-008's bound (mlx.rs:125-147)."""
    cases = [c for c in golden_gpu[1] if c.op == "quantized_matmul"]
    assert len(cases) >= 60
    assert not _failures(cases, lambda c: replay.within_fr008(replay.run_case(c, ORACLE), c.outputs))


def test_gathers_against_mlx_gpu(golden_gpu):
    cases = [c for c in golden_gpu[1] if c.op == "gather_qmm"]
    assert len(cases) >= 18
    assert not _failures(cases, lambda c: replay.within_fr008(replay.run_case(c, ORACLE), c.outputs))
