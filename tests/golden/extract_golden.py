"""Extracts the committed golden subset from the reference's recorded-MLX fixture files.

Reads (as bytes, nothing is imported or executed) the two data files the reference's own
tests replay — crates/nuvec-core/tests/fixtures/mlx.bin (MLX 0.32.4 on the CPU) and
mlx_gpu.bin (MLX 0.32.4 on the GPU) — keeps the cases of the quantized-matmul path
(affine, MXFP4, MXFP8 and NVFP4, the latter also with its global scale) and re-serialises them unchanged in the same
BSMXFIX1 container:

    golden_cpu.bin   every affine quantize / dequantize / quantized_matmul case of mlx.bin
    golden_gpu.bin   every MXFP4 / MXFP8 / NVFP4 quantize / dequantize case and every
                     affine-dequantize case of mlx_gpu.bin, plus a curated set of product and gather
                     cases (float32 and bfloat16, one case per kernel route; the smaller ones for
                     MXFP8 and NVFP4)

Run once, in a checkout that has the reference beside it:
    python tests/golden/extract_golden.py [/root/reference]
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "..", ".."))
from oracle import bsmxfix  # noqa: E402

PATH_OPS = ("quantize", "dequantize", "quantized_matmul", "gather_qmm", "qqmm", "gather_qqmm")


def in_scope(case) -> bool:
    mode = case.params.get("mode", "affine")
    return case.op in PATH_OPS and mode in ("affine", "mxfp4", "mxfp8", "nvfp4")


def keep_gpu(case) -> bool:
    if not in_scope(case):
        return False
    if case.op in ("quantize", "dequantize"):
        return True
    # Products and gathers: float32 and bfloat16 only ("bfloat16" contains "float16"), sized
    # to keep the file near 3 MiB; the MoE-shaped grouped gather (K = 2880) is kept whole.
    if "-float16" in case.name:
        return False
    if case.params.get("gs") == "1":  # gathers with one global scale per expert: the transposed ones that reach a kernel
        return case.params.get("transpose", "1") == "1" and case.nbytes() <= 160_000
    if case.params.get("mode", "affine") in ("mxfp8", "nvfp4"):
        return case.nbytes() <= 40_000
    if case.name.endswith("oss-grouped"):
        return True
    return case.nbytes() <= (160_000 if "float32" in case.name else 100_000)


def main(reference="/root/reference"):
    fixtures = os.path.join(reference, "crates/nuvec-core/tests/fixtures")
    meta, cases = bsmxfix.load(os.path.join(fixtures, "mlx.bin"))
    cpu = [c for c in cases if in_scope(c)]
    bsmxfix.dump(os.path.join(HERE, "golden_cpu.bin"), meta + " subset=quantized-path", cpu)
    meta, cases = bsmxfix.load(os.path.join(fixtures, "mlx_gpu.bin"))
    gpu = [c for c in cases if keep_gpu(c)]
    bsmxfix.dump(os.path.join(HERE, "golden_gpu.bin"), meta + " subset=quantized-path", gpu)
    for name, kept in (("golden_cpu.bin", cpu), ("golden_gpu.bin", gpu)):
        size = os.path.getsize(os.path.join(HERE, name))
        print(f"{name}: {len(kept)} cases, {size / 1024:.0f} KiB")


if __name__ == "__main__":
    main(*sys.argv[1:])
