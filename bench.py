#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

A "step" is one decode-shaped product of BASELINE.json's configs[1]: affine 4-bit g64,
x bf16 [1,4096], W [14336,4096] (packed uint32 + bf16 scales and biases), y bf16 [1,14336].
`value` is the weight stream rate in GB/s: the algorithmic bytes of one product
(packed 29,360,128 + scales 1,835,008 + biases 1,835,008 = 33,030,144 B) over the average
time of one launch, with every operand resident in HBM.  Launches go back to back on one
stream through the C ABI and rotate through enough distinct weight copies that no launch finds
its weights in the 256 MB last-level cache.  The prefill-shaped product (configs[2], M = 2048)
is timed the same way and reported in the same line as `qmm`.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-qmm] [--no-configs] [--no-peaks]

Prints one JSON line.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E, vendor figure
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, vendor figure
MFMA_F32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 MFMA, vendor figure
N, K = 14336, 4096
GROUP, BITS = 64, 4
WEIGHT_BYTES = N * K * BITS // 8 + 2 * (N * (K // GROUP) * 2)  # 33,030,144
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/), scaled by
# what the same counters read for a plain device copy of known size; None until measured.
QMV_TRAFFIC_BYTES = 33_235_175
QMM_TRAFFIC_BYTES = 297_181_328
METRIC = "QMV weight GB/s (% HBM peak) at M=1; QMM TFLOP/s (% MFMA peak) at M=2048"


def make_weights(copies, device):
    import torch

    import nuvec_amd as nv
    out = []
    gen = torch.Generator(device=device)
    for i in range(copies):
        gen.manual_seed(1234 + i)
        w = (torch.randn(N, K, device=device, generator=gen) * 0.02).to(torch.bfloat16)
        out.append(nv.quantize(w, nv.Quant.affine(GROUP, BITS)))
        del w
    torch.cuda.synchronize()
    return out


class Product:
    """One prepared nvq_quantized_matmul call: descriptor and pointers built once, so the timed
    loop is a bare C-ABI call per launch."""

    def __init__(self, lib, m, x, q, y, n=N, k=K, dtype=None, transpose=True):
        from nuvec_amd import _lib
        d = _lib.QmmDescC()
        d.quant = q.quant._c()
        d.dtype = _lib.BF16 if dtype is None else dtype
        d.transpose, d.m, d.n, d.k, d.item_rows, d.batch_ndim = int(transpose), m, n, k, m, 0
        self.d, self.fn = d, lib.nvq_quantized_matmul
        biases = q.biases.data_ptr() if q.biases is not None else None
        import torch
        need = lib.nvq_quantized_matmul_workspace_bytes(C.byref(d))  # the caller's scratch, as the boundary defines it
        workspace = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
        self.args = (C.byref(d), C.c_void_p(x.data_ptr()), C.c_void_p(q.weight.data_ptr()),
                     C.c_void_p(q.scales.data_ptr()), C.c_void_p(biases), C.c_void_p(y.data_ptr()),
                     C.c_void_p(workspace.data_ptr() if need else None))
        self.keep = (x, q, y, workspace)

    def __call__(self, stream):
        rc = self.fn(*self.args, stream)
        if rc:
            from nuvec_amd import _lib
            _lib.check(rc)


class GatherProduct:
    """One prepared nvq_gather_qmm call with one row of x per pair: sorted pairs with their offsets (the grouped route) or
    unsorted ones."""

    def __init__(self, lib, x, q, lhs, rhs, offsets, y, n, k, experts):
        """`offsets` None: unsorted pairs, one product per pair."""
        from nuvec_amd import _lib
        pairs = rhs.numel()
        self.d = _lib.GatherDescC(q.quant._c(), _lib.BF16, 1, 0, 0, 1, n, k, pairs, x.shape[0], experts)
        self.fn = lib.nvq_gather_qmm
        biases = q.biases.data_ptr() if q.biases is not None else None
        self.args = (C.byref(self.d), C.c_void_p(x.data_ptr()), C.c_void_p(q.weight.data_ptr()),
                     C.c_void_p(q.scales.data_ptr()), C.c_void_p(biases), C.c_void_p(lhs.data_ptr()),
                     C.c_void_p(rhs.data_ptr()), C.c_void_p(None if offsets is None else offsets.data_ptr()), C.c_void_p(y.data_ptr()),
                     C.c_void_p(None))
        self.keep = (x, q, lhs, rhs, offsets, y)

    def __call__(self, stream):
        rc = self.fn(*self.args, stream)
        if rc:
            from nuvec_amd import _lib
            _lib.check(rc)


def time_launches(calls, steps, warmup, graph=True):
    """Average milliseconds per launch over `steps` launches, after `warmup` untimed ones, between
    two HIP events recorded on the stream the kernels run on.  `calls` are rotated.

    graph=True: one rotation of the calls is captured into a HIP graph (the same C-ABI calls, made
    once on the capturing stream) and the graph is replayed, so the launches reach the GPU back
    to back without a Python call between them; `steps` is rounded to whole rotations.
    graph=False: one C-ABI call per launch from the Python loop (host-bound for kernels this short)."""
    import torch
    n = len(calls)
    stream = torch.cuda.current_stream()
    for i in range(warmup):
        calls[i % n](C.c_void_p(stream.cuda_stream))
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if not graph:
        start.record()
        for i in range(steps):
            calls[i % n](C.c_void_p(stream.cuda_stream))
        stop.record()
        torch.cuda.synchronize()
        return start.elapsed_time(stop) / steps, steps
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        cap = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        for c in calls:
            c(cap)
    reps = max(1, round(steps / n))
    g.replay()
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        g.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / (reps * n), reps * n


def cpu_baseline(seconds_budget=24.0):
    """The CPU restatement of nuvec's path (dequantize the whole matrix on one thread as the reference does, then the
    product) on this host's cores, on a bounded sample of the same workload: the decode product of configs[1] on one
    thread and on all cores, and rows of the prefill product of configs[2] (the path for more than 16 rows)."""
    import numpy as np

    from oracle import ref
    rng = np.random.default_rng(0)
    w = ref.from_f32((rng.standard_normal((N, K)) * 0.02).astype(np.float32), ref.BF16)
    x = ref.from_f32(rng.standard_normal((1, K)).astype(np.float32), ref.BF16)
    packed, scales, biases = ref.affine_quantize(w, ref.BF16, GROUP, BITS)
    cores = max(1, min(ref.max_threads(), int(os.environ.get("OMP_NUM_THREADS", "0") or os.cpu_count() or 1)))

    def timed(run, budget, least=2, most=40):
        run()
        done, t0 = 0, time.perf_counter()
        while done < least or (time.perf_counter() - t0 < budget and done < most):
            run()
            done += 1
        return (time.perf_counter() - t0) / done, done

    legs = {}
    for name, threads in (("single_thread", 1), ("all_cores", cores)):
        dt, done = timed(lambda: ref.quantized_matmul(x, packed, scales, biases, group=GROUP, bits=BITS, dtype=ref.BF16, threads=threads),
                         seconds_budget / 4)
        legs[name] = {"value": WEIGHT_BYTES / dt / 1e9, "unit": "GB/s", "cores": threads, "ms_per_step": dt * 1e3, "products": done}
    rows = 64  # of the 2048 of configs[2]: more than 16 rows, so the many-row product (float32 products summed in order)
    xm = ref.from_f32(rng.standard_normal((rows, K)).astype(np.float32), ref.BF16)
    dt, done = timed(lambda: ref.quantized_matmul(xm, packed, scales, biases, group=GROUP, bits=BITS, dtype=ref.BF16, threads=cores),
                     seconds_budget / 4, least=1, most=10)
    legs["prefill_all_cores"] = {"value": 2.0 * rows * N * K / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "ms_per_step": dt * 1e3,
                                 "products": done, "sample": f"{rows} of the 2048 rows of configs[2] per product (dequantize included)"}
    return {"value": legs["all_cores"]["value"], "unit": "GB/s", "cores": cores, "kind": "port",
            "ms_per_step": legs["all_cores"]["ms_per_step"],
            "sample": f"{legs['all_cores']['products']} products of the same workload (x bf16 [1,{K}], W [{N},{K}] affine 4-bit g64): "
                      f"whole-matrix dequantize on one thread as the reference does, then the 8-lane fixed-order product over "
                      f"64-column blocks on {cores} threads; `single_thread` is the same on one thread, `prefill_all_cores` "
                      f"{rows} rows of configs[2]",
            **legs}


def measured_peaks(lib, device, qs):
    """What this box gives the simplest kernels, measured in this run with the same event timing: the ceilings the
    roofline fractions can be read against besides the published peaks."""
    import torch

    from nuvec_amd import _lib
    work = C.c_int64(0)
    out = {}

    def best_of(calls, steps):
        return min(time_launches(calls, steps, len(calls), graph=False)[0] for _ in range(3))

    # the decode kernel's grid reading the 29.4 MB of packed codes and nothing else, weights rotated like the headline
    code_bytes = N * K * BITS // 8
    reads = [(lambda stream, q=q: _lib.check(lib.nvq_calibrate(0, C.c_void_p(q.weight.data_ptr()), code_bytes, 0, None, C.byref(work), stream)))
             for q in qs]
    ms = best_of(reads, 2000)
    out["read_codes_decode_grid"] = {"us_per_launch": ms * 1e3, "gbps": code_bytes / (ms * 1e-3) / 1e9, "bytes": code_bytes,
                                     "note": "plain read of one product's packed codes (no scales, no arithmetic), rotating buffers"}
    big = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    ms = best_of([lambda stream: _lib.check(lib.nvq_calibrate(0, C.c_void_p(big.data_ptr()), 1 << 30, 0, None, C.byref(work), stream))], 30)
    out["stream_read_1gib"] = {"us_per_launch": ms * 1e3, "gbps": (1 << 30) / (ms * 1e-3) / 1e9}
    del big
    empty = torch.empty(16384, dtype=torch.uint8, device=device)
    ms = best_of([lambda stream: _lib.check(lib.nvq_calibrate(0, C.c_void_p(empty.data_ptr()), 16384, 0, None, C.byref(work), stream))], 2000)
    out["one_block_launch"] = {"us_per_launch": ms * 1e3, "note": "a launch of one block: the floor of any back-to-back kernel here"}
    iters = 4096
    ms = best_of([lambda stream: _lib.check(lib.nvq_calibrate(1, None, 0, iters, None, C.byref(work), stream))], 10)
    out["mfma_only_loop"] = {"us_per_launch": ms * 1e3, "tflops": work.value / (ms * 1e-3) / 1e12,
                             "note": "v_mfma_f32_32x32x16_bf16 on constant operands, two wavefronts per SIMD"}
    a = torch.randn(2048, K, device=device).to(torch.bfloat16)
    b = torch.randn(N, K, device=device).to(torch.bfloat16)
    c = torch.empty(2048, N, dtype=torch.bfloat16, device=device)
    ms = best_of([lambda stream: torch.matmul(a, b.t(), out=c)], 20)
    out["vendor_dense_gemm"] = {"us_per_launch": ms * 1e3, "tflops": 2.0 * 2048 * N * K / (ms * 1e-3) / 1e12,
                                "note": "torch.matmul bf16 [2048,4096] x [4096,14336] (hipBLASLt, nothing to dequantize): baseline only"}
    # The same two launches on operands that are all zero: the same instruction streams with no bit toggling in the
    # operand paths.  What they gain over random data is what the chip's power management takes from a kernel at this
    # occupancy of the matrix cores, whatever its schedule.
    a.zero_(), b.zero_()
    ms = best_of([lambda stream: torch.matmul(a, b.t(), out=c)], 20)
    out["vendor_dense_gemm_zero_operands"] = {"us_per_launch": ms * 1e3, "tflops": 2.0 * 2048 * N * K / (ms * 1e-3) / 1e12}
    import nuvec_amd as nv
    zq = nv.Quantized(torch.zeros_like(qs[0].weight), torch.zeros_like(qs[0].scales), torch.zeros_like(qs[0].biases), qs[0].quant)
    ms = best_of([Product(lib, 2048, a, zq, c)], 20)
    out["prefill_zero_operands"] = {"us_per_launch": ms * 1e3, "tflops": 2.0 * 2048 * N * K / (ms * 1e-3) / 1e12,
                                    "note": "configs[2]'s own kernel on all-zero x, codes, scales and biases"}
    return out


def all_configs(lib, device, qs):
    """Every BASELINE configuration, each timed like the headline: rotating weight copies beyond the
    last-level cache, one C-ABI call per launch, best of three event-timed runs.  `qs` are the C2 weights."""
    import numpy as np
    import torch

    import nuvec_amd as nv
    from nuvec_amd import _lib
    out = []

    def best_of(calls, steps):
        return min(time_launches(calls, steps, len(calls), graph=False)[0] for _ in range(3))

    def products(label, n, k, quant, tdtype, code, ms_list, copies, wbytes, weights=None, transpose=True, matrix_peak=MFMA_BF16_PEAK_TFLOPS):
        if weights is None:
            gen = torch.Generator(device=device)
            weights = []
            for i in range(copies):
                gen.manual_seed(4321 + i)
                shape = (n, k) if transpose else (k, n)  # (stored [K, N]: quantized along N)
                weights.append(nv.quantize((torch.randn(shape, device=device, generator=gen) * 0.02).to(tdtype), quant))
        for m in ms_list:
            x = torch.randn(m, k, device=device).to(tdtype)
            ys = [torch.empty(m, n, dtype=tdtype, device=device) for _ in weights]
            calls = [Product(lib, m, x, q, y, n, k, code, transpose) for q, y in zip(weights, ys)]
            ms = best_of(calls, 600 if m <= 64 else 48)
            kernel = lib.nvq_quantized_matmul_route(C.byref(calls[0].d))  # from the library's routing code
            gbps, tflops = wbytes / (ms * 1e-3) / 1e9, 2.0 * m * n * k / (ms * 1e-3) / 1e12
            out.append({"config": label, "m": m, "kernel": kernel.decode() if kernel else None, "us_per_launch": ms * 1e3,
                        "weight_gbps": gbps, "tflops": tflops,
                        # the roof that bounds the row: weight bytes over HBM for few rows, the bf16 matrix peak for many
                        "frac_of_peak": gbps / HBM_PEAK_GBPS if m <= 64 else tflops / matrix_peak,
                        "bound": "hbm" if m <= 64 else "mfma"})

    # (C1 is one row; 512 rows beside it: float32 on the matrix cores, against the 157.3 TFLOP/s of the float32 matrix instruction)
    products("C1 f32 4-bit g64 W[4096,4096]", 4096, 4096, nv.Quant.affine(64, 4), torch.float32, _lib.F32, [1, 512], 48, 10_485_760,
             matrix_peak=MFMA_F32_PEAK_TFLOPS)
    products("C2/C3 bf16 4-bit g64 W[14336,4096]", N, K, None, torch.bfloat16, _lib.BF16, [1, 4, 8, 32, 64, 2048], 0, WEIGHT_BYTES,
             weights=qs)
    # Beside C2: the same layer's down projection, whose rows are K = 14336 long
    products("beside C2: bf16 4-bit g64 W[4096,14336]", 4096, 14336, nv.Quant.affine(64, 4), torch.bfloat16, _lib.BF16, [1], 24, WEIGHT_BYTES)
    # ... and C2's shape in 8-bit codes at the rows of batched decode
    products("beside C2: bf16 8-bit g64 W[14336,4096]", N, K, nv.Quant.affine(64, 8), torch.bfloat16, _lib.BF16, [16, 64], 12,
             N * K + 2 * (N * (K // 64) * 2))
    products("C4 bf16 3-bit g64 W[4096,4096]", 4096, 4096, nv.Quant.affine(64, 3), torch.bfloat16, _lib.BF16, [1, 16, 512], 48,
             7_340_032)
    products("C4 bf16 8-bit g32 W[4096,4096]", 4096, 4096, nv.Quant.affine(32, 8), torch.bfloat16, _lib.BF16, [1, 16, 512], 32,
             18_874_368)
    # Beside the BASELINE configurations: 6-bit codes, the width mixed-precision checkpoints give their sensitive layers
    products("beside C4: bf16 6-bit g64 W[4096,4096]", 4096, 4096, nv.Quant.affine(64, 6), torch.bfloat16, _lib.BF16, [1, 4, 16], 32,
             13_631_488)
    # ... and C2's product with the weights stored [K, N] (transpose = false)
    products("bf16 4-bit g64 w[4096,14336] stored [K, N]", N, K, nv.Quant.affine(64, 4), torch.bfloat16, _lib.BF16, [1, 16, 2048], 24,
             WEIGHT_BYTES, transpose=False)
    # ... and with 6-bit codes (a run of eight columns is six bytes): the widths other than 2, 4 and 8 bits on the same kernel
    products("bf16 6-bit g64 w[4096,14336] stored [K, N]", N, K, nv.Quant.affine(64, 6), torch.bfloat16, _lib.BF16, [16, 512], 12,
             K * N * 6 // 8 + 2 * (K * (N // 64) * 2), transpose=False)
    # C5: 32 MXFP4 experts [2880,2880], 256 tokens x 4 distinct experts, pairs sorted by expert
    experts, n, k, tokens, top = 32, 2880, 2880, 256, 4
    weights = [nv.quantize((torch.randn(experts, n, k, device=device) * 0.02).to(torch.bfloat16), nv.QuantMode.MXFP4)
               for _ in range(4)]
    rng = np.random.default_rng(0)
    choice = np.stack([rng.permutation(experts)[:top] for _ in range(tokens)]).reshape(-1)
    rhs = torch.from_numpy(np.sort(choice).astype(np.int32)).to(device)
    lhs = torch.arange(tokens * top, dtype=torch.int32, device=device)
    x = torch.randn(tokens * top, 1, k, device=device).to(torch.bfloat16)
    y = torch.empty(tokens * top, 1, n, dtype=torch.bfloat16, device=device)
    offsets = nv.sorted_offsets(rhs, experts)
    calls = [GatherProduct(lib, x, q, lhs, rhs, offsets, y, n, k, experts) for q in weights]
    ms = best_of(calls, 200)
    out.append({"config": "C5 MXFP4 gather_qmm 32 experts W[2880,2880], 1024 sorted rows", "m": tokens * top, "kernel": "qmg_kernel",
                "us_per_launch": ms * 1e3, "weight_gbps": 141_004_800 / (ms * 1e-3) / 1e9,
                "tflops": 16_986_931_200 / (ms * 1e-3) / 1e12, "frac_of_peak": 141_004_800 / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                "bound": "hbm"})
    # Beside the configurations: the same experts at decode, one token's four experts as unsorted pairs (one product
    # per pair on the decode kernel), and 32 such pairs
    for pairs in (top, 32):
        ids = torch.from_numpy(rng.permutation(experts)[:pairs].astype(np.int32)).to(device)
        calls = [GatherProduct(lib, x[:pairs], q, lhs[:pairs], ids, None, y[:pairs], n, k, experts) for q in weights]
        ms = best_of(calls * 4, 320)
        moved = pairs * (n * k // 2 + n * k // 32)
        out.append({"config": f"C5's experts at decode: {pairs} unsorted rows, one expert each", "m": pairs, "kernel": "qmv4_lds_kernel",
                    "us_per_launch": ms * 1e3, "weight_gbps": moved / (ms * 1e-3) / 1e9, "tflops": 2.0 * pairs * n * k / (ms * 1e-3) / 1e12,
                    "frac_of_peak": moved / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "bound": "hbm"})
    del weights, calls

    # The weights' own kernels at the same shapes: quantize (dense in, packed out) and dequantize (packed in, dense out),
    # inputs rotated beyond the last-level cache, outputs preallocated; GB/s counts every byte read and written.
    def quantizers(label, shape, tdtype, code, quant, copies):
        dense = [(torch.randn(shape, device=device) * 0.02).to(tdtype) for _ in range(copies)]
        q = nv.quantize(dense[0], quant)
        rows, cols = dense[0].numel() // shape[-1], shape[-1]
        qc = q.quant._c()
        ptr = lambda t: C.c_void_p(None if t is None else t.data_ptr())
        packed_bytes = q.weight.numel() * 4 + q.scales.numel() * q.scales.element_size() * (2 if q.biases is not None else 1)
        dense_bytes = dense[0].numel() * dense[0].element_size()

        def quantize_call(w):
            return lambda stream: _lib.check(lib.nvq_quantize(C.byref(qc), code, ptr(w), rows, cols, ptr(q.weight), ptr(q.scales),
                                                              ptr(q.biases), stream))
        ms = best_of([quantize_call(w) for w in dense], 60)
        out.append({"config": f"quantize {label}", "m": 0, "us_per_launch": ms * 1e3,
                    "weight_gbps": (dense_bytes + packed_bytes) / (ms * 1e-3) / 1e9, "tflops": 0.0,
                    "frac_of_peak": (dense_bytes + packed_bytes) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "bound": "hbm"})
        qs_ = [nv.quantize(w, quant) for w in dense]

        def dequantize_call(qq, o):
            return lambda stream: _lib.check(lib.nvq_dequantize(C.byref(qc), code, ptr(qq.weight), ptr(qq.scales), ptr(qq.biases), rows,
                                                                cols, ptr(o), stream))
        ms = best_of([dequantize_call(qq, w) for qq, w in zip(qs_, dense)], 60)
        out.append({"config": f"dequantize {label}", "m": 0, "us_per_launch": ms * 1e3,
                    "weight_gbps": (dense_bytes + packed_bytes) / (ms * 1e-3) / 1e9, "tflops": 0.0,
                    "frac_of_peak": (dense_bytes + packed_bytes) / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "bound": "hbm"})

    quantizers("C2 W[14336,4096] bf16 <-> 4-bit g64", (N, K), torch.bfloat16, _lib.BF16, nv.Quant.affine(GROUP, BITS), 4)
    quantizers("C1 W[4096,4096] f32 <-> 4-bit g64", (4096, 4096), torch.float32, _lib.F32, nv.Quant.affine(64, 4), 8)
    quantizers("C5 W[32,2880,2880] bf16 <-> MXFP4", (32, 2880, 2880), torch.bfloat16, _lib.BF16, nv.Quant.new(nv.QuantMode.MXFP4), 2)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=4000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--copies", type=int, default=24, help="distinct weight copies rotated through (24 x 33 MB = 793 MB)")
    ap.add_argument("--qmm-steps", type=int, default=40)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-qmm", action="store_true", help="skip the M=2048 leg")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip timing every configuration of the reference's benchmark list (C1..C5), reported under \"configs\"")
    ap.add_argument("--no-peaks", action="store_true", help="skip the calibration kernels reported under \"measured_peaks\"")
    ap.add_argument("--only", choices=["qmv", "qmm", "copy", "configs"], default=None,
                    help="profiling aid: run just the rotating decode leg, just the prefill leg, just the table of every "
                         "configuration, or a plain 1 GiB device copy (the known-size kernel the HBM counters are scaled by)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (the path shards along N without exchange: "
                 "each GPU would run the same kernels on its rows of the weight)")

    import torch

    import nuvec_amd  # noqa: F401
    from nuvec_amd import _lib
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU")
    device = torch.device("cuda:0")
    lib = _lib.load()
    _lib.check(lib.nvq_init(0))
    if args.only == "copy":
        src = torch.empty(1 << 29, dtype=torch.bfloat16, device=device).fill_(1.0)  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes_read": src.numel() * 2, "copy_bytes_written": dst.numel() * 2, "launches": 10}))
        return

    only = args.only
    qs = make_weights(args.copies if only != "qmm" else 4, device)
    if only == "configs":
        print(json.dumps({"configs": all_configs(lib, device, qs)}))
        return
    record = {"metric": METRIC, "unit": "GB/s", "n_gpus": 1, "higher_is_better": True, "scaling": "weak",
              "vs_baseline": None, "dtype": "bf16", "data": "synthetic"}

    if only != "qmm":
        x1 = torch.randn(1, K, device=device).to(torch.bfloat16)
        ys = [torch.empty(1, N, dtype=torch.bfloat16, device=device) for _ in qs]
        calls = [Product(lib, 1, x1, q, y) for q, y in zip(qs, ys)]
        # (untimed: the clocks and the caches of a process that has only allocated so far; the W warm-up steps and the K
        # timed steps follow as asked)
        time_launches(calls, 240, 24, graph=False)
        ms, steps = time_launches(calls, args.steps, args.warmup, graph=False)
        gbps = WEIGHT_BYTES / (ms * 1e-3) / 1e9
        record.update({
            "value": gbps, "steps": steps, "warmup": args.warmup, "ms_per_step": ms,
            "config": {"workload": "configs[1]: decode QMV, affine 4-bit g64, x bf16 [1,4096], W [14336,4096], M=1",
                       "weight_copies_rotated": args.copies,
                       "submission": "one C-ABI call per launch, back to back on one stream"},
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": gbps / HBM_PEAK_GBPS, "traffic": QMV_TRAFFIC_BYTES,
                         "kernel": lib.nvq_quantized_matmul_route(C.byref(calls[0].d)).decode(),
                         "bytes_per_launch": WEIGHT_BYTES, "us_per_launch": ms * 1e3},
        })
        if only is None:
            graph_ms, _ = time_launches(calls, min(args.steps, 2000), 50, graph=True)
            hot_ms, _ = time_launches(calls[:1] * len(calls), min(args.steps, 2000), 50, graph=False)
            record["graph_replay"] = {"us_per_launch": graph_ms * 1e3, "gbps": WEIGHT_BYTES / (graph_ms * 1e-3) / 1e9,
                                      "note": "the same launches captured once into a HIP graph per rotation and replayed"}
            record["cache_hot"] = {"us_per_launch": hot_ms * 1e3, "gbps": WEIGHT_BYTES / (hot_ms * 1e-3) / 1e9,
                                   "note": "one weight buffer reused: served from the last-level cache, not an HBM figure"}

    if only == "qmm" or (only is None and not args.no_qmm):
        m = 2048
        xm = torch.randn(m, K, device=device).to(torch.bfloat16)
        ym = torch.empty(m, N, dtype=torch.bfloat16, device=device)
        qcalls = [Product(lib, m, xm, q, ym) for q in qs[:4]]
        # four runs of `qmm_steps` launches; the first sits on the clock ramp and is dropped, the others are averaged
        runs = [time_launches(qcalls, args.qmm_steps, 4, graph=False) for _ in range(4)][1:]
        qms, qsteps = sum(r[0] for r in runs) / len(runs), sum(r[1] for r in runs)
        best_ms = min(r[0] for r in runs)
        flop = 2.0 * m * N * K
        tflops = flop / (qms * 1e-3) / 1e12
        record["qmm"] = {"workload": "configs[2]: prefill QMM, affine 4-bit g64, x bf16 [2048,4096], W [14336,4096]",
                         "value": tflops, "unit": "TFLOP/s", "ms_per_step": qms, "steps": qsteps,
                         "best_run": {"ms_per_step": best_ms, "tflops": flop / (best_ms * 1e-3) / 1e12},
                         "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                      "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": QMM_TRAFFIC_BYTES,
                                      "kernel": "qmm_kernel (256x256 tile)", "flop_per_launch": flop}}

    if only is None and not args.no_peaks:
        record["measured_peaks"] = measured_peaks(lib, device, qs)
    if only is None and not args.no_configs:
        record["configs"] = all_configs(lib, device, qs)
    if only is None and not args.no_cpu:
        record["cpu_baseline"] = cpu_baseline()
    print(json.dumps(record))


if __name__ == "__main__":
    main()
