"""The entry point that allocates nothing, `nvq_quantized_matmul_static`, against `nvq_quantized_matmul` given the
workspace its size query names: bit for bit, on two calls in a row (the second on a smaller product, so that the
scratch still holds the first call's partial sums), then the refusal of a product whose partial sums exceed the scratch."""
import ctypes as C

import numpy as np
import pytest
import torch

import nuvec_amd as nv
from nuvec_amd import _lib
from oracle import ref
from tests.hip_backend import to_dev, to_host
from tests.test_gpu_parity import assert_rows_close, make_w, make_x

pytestmark = pytest.mark.gpu


def desc(quant, m, n, k, transpose=1):
    d = _lib.QmmDescC()
    d.quant, d.dtype, d.transpose = quant._c(), _lib.BF16, transpose
    d.m, d.n, d.k, d.item_rows = m, n, k, m
    return d


def ptr(t):
    return C.c_void_p(t.data_ptr())


def test_static_scratch_matches_the_workspace_entry_point():
    lib = _lib.load()
    rng = np.random.default_rng(77)
    quant = nv.Quant.affine(64, 4)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    # (rows, weight rows, K, transposed): tiled products that split K, then a smaller one, then weights stored [K, N] on
    # the matrix-core kernel (K split) and on the vector kernel (K no multiple of 64)
    for m, n, k, transpose in [(512, 4096, 4096, 1), (1024, 1024, 4096, 1), (40, 256, 2048, 0), (3, 256, 480, 0)]:
        w = make_w(rng, n, k, ref.BF16) if transpose else make_w(rng, k, n, ref.BF16)
        x = make_x(rng, m, k, ref.BF16)
        q = nv.quantize(to_dev(w), quant)
        xd = to_dev(x)
        d = desc(quant, m, n, k, transpose)
        need = lib.nvq_quantized_matmul_workspace_bytes(C.byref(d))
        assert 0 < need <= _lib.STATIC_SCRATCH_BYTES, need
        workspace = torch.empty(need, dtype=torch.uint8, device="cuda")
        want = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        _lib.check(lib.nvq_quantized_matmul(C.byref(d), ptr(xd), ptr(q.weight), ptr(q.scales), ptr(q.biases), ptr(want), ptr(workspace), stream))
        got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        _lib.check(lib.nvq_quantized_matmul_static(C.byref(d), ptr(xd), ptr(q.weight), ptr(q.scales), ptr(q.biases), ptr(got), stream))
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert np.array_equal(to_host(got), to_host(want)), f"{m}x{n}x{k} transpose={transpose}: differs from the workspace entry point"
        packed, scales, biases = to_host(q.weight), to_host(q.scales), to_host(q.biases)
        oracle = ref.quantized_matmul(x, packed, scales, biases, group=64, bits=4, dtype=ref.BF16, transpose=bool(transpose), threads=8)
        assert_rows_close(to_host(got), oracle, ref.BF16, f"static scratch {m}x{n}x{k} transpose={transpose}")


def test_static_scratch_refuses_what_it_cannot_hold():
    lib = _lib.load()
    quant = nv.Quant.affine(64, 4)
    one = torch.zeros(64, dtype=torch.uint8, device="cuda")
    nv.quantized_matmul(torch.zeros((1, 64), dtype=torch.bfloat16, device="cuda"),
                        nv.quantize(torch.zeros((8, 64), dtype=torch.bfloat16, device="cuda"), quant))  # binds the device
    found = False
    for m, n, k in [(512, 8192, 16384), (1024, 8192, 16384), (512, 16384, 16384), (768, 8192, 32768)]:
        d = desc(quant, m, n, k)
        need = lib.nvq_quantized_matmul_workspace_bytes(C.byref(d))
        if need > _lib.STATIC_SCRATCH_BYTES:
            found = True
            rc = lib.nvq_quantized_matmul_static(C.byref(d), ptr(one), ptr(one), ptr(one), ptr(one), ptr(one), None)
            assert rc == _lib.UNSUPPORTED and "static scratch" in _lib.last_error()
    assert found, "no product in the list needed more than the scratch"
