"""Row independence, run-to-run determinism and re-entrancy of the HIP path, through the C ABI.

Mirrors the reference's tests of the same contracts:
  * `few_row_products_equal_one_row_products_bit_for_bit` (crates/nuvec-core/tests/quantized.rs:794-831) and
    `sorted_few_row_gathers_keep_the_one_row_bits` (:1798-1900): under `row_exact` a product of up to eight rows gives
    every row the bits of its one-row product, and a sorted gather the bits of the unsorted one;
  * `kernels_are_deterministic` (crates/nuvec-core/tests/determinism.rs:47-88): every route, run again into reused
    buffers, gives identical bits;
  * many host threads evaluate at once (eval.rs:129-137): eight threads on their own streams get the serial results.
"""
import threading

import numpy as np
import pytest
import torch

import nuvec_amd as nv
from oracle import ref
from tests.hip_backend import TORCH, to_dev, to_host
from tests.test_gpu_parity import assert_rows_close, make_w, make_x

pytestmark = pytest.mark.gpu


def bits_of(t):
    return to_host(t).view(np.uint8)


@pytest.mark.parametrize("dtype", [ref.BF16, ref.F16, ref.F32])
@pytest.mark.parametrize("m,k,n,group,bits", [(6, 4096, 512, 64, 4), (5, 1024, 1000, 32, 4), (4, 2048, 256, 128, 4),
                                              (8, 4096, 14336, 64, 4), (7, 1024, 130, 64, 3), (3, 512, 96, 32, 8),
                                              (8, 768, 64, 64, 2), (2, 640, 72, 128, 6)])
def test_row_exact_rows_equal_their_one_row_products(dtype, m, k, n, group, bits):
    """tests/quantized.rs:794-831, widened to the other code widths: odd and even row counts, N off the block size."""
    rng = np.random.default_rng(m * 1000 + bits)
    w, x = make_w(rng, n, k, dtype), make_x(rng, m, k, dtype)
    q = nv.quantize(to_dev(w), nv.Quant.affine(group, bits))
    xd = to_dev(x)
    both = bits_of(nv.quantized_matmul(xd, q, row_exact=True))
    for r in range(m):
        one = bits_of(nv.quantized_matmul(xd[r:r + 1], q, row_exact=True))
        assert np.array_equal(one[0], both[r]), f"row {r} of {m} differs from its one-row product"
    # the values are the product's
    packed, scales, biases = to_host(q.weight), to_host(q.scales), to_host(q.biases)
    want = ref.quantized_matmul(x, packed, scales, biases, group=group, bits=bits, dtype=dtype)
    assert_rows_close(to_host(nv.quantized_matmul(xd, q, row_exact=True)), want, dtype, f"row-exact b{bits} g{group} M={m} K={k} N={n}")
    # `rows` (every row count on the matrix-vector kernels) keeps rows independent at any count
    many = np.concatenate([x, x[::-1], x, x[:1]])
    wide = bits_of(nv.quantized_matmul(to_dev(many), q, rows=True))
    assert np.array_equal(wide[:m], both) and np.array_equal(wide[-1], both[0])


@pytest.mark.parametrize("mode", ["MXFP4", "MXFP8", "NVFP4"])
def test_row_exact_block_formats_and_untransposed(mode):
    rng = np.random.default_rng(5)
    m, k, n = 7, 1024, 200
    w, x = make_w(rng, n, k, ref.BF16), make_x(rng, m, k, ref.BF16)
    q = nv.quantize(to_dev(w), nv.QuantMode[mode])
    xd = to_dev(x)
    both = bits_of(nv.quantized_matmul(xd, q, row_exact=True))
    for r in range(m):
        assert np.array_equal(bits_of(nv.quantized_matmul(xd[r:r + 1], q, row_exact=True))[0], both[r]), f"{mode}: row {r}"
    # weights stored [K, N]: K is split over the grid by the weight's shape alone
    wt = make_w(rng, k, 256, ref.BF16)
    qt = nv.quantize(to_dev(wt), nv.QuantMode[mode])
    both = bits_of(nv.quantized_matmul(xd, qt, transpose=False, row_exact=True))
    for r in range(m):
        one = bits_of(nv.quantized_matmul(xd[r:r + 1], qt, transpose=False, row_exact=True))
        assert np.array_equal(one[0], both[r]), f"{mode} untransposed: row {r}"


@pytest.mark.parametrize("dtype", [ref.F16, ref.BF16])
@pytest.mark.parametrize("bits", [2, 3, 4, 8])
def test_sorted_few_row_gathers_keep_the_one_row_bits(dtype, bits):
    """tests/quantized.rs:1798-1900: 2 to 8 tokens' top-8 of 16 experts, sorted by expert as a mixture-of-experts
    layer sorts them, against the unsorted per-pair gather and against each token alone."""
    rng = np.random.default_rng(0x1D5 + bits)
    experts, n, k, top = 16, 256, 512, 8
    w = ref.from_f32((rng.standard_normal((experts, n, k)) * 0.1).astype(np.float32), dtype)
    q = nv.quantize(to_dev(w), nv.Quant.affine(64, bits))
    for tokens in (2, 5, 8):
        ids = np.stack([rng.permutation(experts)[:top] for _ in range(tokens)]).astype(np.int64)
        x = to_dev(make_x(rng, tokens, k, dtype)).reshape(1, tokens, 1, 1, k)
        idx = torch.from_numpy(ids).cuda().reshape(1, tokens, top)
        unsorted = nv.gather_qmm(x, q, None, idx, nv.GatherQmm(), row_exact=True)
        assert unsorted.shape == (1, tokens, top, 1, n)
        flat = idx.reshape(-1)
        order = torch.argsort(flat, stable=True)
        token_of = torch.arange(tokens * top, device="cuda") // top
        rows = x.reshape(-1, 1, k)[token_of[order]]
        got = nv.gather_qmm(rows, q, None, flat[order], nv.GatherQmm(sorted_indices=True), row_exact=True)
        restored = got[torch.argsort(order)].reshape(1, tokens, top, 1, n)
        assert np.array_equal(bits_of(restored), bits_of(unsorted)), f"b{bits}, {tokens} tokens: the sorted gather differs"
        for t in range(tokens):
            one = nv.gather_qmm(x[:, t:t + 1], q, None, idx[:, t:t + 1], nv.GatherQmm(), row_exact=True)
            assert np.array_equal(bits_of(one)[0, 0], bits_of(restored)[0, t]), f"b{bits}, token {t} of {tokens} alone differs"


def determinism_cases():
    """One product per route (determinism.rs:47-88 for this path): decode, few rows on both matrix-core kernels, tiled
    with and without a split of K, weights stored [K, N] (both kernels), rows of few outputs, the general kernel's
    modes, grouped and per-pair gathers, the gated activation, quantize and dequantize."""
    rng = np.random.default_rng(123)
    w = make_w(rng, 4096, 4096, ref.BF16)
    wd = to_dev(w)
    q4 = nv.quantize(wd, nv.Quant.affine(64, 4))
    cases = {}
    for rows in (1, 2, 4, 8, 16, 40, 256, 512):
        x = to_dev(make_x(rng, rows, 4096, ref.BF16))
        cases[f"b4 M={rows}"] = lambda x=x: nv.quantized_matmul(x, q4)
    x1, x512 = to_dev(make_x(rng, 1, 4096, ref.BF16)), to_dev(make_x(rng, 512, 4096, ref.BF16))
    cases["b4 M=512 unsplit"] = lambda: nv.quantized_matmul(x512, q4, scratch=False)
    cases["b4 untransposed"] = lambda: nv.quantized_matmul(x1, q4, transpose=False)
    cases["b4 row-exact M=8"] = lambda: nv.quantized_matmul(x512[:8], q4, row_exact=True)
    for group, bits in ((64, 3), (32, 8), (128, 2), (64, 6), (64, 5)):
        q = nv.quantize(wd[:1024], nv.Quant.affine(group, bits))
        for rows in (1, 16, 300):
            cases[f"b{bits} M={rows}"] = lambda q=q, rows=rows: nv.quantized_matmul(x512[:rows], q)
    xf = to_dev(make_x(rng, 3, 4096, ref.F32))
    qf = nv.quantize(wd[:512].float(), nv.Quant.affine(64, 4))
    cases["f32 M=3"] = lambda: nv.quantized_matmul(xf, qf)
    experts = to_dev(make_w(rng, 16 * 512, 1024, ref.BF16)).reshape(16, 512, 1024)
    ids = (torch.arange(512, device="cuda") * 16 // 512)
    xe = to_dev(make_x(rng, 512, 1024, ref.BF16)).reshape(512, 1, 1024)
    eq = nv.quantize(experts, nv.Quant.affine(64, 4))
    cases["grouped gather b4"] = lambda: nv.gather_qmm(xe, eq, None, ids, nv.GatherQmm(sorted_indices=True))
    cases["pair gather b4"] = lambda: nv.gather_qmm(xe[:24], eq, None, ids[:24].flip(0), nv.GatherQmm())
    for mode in ("MXFP4", "MXFP8", "NVFP4"):
        qm = nv.quantize(wd[:512], nv.QuantMode[mode])
        cases[f"{mode} M=64"] = lambda qm=qm: nv.quantized_matmul(x512[:64], qm)
        em = nv.quantize(experts, nv.QuantMode[mode])
        if mode == "NVFP4":
            em = nv.Quantized(em.weight, em.scales, None, em.quant, torch.full((16,), 0.5, device="cuda"))
        cases[f"{mode} grouped gather"] = lambda em=em: nv.gather_qmm(xe, em, None, ids, nv.GatherQmm(sorted_indices=True))
    # weights stored [K, N] on the matrix cores (K split through the workspace, and not), rows of few outputs on the
    # exact-weights kernels, the gated activation alone and as the grouped product's epilogue
    cases["b4 untransposed M=300"] = lambda: nv.quantized_matmul(x512[:300], q4, transpose=False)
    cases["b4 untransposed M=300 unsplit"] = lambda: nv.quantized_matmul(x512[:300], q4, transpose=False, scratch=False)
    qs = nv.quantize(wd[:256], nv.Quant.affine(64, 4))
    for rows in (1, 5, 512):
        cases[f"b4 N=256 M={rows}"] = lambda rows=rows: nv.quantized_matmul(x512[:rows], qs)
    cases["glu"] = lambda: nv.glu(x512[:, :2048], x512[:, 2048:], "swiglu_oai")
    eg = nv.quantize(experts, nv.QuantMode.MXFP4)
    paired = nv.Quantized(nv.pair_rows(eg.weight[:, :256], eg.weight[:, 256:], 1), nv.pair_rows(eg.scales[:, :256], eg.scales[:, 256:], 1), None, eg.quant)
    offsets = nv.sorted_offsets(ids.to(torch.int32), 16)
    tokens = torch.arange(512, device="cuda", dtype=torch.int32)
    cases["grouped gather with the gated epilogue"] = lambda: nv.gather_qmm_glu(xe.reshape(512, 1024), paired, tokens, ids.to(torch.int32), offsets, "swiglu")
    # the decode kernel on the block formats, unsorted pairs on the decode and the short-row kernels, the experts' bias in
    # the grouped and the per-pair epilogues, sorted pairs against weights stored [K, N], the fused attention at 3 bits
    em4 = nv.quantize(experts, nv.QuantMode.MXFP4)
    bias = to_dev(make_x(rng, 16, 512, ref.BF16))
    for mode in ("MXFP4", "MXFP8", "NVFP4"):
        qm = nv.quantize(wd[:1024], nv.QuantMode[mode])
        for rows in (1, 2):
            cases[f"{mode} decode M={rows}"] = lambda qm=qm, rows=rows: nv.quantized_matmul(x512[:rows], qm)
    cases["pair gather MXFP4, short rows"] = lambda: nv.gather_qmm(xe[:24], em4, None, ids[:24].flip(0), nv.GatherQmm())
    cases["pair gather b4, long rows"] = lambda: nv.gather_qmm(x512[:6].reshape(6, 1, 4096), nv.Quantized(q4.weight[None], q4.scales[None], q4.biases[None], q4.quant),
                                                               None, torch.zeros(6, dtype=torch.int64, device="cuda"), nv.GatherQmm())
    cases["grouped gather with the experts' bias"] = lambda: nv.gather_qmm_grouped(xe.reshape(512, 1024), em4, tokens, ids.to(torch.int32), offsets, expert_bias=bias)
    cases["pair gather with the experts' bias"] = lambda: nv.gather_qmm(xe[:24], em4, None, ids[:24].flip(0), nv.GatherQmm(), expert_bias=bias)
    ekn = nv.quantize(experts.transpose(1, 2).contiguous(), nv.QuantMode.MXFP4)  # stored [K, N] = [1024, 512]
    cases["grouped gather, weights stored [K, N]"] = lambda: nv.gather_qmm(xe, ekn, None, ids, nv.GatherQmm(transpose=False, sorted_indices=True))
    kv = nv.quantize(to_dev(make_x(rng, 2 * 700, 128, ref.BF16)).reshape(1, 2, 700, 128), nv.Quant.affine(64, 3))
    qh = to_dev(make_x(rng, 8, 128, ref.BF16)).reshape(1, 8, 1, 128)
    cases["attention, 3-bit cache"] = lambda: nv.ops.quantized_attention(qh, kv, kv, 0.088)
    cases["unsorted pairs with the gated epilogue"] = lambda: nv.gather_qmm_glu(xe.reshape(512, 1024)[:24], paired, tokens[:24], ids.to(torch.int32)[:24].flip(0), None, "geglu")
    q4p = nv.Quantized(nv.pair_rows(q4.weight[:2048], q4.weight[2048:], 0), nv.pair_rows(q4.scales[:2048], q4.scales[2048:], 0),
                       nv.pair_rows(q4.biases[:2048], q4.biases[2048:], 0), q4.quant)
    cases["two rows with the gated epilogue"] = lambda: nv.quantized_matmul_glu(x512[:2], q4p, "swiglu")
    cases["quantize b4"] = lambda: nv.quantize(wd, nv.Quant.affine(64, 4)).weight
    cases["quantize mxfp4"] = lambda: nv.quantize(wd, nv.QuantMode.MXFP4).weight
    cases["dequantize b4"] = lambda: nv.dequantize(q4)
    return cases


def test_kernels_are_deterministic_under_buffer_reuse():
    """Every route three times; between the runs the outputs are dropped, so the allocator hands the same buffers out
    again (and scratch memory holds the previous run's partial sums)."""
    cases = determinism_cases()
    first = {name: bits_of(run()).copy() for name, run in cases.items()}
    torch.cuda.synchronize()
    for again in range(2):
        for name, run in cases.items():
            assert np.array_equal(bits_of(run()), first[name]), f"{name}: run {again + 2} differs from the first"


def test_eight_host_threads_on_their_own_streams():
    """The library is re-entrant: eight threads call the C ABI at once, each on a stream of its own, and every one
    gets the bits of the serial run."""
    cases = determinism_cases()
    names = list(cases)
    serial = {name: bits_of(cases[name]()).copy() for name in names}
    torch.cuda.synchronize()
    failures, barrier = [], threading.Barrier(8)

    def work(t):
        try:
            stream = torch.cuda.Stream()
            barrier.wait()
            with torch.cuda.stream(stream):
                for rep in range(3):
                    for name in names[t % 3::3] + names:  # threads walk the routes in different orders
                        out = cases[name]()
                        stream.synchronize()
                        if not np.array_equal(bits_of(out), serial[name]):
                            failures.append(f"thread {t}: {name} differs from the serial run")
        except Exception as e:  # noqa: BLE001 - reported below
            failures.append(f"thread {t}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=work, args=(t,)) for t in range(8)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not failures, failures[:5]


@pytest.mark.parametrize("transpose", [True, False])
def test_indices_and_offsets_outside_their_operands_are_clamped(transpose):
    """A caller's error must not reach the device as an access outside an operand (the reference's contract for
    primitives built with bad parameters, tests/primitive_fuzz.rs:97-131, 423-431: an error or a result, never a
    crash): expert ids beyond the experts, rows of x beyond x, offsets that do not ascend or leave the pairs.  The
    kernels clamp them; rows whose indices were valid keep their values."""
    rng = np.random.default_rng(77)
    experts, n, k, pairs = 6, 1152, 256, 96
    w = to_dev(make_w(rng, experts * n, k, ref.BF16)).reshape(experts, n, k)
    q = nv.quantize(w if transpose else w.transpose(1, 2).contiguous(), nv.QuantMode.MXFP4)
    x = to_dev(make_x(rng, pairs, k, ref.BF16))
    ids = torch.sort(torch.from_numpy(rng.integers(0, experts, pairs).astype(np.int32)).cuda())[0]
    rows = torch.arange(pairs, dtype=torch.int32, device="cuda")
    offsets = nv.sorted_offsets(ids, experts)
    options = nv.GatherQmm(transpose=transpose)
    good = nv.gather_qmm(x.reshape(pairs, 1, k), q, rows, ids, options)
    # unsorted pairs with indices out of range
    bad_ids, bad_rows = ids.clone(), rows.clone()
    bad_ids[::7] = 1000
    bad_rows[::5] = 5000
    got = nv.gather_qmm(x.reshape(pairs, 1, k), q, bad_rows, bad_ids, options)
    keep = torch.ones(pairs, dtype=torch.bool, device="cuda")
    keep[::7] = False
    keep[::5] = False
    assert torch.isfinite(got.float()).all() and torch.equal(got[keep], good[keep])
    # grouped, with offsets that descend, are negative or leave the pairs
    if transpose:
        for broken in ([5, 3, 900, -4, 50, 20], [0, 0, 0, 0, 0, 0], [96, 96, 96, 96, 96, 96], [-1, -1, 200, 200, 10, 10 ** 6]):
            out = nv.gather_qmm_grouped(x, q, bad_rows, ids, torch.tensor(broken, dtype=torch.int32, device="cuda"))
            torch.cuda.synchronize()
            assert tuple(out.shape) == (pairs, n)
        whole = nv.gather_qmm_grouped(x, q, rows, ids, offsets)
        assert torch.isfinite(whole.float()).all()
    else:
        sorted_out = nv.gather_qmm(x.reshape(pairs, 1, k), q, None, ids, nv.GatherQmm(transpose=False, sorted_indices=True))
        assert torch.isfinite(sorted_out.float()).all()
