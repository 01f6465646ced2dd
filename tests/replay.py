"""Replays recorded golden cases through a backend and compares with the recorded outputs.

A backend is any object with `quantize`, `dequantize`, `quantized_matmul` and `gather_qmm`
taking and returning numpy arrays (float16 as np.float16, bfloat16 as np.uint16 bit
patterns, each call naming its dtype code).  Two backends exist: `OracleBackend` below (the
CPU restatement) and the HIP backend's adapter in the GPU tests, so one replay serves both —
as the reference replays one fixture file on its CPU and its GPU
(reference: crates/nuvec-core/tests/mlx.rs:55-104, tests/common/fixture.rs:442-1065).
"""
from __future__ import annotations

import numpy as np

from oracle import ref

DT = ref.DTYPE_CODE  # "f16"/"bf16"/"f32" -> 9/10/11
EPS = {ref.F16: 2.0 ** -10, ref.BF16: 2.0 ** -7, ref.F32: float(np.finfo(np.float32).eps)}


def quant_of(case):
    """(mode, group, bits) of a case (fixture.rs `quant(case)`; mode defaults to affine)."""
    mode = ref.MODES[case.params.get("mode", "affine")]
    if mode == ref.AFFINE:
        return mode, int(case.params["group_size"]), int(case.params["bits"])
    return (mode,) + ref.FP_PARAMS[mode]


class OracleBackend:
    """Op-level semantics (quantized.rs:385-719) in numpy around the C oracle."""

    name = "oracle"

    def quantize(self, w, dtype, mode, group, bits, global_scale=None):
        if mode == ref.AFFINE:
            return ref.affine_quantize(w, dtype, group, bits)
        packed, scales = ref.fp_quantize(w, dtype, mode, global_scale)
        return packed, scales, None

    def dequantize(self, w, scales, biases, mode, group, bits, scales_dtype, out_dtype=None, global_scale=None):
        if mode == ref.AFFINE:
            out = ref.affine_dequantize(w, scales, biases, scales_dtype, group, bits)
            if out_dtype is not None and out_dtype != scales_dtype:
                out = ref.from_f32(ref.to_f32(out, scales_dtype), out_dtype)
            return out, (out_dtype or scales_dtype)
        out_dtype = out_dtype or ref.BF16
        return ref.fp_dequantize(w, scales, mode, out_dtype, global_scale), out_dtype

    def quantized_matmul(self, x, w, scales, biases, mode, group, bits, dtype, transpose):
        vector = x.ndim == 1
        if vector:
            x = x[None, :]
        if w.ndim > 2:
            batch = np.broadcast_shapes(x.shape[:-2], w.shape[:-2])
            full = lambda a: np.ascontiguousarray(np.broadcast_to(a, batch + a.shape[-2:]))
            x, w, scales = full(x), full(w), full(scales)
            biases = None if biases is None else full(biases)
        y = ref.quantized_matmul(x, w, scales, biases, mode=mode, group=group, bits=bits, dtype=dtype,
                                 transpose=transpose)
        return y[..., 0, :] if vector else y

    def qqmm(self, x, w, dtype, mode, gx, gw, prequantized):
        f = lambda g: None if g is None else float(g)
        return ref.qqmm(x, w, dtype, mode, f(gx), f(gw))

    def gather_qqmm(self, x, w, rhs, dtype, mode, gx, gw, prequantized):
        f = lambda g: None if g is None else float(g)
        return ref.gather_qqmm(x, w, rhs, dtype, mode, f(gx), f(gw))

    def gather_qmm(self, x, w, scales, biases, lhs, rhs, mode, group, bits, dtype, transpose, sorted_indices,
                   global_scales=None):
        xb = int(np.prod(x.shape[:-2], dtype=np.int64))
        eb = int(np.prod(w.shape[:-2], dtype=np.int64))
        lhs = np.arange(xb, dtype=np.uint32).reshape(x.shape[:-2]) if lhs is None else lhs
        rhs = np.arange(eb, dtype=np.uint32).reshape(w.shape[:-2]) if rhs is None else rhs
        lhs, rhs = np.broadcast_arrays(lhs, rhs)
        if global_scales is not None:  # quantized.rs:677-719: each pair against its expert's weights and scale
            xf, wf, sf = (a.reshape((-1,) + a.shape[-2:]) for a in (x, w, scales))
            outs = [ref.fp_quantized_matmul_scaled(xf[l], wf[r], sf[r], mode, dtype, float(global_scales.reshape(-1)[r]), transpose)
                    for l, r in zip(lhs.reshape(-1), rhs.reshape(-1))]
            return np.stack(outs).reshape(rhs.shape + outs[0].shape)
        return ref.gather_qmm(x, w, scales, biases, lhs, rhs, mode=mode, group=group, bits=bits, dtype=dtype,
                              transpose=transpose)


def _run_qq(case, backend, xs, names, mode):
    """fixture.rs:789-819: with `gs=1` the last two inputs are the activations' and the weight's global scales;
    `q=1` hands the weight over quantized, `q=0` dense (quantized for the product): the same values."""
    gx = gw = None
    if case.params.get("gs") == "1":
        gx, gw = xs[-2], xs[-1]
        xs = xs[:-2]
    dtype = DT[names[0]]
    if case.op == "qqmm":
        return [(backend.qqmm(xs[0], xs[1], dtype, mode, gx, gw, case.params.get("q") == "1"), names[0])]
    return [(backend.gather_qqmm(xs[0], xs[1], xs[2], dtype, mode, gx, gw, case.params.get("q") == "1"), names[0])]


def run_case(case, backend):
    """The case's outputs from `backend`: a list of (array, dtype_name)."""
    p = case.params
    xs = [t.array() for t in case.inputs]
    names = [t.dtype for t in case.inputs]
    mode, group, bits = quant_of(case)
    transpose = p.get("transpose", "1") == "1"
    if case.op in ("qqmm", "gather_qqmm"):
        return _run_qq(case, backend, xs, names, mode)
    if case.op == "quantize":
        w = xs[0]
        if p.get("pre") == "t":
            w = np.ascontiguousarray(np.swapaxes(w, -1, -2))
        elif p.get("pre") == "r":
            w = np.ascontiguousarray(w[..., ::-1])
        if p.get("gs") == "1":
            packed, scales, biases = backend.quantize(w, DT[names[0]], mode, group, bits, global_scale=xs[1])
        else:
            packed, scales, biases = backend.quantize(w, DT[names[0]], mode, group, bits)
        out = [(packed, "u32"), (scales, names[0] if mode == ref.AFFINE else "u8")]
        if biases is not None:
            out.append((biases, names[0]))
        return out
    if case.op == "dequantize":
        out_dtype = int(p["dtype"]) if "dtype" in p else None
        sdt = DT.get(names[1])
        if p.get("gs") == "1":
            out, code = backend.dequantize(xs[0], xs[1], None, mode, group, bits, sdt, out_dtype, global_scale=xs[2])
            return [(out, ref_name(code))]
        biases = xs[2] if len(xs) > 2 else None
        out, code = backend.dequantize(xs[0], xs[1], biases, mode, group, bits, sdt, out_dtype)
        return [(out, ref_name(code))]
    if case.op == "quantized_matmul":
        biases = xs[3] if len(xs) > 3 else None
        y = backend.quantized_matmul(xs[0], xs[1], xs[2], biases, mode, group, bits, DT[names[0]], transpose)
        return [(y, names[0])]
    if case.op == "gather_qmm":
        rest = list(xs[3:])
        extra = {"global_scales": rest.pop(0)} if p.get("gs") == "1" else {}
        idx = p.get("idx", "")
        lhs = rest.pop(0) if "l" in idx else None
        rhs = rest.pop(0) if "r" in idx else None
        y = backend.gather_qmm(xs[0], xs[1], xs[2], None, lhs, rhs, mode, group, bits, DT[names[0]], transpose,
                               p.get("sorted") == "1", **extra)
        return [(y, names[0])]
    raise KeyError(case.op)


def ref_name(code):
    return {ref.F16: "f16", ref.BF16: "bf16", ref.F32: "f32"}[code]


def as_f64(a, dtype_name):
    if dtype_name == "bf16":
        return ref.bf16_to_f32(a).astype(np.float64)
    return a.astype(np.float64)


def _is_nan(a, dtype_name):
    if dtype_name in ("u32", "u8"):
        return np.zeros(a.shape, bool)
    return np.isnan(as_f64(a, dtype_name))


def exact_bits(got, expected):
    """fixture.rs:138-185 `check_exact`: equal bytes, or both NaN.  Returns a message or None."""
    for k, ((g, gname), e) in enumerate(zip(got, expected)):
        ea = e.array()
        if gname != e.dtype or g.shape != ea.shape:
            return f"output {k}: {gname}{g.shape} vs recorded {e.dtype}{ea.shape}"
        same = (g.view(np.uint8).reshape(-1) == ea.view(np.uint8).reshape(-1))
        same = same.reshape(-1, ea.dtype.itemsize).all(axis=1)
        ok = same | (_is_nan(g, gname).reshape(-1) & _is_nan(ea, e.dtype).reshape(-1))
        if not ok.all():
            i = int(np.argmin(ok))
            return f"output {k} element {i}: {g.reshape(-1)[i]!r} vs recorded {ea.reshape(-1)[i]!r}"
    return None


def by_value(got, expected, tol=0.0):
    """fixture.rs:1331-1394 `compare`: integers exactly, floats `==` or both NaN or within tol."""
    for k, ((g, gname), e) in enumerate(zip(got, expected)):
        ea = e.array()
        if gname != e.dtype or g.shape != ea.shape:
            return f"output {k}: {gname}{g.shape} vs recorded {e.dtype}{ea.shape}"
        if gname in ("u32", "u8"):
            bad = g != ea
        else:
            a, b = as_f64(g, gname), as_f64(ea, e.dtype)
            with np.errstate(invalid="ignore"):
                bad = ~((a == b) | (np.isnan(a) & np.isnan(b)) | (np.abs(a - b) <= tol))
        if bad.any():
            i = int(np.argmax(bad.reshape(-1)))
            return f"output {k} element {i}: {g.reshape(-1)[i]!r} vs recorded {ea.reshape(-1)[i]!r} (tol {tol:g})"
    return None


def product_bound(case):
    """fixture.rs:1309-1316: 4(K+1) eps max|x| (max|s| (2^bits - 1) + max|b|), maxima floored at 1."""
    bound = lambda t: max(1.0, float(np.nanmax(np.abs(as_f64(t.array(), t.dtype)))))
    bits = int(case.params["bits"])
    k = case.inputs[0].shape[-1]
    eps = EPS[DT[case.outputs[0].dtype]]
    w = bound(case.inputs[2]) * ((1 << bits) - 1) + bound(case.inputs[3])
    return 4.0 * (k + 1.0) * eps * bound(case.inputs[0]) * w


def within_fr008(got, expected):
    """mlx.rs:125-147: |a - b| <= atol * max(1, max|b|) + rtol * |b| against the recorded GPU output."""
    (g, gname), e = got[0], expected[0]
    ea = e.array()
    if gname != e.dtype or g.shape != ea.shape:
        return f"{gname}{g.shape} vs recorded {e.dtype}{ea.shape}"
    atol, rtol = {"f32": (1e-5, 1e-4), "f16": (1e-3, 5e-3)}.get(e.dtype, (1e-2, 4e-2))
    a, b = as_f64(g, gname), as_f64(ea, e.dtype)
    scale = max(1.0, float(np.max(np.abs(b)))) if b.size else 1.0
    bad = np.abs(a - b) > atol * scale + rtol * np.abs(b)
    if bad.any():
        i = int(np.argmax(bad.reshape(-1)))
        return f"element {i}: {a.reshape(-1)[i]} vs recorded {b.reshape(-1)[i]}"
    return None
