"""Quantized KV-cache attention against the cases the reference's own test holds
(crates/nuvec-lm/tests/fixtures/kv_quant_attention.safetensors, copied to tests/golden/ by
tests/golden/copy_checkpoints.py; read by model.rs:3646-3720 `quantized_attention_equals_mlx_lm`): queries
[1, 4, L, 64], keys and values quantized in groups of 32 at 8 and 4 bits over 2 heads and 40 positions, mlx-lm's
outputs; L = 1 unmasked and L = 6 causal; float32 and bfloat16.  The reference's tolerances: 1e-5 and 2e-2."""
import os

import numpy as np
import pytest
import torch

import nuvec_amd as nv
from nuvec_amd import checkpoint as ck
from oracle import ref

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "kv_quant_attention.safetensors")
CASES = [(dt, bits, l) for dt in ("f32", "bf16") for bits in (8, 4) for l in (1, 6)]
CODE = {"f32": ref.F32, "bf16": ref.BF16}
TOL = {"f32": 1e-5, "bf16": 2e-2}
SCALE, GROUP, POSITIONS = 0.125, 32, 40


def host(t):
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.uint32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()


@pytest.fixture(scope="module")
def recorded():
    return ck.load_safetensors(PATH, "cpu")


@pytest.mark.parametrize("dt,bits,l", CASES)
def test_oracle_attention_matches_the_recorded_outputs(recorded, dt, bits, l):
    """Attention in float64 over the oracle's dequantized keys and values reproduces mlx-lm's outputs: pins the
    reading of the case (grouped heads, the causal mask's alignment at the end of the cache, the scale)."""
    code = CODE[dt]
    g = lambda k: host(recorded[f"{dt}_b{bits}_l{l}_{k}"])
    kf = ref.to_f32(ref.affine_dequantize(g("k0"), g("k1"), g("k2"), code, GROUP, bits), code).astype(np.float64)
    vf = ref.to_f32(ref.affine_dequantize(g("v0"), g("v1"), g("v2"), code, GROUP, bits), code).astype(np.float64)
    q = ref.to_f32(g("q"), code).astype(np.float64).reshape(1, 2, 2, l, 64)
    logits = SCALE * np.einsum("bhrld,bhsd->bhrls", q, kf)
    if l > 1:
        hidden = np.arange(POSITIONS)[None, :] > (POSITIONS - l + np.arange(l))[:, None]
        logits = np.where(hidden, -np.inf, logits)
    p = np.exp(logits - logits.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("bhrls,bhsd->bhrld", p, vf).reshape(1, 4, l, 64)
    assert np.abs(ref.to_f32(g("out"), code) - want).max() < TOL[dt]


@pytest.mark.gpu
@pytest.mark.parametrize("dt,bits,l", CASES)
def test_quantized_attention_matches_the_recorded_outputs(recorded, dt, bits, l):
    """`layers.quantized_attention` (both products on the HIP library) within the reference's tolerance of mlx-lm."""
    import nuvec_amd as nv
    from nuvec_amd.layers import quantized_attention
    g = lambda k: recorded[f"{dt}_b{bits}_l{l}_{k}"].cuda()
    quant = nv.Quant.affine(GROUP, bits)
    k, v = nv.Quantized(g("k0"), g("k1"), g("k2"), quant), nv.Quantized(g("v0"), g("v1"), g("v2"), quant)
    want = recorded[f"{dt}_b{bits}_l{l}_out"]
    for fused in (True, False):  # one query row: the fused kernel and the composition; several: the composition twice
        got = quantized_attention(g("q"), k, v, SCALE, causal=l > 1, fused=fused)
        assert got.shape == want.shape and got.dtype == want.dtype
        assert (got.cpu().float() - want.float()).abs().max().item() < TOL[dt]
    from nuvec_amd import ops
    assert ops.quantized_attention_fits(g("q"), k, v) == (l == 1)


@pytest.mark.gpu
@pytest.mark.parametrize("batch,hq,hkv,s,d,bits,group,with_sinks", [
    (1, 32, 8, 8192, 128, 4, 64, False), (2, 8, 8, 1000, 64, 8, 32, True), (1, 4, 1, 777, 128, 8, 128, True),
    (3, 16, 2, 2049, 64, 4, 64, False), (1, 2, 2, 513, 128, 4, 32, True), (2, 8, 2, 1500, 128, 3, 64, True),
    (1, 16, 16, 700, 64, 3, 32, False), (1, 4, 2, 61, 128, 3, 128, True)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_positions_split_over_the_grid(batch, hq, hkv, s, d, bits, group, with_sinks, dtype):
    """Long caches: the positions split over the grid and merged (with the workspace) against one block per head
    (without) and against float32 attention over the dequantized cache; lengths off the tile size, grouped heads,
    sinks; queries, scales, biases and outputs in float32, bfloat16 and float16.  Bound: 2e-3 of the largest output
    in float32 (far under the bfloat16 step of the recorded cases' tolerance); in the 16-bit types one and a half
    rounding steps of the largest output (1.2e-2 bfloat16, inside the reference's 2e-2; 1.5e-3 float16), the output
    being rounded once from float32 sums."""
    from nuvec_amd import ops
    torch.manual_seed(s)
    kd, vd = torch.randn(batch, hkv, s, d, device="cuda").to(dtype), torch.randn(batch, hkv, s, d, device="cuda").to(dtype)
    quant = nv.Quant.affine(group, bits)
    k, v = nv.quantize(kd, quant), nv.quantize(vd, quant)
    q = torch.randn(batch, hq, 1, d, device="cuda").to(dtype)
    sinks = torch.randn(hq, device="cuda").to(dtype) if with_sinks else None
    scale = d ** -0.5
    assert ops.quantized_attention_fits(q, k, v, sinks)
    split = ops.quantized_attention(q, k, v, scale, sinks)
    whole = ops.quantized_attention(q, k, v, scale, sinks, scratch=False)
    assert split.dtype == dtype and whole.dtype == dtype
    kf = nv.dequantize(k).float().repeat_interleave(hq // hkv, dim=1)
    vf = nv.dequantize(v).float().repeat_interleave(hq // hkv, dim=1)
    scores = scale * q.float() @ kf.transpose(-1, -2)
    if with_sinks:
        scores = torch.cat([scores, sinks.float().view(1, hq, 1, 1).expand(batch, hq, 1, 1)], dim=-1)
    p = torch.softmax(scores, dim=-1)[..., :s]
    want = p @ vf
    bound = {torch.float32: 2e-3, torch.bfloat16: 1.2e-2, torch.float16: 1.5e-3}[dtype] * want.abs().max().item()
    assert (split.float() - want).abs().max().item() <= bound, "split"
    assert (whole.float() - want).abs().max().item() <= bound, "one block per head"
