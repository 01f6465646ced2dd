"""The checkpoint loader (nuvec_amd/checkpoint.py) on the small quantized checkpoints the reference's own tests hold
(tests/golden/checkpoints/, copied by tests/golden/copy_checkpoints.py): the safetensors reader against the
`safetensors` library and against the reference's header rules, the `quantization` config and the per-layer rule on
the CPU; on the GPU the loaded layers dequantized by the HIP library against the oracle, bit for bit."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from nuvec_amd import checkpoint as ck
from nuvec_amd.ops import InvalidArgument, Quant, QuantMode
from oracle import formats as fmt_ref
from oracle import ref

ROOT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "checkpoints")
NAMES = ["qwen2_q4", "gpt_oss_mxfp4", "qwen3_moe_nvfp4_gs", "llama_mxfp8", "llama_gptq", "qwen3_awq", "qwen3_gptq8_v2"]
CODE = {torch.float16: ref.F16, torch.bfloat16: ref.BF16, torch.float32: ref.F32}


def host(t):
    t = t.contiguous().cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.uint32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.numpy()


@pytest.mark.parametrize("name", NAMES)
def test_reader_matches_the_safetensors_library(name):
    import safetensors.torch as st
    path = os.path.join(ROOT, name, "model.safetensors")
    mine, theirs = ck.load_safetensors(path, "cpu"), st.load_file(path)
    assert set(mine) == set(theirs) and len(mine) > 30
    for k, t in theirs.items():
        assert mine[k].dtype == t.dtype and mine[k].shape == t.shape, k
        assert torch.equal(mine[k].reshape(-1).view(torch.uint8), t.reshape(-1).view(torch.uint8)), k
    kept = ck.load_safetensors(path, "cpu", keep=lambda n: n.endswith(".scales"))
    assert kept and all(n.endswith(".scales") for n in kept) and len(kept) < len(mine)


def header(entries, data_len, meta=None):
    h = dict(entries)
    if meta is not None:
        h["__metadata__"] = meta
    raw = json.dumps(h).encode()
    return raw, 8 + len(raw), 8 + len(raw) + data_len


def test_header_rules():
    """safetensors.rs:188-272: what a header must satisfy, with the reference's messages."""
    ok = {"a": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 16]}, "b": {"dtype": "U8", "shape": [3], "data_offsets": [16, 19]}}
    tensors, meta = ck.parse_header(*header(ok, 19, {"format": "mlx"}))
    assert [(t.name, t.shape, t.end - t.begin) for t in tensors] == [("a", (2, 2), 16), ("b", (3,), 3)] and meta == {"format": "mlx"}
    bad = [
        ({"a": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 12]}}, 12, "do not hold 16 bytes"),
        ({"a": {"dtype": "F8_E5M2", "shape": [4], "data_offsets": [0, 4]}}, 4, "unsupported dtype F8_E5M2"),
        ({"a": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}, "b": {"dtype": "U8", "shape": [4], "data_offsets": [2, 6]}}, 6, "overlap or leave a gap"),
        ({"a": {"dtype": "U8", "shape": [4], "data_offsets": [1, 5]}}, 5, "overlap or leave a gap"),
        ({"a": {"dtype": "U8", "shape": [4], "data_offsets": [0, 4]}}, 9, "do not cover the data to the end"),
        ({"a": {"shape": [4], "data_offsets": [0, 4]}}, 4, "missing dtype"),
        ({"a": {"dtype": "U8", "data_offsets": [0, 4]}}, 4, "missing shape"),
        ({"a": {"dtype": "U8", "shape": [4]}}, 4, "missing data_offsets"),
        ({"a": {"dtype": "U8", "shape": [-4], "data_offsets": [0, 4]}}, 4, "a dimension must be a non-negative integer"),
        ({"a": 3}, 0, "entry `a` must be an object"),
    ]
    for entries, n, message in bad:
        with pytest.raises(InvalidArgument, match=message):
            ck.parse_header(*header(entries, n))
    with pytest.raises(InvalidArgument, match="metadata values must be strings"):
        ck.parse_header(*header(ok, 19, {"n": 3}))
    twice = b'{"a": {"dtype": "U8", "shape": [1], "data_offsets": [0, 1]}, "a": {"dtype": "U8", "shape": [1], "data_offsets": [1, 2]}}'
    with pytest.raises(InvalidArgument, match="duplicate tensor `a`"):
        ck.parse_header(twice, 8 + len(twice), 8 + len(twice) + 2)
    with pytest.raises(InvalidArgument, match="must be a JSON object"):
        ck.parse_header(b"[1]", 11, 11)
    # an F8_E4M3 / F8_E8M0 tensor reads as bytes (safetensors.rs:47-49)
    t, _ = ck.parse_header(*header({"s": {"dtype": "F8_E8M0", "shape": [5], "data_offsets": [0, 5]}}, 5))
    assert t[0].dtype == torch.uint8


def test_file_errors(tmp_path):
    p = tmp_path / "m.safetensors"
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(InvalidArgument, match="header larger than the file or 100 MB"):
        ck.read_header(str(p))
    raw = json.dumps({"w": {"dtype": "I32", "shape": [3], "data_offsets": [0, 12]}}).encode()
    p.write_bytes(struct.pack("<Q", len(raw)) + raw + np.array([7, -8, 9], np.int32).tobytes())
    assert ck.load_safetensors(str(p), "cpu")["w"].tolist() == [7, -8, 9]
    p.write_bytes(struct.pack("<Q", len(raw)) + raw + b"\0" * 11)
    with pytest.raises(InvalidArgument, match="do not cover the data"):
        ck.load_safetensors(str(p), "cpu")
    empty = json.dumps({"e": {"dtype": "F16", "shape": [0, 4], "data_offsets": [0, 0]}}).encode()
    p.write_bytes(struct.pack("<Q", len(empty)) + empty)
    assert ck.load_safetensors(str(p), "cpu")["e"].shape == (0, 4)


def config_of(name):
    with open(os.path.join(ROOT, name, "config.json")) as f:
        return json.load(f)


def test_quantization_of_the_configs():
    """config.rs:1038-1190 on the reference's own configs."""
    q = ck.Quantization.from_config(config_of("qwen2_q4"))
    assert q.default == Quant.affine(32, 4) and q.layers == () and q.packed is None
    q = ck.Quantization.from_config(config_of("gpt_oss_mxfp4"))
    assert q.default == Quant.new(QuantMode.MXFP4)
    assert q.for_layer("model.layers.0.mlp.router") == ck.LayerQuant("model.layers.0.mlp.router", Quant.affine(64, 8), False)
    assert q.for_layer("model.layers.0.mlp.experts.down_proj") is None
    q = ck.Quantization.from_config(config_of("qwen3_moe_nvfp4_gs"))
    assert q.default == Quant.new(QuantMode.NVFP4)
    assert q.for_layer("model.layers.0.mlp.switch_mlp.up_proj") == ck.LayerQuant("model.layers.0.mlp.switch_mlp.up_proj", Quant.new(QuantMode.NVFP4), True)
    assert q.for_layer("model.layers.0.mlp.gate").quant == Quant.affine(64, 8)
    assert ck.Quantization.from_config(config_of("llama_mxfp8")).default == Quant.new(QuantMode.MXFP8)
    for name, packed, quant in [("llama_gptq", "gptq", Quant.affine(32, 4)), ("qwen3_awq", "awq", Quant.affine(64, 4)),
                                ("qwen3_gptq8_v2", "gptq_v2", Quant.affine(32, 8))]:
        q = ck.Quantization.from_config(config_of(name))
        assert (q.packed, q.default) == (packed, quant)
    assert ck.Quantization.from_config({"model_type": "llama"}) is None


def test_quantization_rules():
    from_config = ck.Quantization.from_config
    assert from_config({"quantization": {"mode": "mxfp8"}}).default == Quant(QuantMode.MXFP8, 32, 8)  # the mode's defaults
    q = from_config({"quantization": {"group_size": 64, "bits": 4, "model.language_model.layers.0.mlp": {"bits": 8},
                                      "language_model.lm_head": False, "note": "x"}})
    assert q.for_layer("model.layers.0.mlp").quant == Quant.affine(64, 8)  # renamed as the loader renames weights
    assert q.for_layer("lm_head") == ck.LayerQuant("lm_head", None, False) and len(q.layers) == 2
    for bad, message in [({"quantization": {"note": 1}}, "needs `group_size` and `bits`"),
                         ({"quantization": {"mode": "int4"}}, "unsupported quantization mode"),
                         ({"quantization": {"bits": 9}}, "9 bits"),
                         ({"quantization": {"bits": 4, "group_size": 0}}, "group size 0"),
                         ({"quantization_config": {"quant_method": "awq", "bits": 8}}, "awq: version"),
                         ({"quantization_config": {"quant_method": "awq", "version": "gemv"}}, "awq: version"),
                         ({"quantization_config": {"quant_method": "gptq", "bits": 3}}, "gptq: 3 bits"),
                         ({"quantization_config": {"quant_method": "gptq", "desc_act": True}}, "desc_act"),
                         ({"quantization_config": {"quant_method": "gptq", "group_size": 48}}, "group size 48"),
                         ({"quantization_config": {"quant_method": "fp8"}}, "not converted yet"),
                         ({"quantization_config": {"quant_method": "mxfp4"}, "model_type": "llama"}, "not converted yet"),
                         ({"quantization_config": {"quant_method": "bnb"}}, "unsupported quantization method")]:
        with pytest.raises(InvalidArgument, match=message):
            from_config(bad)
    assert from_config({"quantization_config": {"quant_method": "mxfp4"}, "model_type": "gpt_oss"}).default == Quant.new(QuantMode.MXFP4)
    assert from_config({"text_config": {"quantization_config": {"quant_method": "gptq"}}}) == ck.Quantization(Quant.affine(128, 4), (), "gptq")


def test_infer_quant():
    """lib.rs:462-479: packed words per group tell the floating-point modes apart."""
    u32 = lambda *s: torch.zeros(s, dtype=torch.int32).view(torch.uint32)
    u8 = lambda *s: torch.zeros(s, dtype=torch.uint8)
    default = Quant.affine(32, 4)
    assert ck.infer_quant(u32(8, 16), u8(8, 8), default) == Quant.new(QuantMode.NVFP4)
    assert ck.infer_quant(u32(8, 16), u8(8, 4), default) == Quant.new(QuantMode.MXFP4)
    assert ck.infer_quant(u32(8, 16), u8(8, 2), default) == Quant.new(QuantMode.MXFP8)
    assert ck.infer_quant(u32(8, 16), torch.zeros(8, 4, dtype=torch.float16), default) == default
    assert ck.infer_quant(u32(8, 16), torch.zeros(8, 4, dtype=torch.float16), Quant.new(QuantMode.MXFP4)) == Quant.new(QuantMode.AFFINE)


def test_layers_of_the_checkpoints():
    """lib.rs:573-590: named layers take their entry, the others are recognised from their tensors."""
    weights = ck.load_safetensors(os.path.join(ROOT, "gpt_oss_mxfp4", "model.safetensors"), "cpu")
    layers, rest = ck.quantized_layers(weights, ck.Quantization.from_config(config_of("gpt_oss_mxfp4")))
    experts = layers["model.layers.0.mlp.experts.down_proj"]
    assert experts.quant == Quant.new(QuantMode.MXFP4) and experts.biases is None and experts.weight.shape == (8, 64, 8)
    assert layers["model.layers.0.mlp.router"].quant == Quant.affine(64, 8) and layers["model.layers.0.mlp.router"].biases is not None
    assert "model.layers.0.mlp.experts.down_proj.bias" in rest and "model.layers.0.mlp.experts.down_proj.weight" not in rest
    assert len(layers) * 2 + sum(l.biases is not None for l in layers.values()) + len(rest) == len(weights)
    weights = ck.load_safetensors(os.path.join(ROOT, "qwen3_moe_nvfp4_gs", "model.safetensors"), "cpu")
    layers, rest = ck.quantized_layers(weights, ck.Quantization.from_config(config_of("qwen3_moe_nvfp4_gs")))
    up = layers["model.layers.0.mlp.switch_mlp.up_proj"]
    assert up.quant == Quant.new(QuantMode.NVFP4) and up.global_scale.shape == (16,) and up.global_scale.dtype == torch.float32
    assert layers["lm_head"].quant == Quant.new(QuantMode.NVFP4) and layers["lm_head"].global_scale is None
    assert not any(n.endswith(".global_scale") for n in rest)
    kept = ck.Quantization(Quant.new(QuantMode.NVFP4), (ck.LayerQuant("lm_head", None),))
    assert "lm_head" not in ck.quantized_layers(weights, kept)[0] and "lm_head.weight" in ck.quantized_layers(weights, kept)[1]
    assert ck.quantized_layers(weights, None) == ({}, weights)


def oracle_dense(q, e=None):
    """The oracle's dequantize of a loaded layer (of expert `e` of a stacked layer with global scales)."""
    w, s = host(q.weight), host(q.scales)
    if q.quant.mode == QuantMode.AFFINE:
        return ref.affine_dequantize(w, s, host(q.biases), CODE[q.scales.dtype], q.quant.group_size, q.quant.bits)
    if e is not None:
        return ref.fp_dequantize(w[e], s[e], int(q.quant.mode), ref.BF16, float(q.global_scale[e]))
    return ref.fp_dequantize(w, s, int(q.quant.mode), ref.BF16)


@pytest.mark.gpu
@pytest.mark.parametrize("name", NAMES)
def test_loaded_layers_dequantize_like_the_oracle(name):
    """Every quantized layer of the checkpoint, read straight into device memory (AWQ / GPTQ repacked there),
    dequantized by the HIP library: bit for bit the oracle's dequantize of the same tensors read on the host."""
    import nuvec_amd as nv
    directory = os.path.join(ROOT, name)
    layers, rest, quantization = ck.load_quantized(directory, "cuda")
    assert layers and all(t.is_cuda for t in rest.values())
    host_weights = ck.load_safetensors(os.path.join(directory, "model.safetensors"), "cpu")
    if quantization.packed is None:
        host_layers, _ = ck.quantized_layers(host_weights, quantization)
    else:  # the oracle's repacking of the Hugging Face layout
        host_layers = {}
        bits, group = quantization.default.bits, quantization.default.group_size
        for n in sorted(host_weights):
            if n.endswith(".qweight"):
                p = n[:-len(".qweight")]
                scales = host_weights[p + ".scales"]
                w, s, b = fmt_ref.convert_packed(host_weights[n].numpy(), host_weights[p + ".qzeros"].numpy(), host(scales),
                                                 CODE[scales.dtype], quantization.packed, bits, group)
                as_t = lambda a, like: torch.from_numpy(a.view(np.int16)).view(like.dtype) if like.dtype == torch.bfloat16 else torch.from_numpy(a)
                host_layers[p] = nv.Quantized(torch.from_numpy(w.view(np.int32)).view(torch.uint32), as_t(s, scales), as_t(b, scales),
                                              quantization.default)
    assert set(layers) == set(host_layers)
    for path, q in layers.items():
        assert q.weight.is_cuda and q.quant == host_layers[path].quant, path
        if q.global_scale is not None:  # one global scale per expert
            for e in range(q.weight.shape[0]):
                one = nv.Quantized(q.weight[e], q.scales[e], None, q.quant, q.global_scale[e:e + 1])
                got = host(nv.dequantize(one, torch.bfloat16))
                assert np.array_equal(got, oracle_dense(host_layers[path], e)), (path, e)
            continue
        dtype = q.scales.dtype if q.quant.mode == QuantMode.AFFINE else torch.bfloat16
        got = host(nv.dequantize(q, dtype))
        want = oracle_dense(host_layers[path])
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), path
