"""Copies the small quantized checkpoints the reference's own tests hold (crates/nuvec-lm/tests/fixtures/<name>/
config.json and model.safetensors: data files, a few hundred KB together) into tests/golden/checkpoints/, where the
loader's tests read them, and the recorded quantized-attention cases (tests/fixtures/kv_quant_attention.safetensors:
queries, quantized keys and values, mlx-lm's outputs) into tests/golden/, and the gated activations mlx-lm recorded
for the reference's test `activations_equal_mlx_lm` (crates/nuvec-nn/tests/rope_scaling.rs:150-172; the `act_*` tensors
of crates/nuvec-nn/tests/fixtures/mlx_lm_ops.safetensors: gate, x, swiglu_oai and geglu in float32 and bfloat16) into
tests/golden/mlx_lm_activations.safetensors.  Run once in a container that has the reference: python tests/golden/copy_checkpoints.py"""
import os
import shutil

SOURCE = "/root/reference/crates/nuvec-lm/tests/fixtures"
NAMES = ["qwen2_q4", "gpt_oss_mxfp4", "qwen3_moe_nvfp4_gs", "llama_mxfp8", "llama_gptq", "qwen3_awq", "qwen3_gptq8_v2"]

if __name__ == "__main__":
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "checkpoints")
    for name in NAMES:
        os.makedirs(os.path.join(here, name), exist_ok=True)
        for part in ("config.json", "model.safetensors"):
            shutil.copyfile(os.path.join(SOURCE, name, part), os.path.join(here, name, part))
            os.chmod(os.path.join(here, name, part), 0o644)
        print(name, os.path.getsize(os.path.join(here, name, "model.safetensors")), "bytes")
    recorded = os.path.join(os.path.dirname(here), "kv_quant_attention.safetensors")
    shutil.copyfile(os.path.join(SOURCE, "kv_quant_attention.safetensors"), recorded)
    os.chmod(recorded, 0o644)
    print("kv_quant_attention", os.path.getsize(recorded), "bytes")
    from safetensors import safe_open
    from safetensors.torch import save_file
    with safe_open("/root/reference/crates/nuvec-nn/tests/fixtures/mlx_lm_ops.safetensors", "pt") as f:
        taken = {k: f.get_tensor(k).contiguous() for k in f.keys() if k.startswith("act_") and not k.endswith(".softcap")}
    activations = os.path.join(os.path.dirname(here), "mlx_lm_activations.safetensors")
    save_file(taken, activations)
    print("mlx_lm_activations", sorted(taken), os.path.getsize(activations), "bytes")
