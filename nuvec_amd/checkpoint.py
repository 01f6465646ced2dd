"""Quantized checkpoints (`config.json` + `model*.safetensors`) as `Quantized` operands in device memory.

Host mirror of the part of nuvec's loader that feeds the quantized path: the safetensors header and its checks
(crates/nuvec-io/src/safetensors.rs:31-52, 177-272), the `quantization` entry of a model's `config.json`
(crates/nuvec-lm/src/config.rs:1038-1110), the rule that tells a layer's quantization from its tensors
(crates/nuvec-lm/src/lib.rs:462-479, 573-590) and the tensor names of a quantized layer
(crates/nuvec-core/src/quantized.rs:292-312: `weight`, `scales`, `biases`, `global_scale`).  The file is memory-mapped
and every tensor's bytes go from the mapping to the device in one copy; nothing of the file is interpreted but its
JSON header.  AWQ / GPTQ layers pass through `formats.convert_packed` when the config names such a packing."""
from __future__ import annotations

import json
import mmap
import os
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple, Union

import torch

from . import formats
from .ops import InvalidArgument, Quant, QuantMode, Quantized

MAX_HEADER = 100_000_000  # safetensors.rs: a header beyond 100 MB is refused

# safetensors.rs:31-52: fp8 tensors are read as bytes (quantization scales); F8_E5M2 has no reading
_DTYPES = {
    "BOOL": torch.bool, "U8": torch.uint8, "U16": torch.uint16, "U32": torch.uint32, "U64": torch.uint64,
    "I8": torch.int8, "I16": torch.int16, "I32": torch.int32, "I64": torch.int64,
    "F16": torch.float16, "BF16": torch.bfloat16, "F32": torch.float32, "F64": torch.float64,
    "C64": torch.complex64, "F8_E4M3": torch.uint8, "F8_E8M0": torch.uint8,
}


def _invalid(msg: str) -> InvalidArgument:
    return InvalidArgument(f"safetensors: {msg}")


@dataclass(frozen=True)
class TensorInfo:
    """One entry of the header: where the tensor's bytes lie in the file."""
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    begin: int  # absolute file offsets
    end: int


def _usize(v, what: str) -> int:
    if isinstance(v, bool) or not isinstance(v, int) or v < 0:
        raise _invalid(f"{what} must be a non-negative integer")
    return v


def _reject_duplicates(pairs):
    seen = {}
    for k, v in pairs:
        if k in seen and k != "__metadata__":
            raise _invalid(f"duplicate tensor `{k}`")
        seen[k] = v
    return seen


def parse_header(raw: bytes, start: int, file_len: int) -> Tuple[List[TensorInfo], Dict[str, str]]:
    """safetensors.rs:188-272: the JSON header `raw` of a file of `file_len` bytes whose data starts at `start`.
    Every entry needs a known dtype, a shape and offsets that hold exactly its bytes; the tensors must tile the data
    from its start to the end of the file."""
    try:
        header = json.loads(raw.decode("utf-8"), object_pairs_hook=_reject_duplicates)
    except (UnicodeDecodeError, json.JSONDecodeError) as e:
        raise _invalid(f"the header is not JSON ({e})") from None
    if not isinstance(header, dict):
        raise _invalid("the header must be a JSON object")
    metadata: Dict[str, str] = {}
    tensors: List[TensorInfo] = []
    for name, entry in header.items():
        if name == "__metadata__":
            if entry is None:
                continue
            if not isinstance(entry, dict):
                raise _invalid("`__metadata__` must be an object")
            for k, v in entry.items():
                if not isinstance(v, str):
                    raise _invalid("metadata values must be strings")
                metadata[k] = v
            continue
        if not isinstance(entry, dict):
            raise _invalid(f"entry `{name}` must be an object")
        d = entry.get("dtype")
        if not isinstance(d, str):
            raise _invalid(f"`{name}`: missing dtype")
        if d not in _DTYPES:
            raise _invalid(f"`{name}`: unsupported dtype {d}")
        dtype = _DTYPES[d]
        if not isinstance(entry.get("shape"), list):
            raise _invalid(f"`{name}`: missing shape")
        shape = tuple(_usize(s, "a dimension") for s in entry["shape"])
        o = entry.get("data_offsets")
        if not isinstance(o, list) or len(o) != 2:
            raise _invalid(f"`{name}`: missing data_offsets")
        begin, end = _usize(o[0], "an offset"), _usize(o[1], "an offset")
        expected = dtype.itemsize
        for s in shape:
            expected *= s
        if end - begin != expected:
            raise _invalid(f"`{name}`: data_offsets [{begin}, {end}] do not hold {expected} bytes")
        tensors.append(TensorInfo(name, dtype, shape, start + begin, start + end))
    at = start
    for t in sorted(tensors, key=lambda t: (t.begin, t.end)):
        if t.begin != at:
            raise _invalid(f"`{t.name}`: data_offsets overlap or leave a gap")
        at = t.end
    if at != file_len:
        raise _invalid("the tensors do not cover the data to the end of the file")
    return tensors, metadata


def read_header(path: str) -> Tuple[List[TensorInfo], Dict[str, str]]:
    """safetensors.rs:274-293: the header of the file at `path`, read with ordinary reads (nothing is mapped)."""
    file_len = os.path.getsize(path)
    with open(path, "rb") as f:
        size = f.read(8)
        if len(size) != 8:
            raise InvalidArgument(f"{path}: safetensors: the file is shorter than its 8-byte header size")
        n = int.from_bytes(size, "little")
        if n > MAX_HEADER or 8 + n > file_len:
            raise InvalidArgument(f"{path}: safetensors: header larger than the file or 100 MB")
        raw = f.read(n)
    try:
        return parse_header(raw, 8 + n, file_len)
    except InvalidArgument as e:
        raise InvalidArgument(f"{path}: {e}") from None


def load_safetensors(path: str, device: Union[str, torch.device] = "cuda",
                     keep: Optional[Callable[[str], bool]] = None) -> Dict[str, torch.Tensor]:
    """safetensors.rs:471-580 (`load_safetensors`, `load_safetensors_filtered`): the tensors `keep` accepts (all by
    default), each copied once from the mapped file into a fresh buffer on `device`.  The bytes travel as bytes and
    are typed on the device, so files whose data is not aligned for its element type (as MLX writes them) load the
    same way."""
    tensors, _ = read_header(path)
    device = torch.device(device)
    out: Dict[str, torch.Tensor] = {}
    wanted = [t for t in tensors if keep is None or keep(t.name)]
    if not wanted:
        return out
    with open(path, "rb") as f:
        # a private mapping: nothing is written, and the buffer protocol hands torch a writable view without a copy
        mapped = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_COPY)
    try:
        for t in wanted:
            n = t.end - t.begin
            if n == 0:
                out[t.name] = torch.empty(t.shape, dtype=t.dtype, device=device)
                continue
            raw = torch.frombuffer(mapped, dtype=torch.uint8, count=n, offset=t.begin)
            moved = raw.to(device) if device.type != "cpu" else raw.clone()
            out[t.name] = moved.view(t.dtype).reshape(t.shape)
            del raw
    finally:
        try:
            mapped.close()
        except BufferError:  # a view still alive somewhere: the mapping goes with it
            pass
    return out


@dataclass(frozen=True)
class LayerQuant:
    """config.rs:49-60: a layer's settings (`None`: kept in full precision, mlx-lm's `false`) and whether it is an
    NVFP4 switch layer with one global scale per expert."""
    path: str
    quant: Optional[Quant]
    global_scale: bool = False


@dataclass(frozen=True)
class Quantization:
    """config.rs:17-28: the default settings and the layers the config names."""
    default: Quant
    layers: Tuple[LayerQuant, ...] = field(default_factory=tuple)
    packed: Optional[str] = None  # formats.AWQ / GPTQ_V1 / GPTQ_V2 for Hugging Face packings

    def for_layer(self, path: str) -> Optional[LayerQuant]:
        for layer in self.layers:
            if layer.path == path:
                return layer
        return None

    @staticmethod
    def from_config(config: dict) -> Optional["Quantization"]:
        """config.rs:848-856, 1038-1110: the `quantization` entry (MLX's), else a Hugging Face `quantization_config`
        (config.rs:1111-1190).  None when the checkpoint is not quantized."""
        q = config.get("quantization")
        if q is None:
            hf = config.get("quantization_config")
            if hf is None and isinstance(config.get("text_config"), dict):
                hf = config["text_config"].get("quantization_config")
            model_type = config.get("model_type") if isinstance(config.get("model_type"), str) else ""
            return _hf_quantization(hf, model_type)
        if not isinstance(q, dict) or not any(k in q for k in ("group_size", "bits", "mode")):
            raise InvalidArgument("quantization needs `group_size` and `bits` (or a `mode`)")
        default = _settings(q)
        layers = []
        for path, v in q.items():
            if not (isinstance(v, dict) or v is False):
                continue
            # under the text model's names, as the loader renames weights
            if path.startswith("model.language_model."):
                path = "model." + path[len("model.language_model."):]
            elif path.startswith("language_model."):
                path = path[len("language_model."):]
            layers.append(LayerQuant(path, None if v is False else _settings(v),
                                     isinstance(v, dict) and v.get("global_scale") is True))
        return Quantization(default, tuple(layers))


def _int(what: str, v) -> int:
    if isinstance(v, bool) or not isinstance(v, int):
        raise InvalidArgument(f"{what} must be an integer")
    return v


def _settings(j: dict) -> Quant:
    """config.rs:1047-1068: a mode (affine by default), then its group size and bits (the mode's defaults when
    absent); the combination is checked by the operations."""
    mode = j.get("mode")
    if mode is None:
        mode = QuantMode.AFFINE
    else:
        try:
            mode = QuantMode.parse(mode) if isinstance(mode, str) else None
        except InvalidArgument:
            mode = None
        if mode is None:
            raise InvalidArgument(f"unsupported quantization mode {j.get('mode')!r}")
    quant = Quant.new(mode)
    group, bits = quant.group_size, quant.bits
    if "group_size" in j:
        group = _int("quantization.group_size", j["group_size"])
    if "bits" in j:
        bits = _int("quantization.bits", j["bits"])
    if group < 1 or not 1 <= bits <= 8:
        raise InvalidArgument(f"quantization: group size {group} and {bits} bits (a group size of at least 1, 1 to 8 bits)")
    return Quant(mode, group, bits)


def _hf_quantization(hf: Optional[dict], model_type: str = "") -> Optional[Quantization]:
    """config.rs:1111-1190: a Hugging Face `quantization_config`: AWQ (4-bit, GEMM version) and GPTQ (4 or 8 bits, v1 or
    v2, no activation reordering) become affine settings plus the packing `formats.convert_packed` undoes; gpt-oss's
    own MXFP4 (`*_blocks`, `formats.mxfp4_from_hf_blocks`) is MXFP4; every other method is refused."""
    if hf is None:
        return None
    if not isinstance(hf, dict):
        raise InvalidArgument("quantization_config must be an object")
    method = hf.get("quant_method") if isinstance(hf.get("quant_method"), str) else ""

    def int_or(key: str, default: int) -> int:
        v = hf.get(key)
        if v is None:
            return default
        if isinstance(v, bool) or not isinstance(v, int):
            raise InvalidArgument(f"quantization_config.{key} must be an integer")
        return v

    bits, group = int_or("bits", 4), int_or("group_size", 128)

    def affine(bits: int) -> Quant:
        if group not in (32, 64, 128):
            raise InvalidArgument(f"{method}: group size {group} (MLX's affine kernels take 32, 64 or 128)")
        return Quant.affine(group, bits)

    if method == "awq":
        version = hf.get("version") if isinstance(hf.get("version"), str) else "gemm"
        if version.lower() != "gemm" or bits != 4:
            raise InvalidArgument(f'awq: version "{version}" with {bits} bits (4-bit GEMM checkpoints load)')
        return Quantization(affine(4), (), formats.AWQ)
    if method == "gptq":
        if bits not in (4, 8):
            raise InvalidArgument(f"gptq: {bits} bits (4 and 8 load)")
        if hf.get("desc_act") is True:
            raise InvalidArgument("gptq: activation reordering (`desc_act`) is not supported; use a checkpoint "
                                  "quantized without it")
        v2 = hf.get("checkpoint_format") == "gptq_v2"
        return Quantization(affine(bits), (), formats.GPTQ_V2 if v2 else formats.GPTQ_V1)
    if method == "mxfp4" and model_type == "gpt_oss":
        return Quantization(Quant.new(QuantMode.MXFP4), (), None)
    if method in ("mxfp4", "mxfp8", "fp8", "compressed-tensors", "modelopt"):
        raise InvalidArgument(f"Hugging Face {method} checkpoints are not converted yet; use an MLX conversion "
                              "(mlx_lm.convert, or an mlx-community checkpoint)")
    raise InvalidArgument(f'unsupported quantization method "{method}"')


def infer_quant(weight: torch.Tensor, scales: torch.Tensor, default: Quant) -> Quant:
    """lib.rs:462-479 (mlx-lm's `infer_quant_config`): uint8 scales mean a floating-point mode, told apart by the packed
    words per group (2: nvfp4, 8: mxfp8, else mxfp4); other scales are affine with the config's settings."""
    if scales.dtype != torch.uint8:
        return default if default.mode == QuantMode.AFFINE else Quant.new(QuantMode.AFFINE)
    packed = weight.shape[-1] if weight.ndim else 0
    groups = max(scales.shape[-1] if scales.ndim else 0, 1)
    per = packed // groups
    return Quant.new(QuantMode.NVFP4 if per == 2 else QuantMode.MXFP8 if per == 8 else QuantMode.MXFP4)


def quantized_layers(weights: Dict[str, torch.Tensor], quantization: Optional[Quantization]
                     ) -> Tuple[Dict[str, Quantized], Dict[str, torch.Tensor]]:
    """lib.rs:573-590: every layer `path` with `path.weight` and `path.scales` as a `Quantized` (with `path.biases`
    and `path.global_scale` where the checkpoint has them): a layer the config names takes its entry, any other is
    recognised from its tensors.  Returns the quantized layers by path and the remaining tensors by name."""
    layers: Dict[str, Quantized] = {}
    rest = dict(weights)
    if quantization is None:
        return layers, rest
    for name in sorted(weights):
        if not name.endswith(".scales"):
            continue
        path = name[:-len(".scales")]
        weight = weights.get(f"{path}.weight")
        if weight is None or weight.dtype != torch.uint32:
            continue
        entry = quantization.for_layer(path)
        if entry is not None and entry.quant is None:
            continue  # named as kept in full precision
        quant = entry.quant if entry is not None else infer_quant(weight, weights[name], quantization.default)
        layers[path] = Quantized(weight, weights[name], weights.get(f"{path}.biases"), quant,
                                 weights.get(f"{path}.global_scale"))
        for part in ("weight", "scales", "biases", "global_scale"):
            rest.pop(f"{path}.{part}", None)
    return layers, rest


def load_quantized(directory: str, device: Union[str, torch.device] = "cuda",
                   keep: Optional[Callable[[str], bool]] = None
                   ) -> Tuple[Dict[str, Quantized], Dict[str, torch.Tensor], Optional[Quantization]]:
    """lib.rs:499-590 as far as the quantized path goes: `config.json` and every `model*.safetensors` of `directory`
    read into device memory, Hugging Face packings repacked on the device, the quantized layers assembled.  Returns
    `(layers, other tensors, quantization)`; building a model from them is the caller's."""
    try:
        with open(os.path.join(directory, "config.json"), "r", encoding="utf-8") as f:
            config = json.load(f)
    except (OSError, json.JSONDecodeError) as e:
        raise InvalidArgument(f"{directory}: {e}") from None
    quantization = Quantization.from_config(config)
    try:
        files = sorted(n for n in os.listdir(directory) if n.startswith("model") and n.endswith(".safetensors"))
    except OSError as e:
        raise InvalidArgument(f"{directory}: {e}") from None
    if not files:
        raise InvalidArgument(f"{directory}: no model*.safetensors file")
    weights: Dict[str, torch.Tensor] = {}
    for name in files:
        weights.update(load_safetensors(os.path.join(directory, name), device, keep))
    if quantization is not None and quantization.packed is not None:
        weights = formats.convert_packed(weights, quantization.packed, quantization.default)
    layers, rest = quantized_layers(weights, quantization)
    return layers, rest, quantization
