"""Model registry: which configuration reader and which model class serve a checkpoint folder, chosen by config.json
("architecture", or the first of "architectures"), and a dependency-free safetensors reader for its weights."""
import json
import mmap
import os
import struct
import warnings
from typing import Dict, Iterator, Tuple

import torch

_ST_DTYPES = {"BF16": torch.bfloat16, "F16": torch.float16, "F32": torch.float32, "F64": torch.float64,
              "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
              "BOOL": torch.bool}


def _llama_config(raw: dict, context_len=None, **_kw):
    from .model_runner import ModelConfig
    ctx = context_len or raw.get("max_position_embeddings", 8192)
    return ModelConfig(raw["hidden_size"], raw["intermediate_size"], raw["num_hidden_layers"], raw["num_attention_heads"],
                       raw.get("num_key_value_heads", raw["num_attention_heads"]), raw["vocab_size"], context_len=ctx,
                       head_dim=raw.get("head_dim"), rms_norm_eps=raw.get("rms_norm_eps", 1e-5),
                       rope_theta=raw.get("rope_theta", 10000.0), rope_scaling=raw.get("rope_scaling"),
                       max_position_embeddings=max(raw.get("max_position_embeddings", 8192), ctx),
                       tie_word_embeddings=raw.get("tie_word_embeddings", False))


def _tizalorn_config(raw: dict, context_len=None, tensor_shapes=None, **_kw):
    from .tizalorn import TizalornConfig
    return TizalornConfig(raw, context_len=context_len or 8192, tensor_shapes=tensor_shapes)


def _sominex_config(raw: dict, context_len=None, tensor_shapes=None, **_kw):
    from .sominex import SominexConfig
    return SominexConfig(raw, context_len=context_len or 8192, tensor_shapes=tensor_shapes)


def _toredra_config(raw: dict, context_len=None, tensor_shapes=None, **_kw):
    from .toredra import ToredraConfig
    return ToredraConfig(raw, context_len=context_len or 8192, tensor_shapes=tensor_shapes)


def _kikurax_config(raw: dict, context_len=None, tensor_shapes=None, **_kw):
    from .kikurax import KikuraxConfig
    return KikuraxConfig(raw, context_len=context_len or 8192, tensor_shapes=tensor_shapes)


def _llama_class():
    from .llama import LlamaForCausalLM
    return LlamaForCausalLM


def _mllama_class():
    from .mllama import MllamaForConditionalGeneration
    return MllamaForConditionalGeneration


def _tizalorn_class():
    from .tizalorn import TizalornForCausalLM
    return TizalornForCausalLM


def _sominex_class():
    from .sominex import SominexForCausalLM
    return SominexForCausalLM


def _toredra_class():
    from .toredra import ToredraForCausalLM
    return ToredraForCausalLM


def _kikurax_class():
    from .kikurax import KikuraxForCausalLM
    return KikuraxForCausalLM


# architecture name -> (configuration from config.json's dict, model class); both lazy so that naming a model does not
# import the others
MODELS = {
    "LlamaForCausalLM": (_llama_config, _llama_class),
    "Tizalorn": (_tizalorn_config, _tizalorn_class),
    "Sominex": (_sominex_config, _sominex_class),
    "Toredra": (_toredra_config, _toredra_class),
    "Kikurax": (_kikurax_config, _kikurax_class),
}


def architecture_of(raw: dict) -> str:
    arch = raw.get("architecture") or (raw.get("architectures") or [None])[0]
    if arch not in MODELS:
        raise ValueError(f"no model class for architecture {arch!r}; known: {sorted(MODELS)}")
    return arch


def load_config(model_dir: str, **kw):
    """the model configuration of a checkpoint folder; tensor shapes of its safetensors files are handed to the reader
    (a design may take sizes from them)"""
    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    shapes = {}
    for path in safetensors_files(model_dir):
        header, _ = _read_header(path)
        shapes.update({k: tuple(v["shape"]) for k, v in header.items() if k != "__metadata__"})
    return MODELS[architecture_of(raw)][0](raw, tensor_shapes=shapes, **kw)


def model_class_for(config):
    """the class ModelRunner instantiates for a configuration object"""
    arch = getattr(config, "architecture", None)
    if arch in MODELS:
        return MODELS[arch][1]()
    if getattr(config, "is_encoder_decoder", False):
        return _mllama_class()
    return _llama_class()


def safetensors_files(model_dir: str):
    return sorted(os.path.join(model_dir, f) for f in os.listdir(model_dir) if f.endswith(".safetensors"))


def _read_header(path: str):
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        return json.loads(f.read(n)), 8 + n


def iter_safetensors(model_dir: str) -> Iterator[Tuple[str, torch.Tensor]]:
    """(name, tensor) of every tensor in the folder's .safetensors files: an 8-byte little-endian header length, a JSON
    header name -> {dtype, shape, data_offsets}, then the data.  Files are memory-mapped; tensors are copies."""
    for path in safetensors_files(model_dir):
        header, base = _read_header(path)
        with open(path, "rb") as f, mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ) as mm:
            for name, info in header.items():
                if name == "__metadata__":
                    continue
                lo, hi = info["data_offsets"]
                dtype = _ST_DTYPES[info["dtype"]]
                if hi == lo:
                    yield name, torch.empty(info["shape"], dtype=dtype)
                    continue
                with warnings.catch_warnings():
                    warnings.simplefilter("ignore", UserWarning)          # (read-only buffer: it is copied right away)
                    flat = torch.frombuffer(mm, dtype=dtype, count=(hi - lo) // dtype.itemsize, offset=base + lo)
                tensor = flat.reshape(info["shape"]).clone()
                del flat
                yield name, tensor


def load_weights(model, model_dir: str) -> None:
    model.load_weights(iter_safetensors(model_dir))
