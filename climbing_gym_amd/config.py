"""Configuration objects of the native LFM2 inference path.

`LFM2Config` keeps the field names and checkpoint normalisation of the reference's model schema
(models/lfm2.py:176-260, models/lfm2_compat.py:8-33) for the fields inference reads;
`LFM25SamplingConfig` is the sampling request of lfm25_engine.py:22-54 with the same validation.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, fields
from pathlib import Path
from typing import Any, Mapping
from ._checks import reject

DEFAULT_LAYER_TYPES = tuple("full_attention" if i in (2, 5, 8, 10, 12, 14) else "conv" for i in range(16))


@dataclass
class LFM2Config:
    vocab_size: int = 65536
    hidden_size: int = 2048
    mlp_hidden_size: int = 8192
    num_hidden_layers: int = 16
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    max_position_embeddings: int = 128000
    rope_theta: float = 1_000_000.0
    norm_eps: float = 1e-5
    conv_kernel_size: int = 3
    conv_bias: bool = False
    layer_types: tuple = DEFAULT_LAYER_TYPES
    tie_embedding: bool = True
    pad_token_id: int = 0
    bos_token_id: int = 1
    eos_token_id: int = 7

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    def validate(self) -> None:
        reject(len(self.layer_types) != self.num_hidden_layers, "len(layer_types) must match num_hidden_layers")
        reject(self.hidden_size % self.num_attention_heads, "hidden_size must be divisible by num_attention_heads")
        reject(self.num_attention_heads % self.num_key_value_heads,
               "num_attention_heads must be divisible by num_key_value_heads")
        reject(self.mlp_hidden_size <= 0 or self.conv_kernel_size <= 0, "mlp_hidden_size and conv_kernel_size must be > 0")
        reject(any(kind not in ("conv", "full_attention") for kind in self.layer_types),
               "layer_types entries must be either 'conv' or 'full_attention'")

    @classmethod
    def from_dict(cls, payload: Mapping[str, Any]) -> "LFM2Config":
        """Accepts this schema as well as Hugging Face LFM2 config.json spellings."""
        data = dict(payload)
        rope = data.get("rope_parameters") or data.get("rope_scaling")
        if rope is not None:
            reject(not isinstance(rope, Mapping), "LFM2 rope_parameters must be an object")
            reject(any(isinstance(v, Mapping) for v in rope.values()), "Unsupported LFM2 per-layer rope_parameters")
            kind = rope.get("rope_type", rope.get("type", "default"))
            reject(kind != "default", f"Unsupported LFM2 rope_type: {kind!r}; expected 'default'")
            if rope.get("rope_theta") is not None:
                data["rope_theta"] = float(rope["rope_theta"])
        if data.get("tie_embedding") is None and data.get("tie_word_embeddings") is not None:
            data["tie_embedding"] = bool(data["tie_word_embeddings"])
        if data.get("mlp_hidden_size") is None:
            data["mlp_hidden_size"] = _mlp_width(data)
        if data.get("conv_kernel_size") is None and data.get("conv_L_cache") is not None:
            data["conv_kernel_size"] = data["conv_L_cache"]
        if data.get("layer_types") is None and data.get("full_attn_idxs") is not None:
            idx = set(data["full_attn_idxs"])
            data["layer_types"] = ["full_attention" if i in idx else "conv" for i in range(int(data["num_hidden_layers"]))]
        if isinstance(data.get("eos_token_id"), (list, tuple)):
            data["eos_token_id"] = int(data["eos_token_id"][0])
        known = {f.name for f in fields(cls)}
        kwargs = {k: (tuple(v) if isinstance(v, list) else v) for k, v in data.items() if k in known and v is not None}
        config = cls(**kwargs)
        config.validate()
        return config

    @classmethod
    def from_pretrained(cls, model_dir) -> "LFM2Config":
        path = Path(model_dir) / "config.json"
        if not path.exists():
            return cls()
        return cls.from_dict(json.loads(path.read_text()))

    def to_dict(self) -> dict:
        return {f.name: (list(v) if isinstance((v := getattr(self, f.name)), tuple) else v) for f in fields(self)}


def _mlp_width(payload: Mapping[str, Any]) -> int:
    """Legacy checkpoints store `intermediate_size` before the 2/3 SwiGLU adjustment (models/lfm2.py:262-279)."""
    size = payload.get("intermediate_size", payload.get("block_ff_dim"))
    if size is None:
        return 8192
    size = int(size)
    if not bool(payload.get("block_auto_adjust_ff_dim", True)):
        return size
    multiple = int(payload.get("block_multiple_of", 256))
    reject(multiple <= 0, "block_multiple_of must be > 0")
    adjusted = int(float(payload.get("block_ffn_dim_multiplier", 1.0)) * int(2 * size / 3))
    return multiple * ((adjusted + multiple - 1) // multiple)


def coerce_config(config: Any) -> LFM2Config:
    if isinstance(config, LFM2Config):
        return config
    reject(config is None, "LFM25 weight synchronization requires a model with an LFM2 config", TypeError)
    to_dict = getattr(config, "to_dict", None)
    reject(not callable(to_dict), "LFM25 weight synchronization requires an LFM2 config exposing to_dict()", TypeError)
    payload = to_dict()
    reject(not isinstance(payload, Mapping), "LFM2 config.to_dict() must return a mapping", TypeError)
    return LFM2Config.from_dict(dict(payload))


@dataclass(frozen=True)
class LFM25SamplingConfig:
    temperature: float = 1.0
    top_k: int = 0
    top_p: float = 1.0
    repetition_penalty: float = 1.0
    max_new_tokens: int = 256
    stop_token_ids: tuple = ()
    return_logprobs: bool = True
    seed: int = 0
    ignore_eos: bool = False
    stop_token_sequences: tuple = ()
    stop_table: Any = None
    behavior_topk: int = 0

    def __post_init__(self) -> None:
        reject(self.temperature < 0, "temperature must be >= 0")
        reject(self.top_k < 0, "top_k must be 0 or positive")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must be in (0, 1]")
        reject(self.repetition_penalty <= 0.0, "repetition_penalty must be > 0")
        reject(self.max_new_tokens <= 0, "max_new_tokens must be > 0")
        reject(type(self.behavior_topk) is not int or not 0 <= self.behavior_topk <= 128,
               "behavior_topk must be an integer between 0 and 128")
        if self.behavior_topk and (not self.return_logprobs or self.temperature != 1.0 or self.top_k
                                   or self.top_p != 1.0 or self.repetition_penalty != 1.0):
            raise ValueError("behavior_topk requires actual full-support temperature-1 logprobs")
        reject(any(not sequence for sequence in self.stop_token_sequences), "Stop token sequences must be nonempty")

    @property
    def filtered(self) -> bool:
        return self.temperature > 0 and (self.top_k > 0 or self.top_p < 1.0)

    @property
    def fixed_length(self) -> bool:
        return (self.ignore_eos and not self.stop_token_ids and not self.stop_token_sequences
                and self.stop_table is None)
