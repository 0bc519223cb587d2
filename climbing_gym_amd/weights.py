"""Packed LFM2 weights on the GPU (lfm25_engine.py:57-367 of the reference).

Per layer the SwiGLU gate/up matrices are stored as one [2I,H] matrix and q/k/v as one
[(QH+2KH)D,H] matrix so that a decode step needs one GEMM for each; the depthwise conv weight
[H,1,3] is kept as [H,3].  `copy_from_model_` overwrites these buffers in place (graphs captured
over them stay valid) and validates every shape before touching the first one.
"""
from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Any, Mapping

import torch

from .config import LFM2Config, coerce_config
from ._checks import reject

SYNC_FIELDS = ("vocab_size", "hidden_size", "mlp_hidden_size", "num_hidden_layers", "num_attention_heads",
               "num_key_value_heads", "max_position_embeddings", "rope_theta", "norm_eps", "conv_kernel_size",
               "conv_bias", "layer_types", "tie_embedding", "pad_token_id", "bos_token_id", "eos_token_id")


@dataclass(frozen=True)
class LFM25AttentionWeights:
    qkv_weight: torch.Tensor
    out_weight: torch.Tensor
    q_norm_weight: torch.Tensor
    k_norm_weight: torch.Tensor
    cache_index: int


@dataclass(frozen=True)
class LFM25ConvWeights:
    in_weight: torch.Tensor
    conv_weight: torch.Tensor
    out_weight: torch.Tensor
    cache_index: int


@dataclass(frozen=True)
class LFM25LayerWeights:
    operator_norm_weight: torch.Tensor
    ffn_norm_weight: torch.Tensor
    w13_weight: torch.Tensor
    w2_weight: torch.Tensor
    attention: LFM25AttentionWeights | None = None
    conv: LFM25ConvWeights | None = None

    @property
    def is_attention_layer(self) -> bool:
        return self.attention is not None


def lookup(state: Mapping[str, torch.Tensor], key: str) -> torch.Tensor:
    """Checkpoints may or may not carry the `model.` prefix."""
    alt = key[len("model."):] if key.startswith("model.") else f"model.{key}"
    for name in (key, alt):
        value = state.get(name)
        if value is not None:
            return value
    raise KeyError(f"Missing tensor {key!r} in LFM2 checkpoint")


def has(state: Mapping[str, torch.Tensor], key: str) -> bool:
    alt = key[len("model."):] if key.startswith("model.") else f"model.{key}"
    return key in state or alt in state


def _layer_sources(cfg: LFM2Config, index: int, kind: str):
    """(packed attribute path, row range or None, checkpoint key) for every tensor of a layer."""
    p = f"model.layers.{index}"
    I, H = cfg.mlp_hidden_size, cfg.hidden_size
    items = [("operator_norm_weight", None, f"{p}.operator_norm.weight"), ("ffn_norm_weight", None, f"{p}.ffn_norm.weight"),
             ("w13_weight", (0, I), f"{p}.feed_forward.w1.weight"), ("w13_weight", (I, 2 * I), f"{p}.feed_forward.w3.weight"),
             ("w2_weight", None, f"{p}.feed_forward.w2.weight")]
    if kind == "full_attention":
        q = cfg.num_attention_heads * cfg.head_dim
        kv = cfg.num_key_value_heads * cfg.head_dim
        items += [("attention.qkv_weight", (0, q), f"{p}.self_attn.q_proj.weight"),
                  ("attention.qkv_weight", (q, q + kv), f"{p}.self_attn.k_proj.weight"),
                  ("attention.qkv_weight", (q + kv, q + 2 * kv), f"{p}.self_attn.v_proj.weight"),
                  ("attention.out_weight", None, f"{p}.self_attn.out_proj.weight"),
                  ("attention.q_norm_weight", None, f"{p}.self_attn.q_layernorm.weight"),
                  ("attention.k_norm_weight", None, f"{p}.self_attn.k_layernorm.weight")]
    elif kind == "conv":
        items += [("conv.in_weight", None, f"{p}.conv.in_proj.weight"), ("conv.conv_weight", "squeeze", f"{p}.conv.conv.weight"),
                  ("conv.out_weight", None, f"{p}.conv.out_proj.weight")]
    else:
        raise ValueError(f"Unsupported LFM2 layer type: {kind!r}")
    return items


@dataclass(frozen=True)
class LFM25PackedWeights:
    config: LFM2Config
    embed_tokens: torch.Tensor
    embedding_norm_weight: torch.Tensor
    lm_head_weight: torch.Tensor
    layers: tuple
    device: torch.device
    dtype: torch.dtype

    @property
    def num_attention_layers(self) -> int:
        return sum(layer.attention is not None for layer in self.layers)

    @property
    def num_conv_layers(self) -> int:
        return sum(layer.conv is not None for layer in self.layers)

    def linear_matrices(self):
        """Every GEMM weight of the model, in execution order of a decode step."""
        for layer in self.layers:
            if layer.attention is not None:
                yield layer.attention.qkv_weight
                yield layer.attention.out_weight
            else:
                yield layer.conv.in_weight
                yield layer.conv.out_weight
            yield layer.w13_weight
            yield layer.w2_weight
        yield self.lm_head_weight

    @classmethod
    def from_state_dict(cls, config: LFM2Config, state: Mapping[str, torch.Tensor], *, device, dtype):
        config.validate()
        device = torch.device(device)

        def put(key):
            return lookup(state, key).detach().to(device=device, dtype=dtype).contiguous()

        embed = put("model.embed_tokens.weight")
        head = put("model.lm_head.weight") if has(state, "model.lm_head.weight") else embed
        layers, n_attn, n_conv = [], 0, 0
        for index, kind in enumerate(config.layer_types):
            parts: dict[str, Any] = {}
            for attr, rows, key in _layer_sources(config, index, kind):
                tensor = put(key)
                if rows == "squeeze":
                    reject(tensor.ndim != 3 or tensor.size(1) != 1,
                           f"Expected depthwise conv weight [H,1,K], got {tuple(tensor.shape)}")
                    tensor = tensor[:, 0, :].contiguous()
                parts.setdefault(attr, []).append(tensor)
            packed = {a: (v[0] if len(v) == 1 else torch.cat(v, 0).contiguous()) for a, v in parts.items()}
            common = {k: packed[k] for k in ("operator_norm_weight", "ffn_norm_weight", "w13_weight", "w2_weight")}
            if kind == "full_attention":
                op = LFM25AttentionWeights(packed["attention.qkv_weight"], packed["attention.out_weight"],
                                           packed["attention.q_norm_weight"], packed["attention.k_norm_weight"], n_attn)
                layers.append(LFM25LayerWeights(**common, attention=op))
                n_attn += 1
            else:
                op = LFM25ConvWeights(packed["conv.in_weight"], packed["conv.conv_weight"], packed["conv.out_weight"], n_conv)
                layers.append(LFM25LayerWeights(**common, conv=op))
                n_conv += 1
        return cls(config, embed, put("model.embedding_norm.weight"), head, tuple(layers), device, dtype)

    @classmethod
    def from_model(cls, model: Any, *, device=None, dtype=None):
        first = next(model.parameters())
        return cls.from_state_dict(coerce_config(getattr(model, "config", None)), model.state_dict(),
                                   device=device or first.device, dtype=dtype or first.dtype)

    @classmethod
    def from_pretrained(cls, model_dir, *, device, dtype):
        path = Path(model_dir)
        return cls.from_state_dict(LFM2Config.from_pretrained(path), load_state_dict(path), device=device, dtype=dtype)

    @torch.inference_mode()
    def copy_from_model_(self, model: Any) -> None:
        """In-place policy sync (lfm25_engine.py:225-367): all checks first, then all copies."""
        source_cfg = coerce_config(getattr(model, "config", None))
        source_cfg.validate()
        bad = [f"{f}: engine={getattr(self.config, f)!r}, model={getattr(source_cfg, f)!r}"
               for f in SYNC_FIELDS if getattr(self.config, f) != getattr(source_cfg, f)]
        reject(bad, "Cannot synchronize an incompatible LFM2 config (" + "; ".join(bad) + ")")
        state = model.state_dict()
        reject(not isinstance(state, Mapping),
               "model.state_dict() must return a mapping of tensor names to tensors", TypeError)
        plan = []

        def add(name, destination, source):
            reject(not torch.is_tensor(source), f"LFM25 sync source {name!r} is not a tensor", TypeError)
            if tuple(source.shape) != tuple(destination.shape):
                raise ValueError(f"LFM25 sync shape mismatch for {name!r}: expected {tuple(destination.shape)}, "
                                 f"got {tuple(source.shape)}")
            plan.append((destination, source))

        add("model.embed_tokens.weight", self.embed_tokens, lookup(state, "model.embed_tokens.weight"))
        add("model.embedding_norm.weight", self.embedding_norm_weight, lookup(state, "model.embedding_norm.weight"))
        head_key = "model.lm_head.weight" if has(state, "model.lm_head.weight") else "model.embed_tokens.weight"
        add("model.lm_head.weight", self.lm_head_weight, lookup(state, head_key))
        for index, (kind, layer) in enumerate(zip(source_cfg.layer_types, self.layers, strict=True)):
            reject((kind == "full_attention") != (layer.attention is not None),
                   f"LFM25 packed layer {index} does not match {kind} config")
            for attr, rows, key in _layer_sources(source_cfg, index, kind):
                target = layer
                for part in attr.split("."):
                    target = getattr(target, part)
                source = lookup(state, key)
                if rows == "squeeze":
                    expected = (target.size(0), 1, target.size(1))
                    reject(not torch.is_tensor(source), f"LFM25 sync source {key!r} is not a tensor", TypeError)
                    reject(tuple(source.shape) != expected,
                           f"LFM25 sync shape mismatch for {key!r}: expected {expected}, got {tuple(source.shape)}")
                    plan.append((target, source[:, 0, :]))
                else:
                    add(key, target if rows is None else target[rows[0]:rows[1]], source)
        for destination, source in plan:
            destination.copy_(source.detach())


def load_state_dict(model_dir: Path) -> dict:
    """First *.safetensors file, else a *.pt / *.bin payload (optionally wrapped in state_dict/model)."""
    shards = sorted(model_dir.glob("*.safetensors"))
    if shards:
        from safetensors.torch import load_file
        return load_file(shards[0], device="cpu")
    others = sorted(model_dir.glob("*.pt")) or sorted(model_dir.glob("*.bin"))
    if others:
        payload = torch.load(others[0], map_location="cpu", weights_only=True)
        for key in ("state_dict", "model"):
            if isinstance(payload, dict) and isinstance(payload.get(key), dict):
                return payload[key]
        if isinstance(payload, dict):
            return payload
    raise FileNotFoundError(f"No safetensors, .pt, or .bin weights found in: {model_dir}")
