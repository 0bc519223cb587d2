"""Seeded random-init LFM2 checkpoints and prompt batches for tests and benchmarks.

Key names follow the Hugging Face LFM2 schema that the reference packs from
(`lfm25_engine.py:134-223`): every matrix is N(0, std), every norm weight is 1.
"""
from __future__ import annotations

import torch

LFM2_1P2B_LAYER_TYPES = tuple(
    "full_attention" if i in (2, 5, 8, 10, 12, 14) else "conv" for i in range(16))


def random_state_dict(*, hidden, mlp_hidden, layer_types, q_heads, kv_heads, vocab,
                      seed=0, std=0.02, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    head_dim = hidden // q_heads

    def mat(*shape):
        return (torch.randn(*shape, generator=g) * std).to(dtype)

    def ones(n):
        return torch.ones(n, dtype=dtype)

    sd = {"model.embed_tokens.weight": mat(vocab, hidden), "model.embedding_norm.weight": ones(hidden)}
    for i, kind in enumerate(layer_types):
        p = f"model.layers.{i}"
        sd[f"{p}.operator_norm.weight"] = ones(hidden)
        sd[f"{p}.ffn_norm.weight"] = ones(hidden)
        sd[f"{p}.feed_forward.w1.weight"] = mat(mlp_hidden, hidden)
        sd[f"{p}.feed_forward.w3.weight"] = mat(mlp_hidden, hidden)
        sd[f"{p}.feed_forward.w2.weight"] = mat(hidden, mlp_hidden)
        if kind == "full_attention":
            sd[f"{p}.self_attn.q_proj.weight"] = mat(q_heads * head_dim, hidden)
            sd[f"{p}.self_attn.k_proj.weight"] = mat(kv_heads * head_dim, hidden)
            sd[f"{p}.self_attn.v_proj.weight"] = mat(kv_heads * head_dim, hidden)
            sd[f"{p}.self_attn.out_proj.weight"] = mat(hidden, q_heads * head_dim)
            sd[f"{p}.self_attn.q_layernorm.weight"] = ones(head_dim)
            sd[f"{p}.self_attn.k_layernorm.weight"] = ones(head_dim)
        else:
            sd[f"{p}.conv.in_proj.weight"] = mat(3 * hidden, hidden)
            sd[f"{p}.conv.conv.weight"] = mat(hidden, 1, 3)
            sd[f"{p}.conv.out_proj.weight"] = mat(hidden, hidden)
    return sd


def random_prompts(count, low, high, vocab, seed=0):
    """`count` prompts with lengths uniform in [low, high] and uniform token ids."""
    g = torch.Generator().manual_seed(seed)
    lengths = torch.randint(low, high + 1, (count,), generator=g).tolist()
    return [torch.randint(0, vocab, (n,), generator=g).tolist() for n in lengths]


TINY = dict(hidden=256, mlp_hidden=768, layer_types=("conv", "full_attention", "conv", "full_attention"),
            q_heads=4, kv_heads=2, vocab=4096)
LFM2_1P2B = dict(hidden=2048, mlp_hidden=5632, layer_types=LFM2_1P2B_LAYER_TYPES,
                 q_heads=32, kv_heads=8, vocab=65536)
