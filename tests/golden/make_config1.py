"""Writes tests/golden/config1_greedy.json: the CPU-runnable benchmark case (tiny LFM2-style model, seed 0, fp32,
prompts of 7/33/64/120 uniform token ids, 64 greedy tokens).

The values come from this repository's CPU oracle, which tests/test_oracle_model.py pins against
transformers' Lfm2ForCausalLM on random-init weights; before writing, this script re-checks the first greedy token of
every prompt against a full Transformers recompute with the same weights.  Nothing of the reference is imported.

    python tests/golden/make_config1.py
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from climbing_gym_amd.synthetic import TINY, random_state_dict  # noqa: E402
from oracle import lfm2_oracle as O  # noqa: E402


def build():
    cfg = O.OracleConfig(vocab_size=TINY["vocab"], hidden_size=TINY["hidden"], mlp_hidden_size=TINY["mlp_hidden"],
                         num_hidden_layers=len(TINY["layer_types"]), num_attention_heads=TINY["q_heads"],
                         num_key_value_heads=TINY["kv_heads"], max_position_embeddings=512, rope_theta=1e6,
                         layer_types=tuple(TINY["layer_types"]))
    state = random_state_dict(**TINY, seed=0)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, 4096, (n,), generator=g).tolist() for n in (7, 33, 64, 120)]
    return cfg, state, prompts


def transformers_first_tokens(cfg, state, prompts):
    from transformers import Lfm2Config, Lfm2ForCausalLM
    hf = Lfm2Config(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size, intermediate_size=cfg.mlp_hidden_size,
                    num_hidden_layers=cfg.num_hidden_layers, num_attention_heads=cfg.num_attention_heads,
                    num_key_value_heads=cfg.num_key_value_heads, max_position_embeddings=cfg.max_position_embeddings,
                    norm_eps=cfg.norm_eps, rope_theta=cfg.rope_theta, conv_bias=False, conv_L_cache=3,
                    block_auto_adjust_ff_dim=False, layer_types=list(cfg.layer_types), tie_word_embeddings=True)
    model = Lfm2ForCausalLM(hf).eval()
    model.load_state_dict({**state, "lm_head.weight": state["model.embed_tokens.weight"]}, strict=False)
    with torch.inference_mode():
        return [int(model(torch.tensor([p]), use_cache=False).logits[0, -1].argmax()) for p in prompts]


def main():
    cfg, state, prompts = build()
    oracle = O.OracleEngine(cfg, state, torch.float32, max_model_len=256)
    with torch.inference_mode():
        tokens, logprobs, trace = oracle.generate(prompts, 64, temperature=0.0, return_logits=True)
    first = transformers_first_tokens(cfg, state, prompts)
    assert first == tokens[:, 0].tolist(), (first, tokens[:, 0].tolist())
    top2 = [t.topk(2, -1).values for t in trace]
    record = {
        "description": "tiny LFM2-style model, seed 0, fp32 CPU oracle, 64 greedy tokens",
        "prompt_lengths": [len(p) for p in prompts],
        "prompt_heads": [p[:4] for p in prompts],
        "token_ids": tokens.tolist(),
        "logprobs": [[round(float(v), 6) for v in row] for row in logprobs],
        "best_logit": [[round(float(t[r, 0]), 5) for t in top2] for r in range(4)],
        "margin_to_second": [[round(float(t[r, 0] - t[r, 1]), 6) for t in top2] for r in range(4)],
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1_greedy.json")
    with open(path, "w") as f:
        json.dump(record, f)
    print("wrote", path)


if __name__ == "__main__":
    main()
