"""ASCII stop strings as a token-level prefix automaton (inference/text_stops.py of the reference).

The table is built once on the host; on the device a row advances with one lookup per sampled token
(`table[state, token]`: low 16 bits = next state, 65536 set = a stop string just completed).
"""
from __future__ import annotations

import numpy as np
import torch


def trim_after_stop(text: str, stops) -> str:
    """Cut `text` right after the earliest completed stop string (display only; tokens are kept whole)."""
    ends = [at + len(stop) for stop in stops if stop and (at := text.find(stop)) >= 0]
    return text[:min(ends)] if ends else text


def build_stop_table(tokenizer, stops, *, vocab_size=None) -> torch.Tensor:
    if any(not s or not s.isascii() for s in stops):
        raise ValueError('Native text stops must be nonempty ASCII strings')
    states = sorted({''} | {s[:i] for s in stops for i in range(1, len(s))}, key=len)
    if len(states) >= 65536:
        raise ValueError('Too many stop-prefix states')
    vocab = len(tokenizer) if vocab_size is None else int(vocab_size)
    if vocab < len(tokenizer):
        raise ValueError('Model vocabulary must cover the tokenizer vocabulary')
    pieces = [tokenizer.decode([i], skip_special_tokens=False, clean_up_tokenization_spaces=False)
              for i in range(len(tokenizer))]
    pieces += [''] * (vocab - len(pieces))  # padded head ids decode to nothing and keep the state
    by_length = sorted(range(len(states)), key=lambda i: -len(states[i]))
    cache: dict = {}
    table = np.zeros((len(states), vocab), dtype=np.int32)
    for si, prefix in enumerate(states):
        for ti, piece in enumerate(pieces):
            key = (si, piece)
            if key not in cache:
                text = prefix + piece
                nxt = next(i for i in by_length if text.endswith(states[i]))
                cache[key] = nxt + (65536 if any(s in text for s in stops) else 0)
            table[si, ti] = cache[key]
    return torch.from_numpy(table)


def advance_text_stops(table, states, tokens, reasons):
    value = table[states, tokens].long()
    return value & 65535, torch.where((reasons == 0) & (value >= 65536), 2, reasons)
