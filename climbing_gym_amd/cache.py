"""Dense slot cache for KV history and short-conv state (lfm25_engine.py:370-431, 1165-1221).

Layout in HBM (one allocation per tensor, all layers of a kind together):

  bf16 KV : k, v          [attn layers, slots, KV heads, capacity, D]   (each head's history is contiguous:
  e4m3 KV : k, v bytes    [attn layers, slots, KV heads, capacity, D]    128 or 64 B / token, so the decode
            scales fp32   [attn layers, slots, KV heads, capacity]       kernel streams whole DRAM pages)
            exposed through [.., capacity, KV heads, ..] views, the index order of the reference's cache
  conv    : state         [conv layers, slots, H, 3]   (index 2 = newest tap)
  seq_lens: int32 [slots]
"""
from __future__ import annotations

from dataclasses import dataclass

import torch

from . import ops


@dataclass
class LFM25HybridCache:
    k_cache: torch.Tensor
    v_cache: torch.Tensor
    conv_state: torch.Tensor
    seq_lens: torch.Tensor
    k_scales: torch.Tensor | None = None
    v_scales: torch.Tensor | None = None

    @classmethod
    def allocate(cls, *, attn_layers, conv_layers, slots, capacity, kv_heads, head_dim, hidden, kernel, dtype, device,
                 fp8_kv=False):
        conv = torch.zeros((conv_layers, slots, hidden, kernel), device=device, dtype=dtype)
        lens = torch.zeros(slots, device=device, dtype=torch.int32)
        if fp8_kv:
            shape = (attn_layers, slots, kv_heads, capacity)
            make = lambda: torch.zeros((*shape, head_dim), device=device, dtype=torch.float8_e4m3fn).permute(0, 1, 3, 2, 4)
            scale = lambda: torch.zeros(shape, device=device, dtype=torch.float32).permute(0, 1, 3, 2)
            return cls(make(), make(), conv, lens, scale(), scale())
        make = lambda: torch.zeros((attn_layers, slots, kv_heads, capacity, head_dim), device=device, dtype=dtype).permute(0, 1, 3, 2, 4)
        return cls(make(), make(), conv, lens)

    def rows(self, start: int, end: int) -> "LFM25HybridCache":
        cut = lambda t: None if t is None else t[:, start:end]
        return LFM25HybridCache(cut(self.k_cache), cut(self.v_cache), cut(self.conv_state), self.seq_lens[start:end],
                                cut(self.k_scales), cut(self.v_scales))

    @property
    def max_slots(self) -> int:
        return int(self.seq_lens.numel())

    @property
    def max_seq_len(self) -> int:
        return int(self.k_cache.size(2))

    @property
    def fp8(self) -> bool:
        return self.k_scales is not None

    def store_prefill(self, layer: int, k: torch.Tensor, v: torch.Tensor, *, start: int = 0) -> None:
        """Write [batch, tokens, KV heads, D] (or one [tokens, KV heads, D]) at positions 0.. of slots start.."""
        keys, values = (k[None], v[None]) if k.ndim == 3 else (k, v)
        rows, span = slice(start, start + keys.size(0)), slice(0, keys.size(1))
        targets = self.k_cache[layer, rows, span], self.v_cache[layer, rows, span]
        if self.fp8:
            ops.store_kv(keys, values, *targets, self.k_scales[layer, rows, span], self.v_scales[layer, rows, span])
        else:
            for target, source in zip(targets, (keys, values)):
                target.copy_(source)

    def copy_prefix_from(self, source: "LFM25HybridCache", slots: torch.Tensor, length: int) -> None:
        """self[i] <- source[slots[i]] for the first `length` positions, conv state and lengths
        (lfm25_engine.py:400-423).  Byte-identical when both caches use the same storage (all layers in one gather per
        tensor); an e4m3 source is dequantised into a model-dtype destination."""
        order = slots.to(self.seq_lens.device, torch.long)
        head = lambda t: _bytes(t[:, :, :length])                     # [layers, slots, positions, ...] as raw bytes
        taken = lambda t: head(t).index_select(1, order)
        mine = [self.k_cache, self.v_cache, self.k_scales, self.v_scales]
        theirs = [source.k_cache, source.v_cache, source.k_scales, source.v_scales]
        if self.fp8 == source.fp8 and self.k_cache.dtype == source.k_cache.dtype:
            for target, origin in zip(mine, theirs):
                if target is not None:
                    head(target).copy_(taken(origin))
        else:
            for layer in range(self.k_cache.size(0)):
                pick = lambda t: t[layer, :, :length].index_select(0, order) if t.element_size() > 1 else \
                    t[layer, :, :length].view(torch.uint8).index_select(0, order).view(t.dtype)
                keys, values = pick(source.k_cache), pick(source.v_cache)
                if source.fp8:
                    keys = (keys.float() * pick(source.k_scales)[..., None]).to(self.conv_state.dtype)
                    values = (values.float() * pick(source.v_scales)[..., None]).to(self.conv_state.dtype)
                self.store_prefill(layer, keys.contiguous(), values.contiguous())
        self.conv_state.copy_(source.conv_state.index_select(1, order))
        self.seq_lens.copy_(source.seq_lens.index_select(0, order))

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in
                   (self.k_cache, self.v_cache, self.conv_state, self.seq_lens, self.k_scales, self.v_scales) if t is not None)


def _bytes(tensor: torch.Tensor) -> torch.Tensor:
    """One-byte element types as uint8, so that gathers and copies move e4m3 codes as they are."""
    return tensor.view(torch.uint8) if tensor.element_size() == 1 else tensor
