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
        if k.ndim == 3:
            k, v = k.unsqueeze(0), v.unsqueeze(0)
        end, length = start + k.size(0), k.size(1)
        kc, vc = self.k_cache[layer, start:end, :length], self.v_cache[layer, start:end, :length]
        if self.k_scales is None:
            kc.copy_(k)
            vc.copy_(v)
        else:
            ops.store_kv(k, v, kc, vc, self.k_scales[layer, start:end, :length], self.v_scales[layer, start:end, :length])

    def copy_prefix_from(self, source: "LFM25HybridCache", slots: torch.Tensor, length: int) -> None:
        """self[i] <- source[slots[i]] for the first `length` positions, conv state and lengths
        (lfm25_engine.py:400-423).  Byte-identical when both caches use the same storage; an e4m3 source is
        dequantised into a model-dtype destination."""
        same = self.k_cache.dtype == source.k_cache.dtype and self.fp8 == source.fp8
        slots = slots.to(self.seq_lens.device, torch.long)
        for layer in range(self.k_cache.size(0)):
            def pick(t):
                part = t[layer, :, :length]
                if part.element_size() == 1:
                    return part.view(torch.uint8).index_select(0, slots).view(part.dtype)
                return part.index_select(0, slots)
            k, v = pick(source.k_cache), pick(source.v_cache)
            if same:
                if k.element_size() == 1:
                    self.k_cache[layer, :, :length].view(torch.uint8).copy_(k.view(torch.uint8))
                    self.v_cache[layer, :, :length].view(torch.uint8).copy_(v.view(torch.uint8))
                else:
                    self.k_cache[layer, :, :length].copy_(k)
                    self.v_cache[layer, :, :length].copy_(v)
                if source.fp8:
                    self.k_scales[layer, :, :length].copy_(pick(source.k_scales))
                    self.v_scales[layer, :, :length].copy_(pick(source.v_scales))
                continue
            if source.fp8:
                k = (k.float() * pick(source.k_scales)[..., None]).to(self.conv_state.dtype)
                v = (v.float() * pick(source.v_scales)[..., None]).to(self.conv_state.dtype)
            self.store_prefill(layer, k.contiguous(), v.contiguous())
        self.conv_state.copy_(source.conv_state.index_select(1, slots))
        self.seq_lens.copy_(source.seq_lens.index_select(0, slots))

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in
                   (self.k_cache, self.v_cache, self.conv_state, self.seq_lens, self.k_scales, self.v_scales) if t is not None)
