"""Token engine of the native LFM2 path on MI355X: prefill, fork, decode step, generate.

Public surface and argument meaning follow the reference's `LFM25Engine`
(lfm25_engine.py:479-1163); the arithmetic runs in this package's HIP kernels.  Two things differ
by design and do not change results beyond GEMM rounding:

* prefill runs a *packed* (varlen) batch through the same fused kernels as decode instead of a
  right-padded batch through eager torch ops; `max_prefill_tokens` (lfm25_engine.py:646-665) bounds the real
  tokens of a chunk, since a packed chunk has no padding to count, and the prompts of a chunk need not be
  neighbours (each has its own cache slot and logits row);
* the engine only exists on the GPU in bf16: there is no eager CPU path in this package.
"""
from __future__ import annotations

import bisect
import itertools
import math
from dataclasses import dataclass
from typing import Any, Sequence

import numpy as np
import torch

from . import ops
from .cache import LFM25HybridCache
from .config import LFM2Config, LFM25SamplingConfig
from .weights import LFM25PackedWeights
from ._checks import reject

MAX_PACKED_TOKENS = 32768  # grid limit of the packed prefill kernels per launch


@dataclass(frozen=True)
class LFM25PrefixBatch:
    cache: LFM25HybridCache
    next_token_logits: torch.Tensor
    prompt_lengths: torch.Tensor
    input_ids: torch.Tensor

    @property
    def batch_size(self) -> int:
        return int(self.prompt_lengths.numel())


@dataclass
class LFM25DecodeBatch:
    cache: LFM25HybridCache
    active_slot_ids: torch.Tensor
    prompt_indices: torch.Tensor
    repeat_indices: torch.Tensor
    alive: torch.Tensor

    @property
    def batch_size(self) -> int:
        return int(self.prompt_indices.numel())


@dataclass(frozen=True)
class LFM25StepOutput:
    token_ids: torch.Tensor
    raw_logprobs: torch.Tensor | None
    sampling_logprobs: torch.Tensor | None
    finished: torch.Tensor
    finish_reasons: torch.Tensor
    logits: torch.Tensor


@dataclass(frozen=True)
class LFM25GenerationOutput:
    token_ids: torch.Tensor
    lengths: torch.Tensor
    logprobs: torch.Tensor | None
    finish_reasons: torch.Tensor
    topk_token_ids: torch.Tensor | None = None
    topk_logprobs: torch.Tensor | None = None


def plan_prefill_chunks(lengths: Sequence[int], budget: int):
    """The reference's planner for right-padded chunks: contiguous groups (start, end, padded width) with
    (count * longest) <= budget; a group always takes its first prompt (lfm25_engine.py:646-665).  This engine packs
    its chunks and plans them with `plan_packed_chunks`; the padded rule is kept for callers that size padded batches."""
    groups, start, total = [], 0, len(lengths)
    while start < total:
        end, width = start, 0
        while end < total:
            widest = max(width, lengths[end])
            if end > start and (end - start + 1) * widest > budget:
                break
            width, end = widest, end + 1
        groups.append((start, end, width))
        start = end
    return groups


def plan_packed_chunks(lengths: Sequence[int], budget: int):
    """Contiguous groups (start, end) of whole prompts whose token counts add up to at most `budget`; a group always
    takes its first prompt.  A packed (varlen) chunk carries no padding, so the budget of lfm25_engine.py:646-665 is
    spent on real tokens: with prompts of 256 to 2048 tokens a 4096-token chunk holds about 3500 instead of 2660."""
    groups, start, total = [], 0, len(lengths)
    while start < total:
        end, used = start + 1, lengths[start]
        while end < total and used + lengths[end] <= budget:
            used += lengths[end]
            end += 1
        groups.append((start, end))
        start = end
    return groups


def plan_packed_bins(lengths: Sequence[int], budget: int):
    """Groups of whole prompts in any order whose token counts add up to at most `budget` (best fit, longest prompt
    first: a prompt goes to the group with the least room that still holds it); a prompt longer than the budget gets a
    group of its own.  Every prompt has its own cache slot and its own row of the logits, and a packed chunk computes
    each sequence by itself, so which prompts share a chunk changes no result, only how full the chunks are: 256
    prompts of 256 to 2048 tokens fill 72 chunks of 4096 to 98 % instead of 84 contiguous ones to 84 %.  Each group
    lists its prompts in their original order."""
    groups, room = [], []   # prompt indices per group; (tokens left, group) sorted by tokens left
    for index in sorted(range(len(lengths)), key=lambda i: (-lengths[i], i)):
        need = lengths[index]
        at = bisect.bisect_left(room, (need, -1))
        if at < len(room):
            left, group = room.pop(at)
        else:
            left, group = budget, len(groups)
            groups.append([])
        groups[group].append(index)
        if left - need > 0:
            bisect.insort(room, (left - need, group))
    return [sorted(group) for group in groups]


def flatten_token_batches(input_ids: Sequence[Sequence[int]], *, device=None):
    """Python prompts -> (flat ids int64, cu_seqlens int32, longest) (lfm25_engine.py:1799-1811)."""
    reject(not input_ids, "input_ids must contain at least one prompt")
    lengths = [len(p) for p in input_ids]
    reject(any(n <= 0 for n in lengths), "empty prompts are not supported")
    device = torch.device(device or "cpu")
    # one pass in C over the concatenated prompts (a Python list comprehension over a few hundred thousand ids is a
    # visible share of an admission)
    total = sum(lengths)
    flat = torch.from_numpy(np.fromiter(itertools.chain.from_iterable(input_ids), dtype=np.int64, count=total)).to(device)
    cu_host = torch.zeros(len(lengths) + 1, dtype=torch.int32)
    cu_host[1:] = torch.tensor(lengths, dtype=torch.int32).cumsum(0)
    return flat, cu_host.to(device), max(lengths)


class LFM25Engine:
    def __init__(self, weights: LFM25PackedWeights, *, max_model_len: int | None = None) -> None:
        reject(weights.device.type != "cuda", "this engine runs on the GPU only; weights must live on a HIP device")
        reject(weights.dtype != torch.bfloat16, "this engine computes in bfloat16")
        cfg = weights.config
        reject(cfg.conv_kernel_size != 3 or cfg.conv_bias, "the short-conv kernels need bias-free convolutions of width 3")
        reject(cfg.head_dim not in (32, 64, 128), "head_dim must be one of {32, 64, 128}")
        self.weights, self.config = weights, cfg
        self.device, self.dtype = weights.device, weights.dtype
        self.max_model_len = int(max_model_len or min(int(cfg.max_position_embeddings), 32768))
        reject(self.max_model_len <= 0, "max_model_len must be > 0")
        reject(self.max_model_len > int(cfg.max_position_embeddings),
               "max_model_len cannot exceed config.max_position_embeddings")
        self._scaling = cfg.head_dim ** -0.5
        self._cuda_decoder = None
        self._step_probe = None   # measurement hook of the decode step, see LFM25HIPDecoder.capture_probed_step
        self.policy_version = 0
        self.last_prefill: dict = {}   # chunk count, tokens and fill of the latest prefill() call
        # fp32 rotary tables [max_model_len, D/2] (lfm25_engine.py:1004-1012)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, cfg.head_dim, 2, dtype=torch.float32, device=self.device) / cfg.head_dim))
        angles = torch.arange(self.max_model_len, dtype=torch.float32, device=self.device)[:, None] * inv[None, :]
        self._rope_cos, self._rope_sin = angles.cos().contiguous(), angles.sin().contiguous()

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_state_dict(cls, config: LFM2Config, state, *, device="cuda", dtype=torch.bfloat16, max_model_len=None):
        return cls(LFM25PackedWeights.from_state_dict(config, state, device=torch.device(device), dtype=dtype),
                   max_model_len=max_model_len)

    @classmethod
    def from_model(cls, model: Any, *, device=None, dtype=None, max_model_len=None):
        first = next(model.parameters())
        return cls(LFM25PackedWeights.from_model(model, device=torch.device(device or first.device),
                                                 dtype=_resolve_dtype(dtype or first.dtype)), max_model_len=max_model_len)

    @classmethod
    def from_pretrained(cls, model_dir, *, device=None, dtype=None, max_model_len=None):
        return cls(LFM25PackedWeights.from_pretrained(model_dir, device=torch.device(device or "cuda"),
                                                      dtype=_resolve_dtype(dtype)), max_model_len=max_model_len)

    # ------------------------------------------------------------------ lifecycle
    @property
    def _decoder_busy(self) -> bool:
        return self._cuda_decoder is not None and self._cuda_decoder._active_session is not None

    @torch.inference_mode()
    def sync_from_model(self, model: Any, *, drain_timeout: int | float = 300) -> "LFM25Engine":
        """In-place policy sync; captured graphs keep working and see the new weights (lfm25_engine.py:556-578)."""
        timeout = float(drain_timeout)
        reject(not math.isfinite(timeout) or timeout < 0.0, "drain_timeout must be finite and >= 0")
        reject(self._decoder_busy, "Close the native generation session before synchronizing weights", RuntimeError)
        self.weights.copy_from_model_(model)
        if self._cuda_decoder is not None:
            self._cuda_decoder.refresh_weights()
        self.policy_version += 1
        return self

    def enable_cuda_graphs(self, *, max_graphs: int = 2, bf16_weight_packing: bool = True, max_prefill_tokens: int = 4096,
                           fp8_mlp: bool = False, fp8_kv: bool = False, adaptive_batching: bool = False,
                           fp8_lm_head: bool = False, fp8_operators: bool = False, capture: bool = True) -> None:
        """Same switch as the reference (lfm25_engine.py:980-997); graphs are HIP graphs.  `fp8_operators` extends
        W8A8 to the QKV/out and conv in/out projections; `bf16_weight_packing` is accepted and ignored."""
        from .decoder import LFM25HIPDecoder
        reject(self._decoder_busy, "Close the native generation session before reconfiguring CUDA graphs", RuntimeError)
        if self._cuda_decoder is not None:
            self._cuda_decoder.clear()
        self._cuda_decoder = LFM25HIPDecoder(self, max_graphs=max_graphs, max_prefill_tokens=max_prefill_tokens,
                                             fp8_mlp=fp8_mlp, fp8_kv=fp8_kv, adaptive_batching=adaptive_batching,
                                             fp8_lm_head=fp8_lm_head, fp8_operators=fp8_operators, capture=capture)

    enable_hip_graphs = enable_cuda_graphs

    def disable_cuda_graphs(self) -> None:
        if self._cuda_decoder is not None:
            self._cuda_decoder.clear()
        self._cuda_decoder = None

    def compile_decode(self, *, mode: str = "reduce-overhead", fullgraph: bool = False) -> None:
        """The reference compiles its eager decode step with a tracing compiler here (lfm25_engine.py:972-978).  This
        engine has no such step to compile: the same request turns on HIP-graph capture of the kernel sequence."""
        del mode, fullgraph
        if self._cuda_decoder is None:
            self.enable_cuda_graphs()

    def release_inference_buffers(self) -> None:
        decoder = self._cuda_decoder
        if decoder is None:
            return
        reject(decoder._active_session is not None,
               "Close the native generation session before releasing inference buffers", RuntimeError)
        if not (decoder.graphs or decoder.fp8_weights):
            return
        torch.cuda.synchronize(self.device)
        decoder.clear()
        torch.cuda.empty_cache()

    def generation_session(self, *, max_batch_size: int, max_new_tokens: int, cache_len: int | None = None,
                           behavior_topk: int = 0, profile_timings: bool = False):
        reject(self._cuda_decoder is None, "generation_session requires enable_cuda_graphs()", RuntimeError)
        from .session import LFM25GenerationSession
        return LFM25GenerationSession(self._cuda_decoder, max_batch_size=max_batch_size, max_new_tokens=max_new_tokens,
                                      cache_len=cache_len, behavior_topk=behavior_topk, profile_timings=profile_timings)

    # ------------------------------------------------------------------ cache
    def _empty_cache(self, *, max_slots: int, max_seq_len: int, fp8_kv: bool = False) -> LFM25HybridCache:
        reject(max_slots <= 0, "max_slots must be > 0")
        reject(max_seq_len <= 0, "max_seq_len must be > 0")
        reject(max_seq_len > self.max_model_len,
               f"max_seq_len={max_seq_len} exceeds engine max_model_len={self.max_model_len}")
        cfg = self.config
        return LFM25HybridCache.allocate(
            attn_layers=self.weights.num_attention_layers, conv_layers=self.weights.num_conv_layers, slots=max_slots,
            capacity=max_seq_len, kv_heads=cfg.num_key_value_heads, head_dim=cfg.head_dim, hidden=cfg.hidden_size,
            kernel=cfg.conv_kernel_size, dtype=self.dtype, device=self.device, fp8_kv=fp8_kv)

    # ------------------------------------------------------------------ shared layer walk
    def _fp8(self):
        return self._cuda_decoder.fp8_weights if self._cuda_decoder is not None else {}

    def _normed(self, x, norm_weight, residual, weight, fp8):
        """residual-add + RMSNorm in front of the projection `weight`: (projection input, new residual).  The input is
        (e4m3 rows, per-row scales) when the projection has an e4m3 copy, a tensor otherwise."""
        if id(weight) in fp8:
            q, scales, residual = ops.rms_norm_fp8(x, norm_weight, self.config.norm_eps, residual)
            return (q, scales), residual
        if isinstance(x, ops.SplitProduct) and residual is None:
            x = x.materialize()
        return ops.rms_norm(x, norm_weight, self.config.norm_eps, residual)

    def _project(self, normed, weight, fp8, place=None):
        """The projection of what `_normed` returned; `place` (an `ops.RowPlacement`) sends the product's rows into an
        existing buffer."""
        packed = fp8.get(id(weight))
        if packed is not None:
            return packed.linear_quantized(normed[0], normed[1], dtype=self.dtype, place=place)
        return ops.linear(normed, weight, place=place)

    def _norm_linear(self, x, norm_weight, residual, weight, fp8, place=None):
        normed, residual = self._normed(x, norm_weight, residual, weight, fp8)
        return self._project(normed, weight, fp8, place), residual

    def _linear(self, x, weight, fp8, defer_reduce=False):
        """Out projection of an operator; `x` is a tensor or, from a fused producer, (e4m3 rows, scales).  With
        `defer_reduce` a product that the plan splits along K is left to the norm that follows."""
        packed = fp8.get(id(weight))
        if isinstance(x, tuple):
            return packed.linear_quantized(x[0], x[1], dtype=self.dtype, defer_reduce=defer_reduce)
        return packed.linear(x) if packed is not None else ops.linear(x, weight, defer_reduce=defer_reduce)

    def _backbone(self, tokens, attention_op, conv_op, fp8, *, defer_reduce=False, projecting_attention_op=None,
                  projecting_conv_op=None):
        """Embedding and all layers with the fused residual chain of lfm25_cuda.py:134-184: every RMSNorm also adds
        the previous block's output into the running residual; the first norm, which has nothing to add, runs in the
        launch that gathers the embedding rows.  Returns (last MLP output, residual).  With `defer_reduce` (decode) a
        split-K down projection hands its partial sums to the next norm.  `projecting_attention_op(op, packed, rows_q,
        row_scales)` (decode), when it takes the layer (returns something), runs the W8A8 QKV projection itself, with the
        head preparation and the KV append as the product's epilogue; `projecting_conv_op(op, normed)` likewise runs the conv
        in-projection with the short-conv update as its epilogue."""
        layers = self.weights.layers
        if not layers:
            return ops.embedding(tokens, self.weights.embed_tokens), None
        operator_weight = lambda layer: layer.attention.qkv_weight if layer.attention is not None else layer.conv.in_weight
        normed, residual = ops.embedding_rms_norm(tokens, self.weights.embed_tokens, layers[0].operator_norm_weight,
                                                  self.config.norm_eps, fp8=id(operator_weight(layers[0])) in fp8)
        hidden = None
        for index, layer in enumerate(layers):
            if index:
                normed, residual = self._normed(hidden, layer.operator_norm_weight, residual, operator_weight(layer), fp8)
            if layer.attention is not None:
                op = layer.attention
                packed = fp8.get(id(op.qkv_weight))
                attended = None
                if projecting_attention_op is not None and packed is not None:
                    attended = projecting_attention_op(op, packed, normed[0], normed[1])
                if attended is None:   # no fused projection for this shape: the plain one, then the head preparation
                    attended = attention_op(op, self._project(normed, op.qkv_weight, fp8))
                mixed = self._linear(attended, op.out_weight, fp8, defer_reduce)
            else:
                op = layer.conv
                gated = projecting_conv_op(op, normed) if projecting_conv_op is not None else None
                if gated is None:   # no fused projection for this shape: the plain one, then the conv launch
                    gated = conv_op(op, self._project(normed, op.in_weight, fp8))
                mixed = self._linear(gated, op.out_weight, fp8, defer_reduce)
            # gate+up projection and SwiGLU: one launch where the product's shape has the fused form (packed prefill
            # chunks), the projection and the SwiGLU launch otherwise (decode); the same bits either way
            normed, residual = self._normed(mixed, layer.ffn_norm_weight, residual, layer.w13_weight, fp8)
            gate_up, down = fp8.get(id(layer.w13_weight)), fp8.get(id(layer.w2_weight))
            if gate_up is not None and down is not None:
                q, scales = gate_up.linear_swiglu_quantized(normed[0], normed[1], dtype=self.dtype)
                hidden = down.linear_quantized(q, scales, dtype=self.dtype, defer_reduce=defer_reduce)
            elif gate_up is None and down is None:
                hidden = ops.linear(ops.linear_swiglu(normed, layer.w13_weight), layer.w2_weight, defer_reduce=defer_reduce)
            else:   # only one of the two MLP projections has an e4m3 copy
                product = self._project(normed, layer.w13_weight, fp8)
                if down is not None:
                    q, scales = ops.swiglu_fp8(product)
                    hidden = down.linear_quantized(q, scales, dtype=self.dtype, defer_reduce=defer_reduce)
                else:
                    hidden = ops.linear(ops.swiglu(product), layer.w2_weight, defer_reduce=defer_reduce)
        return hidden, residual

    def _head(self, hidden, residual, fp8, place=None):
        """Final norm and the vocabulary projection; with `place` the product's rows land in `place.out`."""
        logits, _ = self._norm_linear(hidden, self.weights.embedding_norm_weight, residual, self.weights.lm_head_weight, fp8,
                                      place)
        return logits

    # ------------------------------------------------------------------ decode step (one token per row)
    def _decode_forward(self, cache: LFM25HybridCache, tokens, active=None, *, slot_ids=None, positions=None, fp8=None,
                        logits_out=None, gather=None):
        """One token for every row (lfm25_cuda.py:128-192).  Rows index cache slots directly, or through `slot_ids`
        (then `positions` are the rows' lengths and -1 marks padding).  With `logits_out` ([slots, vocab]) the head
        projection writes the live rows' logits there (row -> its slot) and the other rows keep theirs: the
        `_scatter_logits` step of lfm25_batching.py:99-101 without a copy."""
        cfg = self.config
        fp8 = self._fp8() if fp8 is None else fp8
        rows = tokens.numel()
        # The attention layers of one step see the same lengths: the work list of the attention kernel is built once.
        # When the step owns its rows' bookkeeping (rows are the cache's slots, or a compact batch gathered from them:
        # `gather` = (the slots' input tokens, the slots' activity flags)) the same launch snapshots the positions,
        # gathers the inputs and advances the lengths; otherwise the caller's positions are used and the lengths are
        # advanced at the end.
        advance_after = False
        if positions is None:
            positions, schedule = ops.decode_begin(cache.seq_lens, active, capacity=cache.max_seq_len)
        elif gather is not None:
            positions, schedule = ops.decode_begin(cache.seq_lens, capacity=cache.max_seq_len,
                                                   gather=(gather[0], gather[1], slot_ids, tokens, positions, active))
        else:
            schedule = ops.decode_schedule(positions, active, slot_ids, capacity=cache.max_seq_len)
            advance_after = True

        probe = self._step_probe

        def attend(i, q, k_scales, v_scales, quantized):
            # `probe(kind, index, phase)`, when a measurement asks for it, brackets the call on the launch stream
            if probe is not None:
                probe("attention", i, 0)
            out = ops.attend(q, cache.k_cache[i], cache.v_cache[i], k_scales, v_scales, positions, active=active,
                             scale=self._scaling, slot_ids=slot_ids, schedule=schedule, quantized=quantized)
            if probe is not None:
                probe("attention", i, 1)
            return out

        def attention_op(op, qkv):
            # QK norm + RoPE with the new token's keys and values written straight into the cache, then attention over
            # [0, position]; rows come back already quantised when the out projection is W8A8
            i = op.cache_index
            k_scales = cache.k_scales[i] if cache.fp8 else None
            v_scales = cache.v_scales[i] if cache.fp8 else None
            q = ops.prepare_qkv_store(qkv, op.q_norm_weight, op.k_norm_weight, self._rope_cos, self._rope_sin, positions,
                                      cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.norm_eps,
                                      cache.k_cache[i], cache.v_cache[i], k_scales, v_scales, active=active,
                                      slot_ids=slot_ids)
            quantized = (id(op.out_weight) in fp8
                         and -(-cfg.num_attention_heads // 16) * -(-cfg.head_dim // 64) <= 4)  # the fused combine's row limit
            out = attend(i, q, k_scales, v_scales, quantized)
            return out if quantized else out.view(rows, -1)

        def conv_op(op, bcx):
            state = cache.conv_state[op.cache_index]
            if id(op.out_weight) in fp8 and op.conv_weight.size(0) <= 4096 and op.conv_weight.size(0) % 8 == 0:
                return ops.conv_update_fp8(bcx, op.conv_weight, state, active, slot_ids)
            return ops.conv_update(bcx, op.conv_weight, state, active, slot_ids)

        def projecting_attention_op(op, packed, rows_q, row_scales):
            i = op.cache_index
            if not ops.qkv_project_store_supported(packed, cfg.head_dim, self.dtype, cache.k_cache[i]):
                return None
            k_scales = cache.k_scales[i] if cache.fp8 else None
            v_scales = cache.v_scales[i] if cache.fp8 else None
            q = ops.qkv_project_store(rows_q, row_scales, packed, op.q_norm_weight, op.k_norm_weight, self._rope_cos,
                                      self._rope_sin, positions, cfg.num_attention_heads, cfg.num_key_value_heads,
                                      cfg.head_dim, cfg.norm_eps, cache.k_cache[i], cache.v_cache[i], k_scales, v_scales,
                                      active=active, slot_ids=slot_ids)
            quantized = (id(op.out_weight) in fp8
                         and -(-cfg.num_attention_heads // 16) * -(-cfg.head_dim // 64) <= 4)
            out = attend(i, q, k_scales, v_scales, quantized)
            return out if quantized else out.view(rows, -1)

        def projecting_conv_op(op, normed):
            # With a W8A8 out projection the conv launch that also quantises its rows is as fast as this form plus a
            # quantise launch (1.5438 against 1.5454 ms per step), so the fused projection serves the model-dtype path,
            # where it removes a launch per conv layer (all-bf16 step 2.178 -> 2.150 ms).
            if id(op.out_weight) in fp8:
                return None
            state = cache.conv_state[op.cache_index]
            packed = fp8.get(id(op.in_weight))
            if packed is not None:
                return packed.linear_conv_update(normed[0], normed[1], op.conv_weight, state, active, slot_ids, dtype=self.dtype)
            return ops.linear_conv_update(normed, op.in_weight, op.conv_weight, state, active, slot_ids)

        hidden, residual = self._backbone(tokens, attention_op, conv_op, fp8, defer_reduce=True,
                                          projecting_attention_op=projecting_attention_op, projecting_conv_op=projecting_conv_op)
        place = None if logits_out is None else ops.RowPlacement(logits_out, slot_ids, active)
        logits = self._head(hidden, residual, fp8, place)
        if advance_after:
            ops.advance_positions(cache.seq_lens, positions, slot_ids, active)
        return logits

    # ------------------------------------------------------------------ prefill
    def _prefill_packed(self, cache: LFM25HybridCache, tokens, lengths: Sequence[int], fp8, lengths_device, slots, logits_out):
        """Forward a packed batch of whole prompts; sequence i goes to cache slot `slots[i]` (int32 on the device) and
        its next-token logits to row `slots[i]` of `logits_out`.  `lengths_device` holds the same numbers as `lengths`
        on the device: a caller with many chunks copies all lengths once, because a host-to-device copy per chunk waits
        for the stream and stops the host from running ahead of the GPU."""
        cfg = self.config
        count, total, longest = len(lengths), int(sum(lengths)), int(max(lengths))
        reject(longest > cache.max_seq_len, "cache capacity exceeded", RuntimeError)
        reject(longest > self.max_model_len, "position exceeds engine max_model_len", RuntimeError)
        cu = torch.zeros(count + 1, device=self.device, dtype=torch.int32)
        cu[1:] = lengths_device.cumsum(0)
        seq_of_token, positions = ops.build_token_map(cu, total)

        def attention_op(op, qkv):
            q, k, v = ops.prepare_qkv(qkv, op.q_norm_weight, op.k_norm_weight, self._rope_cos, self._rope_sin, positions,
                                      cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.norm_eps)
            i = op.cache_index
            q, k, v = q.view(total, -1, cfg.head_dim), k.view(total, -1, cfg.head_dim), v.view(total, -1, cfg.head_dim)
            ops.store_kv_packed(k, v, cache.k_cache[i], cache.v_cache[i],
                                None if cache.k_scales is None else cache.k_scales[i],
                                None if cache.v_scales is None else cache.v_scales[i], cu, seq_of_token, slots)
            return ops.prefill_attention(q, k, v, cu, longest, self._scaling).view(total, -1)

        def conv_op(op, bcx):
            # a W8A8 out projection takes the rows quantised: the conv launch does that itself
            form = ops.conv_prefill_fp8 if id(op.out_weight) in fp8 else ops.conv_prefill
            return form(bcx, op.conv_weight, cache.conv_state[op.cache_index], cu, seq_of_token, slots)

        hidden, residual = self._backbone(tokens, attention_op, conv_op, fp8)
        last = (cu[1:] - 1).long()
        # the head projection places each sequence's logits in its slot's row of the destination
        self._head(hidden.index_select(0, last), residual.index_select(0, last), fp8, ops.RowPlacement(logits_out, slots))
        cache.seq_lens.index_copy_(0, slots.long(), lengths_device)

    @torch.inference_mode()
    def prefill(self, input_ids, cu_seqlens, max_seqlen: int, *, max_cache_len: int | None = None,
                cache: LFM25HybridCache | None = None, max_prefill_tokens: int | None = None,
                logits_buffer: torch.Tensor | None = None, slots: Sequence[int] | None = None) -> LFM25PrefixBatch:
        """Prefill whole prompts (lfm25_engine.py:605-684) as packed chunks of at most `max_prefill_tokens` real tokens.
        Without `slots`, prompt i fills cache slot i of a cache with exactly that many slots, as in the reference.
        With `slots` (distinct slot indices, one per prompt) the prompts go to those slots of a larger cache and their
        logits to the same rows of `logits_buffer` ([cache slots, vocab]); the other slots are not touched."""
        input_ids = input_ids.to(device=self.device, dtype=torch.long).reshape(-1)
        bounds = cu_seqlens.to(device="cpu", dtype=torch.long).reshape(-1)
        reject(bounds.numel() < 2, "cu_seqlens must contain at least [0, total_tokens]")
        reject(int(bounds[0]) != 0, "cu_seqlens must start at 0")
        reject(int(bounds[-1]) != int(input_ids.numel()), "cu_seqlens[-1] must equal input_ids.numel()")
        offsets = bounds.tolist()
        lengths = [b - a for a, b in zip(offsets[:-1], offsets[1:])]
        reject(min(lengths) <= 0, "empty prompts are not supported")
        reject(max(lengths) > int(max_seqlen), "max_seqlen is smaller than at least one prompt")
        reject(max_prefill_tokens is not None and max_prefill_tokens <= 0, "max_prefill_tokens must be positive")
        count = len(lengths)
        cache_len = int(max_cache_len or max_seqlen)
        if cache is None:
            reject(slots is not None, "slots address an existing cache")
            cache = self._empty_cache(max_slots=count, max_seq_len=cache_len)
        elif cache.max_seq_len < cache_len or (slots is None and cache.max_slots != count):
            raise ValueError("destination cache does not fit the prompt batch")
        if slots is None:
            slot_list = list(range(count))
        else:
            slot_list = [int(slot) for slot in slots]
            reject(len(slot_list) != count or len(set(slot_list)) != count or min(slot_list) < 0 or max(slot_list) >= cache.max_slots,
                   "slots must be distinct cache slots, one per prompt")
        shape = (cache.max_slots, self.config.vocab_size)
        if logits_buffer is None:
            logits_out = torch.empty(shape, device=self.device, dtype=self.dtype)
        else:
            reject(logits_buffer.shape != shape or logits_buffer.dtype != self.dtype or logits_buffer.device != self.weights.embed_tokens.device,
                   "logits buffer must match the prompt batch, vocabulary, device, and model dtype")
            logits_out = logits_buffer
        budget = MAX_PACKED_TOKENS if max_prefill_tokens is None else min(int(max_prefill_tokens), MAX_PACKED_TOKENS)
        fp8 = self._fp8()
        plan = plan_packed_chunks(lengths, budget)
        chunk_tokens, chunk_lengths, chunk_slots, chunk_offsets = input_ids, lengths, slot_list, offsets
        bins = plan_packed_bins(lengths, budget) if len(plan) > 2 else plan
        if len(bins) < len(plan):
            # fuller chunks out of prompts that are not neighbours: the prompts are put in the bins' order once (one
            # gather of the token ids), after which every chunk is a contiguous range again
            order = [index for group in bins for index in group]
            chunk_lengths, chunk_slots = [lengths[i] for i in order], [slot_list[i] for i in order]
            chunk_offsets = [0, *itertools.accumulate(chunk_lengths)]
            # token t of the reordered batch is token t + (where its prompt was) - (where its prompt is now) of the given one
            shift = torch.tensor([offsets[i] for i in order]) - torch.tensor(chunk_offsets[:-1])
            gather = torch.arange(offsets[-1]) + shift.repeat_interleave(torch.tensor(chunk_lengths))
            chunk_tokens = input_ids.index_select(0, gather.to(self.device))
            ends = list(itertools.accumulate(len(group) for group in bins))
            plan = list(zip([0] + ends[:-1], ends))
        # one upload for the whole call: lengths (as given, and in chunk order) and destination slots
        meta = torch.tensor([lengths, chunk_lengths, chunk_slots], dtype=torch.int32).to(self.device)
        lengths_device, chunk_lengths_device, slots_device = meta[0], meta[1], meta[2]
        in_flight = []   # the host stays at most two chunks (a few hundred launches) ahead of the GPU
        for start, end in plan:
            self._prefill_packed(cache, chunk_tokens[chunk_offsets[start]:chunk_offsets[end]], chunk_lengths[start:end], fp8,
                                 chunk_lengths_device[start:end], slots_device[start:end], logits_out)
            marker = torch.cuda.Event()
            marker.record()
            in_flight.append(marker)
            if len(in_flight) > 2:
                in_flight.pop(0).synchronize()
        self.last_prefill = {"chunks": len(plan), "tokens": offsets[-1], "budget": budget,
                             "fill": offsets[-1] / (len(plan) * budget)}
        return LFM25PrefixBatch(cache, logits_out, lengths_device, input_ids)

    # ------------------------------------------------------------------ fork / decode_step
    @torch.inference_mode()
    def fork(self, prefix: LFM25PrefixBatch, repeats: int, *, max_cache_len: int | None = None) -> LFM25DecodeBatch:
        reject(repeats <= 0, "repeats must be > 0")
        prompts = prefix.batch_size
        total = prompts * int(repeats)
        cache_len = int(max_cache_len or prefix.cache.max_seq_len)
        reject(cache_len < prefix.cache.max_seq_len, "max_cache_len cannot be smaller than the prefix cache")
        cache = self._empty_cache(max_slots=total, max_seq_len=cache_len)
        arange = lambda n: torch.arange(n, device=self.device, dtype=torch.long)
        cache.copy_prefix_from(prefix.cache, arange(prompts).repeat_interleave(repeats), prefix.cache.max_seq_len)
        return LFM25DecodeBatch(cache, arange(total), arange(prompts).repeat_interleave(repeats),
                                arange(repeats).repeat(prompts), torch.ones(total, device=self.device, dtype=torch.bool))

    @torch.inference_mode()
    def _append_decode_tokens(self, cache: LFM25HybridCache, slot_ids, input_tokens):
        """Eager decode of one token for the given slots with the reference's capacity checks
        (lfm25_engine.py:1232-1243)."""
        slot_ids = slot_ids.to(device=self.device, dtype=torch.long).reshape(-1)
        input_tokens = input_tokens.to(device=self.device, dtype=torch.long).reshape(-1)
        reject(slot_ids.numel() != input_tokens.numel(), "slot_ids and input_tokens must have matching lengths")
        reject(torch.any(slot_ids < 0) or torch.any(slot_ids >= cache.max_slots),
               "slot_ids contain an out-of-range cache slot")
        positions = cache.seq_lens.index_select(0, slot_ids)
        reject(torch.any(positions >= cache.max_seq_len), "cache capacity exceeded", RuntimeError)
        reject(torch.any(positions >= self.max_model_len), "position exceeds engine max_model_len", RuntimeError)
        active = torch.ones(slot_ids.numel(), device=self.device, dtype=torch.bool)
        return self._decode_forward(cache, input_tokens, active, slot_ids=slot_ids.to(torch.int32), positions=positions.contiguous())

    @torch.inference_mode()
    def decode_step(self, state: LFM25DecodeBatch, input_tokens, sampling: LFM25SamplingConfig | None = None) -> LFM25StepOutput:
        sampling = sampling or LFM25SamplingConfig()
        input_tokens = input_tokens.to(device=self.device, dtype=torch.long).reshape(-1)
        reject(input_tokens.numel() != state.active_slot_ids.numel(), "input_tokens must have one token per active slot")
        logits = self._append_decode_tokens(state.cache, state.active_slot_ids, input_tokens)
        tokens, raw, tempered = self._sample(logits, sampling, step=0, sampling_logprobs=sampling.return_logprobs)
        reasons = self._finish_reasons(tokens, sampling)
        keep = sampling.return_logprobs
        return LFM25StepOutput(tokens, raw if keep else None, tempered if keep else None, reasons != 0, reasons, logits)

    # ------------------------------------------------------------------ sampling helpers
    def _sample(self, logits, sampling: LFM25SamplingConfig, *, step: int, seen_token_mask=None, sampling_logprobs: bool = False):
        """Greedy, a full-support categorical draw, or temperature/top-k/top-p on the device (lfm25_engine.py:1574-1609):
        (tokens, raw log-softmax of the draw, its log-probability under the tempered and filtered distribution that was
        sampled from — None unless `sampling_logprobs`).  A repetition penalty is applied to an fp32 copy first."""
        if seen_token_mask is not None and sampling.repetition_penalty != 1.0:
            lf = logits.float()
            penalised = torch.where(lf < 0, lf * sampling.repetition_penalty, lf / sampling.repetition_penalty)
            logits = torch.where(seen_token_mask, penalised, lf)
        tempered = torch.empty(logits.size(0), device=logits.device, dtype=torch.float32) if sampling_logprobs else None
        if sampling.filtered:
            tokens, raw = ops.sample_filtered(logits, temperature=sampling.temperature, top_k=sampling.top_k, top_p=sampling.top_p,
                                              seed=sampling.seed, step=step, sampling_logprobs=tempered)
        else:
            tokens, raw = ops.sample_logits(logits, temperature=sampling.temperature, seed=sampling.seed, step=step,
                                            return_logprobs=True, sampling_logprobs=tempered)
        return tokens, raw, tempered

    def _finish_reasons(self, token_ids, sampling: LFM25SamplingConfig):
        reasons = torch.zeros_like(token_ids, dtype=torch.int8)
        if not sampling.ignore_eos:
            reasons[token_ids == int(self.config.eos_token_id)] = 1
        for stop_id in sampling.stop_token_ids:
            reasons[(reasons == 0) & (token_ids == int(stop_id))] = 2
        return reasons

    def _build_seen_token_mask(self, prefix: LFM25PrefixBatch, repeats: int, sampling: LFM25SamplingConfig):
        if float(sampling.repetition_penalty) == 1.0:
            return None
        mask = torch.zeros((prefix.batch_size * repeats, self.config.vocab_size), device=self.device, dtype=torch.bool)
        bounds = [0, *prefix.prompt_lengths.long().cumsum(0).tolist()]
        for i, (a, b) in enumerate(zip(bounds[:-1], bounds[1:])):
            mask[i * repeats:(i + 1) * repeats, prefix.input_ids[a:b].unique()] = True
        return mask

    # ------------------------------------------------------------------ generate
    @torch.inference_mode()
    def generate(self, input_ids, cu_seqlens, max_seqlen: int, repeats: int,
                 sampling: LFM25SamplingConfig | None = None) -> LFM25GenerationOutput:
        sampling = sampling or LFM25SamplingConfig()
        if self._cuda_decoder is None:
            # no graphs requested: the same loop with each step launched kernel by kernel
            self.enable_cuda_graphs(capture=False)
        return self._cuda_decoder.generate(input_ids, cu_seqlens, max_seqlen, repeats, sampling)

    @torch.inference_mode()
    def score_completions(self, prompts, completions, *, max_prefill_tokens: int = 4096, head_chunk_size: int = 256):
        """Raw log-probabilities of given completions through the packed prefill kernels (lfm25_engine.py:1108-1163)."""
        reject(len(prompts) != len(completions), 'prompts and completions must have equal lengths')
        reject(max_prefill_tokens <= 0 or head_chunk_size <= 0, 'scoring chunk sizes must be positive')
        reject(any(not p or not c for p, c in zip(prompts, completions)),
               'scoring requires nonempty prompts and completions')
        sequences = [list(p) + list(c) for p, c in zip(prompts, completions)]
        reject(any(len(s) > self.max_model_len for s in sequences), 'scored sequence exceeds max_model_len')
        cfg, fp8 = self.config, self._fp8()
        result = [()] * len(sequences)
        order = sorted(range(len(sequences)), key=lambda i: len(sequences[i]))
        lengths = [len(sequences[i]) for i in order]
        for start, end in plan_packed_chunks(lengths, min(int(max_prefill_tokens), MAX_PACKED_TOKENS)):
            group = order[start:end]
            cache = self._empty_cache(max_slots=len(group), max_seq_len=max(lengths[start:end]))
            tokens = torch.tensor([t for i in group for t in sequences[i]], device=self.device, dtype=torch.long)
            hidden = self._prefill_hidden(cache, tokens, [len(sequences[i]) for i in group], fp8)
            rows, targets, base = [], [], 0
            for i in group:
                rows.extend(range(base + len(prompts[i]) - 1, base + len(sequences[i]) - 1))
                targets.extend(completions[i])
                base += len(sequences[i])
            selected = hidden.index_select(0, torch.tensor(rows, device=self.device))
            target = torch.tensor(targets, device=self.device, dtype=torch.long)
            scores = []
            for off in range(0, target.numel(), head_chunk_size):
                logits = self._linear(selected[off:off + head_chunk_size].contiguous(), self.weights.lm_head_weight, {}).float()
                pick = target[off:off + head_chunk_size]
                scores.append(logits.gather(1, pick[:, None])[:, 0] - torch.logsumexp(logits, -1))
            flat, cursor = torch.cat(scores).cpu().tolist(), 0
            for i in group:
                result[i] = tuple(flat[cursor:cursor + len(completions[i])])
                cursor += len(completions[i])
        return result

    def _prefill_hidden(self, cache, tokens, lengths, fp8):
        """Final-norm hidden states of every packed token (the `return_hidden` form of lfm25_engine.py:1097-1098)."""
        count, total = len(lengths), int(sum(lengths))
        cu_host = torch.zeros(count + 1, dtype=torch.int32)
        cu_host[1:] = torch.tensor(lengths, dtype=torch.int32).cumsum(0)
        cu = cu_host.to(self.device)
        seq_of_token, positions = ops.build_token_map(cu, total)
        slots = torch.arange(count, device=self.device, dtype=torch.int32)
        cfg = self.config

        def attention_op(op, qkv):
            q, k, v = ops.prepare_qkv(qkv, op.q_norm_weight, op.k_norm_weight, self._rope_cos, self._rope_sin, positions,
                                      cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim, cfg.norm_eps)
            q, k, v = q.view(total, -1, cfg.head_dim), k.view(total, -1, cfg.head_dim), v.view(total, -1, cfg.head_dim)
            return ops.prefill_attention(q, k, v, cu, int(max(lengths)), self._scaling).view(total, -1)

        def conv_op(op, bcx):
            return ops.conv_prefill(bcx, op.conv_weight, cache.conv_state[op.cache_index], cu, seq_of_token, slots)

        hidden, residual = self._backbone(tokens, attention_op, conv_op, fp8)
        return ops.rms_norm(hidden, self.weights.embedding_norm_weight, cfg.norm_eps, residual)[0]


def _resolve_dtype(dtype):
    if isinstance(dtype, torch.dtype):
        return dtype
    if dtype is None or str(dtype).lower() == "auto":
        return torch.bfloat16
    names = {"bf16": torch.bfloat16, "bfloat16": torch.bfloat16, "fp16": torch.float16, "float16": torch.float16,
             "fp32": torch.float32, "float32": torch.float32}
    try:
        return names[str(dtype).strip().lower()]
    except KeyError as exc:
        raise ValueError(f"Unsupported dtype: {dtype!r}") from exc
