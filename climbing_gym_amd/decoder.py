"""HIP-graph decode over the packed weights: the stand-in for the reference's `LFM25CUDADecoder`
(lfm25_cuda.py:30-380) and compact graphs (lfm25_batching.py:72-120).

A graph entry owns a slot cache with stable addresses, an input-token buffer, a logits buffer and one
captured decode step.  Prompts prefill straight into that cache; each new token is one replay.  Per-token
bookkeeping (sampling, recording, stop detection, finish codes) runs in device kernels, and the host
looks at the `alive` flags only every `finish_check_interval` steps.
"""
from __future__ import annotations

import gc
from collections import OrderedDict
from dataclasses import dataclass, field

import torch

from . import ops
from .cache import LFM25HybridCache
from .config import LFM25SamplingConfig
from .engine import LFM25GenerationOutput
from ._checks import reject


class _EagerStep:
    """Stands in for a captured graph when capture is switched off: replay() launches the step directly."""

    def __init__(self, fn):
        self._fn = fn

    def replay(self):
        self._fn()


@dataclass
class _DecodeGraph:
    cache: LFM25HybridCache
    input_tokens: torch.Tensor
    logits: torch.Tensor
    graph: object
    active: torch.Tensor | None = None
    compact_graphs: dict = field(default_factory=dict)


@dataclass
class CompactDecodeGraph:
    """A smaller compute batch over the same physical cache; rows reach their slots through `slots`."""
    graph: object
    slots: torch.Tensor
    buffers: tuple
    mapped_slots: tuple = ()

    def set_slots(self, slots):
        mapping = tuple(slots)
        if mapping != self.mapped_slots:
            padded = mapping + (-1,) * (self.slots.numel() - len(mapping))
            self.slots.copy_(torch.tensor(padded, dtype=torch.int32), non_blocking=False)
            self.mapped_slots = mapping


def graph_capacity(cache_len: int, batch_size: int, max_model_len: int) -> int:
    """Context capacity of a graph's cache: finer rounding for large batches (lfm25_cuda.py:216-217)."""
    step = 32 if batch_size >= 64 else 128
    return min(max_model_len, -(-cache_len // step) * step)


class LFM25HIPDecoder:
    def __init__(self, engine, *, max_graphs: int = 2, max_prefill_tokens: int = 4096, finish_check_interval: int = 32,
                 skip_finished_attention: bool = True, fp8_mlp: bool = False, fp8_kv: bool = False,
                 adaptive_batching: bool = False, fp8_lm_head: bool = False, fp8_operators: bool = False,
                 capture: bool = True):
        reject(max_graphs <= 0, "max_graphs must be > 0")
        reject(max_prefill_tokens <= 0, "max_prefill_tokens must be positive")
        reject(type(finish_check_interval) is not int or finish_check_interval <= 0,
               "finish_check_interval must be a positive integer")
        self.engine = engine
        self.max_graphs = max_graphs
        self.max_prefill_tokens = max_prefill_tokens
        self.finish_check_interval = finish_check_interval
        self.skip_finished_attention = bool(skip_finished_attention)
        self.fp8_mlp, self.fp8_kv = bool(fp8_mlp), bool(fp8_kv)
        self.fp8_lm_head, self.fp8_operators = bool(fp8_lm_head), bool(fp8_operators)
        self.adaptive_batching = bool(adaptive_batching)
        self.capture = bool(capture)
        self.fp8_weights: dict = {}
        self.graphs: "OrderedDict[tuple, _DecodeGraph]" = OrderedDict()
        self._active_session = None
        # One stream for every capture of this decoder's lifetime (captures may come from different host threads).
        self._capture_stream = torch.cuda.Stream(device=engine.device)
        self._prepare_fp8_weights()

    # ------------------------------------------------------------------ weights
    def _prepare_fp8_weights(self) -> None:
        if self.fp8_weights or not (self.fp8_mlp or self.fp8_lm_head or self.fp8_operators):
            return
        weights = self.engine.weights
        chosen = []
        for layer in weights.layers:
            if self.fp8_operators:
                op = layer.attention or layer.conv
                chosen += [op.qkv_weight if layer.attention is not None else op.in_weight, op.out_weight]
            if self.fp8_mlp:
                chosen += [layer.w13_weight, layer.w2_weight]
        if self.fp8_lm_head:
            chosen.append(weights.lm_head_weight)
        self.fp8_weights = {id(w): ops.PackedFP8Weight.from_weight(w) for w in chosen}

    def refresh_weights(self) -> None:
        for packed in self.fp8_weights.values():
            packed.refresh()

    def clear(self) -> None:
        if self._active_session is not None:
            self._active_session.close()
        self.graphs.clear()
        self.fp8_weights.clear()

    # ------------------------------------------------------------------ capture
    def _forward(self, cache, tokens, active=None, *, slot_ids=None, positions=None, logits_out=None, gather=None):
        return self.engine._decode_forward(cache, tokens, active, slot_ids=slot_ids, positions=positions, fp8=self.fp8_weights,
                                           logits_out=logits_out, gather=gather)

    def _capture(self, step, before_warmup=None, probe=None):
        """Two warm-up launches, then record `step` into a HIP graph on the decoder's capture stream.  `probe` is
        installed as the engine's step probe for the recorded run only."""
        if not self.capture:
            return _EagerStep(step)
        device = self.engine.device
        stream, current = self._capture_stream, torch.cuda.current_stream(device)
        stream.wait_stream(current)
        with torch.cuda.stream(stream):
            for _ in range(2):
                if before_warmup is not None:
                    before_warmup()
                step()
            if before_warmup is not None:
                before_warmup()
        current.wait_stream(stream)
        torch.cuda.synchronize(device)
        graph = torch.cuda.CUDAGraph()
        # Destroying a graph, a graph executable or a stream is one of the calls HIP forbids while a capture is open:
        # under the default (global) capture mode any thread that makes one invalidates the capture and the runtime
        # aborts the process.  Two sources of such calls exist here: the cyclic collector finalising an unreachable
        # engine's graphs and streams in the middle of this capture (torch.cuda.graph collects once before the capture
        # begins; the collector stays off until it ends), and another host thread dropping the last reference to such
        # an object (thread-local capture mode confines the check to the capturing thread).
        collector_was_on = gc.isenabled()
        gc.disable()
        self.engine._step_probe = probe
        try:
            with torch.cuda.graph(graph, stream=stream, capture_error_mode="thread_local"):
                step()
        finally:
            self.engine._step_probe = None
            if collector_was_on:
                gc.enable()
        current.wait_stream(stream)
        return graph

    @torch.inference_mode()
    def _get_graph(self, batch_size: int, cache_len: int, *, masked: bool = False) -> _DecodeGraph:
        capacity = graph_capacity(cache_len, batch_size, self.engine.max_model_len)
        key = (batch_size, capacity, masked)
        if key in self.graphs:
            self.graphs.move_to_end(key)
            return self.graphs[key]
        if len(self.graphs) >= self.max_graphs:  # evict first: bounds peak residency too
            self.graphs.popitem(last=False)
        self._prepare_fp8_weights()
        engine = self.engine
        cache = engine._empty_cache(max_slots=batch_size, max_seq_len=capacity, fp8_kv=self.fp8_kv)
        tokens = torch.zeros(batch_size, device=engine.device, dtype=torch.long)
        active = torch.ones(batch_size, device=engine.device, dtype=torch.bool) if masked else None
        # masked graphs keep the last logits of rows that sit out a step (fresh prefill logits included)
        saved = torch.zeros((batch_size, engine.config.vocab_size), device=engine.device, dtype=engine.dtype) if masked else None
        if saved is None and not self.capture:
            saved = torch.zeros((batch_size, engine.config.vocab_size), device=engine.device, dtype=engine.dtype)
        holder = {}

        def step():
            # masked steps write only the live rows of `saved`; uncaptured steps write all of it, so that one stable
            # buffer holds the logits either way
            holder["logits"] = self._forward(cache, tokens, active, logits_out=saved)

        graph = self._capture(step, before_warmup=cache.seq_lens.zero_)
        entry = _DecodeGraph(cache, tokens, holder["logits"] if self.capture else saved, graph, active)
        self.graphs[key] = entry
        if batch_size >= 64:
            torch.cuda.empty_cache()
        return entry

    @torch.inference_mode()
    def capture_probed_step(self, entry: _DecodeGraph, probe):
        """`entry`'s decode step recorded once more, over the same cache and buffers, with `probe(kind, index, phase)`
        called on the capture stream before (phase 0) and after (phase 1) each decode-attention call (`kind` is
        "attention", `index` the attention layer).  A probe that records events made with `external=True` puts
        event-record nodes around those kernels, so their time inside a replayed step can be read with
        `Event.elapsed_time`.  For measurement: the two warm-up runs advance the rolling conv state, which is put back
        together with the lengths; the rows they append to the KV cache are overwritten by the next real step."""
        reject(not self.capture, "a probed step needs graph capture", RuntimeError)
        cache = entry.cache
        lengths, conv_state = cache.seq_lens.clone(), cache.conv_state.clone()
        logits = entry.logits

        def restore():
            cache.seq_lens.copy_(lengths)
            cache.conv_state.copy_(conv_state)

        def step():
            self._forward(cache, entry.input_tokens, entry.active, logits_out=logits)

        graph = self._capture(step, before_warmup=restore, probe=probe)
        return graph

    @torch.inference_mode()
    def capture_compact(self, entry: _DecodeGraph, batch_size: int) -> CompactDecodeGraph:
        """Capture a `batch_size`-row step over `entry`'s cache.  Every slot id is -1 during warm-up and capture,
        so no resident request is touched (lfm25_batching.py:87-120)."""
        device = self.engine.device
        slots = torch.full((batch_size,), -1, device=device, dtype=torch.int32)
        tokens = torch.zeros(batch_size, device=device, dtype=torch.long)
        positions = torch.zeros(batch_size, device=device, dtype=torch.int32)
        active = torch.zeros(batch_size, device=device, dtype=torch.bool)

        def step():
            # the rows' tokens, positions and activity flags are gathered from the slots by the step's first launch
            self._forward(entry.cache, tokens, active, slot_ids=slots, positions=positions, logits_out=entry.logits,
                          gather=(entry.input_tokens, entry.active))

        graph = self._capture(step)
        return CompactDecodeGraph(graph, slots, (tokens, positions, active))

    def _select_graph(self, entry: _DecodeGraph, live_slots):
        """(graph, compute rows) for the rows that are live: with adaptive batching the smallest power of two that holds
        them, 16 at least, as a compact graph over the same cache; the full graph when that is no smaller than it
        (lfm25_cuda.py:194-209)."""
        rows = entry.input_tokens.numel()
        if self.adaptive_batching:
            width = max(16, 1 << max(len(live_slots) - 1, 0).bit_length())
            if width < rows:
                compact = entry.compact_graphs.get(width)
                if compact is None:
                    compact = entry.compact_graphs[width] = self.capture_compact(entry, width)
                compact.set_slots(live_slots)
                return compact.graph, width
        return entry.graph, rows

    # ------------------------------------------------------------------ generate
    @torch.inference_mode()
    def generate(self, input_ids, cu_seqlens, max_seqlen: int, repeats: int, sampling: LFM25SamplingConfig):
        reject(self._active_session is not None,
               "Close the native generation session before calling generate", RuntimeError)
        reject(repeats <= 0, "repeats must be > 0")
        engine = self.engine
        device, vocab = engine.device, engine.config.vocab_size
        new_tokens = sampling.max_new_tokens
        cache_len = int(max_seqlen) + new_tokens
        reject(cache_len > engine.max_model_len,
               f"max_seq_len={cache_len} exceeds engine max_model_len={engine.max_model_len}")
        prompts = cu_seqlens.numel() - 1
        batch = prompts * repeats
        k = sampling.behavior_topk
        reject(k > vocab, 'Behavior head exceeds the vocabulary')
        entry = self._get_graph(batch, cache_len, masked=self.adaptive_batching) if new_tokens > 1 else None
        direct = entry is not None and repeats == 1
        prefix = engine.prefill(input_ids, cu_seqlens, max_seqlen, max_cache_len=max_seqlen,
                                cache=entry.cache if direct else None, max_prefill_tokens=self.max_prefill_tokens,
                                logits_buffer=entry.logits if direct else None)
        if entry is not None and not direct:
            rows = torch.arange(prefix.batch_size, device=device).repeat_interleave(repeats)
            entry.cache.copy_prefix_from(prefix.cache, rows, max_seqlen)
        logits = prefix.next_token_logits if repeats == 1 else prefix.next_token_logits.repeat_interleave(repeats, dim=0)
        seen = engine._build_seen_token_mask(prefix, repeats, sampling)
        del prefix

        zeros = lambda *shape, dtype: torch.zeros(shape, device=device, dtype=dtype)
        tokens, logprobs = zeros(batch, new_tokens, dtype=torch.long), zeros(batch, new_tokens, dtype=torch.float32)
        lengths, limits = zeros(batch, dtype=torch.int32), torch.full((batch,), new_tokens, device=device, dtype=torch.int32)
        reasons, alive = zeros(batch, dtype=torch.int8), torch.ones(batch, device=device, dtype=torch.bool)
        pending = entry.active if entry is not None and entry.active is not None else torch.ones_like(alive)
        pending.fill_(True)
        feed = entry.input_tokens if entry is not None else zeros(batch, dtype=torch.long)
        rng_positions, stop_states = zeros(batch, dtype=torch.long), zeros(batch, dtype=torch.long)
        ignore_eos = torch.full((batch,), bool(sampling.ignore_eos), device=device, dtype=torch.bool)
        stop_table, offset = self._stop_table(sampling, vocab, device)
        stop_offsets = torch.full((batch,), offset, device=device, dtype=torch.long)
        head_ids = zeros(batch, new_tokens, k, dtype=torch.int32) if k else None
        head_logprobs = zeros(batch, new_tokens, k, dtype=torch.float32) if k else None
        patterns = [torch.tensor(s, device=device) for s in sampling.stop_token_sequences]
        fixed = sampling.fixed_length
        decode_graph = entry.graph if entry is not None else None
        interval = self.finish_check_interval if batch >= 16 else 1

        for step in range(new_tokens):
            sampled, raw, _ = engine._sample(logits, sampling, step=step, seen_token_mask=seen)
            if k:
                ids, probs = ops.behavior_topk(logits, sampled, raw, k)
                ops.record_head(ids, probs, head_ids, head_logprobs, lengths, alive, k, new_tokens)
            if seen is not None:
                seen[torch.arange(batch, device=device), sampled] = True
            # token, log-probability, length, stop automaton, finish code and next input in one launch
            ops.record_sample(sampled, raw, tokens, logprobs, lengths, limits, reasons, alive, pending, feed, stop_states,
                              stop_offsets, stop_table, ignore_eos, rng_positions, engine.config.eos_token_id, vocab, new_tokens)
            if patterns:
                hit = _sequence_stops(tokens[:, :step + 1], lengths, patterns) & alive
                reasons.masked_fill_(hit, 2)
                alive.logical_and_(~hit)
                pending.logical_and_(~hit)
            if not fixed and ((step + 1) % interval == 0 or step + 1 == new_tokens):
                if self.adaptive_batching:
                    live = [i for i, on in enumerate(alive.cpu().tolist()) if on]
                    if not live:
                        break
                    if step + 1 < new_tokens:
                        decode_graph, _ = self._select_graph(entry, live)
                elif not bool(alive.any().item()):
                    break
            if step + 1 < new_tokens:
                if not fixed and self.skip_finished_attention and entry.active is None:
                    entry.cache.seq_lens.masked_fill_(~alive, 0)  # finished rows stop reading their history
                decode_graph.replay()
                logits = entry.logits
        shape = (prompts, repeats)
        return LFM25GenerationOutput(
            token_ids=tokens.view(*shape, new_tokens), lengths=lengths.view(*shape),
            logprobs=logprobs.view(*shape, new_tokens) if sampling.return_logprobs else None,
            finish_reasons=reasons.view(*shape),
            topk_token_ids=None if head_ids is None else head_ids.view(*shape, new_tokens, k),
            topk_logprobs=None if head_logprobs is None else head_logprobs.view(*shape, new_tokens, k))

    @staticmethod
    def _stop_table(sampling: LFM25SamplingConfig, vocab: int, device):
        """Flat int32 automaton: entry state*V + token -> next state (+65536 when a stop completes).  Offset 0 is the
        empty table; stop token ids are encoded as 65536 in every state (lfm25_session.py:228-241)."""
        empty = torch.zeros(vocab, device=device, dtype=torch.int32)
        if sampling.stop_table is None and not sampling.stop_token_ids:
            return empty, 0
        table = (torch.zeros((1, vocab), dtype=torch.int32, device=device) if sampling.stop_table is None
                 else sampling.stop_table.to(device).clone())
        reject(table.ndim != 2 or table.size(1) != vocab or table.dtype != torch.int32,
               "stop_table must be an int32 state-by-vocabulary table")
        if sampling.stop_token_ids:
            table[:, list(sampling.stop_token_ids)] = 65536
        return torch.cat((empty, table.reshape(-1))), vocab


def _sequence_stops(history, lengths, patterns):
    """Rows whose generated tokens end with one of the multi-token stop patterns (lfm25_engine.py:1620-1626)."""
    hit = torch.zeros(history.size(0), device=history.device, dtype=torch.bool)
    for pattern in patterns:
        n = pattern.numel()
        if history.size(1) >= n:
            hit |= (history[:, -n:] == pattern).all(dim=1) & (lengths == history.size(1))
    return hit


LFM25CUDADecoder = LFM25HIPDecoder
