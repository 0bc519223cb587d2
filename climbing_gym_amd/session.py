"""Continuous batching over one graph entry: admit, poll, resume, release, fork, snapshot.

Mirrors `LFM25GenerationSession` of the reference (lfm25_session.py:109-533).  Row lifecycle: a finished
request keeps every token except its last sampled one in the KV/conv cache; `pending[row]` says that
token still has to be consumed.  The first step after `admit` leaves a fresh row inactive, so the sampler
reads the prefill logits kept in the entry's logits buffer.

All per-token state (lengths, limits, finish reasons, stop automaton state, RNG positions) lives in device
tensors updated by the record kernel; the host reads `reasons` once per poll.

Beyond the reference, rows may use temperature/top-k/top-p sampling as long as every filtered row of the
session shares one (top_k, top_p) pair; the draw then comes from the on-device filtered sampler.
"""
from __future__ import annotations

from contextlib import contextmanager
from dataclasses import dataclass
from typing import Sequence

import torch

from . import ops
from .cache import LFM25HybridCache
from .config import LFM25SamplingConfig
from .engine import flatten_token_batches
from .types import BehaviorTopK

STAT_KEYS = ("prefilled_tokens", "resumed_prefix_tokens", "appended_tokens", "admitted_requests", "resumed_requests",
             "decode_steps", "slot_refills", "peak_live_slots", "decode_row_steps", "reserved_row_steps",
             "adaptive_graph_captures", "forked_requests", "copied_prefix_tokens", "snapshot_prefilled_tokens",
             "snapshot_count", "peak_snapshots", "peak_snapshot_bytes")


@dataclass(frozen=True)
class LFM25ContinuationHandle:
    """Single-use lease on one session slot; invalid after release or close."""
    session: object
    slot: int
    version: int
    prefix_token_ids: tuple


@dataclass(frozen=True)
class LFM25SessionResult:
    handle: LFM25ContinuationHandle
    prompt_token_ids: tuple
    token_ids: tuple
    logprobs: tuple | None
    finish_reason: int
    behavior_topk: BehaviorTopK | None = None


@dataclass(frozen=True)
class LFM25PrefixSnapshot:
    """Opaque immutable lease; the tensors belong to the session that made it."""
    session: object
    identity: int
    policy_version: int
    prefix_token_ids: tuple


@dataclass
class _Snapshot:
    lease: LFM25PrefixSnapshot
    cache: LFM25HybridCache
    logits: torch.Tensor
    pending_token: int | None
    seed: int
    rng_position: int
    stop_state: int


@dataclass
class _Request:
    prompt: tuple
    sampling: LFM25SamplingConfig
    version: int
    delivered: bool = False
    handle: LFM25ContinuationHandle | None = None


class LFM25GenerationSession:
    @torch.inference_mode()
    def __init__(self, decoder, *, max_batch_size: int, max_new_tokens: int, cache_len: int | None = None,
                 behavior_topk: int = 0, profile_timings: bool = False):
        if decoder._active_session is not None:
            raise RuntimeError("A native generation session is already open")
        if type(max_batch_size) is not int or max_batch_size <= 0:
            raise ValueError("max_batch_size must be a positive integer")
        if type(max_new_tokens) is not int or max_new_tokens <= 0:
            raise ValueError("max_new_tokens must be a positive integer")
        engine = decoder.engine
        vocab = engine.config.vocab_size
        if type(behavior_topk) is not int or not 0 <= behavior_topk <= min(128, vocab):
            raise ValueError('behavior_topk must be an integer between 0 and min(vocab, 128)')
        self.decoder, self.engine = decoder, engine
        self.batch_size, self.max_new_tokens, self.behavior_topk = max_batch_size, max_new_tokens, behavior_topk
        self.entry = decoder._get_graph(max_batch_size, cache_len or engine.max_model_len, masked=True)
        self.entry.active.zero_()
        self.entry.cache.seq_lens.zero_()
        self.requests: list = [None] * max_batch_size
        self.versions = [0] * max_batch_size
        self.closed = False
        self.policy_version = engine.policy_version
        self.profile_timings = profile_timings
        self._snapshots: dict = {}
        self._snapshot_ids = 0
        self._events: list = []
        self._filter = None  # (top_k, top_p) shared by filtered rows
        device = engine.device
        col = lambda dtype, fill=0: torch.full((max_batch_size,), fill, device=device, dtype=dtype)
        self.lengths, self.limits = col(torch.int32), col(torch.int32)
        self.rng_positions, self.seeds = col(torch.int64), col(torch.int64)
        self.reasons = col(torch.int8)
        self.alive, self.pending, self.ignore_eos = col(torch.bool), col(torch.bool), col(torch.bool)
        self.temperatures = col(torch.float32)
        self.stop_states, self.stop_offsets = col(torch.int64), col(torch.int64)
        self.tokens = torch.empty((max_batch_size, max_new_tokens), device=device, dtype=torch.long)
        self.logprobs = torch.empty((max_batch_size, max_new_tokens), device=device, dtype=torch.float32)
        self.head_ids = (torch.empty((max_batch_size, max_new_tokens, behavior_topk), device=device, dtype=torch.int32)
                         if behavior_topk else None)
        self.head_logprobs = torch.empty_like(self.head_ids, dtype=torch.float32) if behavior_topk else None
        self.sampler = ops.RowSampler(self.entry.logits)
        self.stop_table = torch.zeros(vocab, device=device, dtype=torch.int32)
        self._stop_tables: dict = {}
        self.stats = {key: 0 for key in STAT_KEYS}
        self.stats["decode_batches"] = {}
        decoder._active_session = self

    # ------------------------------------------------------------------ guards
    def _check_open(self):
        if self.closed or self.decoder._active_session is not self or self.engine._cuda_decoder is not self.decoder:
            raise RuntimeError("Native generation session is closed")
        if self.engine.policy_version != self.policy_version:
            raise ValueError('Session cache belongs to another policy version')

    @contextmanager
    def _timed(self, phase):
        if not self.profile_timings:
            yield
            return
        begin, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        begin.record()
        try:
            yield
        finally:
            end.record()
            self._events.append((phase, begin, end))

    def timing_stats(self):
        """GPU seconds per phase, resolved once at the end (outside the hot loop)."""
        if self._events:
            self._events[-1][2].synchronize()
        totals: dict = {}
        for phase, begin, end in self._events:
            key = phase + '_gpu_seconds'
            totals[key] = totals.get(key, 0.0) + begin.elapsed_time(end) / 1000
        return totals

    def _validate(self, prompt, sampling):
        vocab = self.engine.config.vocab_size
        if sampling.behavior_topk > self.behavior_topk:
            raise ValueError('Request behavior head exceeds the session reservation')
        if not prompt:
            raise ValueError("Empty prompts are not supported")
        if set(map(type, prompt)) != {int} or min(prompt) < 0 or max(prompt) >= vocab:   # C-level passes over the ids
            raise ValueError("Prompt token outside the model vocabulary")
        if len(prompt) + sampling.max_new_tokens > self.entry.cache.max_seq_len:
            raise ValueError("Request exceeds reserved session context capacity")
        if sampling.max_new_tokens > self.max_new_tokens:
            raise ValueError("Request exceeds the session generation buffer")
        if sampling.repetition_penalty != 1.0:
            raise ValueError("Sessions support greedy/full-support/filtered sampling without repetition penalties")
        if sampling.filtered and self._filter not in (None, (sampling.top_k, sampling.top_p)):
            raise ValueError("Filtered rows of one session must share top_k and top_p")
        if sampling.stop_token_sequences:
            raise ValueError("Sessions use stop_token_ids or stop_table; encode string stops with build_stop_table")
        if any(not 0 <= t < vocab for t in sampling.stop_token_ids):
            raise ValueError("Stop token outside the model vocabulary")
        table = sampling.stop_table
        if table is not None and (table.ndim != 2 or table.size(1) != vocab or table.dtype != torch.int32):
            raise ValueError("stop_table must be an int32 state-by-vocabulary table")

    def _stop_offset(self, sampling) -> int:
        """Offset of the request's automaton inside the flat table; entry 0..V-1 is the empty automaton."""
        if sampling.stop_table is None and not sampling.stop_token_ids:
            return 0
        key = (id(sampling.stop_table), sampling.stop_token_ids)
        if key not in self._stop_tables:
            vocab, device = self.engine.config.vocab_size, self.engine.device
            table = (torch.zeros((1, vocab), dtype=torch.int32, device=device) if sampling.stop_table is None
                     else sampling.stop_table.to(device).clone())
            if sampling.stop_token_ids:
                table[:, list(sampling.stop_token_ids)] = 65536
            offset = self.stop_table.numel()
            self.stop_table = torch.cat((self.stop_table, table.reshape(-1)))
            self._stop_tables[key] = (offset, sampling.stop_table)  # keep the source alive: ids must stay unique
        return self._stop_tables[key][0]

    def _configure(self, slot, prompt, sampling, *, rng_position=0, stop_state=0):
        self._configure_many([(slot, prompt, sampling)], rng_position=rng_position, stop_state=stop_state)

    def _configure_many(self, work, *, rng_position=0, stop_state=0):
        """Per-row state of newly admitted (slot, prompt, sampling) requests: one indexed write per state tensor for
        the whole group (a write per row and tensor is eleven tiny launches per request)."""
        for slot, prompt, sampling in work:
            self.versions[slot] += 1
            self.requests[slot] = _Request(tuple(prompt), sampling, self.versions[slot])
            if sampling.filtered:
                self._filter = (sampling.top_k, sampling.top_p)
        samplings = [sampling for _, _, sampling in work]
        columns = ((self.lengths, [0] * len(work)), (self.reasons, [0] * len(work)),
                   (self.stop_states, [stop_state] * len(work)), (self.rng_positions, [rng_position] * len(work)),
                   (self.limits, [s.max_new_tokens for s in samplings]),
                   (self.seeds, [s.seed & 0x7FFFFFFFFFFFFFFF for s in samplings]),
                   (self.temperatures, [s.temperature for s in samplings]), (self.ignore_eos, [s.ignore_eos for s in samplings]),
                   (self.stop_offsets, [self._stop_offset(s) for s in samplings]), (self.alive, [True] * len(work)),
                   (self.pending, [False] * len(work)))
        if len(work) == 1:
            slot = work[0][0]
            for tensor, values in columns:
                tensor[slot] = values[0]
            return
        index = torch.tensor([slot for slot, _, _ in work], dtype=torch.long).to(self.lengths.device)
        for tensor, values in columns:
            tensor[index] = torch.tensor(values, dtype=tensor.dtype).to(tensor.device)

    def _free_slots(self):
        return [i for i, r in enumerate(self.requests) if r is None]

    def _live_count(self):
        return sum(r is not None for r in self.requests)

    def _pick_slots(self, slots, count, what):
        free = self._free_slots()
        slots = list(free[:count] if slots is None else slots)
        if len(slots) != count or len(set(slots)) != len(slots) or any(s not in free for s in slots):
            raise ValueError(f"{what} requires distinct free session slots")
        return slots

    # ------------------------------------------------------------------ admission
    @torch.inference_mode()
    def admit(self, prompts: Sequence[Sequence[int]], samplings: Sequence[LFM25SamplingConfig], *,
              slots: Sequence[int] | None = None) -> list:
        self._check_open()
        if len(prompts) != len(samplings):
            raise ValueError("One sampling configuration is required per prompt")
        slots = self._pick_slots(slots, len(prompts), "Admission")
        work = sorted(zip(slots, prompts, samplings), key=lambda item: item[0])
        for _, prompt, sampling in work:
            self._validate(prompt, sampling)
        # runs of consecutive slots prefill straight into views of the session cache
        begin = 0
        while begin < len(work):
            end = begin + 1
            while end < len(work) and work[end][0] == work[end - 1][0] + 1:
                end += 1
            first, last = work[begin][0], work[end - 1][0] + 1
            flat = flatten_token_batches([list(p) for _, p, _ in work[begin:end]], device=self.engine.device)
            with self._timed('prefill'):
                self.engine.prefill(*flat, cache=self.entry.cache.rows(first, last),
                                    max_prefill_tokens=self.decoder.max_prefill_tokens,
                                    logits_buffer=self.entry.logits[first:last])
            begin = end
        for slot, prompt, sampling in work:
            self.stats['slot_refills'] += int(self.versions[slot] > 0)
            self.stats['prefilled_tokens'] += len(prompt)
            self.stats['admitted_requests'] += 1
        self._configure_many(work)
        self.stats['peak_live_slots'] = max(self.stats['peak_live_slots'], self._live_count())
        return slots

    # ------------------------------------------------------------------ snapshots and forks
    def _remember(self, prompt, cache, logits, pending_token=None, seed=0, rng_position=0, stop_state=0):
        self._snapshot_ids += 1
        lease = LFM25PrefixSnapshot(self, self._snapshot_ids, self.policy_version, tuple(prompt))
        self._snapshots[lease.identity] = _Snapshot(lease, cache, logits, pending_token, seed, rng_position, stop_state)
        held = sum(s.cache.nbytes() + s.logits.numel() * s.logits.element_size() for s in self._snapshots.values())
        self.stats['snapshot_count'] += 1
        self.stats['peak_snapshots'] = max(self.stats['peak_snapshots'], len(self._snapshots))
        self.stats['peak_snapshot_bytes'] = max(self.stats['peak_snapshot_bytes'], held)
        return lease

    @torch.inference_mode()
    def prefill_snapshot(self, prompt: Sequence[int]) -> LFM25PrefixSnapshot:
        """Prefill one exact prefix once under the current weights."""
        self._check_open()
        prompt = tuple(prompt)
        self._validate(prompt, LFM25SamplingConfig(max_new_tokens=1))
        cache = self.engine._empty_cache(max_slots=1, max_seq_len=len(prompt), fp8_kv=self.entry.cache.fp8)
        with self._timed('prefill'):
            prefix = self.engine.prefill(*flatten_token_batches([list(prompt)], device=self.engine.device), cache=cache,
                                         max_prefill_tokens=self.decoder.max_prefill_tokens)
        self.stats['prefilled_tokens'] += len(prompt)
        self.stats['snapshot_prefilled_tokens'] += len(prompt)
        return self._remember(prompt, cache, prefix.next_token_logits)

    @torch.inference_mode()
    def snapshot(self, handle: LFM25ContinuationHandle) -> LFM25PrefixSnapshot:
        """Copy the valid KV bytes/scales, conv state, logits and the pending token of a delivered row."""
        request = self._request_for(handle)
        length = len(handle.prefix_token_ids) - 1
        if int(self.entry.cache.seq_lens[handle.slot]) != length:
            raise ValueError('Cached position does not match the pending-token prefix')
        with self._timed('cache_copy'):
            src = self.entry.cache.rows(handle.slot, handle.slot + 1)
            part = lambda t: None if t is None else t[:, :, :length].clone()
            cache = LFM25HybridCache(part(src.k_cache), part(src.v_cache), src.conv_state.clone(), src.seq_lens.clone(),
                                     part(src.k_scales), part(src.v_scales))
            logits = self.entry.logits[handle.slot:handle.slot + 1].clone()
        return self._remember(handle.prefix_token_ids, cache, logits, handle.prefix_token_ids[-1], request.sampling.seed,
                              int(self.rng_positions[handle.slot]), int(self.stop_states[handle.slot]))

    def _snapshot_for(self, snapshot):
        self._check_open()
        if snapshot.policy_version != self.engine.policy_version:
            raise ValueError('Snapshot belongs to another policy version')
        state = self._snapshots.get(snapshot.identity)
        if snapshot.session is not self or state is None or state.lease is not snapshot:
            raise ValueError('Snapshot is released or belongs to another session')
        return state

    @torch.inference_mode()
    def fork(self, snapshot: LFM25PrefixSnapshot, samplings: Sequence[LFM25SamplingConfig], *,
             slots: Sequence[int] | None = None) -> list:
        """Start independent children of a snapshot in free rows without any prefill."""
        state = self._snapshot_for(snapshot)
        slots = self._pick_slots(slots, len(samplings), "Fork")
        for sampling in samplings:
            self._validate(snapshot.prefix_token_ids, sampling)
        length = state.cache.max_seq_len
        with self._timed('cache_copy'):
            for slot in slots:
                dst = self.entry.cache.rows(slot, slot + 1)
                for target, source in ((dst.k_cache, state.cache.k_cache), (dst.v_cache, state.cache.v_cache),
                                       (dst.k_scales, state.cache.k_scales), (dst.v_scales, state.cache.v_scales)):
                    if target is not None:
                        _copy_bytes(target[:, :, :length], source)
                dst.conv_state.copy_(state.cache.conv_state)
                dst.seq_lens.copy_(state.cache.seq_lens)
                self.entry.logits[slot].copy_(state.logits[0])
        if slots and state.pending_token is not None:
            # the snapshot's last sampled token is not in the cache yet: consume it once in every child
            with self._timed('append'):
                keep = self.entry.input_tokens.clone()
                self.entry.input_tokens[slots] = state.pending_token
                self.entry.active.zero_()
                self.entry.active[slots] = True
                self._select_graph(slots)[0].replay()
                self.entry.input_tokens.copy_(keep)
        for slot, sampling in zip(slots, samplings):
            self.stats['slot_refills'] += int(self.versions[slot] > 0)
            self._configure(slot, snapshot.prefix_token_ids, sampling)
        self.stats['forked_requests'] += len(slots)
        self.stats['copied_prefix_tokens'] += length * len(slots)
        self.stats['peak_live_slots'] = max(self.stats['peak_live_slots'], self._live_count())
        return slots

    def release_snapshot(self, snapshot: LFM25PrefixSnapshot) -> None:
        self._snapshot_for(snapshot)
        del self._snapshots[snapshot.identity]

    # ------------------------------------------------------------------ continuation
    def _request_for(self, handle):
        self._check_open()
        if handle.session is not self or not 0 <= handle.slot < self.batch_size:
            raise ValueError("Continuation handle belongs to another session")
        request = self.requests[handle.slot]
        if request is None or request.version != handle.version or not request.delivered or request.handle is not handle:
            raise ValueError("Continuation handle is stale or already consumed")
        return request

    def _select_graph(self, slots):
        before = len(self.entry.compact_graphs)
        graph, size = self.decoder._select_graph(self.entry, slots)
        self.stats['adaptive_graph_captures'] += len(self.entry.compact_graphs) - before
        return graph, size

    @torch.inference_mode()
    def resume(self, handles: Sequence[LFM25ContinuationHandle], prompts: Sequence[Sequence[int]],
               samplings: Sequence[LFM25SamplingConfig], *, preserve_rng: bool = False) -> None:
        """Continue delivered rows from an exact extension of their cached prefix: the pending token and the new
        suffix are appended one token per replay with per-row masks."""
        if not len(handles) == len(prompts) == len(samplings):
            raise ValueError("One prompt and sampling configuration is required per handle")
        if len({h.slot for h in handles}) != len(handles):
            raise ValueError("Cannot resume a handle twice")
        appends, carried = [], []
        for handle, prompt, sampling in zip(handles, prompts, samplings):
            request = self._request_for(handle)
            self._validate(prompt, sampling)
            prefix = handle.prefix_token_ids
            if tuple(prompt[:len(prefix)]) != prefix:
                raise ValueError("Continuation requires the exact cached token prefix")
            if preserve_rng and (tuple(prompt) != prefix or sampling.seed != request.sampling.seed
                                 or sampling.stop_table is not request.sampling.stop_table
                                 or sampling.stop_token_ids != request.sampling.stop_token_ids):
                raise ValueError('Internal pauses must preserve the exact context, seed and stop rules')
            carried.append((int(self.rng_positions[handle.slot]), int(self.stop_states[handle.slot])) if preserve_rng else (0, 0))
            appends.append((handle.slot, (prefix[-1], *prompt[len(prefix):])))
        if not appends:
            return
        width = max(len(t) for _, t in appends)
        feed = torch.zeros((width, self.batch_size), dtype=torch.long)
        mask = torch.zeros((width, self.batch_size), dtype=torch.bool)
        for slot, toks in appends:
            feed[:len(toks), slot] = torch.tensor(toks)
            mask[:len(toks), slot] = True
        feed, mask = feed.to(self.engine.device), mask.to(self.engine.device)
        keep = self.entry.input_tokens.clone()  # other live rows still owe their own pending tokens
        graph, _ = self._select_graph([slot for slot, _ in appends])
        for i in range(width):
            self.entry.input_tokens.copy_(feed[i])
            self.entry.active.copy_(mask[i])
            graph.replay()
        self.entry.input_tokens.copy_(keep)
        for handle, prompt, sampling, (position, stop_state) in zip(handles, prompts, samplings, carried):
            self._configure(handle.slot, prompt, sampling, rng_position=position, stop_state=stop_state)
            self.stats['resumed_prefix_tokens'] += len(handle.prefix_token_ids) - 1
            self.stats['appended_tokens'] += len(prompt) - len(handle.prefix_token_ids) + 1
            self.stats['resumed_requests'] += 1

    # ------------------------------------------------------------------ the hot loop
    def _sample(self):
        logits = self.entry.logits
        if self._filter is None:
            return self.sampler.sample(logits, self.seeds, self.rng_positions, self.temperatures)
        # one shared (top_k, top_p); temperature is per request but must be positive for filtered rows
        top_k, top_p = self._filter
        temperature = max(r.sampling.temperature for r in self.requests if r is not None and r.sampling.filtered)
        return ops.sample_filtered(logits, temperature=temperature, top_k=top_k, top_p=top_p, seeds=self.seeds,
                                   steps=self.rng_positions, out=(self.sampler.tokens, self.sampler.logprobs))

    @torch.inference_mode()
    def poll(self, *, steps: int | None = None) -> list:
        self._check_open()
        steps = self.decoder.finish_check_interval if steps is None else steps
        if type(steps) is not int or steps <= 0:
            raise ValueError("steps must be a positive integer")
        live = [i for i, r in enumerate(self.requests) if r is not None and not r.delivered]
        if not live:
            return []
        graph, batch = self._select_graph(live)
        cfg = self.engine.config
        for _ in range(steps):
            self.entry.active.copy_(self.pending)
            graph.replay()
            sampled, logp = self._sample()
            if self.behavior_topk:
                ids, probs = ops.behavior_topk(self.entry.logits, sampled, logp, self.behavior_topk)
                ops.record_head(ids, probs, self.head_ids, self.head_logprobs, self.lengths, self.alive,
                                self.behavior_topk, self.max_new_tokens)
            ops.record_sample(sampled, logp, self.tokens, self.logprobs, self.lengths, self.limits, self.reasons, self.alive,
                              self.pending, self.entry.input_tokens, self.stop_states, self.stop_offsets, self.stop_table,
                              self.ignore_eos, self.rng_positions, cfg.eos_token_id, cfg.vocab_size, self.max_new_tokens)
        self.stats['decode_steps'] += steps
        self.stats['decode_row_steps'] += batch * steps
        self.stats['reserved_row_steps'] += self.batch_size * steps
        hist = self.stats['decode_batches']
        hist[str(batch)] = hist.get(str(batch), 0) + steps
        reasons = self.reasons.cpu().tolist()
        done = [i for i in live if reasons[i]]
        if not done:
            return []
        index = torch.tensor(done, device=self.engine.device)
        lengths = self.lengths[index].cpu().tolist()
        longest = max(lengths)
        tokens = self.tokens[:, :longest].index_select(0, index).cpu().tolist()
        logprobs = self.logprobs[:, :longest].index_select(0, index).cpu().tolist()
        results = []
        for slot, length, ids, probs in zip(done, lengths, tokens, logprobs):
            request = self.requests[slot]
            request.delivered = True
            ids = tuple(ids[:length])
            request.handle = LFM25ContinuationHandle(self, slot, request.version, request.prompt + ids)
            k = request.sampling.behavior_topk
            head = BehaviorTopK(self.head_ids[slot, :length, :k].cpu(), self.head_logprobs[slot, :length, :k].cpu()) if k else None
            results.append(LFM25SessionResult(request.handle, request.prompt, ids,
                                              tuple(probs[:length]) if request.sampling.return_logprobs else None,
                                              reasons[slot], head))
        return results

    @torch.inference_mode()
    def release(self, handle: LFM25ContinuationHandle) -> None:
        self._request_for(handle)
        slot = handle.slot
        self.requests[slot] = None
        self.versions[slot] += 1
        self.alive[slot] = False
        self.pending[slot] = False
        self.entry.cache.seq_lens[slot] = 0
        if not any(r is not None and r.sampling.filtered for r in self.requests):
            self._filter = None

    def close(self):
        if self.closed:
            return
        self.closed = True
        self.requests = [None] * self.batch_size
        self._snapshots.clear()
        if self.decoder._active_session is self:
            self.decoder._active_session = None

    def __enter__(self):
        self._check_open()
        return self

    def __exit__(self, *_):
        self.close()


def _copy_bytes(target: torch.Tensor, source: torch.Tensor) -> None:
    """Copy without dequantising: one-byte element types go through a uint8 view."""
    if target.element_size() == 1:
        target.view(torch.uint8).copy_(source.view(torch.uint8))
    else:
        target.copy_(source)
