"""Continuous batching over one captured decode step: the stand-in for `LFM25GenerationSession`
(lfm25_session.py:109-533) with its public methods, argument meanings, error texts and statistics keys.

How this one is built:

* the per-row device state is one struct of tensors (`_RowTable`); an admission writes all of its rows with one
  upload and one kernel (`lfm2_configure_rows`), whatever the number of requests;
* a slot is a small host record (`_Slot`) with a generation counter; a continuation handle is valid while it is the
  record's current lease, so "stale", "consumed" and "other session" are one comparison;
* the flag "this row still owes the model its last sampled token" IS the graph's activity mask: the record kernel
  writes it, the next replay reads it, and no copy runs between the two;
* a whole admission is one packed prefill, whichever slots are free: the prefill kernels scatter every sequence to its
  slot, so fragmented free slots cost nothing;
* every row is drawn by the full-support sampler; rows that ask for top-k / top-p (an extension: the reference's
  sessions refuse them, lfm25_session.py:217-218) are then redrawn by the filtered sampler with their own
  temperature, k and p, so a request's tokens never depend on what its neighbours asked for.

A finished request keeps every token except its last sampled one in the KV/conv cache; resuming it feeds that token
(and any new suffix) one position per replay under a per-row mask.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass
from typing import Sequence

import torch

from . import ops
from .cache import LFM25HybridCache
from .config import LFM25SamplingConfig
from .engine import flatten_token_batches
from .types import BehaviorTopK
from ._checks import reject

_no_grad = torch.inference_mode   # every public method runs without autograd state
STAT_KEYS = ("prefilled_tokens", "resumed_prefix_tokens", "appended_tokens", "admitted_requests", "resumed_requests",
             "decode_steps", "slot_refills", "peak_live_slots", "decode_row_steps", "reserved_row_steps",
             "adaptive_graph_captures", "forked_requests", "copied_prefix_tokens", "snapshot_prefilled_tokens",
             "snapshot_count", "peak_snapshots", "peak_snapshot_bytes")
_SEED_MASK = (1 << 63) - 1
# the reference's error texts (callers and tests match on them), by the condition that raises them
_REFUSALS = {
    "already_open": (RuntimeError, "A native generation session is already open"),
    "head_width": (ValueError, "behavior_topk must be an integer between 0 and min(vocab, 128)"),
    "closed": (RuntimeError, "Native generation session is closed"),
    "session_policy": (ValueError, "Session cache belongs to another policy version"),
    "sampling_per_prompt": (ValueError, "One sampling configuration is required per prompt"),
    "snapshot_policy": (ValueError, "Snapshot belongs to another policy version"),
    "snapshot_gone": (ValueError, "Snapshot is released or belongs to another session"),
    "position_mismatch": (ValueError, "Cached position does not match the pending-token prefix"),
    "foreign_handle": (ValueError, "Continuation handle belongs to another session"),
    "stale_handle": (ValueError, "Continuation handle is stale or already consumed"),
    "per_handle": (ValueError, "One prompt and sampling configuration is required per handle"),
    "twice": (ValueError, "Cannot resume a handle twice"),
    "prefix_differs": (ValueError, "Continuation requires the exact cached token prefix"),
    "pause_rules": (ValueError, "Internal pauses must preserve the exact context, seed and stop rules"),
    "steps": (ValueError, "steps must be a positive integer"),
}


def filtered_on_device(sampling: LFM25SamplingConfig) -> bool:
    """Whether the filtered sampler draws this request's rows.  The kernels decide per row from the float32 columns
    of the row table, so the host decides from the same float32 values: a top_p such as 1 - 1e-9 is 1.0f there and a
    temperature below the smallest float32 is 0 (greedy), and such a row belongs to the full-support sampler."""
    as_f32 = lambda value: struct.unpack("<f", struct.pack("<f", float(value)))[0]
    return as_f32(sampling.temperature) > 0.0 and (sampling.top_k > 0 or as_f32(sampling.top_p) < 1.0)


def _refuse(condition: str):
    kind, text = _REFUSALS[condition]
    raise kind(text)


# ---------------------------------------------------------------------------------------------- what callers hold
@dataclass(frozen=True)
class LFM25ContinuationHandle:
    """Single-use lease on one session slot; invalid after release, resume or close."""
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
    """Opaque immutable lease on a stored prefix; the tensors stay with the session that made it."""
    session: object
    identity: int
    policy_version: int
    prefix_token_ids: tuple


# ---------------------------------------------------------------------------------------------- host-side records
@dataclass
class _Slot:
    generation: int = 0                    # bumped every time the slot is configured or given back
    prompt: tuple | None = None
    sampling: LFM25SamplingConfig | None = None
    lease: LFM25ContinuationHandle | None = None   # set once the result has been handed out
    used_before: bool = False

    @property
    def busy(self) -> bool:
        return self.prompt is not None

    @property
    def running(self) -> bool:
        return self.prompt is not None and self.lease is None


@dataclass
class _StoredPrefix:
    lease: LFM25PrefixSnapshot
    cache: LFM25HybridCache
    logits: torch.Tensor
    pending_token: int | None = None
    seed: int = 0
    rng_position: int = 0
    stop_state: int = 0

    def nbytes(self) -> int:
        return self.cache.nbytes() + self.logits.numel() * self.logits.element_size()


class _RowTable:
    """Device state of the session's rows, one column per field (the tensors of lfm25_session.py:150-165 plus the
    per-row filter parameters)."""

    def __init__(self, rows: int, new_tokens: int, head: int, pending: torch.Tensor, device):
        column = lambda dtype: torch.zeros(rows, device=device, dtype=dtype)
        self.lengths, self.limits, self.top_ks = column(torch.int32), column(torch.int32), column(torch.int32)
        self.seeds, self.rng_positions = column(torch.int64), column(torch.int64)
        self.stop_states, self.stop_offsets = column(torch.int64), column(torch.int64)
        self.reasons = column(torch.int8)
        self.alive, self.ignore_eos = column(torch.bool), column(torch.bool)
        self.temperatures, self.top_ps = column(torch.float32), column(torch.float32)
        self.pending = pending.zero_()     # the decode graph's activity mask
        self.tokens = torch.empty((rows, new_tokens), device=device, dtype=torch.long)
        self.logprobs = torch.empty((rows, new_tokens), device=device, dtype=torch.float32)
        self.head_ids = torch.empty((rows, new_tokens, head), device=device, dtype=torch.int32) if head else None
        self.head_logprobs = torch.empty((rows, new_tokens, head), device=device, dtype=torch.float32) if head else None
        self.device = device

    @staticmethod
    def spec(slot: int, sampling: LFM25SamplingConfig, stop_offset: int, rng_position: int, stop_state: int) -> list:
        """The eight words `lfm2_configure_rows` reads for one request."""
        floats = struct.unpack("<q", struct.pack("<ff", float(sampling.temperature), float(sampling.top_p)))[0]
        flags = int(bool(sampling.ignore_eos)) | (int(sampling.top_k if filtered_on_device(sampling) else 0) << 8)
        return [slot, sampling.max_new_tokens, sampling.seed & _SEED_MASK, rng_position, stop_state, stop_offset, flags, floats]

    def write(self, specs: list) -> None:
        ops.configure_rows(torch.tensor(specs, dtype=torch.int64).to(self.device), self)

    def retire(self, slot: int) -> None:
        self.alive[slot] = False
        self.pending[slot] = False


class _StopTables:
    """One flat int32 table: entries 0..V-1 are the automaton that never stops; each distinct (stop table, stop ids)
    pair appends its states x V entries, with stop ids marked 65536 in every state (lfm25_session.py:228-241)."""

    def __init__(self, vocab: int, device):
        self.vocab, self.device = vocab, device
        self.flat = torch.zeros(vocab, device=device, dtype=torch.int32)
        self._known: dict = {}

    def offset(self, sampling: LFM25SamplingConfig) -> int:
        if sampling.stop_table is None and not sampling.stop_token_ids:
            return 0
        key = (id(sampling.stop_table), tuple(sampling.stop_token_ids))
        found = self._known.get(key)
        if found is None:
            states = (torch.zeros((1, self.vocab), dtype=torch.int32, device=self.device) if sampling.stop_table is None
                      else sampling.stop_table.to(self.device).clone())
            if sampling.stop_token_ids:
                states[:, list(sampling.stop_token_ids)] = 65536
            found = (self.flat.numel(), sampling.stop_table)   # holding the table keeps its id() from being reused
            self.flat = torch.cat((self.flat, states.reshape(-1)))
            self._known[key] = found
        return found[0]


class _PhaseClock:
    """Optional GPU timing of the session's phases with event pairs, read once at the end."""

    def __init__(self, enabled: bool):
        self.enabled, self.spans = enabled, []

    def __call__(self, phase: str):
        return _PhaseSpan(self, phase)

    def totals(self) -> dict:
        if self.spans:
            self.spans[-1][2].synchronize()
        out: dict = {}
        for phase, begin, end in self.spans:
            out[f"{phase}_gpu_seconds"] = out.get(f"{phase}_gpu_seconds", 0.0) + begin.elapsed_time(end) / 1000
        return out


class _PhaseSpan:
    def __init__(self, clock: _PhaseClock, phase: str):
        self.clock, self.phase = clock, phase

    def __enter__(self):
        if self.clock.enabled:
            self.begin = torch.cuda.Event(enable_timing=True)
            self.begin.record()

    def __exit__(self, *_):
        if self.clock.enabled:
            end = torch.cuda.Event(enable_timing=True)
            end.record()
            self.clock.spans.append((self.phase, self.begin, end))


# ---------------------------------------------------------------------------------------------- the session
class LFM25GenerationSession:
    @_no_grad()
    def __init__(self, decoder, *, max_batch_size: int, max_new_tokens: int, cache_len: int | None = None,
                 behavior_topk: int = 0, profile_timings: bool = False):
        if decoder._active_session is not None:
            _refuse("already_open")
        for name, value in (("max_batch_size", max_batch_size), ("max_new_tokens", max_new_tokens)):
            reject(type(value) is not int or value <= 0, f"{name} must be a positive integer")
        engine = decoder.engine
        vocab = engine.config.vocab_size
        if type(behavior_topk) is not int or not 0 <= behavior_topk <= min(128, vocab):
            _refuse("head_width")
        self.decoder, self.engine = decoder, engine
        self.batch_size, self.max_new_tokens, self.behavior_topk = max_batch_size, max_new_tokens, behavior_topk
        self.policy_version = engine.policy_version
        self.closed = False
        self.entry = decoder._get_graph(max_batch_size, cache_len or engine.max_model_len, masked=True)
        self.entry.cache.seq_lens.zero_()
        self.rows = _RowTable(max_batch_size, max_new_tokens, behavior_topk, self.entry.active, engine.device)
        self.slots = [_Slot() for _ in range(max_batch_size)]
        self.stops = _StopTables(vocab, engine.device)
        self.sampler = ops.RowSampler(self.entry.logits)
        self.clock = _PhaseClock(profile_timings)
        self._stored: dict = {}
        self._stored_ids = 0
        self._filtered_rows: set = set()
        self.stats: dict = dict.fromkeys(STAT_KEYS, 0)
        self.stats["decode_batches"] = {}
        decoder._active_session = self

    # ------------------------------------------------------------------ state checks
    def _require_open(self) -> None:
        mine = self.decoder._active_session is self and self.engine._cuda_decoder is self.decoder
        if self.closed or not mine:
            _refuse("closed")
        if self.engine.policy_version != self.policy_version:
            _refuse("session_policy")

    def timing_stats(self) -> dict:
        """GPU seconds per phase (`prefill`, `cache_copy`, `append`), resolved once, outside the hot loop."""
        return self.clock.totals()

    def _violations(self, prompt, sampling: LFM25SamplingConfig):
        """(broken, message) for every rule a request must meet, in checking order; evaluated lazily, so a later rule
        may rely on the earlier ones."""
        vocab, table = self.engine.config.vocab_size, sampling.stop_table
        # the order and the texts of lfm25_session.py:205-225; top-k / top-p requests, which the reference refuses with
        # the same sentence, are accepted here (an extension: such rows are redrawn by the filtered sampler)
        yield sampling.behavior_topk > self.behavior_topk, "Request behavior head exceeds the session reservation"
        yield not prompt, "Empty prompts are not supported"
        # three C-level passes over the ids instead of a Python loop
        yield (set(map(type, prompt)) != {int} or min(prompt) < 0 or max(prompt) >= vocab), "Prompt token outside the model vocabulary"
        yield (len(prompt) + sampling.max_new_tokens > self.entry.cache.max_seq_len), "Request exceeds reserved session context capacity"
        yield sampling.max_new_tokens > self.max_new_tokens, "Request exceeds the session generation buffer"
        yield (sampling.repetition_penalty != 1.0,
               "Sessions support greedy/full-support sampling without repetition penalties")
        yield (bool(sampling.stop_token_sequences),
               "Sessions use stop_token_ids or stop_table; encode string stops with build_stop_table")
        yield any(not 0 <= token < vocab for token in sampling.stop_token_ids), "Stop token outside the model vocabulary"
        yield (table is not None and (table.ndim != 2 or table.size(1) != vocab or table.dtype != torch.int32),
               "stop_table must be an int32 state-by-vocabulary table")

    def _validate(self, prompt, sampling: LFM25SamplingConfig) -> None:
        for broken, message in self._violations(prompt, sampling):
            reject(broken, message)

    def _claim(self, wanted, count: int, purpose: str) -> list:
        """`count` free slots: the lowest ones, or exactly the requested ones."""
        if wanted is None:
            chosen = [i for i, slot in enumerate(self.slots) if not slot.busy][:count]
        else:
            chosen = [int(i) for i in wanted]
        ok = (len(chosen) == count and len(set(chosen)) == count
              and all(0 <= i < self.batch_size and not self.slots[i].busy for i in chosen))
        reject(not ok, f"{purpose} requires distinct free session slots")
        return chosen

    def _start(self, work, *, carried=None) -> None:
        """Make (slot, prompt, sampling) the running request of each slot: host records, then every device column of
        every row in one launch.  `carried[slot]` = (random-stream position, stop state) for rows that keep them."""
        specs = []
        for index, prompt, sampling in work:
            slot = self.slots[index]
            slot.generation += 1
            slot.prompt, slot.sampling, slot.lease, slot.used_before = tuple(prompt), sampling, None, True
            (self._filtered_rows.add if filtered_on_device(sampling) else self._filtered_rows.discard)(index)
            position, stop_state = (0, 0) if carried is None else carried[index]
            specs.append(_RowTable.spec(index, sampling, self.stops.offset(sampling), position, stop_state))
        self.rows.write(specs)
        self.stats["peak_live_slots"] = max(self.stats["peak_live_slots"], sum(slot.busy for slot in self.slots))

    def _graph_for(self, rows):
        known = len(self.entry.compact_graphs)
        graph, width = self.decoder._select_graph(self.entry, rows)
        self.stats["adaptive_graph_captures"] += len(self.entry.compact_graphs) - known
        return graph, width

    # ------------------------------------------------------------------ admission
    @_no_grad()
    def admit(self, prompts: Sequence[Sequence[int]], samplings: Sequence[LFM25SamplingConfig], *,
              slots: Sequence[int] | None = None) -> list:
        self._require_open()
        if len(prompts) != len(samplings):
            _refuse("sampling_per_prompt")
        chosen = self._claim(slots, len(prompts), "Admission")
        for prompt, sampling in zip(prompts, samplings):
            self._validate(prompt, sampling)
        if not chosen:
            return chosen
        refills = sum(self.slots[i].used_before for i in chosen)
        flat, bounds, longest = flatten_token_batches(prompts, device=self.engine.device)
        with self.clock("prefill"):
            # one packed prefill for the whole admission: each sequence lands in its own slot of the session cache
            self.engine.prefill(flat, bounds, longest, cache=self.entry.cache, slots=chosen, logits_buffer=self.entry.logits,
                                max_prefill_tokens=self.decoder.max_prefill_tokens)
        self.stats["slot_refills"] += refills
        self.stats["prefilled_tokens"] += int(flat.numel())
        self.stats["admitted_requests"] += len(chosen)
        self._start(list(zip(chosen, prompts, samplings)))
        return chosen

    # ------------------------------------------------------------------ stored prefixes
    def _store(self, prefix: _StoredPrefix) -> LFM25PrefixSnapshot:
        self._stored[prefix.lease.identity] = prefix
        self.stats["snapshot_count"] += 1
        self.stats["peak_snapshots"] = max(self.stats["peak_snapshots"], len(self._stored))
        self.stats["peak_snapshot_bytes"] = max(self.stats["peak_snapshot_bytes"], sum(p.nbytes() for p in self._stored.values()))
        return prefix.lease

    def _new_lease(self, tokens) -> LFM25PrefixSnapshot:
        self._stored_ids += 1
        return LFM25PrefixSnapshot(self, self._stored_ids, self.policy_version, tuple(tokens))

    def _lookup(self, snapshot: LFM25PrefixSnapshot) -> _StoredPrefix:
        self._require_open()
        if snapshot.policy_version != self.engine.policy_version:
            _refuse("snapshot_policy")
        stored = self._stored.get(snapshot.identity) if snapshot.session is self else None
        if stored is None or stored.lease is not snapshot:
            _refuse("snapshot_gone")
        return stored

    @_no_grad()
    def prefill_snapshot(self, prompt: Sequence[int]) -> LFM25PrefixSnapshot:
        """Prefill one exact prefix once under the current weights, outside the session's slots."""
        self._require_open()
        prompt = tuple(prompt)
        self._validate(prompt, LFM25SamplingConfig(max_new_tokens=1))
        cache = self.engine._empty_cache(max_slots=1, max_seq_len=len(prompt), fp8_kv=self.entry.cache.fp8)
        with self.clock("prefill"):
            done = self.engine.prefill(*flatten_token_batches([prompt], device=self.engine.device), cache=cache,
                                       max_prefill_tokens=self.decoder.max_prefill_tokens)
        self.stats["prefilled_tokens"] += len(prompt)
        self.stats["snapshot_prefilled_tokens"] += len(prompt)
        return self._store(_StoredPrefix(self._new_lease(prompt), cache, done.next_token_logits))

    @_no_grad()
    def snapshot(self, handle: LFM25ContinuationHandle) -> LFM25PrefixSnapshot:
        """Copy a delivered row: the valid part of its KV bytes and scales, its conv state, its logits and the token it
        still owes the model."""
        slot = self._leased(handle)
        cached = len(handle.prefix_token_ids) - 1
        if int(self.entry.cache.seq_lens[handle.slot]) != cached:
            _refuse("position_mismatch")
        with self.clock("cache_copy"):
            row = self.entry.cache.rows(handle.slot, handle.slot + 1)
            history = [None if t is None else t[:, :, :cached].clone() for t in (row.k_cache, row.v_cache, row.k_scales, row.v_scales)]
            copy = LFM25HybridCache(history[0], history[1], row.conv_state.clone(), row.seq_lens.clone(), history[2], history[3])
            logits = self.entry.logits[handle.slot:handle.slot + 1].clone()
        state = self.rows
        return self._store(_StoredPrefix(self._new_lease(handle.prefix_token_ids), copy, logits, handle.prefix_token_ids[-1],
                                         slot.sampling.seed, int(state.rng_positions[handle.slot]), int(state.stop_states[handle.slot])))

    def release_snapshot(self, snapshot: LFM25PrefixSnapshot) -> None:
        del self._stored[self._lookup(snapshot).lease.identity]

    @_no_grad()
    def fork(self, snapshot: LFM25PrefixSnapshot, samplings: Sequence[LFM25SamplingConfig], *,
             slots: Sequence[int] | None = None) -> list:
        """Start independent children of a stored prefix in free slots without any prefill."""
        stored = self._lookup(snapshot)
        chosen = self._claim(slots, len(samplings), "Fork")
        for sampling in samplings:
            self._validate(snapshot.prefix_token_ids, sampling)
        if not chosen:
            return chosen
        cached = stored.cache.max_seq_len
        where = torch.tensor(chosen, device=self.engine.device)
        target, source = self.entry.cache, stored.cache
        with self.clock("cache_copy"):
            for mine, theirs in ((target.k_cache, source.k_cache), (target.v_cache, source.v_cache),
                                 (target.k_scales, source.k_scales), (target.v_scales, source.v_scales)):
                if mine is not None:   # bytes as they are (an e4m3 cache is never dequantised), broadcast over the children
                    _raw(mine)[:, where, :cached] = _raw(theirs)
            target.conv_state[:, where] = source.conv_state
            target.seq_lens[where] = source.seq_lens
            self.entry.logits[where] = stored.logits
        if stored.pending_token is not None:
            # the stored row's last sampled token is not in the cache yet: every child consumes it once
            with self.clock("append"):
                self._feed({index: [stored.pending_token] for index in chosen})
        self.stats["slot_refills"] += sum(self.slots[i].used_before for i in chosen)
        self.stats["forked_requests"] += len(chosen)
        self.stats["copied_prefix_tokens"] += cached * len(chosen)
        self._start([(index, snapshot.prefix_token_ids, sampling) for index, sampling in zip(chosen, samplings)])
        return chosen

    # ------------------------------------------------------------------ continuation
    def _leased(self, handle: LFM25ContinuationHandle) -> _Slot:
        self._require_open()
        if handle.session is not self or not 0 <= handle.slot < self.batch_size:
            _refuse("foreign_handle")
        slot = self.slots[handle.slot]
        if slot.lease is not handle or slot.generation != handle.version:
            _refuse("stale_handle")
        return slot

    def _feed(self, queues: dict) -> None:
        """Append tokens to cached rows: `queues[slot]` is consumed one position per replay while the other rows sit
        out; their own pending flags and next inputs are put back afterwards."""
        depth = max(map(len, queues.values()))
        plan = torch.full((depth, self.batch_size), -1, dtype=torch.long)
        for index, tokens in queues.items():
            plan[:len(tokens), index] = torch.tensor(tokens, dtype=torch.long)
        plan = plan.to(self.engine.device)
        feeding = plan >= 0
        owed_tokens, owed_flags = self.entry.input_tokens.clone(), self.rows.pending.clone()
        graph, _ = self._graph_for(sorted(queues))
        for step in range(depth):
            self.entry.input_tokens.copy_(plan[step].clamp_min(0))
            self.rows.pending.copy_(feeding[step])
            graph.replay()
        self.entry.input_tokens.copy_(owed_tokens)
        self.rows.pending.copy_(owed_flags)

    @_no_grad()
    def resume(self, handles: Sequence[LFM25ContinuationHandle], prompts: Sequence[Sequence[int]],
               samplings: Sequence[LFM25SamplingConfig], *, preserve_rng: bool = False) -> None:
        """Continue delivered rows from an exact extension of what they hold: the owed token and the new suffix are
        appended under per-row masks, then the rows run again.  `preserve_rng` keeps the random stream's position and
        the stop automaton's state (an internal pause of the same request)."""
        if not len(handles) == len(prompts) == len(samplings):
            _refuse("per_handle")
        if len({handle.slot for handle in handles}) != len(handles):
            _refuse("twice")
        queues, carried = {}, {}
        for handle, prompt, sampling in zip(handles, prompts, samplings):
            slot = self._leased(handle)
            self._validate(prompt, sampling)
            held = handle.prefix_token_ids
            if tuple(prompt[:len(held)]) != held:
                _refuse("prefix_differs")
            if preserve_rng:
                before = slot.sampling
                if (len(prompt) != len(held) or sampling.seed != before.seed or sampling.stop_table is not before.stop_table
                        or sampling.stop_token_ids != before.stop_token_ids):
                    _refuse("pause_rules")
            queues[handle.slot] = [held[-1], *prompt[len(held):]]
        if not queues:
            return
        if preserve_rng:
            positions, states = self.rows.rng_positions.cpu().tolist(), self.rows.stop_states.cpu().tolist()
            carried = {index: (positions[index], states[index]) for index in queues}
        with self.clock("append"):
            self._feed(queues)
        for handle, prompt in zip(handles, prompts):
            self.stats["resumed_prefix_tokens"] += len(handle.prefix_token_ids) - 1
            self.stats["appended_tokens"] += len(prompt) - len(handle.prefix_token_ids) + 1
        self.stats["resumed_requests"] += len(handles)
        self._start([(handle.slot, prompt, sampling) for handle, prompt, sampling in zip(handles, prompts, samplings)],
                    carried=carried or None)

    # ------------------------------------------------------------------ the hot loop
    def _draw(self, every_row_filtered=False):
        state = self.rows
        if every_row_filtered:    # no running row keeps the full-support draw: its two launches are left out
            tokens, logprobs = self.sampler.tokens, self.sampler.logprobs
        else:
            tokens, logprobs = self.sampler.sample(self.entry.logits, state.seeds, state.rng_positions, state.temperatures)
        if self._filtered_rows:   # rows with top-k / top-p are redrawn with their own parameters; the others are skipped
            ops.sample_filtered(self.entry.logits, seeds=state.seeds, steps=state.rng_positions, temperatures=state.temperatures,
                                top_ks=state.top_ks, top_ps=state.top_ps, out=(tokens, logprobs))
        return tokens, logprobs

    @_no_grad()
    def poll(self, *, steps: int | None = None) -> list:
        """Run `steps` decode steps (default: the decoder's finish-check interval) and hand out what finished."""
        self._require_open()
        steps = self.decoder.finish_check_interval if steps is None else steps
        if type(steps) is not int or steps <= 0:
            _refuse("steps")
        running = [index for index, slot in enumerate(self.slots) if slot.running]
        if not running:
            return []
        graph, width = self._graph_for(running)
        state, config = self.rows, self.engine.config
        fused_record = not self._filtered_rows and not self.behavior_topk
        every_row_filtered = self._filtered_rows.issuperset(running)
        for _ in range(steps):
            graph.replay()       # consumes the owed token of every row whose pending flag is set
            if fused_record:     # no redraw and no behaviour head between the draw and its record: one launch less
                ops.sample_and_record(self.sampler, self.entry.logits, state, self.entry.input_tokens, self.stops.flat,
                                      config.eos_token_id, self.max_new_tokens)
                continue
            tokens, logprobs = self._draw(every_row_filtered)
            if self.behavior_topk:
                ids, values = ops.behavior_topk(self.entry.logits, tokens, logprobs, self.behavior_topk)
                ops.record_head(ids, values, state.head_ids, state.head_logprobs, state.lengths, state.alive,
                                self.behavior_topk, self.max_new_tokens)
            ops.record_sample(tokens, logprobs, state.tokens, state.logprobs, state.lengths, state.limits, state.reasons,
                              state.alive, state.pending, self.entry.input_tokens, state.stop_states, state.stop_offsets,
                              self.stops.flat, state.ignore_eos, state.rng_positions, config.eos_token_id, config.vocab_size,
                              self.max_new_tokens)
        self.stats["decode_steps"] += steps
        self.stats["decode_row_steps"] += width * steps
        self.stats["reserved_row_steps"] += self.batch_size * steps
        histogram = self.stats["decode_batches"]
        histogram[str(width)] = histogram.get(str(width), 0) + steps
        return self._hand_out(running)

    def _hand_out(self, running) -> list:
        """Results of the running rows that now carry a finish code (one device read for the codes, one per column for
        the finished rows only)."""
        codes = self.rows.reasons.cpu().tolist()
        finished = [index for index in running if codes[index]]
        if not finished:
            return []
        state = self.rows
        where = torch.tensor(finished, device=self.engine.device)
        counts = state.lengths[where].cpu().tolist()
        span = max(counts)
        token_rows = state.tokens[where, :span].cpu().tolist()
        logprob_rows = state.logprobs[where, :span].cpu().tolist()
        results = []
        for index, count, ids, values in zip(finished, counts, token_rows, logprob_rows):
            slot = self.slots[index]
            ids = tuple(ids[:count])
            slot.lease = LFM25ContinuationHandle(self, index, slot.generation, slot.prompt + ids)
            head = None
            if slot.sampling.behavior_topk:
                k = slot.sampling.behavior_topk
                head = BehaviorTopK(state.head_ids[index, :count, :k].cpu(), state.head_logprobs[index, :count, :k].cpu())
            results.append(LFM25SessionResult(slot.lease, slot.prompt, ids,
                                              tuple(values[:count]) if slot.sampling.return_logprobs else None,
                                              codes[index], head))
        return results

    @_no_grad()
    def release(self, handle: LFM25ContinuationHandle) -> None:
        """Give a delivered row's slot back."""
        slot = self._leased(handle)
        slot.generation += 1
        slot.prompt = slot.sampling = slot.lease = None
        self._filtered_rows.discard(handle.slot)
        self.rows.retire(handle.slot)
        self.entry.cache.seq_lens[handle.slot] = 0

    def close(self) -> None:
        if self.closed:
            return
        self.closed = True
        for slot in self.slots:
            slot.generation += 1
            slot.prompt = slot.sampling = slot.lease = None
        self._stored.clear()
        if self.decoder._active_session is self:
            self.decoder._active_session = None

    def __enter__(self):
        self._require_open()
        return self

    def __exit__(self, *_):
        self.close()


def _raw(tensor: torch.Tensor) -> torch.Tensor:
    """One-byte element types as uint8, so that indexed copies move e4m3 codes as they are."""
    return tensor.view(torch.uint8) if tensor.element_size() == 1 else tensor
