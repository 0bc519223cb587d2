"""Async batching adapter over the token engine (lfm25_async_engine.py of the reference).

Text requests are rendered and tokenised on the caller's event loop, queued, grouped by sampling settings and run as
one `LFM25Engine.generate` call per group on a worker thread; `generate_chains` drives multi-phase requests through
a generation session with continuous admission.  The adapter is host code only: every device operation happens
inside the engine it wraps.  One lock serialises engine work (`sync_from_model` drains through the same lock).
"""
from __future__ import annotations

import asyncio
import gc
import math
import threading
import uuid
from dataclasses import dataclass, replace
from typing import Any, Callable, Mapping, Sequence

import torch

from .config import LFM25SamplingConfig
from .inference_config import InferenceEngineConfig, SamplingConfig
from .text_stops import build_stop_table, trim_after_stop
from .types import BehaviorTopK, GenerationOutput, GenerationResult, PromptInput
from ._checks import reject

_MASK63 = 0x7FFFFFFFFFFFFFFF
_CHAIN_STRIDE = 0x517CC1B727220A95   # odd 64-bit constants: chain and phase index spread over the whole key
_PHASE_STRIDE = 0x6C8E9CF570932BD5
_FINISH = {1: ("stop", "eos"), 2: ("stop", "stop"), 3: ("length", None)}
_STOP_PREFIXES = ("", " ", "\n", ">")


def decode_finish_reason(code: int):
    """Engine finish code -> (finish_reason, stop_reason) (lfm25_async_engine.py:712-719)."""
    return _FINISH.get(int(code), (None, None))


def chain_seed(base: int, chain: int, phase: int) -> int:
    """RNG key of one phase of one chain: independent of slot assignment and of which other chains finished at the
    same time (lfm25_async_engine.py:349)."""
    return (base + chain * _CHAIN_STRIDE + phase * _PHASE_STRIDE) & _MASK63


def to_native_sampling(sampling: SamplingConfig, *, seed: int, tokenizer=None) -> LFM25SamplingConfig:
    """Request-level sampling -> engine sampling (lfm25_async_engine.py:688-709).  String stops become the token
    sequences of the stop text after the usual joiners; `top_k == -1` means no top-k."""
    reject(int(sampling.n) != 1, "LFM25AsyncInferenceEngine requires sampling.n == 1")
    reject(sampling.stop and tokenizer is None, "A tokenizer is required for string stop sequences")
    extra = dict(sampling.extra_params)
    sequences = []
    for text in sampling.stop:
        for prefix in _STOP_PREFIXES:
            ids = tuple(tokenizer.encode(prefix + text, add_special_tokens=False))
            if ids not in sequences:
                sequences.append(ids)
    return LFM25SamplingConfig(
        temperature=float(sampling.temperature), top_k=max(int(sampling.top_k), 0), top_p=float(sampling.top_p),
        repetition_penalty=float(extra.get("repetition_penalty", 1.0)), max_new_tokens=int(sampling.max_tokens),
        return_logprobs=sampling.logprobs is not None, seed=seed, ignore_eos=bool(extra.get("ignore_eos", False)),
        stop_token_sequences=tuple(sequences), behavior_topk=extra.get("behavior_topk", 0))


def _batch_limit(config: InferenceEngineConfig, requested) -> int:
    reject(requested is not None and (type(requested) is not int or requested <= 0),
           "max_batch_size must be a positive integer")
    limit = requested if requested is not None else (config.max_num_seqs or 64)
    return limit if config.max_num_seqs is None else min(limit, config.max_num_seqs)


@dataclass
class _Queued:
    prompt: Any
    prompt_text: str
    prompt_token_ids: tuple
    sampling: SamplingConfig
    request_id: str
    future: asyncio.Future


class _PromptRenderer:
    """Prompt -> (echoed prompt, text, token ids) exactly as generation sees it (lfm25_async_engine.py:594-672)."""

    def __init__(self, config: InferenceEngineConfig, tokenizer):
        self.config, self.tokenizer = config, tokenizer

    def encode(self, text: str) -> tuple:
        return tuple(int(t) for t in self.tokenizer.encode(str(text), add_special_tokens=False))

    def chat(self, prompt: str, enable_thinking) -> str:
        if not self.config.apply_chat_template:
            return str(prompt)
        template = getattr(self.tokenizer, "apply_chat_template", None)
        reject(not callable(template),
               "apply_chat_template=true requires a tokenizer with apply_chat_template(...)", TypeError)
        thinking = self.config.chat_template_enable_thinking if enable_thinking is None else enable_thinking
        messages = [{"role": "user", "content": str(prompt)}]
        options = {"tokenize": False, "add_generation_prompt": True}
        try:
            return str(template(messages, enable_thinking=bool(thinking), **options))
        except TypeError as error:  # tokenizers whose template has no thinking switch
            text = str(error)
            if "enable_thinking" in text and ("unexpected keyword" in text or "got an unexpected" in text):
                return str(template(messages, **options))
            raise

    def __call__(self, prompt: PromptInput, *, assistant_prefill: str = "", enable_thinking=None):
        prefill = str(assistant_prefill or "")
        if isinstance(prompt, Mapping):
            text = str(prompt.get("prompt", prompt.get("text", "")) or "")
            given = prompt.get("prompt_token_ids")
            ids = self.encode(text) if given is None else tuple(int(t) for t in given or ())
            if not prefill:
                return prompt, text, ids
            text, ids = text + prefill, ids + self.encode(prefill)
            echoed = dict(prompt)
            for key in ("prompt", "text"):
                if key in echoed:
                    echoed[key] = text
                    break
            echoed["prompt_token_ids"] = list(ids)
            return echoed, text, ids
        if isinstance(prompt, str):
            text = self.chat(prompt, enable_thinking) + prefill
            return text, text, self.encode(text)
        ids = tuple(int(t) for t in prompt)
        text = self.tokenizer.decode(ids, skip_special_tokens=False)
        if prefill:
            text, ids = text + prefill, ids + self.encode(prefill)
        return list(ids), text, ids


class LFM25AsyncInferenceEngine:
    """lfm25_async_engine.py:35-729: `generate`, `generate_many`, `generate_chains`, `sync_from_model`, `abort`,
    `close`, `sleep`/`wake`, with the reference's seed ledger (`seed + index mod 2^64` per engine call)."""

    def __init__(self, config: InferenceEngineConfig, *, batch_wait_seconds: float = 0.001, max_batch_size=None,
                 cuda_graphs: bool = True, max_cuda_graphs: int = 1, max_prefill_tokens: int = 4096,
                 fp8_mlp: bool = False, fp8_kv: bool = False, adaptive_batching: bool = False,
                 fp8_lm_head: bool = False, fp8_operators: bool = False, compile_decode: bool = True,
                 bf16_weight_packing: bool = True):
        del compile_decode, bf16_weight_packing  # no tracing compiler and no separate bf16 packing on this path
        for flag, name in ((fp8_mlp, "FP8 MLP"), (fp8_kv, "FP8 KV cache"), (adaptive_batching, "adaptive batching"),
                           (fp8_lm_head, "FP8 vocabulary head"), (fp8_operators, "FP8 operators")):
            reject(flag and not cuda_graphs, f"Native {name} requires cuda_graphs=True")
        from transformers import AutoTokenizer
        from .engine import LFM25Engine
        tokenizer = AutoTokenizer.from_pretrained(config.model_path, local_files_only=True)
        dtype = torch.bfloat16 if config.dtype in ("auto", "bfloat16", "bf16") else getattr(torch, str(config.dtype))
        engine = LFM25Engine.from_pretrained(config.model_path, device="cuda", dtype=dtype,
                                             max_model_len=config.max_model_len)
        self._setup(engine, tokenizer, config, batch_wait_seconds, _batch_limit(config, max_batch_size), owned=True)
        try:
            if cuda_graphs:
                engine.enable_cuda_graphs(max_graphs=max_cuda_graphs, max_prefill_tokens=max_prefill_tokens,
                                          fp8_mlp=fp8_mlp, fp8_kv=fp8_kv, adaptive_batching=adaptive_batching,
                                          fp8_lm_head=fp8_lm_head, fp8_operators=fp8_operators)
        except BaseException:
            self.close()
            raise

    @classmethod
    def from_components(cls, *, engine, tokenizer, config: InferenceEngineConfig | None = None,
                        batch_wait_seconds: float = 0.0, max_batch_size: int = 64):
        """Wrap an engine and tokenizer the caller owns (lfm25_async_engine.py:107-130)."""
        self = cls.__new__(cls)
        config = config or InferenceEngineConfig(model_path="")
        self._setup(engine, tokenizer, config, batch_wait_seconds, _batch_limit(config, max_batch_size), owned=False)
        return self

    def _setup(self, engine, tokenizer, config, wait, limit, *, owned):
        self.config, self.tokenizer = config, tokenizer
        self.batch_wait_seconds = max(0.0, float(wait))
        self.max_batch_size = limit
        self._engine, self._owns_engine = engine, owned
        self._render = _PromptRenderer(config, tokenizer)
        self._pending: list[_Queued] = []
        self._pending_lock: asyncio.Lock | None = None
        self._flush_task: asyncio.Task | None = None
        self._closed = False
        self._engine_lock = threading.Lock()
        self._seed_lock = threading.Lock()
        self._generation_index = 0
        self._stop_tables: dict = {}
        self.last_session_stats: dict = {}

    # ------------------------------------------------------------------ small public surface
    @property
    def raw_engine(self):
        reject(self._engine is None, "LFM25AsyncInferenceEngine is closed", RuntimeError)
        return self._engine

    def supports_token_prompt_bridge(self) -> bool:
        return True

    def tokenize_prompt(self, prompt: PromptInput, *, assistant_prefill: str | None = None,
                        chat_template_enable_thinking: bool | None = None) -> tuple:
        """Render and tokenise without generating."""
        prefill = self.config.assistant_prefill if assistant_prefill is None else assistant_prefill
        return self._render(prompt, assistant_prefill=str(prefill), enable_thinking=chat_template_enable_thinking)[2]

    @classmethod
    def tokenize_for_config(cls, config: InferenceEngineConfig, tokenizer, prompt: PromptInput, *,
                            assistant_prefill: str | None = None, chat_template_enable_thinking: bool | None = None):
        """The same rendering with only a tokenizer at hand (no engine, no device state)."""
        prefill = config.assistant_prefill if assistant_prefill is None else assistant_prefill
        return _PromptRenderer(config, tokenizer)(prompt, assistant_prefill=str(prefill),
                                                  enable_thinking=chat_template_enable_thinking)[2]

    def _check_open(self):
        reject(self._closed, "LFM25AsyncInferenceEngine is closed", RuntimeError)

    def sync_from_model(self, model, *, drain_timeout: int | float = 300):
        """Wait for running generation to drain, then update the packed weights in place."""
        timeout = float(drain_timeout)
        reject(not math.isfinite(timeout) or timeout < 0.0, "drain_timeout must be finite and >= 0")
        self._check_open()
        if not self._engine_lock.acquire(timeout=timeout):
            raise TimeoutError(f"Timed out after {timeout:g}s waiting for native LFM2.5 generation to drain")
        try:
            self._check_open()
            return self._engine.sync_from_model(model, drain_timeout=drain_timeout)
        finally:
            self._engine_lock.release()

    def release_inference_buffers(self) -> None:
        with self._engine_lock:
            if self._engine is not None:
                self._engine.release_inference_buffers()

    def sleep(self, *, level: int = 1, mode: str = "abort") -> None:
        del level, mode
        self.release_inference_buffers()

    def wake(self, *, tags: Sequence[str] | None = None) -> None:
        del tags

    def close(self) -> None:
        """Cancel queued requests, wait for the running call, drop the engine (and free it when this adapter loaded it)."""
        self._closed = True
        queued, self._pending = self._pending, []
        for item in queued:
            if not item.future.done():
                item.future.cancel()
        with self._engine_lock:
            engine, self._engine = self._engine, None
            if engine is None:
                return
            self._stop_tables.clear()
            if self._owns_engine:
                engine.release_inference_buffers()
        if self._owns_engine:
            del engine
            gc.collect()
            if torch.cuda.is_available():
                torch.cuda.empty_cache()

    # ------------------------------------------------------------------ sampling helpers
    def _resolve_sampling(self, sampling) -> SamplingConfig:
        if sampling is None:
            return self.config.default_sampling
        if isinstance(sampling, SamplingConfig):
            return sampling
        reject(isinstance(sampling, Mapping),
               "sampling must be a SamplingConfig or a sampling-attribute object, not a mapping", TypeError)
        read = lambda name, default: getattr(sampling, name, default)
        return SamplingConfig(temperature=float(read("temperature", 0.0)), top_k=int(read("top_k", -1)),
                              top_p=float(read("top_p", 1.0)),
                              max_tokens=int(read("max_tokens", read("max_new_tokens", 256))), n=int(read("n", 1)),
                              logprobs=read("logprobs", None), stop=read("stop", ()) or (),
                              extra_params=read("extra_params", {}) or {})

    def _native_sampling(self, sampling: SamplingConfig, seed: int) -> LFM25SamplingConfig:
        native = to_native_sampling(sampling, seed=seed, tokenizer=self.tokenizer)
        if not sampling.stop:
            return native
        key = tuple(sampling.stop)
        if key not in self._stop_tables:  # one automaton per distinct stop set, kept on the device
            table = build_stop_table(self.tokenizer, key, vocab_size=self._engine.config.vocab_size)
            self._stop_tables[key] = table.to(self._engine.device)
        return replace(native, stop_token_sequences=(), stop_table=self._stop_tables[key])

    def _next_generation_seed(self) -> int:
        with self._seed_lock:
            index = self._generation_index
            self._generation_index += 1
        return (int(self.config.seed) + index) % (1 << 64)

    def _output(self, sampling: SamplingConfig, token_ids, logprobs, code, head) -> GenerationOutput:
        finish, stop = decode_finish_reason(code)
        text = self.tokenizer.decode(token_ids, skip_special_tokens=False)
        if stop == "stop" and sampling.stop:  # a string stop may end inside the last token: ids stay, text is cut
            text = trim_after_stop(text, sampling.stop)
        return GenerationOutput(0, text, tuple(token_ids), logprobs, finish, stop, head)

    # ------------------------------------------------------------------ single-phase requests
    async def generate(self, prompt: PromptInput, *, sampling=None, request_id: str | None = None,
                       chat_template_enable_thinking: bool | None = None, assistant_prefill: str = "") -> GenerationResult:
        self._check_open()
        resolved = self._resolve_sampling(sampling)
        echoed, text, ids = self._render(prompt, assistant_prefill=str(assistant_prefill or self.config.assistant_prefill),
                                         enable_thinking=chat_template_enable_thinking)
        future = asyncio.get_running_loop().create_future()
        await self._enqueue(_Queued(echoed, text, ids, resolved, request_id or f"req-{uuid.uuid4().hex}", future))
        return await future

    async def generate_many(self, prompts: Sequence[PromptInput], *, sampling=None) -> list:
        return list(await asyncio.gather(*(self.generate(p, sampling=sampling) for p in prompts)))

    def _lock(self) -> asyncio.Lock:
        if self._pending_lock is None:
            self._pending_lock = asyncio.Lock()
        return self._pending_lock

    async def _enqueue(self, item: _Queued) -> None:
        async with self._lock():
            self._check_open()
            self._pending.append(item)
            if self._flush_task is None or self._flush_task.done():
                self._flush_task = asyncio.create_task(self._drain_queue())

    async def _drain_queue(self) -> None:
        """Repeatedly take the oldest request and everything queued with the same sampling key (up to the batch
        limit) and run them as one engine call."""
        if self.batch_wait_seconds > 0:
            await asyncio.sleep(self.batch_wait_seconds)
        while True:
            async with self._lock():
                if not self._pending:
                    return
                key = self._pending[0].sampling.batching_key()
                batch, rest = [], []
                for item in self._pending:
                    mine = len(batch) < self.max_batch_size and item.sampling.batching_key() == key
                    (batch if mine else rest).append(item)
                self._pending = rest
            loop = asyncio.get_running_loop()
            try:
                results = await loop.run_in_executor(None, self._run_batch, tuple(batch))
            except Exception as error:
                for item in batch:
                    if not item.future.done():
                        item.future.set_exception(error)
                continue
            for item, result in zip(batch, results):
                if not item.future.done():
                    item.future.set_result(result)

    def _run_batch(self, batch: tuple) -> list:
        from .engine import flatten_token_batches
        with self._engine_lock:
            self._check_open()
            native = self._native_sampling(batch[0].sampling, self._next_generation_seed())
            flat = flatten_token_batches([list(item.prompt_token_ids) for item in batch], device=self._engine.device)
            output = self._engine.generate(*flat, repeats=1, sampling=native)
            if torch.cuda.is_available():
                torch.cuda.synchronize()
            return self._collect(batch, output)

    def _collect(self, batch, output) -> list:
        """One host transfer per output tensor, then per-request slices."""
        lengths = output.lengths[:, 0].cpu().tolist()
        longest = max(lengths, default=0)
        tokens = output.token_ids[:, 0, :longest].cpu().tolist()
        reasons = output.finish_reasons[:, 0].cpu().tolist()
        logprobs = None if output.logprobs is None else output.logprobs[:, 0, :longest].cpu().tolist()
        head_ids = getattr(output, "topk_token_ids", None)
        head_lp = getattr(output, "topk_logprobs", None)
        if head_ids is not None:
            head_ids, head_lp = head_ids[:, 0, :longest].cpu(), head_lp[:, 0, :longest].cpu()
        results = []
        for row, item in enumerate(batch):
            n = lengths[row]
            head = None if head_ids is None else BehaviorTopK(head_ids[row, :n].clone(), head_lp[row, :n].clone())
            completion = self._output(item.sampling, tokens[row][:n],
                                      None if logprobs is None else tuple(logprobs[row][:n]), reasons[row], head)
            results.append(GenerationResult(item.request_id, item.prompt, item.prompt_token_ids, (completion,), True,
                                            output if head_ids is None else None))
        return results

    async def abort_async(self, request_id) -> None:
        wanted = {str(request_id)} if isinstance(request_id, str) else {str(r) for r in request_id}
        async with self._lock():
            keep = []
            for item in self._pending:
                if item.request_id in wanted:
                    item.future.cancel()
                else:
                    keep.append(item)
            self._pending = keep

    def abort(self, request_id) -> None:
        try:
            loop = asyncio.get_running_loop()
        except RuntimeError:
            asyncio.run(self.abort_async(request_id))
        else:
            loop.create_task(self.abort_async(request_id))

    # ------------------------------------------------------------------ multi-phase chains
    async def generate_chains(self, requests: Sequence, *, on_result: Callable, max_new_tokens: int,
                              reuse_cache: bool = True, poll_interval: int | None = None) -> list:
        """Run independent, possibly multi-phase requests with continuous admission (lfm25_async_engine.py:278-409).
        `on_result(index, result)` runs on the worker thread and returns the next (prompt, sampling) of that chain or
        None.  A next prompt that extends the cached prefix exactly resumes in place; anything else starts fresh."""
        self._check_open()
        if not requests:
            return []
        cancelled = threading.Event()
        worker = asyncio.get_running_loop().run_in_executor(
            None, self._run_chains, tuple(requests), on_result, max_new_tokens, reuse_cache, poll_interval, cancelled)
        try:
            return await asyncio.shield(worker)
        except asyncio.CancelledError:
            cancelled.set()
            try:  # the session (and its cache lease) must be gone before the caller continues
                await asyncio.shield(worker)
            except Exception:
                pass
            raise

    def _run_chains(self, requests, on_result, max_new_tokens, reuse_cache, poll_interval, cancelled):
        with self._engine_lock:
            self._check_open()
            results = [[] for _ in requests]
            if cancelled.is_set():
                return results
            base = self._next_generation_seed()
            phase = [0] * len(requests)
            prefill = str(self.config.assistant_prefill)

            def prepare(index, request):
                prompt, sampling = request
                sampling = self._resolve_sampling(sampling)
                echoed, _, ids = self._render(prompt, assistant_prefill=prefill)
                native = self._native_sampling(sampling, chain_seed(base, index, phase[index]))
                return index, echoed, ids, sampling, native

            backlog = iter(enumerate(requests))
            head = max(int(dict(self._resolve_sampling(s).extra_params).get("behavior_topk", 0)) for _, s in requests)
            options = {"behavior_topk": head} if head else {}
            running = {}
            with self._engine.generation_session(max_batch_size=min(self.max_batch_size, len(requests)),
                                                 max_new_tokens=max_new_tokens, **options) as session:
                first = [prepare(*item) for _, item in zip(range(session.batch_size), backlog)]
                slots = session.admit([job[2] for job in first], [job[4] for job in first])
                running.update(zip(slots, first))
                while running and not cancelled.is_set() and not self._closed:
                    continued, restarted = [], []
                    for done in session.poll(steps=poll_interval):
                        slot = done.handle.slot
                        index, echoed, ids, sampling, _ = running.pop(slot)
                        completion = self._output(sampling, done.token_ids, done.logprobs, done.finish_reason,
                                                  getattr(done, "behavior_topk", None))
                        result = GenerationResult(f"chain-{index}-phase-{phase[index]}", echoed, ids, (completion,),
                                                  True, None)
                        results[index].append(result)
                        following = on_result(index, result)
                        if following is None:
                            session.release(done.handle)
                            queued = next(backlog, None)
                            if queued is not None:
                                restarted.append((slot, prepare(*queued)))
                            continue
                        phase[index] += 1
                        job = prepare(index, following)
                        cached = done.handle.prefix_token_ids
                        if reuse_cache and job[2][:len(cached)] == cached:
                            continued.append((done.handle, job))
                        else:
                            session.release(done.handle)
                            restarted.append((slot, job))
                    if continued:
                        session.resume([h for h, _ in continued], [job[2] for _, job in continued],
                                       [job[4] for _, job in continued])
                        running.update((h.slot, job) for h, job in continued)
                    if restarted:
                        session.admit([job[2] for _, job in restarted], [job[4] for _, job in restarted],
                                      slots=[slot for slot, _ in restarted])
                        running.update(restarted)
                self.last_session_stats = dict(session.stats)
            reject(self._closed and not cancelled.is_set(),
                   "LFM25AsyncInferenceEngine closed during generation", RuntimeError)
            return results


__all__ = ["LFM25AsyncInferenceEngine", "chain_seed", "decode_finish_reason", "to_native_sampling"]
