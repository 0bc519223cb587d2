"""Host logic of the async adapter (CPU): request queueing and grouping, the seed ledger, chain keys, prompt
rendering, finish-reason decoding, stop trimming, abort/close.  A scripted engine stands in for the GPU engine; the
scenarios follow tests/test_lfm25_async_engine.py and tests/test_native_chains.py of the reference in spirit
(lfm25_async_engine.py:235-729 is the behaviour under test)."""
import asyncio
from dataclasses import dataclass
from types import SimpleNamespace

import pytest
import torch

from climbing_gym_amd.async_engine import (LFM25AsyncInferenceEngine, chain_seed, decode_finish_reason,
                                           to_native_sampling)
from climbing_gym_amd.inference_config import InferenceEngineConfig, SamplingConfig


class CharTokenizer:
    """One token per character (code point); enough for rendering, stops and decode."""

    def encode(self, text, add_special_tokens=False):
        return [ord(c) for c in text]

    def __len__(self):
        return 128

    def decode(self, ids, skip_special_tokens=False, clean_up_tokenization_spaces=False):
        return "".join(chr(i) for i in ids)

    def apply_chat_template(self, messages, tokenize=False, add_generation_prompt=True, enable_thinking=True):
        body = "".join(f"<{m['role']}>{m['content']}" for m in messages)
        return body + ("<assistant>" if add_generation_prompt else "") + ("" if enable_thinking else "<nothink>")


@dataclass
class _Handle:
    slot: int
    prefix_token_ids: tuple


class ScriptedSession:
    """Finishes every live row at each poll with tokens derived from its seed; records what it was asked."""

    def __init__(self, log, batch_size):
        self.log, self.batch_size, self.rows, self.stats = log, batch_size, {}, {"polls": 0}

    def __enter__(self):
        return self

    def __exit__(self, *_):
        self.log.append(("close",))

    def admit(self, prompts, samplings, slots=None):
        free = [s for s in range(self.batch_size) if s not in self.rows]
        slots = list(slots) if slots is not None else free[:len(prompts)]
        for slot, prompt, sampling in zip(slots, prompts, samplings):
            self.rows[slot] = (tuple(prompt), sampling)
        self.log.append(("admit", tuple(slots), tuple(s.seed for s in samplings)))
        return slots

    def resume(self, handles, prompts, samplings):
        for handle, prompt, sampling in zip(handles, prompts, samplings):
            self.rows[handle.slot] = (tuple(prompt), sampling)
        self.log.append(("resume", tuple(h.slot for h in handles), tuple(s.seed for s in samplings)))

    def release(self, handle):
        self.rows.pop(handle.slot, None)
        self.log.append(("release", handle.slot))

    def poll(self, steps=None):
        self.stats["polls"] += 1
        done = []
        for slot, (prompt, sampling) in sorted(self.rows.items()):
            tokens = tuple(ord("a") + (sampling.seed + i) % 26 for i in range(2))
            done.append(SimpleNamespace(handle=_Handle(slot, prompt + tokens), token_ids=tokens, logprobs=(-0.5, -0.25),
                                        finish_reason=3, behavior_topk=None))
        return done


class ScriptedEngine:
    device = torch.device("cpu")
    config = SimpleNamespace(vocab_size=512)

    def __init__(self):
        self.calls, self.log = [], []

    def generate(self, flat, cu, longest, repeats, sampling):
        rows = cu.numel() - 1
        self.calls.append((rows, sampling))
        length = min(sampling.max_new_tokens, 3)
        tokens = torch.full((rows, 1, length), ord("x"), dtype=torch.long)
        tokens[:, 0, -1] = ord("!")
        return SimpleNamespace(token_ids=tokens, lengths=torch.full((rows, 1), length, dtype=torch.int32),
                               logprobs=torch.zeros(rows, 1, length), finish_reasons=torch.full((rows, 1), 2, dtype=torch.int8),
                               topk_token_ids=None, topk_logprobs=None)

    def generation_session(self, *, max_batch_size, max_new_tokens, **options):
        self.log.append(("session", max_batch_size, max_new_tokens))
        return ScriptedSession(self.log, max_batch_size)

    def sync_from_model(self, model, drain_timeout=300):
        self.log.append(("sync", model))
        return self

    def release_inference_buffers(self):
        self.log.append(("release_buffers",))


def _adapter(engine=None, **config):
    engine = engine or ScriptedEngine()
    adapter = LFM25AsyncInferenceEngine.from_components(
        engine=engine, tokenizer=CharTokenizer(), config=InferenceEngineConfig(model_path="", **config), max_batch_size=4)
    return adapter, engine


def test_requests_group_by_sampling_key_and_respect_the_batch_limit():
    adapter, engine = _adapter(seed=100)
    hot, cold = SamplingConfig(temperature=1.0, max_tokens=8), SamplingConfig(temperature=0.0, max_tokens=8)

    async def scenario():
        jobs = [adapter.generate(f"p{i}", sampling=hot if i % 2 == 0 else cold) for i in range(6)]
        jobs += [adapter.generate(f"q{i}", sampling=hot) for i in range(3)]
        return await asyncio.gather(*jobs)
    results = asyncio.run(scenario())
    assert [r.text for r in results] == ["xx!"] * 9
    # six hot requests: a batch of 4 (the limit) and a batch of 2; three cold ones share one call
    assert sorted(rows for rows, _ in engine.calls) == [2, 3, 4]
    assert [s.seed for _, s in engine.calls] == [100, 101, 102]  # seed ledger: config.seed + call index
    assert {s.temperature for rows, s in engine.calls if rows != 3} == {1.0}
    first = results[0]
    assert first.prompt == "p0" and first.prompt_token_ids == (ord("p"), ord("0")) and first.finished
    assert first.outputs[0].finish_reason == "stop" and first.outputs[0].stop_reason == "stop"
    assert first.request_id.startswith("req-")


def test_string_stops_trim_text_but_keep_token_ids():
    adapter, engine = _adapter()
    result = asyncio.run(adapter.generate("hello", sampling=SamplingConfig(stop=("x!",), max_tokens=8, logprobs=1)))
    assert result.token_ids == (ord("x"), ord("x"), ord("!")) and result.text == "xx!"[:"xx!".index("x!") + 2]
    native = engine.calls[0][1]
    assert native.stop_table is not None and native.stop_token_sequences == () and native.return_logprobs
    assert result.completion_logprobs == (0.0, 0.0, 0.0)


def test_prompt_rendering_of_text_tokens_and_mappings():
    adapter, _ = _adapter(apply_chat_template=True, chat_template_enable_thinking=False, assistant_prefill="OK")
    text_ids = adapter.tokenize_prompt("hi")
    assert CharTokenizer().decode(text_ids) == "<user>hi<assistant><nothink>OK"
    assert adapter.tokenize_prompt("hi", chat_template_enable_thinking=True, assistant_prefill="") == tuple(
        map(ord, "<user>hi<assistant>"))
    assert adapter.tokenize_prompt([104, 105]) == (104, 105, ord("O"), ord("K"))  # token prompts are not templated
    mapped = adapter.tokenize_prompt({"prompt": "ignored", "prompt_token_ids": [1, 2]}, assistant_prefill="")
    assert mapped == (1, 2)
    config = InferenceEngineConfig(model_path="", assistant_prefill="!")
    assert LFM25AsyncInferenceEngine.tokenize_for_config(config, CharTokenizer(), {"text": "ab"}) == (97, 98, 33)
    with pytest.raises(TypeError):
        asyncio.run(adapter.generate("x", sampling={"temperature": 1.0}))


def test_native_sampling_translation_and_finish_codes():
    native = to_native_sampling(SamplingConfig(temperature=0.7, top_k=-1, top_p=0.9, max_tokens=5, stop=("ab",),
                                               extra_params={"ignore_eos": True, "repetition_penalty": 1.5}),
                                seed=9, tokenizer=CharTokenizer())
    assert (native.temperature, native.top_k, native.top_p, native.max_new_tokens) == (0.7, 0, 0.9, 5)
    assert native.ignore_eos and native.repetition_penalty == 1.5 and native.seed == 9 and not native.return_logprobs
    assert native.stop_token_sequences == ((97, 98), (32, 97, 98), (10, 97, 98), (62, 97, 98))
    with pytest.raises(ValueError):
        to_native_sampling(SamplingConfig(n=2), seed=0)
    with pytest.raises(ValueError):
        to_native_sampling(SamplingConfig(stop=("a",)), seed=0)
    assert [decode_finish_reason(c) for c in (0, 1, 2, 3)] == [(None, None), ("stop", "eos"), ("stop", "stop"), ("length", None)]
    with pytest.raises(ValueError):
        SamplingConfig(top_k=0)
    with pytest.raises(ValueError):
        SamplingConfig(extra_params={"min_p": 0.1})


def test_chain_keys_do_not_depend_on_slots_and_exact_extensions_resume():
    assert chain_seed(5, 0, 0) == 5
    assert chain_seed(5, 3, 2) == (5 + 3 * 0x517CC1B727220A95 + 2 * 0x6C8E9CF570932BD5) & 0x7FFFFFFFFFFFFFFF
    adapter, engine = _adapter(seed=7)
    adapter.max_batch_size = 2
    sampling = SamplingConfig(temperature=1.0, max_tokens=2)
    requests = [([10 + i], sampling) for i in range(3)]
    seen = []

    def on_result(index, result):
        seen.append((index, result.request_id, result.token_ids))
        phase = int(result.request_id.rsplit("-", 1)[1])
        if index == 0 and phase == 0:   # exact extension of prompt + completion: resumes in place
            return (list(result.prompt_token_ids + result.token_ids) + [99], sampling)
        if index == 1 and phase == 0:   # a different prompt: the slot starts fresh
            return ([77, 78], sampling)
        return None
    results = asyncio.run(adapter.generate_chains(requests, on_result=on_result, max_new_tokens=4, poll_interval=8))
    assert [len(r) for r in results] == [2, 2, 1]
    log = engine.log
    assert log[0] == ("session", 2, 4)
    base = 7
    assert log[1] == ("admit", (0, 1), (chain_seed(base, 0, 0), chain_seed(base, 1, 0)))
    resumes = [e for e in log if e[0] == "resume"]
    assert resumes == [("resume", (0,), (chain_seed(base, 0, 1),))]
    later_admits = [e for e in log if e[0] == "admit"][1:]
    assert later_admits[0] == ("admit", (1,), (chain_seed(base, 1, 1),))           # chain 1 restarted in its own slot
    assert later_admits[-1][2] == (chain_seed(base, 2, 0),)                         # the queued chain got a freed slot
    assert [r.request_id for r in results[0]] == ["chain-0-phase-0", "chain-0-phase-1"]
    assert results[0][0].outputs[0].finish_reason == "length" and adapter.last_session_stats["polls"] >= 2
    assert log[-1] == ("close",)


def test_abort_close_and_weight_sync_go_through_the_engine_lock():
    adapter, engine = _adapter()

    async def scenario():
        adapter.batch_wait_seconds = 0.05
        kept = asyncio.ensure_future(adapter.generate("keep", request_id="keep"))
        dropped = asyncio.ensure_future(adapter.generate("drop", request_id="drop"))
        await asyncio.sleep(0)
        await adapter.abort_async("drop")
        result = await kept
        with pytest.raises(asyncio.CancelledError):
            await dropped
        return result
    assert asyncio.run(scenario()).request_id == "keep"
    assert adapter.sync_from_model("policy") is engine and ("sync", "policy") in engine.log
    with pytest.raises(ValueError):
        adapter.sync_from_model("policy", drain_timeout=float("inf"))
    adapter.sleep()
    assert ("release_buffers",) in engine.log
    adapter.close()
    with pytest.raises(RuntimeError):
        asyncio.run(adapter.generate("late"))
    with pytest.raises(RuntimeError):
        adapter.raw_engine
