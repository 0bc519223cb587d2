"""Fixed-budget prefill + decode throughput report of the native engine (`python -m climbing_gym_amd.benchmark`).

Same switches and the same report as the reference's `inference/benchmark.py:23-157`: a JSON file that
`preflight.validate_preflight` (`preflight.py:60-135`) reads before a training run, and a Markdown file beside it with
the first rows' prompts and complete responses.  Every timed rollout includes the device-to-host copies of tokens,
log-probabilities and lengths and excludes loading and warm-up.

One switch has no counterpart there: `--synthetic-shape` runs a seeded random-init model of a named shape with an
id-echo tokenizer, for machines that hold no checkpoint (the report then says `workload.kind = "synthetic"`, which the
preflight check rejects on purpose, like the reference's own synthetic prompts).
"""
from __future__ import annotations

import argparse
import hashlib
import json
import statistics
import time
from dataclasses import asdict
from datetime import datetime, timezone
from pathlib import Path

import torch

from .config import LFM2Config, LFM25SamplingConfig
from .engine import LFM25Engine, flatten_token_batches
from ._checks import reject

SCHEDULER_NOTE = "synchronous fixed batches; no hidden request concurrency cap"
SHAPES = ("tiny", "lfm2-1.2b")


class EchoTokenizer:
    """Stand-in for runs without a checkpoint: token ids are their own text."""

    def __init__(self, vocab: int):
        self.vocab = int(vocab)

    def encode(self, text, add_special_tokens=False):
        return [ord(ch) % self.vocab for ch in str(text)]

    def decode(self, ids, skip_special_tokens=False):
        return " ".join(str(int(t)) for t in ids)


def build_arg_parser() -> argparse.ArgumentParser:
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    source = p.add_mutually_exclusive_group(required=True)
    source.add_argument("--model", help="Local checkpoint directory")
    source.add_argument("--synthetic-shape", choices=SHAPES, help="Seeded random-init model instead of a checkpoint")
    p.add_argument("--batches", type=int, nargs="+", default=[1, 32, 128])
    p.add_argument("--prompt-tokens", type=int, default=128)
    p.add_argument("--prompts-json", type=Path, help="JSON containing a prompts list of token-ID rows")
    p.add_argument("--output-tokens", type=int, default=4096)
    p.add_argument("--max-model-len", type=int)
    p.add_argument("--device", default="cuda" if torch.cuda.is_available() else "cpu")
    p.add_argument("--dtype", default="auto", choices=["auto", "bfloat16", "float16", "float32"])
    p.add_argument("--temperature", type=float, default=1.0)
    p.add_argument("--top-k", type=int, default=-1, help="-1 disables top-k, matching rollout sampling")
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--repetition-penalty", type=float, default=1.0)
    p.add_argument("--behavior-topk", type=int, default=0)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--warmups", type=int, default=1)
    p.add_argument("--repeats", type=int, default=2)
    p.add_argument("--cuda-graphs", action="store_true")
    p.add_argument("--compile-decode", action="store_true")
    p.add_argument("--fp8-mlp", action="store_true")
    p.add_argument("--fp8-kv", action="store_true")
    p.add_argument("--fp8-lm-head", action="store_true")
    p.add_argument("--adaptive-batching", action="store_true")
    p.add_argument("--bf16-weight-packing", action="store_true")
    p.add_argument("--max-prefill-tokens", type=int, default=4096)
    p.add_argument("--park-gib", type=float, default=0, help="Reserve optimizer-equivalent GPU memory")
    p.add_argument("--output", type=Path, required=True)
    return p


def synthetic_prompts(tokenizer, batch: int, length: int):
    """The reference's filler sentence repeated to `length` tokens, one document number per row
    (`inference/benchmark.py:53-59`)."""
    rows = []
    for index in range(batch):
        ids = list(tokenizer.encode(f"Document {index}: Check each arithmetic operation carefully before continuing. ",
                                    add_special_tokens=False))
        rows.append((ids * (length // len(ids) + 1))[:length])
    return rows


def _load_tokenizer(model_dir):
    from transformers import AutoTokenizer
    return AutoTokenizer.from_pretrained(str(model_dir), local_files_only=True)


def _synthetic_engine(shape: str, *, device, dtype, max_model_len):
    from . import synthetic
    spec = synthetic.TINY if shape == "tiny" else synthetic.LFM2_1P2B
    config = LFM2Config(vocab_size=spec["vocab"], hidden_size=spec["hidden"], mlp_hidden_size=spec["mlp_hidden"],
                        num_hidden_layers=len(spec["layer_types"]), num_attention_heads=spec["q_heads"],
                        num_key_value_heads=spec["kv_heads"], layer_types=tuple(spec["layer_types"]),
                        max_position_embeddings=max(int(max_model_len), 128000))
    state = synthetic.random_state_dict(**spec, seed=0, dtype=torch.bfloat16)
    torch_dtype = torch.bfloat16 if dtype == "auto" else getattr(torch, dtype)
    return LFM25Engine.from_state_dict(config, state, device=device, dtype=torch_dtype, max_model_len=max_model_len), \
        EchoTokenizer(spec["vocab"])


def validate(parser, args, saved):
    """Argument rules of `inference/benchmark.py:64-82`, same messages."""
    positive = [*args.batches, args.prompt_tokens, args.output_tokens, args.warmups, args.repeats, args.max_prefill_tokens]
    if min(positive) <= 0 or args.park_gib < 0:
        parser.error("batch sizes, token counts and repetitions must be positive; parked memory must be nonnegative")
    if any((args.fp8_mlp, args.fp8_kv, args.fp8_lm_head, args.adaptive_batching)) and not args.cuda_graphs:
        parser.error("FP8 and adaptive batching require --cuda-graphs")
    if (args.cuda_graphs or args.park_gib) and torch.device(args.device).type != "cuda":
        parser.error("CUDA graphs and parked GPU memory require --device cuda")
    if saved is not None and (not saved or any(
            not row or any(type(token) is not int or token < 0 for token in row) for row in saved)):
        parser.error("--prompts-json must contain nonempty rows of nonnegative integer token IDs")
    if args.top_k == 0 or args.top_k < -1:
        parser.error("--top-k must be -1 or positive")


def new_report(args, sampling, context, device, saved):
    """Head of the report: the keys and value types of `inference/benchmark.py:93-103`."""
    return {
        "engine": "native_lfm25",
        "created_at": datetime.now(timezone.utc).isoformat(),
        "hardware": {"device": str(device),
                     "name": torch.cuda.get_device_name(device) if device.type == "cuda" else "cpu",
                     "torch_version": torch.__version__},
        "workload": {"kind": "representative" if saved else "synthetic",
                     "prompts_sha256": hashlib.sha256(args.prompts_json.read_bytes()).hexdigest() if saved else None,
                     "prompt_lengths": [len(row) for row in saved] if saved else [args.prompt_tokens]},
        "config": {key: str(value) if isinstance(value, Path) else value for key, value in vars(args).items()},
        "sampling": asdict(sampling),
        "max_model_len": context,
        "scheduler": SCHEDULER_NOTE,
        "batches": [],
    }


def measure_batch(engine, rows, sampling, *, batch, output_tokens, warmups, repeats, device):
    """Warm up, then time `repeats` full rollouts of one batch; returns (report entry, last tokens, last lengths)."""
    cuda = device.type == "cuda"
    sync = (lambda: torch.cuda.synchronize(device)) if cuda else (lambda: None)
    flat = flatten_token_batches(rows, device=device)
    for _ in range(warmups):
        engine.generate(*flat, repeats=1, sampling=sampling)
    sync()
    if cuda:
        torch.cuda.reset_peak_memory_stats(device)
    runs, tokens, lengths = [], None, None
    for _ in range(repeats):
        sync()
        started = time.perf_counter()
        output = engine.generate(*flat, repeats=1, sampling=sampling)
        tokens, logprobs, lengths = output.token_ids.cpu(), output.logprobs.cpu(), output.lengths.cpu()
        if output.topk_token_ids is not None:
            output.topk_token_ids.cpu()
            reject(not bool(torch.isfinite(output.topk_logprobs.cpu()).all()),
                   "Native rollout returned non-finite sparse behavior logprobs", RuntimeError)
        sync()
        seconds = time.perf_counter() - started
        count = int(lengths.sum())
        reject(count != batch * output_tokens or not bool(torch.isfinite(logprobs).all()),
               "Native rollout returned an incomplete budget or non-finite logprobs", RuntimeError)
        runs.append({"seconds": seconds, "output_tokens": count, "tokens_per_second": count / seconds})
    entry = {"batch_size": batch, "max_num_seqs": batch, "max_inflight_requests": batch, "runs": runs,
             "median_tokens_per_second": statistics.median(run["tokens_per_second"] for run in runs),
             "peak_allocated_bytes": torch.cuda.max_memory_allocated(device) if cuda else None,
             "peak_reserved_bytes": torch.cuda.max_memory_reserved(device) if cuda else None}
    return entry, tokens, lengths


def trace_rows(tokenizer, rows, tokens, lengths, batch, representative):
    """Markdown of the first three rows of a batch (`inference/benchmark.py:142-150`)."""
    lines = []
    for row in range(min(3, batch)):
        completion = tokens[row, 0, :int(lengths[row, 0])].tolist()
        lines += [f"## Batch {batch}, row {row}", "", "Prompt:", "",
                  "```text", tokenizer.decode(rows[row], skip_special_tokens=False), "```", "",
                  "Complete model response:", "", "```text", tokenizer.decode(completion, skip_special_tokens=False), "```", "",
                  ("Expected answer: not scored (representative throughput workload)." if representative else
                   "Expected answer: not applicable (synthetic throughput workload)."),
                  f"Outcome: {len(completion)} tokens; sampled log probabilities finite.", ""]
    return lines


def check_report(report, batch_size: int) -> dict:
    """What the report's reader requires of the entry for `batch_size` (`preflight.py:60-79`): positive median rate,
    positive peak memory on a GPU, at least one run, every run complete.  Returns the entry."""
    def positive(value, name):
        reject(not isinstance(value, (int, float)) or not value > 0, f"Native preflight report has no positive {name}")
    for entry in report.get("batches", []):
        if int(entry.get("batch_size", 0)) != batch_size:
            continue
        positive(entry.get("median_tokens_per_second", 0), "tokens_per_second")
        if str(report["config"].get("device", "cuda")).startswith("cuda"):
            positive(entry.get("peak_allocated_bytes", 0), "peak_allocated_bytes")
            positive(entry.get("peak_reserved_bytes", 0), "peak_reserved_bytes")
        reject(not entry.get("runs"), "Native preflight report contains no measured rollouts")
        for run in entry["runs"]:
            positive(run.get("seconds", 0), "rollout seconds")
            positive(run.get("tokens_per_second", 0), "rollout tokens_per_second")
            reject(int(run.get("output_tokens", 0)) != batch_size * int(report["config"]["output_tokens"]),
                   "Native preflight report did not complete the intended token budget")
        return entry
    raise ValueError(f"Native preflight report must benchmark resolved batch size {batch_size}")


def main(argv=None, *, engine_factory=None) -> dict:
    """Runs the benchmark and writes `<output>` (JSON) and `<output stem>.md`.  `engine_factory(args, context)` ->
    (engine, tokenizer) replaces checkpoint loading (tests)."""
    parser = build_arg_parser()
    args = parser.parse_args(argv)
    saved = json.loads(args.prompts_json.read_text())["prompts"] if args.prompts_json else None
    validate(parser, args, saved)
    device = torch.device(args.device)
    context = args.max_model_len or max(args.prompt_tokens, max(map(len, saved)) if saved else 0) + args.output_tokens
    if engine_factory is not None:
        engine, tokenizer = engine_factory(args, context)
    elif args.synthetic_shape:
        engine, tokenizer = _synthetic_engine(args.synthetic_shape, device=device, dtype=args.dtype, max_model_len=context)
    else:
        tokenizer = _load_tokenizer(args.model)
        engine = LFM25Engine.from_pretrained(args.model, device=device, dtype=args.dtype, max_model_len=context)
    parked = torch.empty(int(args.park_gib * 1024 ** 3), device=device, dtype=torch.uint8) if args.park_gib else None
    if args.cuda_graphs:
        engine.enable_cuda_graphs(max_graphs=1, max_prefill_tokens=args.max_prefill_tokens,
                                  bf16_weight_packing=args.bf16_weight_packing, fp8_mlp=args.fp8_mlp, fp8_kv=args.fp8_kv,
                                  fp8_lm_head=args.fp8_lm_head, adaptive_batching=args.adaptive_batching)
    elif args.compile_decode:
        engine.compile_decode()
    sampling = LFM25SamplingConfig(max_new_tokens=args.output_tokens, temperature=args.temperature, seed=args.seed,
                                   ignore_eos=True, return_logprobs=True, top_k=0 if args.top_k == -1 else args.top_k,
                                   top_p=args.top_p, repetition_penalty=args.repetition_penalty,
                                   behavior_topk=args.behavior_topk)
    report = new_report(args, sampling, context, device, saved)
    traces = ["# Native throughput traces", "",
              ("Fixed-budget representative task prompts; environment answers are not scored." if saved else
               "Fixed-budget synthetic prompts; expected answer: not applicable (throughput validation)."), ""]
    for batch in args.batches:
        rows = [saved[i % len(saved)] for i in range(batch)] if saved else synthetic_prompts(tokenizer, batch, args.prompt_tokens)
        if any(len(row) + args.output_tokens > context for row in rows):
            parser.error("prompt plus output token budget exceeds --max-model-len")
        entry, tokens, lengths = measure_batch(engine, rows, sampling, batch=batch, output_tokens=args.output_tokens,
                                               warmups=args.warmups, repeats=args.repeats, device=device)
        report["batches"].append(entry)
        traces += trace_rows(tokenizer, rows, tokens, lengths, batch, bool(saved))
        print(json.dumps(entry), flush=True)
        engine.release_inference_buffers()
    args.output.parent.mkdir(parents=True, exist_ok=True)
    args.output.write_text(json.dumps(report, indent=2) + "\n")
    args.output.with_suffix(".md").write_text("\n".join(traces) + "\n")
    del parked
    return report


if __name__ == "__main__":
    main()
