"""The `benchmark` command: argument rules, report schema and the reader's checks (reference
`inference/benchmark.py:23-157`, `preflight.py:60-79`).  The CPU tests drive the command with a scripted engine;
the GPU test runs it end to end on the small synthetic shape."""
import json

import pytest
import torch

from climbing_gym_amd import benchmark
from climbing_gym_amd.engine import LFM25GenerationOutput


class ScriptedEngine:
    """Returns the full budget for every row: token = row index, log-probability -1."""

    def __init__(self, short=False):
        self.calls, self.released, self.graphs, self.short = 0, 0, None, short

    def enable_cuda_graphs(self, **kw):
        self.graphs = kw

    def generate(self, input_ids, cu_seqlens, max_seqlen, repeats, sampling):
        self.calls += 1
        rows, budget = cu_seqlens.numel() - 1, sampling.max_new_tokens
        tokens = torch.arange(rows).view(rows, 1, 1).expand(rows, 1, budget).clone()
        lengths = torch.full((rows, 1), budget - (1 if self.short else 0), dtype=torch.int32)
        return LFM25GenerationOutput(tokens, lengths, torch.full((rows, 1, budget), -1.0), torch.full((rows, 1), 3, dtype=torch.int8))

    def release_inference_buffers(self):
        self.released += 1


def run(tmp_path, extra=(), engine=None):
    engine = engine or ScriptedEngine()
    out = tmp_path / "report.json"
    argv = ["--synthetic-shape", "tiny", "--device", "cpu", "--batches", "2", "5", "--prompt-tokens", "9",
            "--output-tokens", "6", "--repeats", "3", "--output", str(out), *extra]
    report = benchmark.main(argv, engine_factory=lambda args, context: (engine, benchmark.EchoTokenizer(4096)))
    return report, json.loads(out.read_text()), out.with_suffix(".md").read_text(), engine


def test_report_has_the_reference_schema_and_passes_the_readers_checks(tmp_path):
    report, on_disk, traces, engine = run(tmp_path)
    assert on_disk == json.loads(json.dumps(report))
    assert set(report) == {"engine", "created_at", "hardware", "workload", "config", "sampling", "max_model_len",
                           "scheduler", "batches"}
    assert report["engine"] == "native_lfm25" and report["scheduler"] == benchmark.SCHEDULER_NOTE
    assert report["workload"] == {"kind": "synthetic", "prompts_sha256": None, "prompt_lengths": [9]}
    assert report["max_model_len"] == 9 + 6
    assert report["sampling"]["return_logprobs"] is True and report["sampling"]["ignore_eos"] is True
    assert report["sampling"]["top_k"] == 0 and report["sampling"]["max_new_tokens"] == 6   # --top-k -1 -> 0
    assert report["config"]["output"].endswith("report.json") and report["config"]["output_tokens"] == 6
    assert [b["batch_size"] for b in report["batches"]] == [2, 5]
    for entry in report["batches"]:
        assert set(entry) == {"batch_size", "max_num_seqs", "max_inflight_requests", "runs", "median_tokens_per_second",
                              "peak_allocated_bytes", "peak_reserved_bytes"}
        assert len(entry["runs"]) == 3 and entry["peak_allocated_bytes"] is None
        assert all(run_["output_tokens"] == entry["batch_size"] * 6 for run_ in entry["runs"])
        assert benchmark.check_report(report, entry["batch_size"]) is entry
    assert engine.calls == 2 * (1 + 3) and engine.released == 2            # one warm-up + three timed per batch
    assert traces.startswith("# Native throughput traces") and "## Batch 5, row 2" in traces and "## Batch 5, row 3" not in traces
    assert "Outcome: 6 tokens; sampled log probabilities finite." in traces
    with pytest.raises(ValueError, match="resolved batch size 7"):
        benchmark.check_report(report, 7)


def test_representative_prompts_are_hashed_and_cycled(tmp_path):
    prompts = tmp_path / "prompts.json"
    prompts.write_text(json.dumps({"prompts": [[1, 2, 3], [4, 5, 6, 7, 8]]}))
    report, _, traces, _ = run(tmp_path, ["--prompts-json", str(prompts)])
    assert report["workload"]["kind"] == "representative" and report["workload"]["prompt_lengths"] == [3, 5]
    assert len(report["workload"]["prompts_sha256"]) == 64
    assert report["max_model_len"] == 9 + 6          # the longer of --prompt-tokens and the saved prompts, plus the budget
    assert "representative task prompts" in traces and "```text\n4 5 6 7 8\n```" in traces


def test_an_incomplete_budget_is_an_error_and_so_are_bad_arguments(tmp_path):
    with pytest.raises(RuntimeError, match="incomplete budget"):
        run(tmp_path, engine=ScriptedEngine(short=True))
    for extra in (["--top-k", "0"], ["--fp8-kv"], ["--cuda-graphs"], ["--repeats", "0"], ["--park-gib", "1"]):
        with pytest.raises(SystemExit):
            run(tmp_path, extra)
    bad = tmp_path / "bad.json"
    bad.write_text(json.dumps({"prompts": [[1, -2]]}))
    with pytest.raises(SystemExit):
        run(tmp_path, ["--prompts-json", str(bad)])
    with pytest.raises(SystemExit):      # prompt + budget beyond the context
        run(tmp_path, ["--max-model-len", "12"])


def test_reader_checks_reject_broken_reports():
    good = {"config": {"device": "cuda", "output_tokens": 4},
            "batches": [{"batch_size": 2, "median_tokens_per_second": 10.0, "peak_allocated_bytes": 5, "peak_reserved_bytes": 6,
                         "runs": [{"seconds": 1.0, "tokens_per_second": 8.0, "output_tokens": 8}]}]}
    assert benchmark.check_report(good, 2)["batch_size"] == 2
    for path, value, message in ((("batches", 0, "median_tokens_per_second"), 0, "tokens_per_second"),
                                 (("batches", 0, "peak_allocated_bytes"), None, "peak_allocated_bytes"),
                                 (("batches", 0, "runs"), [], "no measured rollouts"),
                                 (("batches", 0, "runs", 0, "output_tokens"), 7, "intended token budget")):
        broken = json.loads(json.dumps(good))
        node = broken
        for key in path[:-1]:
            node = node[key]
        node[path[-1]] = value
        with pytest.raises(ValueError, match=message):
            benchmark.check_report(broken, 2)


@pytest.mark.gpu
def test_command_runs_end_to_end_on_the_small_synthetic_shape(tmp_path):
    out = tmp_path / "gpu.json"
    report = benchmark.main(["--synthetic-shape", "tiny", "--batches", "3", "--prompt-tokens", "24", "--output-tokens", "16",
                             "--cuda-graphs", "--fp8-mlp", "--fp8-kv", "--fp8-lm-head", "--behavior-topk", "4",
                             "--output", str(out)])
    entry = benchmark.check_report(report, 3)
    assert entry["peak_allocated_bytes"] > 0 and len(entry["runs"]) == 2
    assert report["hardware"]["device"].startswith("cuda") and report["workload"]["kind"] == "synthetic"
    assert out.exists() and out.with_suffix(".md").read_text().count("## Batch 3, row") == 3
