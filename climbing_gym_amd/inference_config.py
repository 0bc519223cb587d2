"""Request-level configuration of the async adapter (inference/config.py of the reference: same fields, same
validation messages, so rollout code written against the reference constructs these unchanged)."""
from __future__ import annotations

import math
from collections.abc import Mapping, Sequence
from dataclasses import dataclass, field
from numbers import Real
from pathlib import Path
from typing import Any
from ._checks import reject

DEFAULT_STAGED_CHECKPOINT_ROOT = Path.home() / ".cache" / "climbing-gym" / "checkpoints"
_EXTRA_KEYS = {"repetition_penalty", "ignore_eos", "behavior_topk"}


def _is_number(value: Any) -> bool:
    return isinstance(value, Real) and not isinstance(value, bool) and math.isfinite(value)


@dataclass(frozen=True)
class SamplingConfig:
    """inference/config.py:17-62."""
    temperature: float = 0.0
    top_k: int = -1
    top_p: float = 1.0
    max_tokens: int = 256
    n: int = 1
    stop: tuple = ()
    logprobs: int | None = None
    extra_params: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        checks = (
            (_is_number(self.temperature) and self.temperature >= 0, "temperature must be finite and >= 0"),
            (type(self.top_k) is int and (self.top_k == -1 or self.top_k >= 1), "top_k must be -1 or >= 1"),
            (_is_number(self.top_p) and 0.0 < self.top_p <= 1.0, "top_p must be finite and in (0, 1]"),
            (type(self.max_tokens) is int and self.max_tokens > 0, "max_tokens must be a positive integer"),
            (type(self.n) is int and self.n > 0, "n must be a positive integer"),
            (self.logprobs is None or (type(self.logprobs) is int and self.logprobs > 0),
             "logprobs must be a positive integer when provided"),
            (isinstance(self.stop, Sequence) and not isinstance(self.stop, (str, bytes))
             and all(isinstance(s, str) and s for s in self.stop), "stop must be a sequence of nonempty strings"),
            (isinstance(self.extra_params, Mapping), "extra_params must be a mapping"),
        )
        for ok, message in checks:
            reject(not ok, message)
        object.__setattr__(self, "stop", tuple(self.stop))
        unknown = sorted(str(k) for k in set(self.extra_params) - _EXTRA_KEYS)
        reject(unknown, f"Unsupported native sampling extra_params: {unknown}")
        penalty = self.extra_params.get("repetition_penalty", 1.0)
        reject(not _is_number(penalty) or penalty <= 0, "repetition_penalty must be finite and > 0")
        reject(type(self.extra_params.get("ignore_eos", False)) is not bool, "ignore_eos must be a boolean")
        head = self.extra_params.get("behavior_topk", 0)
        reject(type(head) is not int or not 0 <= head <= 128, "behavior_topk must be an integer between 0 and 128")

    def batching_key(self) -> tuple:
        """Requests with equal keys may share one engine.generate call (lfm25_async_engine.py:675-685)."""
        return (float(self.temperature), int(self.top_k), float(self.top_p), int(self.max_tokens), int(self.n),
                tuple(self.stop), self.logprobs, tuple(sorted(dict(self.extra_params).items())))


@dataclass(frozen=True)
class InferenceEngineConfig:
    """inference/config.py:66-87."""
    model_path: str
    dtype: str = "auto"
    seed: int = 0
    gpu_memory_utilization: float = 0.9
    max_model_len: int | None = None
    max_num_seqs: int | None = None
    enforce_eager: bool = False
    enable_sleep_mode: bool = True
    apply_chat_template: bool = False
    chat_template_enable_thinking: bool = True
    assistant_prefill: str = ""
    default_sampling: SamplingConfig = field(default_factory=SamplingConfig)
    staged_checkpoint_root: Path = field(default_factory=lambda: DEFAULT_STAGED_CHECKPOINT_ROOT)

    def __post_init__(self) -> None:
        reject(not 0.0 < self.gpu_memory_utilization <= 1.0, "gpu_memory_utilization must be between 0 and 1")
        reject(self.max_model_len is not None and self.max_model_len <= 0, "max_model_len must be > 0 when provided")
        reject(self.max_num_seqs is not None and self.max_num_seqs <= 0, "max_num_seqs must be > 0 when provided")
