"""Result containers shared by the session and adapter layers (inference/types.py of the reference)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Sequence, Union

import torch


@dataclass(frozen=True)
class BehaviorTopK:
    """Top-k ids and log-probabilities of the unfiltered sampling distribution, one row per generated token."""
    token_ids: torch.Tensor
    logprobs: torch.Tensor

    def __post_init__(self):
        if self.token_ids.ndim != 2 or self.token_ids.shape != self.logprobs.shape:
            raise ValueError('Behavior head IDs/logprobs must be aligned [tokens, k] tensors')
        if self.token_ids.dtype not in (torch.int32, torch.int64) or self.logprobs.dtype != torch.float32:
            raise ValueError('Behavior head requires integer IDs and FP32 logprobs')


# A prompt is chat text, a list of token ids, or a mapping with "prompt"/"text" and optionally "prompt_token_ids".
PromptInput = Union[str, Sequence[int], Mapping[str, Any]]


@dataclass(frozen=True)
class GenerationOutput:
    """One completion of a request (inference/types.py:30-39 of the reference)."""
    index: int
    text: str
    token_ids: tuple
    completion_logprobs: Optional[tuple]
    finish_reason: Optional[str]
    stop_reason: Optional[str]
    behavior_topk: Optional[BehaviorTopK] = None


@dataclass(frozen=True)
class GenerationResult:
    """A finished request (inference/types.py:42-66); the properties read the first completion."""
    request_id: str
    prompt: Any
    prompt_token_ids: tuple
    outputs: tuple
    finished: bool
    raw_output: Any

    def _first(self, name, default):
        return getattr(self.outputs[0], name) if self.outputs else default

    @property
    def text(self) -> str:
        return self._first("text", "")

    @property
    def token_ids(self) -> tuple:
        return self._first("token_ids", ())

    @property
    def completion_logprobs(self):
        return self._first("completion_logprobs", None)
