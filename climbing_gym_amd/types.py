"""Result containers shared by the session and adapter layers (inference/types.py of the reference)."""
from __future__ import annotations

from dataclasses import dataclass

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
