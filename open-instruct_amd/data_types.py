"""Batch container on the input side of the GRPO path (layout contract only)."""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass
class CollatedBatchData:
    """Six parallel lists of ``[B, T]`` tensors, one entry per micro-batch sample.

    Same fields as open_instruct/data_types.py:104-128: ``query_responses`` int64 token ids,
    ``attention_masks`` int64 (document ids for packed rows), ``position_ids`` int64,
    ``advantages`` fp32 per token, ``response_masks`` bool, ``vllm_logprobs`` fp32 ``[B, T]`` or
    ``[B, T-1]`` with NaN on query tokens.
    """

    query_responses: list[torch.Tensor]
    attention_masks: list[torch.Tensor]
    position_ids: list[torch.Tensor]
    advantages: list[torch.Tensor]
    response_masks: list[torch.Tensor]
    vllm_logprobs: list[torch.Tensor]

    def __len__(self) -> int:
        return len(self.query_responses)

    def to(self, device: torch.device) -> "CollatedBatchData":
        move = lambda ts: [t.to(device) for t in ts]  # noqa: E731
        return CollatedBatchData(
            move(self.query_responses), move(self.attention_masks), move(self.position_ids), move(self.advantages),
            move(self.response_masks), move(self.vllm_logprobs),
        )  # fmt: skip
