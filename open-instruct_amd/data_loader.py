"""Collation of packed rows into per-rank micro-batches; same names as
open_instruct/data_loader.py (``collate_fn`` :636-641, ``prepare_collated_data_for_workers``
:1205-1289).  Index and padding plumbing on tensors that already live on the GPU after
``rl_utils.pack_sequences``: no host copies, no pinned staging buffers."""

from __future__ import annotations

import logging

import numpy as np
import torch

from .data_types import CollatedBatchData

logger = logging.getLogger(__name__)


def collate_fn(tensors_list: list[torch.Tensor], pad_token_id: int | float) -> torch.Tensor:
    """Right-pad to the longest row and stack, ``[B, T_max]``; open_instruct/data_loader.py:636-641
    (the reference also pins the result for the host-to-device copy, which does not exist here)."""
    padded = torch.nn.utils.rnn.pad_sequence(tensors_list, batch_first=True, padding_value=pad_token_id)
    return torch.atleast_2d(padded)


def prepare_collated_data_for_workers(
    packed_sequences, dp_world_size: int, per_device_train_batch_size: int, pad_token_id: int
) -> list[CollatedBatchData]:
    """Split the packed rows over ``dp_world_size`` ranks, shuffle each rank's rows and collate
    them into micro-batches of ``per_device_train_batch_size`` rows; open_instruct/data_loader.py:1205-1289.

    Rows that do not divide evenly over the ranks are dropped from the end (with a warning); the
    shuffle draws from ``numpy.random`` exactly as the reference does, so a seeded run orders its
    micro-batches the same way.  Padding: ``pad_token_id`` for token ids, 0 for everything else.
    """
    total = len(packed_sequences.query_responses)
    if total % dp_world_size != 0:
        kept = (total // dp_world_size) * dp_world_size
        logger.warning(
            f"Total packed sequences ({total}) is not evenly divisible by dp_world_size ({dp_world_size}). "
            f"Truncating to {kept} sequences (dropping {total - kept})."
        )
    per_rank = total // dp_world_size
    assert packed_sequences.position_ids is not None
    assert packed_sequences.advantages is not None
    assert packed_sequences.vllm_logprobs is not None
    fields = (
        ("query_responses", packed_sequences.query_responses, pad_token_id),
        ("attention_masks", packed_sequences.attention_masks, 0),
        ("position_ids", packed_sequences.position_ids, 0),
        ("advantages", packed_sequences.advantages, 0),
        ("response_masks", packed_sequences.response_masks, 0),
        ("vllm_logprobs", packed_sequences.vllm_logprobs, 0),
    )
    out = []
    for rank in range(dp_world_size):
        lo = per_rank * rank
        order = np.random.permutation(per_rank)
        collated = {name: [] for name, _, _ in fields}
        for j in range(0, per_rank, per_device_train_batch_size):
            micro = order[j : j + per_device_train_batch_size]
            for name, rows, pad in fields:
                collated[name].append(collate_fn([rows[lo + int(idx)] for idx in micro], pad))
        out.append(CollatedBatchData(**collated))
    return out
