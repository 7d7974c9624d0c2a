"""Document-length plumbing for models that take ``doc_lens`` / ``max_doc_lens`` instead of an
attention mask (the olmo-core transformer interface).

Same names, arguments and results as ``doc_lens_from_attention_mask`` and
``doc_lens_from_cu_seq_lens`` in open_instruct/olmo_core_utils.py:628-665.  Integer work only:
results are bit-exact.  Both run as a handful of whole-tensor operations on the device the input
lives on (no per-row Python loop); like the reference they read one number back to the host (the
output's width), because the result's shape depends on the data.
"""

from __future__ import annotations

import torch


def doc_lens_from_attention_mask(attention_mask_BS: torch.Tensor) -> tuple[torch.Tensor, list[int]]:
    """Run lengths of every row of an integer-coded packed attention mask.

    ``attention_mask_BS`` is ``[batch, seq]``; a token's value is the 1-based id of its document
    within the row, 0 marks padding, equal values are contiguous.  Every maximal run of equal values
    is one segment, padding runs included (the consumer lays all rows' segments end to end, so a
    dropped padding run would shift the boundaries of the rows behind it).  Returns ``doc_lens``
    ``[batch, max_segments]`` int32, rows with fewer segments padded with zeros, and the longest
    segment of every row as a list.  open_instruct/olmo_core_utils.py:628-647.
    """
    if attention_mask_BS.ndim != 2:
        raise ValueError(f"expected a [batch, seq] mask, got shape {tuple(attention_mask_BS.shape)}")
    batch, seq = attention_mask_BS.shape
    if seq == 0:
        return torch.zeros((batch, 0), dtype=torch.int32, device=attention_mask_BS.device), [0] * batch
    # a token opens a new segment when its value differs from its left neighbour's
    opens = attention_mask_BS[:, 1:] != attention_mask_BS[:, :-1]
    segment = torch.zeros((batch, seq), dtype=torch.int64, device=attention_mask_BS.device)
    segment[:, 1:] = opens.cumsum(dim=1)
    width = int(segment[:, -1].max().item()) + 1
    doc_lens = torch.zeros((batch, width), dtype=torch.int32, device=attention_mask_BS.device)
    doc_lens.scatter_add_(1, segment, torch.ones_like(segment, dtype=torch.int32))
    return doc_lens, doc_lens.max(dim=1).values.tolist()


def doc_lens_from_cu_seq_lens(cu_seq_lens_k_D1: torch.Tensor, seq_len: int) -> tuple[torch.Tensor, list[int]]:
    """Document lengths of one packed row from flash-attention style cumulative offsets.

    ``cu_seq_lens_k_D1`` is ``[num_docs + 1]`` with a leading 0; ``seq_len`` the (possibly padded)
    length of the row.  A trailing pad span becomes a segment of its own so that the lengths add up
    to ``seq_len``.  Returns ``doc_lens`` ``[1, segments]`` int32 and ``[longest segment]``.
    open_instruct/olmo_core_utils.py:650-665.
    """
    if cu_seq_lens_k_D1.ndim != 1 or cu_seq_lens_k_D1.numel() < 1:
        raise ValueError("cu_seq_lens must be a 1-D tensor with a leading 0")
    offsets = cu_seq_lens_k_D1.to(torch.int64)
    covered = int(offsets[-1].item())
    if covered < seq_len:
        offsets = torch.cat([offsets, offsets.new_tensor([seq_len])])
    lens = (offsets[1:] - offsets[:-1]).to(torch.int32)
    longest = int(lens.max().item()) if lens.numel() else 0
    return lens.unsqueeze(0), [longest]
