"""Oracle: masked means and per-sequence log-probability sums (test infrastructure only)."""

from __future__ import annotations

import torch


def masked_mean(
    values: torch.Tensor, mask: torch.Tensor, axis: int | None = None, denominator: float | None = None
) -> torch.Tensor:
    """Masked mean with the reference's axis / extra-leading-dim / empty-mask rules.

    Restates open_instruct/rl_utils.py:426-448:
    * ``values`` may carry extra leading dims over ``mask`` (e.g. ``[4, B, T]`` vs ``[B, T]``);
      they are kept.
    * ``axis=None``: sum over all mask dims, divide by ``mask.sum()`` (or ``denominator``).
    * ``axis=k``: per-slice means along mask axis ``k``; the remaining mask dims are then
      averaged with a plain mean.
    * A non-positive denominator gives 0, not NaN.
    """
    extra = values.ndim - mask.ndim
    if axis is None:
        dims: tuple[int, ...] | int = tuple(range(extra, values.ndim))
    else:
        dims = axis + extra if axis >= 0 else axis
    top = (values * mask).sum(dim=dims)
    if denominator is None:
        bottom: torch.Tensor | float = mask.sum(dim=axis) if axis is not None else mask.sum()
    else:
        bottom = denominator
    if torch.is_tensor(bottom):
        out = torch.where(bottom > 0, top / bottom, torch.zeros_like(top))
    elif bottom > 0:
        out = top / bottom
    else:
        out = torch.zeros_like(top)
    if out.ndim > extra:
        out = out.flatten(extra).mean(-1)
    return out


def get_batch_logps_padded(
    per_token_logps: torch.Tensor, labels: torch.Tensor, average_log_prob: bool = False
) -> torch.Tensor:
    """Per-row sum (or mean) of per-token logps over positions whose *next* label is kept.

    Restates open_instruct/dpo_utils.py:689-712: drops the last position, mask is
    ``labels[:, 1:] != -100``, the mean divides by ``max(count, 1)``.
    """
    keep = (labels[:, 1:] != -100).to(per_token_logps.dtype)
    total = (per_token_logps[:, :-1] * keep).sum(-1)
    if average_log_prob:
        return total / keep.sum(-1).clamp(min=1)
    return total


def packed_segment_ids(cu_seq_lens: torch.Tensor, num_positions: int) -> torch.Tensor:
    """Segment id of each of the first ``num_positions`` positions of a packed row after the shift.

    Restates open_instruct/padding_free_collator.py:208-218: every boundary but the leading 0
    moves left by one (the last position of each sequence scores the first token of the next and
    is attributed to the *next* segment, where its label is normally masked), ids are clamped to
    the last segment.
    """
    bounds = cu_seq_lens.to(torch.int64)[1:] - 1
    num_seqs = bounds.numel()
    t = torch.arange(num_positions, dtype=torch.int64)
    # number of (shifted) end boundaries at or before t == index of the segment t falls in
    ids = (t.unsqueeze(1) >= bounds.unsqueeze(0)).sum(dim=1)
    return ids.clamp(max=num_seqs - 1)


def get_batch_logps_packed(
    per_token_logps: torch.Tensor, labels: torch.Tensor, cu_seq_lens: torch.Tensor, average_log_prob: bool = False
) -> torch.Tensor:
    """Per-sequence sum (or mean) over a packed ``[1, T]`` row.

    Restates open_instruct/padding_free_collator.py:202-229 with an ``index_add_`` in place of the
    reference's ``scatter_add_`` (same sums, deterministic order on CPU).
    """
    logps = per_token_logps[0, :-1]
    keep = (labels[0, 1:] != -100).to(logps.dtype)
    num_seqs = cu_seq_lens.numel() - 1
    ids = packed_segment_ids(cu_seq_lens.cpu(), logps.numel()).to(logps.device)
    sums = torch.zeros(num_seqs, dtype=logps.dtype, device=logps.device).index_add_(0, ids, logps * keep)
    if average_log_prob:
        counts = torch.zeros(num_seqs, dtype=logps.dtype, device=logps.device).index_add_(0, ids, keep)
        return sums / counts.clamp(min=1)
    return sums
