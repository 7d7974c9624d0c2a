"""Per-token and per-sequence log-probabilities for padded and packed (padding-free) batches.

Names and signatures follow open_instruct/padding_free_collator.py in the reference
(``calculate_per_token_logps`` :10-16, ``concatenated_inputs`` :166-199, ``get_batch_logps`` :202-229).
"""

from __future__ import annotations

import torch

from . import _lib, model_utils


def shift_labels(labels: torch.Tensor) -> torch.Tensor:
    """``out[:, i] = labels[:, i + 1]`` with ``-100`` in the last position (index plumbing, bit-exact)."""
    out = torch.full_like(labels, -100)
    out[:, :-1] = labels[:, 1:]
    return out


def calculate_per_token_logps(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """fp32 log-probability of the next label at every position; open_instruct/padding_free_collator.py:10-16.

    ``out[b, i] = log p(labels[b, i+1] | logits[b, i])``; positions whose next label is ignored
    (``-100``) and the last position score token 0, exactly as the reference's ``clamp(min=0)``.
    The logits are read once in their own dtype and accumulated in fp32; no fp32 copy is made.
    """
    safe = shift_labels(labels).clamp(min=0)
    return model_utils.log_softmax_and_gather(logits, safe)


class _SeqLogps(torch.autograd.Function):
    @staticmethod
    def forward(ctx, per_token_logps, labels, cu_seq_lens, n_seqs, total, average):
        dev = _lib.require_gpu(per_token_logps, labels, cu_seq_lens)
        lp = _lib.f32c(per_token_logps)
        lab = labels.contiguous() if labels.dtype == torch.int64 else labels.long().contiguous()
        cu = None
        if cu_seq_lens is not None:
            cu = cu_seq_lens.to(device=dev, dtype=torch.int32).contiguous()
        out = torch.empty(n_seqs, dtype=torch.float32, device=dev)
        counts = torch.empty(n_seqs, dtype=torch.float32, device=dev)
        _lib.call(
            "oi_seq_logp_fwd", lp.data_ptr(), lab.data_ptr(), _lib.ptr(cu), n_seqs, total, int(average),
            out.data_ptr(), counts.data_ptr(), _lib.stream_of(lp),
        )  # fmt: skip
        ctx.save_for_backward(lab, cu, counts)
        ctx.meta = (n_seqs, total, int(average), per_token_logps.shape, per_token_logps.dtype)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        lab, cu, counts = ctx.saved_tensors
        n_seqs, total, average, shape, dtype = ctx.meta
        g = _lib.f32c(grad_out)
        d = torch.empty(shape, dtype=torch.float32, device=g.device)
        _lib.call(
            "oi_seq_logp_bwd", g.data_ptr(), lab.data_ptr(), _lib.ptr(cu), counts.data_ptr(), n_seqs, total, average,
            d.data_ptr(), _lib.stream_of(g),
        )  # fmt: skip
        return d.to(dtype), None, None, None, None, None


def get_batch_logps(
    per_token_logps: torch.Tensor, labels: torch.Tensor, cu_seq_lens: torch.Tensor, average_log_prob: bool = False
) -> torch.Tensor:
    """Per-sequence sum (or mean) of kept per-token logps over one packed row.

    Drop-in for open_instruct/padding_free_collator.py:202-229 (``per_token_logps``/``labels`` are
    ``[1, T]``, ``cu_seq_lens`` is ``[S + 1]``).  The reference's ``scatter_add_`` sums in an
    unspecified order on a GPU; here every sequence is reduced by one workgroup in a fixed order.
    """
    if per_token_logps.ndim != 2 or per_token_logps.shape[0] != 1:
        raise ValueError("packed per_token_logps must have shape [1, T]")
    total = per_token_logps.shape[1]
    n_seqs = cu_seq_lens.shape[0] - 1
    if n_seqs < 1:
        raise ValueError("cu_seq_lens needs at least two entries")
    return _SeqLogps.apply(per_token_logps, labels, cu_seq_lens, n_seqs, total, average_log_prob)


def get_batch_logps_padded(
    per_token_logps: torch.Tensor, labels: torch.Tensor, average_log_prob: bool = False
) -> torch.Tensor:
    """Per-row sum (or mean) for a padded ``[B, T]`` batch; open_instruct/dpo_utils.py:689-712."""
    if per_token_logps.ndim != 2:
        raise ValueError("per_token_logps must have shape [B, T]")
    b, t = per_token_logps.shape
    return _SeqLogps.apply(per_token_logps, labels, None, b, t, average_log_prob)


def _split_prefixed_batch(batch: dict) -> tuple[dict, dict]:
    chosen = {k[len("chosen_") :]: v for k, v in batch.items() if k.startswith("chosen_")}
    rejected = {k[len("rejected_") :]: v for k, v in batch.items() if k.startswith("rejected_")}
    return chosen, rejected


def concatenated_inputs(batch: dict, tag: str = "concatenated_") -> tuple[dict, int]:
    """Chosen then rejected along the token dim of a packed batch; open_instruct/padding_free_collator.py:166-199.

    Integer plumbing only (``torch.cat`` on ids and boundaries); returns the number of pairs.
    """
    chosen, rejected = _split_prefixed_batch(batch)
    ret = {f"{tag}input_ids": torch.cat([chosen["input_ids"], rejected["input_ids"]], dim=-1)}
    if "labels" in chosen:
        ret[f"{tag}labels"] = torch.cat([chosen["labels"], rejected["labels"]], dim=-1)
    if "cu_seq_lens_q" in chosen:
        offset = chosen["input_ids"].shape[-1]
        for side in ("q", "k"):
            key = f"cu_seq_lens_{side}"
            ret[f"{tag}{key}"] = torch.cat([chosen[key], rejected[key][1:] + offset])
            mkey = f"max_length_{side}"
            ret[f"{tag}{mkey}"] = max(chosen[mkey], rejected[mkey])
    if "position_ids" in chosen:
        ret[f"{tag}position_ids"] = torch.cat([chosen["position_ids"], rejected["position_ids"]], dim=-1)
    if "seq_idx" in chosen:
        n_chosen = len(chosen["cu_seq_lens_k"]) - 1
        ret[f"{tag}seq_idx"] = torch.cat([chosen["seq_idx"], rejected["seq_idx"] + n_chosen], dim=-1)
    return ret, len(chosen["cu_seq_lens_k"]) - 1


def _cu_seq_lens_of(batch: dict) -> list[torch.Tensor]:
    """The key-side boundary tensors of a packed batch: ``cu_seq_lens_k`` (GRPO) or the chosen and rejected
    ones (DPO)."""
    return [v for k, v in batch.items() if k.endswith("cu_seq_lens_k")]


def get_num_tokens(batch: dict) -> int:
    """Real (non-padding) tokens of a training batch; open_instruct/padding_free_collator.py:232-249.

    Packed: the last boundary of every ``*cu_seq_lens_k``; padded: the sum of every ``*attention_mask``;
    otherwise the element count of the ``input_ids`` tensors.  Returns a Python number (one host read),
    as the reference does.
    """
    cu = _cu_seq_lens_of(batch)
    if cu:
        return sum(c[-1].item() for c in cu)
    masks = [v for k, v in batch.items() if k.endswith("attention_mask")]
    if masks:
        return sum(m.sum().item() for m in masks)
    return sum(v.numel() for k, v in batch.items() if "input_ids" in k and isinstance(v, torch.Tensor))


def get_num_padded_tokens(batch: dict) -> int:
    """All token positions of a batch, padding included; open_instruct/padding_free_collator.py:252-257."""
    return sum(v.numel() for k, v in batch.items() if k.endswith("input_ids") and isinstance(v, torch.Tensor))


def get_num_sequences(batch: dict) -> torch.Tensor:
    """Sequences of a batch as a scalar tensor (no host read); open_instruct/padding_free_collator.py:260-273.

    Packed: the strictly increasing steps of every ``*cu_seq_lens_k`` (repeated boundaries are padding);
    padded: the rows of every ``*input_ids``.
    """
    cu = _cu_seq_lens_of(batch)
    if cu:
        return sum((c[..., 1:] > c[..., :-1]).sum() for c in cu)
    return torch.tensor(sum(v.shape[0] for k, v in batch.items() if k.endswith("input_ids")))
