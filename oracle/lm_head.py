"""Oracle: lm_head projection followed by per-token logprob / entropy (test infrastructure only).

The projection itself is third-party code in the reference (a bias-free ``nn.Linear(H, V)`` in
HuggingFace causal-LM classes, reached at open_instruct/grpo_utils.py:558-559 and
open_instruct/dpo_utils.py:859-863; ``olmo_core.nn.lm_head.LMHead.w_out`` reached at
open_instruct/olmo_core_train_modules.py:71-72).  It is restated with the textbook routine
``F.linear`` on inputs upcast to the compute dtype, i.e. bf16 products accumulated in fp32/fp64
without an intermediate rounding of the logits to bf16.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from oracle import logprob


def lm_head_logits(hidden: torch.Tensor, weight: torch.Tensor, compute_dtype=torch.float32) -> torch.Tensor:
    return F.linear(hidden.to(compute_dtype), weight.to(compute_dtype))


def lm_head_logprobs(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    return_entropy: bool = False,
    compute_dtype=torch.float32,
    row_chunk: int = 2048,
):
    """``(logprob[N], entropy[N] or None)`` for ``hidden [N,H]``, ``weight [V,H]``, ``labels [N]``.

    Negative (ignored) labels are scored as token 0, matching the ``clamp(min=0)`` at
    open_instruct/padding_free_collator.py:15.  Rows are processed in chunks so the ``[N, V]``
    product never has to exist at once; autograd still flows to ``hidden`` and ``weight``.
    """
    safe = labels.clamp(min=0)
    lps, ents = [], []
    for s in range(0, hidden.shape[0], row_chunk):
        z = lm_head_logits(hidden[s : s + row_chunk], weight, compute_dtype)
        lps.append(logprob.log_softmax_and_gather(z, safe[s : s + row_chunk], None, temperature))
        if return_entropy:
            with torch.no_grad():
                ents.append(logprob.entropy_from_logits(z, None, temperature))
    lp = torch.cat(lps) if lps else hidden.new_zeros(0, dtype=compute_dtype)
    ent = (torch.cat(ents) if ents else hidden.new_zeros(0, dtype=compute_dtype)) if return_entropy else None
    return lp, ent


def linear_cross_entropy(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    num_items_in_batch=None,
    ignore_index: int = -100,
    compute_dtype=torch.float32,
):
    """Causal-LM cross-entropy as the HuggingFace model forward computes it for the reference's SFT
    loop (open_instruct/finetune.py:818-824; third-party ``transformers.loss.loss_utils.ForCausalLMLoss``):
    labels padded with ``ignore_index`` and shifted left by one, ``F.cross_entropy`` over the
    flattened positions with reduction "mean", or "sum" divided by ``num_items_in_batch``."""
    logits = lm_head_logits(hidden, weight, compute_dtype)
    shifted = F.pad(labels, (0, 1), value=ignore_index)[..., 1:].reshape(-1)
    flat = logits.reshape(-1, logits.shape[-1])
    if num_items_in_batch is None:
        return F.cross_entropy(flat, shifted, ignore_index=ignore_index, reduction="mean")
    return F.cross_entropy(flat, shifted, ignore_index=ignore_index, reduction="sum") / num_items_in_batch
