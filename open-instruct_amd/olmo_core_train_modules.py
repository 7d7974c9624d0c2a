"""DPO LM head that returns per-token log-probabilities, backed by the fused lm_head kernel.

Mirrors ``DPOLMHead`` of the reference (open_instruct/olmo_core_train_modules.py:39-85), which
subclasses ``olmo_core.nn.lm_head.LMHead``.  olmo-core is a third-party package outside this
build, so this class is a plain ``torch.nn.Module`` with the attributes the reference's forward
touches (``norm``, ``w_out``) and the same ``forward`` keyword signature and return fields.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Literal

import torch

from . import lm_head, padding_free_collator


@dataclass
class LMOutputWithLoss:
    """Same fields as ``olmo_core.nn.lm_head.LMOutputWithLoss``."""

    logits: torch.Tensor | None
    loss: torch.Tensor
    ce_loss: torch.Tensor
    z_loss: torch.Tensor | None


class DPOLMHead(torch.nn.Module):
    """``norm(x) -> w_out -> per-token logps`` in one fused call.

    ``output.loss[b, i] = log p(labels[b, i+1] | x[b, i])`` with the label shift done internally,
    as ``calculate_per_token_logps`` does (open_instruct/padding_free_collator.py:10-16).  The
    ``[B, T, V]`` logits are never formed when labels are given.

    Positions whose next label is ``ignore_index`` (prompt and padding tokens, the last position)
    are not multiplied at all: their entry of ``output.loss`` is 0 and they receive no gradient.
    The reference scores token 0 there (its ``clamp(min=0)``) and throws the number away when the
    per-sequence sums mask those positions (open_instruct/dpo_utils.py:689-712,
    open_instruct/padding_free_collator.py:202-229), so every result downstream is the same; set
    ``score_ignored_positions = True`` on the module to reproduce the discarded numbers too.
    """

    score_ignored_positions = False
    # Set for the duration of one model call by open_instruct_amd.dpo_utils.fused_loss_olmo: the keyword
    # arguments of dpo_loss_on_hidden.  The head then computes the preference loss and both gradients in the
    # same call as the logps (nothing recomputed) and leaves the result in `fused_result`.
    fused_loss: dict | None = None
    fused_result = None

    def __init__(self, d_model: int, vocab_size: int, bias: bool = False, norm: torch.nn.Module | None = None,
                 dtype: torch.dtype = torch.bfloat16, device=None):  # fmt: skip
        super().__init__()
        if bias:
            raise NotImplementedError("the fused lm_head path is bias-free, like the reference's lm heads")
        self.norm = norm
        self.w_out = torch.nn.Linear(d_model, vocab_size, bias=False, dtype=dtype, device=device)
        self.tp_enabled = False

    def forward(
        self,
        x: torch.Tensor,
        *,
        labels: torch.Tensor | None = None,
        ignore_index: int = -100,
        loss_reduction: Literal["mean", "sum", "none"] = "mean",
        z_loss_multiplier: float | None = None,
        loss_div_factor: torch.Tensor | float | None = None,
        return_logits: bool | None = None,
        logits_to_keep: int | torch.Tensor = 0,
    ) -> torch.Tensor | LMOutputWithLoss:
        h = self.norm(x) if self.norm is not None else x
        if labels is None:
            # no labels: the parent class returns plain logits (library GEMM; not the fused path)
            return self.w_out(h)
        if self.fused_loss is not None:
            from . import dpo_utils

            if ignore_index != -100:
                raise ValueError("the fused preference loss scores against -100 as the ignored label")
            self.fused_result = dpo_utils.dpo_loss_on_hidden(h, self.w_out.weight, labels, **self.fused_loss)
            logps = self.fused_result.per_token_logps
            return LMOutputWithLoss(logits=None, loss=logps, ce_loss=logps.clone(), z_loss=None)
        shifted = padding_free_collator.shift_labels(labels)
        keep = None if self.score_ignored_positions else shifted != ignore_index
        per_token_logps, _ = lm_head.fused_lm_head_logprobs(h, self.w_out.weight, shifted, mask=keep)
        return LMOutputWithLoss(
            logits=None, loss=per_token_logps, ce_loss=per_token_logps.detach().clone(), z_loss=None
        )
