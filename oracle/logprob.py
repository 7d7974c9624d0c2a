"""Oracle: per-token log-probability, entropy and KL estimators (test infrastructure only).

Each function names the reference lines it restates.  ``compute_dtype`` selects the arithmetic
type the restatement runs in: ``None`` keeps the input dtype (what the reference's GRPO path does),
``torch.float32`` is the fp32-accumulate target the HIP kernels are held to, ``torch.float64``
is used by the tests that pin the oracle itself.
"""

from __future__ import annotations

import torch


def _as(x: torch.Tensor, compute_dtype: torch.dtype | None) -> torch.Tensor:
    return x if compute_dtype is None else x.to(compute_dtype)


def log_softmax_and_gather(
    logits: torch.Tensor,
    index: torch.Tensor,
    compute_dtype: torch.dtype | None = torch.float32,
    temperature: float = 1.0,
) -> torch.Tensor:
    """``z[..., idx] - logsumexp(z, -1)``.

    Restates open_instruct/model_utils.py:587-600 (``log_softmax`` then ``gather`` on the last
    dim).  The division by ``temperature`` that the caller performs first
    (open_instruct/grpo_utils.py:560) is folded in here so the oracle and the kernel see the same
    unscaled logits.
    """
    z = _as(logits, compute_dtype)
    if temperature != 1.0:
        z = z / temperature
    picked = torch.take_along_dim(z, index.unsqueeze(-1), dim=-1).squeeze(-1)
    return picked - torch.logsumexp(z, dim=-1)


def entropy_from_logits(
    logits: torch.Tensor, compute_dtype: torch.dtype | None = torch.float32, temperature: float = 1.0
) -> torch.Tensor:
    """``logsumexp(z) - sum_j softmax(z)_j z_j``; restates open_instruct/model_utils.py:326-333."""
    z = _as(logits, compute_dtype)
    if temperature != 1.0:
        z = z / temperature
    lse = torch.logsumexp(z, dim=-1)
    p = torch.exp(z - lse.unsqueeze(-1))
    return lse - (p * z).sum(dim=-1)


def estimate_kl(ref_logprobs_diff: torch.Tensor, ratio: torch.Tensor) -> torch.Tensor:
    """Four KL estimators stacked on a new leading dim; restates open_instruct/model_utils.py:793-818.

    ``d`` is ``new - ref`` already clamped to +-40 by the caller (open_instruct/grpo_utils.py:532).
    """
    d = ref_logprobs_diff
    k0 = d
    k1 = d * d / 2
    k2 = torch.expm1(-d) + d
    k3 = ratio * d
    return torch.stack((k0, k1, k2, k3), dim=0)


def shift_labels(labels: torch.Tensor, ignore_index: int = -100) -> torch.Tensor:
    """``out[:, i] = labels[:, i + 1]``, last position ``ignore_index``.

    Restates the first two lines of open_instruct/padding_free_collator.py:10-16.
    """
    out = torch.full_like(labels, ignore_index)
    out[:, :-1] = labels[:, 1:]
    return out


def calculate_per_token_logps(
    logits: torch.Tensor, labels: torch.Tensor, compute_dtype: torch.dtype = torch.float32
) -> torch.Tensor:
    """Per-token log-probability of the *next* label, always computed in (at least) fp32.

    Restates open_instruct/padding_free_collator.py:10-16: the labels are shifted left by one
    inside the function, ignored labels (negative) are clamped to token 0, and the logits are
    upcast to fp32 before ``log_softmax``.
    """
    safe = shift_labels(labels).clamp(min=0)
    return log_softmax_and_gather(logits, safe, compute_dtype=compute_dtype)
