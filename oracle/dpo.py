"""Oracle: DPO-family sequence losses (test infrastructure only)."""

from __future__ import annotations

import torch
import torch.nn.functional as F


def _sigmoid_pair_loss(x: torch.Tensor, beta: float, label_smoothing: float) -> torch.Tensor:
    """``-(1-ls) log sigma(beta x) - ls log sigma(-beta x)`` written through softplus
    (``-log sigma(u) = softplus(-u)``)."""
    u = beta * x
    return F.softplus(-u) * (1 - label_smoothing) + F.softplus(u) * label_smoothing


def dpo_loss(
    policy_chosen_logps,
    policy_rejected_logps,
    reference_chosen_logps,
    reference_rejected_logps,
    beta: float,
    reference_free: bool = False,
    label_smoothing: float = 0.0,
):
    """Sigmoid DPO loss per pair plus detached rewards; restates open_instruct/dpo_utils.py:523-563."""
    x = policy_chosen_logps - policy_rejected_logps
    if not reference_free:
        x = x - (reference_chosen_logps - reference_rejected_logps)
    losses = _sigmoid_pair_loss(x, beta, label_smoothing)
    chosen_rewards = (beta * (policy_chosen_logps - reference_chosen_logps)).detach()
    rejected_rewards = (beta * (policy_rejected_logps - reference_rejected_logps)).detach()
    return losses, chosen_rewards, rejected_rewards


def simpo_loss(policy_chosen_logps, policy_rejected_logps, beta: float, gamma_beta_ratio: float, label_smoothing=0.0):
    """SimPO: margin ``gamma/beta`` in place of the reference model; restates
    open_instruct/dpo_utils.py:617-642."""
    x = policy_chosen_logps - policy_rejected_logps - gamma_beta_ratio
    losses = _sigmoid_pair_loss(x, beta, label_smoothing)
    return losses, (beta * policy_chosen_logps).detach(), (beta * policy_rejected_logps).detach()


def wpo_loss(
    policy_chosen_logps,
    policy_rejected_logps,
    reference_chosen_logps,
    reference_rejected_logps,
    beta: float,
    chosen_loss_mask,
    rejected_loss_mask,
    label_smoothing: float = 0.0,
):
    """WPO: DPO weighted by ``min(1, exp(avg_c + avg_r))``; restates open_instruct/dpo_utils.py:566-613.

    The "averages" follow the reference literally: the per-sequence logps are broadcast against
    the ``[bs, T]`` token masks, summed over the last dim and divided by the mask count.
    """
    x = (policy_chosen_logps - policy_rejected_logps) - (reference_chosen_logps - reference_rejected_logps)
    avg_c = (policy_chosen_logps * chosen_loss_mask).sum(-1) / chosen_loss_mask.sum(-1)
    avg_r = (policy_rejected_logps * rejected_loss_mask).sum(-1) / rejected_loss_mask.sum(-1)
    w = torch.exp(avg_c + avg_r).clamp(max=1)
    losses = _sigmoid_pair_loss(x, beta, label_smoothing) * w
    chosen_rewards = (beta * (policy_chosen_logps - reference_chosen_logps)).detach()
    rejected_rewards = (beta * (policy_rejected_logps - reference_rejected_logps)).detach()
    return losses, chosen_rewards, rejected_rewards
