"""Oracle: GRPO per-token loss, rho correction and group advantages (test infrastructure only).

``config`` arguments are duck-typed exactly as in the reference (attribute reads only), so the
reference's own ``MagicMock`` style configs or a ``types.SimpleNamespace`` both work.
"""

from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch

from oracle import logprob, reductions

INVALID_LOGPROB = 1.0  # open_instruct/utils.py:83


def mask_logprobs(logprobs: torch.Tensor, response_mask: torch.Tensor) -> torch.Tensor:
    """Off-mask positions and NaNs become +1.0; restates open_instruct/grpo_utils.py:340-344."""
    out = torch.where(response_mask, logprobs, torch.full_like(logprobs, INVALID_LOGPROB))
    return torch.where(torch.isnan(out), torch.full_like(out, INVALID_LOGPROB), out)


def _row_mean_over_mask(values: torch.Tensor, response_mask: torch.Tensor) -> torch.Tensor:
    """Per-row masked mean broadcast to every token (open_instruct/grpo_utils.py:380-390)."""
    w = response_mask.to(values.dtype)
    mean = (values * w).sum(-1, keepdim=True) / w.sum(-1, keepdim=True).clamp_min(1.0)
    return mean.expand_as(values)


def _drops(rho: torch.Tensor, response_mask: torch.Tensor, lower: float, upper: float):
    """Below-``lower`` / above-``upper`` drop masks; a bound of 0 disables that side
    (open_instruct/grpo_utils.py:372-377)."""
    none = torch.zeros_like(response_mask)
    low = (rho < lower) & response_mask if lower > 0.0 else none
    high = (rho > upper) & response_mask if upper > 0.0 else none
    return low, high


@dataclass
class RhoCorrection:
    weights: torch.Tensor
    metrics: dict[str, torch.Tensor]
    histogram_metrics: dict[str, torch.Tensor] = field(default_factory=dict)


def compute_rho_correction(old_logprob, vllm_logprobs, response_mask, advantages, config) -> RhoCorrection:
    """Train/infer mismatch weights; restates open_instruct/grpo_utils.py:410-463.

    Order of operations that the reference's tests fix: clamp the log-difference to +-10 on the
    mask (0 elsewhere); optional per-row geometric mean; drop masks from the *effective* rho (or,
    in TV mode, from the row mean of ``|rho - 1|`` restricted to tokens whose sign(logdiff) *
    advantage is positive); clamp; zero the dropped and the off-mask tokens.
    """
    diff = torch.where(response_mask, (old_logprob - vllm_logprobs).clamp(-10.0, 10.0), torch.zeros_like(old_logprob))
    rho = diff.exp()
    hist = {"val/rho_hist": rho[response_mask].detach().float()}
    if not config.use_rho_correction:
        return RhoCorrection(torch.ones_like(rho), {}, hist)

    effective = _row_mean_over_mask(diff, response_mask).exp() if config.rho_mask_sequence_level else rho
    if config.rho_mask_tv_divergence:
        tv_row = _row_mean_over_mask((rho - 1.0).abs(), response_mask)
        low, high = _drops(tv_row, response_mask, config.rho_mask_lower_bound, config.rho_mask_upper_bound)
        grows_tv = torch.sign(diff) * advantages > 0
        low, high = low & grows_tv, high & grows_tv
    else:
        low, high = _drops(effective, response_mask, config.rho_mask_lower_bound, config.rho_mask_upper_bound)
    keep = response_mask & ~low & ~high

    clamped = effective
    if config.rho_clamp_lower_bound > 0.0:
        clamped = clamped.clamp(min=config.rho_clamp_lower_bound)
    if config.rho_clamp_upper_bound > 0.0:
        clamped = clamped.clamp(max=config.rho_clamp_upper_bound)
    weights = torch.where(keep, clamped, torch.zeros_like(clamped))
    metrics = {
        "val/rho_drop_frac": (low | high).float(),
        "val/rho_drop_low_frac": low.float(),
        "val/rho_drop_high_frac": high.float(),
        "val/rho_weight": weights.float(),
        "val/rho_clipfrac": (clamped != effective).float(),
    }
    return RhoCorrection(weights, metrics, hist)


def compute_grpo_loss(new_logprobs, ratio, advantages, ref_logprobs, config, rho_weights):
    """Per-token policy-gradient loss, clip indicator and KL; restates open_instruct/grpo_utils.py:504-538.

    DAPO: ``max(-A r, -A clamp(r, 1-eps_lo, 1+eps_hi))``, indicator where the clipped branch is
    strictly larger.  CISPO: ``-A clamp(stopgrad(r), max=1+eps_hi) * new_logprobs``.  Both are then
    multiplied by ``rho_weights`` (indicator by ``rho_weights != 0``).  KL is estimator
    ``config.kl_estimator`` of ``clamp(new - ref, +-40)`` or zeros without a reference.
    """
    name = str(getattr(config.loss_fn, "value", config.loss_fn))
    hi = 1.0 + config.clip_higher
    if name == "dapo":
        lo = 1.0 - config.clip_lower
        plain = -advantages * ratio
        clipped = -advantages * ratio.clamp(lo, hi)
        clipfrac = (clipped > plain).float()
        pg = torch.maximum(plain, clipped)
    elif name == "cispo":
        clipfrac = (ratio > hi).float()
        pg = -advantages * ratio.detach().clamp(max=hi) * new_logprobs
    else:
        raise ValueError(f"Invalid loss function: {config.loss_fn}")
    pg = pg * rho_weights
    clipfrac = clipfrac * (rho_weights != 0).float()
    if ref_logprobs is None:
        kl = torch.zeros_like(pg)
    else:
        d = (new_logprobs - ref_logprobs).clamp(-40.0, 40.0)
        kl = logprob.estimate_kl(d, ratio)[config.kl_estimator]
    return pg, clipfrac, kl


def group_advantages(scores: np.ndarray, group_size: int, normalization: str = "standard") -> np.ndarray:
    """Group-normalised advantages in float64 numpy; restates open_instruct/data_loader.py:1472-1484.

    Population std (ddof=0), ``+1e-8`` in the denominator; "centered" subtracts the mean only.
    """
    s = np.asarray(scores, dtype=np.float64)
    g = s.reshape(-1, group_size)
    mean = np.repeat(g.mean(axis=-1), group_size)
    if normalization == "standard":
        std = np.repeat(g.std(axis=-1), group_size)
        return (s - mean) / (std + 1e-8)
    if normalization == "centered":
        return s - mean
    raise ValueError(f"Invalid advantage normalization type: {normalization}")


def grpo_token_loss(
    new_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor,
    ref_logprobs: torch.Tensor | None,
    advantages: torch.Tensor,
    response_mask: torch.Tensor,
    config,
    rho_weights: torch.Tensor | None = None,
    loss_denominator: float | None = None,
    axis: int | None = None,
    dp_scale: float = 1.0,
):
    """Scalar loss assembled as the callers do; restates open_instruct/grpo_fast.py:702-724 and
    open_instruct/olmo_core_train_modules.py:547-568.

    ``ratio = exp(new - old)``; ``loss = masked_mean(pg + beta kl, mask, axis, denominator) * dp_scale``.
    Returns ``(loss, pg, clipfrac, kl, ratio)``.
    """
    ratio = (new_logprobs - old_logprobs).exp()
    if rho_weights is None:
        rho_weights = torch.ones_like(ratio)
    pg, clipfrac, kl = compute_grpo_loss(new_logprobs, ratio, advantages, ref_logprobs, config, rho_weights)
    loss = reductions.masked_mean(pg + config.beta * kl, response_mask, axis, loss_denominator) * dp_scale
    return loss, pg, clipfrac, kl, ratio


def forward_for_logprobs(
    logits: torch.Tensor,
    query_responses: torch.Tensor,
    pad_token_id: int,
    temperature: float,
    return_entropy: bool = False,
    compute_dtype: torch.dtype | None = torch.float32,
):
    """Tail of open_instruct/grpo_utils.py:541-574 after the model call: scale by temperature,
    drop the last position, labels are the ids shifted left with pad ids replaced by 0."""
    z = logits[:, :-1]
    labels = query_responses[:, 1:].clone()
    labels[labels == pad_token_id] = 0
    lp = logprob.log_softmax_and_gather(z, labels, compute_dtype=compute_dtype, temperature=temperature)
    ent = None
    if return_entropy:
        with torch.no_grad():
            ent = logprob.entropy_from_logits(z, compute_dtype=compute_dtype, temperature=temperature)
    return lp, ent


def compute_vllm_local_debug_metrics(
    local_logprobs: torch.Tensor, vllm_logprobs: torch.Tensor, response_mask: torch.Tensor
) -> dict[str, float]:
    """Restates open_instruct/grpo_utils.py:345-369: statistics of ``|local - vllm|`` and of
    ``exp(vllm) * (vllm - local)`` over positions that are in the mask and not NaN on the vLLM side."""
    valid = response_mask.bool() & ~torch.isnan(vllm_logprobs)
    count = int(valid.sum())
    zero = torch.tensor(0.0)
    diff = (local_logprobs - vllm_logprobs).abs().masked_fill(~valid, 0.0)
    rkl = (torch.exp(vllm_logprobs) * (vllm_logprobs - local_logprobs)).masked_fill(~valid, 0.0)
    return {
        "debug/vllm_vs_local_logprob_diff_mean": float(diff.sum() / count if count > 0 else zero),
        "debug/vllm_vs_local_logprob_diff_max": float(diff.max() if count > 0 else zero),
        "debug/vllm_vs_local_logprob_diff_std": float(diff[valid].std() if count > 1 else zero),
        "debug/vllm_local_reverse_kl": float(rkl.sum() / count if count > 0 else zero),
    }


LOSS_STAT_KEYS = (
    "loss/kl_avg", "loss/policy_avg", "loss/total_avg", "objective/kl0_avg", "objective/kl1_avg",
    "objective/kl2_avg", "objective/kl3_avg", "policy/clipfrac_avg", "val/ratio", "val/rho_clipfrac",
    "val/rho_weight", "val/rho_drop_frac", "val/rho_drop_low_frac", "val/rho_drop_high_frac",
)  # fmt: skip


def create_loss_stats(num_samples: int, record_entropy: bool = False) -> dict[str, torch.Tensor]:
    """One zero vector per key; restates open_instruct/grpo_utils.py:674-696."""
    keys = LOSS_STAT_KEYS + (("policy/entropy_avg",) if record_entropy else ())
    return {k: torch.zeros(num_samples) for k in keys}


def populate_sample_loss_stats(
    stats, sample_idx, pg_loss, clipfrac, ratio, loss, response_mask, new_logprobs, ref_logprobs, entropy, config,
    rho_metrics=None,
) -> None:  # fmt: skip
    """Masked means of one sample written at ``sample_idx``; restates open_instruct/grpo_utils.py:699-729.

    KL entries only with ``config.load_ref_policy`` and reference logprobs (the four estimators of
    ``clamp(new - ref, +-40)`` and ``beta`` times the selected one); rho entries only when the
    metric tensors are given; entropy only when given; the loss is stored as passed."""
    mm = lambda t: reductions.masked_mean(t, response_mask)  # noqa: E731
    if config.load_ref_policy and ref_logprobs is not None:
        kls = mm(logprob.estimate_kl((new_logprobs - ref_logprobs).clamp(-40.0, 40.0), ratio)).float()
        for j in range(4):
            stats[f"objective/kl{j}_avg"][sample_idx] = kls[j]
        stats["loss/kl_avg"][sample_idx] = kls[config.kl_estimator] * config.beta
    for key, value in (rho_metrics or {}).items():
        stats[key][sample_idx] = mm(value)
    stats["policy/clipfrac_avg"][sample_idx] = mm(clipfrac)
    stats["loss/policy_avg"][sample_idx] = mm(pg_loss)
    stats["loss/total_avg"][sample_idx] = loss
    stats["val/ratio"][sample_idx] = mm(ratio)
    if entropy is not None:
        stats["policy/entropy_avg"][sample_idx] = mm(entropy).float()


def compute_metrics_from_loss_stats(stats: dict[str, torch.Tensor], token_counts: torch.Tensor) -> dict[str, float]:
    """Token-weighted average of every key over the samples and the weighted variance of
    ``val/ratio``; restates open_instruct/grpo_utils.py:732-742."""
    total = token_counts.sum()
    w = token_counts / total if total > 0 else torch.zeros_like(token_counts)
    out = {k: float((v * w).sum()) for k, v in stats.items()}
    out["val/ratio_var"] = float((w * (stats["val/ratio"] - out["val/ratio"]) ** 2).sum())
    return out
