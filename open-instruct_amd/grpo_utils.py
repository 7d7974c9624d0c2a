"""GRPO logprob forward and loss functions on the GPU.

Names, signatures and argument meaning follow open_instruct/grpo_utils.py in the reference
(``mask_logprobs`` :340-344, ``compute_rho_correction`` :410-463, ``resolve_old_logprob`` :475-501,
``compute_grpo_loss`` :504-538, ``forward_for_logprobs`` :541-574, ``compute_logprobs`` :577-648,
``calculate_token_counts`` :651-671, loss-stat helpers :674-742).  ``config`` is duck-typed as in
the reference: only attributes are read.

``grpo_loss_fused`` and ``group_advantages`` have no single counterpart in the reference; they
carry the loss assembly of open_instruct/grpo_fast.py:702-724 and the advantage formula of
open_instruct/data_loader.py:1472-1484 in one or two kernel launches each.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass, field

import torch

from . import _lib, model_utils, olmo_core_utils
from .rl_utils import masked_mean


class GRPOLossType(str, enum.Enum):
    """The policy-gradient terms of the reference; open_instruct/grpo_utils.py:69-71.  A string enum: members
    compare equal to their names, which is also what ``config.loss_fn`` may hold."""

    dapo = "dapo"
    cispo = "cispo"

    def __str__(self) -> str:
        return self.value

INVALID_LOGPROB = 1.0  # open_instruct/utils.py:83


# ----------------------------------------------------------------------------------------------
# mask_logprobs
# ----------------------------------------------------------------------------------------------
class _MaskLogprobs(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logprobs, mask):
        _lib.require_gpu(logprobs, mask)
        lp, m = _lib.f32c(logprobs), _lib.mask_u8(mask)
        out = torch.empty_like(lp)
        _lib.call(
            "oi_mask_logprobs_fwd", lp.data_ptr(), m.data_ptr(), lp.numel(), INVALID_LOGPROB, out.data_ptr(),
            _lib.stream_of(lp),
        )  # fmt: skip
        ctx.save_for_backward(lp, m)
        ctx.in_dtype = logprobs.dtype
        return out.to(logprobs.dtype)

    @staticmethod
    def backward(ctx, grad_out):
        lp, m = ctx.saved_tensors
        g = _lib.f32c(grad_out)
        d = torch.empty_like(lp)
        _lib.call(
            "oi_mask_logprobs_bwd", lp.data_ptr(), m.data_ptr(), g.data_ptr(), lp.numel(), d.data_ptr(),
            _lib.stream_of(lp),
        )  # fmt: skip
        return d.to(ctx.in_dtype), None


def mask_logprobs(vllm_logprobs: torch.Tensor, response_mask: torch.Tensor) -> torch.Tensor:
    """Set non-response positions and NaNs to ``INVALID_LOGPROB`` (+1.0); open_instruct/grpo_utils.py:340-344."""
    if tuple(vllm_logprobs.shape) != tuple(response_mask.shape):
        response_mask = response_mask.expand_as(vllm_logprobs)
    return _MaskLogprobs.apply(vllm_logprobs, response_mask)


# ----------------------------------------------------------------------------------------------
# rho correction
# ----------------------------------------------------------------------------------------------
@dataclass
class RhoCorrection:
    """Same fields as the reference's dataclass (open_instruct/grpo_utils.py:393-407)."""

    weights: torch.Tensor
    metrics: dict[str, torch.Tensor]
    histogram_metrics: dict[str, torch.Tensor] = field(default_factory=dict)


def _expand_to(t: torch.Tensor, shape: tuple[int, ...], name: str) -> torch.Tensor:
    """``t`` broadcast to ``shape`` (a view), ``ValueError`` when it does not broadcast."""
    if tuple(t.shape) == tuple(shape):
        return t
    try:
        return t.expand(shape)
    except RuntimeError:
        raise ValueError(f"{name} of shape {tuple(t.shape)} does not broadcast to {tuple(shape)}") from None


def compute_rho_correction(
    old_logprob: torch.Tensor,
    vllm_logprobs: torch.Tensor,
    response_mask: torch.Tensor,
    advantages: torch.Tensor,
    config,
) -> RhoCorrection:
    """Train/infer mismatch weights rho = pi_train_old / pi_infer_old; open_instruct/grpo_utils.py:410-463.

    Stop-gradient by construction (the reference's inputs carry no grad either).
    """
    shape = tuple(old_logprob.shape)
    # the kernel indexes every side tensor per token: broadcastable inputs are expanded first
    vllm_logprobs = _expand_to(vllm_logprobs.detach(), shape, "vllm_logprobs")
    advantages = _expand_to(advantages.detach(), shape, "advantages")
    response_mask = _expand_to(response_mask, shape, "response_mask")
    dev = _lib.require_gpu(old_logprob, vllm_logprobs, response_mask, advantages)
    with torch.no_grad():
        old, vl, adv = _lib.f32c(old_logprob.detach()), _lib.f32c(vllm_logprobs), _lib.f32c(advantages)
        m = _lib.mask_u8(response_mask)
        cols = shape[-1] if shape else 1
        rows = old.numel() // max(cols, 1)
        bufs = torch.empty((6,) + shape, dtype=torch.float32, device=dev)
        use = bool(config.use_rho_correction)
        _lib.call(
            "oi_rho_correction", old.data_ptr(), vl.data_ptr(), m.data_ptr(), adv.data_ptr(), rows, cols,
            int(bool(config.rho_mask_sequence_level)) if use else 0,
            int(bool(config.rho_mask_tv_divergence)) if use else 0,
            float(config.rho_mask_lower_bound) if use else 0.0, float(config.rho_mask_upper_bound) if use else 0.0,
            float(config.rho_clamp_lower_bound) if use else 0.0, float(config.rho_clamp_upper_bound) if use else 0.0,
            *[bufs[k].data_ptr() for k in range(6)], _lib.stream_of(old),
        )  # fmt: skip
        rho, weights, drop_any, drop_low, drop_high, clipped = bufs.unbind(0)
        hist = {"val/rho_hist": rho[response_mask.bool()].detach().float()}
        if not use:
            return RhoCorrection(weights=torch.ones_like(rho), metrics={}, histogram_metrics=hist)
        metrics = {
            "val/rho_drop_frac": drop_any,
            "val/rho_drop_low_frac": drop_low,
            "val/rho_drop_high_frac": drop_high,
            "val/rho_weight": weights,
            "val/rho_clipfrac": clipped,
        }
        return RhoCorrection(weights=weights, metrics=metrics, histogram_metrics=hist)


def accumulate_rho_histograms(acc: dict[str, list[torch.Tensor]], correction: RhoCorrection) -> None:
    for key, values in correction.histogram_metrics.items():
        acc.setdefault(key, []).append(values.detach().cpu())


def finalize_rho_histograms(acc: dict[str, list[torch.Tensor]]) -> dict:
    return {key: torch.cat(chunks).numpy() for key, chunks in acc.items()}


def resolve_old_logprob(
    old_logprobs_cache: list,
    sample_idx: int,
    epoch_idx: int,
    num_mini_batches: int,
    use_vllm_logprobs: bool,
    vllm_logprobs: torch.Tensor,
    new_logprobs: torch.Tensor,
) -> torch.Tensor:
    """Baseline ("old") logprobs of one sample; host bookkeeping of open_instruct/grpo_utils.py:475-501.

    With several mini-batches the cache was filled by a separate no-grad pass and is only read.
    With a single mini-batch the first epoch's own logprobs (detached), or the sampler's when
    ``use_vllm_logprobs``, become the baseline of the later epochs, so the first epoch runs at
    ratio 1.
    """
    fills_cache = num_mini_batches <= 1 and epoch_idx == 0
    if fills_cache:
        old_logprobs_cache[sample_idx] = vllm_logprobs if use_vllm_logprobs else new_logprobs.detach()
    baseline = old_logprobs_cache[sample_idx]
    if baseline is None:
        raise AssertionError(f"no old logprobs cached for sample {sample_idx}")
    return baseline


# ----------------------------------------------------------------------------------------------
# compute_grpo_loss
# ----------------------------------------------------------------------------------------------
def _loss_fn_tag(config) -> int:
    name = str(getattr(config.loss_fn, "value", config.loss_fn))
    if name not in _lib.LOSS_FN_TAGS:
        raise ValueError(f"Invalid loss function: {config.loss_fn}")
    return _lib.LOSS_FN_TAGS[name]


def _clip_bounds(config) -> tuple[float, float]:
    # evaluated in double and rounded to fp32 once at the C boundary, like a Python scalar in torch.clamp
    return 1.0 - float(config.clip_lower), 1.0 + float(config.clip_higher)


class _GrpoTerms(torch.autograd.Function):
    @staticmethod
    def forward(ctx, new_logprobs, ratio, advantages, ref_logprobs, rho_weights, loss_fn, lo, hi, kl_estimator):
        dev = _lib.require_gpu(new_logprobs, ratio, advantages, ref_logprobs, rho_weights)
        shape = torch.broadcast_shapes(new_logprobs.shape, ratio.shape, advantages.shape, rho_weights.shape)
        nl = _lib.f32c(new_logprobs.expand(shape))
        rt = _lib.f32c(ratio.expand(shape))
        adv = _lib.f32c(advantages.expand(shape))
        w = _lib.f32c(rho_weights.expand(shape))
        ref = _lib.f32c(ref_logprobs.expand(shape)) if ref_logprobs is not None else None
        out = torch.empty((3,) + tuple(shape), dtype=torch.float32, device=dev)
        n = nl.numel()
        _lib.call(
            "oi_grpo_terms_fwd", nl.data_ptr(), rt.data_ptr(), adv.data_ptr(), _lib.ptr(ref), w.data_ptr(), n, loss_fn,
            lo, hi, kl_estimator, out[0].data_ptr(), out[1].data_ptr(), out[2].data_ptr(), _lib.stream_of(nl),
        )  # fmt: skip
        ctx.save_for_backward(nl, rt, adv, ref, w)
        ctx.cfg = (loss_fn, lo, hi, kl_estimator)
        ctx.in_shapes = (new_logprobs.shape, ratio.shape)
        pg, clipfrac, kl = out.unbind(0)
        ctx.mark_non_differentiable(clipfrac)
        return pg, clipfrac, kl

    @staticmethod
    def backward(ctx, g_pg, _g_clip, g_kl):
        nl, rt, adv, ref, w = ctx.saved_tensors
        loss_fn, lo, hi, kl_estimator = ctx.cfg
        need_new, need_ratio = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        g_pg = _lib.f32c(g_pg) if g_pg is not None else None
        g_kl = _lib.f32c(g_kl) if g_kl is not None else None
        d_new = torch.empty_like(nl) if need_new else None
        d_ratio = torch.empty_like(rt) if need_ratio else None
        _lib.call(
            "oi_grpo_terms_bwd", nl.data_ptr(), rt.data_ptr(), adv.data_ptr(), _lib.ptr(ref), w.data_ptr(),
            _lib.ptr(g_pg), _lib.ptr(g_kl), nl.numel(), loss_fn, lo, hi, kl_estimator, _lib.ptr(d_new),
            _lib.ptr(d_ratio), _lib.stream_of(nl),
        )  # fmt: skip
        if d_new is not None and d_new.shape != ctx.in_shapes[0]:
            d_new = d_new.sum_to_size(ctx.in_shapes[0])
        if d_ratio is not None and d_ratio.shape != ctx.in_shapes[1]:
            d_ratio = d_ratio.sum_to_size(ctx.in_shapes[1])
        return d_new, d_ratio, None, None, None, None, None, None, None


def compute_grpo_loss(
    new_logprobs: torch.Tensor,
    ratio: torch.Tensor,
    advantages: torch.Tensor,
    ref_logprobs: torch.Tensor | None,
    config,
    rho_weights: torch.Tensor,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Per-token ``(pg_loss, clipfrac, kl)``; drop-in for open_instruct/grpo_utils.py:504-538.

    DAPO gradients flow to ``ratio``; CISPO uses the detached ratio and sends its gradient to
    ``new_logprobs``; the KL term flows to ``new_logprobs`` (and to ``ratio`` for estimator 3).
    """
    tag = _loss_fn_tag(config)
    lo, hi = _clip_bounds(config)
    return _GrpoTerms.apply(
        new_logprobs, ratio, advantages, ref_logprobs, rho_weights, tag, lo, hi, int(config.kl_estimator)
    )


# ----------------------------------------------------------------------------------------------
# fused scalar loss (+ statistics) of one micro-batch
# ----------------------------------------------------------------------------------------------
# entry q of the kernels' statistics vector (OI_GRPO_NUM_STATS entries)
GRPO_STAT_NAMES = (
    "loss/total_avg",
    "loss/policy_avg",
    "objective/kl0_avg",
    "objective/kl1_avg",
    "objective/kl2_avg",
    "objective/kl3_avg",
    "policy/clipfrac_avg",
    "val/ratio",
    "policy/entropy_avg",
    "num_response_tokens",
    "val/rho_drop_frac",
    "val/rho_drop_low_frac",
    "val/rho_drop_high_frac",
    "val/rho_weight",
    "val/rho_clipfrac",
    "loss/kl_avg",
)
_STAT_ROW = {name: i for i, name in enumerate(GRPO_STAT_NAMES)}
# per-token indicator tensors of compute_rho_correction that the statistics kernels only average
_RHO_INDICATOR_KEYS = ("val/rho_drop_frac", "val/rho_drop_low_frac", "val/rho_drop_high_frac", "val/rho_clipfrac")


def _rho_indicator_ptrs(rho_metrics: dict[str, torch.Tensor] | None, shape) -> tuple[list, list]:
    """Device pointers (or None) of the four indicator tensors in the kernels' argument order, and the
    tensors that must stay alive for the duration of the call."""
    if not rho_metrics:
        return [None] * 4, []
    keep = [
        _lib.f32c(_expand_to(rho_metrics[k].detach(), shape, k)) if k in rho_metrics else None
        for k in _RHO_INDICATOR_KEYS
    ]
    return [_lib.ptr(t) for t in keep], keep


class _GrpoFused(torch.autograd.Function):
    @staticmethod
    def forward(ctx, new_logprobs, old, ref, adv, mask, rho, entropy, cfg, rho_metrics=None):
        dev = _lib.require_gpu(new_logprobs, old, ref, adv, mask, rho, entropy)
        loss_fn, lo, hi, kl_estimator, beta, axis_mode, denominator, scale = cfg
        nl = _lib.f32c(new_logprobs)
        if nl.ndim != 2:
            raise ValueError("grpo_loss_fused expects [rows, cols] tensors")
        rows, cols = nl.shape
        sides = [None if t is None else _lib.f32c(t.expand(rows, cols)) for t in (old, ref, adv, rho, entropy)]
        old_c, ref_c, adv_c, rho_c, ent_c = sides
        m = _lib.mask_u8(mask.expand(rows, cols))
        stats = torch.empty(len(GRPO_STAT_NAMES), dtype=torch.float32, device=dev)
        row_denoms = torch.empty(rows, dtype=torch.float32, device=dev)
        ws_bytes = _lib.load().oi_grpo_fused_workspace_bytes(rows, cols)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        rho_ptrs, _alive = _rho_indicator_ptrs(rho_metrics, (rows, cols))
        _lib.call(
            "oi_grpo_fused_fwd", nl.data_ptr(), _lib.ptr(old_c), _lib.ptr(ref_c), adv_c.data_ptr(), m.data_ptr(),
            _lib.ptr(rho_c), _lib.ptr(ent_c), *rho_ptrs, rows, cols, loss_fn, lo, hi, kl_estimator, beta, axis_mode,
            denominator, scale, stats.data_ptr(), row_denoms.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_of(nl),
        )  # fmt: skip
        ctx.save_for_backward(nl, old_c, ref_c, adv_c, m, rho_c, row_denoms)
        ctx.cfg = cfg
        ctx.in_dtype = new_logprobs.dtype
        loss = stats[0]
        ctx.mark_non_differentiable(stats)
        return loss.clone(), stats

    @staticmethod
    def backward(ctx, g_loss, _g_stats):
        nl, old_c, ref_c, adv_c, m, rho_c, row_denoms = ctx.saved_tensors
        loss_fn, lo, hi, kl_estimator, beta, _axis_mode, _denominator, scale = ctx.cfg
        g = _lib.f32c(g_loss).reshape(1)
        d_new = torch.empty_like(nl)
        rows, cols = nl.shape
        _lib.call(
            "oi_grpo_fused_bwd", nl.data_ptr(), _lib.ptr(old_c), _lib.ptr(ref_c), adv_c.data_ptr(), m.data_ptr(),
            _lib.ptr(rho_c), rows, cols, loss_fn, lo, hi, kl_estimator, beta, scale, row_denoms.data_ptr(),
            g.data_ptr(), d_new.data_ptr(), _lib.stream_of(nl),
        )  # fmt: skip
        return d_new.to(ctx.in_dtype), None, None, None, None, None, None, None, None


def grpo_loss_fused(
    new_logprobs: torch.Tensor,
    old_logprobs: torch.Tensor | None,
    ref_logprobs: torch.Tensor | None,
    advantages: torch.Tensor,
    response_mask: torch.Tensor,
    config,
    rho_weights: torch.Tensor | None = None,
    entropy: torch.Tensor | None = None,
    loss_denominator: float | None = None,
    axis: int | None = None,
    dp_scale: float = 1.0,
    rho_metrics: dict[str, torch.Tensor] | None = None,
) -> tuple[torch.Tensor, dict[str, torch.Tensor]]:
    """Scalar GRPO loss of a ``[B, T]`` micro-batch and its statistics in two launches.

    Equivalent to the reference sequence ``ratio = exp(new - old)`` → ``compute_grpo_loss`` →
    ``masked_mean(pg + beta * kl, mask, axis, loss_denominator) * dp_scale``
    (open_instruct/grpo_fast.py:702-724) plus the masked means that
    ``populate_sample_loss_stats`` records (open_instruct/grpo_utils.py:699-729).
    ``old_logprobs=None`` means ``old = new.detach()`` (ratio 1 with a live gradient).
    Differentiable with respect to ``new_logprobs`` only; ``old``/``ref``/``advantages``/``rho`` are
    constants, as in the reference.  ``rho_metrics`` (the ``metrics`` of
    :func:`compute_rho_correction`) adds the masked means of the rho indicators to the same pass.
    Returns ``(loss, stats)`` with ``stats`` keyed by ``GRPO_STAT_NAMES`` (0-dim views of one device
    vector, no host sync); ``populate_sample_loss_stats(..., fused_stats=stats)`` records them.
    """
    if axis not in (None, 1, -1):
        raise ValueError("axis must be None or the token axis (1)")
    if loss_denominator is not None and float(loss_denominator) <= 0.0:
        raise ValueError("loss_denominator must be positive when given")
    lo, hi = _clip_bounds(config)
    cfg = (
        _loss_fn_tag(config), lo, hi, int(config.kl_estimator), float(config.beta), 0 if axis is None else 1,
        0.0 if loss_denominator is None else float(loss_denominator), float(dp_scale),
    )  # fmt: skip
    detach = lambda t: None if t is None else t.detach()  # noqa: E731
    loss, stats = _GrpoFused.apply(
        new_logprobs, detach(old_logprobs), detach(ref_logprobs), advantages.detach(), response_mask,
        detach(rho_weights), detach(entropy), cfg, rho_metrics,
    )  # fmt: skip
    return loss, _StatsView(stats)


class _StatsView(dict):
    """The statistics of one micro-batch keyed by ``GRPO_STAT_NAMES``; ``vector`` is the device
    vector the 0-dim entries are views of."""

    def __init__(self, vector: torch.Tensor):
        super().__init__((name, vector[i]) for i, name in enumerate(GRPO_STAT_NAMES))
        self.vector = vector


# ----------------------------------------------------------------------------------------------
# GRPO on materialised logits: forward + gradient in one read and one write of the logits
# ----------------------------------------------------------------------------------------------
def _token_coef(mask: torch.Tensor, axis: int | None, loss_denominator: float | None, dp_scale: float) -> torch.Tensor:
    """``scale / denominator`` on response tokens, 0 elsewhere: the factor that ``masked_mean``
    (open_instruct/rl_utils.py:426-448) puts in front of every token's loss.  Device arithmetic only."""
    m = mask.to(torch.float32)
    if axis is None:
        den = m.sum() if loss_denominator is None else torch.full((), float(loss_denominator), device=m.device)
        inv = torch.where(den > 0, 1.0 / den.clamp(min=1e-30), torch.zeros_like(den))
        return m * (inv * float(dp_scale))
    den = m.sum(dim=1, keepdim=True) if loss_denominator is None else torch.full_like(m[:, :1], float(loss_denominator))
    inv = torch.where(den > 0, 1.0 / den.clamp(min=1e-30), torch.zeros_like(den))
    return m * (inv * (float(dp_scale) / m.shape[0]))


def _single_pass_ok(view: torch.Tensor, so: int, si: int) -> bool:
    """Rows must start on 16-byte boundaries for the fused kernel (the gradient tensor is allocated
    contiguous here, so with an aligned vocabulary size it qualifies whenever the logits do)."""
    vec = 16 // view.element_size()
    return view.data_ptr() % 16 == 0 and so % vec == 0 and si % vec == 0 and view.shape[-1] % vec == 0


def _grpo_on_logits_launch(logits, labels, old, ref, adv, rho, coef, inv_temperature, cfg, drop_last):
    """One launch: logprob, entropy and the gradient of the loss with respect to ``logits``."""
    dev = _lib.require_gpu(logits, labels, adv, coef)
    view = logits[..., :-1, :] if drop_last else logits
    view, n_outer, n_inner, so, si = model_utils._row_layout(view)
    dlogits = torch.empty(logits.shape, dtype=logits.dtype, device=dev)
    out_view = dlogits[..., :-1, :] if drop_last else dlogits
    if drop_last:
        dlogits[..., -1, :].zero_()
    _, _, _, oso, osi = model_utils._row_layout(out_view)
    loss_fn, lo, hi, kl_estimator, beta = cfg
    logprob = torch.empty(labels.shape, dtype=torch.float32, device=dev)
    entropy = torch.empty(labels.shape, dtype=torch.float32, device=dev)
    if n_outer * n_inner > 0:
        _lib.call(
            "oi_lsg_grpo_fwd_bwd", view.data_ptr(), _lib.DTYPE_TAGS[view.dtype], n_outer, n_inner, so, si,
            view.shape[-1], labels.data_ptr(), inv_temperature, _lib.ptr(old), _lib.ptr(ref), adv.data_ptr(),
            _lib.ptr(rho), coef.data_ptr(), loss_fn, lo, hi, kl_estimator, beta, logprob.data_ptr(),
            entropy.data_ptr(), None, out_view.data_ptr(), oso, osi, _lib.stream_of(view),
        )  # fmt: skip
    return logprob, entropy, dlogits


def _hand_out_once(ctx) -> None:
    """The stored gradients are scaled by the upstream gradient in place (the host never reads that
    scalar, so it cannot tell whether it is 1), which can be done once: a second backward over a
    retained graph would scale what the first one left.  It raises instead of returning that."""
    if ctx.handed_out:
        raise RuntimeError(
            "the gradients of this fused loss were computed inside its forward call and have been handed out "
            "(scaled in place by the upstream gradient) by an earlier backward(); call the loss function again "
            "instead of backpropagating through it a second time"
        )
    ctx.handed_out = True


class _AttachLogitsGrad(torch.autograd.Function):
    """Identity on the loss value whose backward hands out the gradient computed in the forward."""

    @staticmethod
    def forward(ctx, loss, logits, dlogits):
        ctx.save_for_backward(dlogits)
        ctx.handed_out = False
        return loss.clone()

    @staticmethod
    def backward(ctx, grad_loss):
        (dlogits,) = ctx.saved_tensors
        _hand_out_once(ctx)
        # The usual upstream gradient of a loss is exactly 1 and the stored tensor is the answer as it
        # is.  The kernel reads the device scalar and returns at once in that case; anything else is
        # applied in place.  The host never looks at the value.
        g = _lib.f32c(grad_loss.detach()).reshape(1)
        _lib.call(
            "oi_scale_by_device_scalar", dlogits.data_ptr(), _lib.DTYPE_TAGS[dlogits.dtype], dlogits.numel(),
            g.data_ptr(), _lib.stream_of(dlogits),
        )  # fmt: skip
        return None, dlogits, None


def grpo_loss_on_logits(
    logits: torch.Tensor,
    labels: torch.Tensor,
    old_logprobs: torch.Tensor | None,
    ref_logprobs: torch.Tensor | None,
    advantages: torch.Tensor,
    response_mask: torch.Tensor,
    config,
    temperature: float = 1.0,
    rho_weights: torch.Tensor | None = None,
    loss_denominator: float | None = None,
    axis: int | None = None,
    dp_scale: float = 1.0,
    drop_last: bool = False,
) -> tuple[torch.Tensor, dict[str, torch.Tensor], torch.Tensor, torch.Tensor]:
    """GRPO loss straight from materialised logits; returns ``(loss, stats, logprobs, entropy)``.

    Same result as ``forward_for_logprobs`` → ``grpo_loss_fused`` (open_instruct/grpo_utils.py:541-574,
    open_instruct/grpo_fast.py:702-724) and the same gradient with respect to ``logits`` after
    ``loss.backward()``, but HBM sees the ``[B, T, V]`` tensor read once and its gradient written
    once (a row waits on its CU between the two passes): a token's upstream gradient depends only on its own logprob and side inputs once the
    denominators are known, and those come from the mask.  The gradient is computed in the
    forward call and stored (one tensor of the logits' shape and dtype, which the backward pass
    would allocate anyway).  ``logits`` is ``[B, T, V]`` (``[B, T + 1, V]`` with ``drop_last``),
    ``labels`` and the side tensors ``[B, T]``.  ``old_logprobs=None`` means ``old =
    new.detach()``.  ``logprobs`` and ``entropy`` are returned detached, for logging.  Side tensors
    may be anything that broadcasts to ``labels.shape`` (``[B, 1]`` advantages, a 0-dim weight).
    Rows that do not fit the single-pass kernel (vocabulary not a multiple of the 16-byte vector,
    unaligned views), and calls that need no gradient (``torch.no_grad()``, logits without
    ``requires_grad``), go through the two-pass kernels with identical results.
    """
    if axis not in (None, 1, -1):
        raise ValueError("axis must be None or the token axis (1)")
    if loss_denominator is not None and float(loss_denominator) <= 0.0:
        raise ValueError("loss_denominator must be positive when given")
    if labels.ndim != 2 or tuple(response_mask.shape) != tuple(labels.shape):
        raise ValueError("labels and response_mask must be [B, T]")
    inv_t = model_utils._inv_temperature(temperature)
    view = logits[..., :-1, :] if drop_last else logits
    if tuple(view.shape[:-1]) != tuple(labels.shape):
        raise ValueError(f"labels {tuple(labels.shape)} do not match logits rows {tuple(view.shape[:-1])}")
    layout_view, _, _, so, si = model_utils._row_layout(view)
    wants_grad = torch.is_grad_enabled() and logits.requires_grad
    if not wants_grad or not _single_pass_ok(layout_view, so, si) or logits.dtype not in _lib.DTYPE_TAGS:
        logprob, entropy = model_utils.logprob_and_entropy(logits, labels, temperature=temperature, drop_last=drop_last)
        loss, stats = grpo_loss_fused(
            logprob, old_logprobs, ref_logprobs, advantages, response_mask, config, rho_weights=rho_weights,
            entropy=entropy, loss_denominator=loss_denominator, axis=axis, dp_scale=dp_scale,
        )  # fmt: skip
        return loss, stats, logprob.detach(), entropy
    lo, hi = _clip_bounds(config)
    cfg = (_loss_fn_tag(config), lo, hi, int(config.kl_estimator), float(config.beta))
    mask = response_mask if response_mask.dtype == torch.bool else response_mask != 0
    coef = _token_coef(mask, None if axis is None else 1, loss_denominator, dp_scale).contiguous()
    shape = tuple(labels.shape)
    # the kernel indexes every side tensor per token: broadcastable inputs are expanded first
    f32 = lambda t, name: None if t is None else _lib.f32c(_expand_to(t.detach(), shape, name))  # noqa: E731
    with torch.no_grad():
        logprob, entropy, dlogits = _grpo_on_logits_launch(
            logits.detach(), labels.long().contiguous(), f32(old_logprobs, "old_logprobs"),
            f32(ref_logprobs, "ref_logprobs"), f32(advantages, "advantages"), f32(rho_weights, "rho_weights"), coef,
            inv_t, cfg, drop_last,
        )  # fmt: skip
        loss, stats = grpo_loss_fused(
            logprob, old_logprobs, ref_logprobs, advantages, response_mask, config, rho_weights=rho_weights,
            entropy=entropy, loss_denominator=loss_denominator, axis=axis, dp_scale=dp_scale,
        )  # fmt: skip
    return _AttachLogitsGrad.apply(loss, logits, dlogits), stats, logprob, entropy


class _AttachHeadGrads(torch.autograd.Function):
    """Identity on the loss value whose backward hands out the gradients computed in the forward."""

    @staticmethod
    def forward(ctx, loss, hidden, weight, d_hidden, d_weight):
        ctx.save_for_backward(d_hidden, d_weight)
        ctx.handed_out = False
        return loss.clone()

    @staticmethod
    def backward(ctx, grad_loss):
        d_hidden, d_weight = ctx.saved_tensors
        _hand_out_once(ctx)
        g = _lib.f32c(grad_loss.detach()).reshape(1)
        for t in (d_hidden, d_weight):  # nothing is touched when the device scalar is exactly 1
            if t is not None:
                _lib.call(
                    "oi_scale_by_device_scalar", t.data_ptr(), _lib.DTYPE_TAGS[t.dtype], t.numel(), g.data_ptr(),
                    _lib.stream_of(t),
                )  # fmt: skip
        need_h, need_w = ctx.needs_input_grad[1], ctx.needs_input_grad[2]
        return None, (d_hidden if need_h else None), (d_weight if need_w else None), None, None


# slab size of the no-recompute step when the caller names none (selected tokens per slab)
DEFAULT_SLAB_TOKENS = 8192


def grpo_loss_on_hidden(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    old_logprobs: torch.Tensor | None,
    ref_logprobs: torch.Tensor | None,
    advantages: torch.Tensor,
    response_mask: torch.Tensor,
    config,
    temperature: float = 1.0,
    rho_weights: torch.Tensor | None = None,
    loss_denominator: float | None = None,
    axis: int | None = None,
    dp_scale: float = 1.0,
    token_slabs: bool | int = True,
) -> tuple[torch.Tensor, dict[str, torch.Tensor], torch.Tensor, torch.Tensor]:
    """GRPO loss straight from final hidden states; returns ``(loss, stats, logprobs, entropy)``.

    One call for ``fused_lm_head_logprobs`` → ``grpo_loss_fused`` → backward
    (open_instruct/grpo_utils.py:558-572 → :504-538 → open_instruct/grpo_fast.py:702-724): the
    ``[tokens, vocab]`` logits are never formed, rows off ``response_mask`` are not multiplied, and
    the gradients with respect to ``hidden`` and ``weight`` are computed inside the same call and
    handed out by ``loss.backward()`` (a token's upstream gradient depends only on its own logprob
    once the denominators are known, and those come from the mask).  ``hidden`` is ``[B, T, H]``
    bf16, ``weight`` ``[V, H]`` bf16, ``labels`` and the side tensors ``[B, T]`` (anything that
    broadcasts).  ``logprobs`` and ``entropy`` are returned detached, 0 off the mask.  Without a
    gradient to compute (``torch.no_grad()``, inputs without ``requires_grad``) only the forward runs.

    ``token_slabs`` (default ``True`` = slabs of at most ``DEFAULT_SLAB_TOKENS`` selected tokens; or a
    number of tokens) runs the step slab by slab without recomputing anything: the selected rows are
    split on the device into the fewest equal slabs, a slab's forward leaves its exponentials (all
    vocabulary columns, bf16, relative to each token's own label logit) in a slab-sized scratch
    buffer, the slab's tokens get their upstream gradient at once, and both backward products read
    that buffer before the next slab overwrites it (``d_weight`` accumulates in fp32 over the
    slabs).  6·N·H·V of matrix work instead of 8·N·H·V; the scratch is ``[slab, vocab]`` bf16 plus an
    fp32 ``[vocab, hidden]``, never ``[tokens, vocab]``.  The slab size hardly matters for the time of the step
    (8192 to 32768 tokens measured within 1 %); smaller slabs need less scratch.  The route has no limit on the size of the logits or on the
    temperature: a token whose label is extremely unlikely (largest logit more than 44 nats above the
    label's) or whose logits hold a NaN is flagged on the device and served by a recomputing backward
    over the flagged rows inside the same call.  ``token_slabs=False`` is the recomputing step: one
    forward over all selected rows, then a backward that recomputes the logits one vocabulary chunk at
    a time (8·N·H·V, scratch ``[tokens, 32768]`` bf16).

    ``loss.backward()`` may be called once per call of this function.
    """
    if axis not in (None, 1, -1):
        raise ValueError("axis must be None or the token axis (1)")
    if loss_denominator is not None and float(loss_denominator) <= 0.0:
        raise ValueError("loss_denominator must be positive when given")
    if labels.ndim != 2 or tuple(response_mask.shape) != tuple(labels.shape):
        raise ValueError("labels and response_mask must be [B, T]")
    if tuple(hidden.shape[:-1]) != tuple(labels.shape):
        raise ValueError(f"labels {tuple(labels.shape)} do not match hidden rows {tuple(hidden.shape[:-1])}")
    inv_t = model_utils._inv_temperature(temperature)
    wants_grad = torch.is_grad_enabled() and (hidden.requires_grad or weight.requires_grad)
    if not wants_grad:
        from . import lm_head

        with torch.no_grad():
            logprob, entropy = lm_head.fused_lm_head_logprobs(
                hidden, weight, labels, temperature=temperature, mask=response_mask, return_entropy=True
            )
            loss, stats = grpo_loss_fused(
                logprob, old_logprobs, ref_logprobs, advantages, response_mask, config, rho_weights=rho_weights,
                entropy=entropy, loss_denominator=loss_denominator, axis=axis, dp_scale=dp_scale,
            )  # fmt: skip
        return loss, stats, logprob, entropy
    dev = _lib.require_gpu(hidden, weight, labels, response_mask, advantages)
    if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise ValueError("the fused lm_head expects bf16 hidden states and weight")
    rows, cols = labels.shape
    h, v = hidden.shape[-1], weight.shape[0]
    if weight.ndim != 2 or weight.shape[1] != h or h % 64:
        raise ValueError(f"weight {tuple(weight.shape)} does not fit hidden size {h} (a multiple of 64)")
    shape = (rows, cols)
    f32 = lambda t, name: None if t is None else _lib.f32c(_expand_to(t.detach(), shape, name))  # noqa: E731
    old_c, ref_c = f32(old_logprobs, "old_logprobs"), f32(ref_logprobs, "ref_logprobs")
    adv_c, rho_c = f32(advantages, "advantages"), f32(rho_weights, "rho_weights")
    m = _lib.mask_u8(response_mask)
    hid = hidden.detach().reshape(rows * cols, h).contiguous()
    w = weight.detach().contiguous()
    lab = labels.to(torch.int64).contiguous()
    lo, hi = _clip_bounds(config)
    logprob = torch.empty(shape, dtype=torch.float32, device=dev)
    entropy = torch.empty(shape, dtype=torch.float32, device=dev)
    stats = torch.empty(len(GRPO_STAT_NAMES), dtype=torch.float32, device=dev)
    d_hidden = torch.empty_like(hid)
    d_weight = torch.empty_like(w) if weight.requires_grad else None
    lib = _lib.load()
    slab_tokens = 0
    if token_slabs:
        slab_tokens = DEFAULT_SLAB_TOKENS if token_slabs is True else int(token_slabs)
        if slab_tokens < 256:
            raise ValueError("token_slabs must be True, False or a number of tokens (at least 256)")
    ws_bytes = lib.oi_lmhead_grpo_workspace_bytes(rows, cols, h, v, int(d_weight is not None), slab_tokens)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    _lib.call(
        "oi_lmhead_grpo_fwd_bwd", hid.data_ptr(), w.data_ptr(), lab.data_ptr(), m.data_ptr(), _lib.ptr(old_c),
        _lib.ptr(ref_c), adv_c.data_ptr(), _lib.ptr(rho_c), rows, cols, h, v, inv_t, _loss_fn_tag(config), lo, hi,
        int(config.kl_estimator), float(config.beta), 0 if axis is None else 1,
        0.0 if loss_denominator is None else float(loss_denominator), float(dp_scale), logprob.data_ptr(),
        entropy.data_ptr(), stats.data_ptr(), d_hidden.data_ptr(), _lib.ptr(d_weight), slab_tokens, ws.data_ptr(),
        ws_bytes, _lib.stream_of(hid),
    )  # fmt: skip
    loss = _AttachHeadGrads.apply(stats[0], hidden, weight, d_hidden.reshape(hidden.shape), d_weight)
    return loss, _StatsView(stats), logprob, entropy


def group_advantages(scores: torch.Tensor, group_size: int, normalization: str = "standard") -> torch.Tensor:
    """Group-normalised advantages; open_instruct/data_loader.py:1472-1484 on the device.

    ``scores`` holds ``n_groups * group_size`` rewards, groups contiguous.  fp64 arithmetic with a
    population std and ``+1e-8`` like the reference's numpy code, fp32 result.
    """
    dev = _lib.require_gpu(scores)
    if normalization not in ("standard", "centered"):
        raise ValueError(f"Invalid advantage normalization type: {normalization}")
    s = scores.reshape(-1).to(torch.float64).contiguous()
    if group_size <= 0 or s.numel() % group_size:
        raise ValueError(f"{s.numel()} scores do not split into groups of {group_size}")
    out = torch.empty(s.numel(), dtype=torch.float32, device=dev)
    _lib.call(
        "oi_group_advantages", s.data_ptr(), s.numel() // group_size, group_size,
        0 if normalization == "standard" else 1, out.data_ptr(), _lib.stream_of(s),
    )  # fmt: skip
    return out


# ----------------------------------------------------------------------------------------------
# sampler-vs-trainer logprob debug metrics
# ----------------------------------------------------------------------------------------------
VLLM_LOCAL_DEBUG_KEYS = (
    "debug/vllm_vs_local_logprob_diff_mean",
    "debug/vllm_vs_local_logprob_diff_max",
    "debug/vllm_vs_local_logprob_diff_std",
    "debug/vllm_local_reverse_kl",
)


def vllm_local_debug_stats(
    local_logprobs: torch.Tensor, vllm_logprobs: torch.Tensor, response_mask: torch.Tensor
) -> torch.Tensor:
    """The four statistics of :func:`compute_vllm_local_debug_metrics` as one device vector
    (order of ``VLLM_LOCAL_DEBUG_KEYS``), one launch, no host synchronisation."""
    _lib.require_gpu(local_logprobs, vllm_logprobs, response_mask)
    if local_logprobs.shape != vllm_logprobs.shape or local_logprobs.shape != response_mask.shape:
        raise ValueError("local_logprobs, vllm_logprobs and response_mask must have one shape")
    lo, vl, m = _lib.f32c(local_logprobs.detach()), _lib.f32c(vllm_logprobs.detach()), _lib.mask_u8(response_mask)
    out = torch.empty(len(VLLM_LOCAL_DEBUG_KEYS), dtype=torch.float32, device=lo.device)
    _lib.call("oi_logprob_diff_stats", lo.data_ptr(), vl.data_ptr(), m.data_ptr(), lo.numel(), out.data_ptr(),
              _lib.stream_of(lo))  # fmt: skip
    return out


def compute_vllm_local_debug_metrics(
    local_logprobs: torch.Tensor, vllm_logprobs: torch.Tensor, response_mask: torch.Tensor
) -> dict[str, float]:
    """Mean / max / std of ``|local - vllm|`` and the mean reverse KL over valid response tokens;
    drop-in for open_instruct/grpo_utils.py:345-369 (returns Python floats, i.e. synchronises,
    exactly as the reference does)."""
    values = vllm_local_debug_stats(local_logprobs, vllm_logprobs, response_mask).tolist()
    return dict(zip(VLLM_LOCAL_DEBUG_KEYS, values))


# ----------------------------------------------------------------------------------------------
# model forward -> logprobs
# ----------------------------------------------------------------------------------------------
def forward_for_logprobs(
    model: torch.nn.Module,
    query_responses: torch.Tensor,
    attention_mask: torch.Tensor | None,
    position_ids: torch.Tensor,
    pad_token_id: int,
    temperature: float,
    return_entropy: bool = False,
    pass_olmo_core_doc_lens: bool = False,
    fused_head: bool = False,
    response_mask: torch.Tensor | None = None,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Model forward, then logprob (and entropy) of each next token; open_instruct/grpo_utils.py:541-574.

    Differences from the reference that do not change results: the temperature is applied inside
    the kernel instead of through a scaled copy of the logits, the ``[:, :-1]`` slice is an
    argument of the kernel instead of a view, and entropy comes out of the same pass over the
    logits as the logprob.  With ``pass_olmo_core_doc_lens`` the integer-coded attention mask is
    turned into ``doc_lens`` / ``max_doc_lens`` for models with the olmo-core interface and no
    attention mask is passed, as in the reference.

    ``fused_head=True`` (not in the reference; HuggingFace-style models) runs the model's trunk only
    and sends its final hidden states through the fused lm_head: the ``[B, T, V]`` logits are never
    formed.  With ``response_mask`` (``[B, T]``, the caller's mask before the shift) positions off
    the mask are not multiplied and hold 0; the callers mask them anyway
    (open_instruct/grpo_utils.py:340-344, open_instruct/grpo_fast.py:702-724).
    """
    extra_kwargs = {}
    if pass_olmo_core_doc_lens:
        if attention_mask is None:
            raise AssertionError("pass_olmo_core_doc_lens needs the integer-coded attention mask")
        doc_lens, max_doc_lens = olmo_core_utils.doc_lens_from_attention_mask(attention_mask)
        extra_kwargs = {"doc_lens": doc_lens, "max_doc_lens": max_doc_lens}
        attention_mask = None
    if fused_head:
        from . import lm_head

        trunk, weight = lm_head.split_causal_lm(model)
        out = trunk(input_ids=query_responses, attention_mask=attention_mask, position_ids=position_ids, **extra_kwargs)
        hidden = getattr(out, "last_hidden_state", out[0] if isinstance(out, (tuple, list)) else out)
        labels = query_responses[:, 1:].clone().to(hidden.device)
        labels[labels == pad_token_id] = 0
        keep = None if response_mask is None else response_mask[:, 1:].to(hidden.device) != 0
        return lm_head.fused_lm_head_logprobs(
            hidden[:, :-1], weight, labels, temperature=temperature, mask=keep, return_entropy=return_entropy
        )
    output = model(input_ids=query_responses, attention_mask=attention_mask, position_ids=position_ids, **extra_kwargs)
    logits = getattr(output, "logits", output)
    labels = query_responses[:, 1:].clone().to(logits.device)
    labels[labels == pad_token_id] = 0
    logprob, entropy = model_utils.logprob_and_entropy(
        logits, labels, temperature=temperature, drop_last=True, want_entropy=return_entropy
    )
    return logprob, entropy


def compute_logprobs(
    model: torch.nn.Module,
    data_BT,
    pad_token_id: int,
    temperature: float,
    use_grad: bool = False,
    batch_size: int | None = None,
    pass_olmo_core_doc_lens: bool = False,
) -> list[torch.Tensor]:
    """Masked logprobs of every sample in a collated batch; open_instruct/grpo_utils.py:577-648.

    Samples of one shape are concatenated along the batch dim for a single forward, others are
    run one by one; off-response positions hold ``INVALID_LOGPROB``.
    """
    out: list[torch.Tensor] = []
    n = len(data_BT.query_responses)
    step = 1 if batch_size is None else batch_size
    with torch.enable_grad() if use_grad else torch.no_grad():
        for start in range(0, n, step):
            idx = list(range(start, min(start + step, n)))
            same_shape = len({tuple(data_BT.query_responses[i].shape) for i in idx}) == 1
            groups = [idx] if same_shape else [[i] for i in idx]
            for grp in groups:
                qr = torch.cat([data_BT.query_responses[i] for i in grp], dim=0)
                pos = torch.cat([data_BT.position_ids[i] for i in grp], dim=0)
                att = (
                    torch.cat([data_BT.attention_masks[i] for i in grp], dim=0) if pass_olmo_core_doc_lens else None
                )
                lp, _ = forward_for_logprobs(
                    model, qr, att, pos, pad_token_id, temperature, False,
                    pass_olmo_core_doc_lens=pass_olmo_core_doc_lens,
                )  # fmt: skip
                sizes = [data_BT.query_responses[i].shape[0] for i in grp]
                for i, part in zip(grp, torch.split(lp, sizes, dim=0)):
                    out.append(mask_logprobs(part, data_BT.response_masks[i][:, 1:]))
    return out


def calculate_token_counts(
    accumulation_steps: int, data_BT, device: torch.device, process_group=None
) -> dict[int, float]:
    """Response-token count per accumulation group; open_instruct/grpo_utils.py:651-671.

    The reference all-reduces the counts over the data-parallel group; this build is single-GPU,
    so the sum over ranks is the local value (a ``process_group`` is used when one is initialised).
    """
    counts: dict[int, float] = {}
    local = [mask[:, 1:].sum().float() for mask in data_BT.response_masks]
    if not local:
        return counts
    t = torch.stack(local).to(device)
    if torch.distributed.is_available() and torch.distributed.is_initialized():
        torch.distributed.all_reduce(t, op=torch.distributed.ReduceOp.SUM, group=process_group)
    for i, c in enumerate(t.tolist()):
        key = int((i // accumulation_steps) * accumulation_steps)
        counts[key] = counts.get(key, 0.0) + c
    return counts


# ----------------------------------------------------------------------------------------------
# loss statistics (open_instruct/grpo_utils.py:674-742)
# ----------------------------------------------------------------------------------------------
# the keys the reference's training loops read back (open_instruct/grpo_utils.py:674-689)
_SCALAR_LOSS_STAT_KEYS = [
    "loss/kl_avg",
    "loss/policy_avg",
    "loss/total_avg",
    "objective/kl0_avg",
    "objective/kl1_avg",
    "objective/kl2_avg",
    "objective/kl3_avg",
    "policy/clipfrac_avg",
    "val/ratio",
    "val/rho_clipfrac",
    "val/rho_weight",
    "val/rho_drop_frac",
    "val/rho_drop_low_frac",
    "val/rho_drop_high_frac",
]
_KL_ROWS = [_STAT_ROW[f"objective/kl{j}_avg"] for j in range(4)] + [_STAT_ROW["loss/kl_avg"]]
_RHO_ROWS = [_STAT_ROW[k] for k in _RHO_INDICATOR_KEYS] + [_STAT_ROW["val/rho_weight"]]
_ALWAYS_ROWS = [_STAT_ROW[k] for k in ("loss/policy_avg", "policy/clipfrac_avg", "val/ratio")]


class LossStats(dict):
    """Per-sample loss statistics: the reference's ``dict[key -> tensor[num_samples]]`` whose entries
    are the rows of ONE ``[len(GRPO_STAT_NAMES), num_samples]`` device table (``self.table``), laid
    out like the statistics vector of the kernels.  A sample's column is then filled by the
    kernel itself, and the epoch summary is one reduction over the table."""

    def __init__(self, num_samples: int, device, record_entropy: bool):
        self.table = torch.zeros(len(GRPO_STAT_NAMES), num_samples, dtype=torch.float32, device=device)
        keys = list(_SCALAR_LOSS_STAT_KEYS) + (["policy/entropy_avg"] if record_entropy else [])
        super().__init__((key, self.table[_STAT_ROW[key]]) for key in keys)

    def is_intact(self) -> bool:
        """True while every entry is still the table row it was created as."""
        base = self.table.data_ptr()
        width = self.table.shape[1]
        return all(
            key in _STAT_ROW and t.data_ptr() == base + 4 * width * _STAT_ROW[key] and t.shape == (width,)
            for key, t in self.items()
        )


def create_loss_stats(num_samples: int, device: torch.device, record_entropy: bool = False) -> dict[str, torch.Tensor]:
    """Zeroed per-sample statistics with the keys of open_instruct/grpo_utils.py:692-696."""
    return LossStats(num_samples, device, record_entropy)


_ROW_SELECTORS: dict[tuple, torch.Tensor] = {}


def _row_selector(rows: tuple[int, ...], device) -> torch.Tensor:
    """Index tensor of the table rows to record, made once per combination and device."""
    key = (rows, str(device))
    if key not in _ROW_SELECTORS:
        _ROW_SELECTORS[key] = torch.tensor(rows, dtype=torch.int64, device=device)
    return _ROW_SELECTORS[key]


def _rows_to_record(config, ref_logprobs, entropy, rho_metrics) -> list[int]:
    rows = list(_ALWAYS_ROWS)
    if config.load_ref_policy and ref_logprobs is not None:
        rows += _KL_ROWS
    if rho_metrics is not None:
        rows += [_STAT_ROW[k] for k in rho_metrics if k in _STAT_ROW]
    if entropy is not None:
        rows.append(_STAT_ROW["policy/entropy_avg"])
    return sorted(set(rows))


def populate_sample_loss_stats(
    loss_stats_B: dict[str, torch.Tensor],
    sample_idx: int,
    pg_loss: torch.Tensor | None,
    clipfrac: torch.Tensor | None,
    ratio: torch.Tensor | None,
    loss: torch.Tensor,
    response_mask: torch.Tensor,
    new_logprobs: torch.Tensor,
    ref_logprobs: torch.Tensor | None,
    entropy: torch.Tensor | None,
    config,
    rho_metrics: dict[str, torch.Tensor] | None = None,
    fused_stats: dict | torch.Tensor | None = None,
) -> None:
    """Record the masked means of one sample; same arguments and recorded keys as
    open_instruct/grpo_utils.py:699-729.

    With the per-token tensors (the reference's call) all means come from one pass over them
    (``oi_grpo_stats_from_terms``), written straight into the sample's column when ``loss_stats_B``
    is the table made by :func:`create_loss_stats`.  With ``fused_stats`` (the statistics that
    :func:`grpo_loss_fused` returned for this sample) nothing is recomputed: the entries are
    copied, and ``pg_loss`` / ``clipfrac`` / ``ratio`` may be None.  No host synchronisation either
    way.
    """
    rows = _rows_to_record(config, ref_logprobs, entropy, rho_metrics)
    table = loss_stats_B.table if isinstance(loss_stats_B, LossStats) and loss_stats_B.is_intact() else None
    with torch.no_grad():
        if fused_stats is not None:
            vec = getattr(fused_stats, "vector", fused_stats)
            if isinstance(vec, dict):
                vec = torch.stack([vec[name].float() for name in GRPO_STAT_NAMES])
        else:
            dev = _lib.require_gpu(pg_loss, clipfrac, ratio, response_mask)
            shape = tuple(pg_loss.shape)
            cols = shape[-1] if shape else 1
            n_rows = pg_loss.numel() // max(cols, 1)
            f32 = lambda t, name: None if t is None else _lib.f32c(_expand_to(t.detach(), shape, name))  # noqa: E731
            pg_c, cf_c, rt_c = f32(pg_loss, "pg_loss"), f32(clipfrac, "clipfrac"), f32(ratio, "ratio")
            with_kl = config.load_ref_policy and ref_logprobs is not None
            nl_c = f32(new_logprobs, "new_logprobs") if with_kl else None
            ref_c = f32(ref_logprobs, "ref_logprobs") if with_kl else None
            ent_c = f32(entropy, "entropy")
            m = _lib.mask_u8(_expand_to(response_mask, shape, "response_mask"))
            w_c = f32(rho_metrics.get("val/rho_weight"), "val/rho_weight") if rho_metrics else None
            rho_ptrs, _alive = _rho_indicator_ptrs(rho_metrics, shape)
            write_mask = sum(1 << r for r in rows)
            ws_bytes = _lib.load().oi_grpo_fused_workspace_bytes(n_rows, cols)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            if table is not None:
                out_ptr, out_stride, vec = table.data_ptr() + 4 * sample_idx, table.shape[1], None
            else:
                vec = torch.zeros(len(GRPO_STAT_NAMES), dtype=torch.float32, device=dev)
                out_ptr, out_stride = vec.data_ptr(), 1
            _lib.call(
                "oi_grpo_stats_from_terms", pg_c.data_ptr(), cf_c.data_ptr(), rt_c.data_ptr(), _lib.ptr(nl_c),
                _lib.ptr(ref_c), m.data_ptr(), _lib.ptr(ent_c), _lib.ptr(w_c), *rho_ptrs, n_rows, cols,
                int(config.kl_estimator), float(config.beta), out_ptr, out_stride, write_mask, ws.data_ptr(), ws_bytes,
                _lib.stream_of(pg_c),
            )  # fmt: skip
        if vec is not None:
            if table is not None:
                sel = _row_selector(tuple(rows), table.device)
                table[:, sample_idx].index_copy_(0, sel, vec.to(table.device).index_select(0, sel))
            else:
                for r in rows:
                    name = GRPO_STAT_NAMES[r]
                    if name in loss_stats_B:
                        loss_stats_B[name][sample_idx] = vec[r]
        loss_stats_B["loss/total_avg"][sample_idx] = loss.detach() if torch.is_tensor(loss) else loss


def compute_metrics_from_loss_stats(
    loss_stats_B: dict[str, torch.Tensor], token_counts: torch.Tensor
) -> dict[str, float]:
    """Token-weighted averages over the samples plus the weighted variance of ``val/ratio``;
    open_instruct/grpo_utils.py:732-742.  One reduction over the stacked statistics and one
    device-to-host copy for all keys (the reference reads every key back on its own)."""
    keys = list(loss_stats_B)
    counts = token_counts.to(torch.float32)
    stacked = torch.stack([loss_stats_B[k].to(torch.float32) for k in keys])  # [keys, samples]
    total = counts.sum()
    weights = torch.where(total > 0, counts / total.clamp(min=1e-30), torch.zeros_like(counts))
    means = stacked @ weights
    spread = (weights * (loss_stats_B["val/ratio"].to(torch.float32) - means[keys.index("val/ratio")]) ** 2).sum()
    values = torch.cat([means, spread.reshape(1)]).tolist()
    metrics = dict(zip(keys, values[:-1]))
    metrics["val/ratio_var"] = values[-1]
    return metrics
