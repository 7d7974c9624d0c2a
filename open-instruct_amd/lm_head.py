"""Fused lm_head projection + per-token logprob / entropy (no ``[tokens, vocab]`` logits tensor).

There is no single counterpart in the reference: this replaces the pair "lm_head GEMM, then
``calculate_per_token_logps`` / ``log_softmax_and_gather`` (+ ``entropy_from_logits``)" at
open_instruct/olmo_core_train_modules.py:71-76 and open_instruct/grpo_utils.py:558-572.

``fused_linear_cross_entropy`` is the supervised fine-tuning loss through the same kernels: the
causal-LM cross-entropy that the reference obtains from the model's own forward
(open_instruct/finetune.py:818-824) or from a fused linear + cross-entropy implementation
(open_instruct/finetune.py:571-586, ``loss_implementation`` at open_instruct/olmo_core_utils.py:64-66).
"""

from __future__ import annotations

import torch

from . import _lib


class _FusedLMHead(torch.autograd.Function):
    @staticmethod
    def forward(ctx, hidden, weight, labels, mask, inv_temperature, want_entropy, compact_backward=False,
                dhidden_in_forward="auto"):
        dev = _lib.require_gpu(hidden, weight, labels, mask)
        if hidden.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
            raise ValueError("fused lm_head expects bf16 hidden states and weight")
        if hidden.ndim != 2 or weight.ndim != 2 or hidden.shape[1] != weight.shape[1]:
            raise ValueError(f"shape mismatch: hidden {tuple(hidden.shape)} weight {tuple(weight.shape)}")
        n, h = hidden.shape
        v = weight.shape[0]
        if h % 64:
            raise ValueError("hidden size must be a multiple of 64")
        hid, w = hidden.contiguous(), weight.contiguous()
        lab = labels.reshape(-1).to(torch.int64).contiguous()
        if lab.numel() != n:
            raise ValueError(f"{lab.numel()} labels for {n} hidden rows")
        m = None
        if mask is not None:
            m = _lib.mask_u8(mask.reshape(-1))
            if m.numel() != n:
                raise ValueError(f"mask of {m.numel()} entries for {n} hidden rows")
        logprob = torch.empty(n, dtype=torch.float32, device=dev)
        entropy = torch.empty(n, dtype=torch.float32, device=dev) if want_entropy else None
        lse = torch.empty(n, dtype=torch.float32, device=dev)
        # a backward pass that only needs d_hidden is prepared while the logits exist (no recomputation)
        if dhidden_in_forward == "auto":
            dhidden_in_forward = not compact_backward
        wsum_mode = bool(dhidden_in_forward) and ctx.needs_input_grad[0] and not ctx.needs_input_grad[1] and n > 0
        if wsum_mode and compact_backward:
            raise ValueError("dhidden_in_forward cannot be combined with compact_backward")
        wsum = xref = unsafe = None
        if wsum_mode:
            lib = _lib.load()
            wsum = torch.empty(n, h, dtype=torch.float32, device=dev)
            xref = torch.empty(n, dtype=torch.float32, device=dev)
            unsafe = torch.empty(n, dtype=torch.uint8, device=dev)
            ws_bytes = lib.oi_lmhead_fwd_wsum_workspace_bytes(n, h, v, int(m is not None))
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            _lib.call(
                "oi_lmhead_logp_fwd_wsum", hid.data_ptr(), w.data_ptr(), lab.data_ptr(), _lib.ptr(m), n, h, v,
                inv_temperature, logprob.data_ptr(), _lib.ptr(entropy), lse.data_ptr(), wsum.data_ptr(),
                xref.data_ptr(), unsafe.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_of(hid),
            )  # fmt: skip
        elif n > 0:
            lib = _lib.load()
            ws_bytes = lib.oi_lmhead_fwd_workspace_bytes(n, h, v, int(m is not None))
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            _lib.call(
                "oi_lmhead_logp_fwd", hid.data_ptr(), w.data_ptr(), lab.data_ptr(), _lib.ptr(m), n, h, v,
                inv_temperature, logprob.data_ptr(), _lib.ptr(entropy), lse.data_ptr(), ws.data_ptr(), ws_bytes,
                _lib.stream_of(hid),
            )  # fmt: skip
        ctx.save_for_backward(hid, w, lab, lse, m, logprob, wsum, xref, unsafe)
        ctx.inv_temperature = inv_temperature
        ctx.compact_backward = bool(compact_backward)
        if want_entropy:
            ctx.mark_non_differentiable(entropy)
        return logprob, entropy

    @staticmethod
    def backward(ctx, grad_logprob, _grad_entropy):
        hid, w, lab, lse, m, logprob, wsum, xref, unsafe = ctx.saved_tensors
        n, h = hid.shape
        v = w.shape[0]
        need_h, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if grad_logprob is None or not (need_h or need_w):
            return (None,) * 8
        g = _lib.f32c(grad_logprob)
        d_hidden = torch.empty_like(hid)
        if wsum is not None:
            ws_bytes = _lib.load().oi_lmhead_dh_workspace_bytes(n, h, v)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=hid.device)
            _lib.call(
                "oi_lmhead_dh_from_wsum", hid.data_ptr(), w.data_ptr(), lab.data_ptr(), lse.data_ptr(),
                logprob.data_ptr(), g.data_ptr(), _lib.ptr(m), wsum.data_ptr(), xref.data_ptr(), unsafe.data_ptr(), n, h,
                v, ctx.inv_temperature, d_hidden.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_of(hid),
            )  # fmt: skip
            return (d_hidden,) + (None,) * 7
        d_weight = torch.empty_like(w) if need_w else None
        if n > 0:
            selecting = m is not None or ctx.compact_backward
            ws_bytes = _lib.load().oi_lmhead_bwd_workspace_bytes(n, h, v, int(need_w), int(selecting))
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=hid.device)
            _lib.call(
                "oi_lmhead_logp_bwd", hid.data_ptr(), w.data_ptr(), lab.data_ptr(), lse.data_ptr(), g.data_ptr(),
                _lib.ptr(m), int(ctx.compact_backward), n, h, v, ctx.inv_temperature, _lib.ptr(logprob),
                d_hidden.data_ptr(), _lib.ptr(d_weight), ws.data_ptr(), ws_bytes, _lib.stream_of(hid),
            )  # fmt: skip
        elif d_weight is not None:
            d_weight.zero_()
        return (d_hidden if need_h else None), d_weight, None, None, None, None, None, None


def fused_lm_head_logprobs(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor,
    temperature: float = 1.0,
    mask: torch.Tensor | None = None,
    return_entropy: bool = False,
    compact_backward: bool = False,
    dhidden_in_forward: bool | str = "auto",
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """``log_softmax(hidden @ weight.T / temperature)[labels]`` (+ entropy) per token, fp32.

    ``hidden`` is ``[N, H]`` bf16 (or any leading shape ``[..., H]``), ``weight`` ``[V, H]`` bf16,
    ``labels`` int64 with the leading shape of ``hidden``; negative labels are scored as token 0
    (the reference's ``clamp(min=0)``, open_instruct/padding_free_collator.py:15).  ``mask`` (bool,
    same leading shape) selects the rows that are computed at all: masked-out rows cost nothing,
    return 0 and receive a zero gradient.  The selection is made on the device (a row index built
    from the mask, the selected rows gathered into the workspace), so neither pass waits for the
    GPU.  Differentiable with respect to ``hidden`` and ``weight``; the entropy carries no
    gradient, as in the reference.  ``compact_backward=True`` additionally leaves rows whose
    upstream gradient is exactly zero (zero-advantage completions, clipped ratios without a KL
    term) out of the backward products; it changes no result.

    Nothing of size ``[tokens, vocab]`` ever exists.  When ``weight`` takes a gradient the backward
    recomputes the logits one vocabulary chunk at a time (for a step without that recomputation see
    :func:`open_instruct_amd.grpo_utils.grpo_loss_on_hidden` and
    :func:`open_instruct_amd.dpo_utils.dpo_loss_on_hidden`, which know the loss and can therefore
    finish a slab of tokens before they start the next).

    ``dhidden_in_forward`` (default ``"auto"``: on whenever ``hidden`` takes a gradient and ``weight``
    does not, e.g. a frozen lm_head) lets the forward also accumulate, per token, the
    softmax-weighted sum of the weight rows, which is all the backward to ``hidden`` needs besides
    the upstream gradient: the backward is then one pass over ``[tokens, hidden]`` and the logits
    are never recomputed (4·N·H·V matrix work for both passes instead of 6·N·H·V).  It holds an
    fp32 ``[tokens, hidden]`` tensor between the passes.  The exponentials behind that sum are kept
    relative to each token's own label logit, so the route has no limit on the size of the logits or
    on the temperature; a token whose label is extremely unlikely (its largest logit more than 44
    nats above the label's) or whose logits hold a NaN is flagged on the device and recomputed in the
    backward pass like a row of the recomputing route, with the same results.
    """
    lead = hidden.shape[:-1]
    hid2 = hidden.reshape(-1, hidden.shape[-1])
    lab1 = labels.reshape(-1)
    inv_t = 1.0 / float(temperature)
    if not float(temperature) > 0.0:
        raise ValueError(f"temperature must be positive, got {temperature}")
    if mask is not None and tuple(mask.shape) != tuple(lead):
        raise ValueError(f"mask {tuple(mask.shape)} does not match the rows of hidden {tuple(lead)}")
    if dhidden_in_forward == "auto":
        dhidden_in_forward = not compact_backward
    # without a backward pass to come (torch.no_grad(): scoring passes, the reference-logprob cache) there is
    # nothing to prepare; inside an autograd Function the grad mode is off, so it is read here
    dhidden_in_forward = bool(dhidden_in_forward) and torch.is_grad_enabled()
    lp, ent = _FusedLMHead.apply(hid2, weight, lab1, mask, inv_t, return_entropy, compact_backward, dhidden_in_forward)
    return lp.reshape(lead), (ent.reshape(lead) if ent is not None else None)


def fused_linear_cross_entropy(
    hidden: torch.Tensor,
    weight: torch.Tensor,
    labels: torch.Tensor | None = None,
    *,
    shift_labels: torch.Tensor | None = None,
    num_items_in_batch: torch.Tensor | int | float | None = None,
    ignore_index: int = -100,
    token_slabs: bool | int = False,
) -> torch.Tensor:
    """Causal-LM cross-entropy of ``hidden @ weight.T`` against next-token labels, scalar fp32.

    ``labels`` ``[B, T]`` are shifted here (position ``t`` is scored against ``labels[:, t + 1]``,
    the last position is ignored); pass ``shift_labels`` instead when the caller has already
    shifted them (sequence-parallel batches, open_instruct/finetune.py:826-829).  Positions whose
    label equals ``ignore_index`` are never multiplied.  The result is the mean over kept tokens,
    or ``sum / num_items_in_batch`` when that count is given (gradient accumulation over several
    micro-batches).  Differentiable with respect to ``hidden`` and ``weight``.

    ``token_slabs`` (``True`` = the default slab size, or a number of tokens) computes the loss and
    both gradients in one call with nothing recomputed: every token's upstream gradient is the known
    constant ``-1 / count``, so the step can run slab by slab like
    :func:`open_instruct_amd.grpo_utils.grpo_loss_on_hidden` (whose ``loss_fn="cispo"`` term with
    unit advantages, ratio 1 and no KL term *is* the negative log-likelihood); the gradients are
    handed out by ``loss.backward()``.  Needs a 2-D ``[B, T]`` batch.
    """
    if (labels is None) == (shift_labels is None):
        raise ValueError("pass exactly one of labels / shift_labels")
    if shift_labels is None:
        shift_labels = torch.full_like(labels, ignore_index)
        shift_labels[..., :-1] = labels[..., 1:]
    if shift_labels.shape != hidden.shape[:-1]:
        raise ValueError(f"labels {tuple(shift_labels.shape)} do not match hidden {tuple(hidden.shape)}")
    keep = shift_labels != ignore_index
    if token_slabs:
        import types

        from . import grpo_utils

        if shift_labels.ndim != 2:
            raise ValueError("token_slabs needs [B, T] labels")
        # masked_mean(-logprob, keep, denominator): the CISPO term with advantage 1, ratio 1, beta 0
        nll = types.SimpleNamespace(loss_fn="cispo", clip_lower=0.0, clip_higher=0.0, beta=0.0, kl_estimator=2)
        denominator = None
        if num_items_in_batch is not None:
            denominator = float(num_items_in_batch)  # a device tensor is read here: the C entry takes a number
        loss, _, _, _ = grpo_utils.grpo_loss_on_hidden(
            hidden, weight, shift_labels, None, None, torch.ones((), device=hidden.device), keep, nll,
            loss_denominator=denominator, token_slabs=token_slabs,
        )  # fmt: skip
        return loss
    logps, _ = fused_lm_head_logprobs(hidden, weight, shift_labels, mask=keep)
    total = -logps.sum()
    if num_items_in_batch is None:
        return total / keep.sum().clamp(min=1)
    if torch.is_tensor(num_items_in_batch):
        num_items_in_batch = num_items_in_batch.to(total.device)
    return total / num_items_in_batch


def split_causal_lm(model) -> tuple[torch.nn.Module, torch.Tensor]:
    """``(trunk, lm_head weight)`` of a HuggingFace-style causal LM: the module that returns
    ``last_hidden_state`` and the ``[V, H]`` matrix its logits are projected with (the pieces the
    reference reaches through ``model(...)`` at open_instruct/grpo_utils.py:558-559 and
    open_instruct/dpo_utils.py:859-863).  Raises ``TypeError`` when the model does not expose them
    or projects with a bias."""
    head = model.get_output_embeddings() if hasattr(model, "get_output_embeddings") else getattr(model, "lm_head", None)
    trunk = getattr(model, "base_model", None)
    if trunk is None or trunk is model:
        trunk = getattr(model, "model", None)
    if head is None or trunk is None or not hasattr(head, "weight"):
        raise TypeError("fused_head needs a causal LM with a trunk (base_model / model) and an output embedding")
    if getattr(head, "bias", None) is not None:
        raise TypeError("fused_head needs a bias-free lm_head")
    return trunk, head.weight


def per_token_logps_from_trunk(model, labels: torch.Tensor, ignore_index: int = -100, **inputs) -> torch.Tensor:
    """``calculate_per_token_logps(model(**inputs).logits, labels)``
    (open_instruct/padding_free_collator.py:10-16) without the logits: the trunk's final hidden
    states go through the fused head.  Positions whose next label is ``ignore_index`` are not
    multiplied and hold 0 (the per-sequence sums mask them anyway)."""
    trunk, weight = split_causal_lm(model)
    out = trunk(**inputs)
    hidden = getattr(out, "last_hidden_state", out[0] if isinstance(out, (tuple, list)) else out)
    shifted = torch.full_like(labels, ignore_index)
    shifted[..., :-1] = labels[..., 1:]
    logps, _ = fused_lm_head_logprobs(hidden, weight, shifted, mask=shifted != ignore_index)
    return logps
