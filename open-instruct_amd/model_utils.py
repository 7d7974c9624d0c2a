"""Per-token log-probability, entropy and KL estimators on the GPU.

Same names and call signatures as open_instruct/model_utils.py in the reference
(``log_softmax_and_gather`` :587-600, ``entropy_from_logits`` :326-333, ``estimate_kl`` :793-818);
the arithmetic runs in hand-written HIP kernels reached through the C-ABI.

Numerics: everything is accumulated in fp32.  For fp32 logits the result is fp32 like the
reference's; for bf16 / fp16 logits the result is fp32 by default (the reference would round it
to the logits' dtype) - pass ``out_dtype=logits.dtype`` to get the reference's dtype back.
"""

from __future__ import annotations

import os
import pathlib

import torch

from . import _lib


class TensorCache:
    """Device-resident tables with one row per dataset sample (the reference-logprob cache of DPO).

    Same constructor, attribute and methods as open_instruct/model_utils.py:92-115:
    ``TensorCache(tensors={...})``, ``cache[indices]`` gathers the rows of every table, ``to_disk`` /
    ``from_disk`` move the whole cache through one ``torch.save`` file (readable by the reference).
    """

    def __init__(self, tensors: dict[str, torch.Tensor]):
        self.tensors = dict(tensors)

    def __getitem__(self, indices: torch.Tensor) -> dict[str, torch.Tensor]:
        out = {}
        for name, table in self.tensors.items():
            idx = indices.to(device=table.device, dtype=torch.int64)
            out[name] = table.index_select(0, idx.reshape(-1)).reshape(idx.shape + table.shape[1:])
        return out

    def __eq__(self, other) -> bool:
        return isinstance(other, TensorCache) and self.tensors.keys() == other.tensors.keys() and all(
            torch.equal(v, other.tensors[k]) for k, v in self.tensors.items()
        )

    def to_disk(self, path: str | pathlib.Path) -> None:
        """The file appears under its final name only when it is complete (written next to it under
        a process-private name, then moved over)."""
        target = pathlib.Path(path)
        target.parent.mkdir(parents=True, exist_ok=True)
        partial = target.with_name(f".{target.name}.{os.getpid()}.partial")
        torch.save({name: table.detach().to("cpu") for name, table in self.tensors.items()}, partial)
        os.replace(partial, target)

    @classmethod
    def from_disk(cls, path: str | pathlib.Path, device: torch.device) -> "TensorCache":
        """Tensors only: the file is read with ``weights_only=True``."""
        return cls(tensors=torch.load(pathlib.Path(path), weights_only=True, map_location=device))


def _row_layout(logits: torch.Tensor) -> tuple[torch.Tensor, int, int, int, int]:
    """Describe ``logits[..., V]`` as (tensor, n_outer, n_inner, stride_outer, stride_inner).

    The kernels address rows through two strides, which covers contiguous tensors and the
    reference's ``logits[:, :-1]`` view without a copy.  Anything more exotic is made contiguous.
    """
    if logits.ndim < 1:
        raise ValueError("logits needs at least one dimension")
    if logits.stride(-1) != 1 and logits.shape[-1] > 1:
        logits = logits.contiguous()
    if any(st < logits.shape[-1] and n > 1 for st, n in zip(logits.stride()[:-1], logits.shape[:-1])):
        logits = logits.contiguous()  # overlapping rows (expanded / transposed views)
    lead = logits.shape[:-1]
    if len(lead) == 0:
        return logits, 1, 1, 0, 0
    if len(lead) == 1:
        return logits, 1, lead[0], 0, logits.stride(0)
    # collapse all leading dims but the last into one outer dim when their strides allow it
    inner, s_inner = lead[-1], logits.stride(-2)
    outer_shape, outer_strides = lead[:-1], logits.stride()[: len(lead) - 1]
    n_outer = 1
    for d in outer_shape:
        n_outer *= d
    collapsible = True
    for k in range(len(outer_shape) - 1):
        if outer_shape[k] != 1 and outer_strides[k] != outer_strides[k + 1] * outer_shape[k + 1]:
            collapsible = False
    if not collapsible:
        logits = logits.contiguous()
        return logits, n_outer, inner, inner * logits.shape[-1], logits.shape[-1]
    return logits, n_outer, inner, outer_strides[-1] if n_outer > 1 else 0, s_inner


class _LogSoftmaxGather(torch.autograd.Function):
    """logprob (+ optional entropy) of the selected token; backward writes dlogits in one pass."""

    @staticmethod
    def forward(ctx, logits, index, inv_temperature, want_entropy, drop_last):
        dev = _lib.require_gpu(logits, index)
        if logits.dtype not in _lib.DTYPE_TAGS:
            raise ValueError(f"unsupported logits dtype {logits.dtype}")
        if index.dtype != torch.int64:
            index = index.long()
        view = logits[..., :-1, :] if drop_last else logits
        if tuple(index.shape) != tuple(view.shape[:-1]):
            raise ValueError(f"index shape {tuple(index.shape)} does not match logits rows {tuple(view.shape[:-1])}")
        view, n_outer, n_inner, so, si = _row_layout(view)
        index = index.contiguous()
        vocab = view.shape[-1]
        rows = n_outer * n_inner
        logprob = torch.empty(index.shape, dtype=torch.float32, device=dev)
        entropy = torch.empty(index.shape, dtype=torch.float32, device=dev) if want_entropy else None
        lse = torch.empty(index.shape, dtype=torch.float32, device=dev)
        if rows > 0:
            _lib.call(
                "oi_lsg_entropy_fwd", view.data_ptr(), _lib.DTYPE_TAGS[view.dtype], n_outer, n_inner, so, si, vocab,
                index.data_ptr(), inv_temperature, logprob.data_ptr(), _lib.ptr(entropy), lse.data_ptr(),
                _lib.stream_of(view),
            )  # fmt: skip
        ctx.save_for_backward(logits, index, lse)
        ctx.inv_temperature = inv_temperature
        ctx.drop_last = drop_last
        if want_entropy:
            ctx.mark_non_differentiable(entropy)
            return logprob, entropy
        return logprob, None

    @staticmethod
    def backward(ctx, grad_logprob, _grad_entropy):
        logits, index, lse = ctx.saved_tensors
        if grad_logprob is None:
            return None, None, None, None, None
        grad = _lib.f32c(grad_logprob)
        dlogits = torch.empty(logits.shape, dtype=logits.dtype, device=logits.device)
        view = logits[..., :-1, :] if ctx.drop_last else logits
        out_view = dlogits[..., :-1, :] if ctx.drop_last else dlogits
        if ctx.drop_last:
            dlogits[..., -1, :].zero_()
        # (n_outer, n_inner) depend on the shape only, so the input and output descriptions agree
        view, n_outer, n_inner, so, si = _row_layout(view)
        _, _, _, oso, osi = _row_layout(out_view)
        if n_outer * n_inner > 0:
            _lib.call(
                "oi_lsg_bwd", view.data_ptr(), _lib.DTYPE_TAGS[view.dtype], n_outer, n_inner, so, si, view.shape[-1],
                index.data_ptr(), lse.data_ptr(), grad.data_ptr(), ctx.inv_temperature, out_view.data_ptr(), oso, osi,
                _lib.stream_of(view),
            )  # fmt: skip
        return dlogits, None, None, None, None


def _inv_temperature(temperature: float) -> float:
    t = float(temperature)
    if not t > 0.0:
        raise ValueError(f"temperature must be positive, got {temperature}")
    return 1.0 / t


def log_softmax_and_gather(
    logits: torch.Tensor,
    index: torch.Tensor,
    *,
    temperature: float = 1.0,
    out_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    """``log_softmax(logits / temperature, -1)`` gathered at ``index`` without a ``[..., V]`` temporary.

    Drop-in for open_instruct/model_utils.py:587-600.  ``logits`` may be a non-contiguous view such
    as ``logits_full[:, :-1]``.  Differentiable with respect to ``logits``.
    """
    out, _ = _LogSoftmaxGather.apply(logits, index, _inv_temperature(temperature), False, False)
    return out if out_dtype is None else out.to(out_dtype)


def entropy_from_logits(
    logits: torch.Tensor, *, temperature: float = 1.0, out_dtype: torch.dtype | None = None
) -> torch.Tensor:
    """Entropy of ``softmax(logits / temperature)`` per row; drop-in for open_instruct/model_utils.py:326-333.

    The reference only calls it under ``torch.no_grad()`` (open_instruct/grpo_utils.py:569-572); the
    result carries no gradient here either.
    """
    with torch.no_grad():
        index = torch.zeros(logits.shape[:-1], dtype=torch.int64, device=logits.device)
        _, ent = _LogSoftmaxGather.apply(logits.detach(), index, _inv_temperature(temperature), True, False)
    return ent if out_dtype is None else ent.to(out_dtype)


def logprob_and_entropy(
    logits: torch.Tensor,
    index: torch.Tensor,
    *,
    temperature: float = 1.0,
    drop_last: bool = False,
    want_entropy: bool = True,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """Both results from ONE pass over the logits (the reference makes two separate calls).

    With ``drop_last=True`` the last position along dim -2 is skipped and ``index`` has one
    position fewer; the gradient then comes back for the full ``logits`` tensor with a zero last
    position, which saves autograd's extra copy through the ``[:, :-1]`` slice.
    """
    return _LogSoftmaxGather.apply(logits, index, _inv_temperature(temperature), want_entropy, drop_last)


class _EstimateKL(torch.autograd.Function):
    @staticmethod
    def forward(ctx, diff, ratio):
        dev = _lib.require_gpu(diff, ratio)
        d, r = _lib.f32c(diff), _lib.f32c(ratio.expand_as(diff))
        out = torch.empty((4,) + tuple(d.shape), dtype=torch.float32, device=dev)
        _lib.call("oi_estimate_kl_fwd", d.data_ptr(), r.data_ptr(), d.numel(), out.data_ptr(), _lib.stream_of(d))
        ctx.save_for_backward(d, r)
        ctx.in_dtypes = (diff.dtype, ratio.dtype)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        d, r = ctx.saved_tensors
        g = _lib.f32c(grad_out)
        dd = torch.empty_like(d) if ctx.needs_input_grad[0] else None
        dr = torch.empty_like(r) if ctx.needs_input_grad[1] else None
        _lib.call(
            "oi_estimate_kl_bwd", d.data_ptr(), r.data_ptr(), g.data_ptr(), d.numel(), _lib.ptr(dd), _lib.ptr(dr),
            _lib.stream_of(d),
        )  # fmt: skip
        if dd is not None:
            dd = dd.to(ctx.in_dtypes[0])
        if dr is not None:
            dr = dr.to(ctx.in_dtypes[1])
        return dd, dr


def estimate_kl(ref_logprobs_diff: torch.Tensor, ratio: torch.Tensor) -> torch.Tensor:
    """Four KL estimators stacked on a new leading dim; drop-in for open_instruct/model_utils.py:793-818."""
    return _EstimateKL.apply(ref_logprobs_diff, ratio)
