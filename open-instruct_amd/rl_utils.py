"""Masked mean on the GPU; same name and signature as open_instruct/rl_utils.py:426-448."""

from __future__ import annotations

import torch

from . import _lib


def _as_rows(values: torch.Tensor, mask: torch.Tensor, axis: int | None):
    """Reshape to values [extra, rows, cols] / mask [rows, cols] for the two reduction modes.

    axis=None: one row holding every mask element.  axis=k: the reduced mask dim becomes the
    column dim (moved last when it is not already), every other mask dim is a row.
    """
    extra_dims = values.ndim - mask.ndim
    if extra_dims < 0:
        raise ValueError(f"values {tuple(values.shape)} has fewer dims than mask {tuple(mask.shape)}")
    if tuple(values.shape[extra_dims:]) != tuple(mask.shape):
        try:  # the reference relies on broadcasting; make it explicit
            mask = mask.expand(values.shape[extra_dims:])
        except RuntimeError:
            raise ValueError(f"mask shape {tuple(mask.shape)} does not match values {tuple(values.shape)}") from None
    extra = 1
    for d in values.shape[:extra_dims]:
        extra *= d
    if axis is None:
        cols = mask.numel()
        return values.reshape(extra, 1, cols), mask.reshape(1, cols), extra_dims, 0
    ax = axis if axis >= 0 else axis + mask.ndim
    if not 0 <= ax < mask.ndim:
        raise IndexError(f"axis {axis} out of range for a mask with {mask.ndim} dims")
    if ax != mask.ndim - 1:
        mask = mask.movedim(ax, -1)
        values = values.movedim(extra_dims + ax, -1)
    cols = mask.shape[-1]
    rows = mask.numel() // max(cols, 1)
    return values.reshape(extra, rows, cols), mask.reshape(rows, cols), extra_dims, 1


class _MaskedMean(torch.autograd.Function):
    @staticmethod
    def forward(ctx, values3, mask2, axis_mode, denominator):
        dev = _lib.require_gpu(values3, mask2)
        v = _lib.f32c(values3)
        is_float = mask2.dtype.is_floating_point
        m = _lib.f32c(mask2) if is_float else _lib.mask_u8(mask2)
        extra, rows, cols = v.shape
        out = torch.empty(extra, dtype=torch.float32, device=dev)
        row_denoms = torch.empty(rows, dtype=torch.float32, device=dev)
        ws_bytes = _lib.load().oi_masked_mean_workspace_bytes(extra, rows, cols)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        _lib.call(
            "oi_masked_mean_fwd", v.data_ptr(), m.data_ptr(), int(is_float), extra, rows, cols, axis_mode,
            float(denominator), out.data_ptr(), row_denoms.data_ptr(), ws.data_ptr(), ws_bytes, _lib.stream_of(v),
        )  # fmt: skip
        ctx.save_for_backward(m, row_denoms)
        ctx.is_float = is_float
        ctx.shape = (extra, rows, cols)
        ctx.in_dtype = values3.dtype
        return out

    @staticmethod
    def backward(ctx, grad_out):
        m, row_denoms = ctx.saved_tensors
        extra, rows, cols = ctx.shape
        g = _lib.f32c(grad_out)
        dv = torch.empty(ctx.shape, dtype=torch.float32, device=g.device)
        _lib.call(
            "oi_masked_mean_bwd", g.data_ptr(), m.data_ptr(), int(ctx.is_float), row_denoms.data_ptr(), extra, rows,
            cols, dv.data_ptr(), _lib.stream_of(g),
        )  # fmt: skip
        return dv.to(ctx.in_dtype), None, None, None


def masked_mean(
    values: torch.Tensor, mask: torch.Tensor, axis: int | None = None, denominator: float | None = None
) -> torch.Tensor:
    """Mean of ``values`` over the positions selected by ``mask``.

    Drop-in for open_instruct/rl_utils.py:426-448: extra leading dims of ``values`` are kept;
    ``axis=None`` divides the masked sum by ``mask.sum()`` (or ``denominator``); ``axis=k`` takes
    per-slice means along mask dim ``k`` and averages them; an empty mask gives 0.
    """
    if denominator is not None and not isinstance(denominator, (int, float)):
        denominator = float(denominator)
    if values.numel() == 0 or mask.numel() == 0:
        raise ValueError("masked_mean needs non-empty tensors")
    v3, m2, extra_dims, axis_mode = _as_rows(values, mask, axis)
    if denominator is not None and denominator <= 0:
        # the reference returns zeros for a non-positive constant denominator
        return (v3.sum(dim=(1, 2)) * 0.0).reshape(values.shape[:extra_dims])
    out = _MaskedMean.apply(v3, m2, axis_mode, 0.0 if denominator is None else float(denominator))
    return out.reshape(values.shape[:extra_dims])
