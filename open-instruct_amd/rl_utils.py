"""Masked mean and sequence packing on the GPU; same names and signatures as
open_instruct/rl_utils.py (``masked_mean`` :426-448, ``pack_sequences`` :227-375,
``PackedSequences`` :181-213)."""

from __future__ import annotations

import itertools
from dataclasses import dataclass

import numpy as np
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


# ----------------------------------------------------------------------------------------------
# sequence packing
# ----------------------------------------------------------------------------------------------
@dataclass
class PackedSequences:
    """Same fields as open_instruct/rl_utils.py:181-213; every tensor lives on the GPU and the
    per-row tensors of one field are views into one flat buffer (rows back to back)."""

    query_responses: list[torch.Tensor]
    attention_masks: list[torch.Tensor]
    response_masks: list[torch.Tensor]
    original_responses: list[list[int]]
    advantages: list[torch.Tensor] | None = None
    num_actions: list[torch.Tensor] | None = None
    position_ids: list[torch.Tensor] | None = None
    packed_seq_lens: list[torch.Tensor] | None = None
    vllm_logprobs: list[torch.Tensor] | None = None
    dones: list[torch.Tensor] | None = None
    rewards: list[torch.Tensor] | None = None


def _csr(seqs: list, dtype) -> tuple[np.ndarray, np.ndarray]:
    lens = np.fromiter((len(x) for x in seqs), dtype=np.int64, count=len(seqs))
    offsets = np.zeros(len(seqs) + 1, dtype=np.int64)
    np.cumsum(lens, out=offsets[1:])
    flat = np.fromiter(itertools.chain.from_iterable(seqs), dtype=dtype, count=int(offsets[-1]))
    return flat, offsets


def pack_sequences(
    queries: list[list[int]],
    responses: list[list[int]],
    masks: list[list[int]],
    pack_length: int,
    pad_token_id: int,
    vllm_logprobs: list[list[float]],
    min_num_batches: int = 1,
    mask_tool_use: bool = False,
    advantages=None,
    device: torch.device | str = "cuda",
) -> PackedSequences:
    """Pack query-response pairs into rows of at most ``pack_length`` tokens.

    Drop-in for open_instruct/rl_utils.py:227-375 (same greedy rule: a sequence that does not fit
    the current row starts a new one; ``min_num_batches`` shrinks the row length to
    ``total_tokens // min_num_batches``).  The ragged lists are flattened once on the host; the
    seven per-token outputs are written by one kernel launch and returned as GPU tensors.
    ``advantages`` (one value per sequence, optional) fills ``PackedSequences.advantages`` with
    the broadcast of open_instruct/data_loader.py:1509-1514 in the same launch; response masks
    keep the reference's int64 document ids (``.bool()`` them after use, as the reference does).
    """
    n = len(queries)
    if not (len(responses) == len(masks) == len(vllm_logprobs) == n):
        raise ValueError("queries, responses, masks and vllm_logprobs must have one length")
    assert not any(pad_token_id in query for query in queries)
    for i in range(n):
        assert len(vllm_logprobs[i]) == len(responses[i]), (
            f"Response {i}: logprobs length ({len(vllm_logprobs[i])}) != response length ({len(responses[i])})"
        )
        if len(masks[i]) != len(responses[i]):
            raise ValueError(f"Response {i}: mask length ({len(masks[i])}) != response length ({len(responses[i])})")
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("pack_sequences writes its outputs on an AMD GPU; there is no CPU implementation")
    q_flat, q_off = _csr(queries, np.int64)
    r_flat, r_off = _csr(responses, np.int64)
    m_flat = _csr(masks, np.int64)[0] if mask_tool_use else None  # only read when tool tokens are masked out
    lp_flat, _ = _csr(vllm_logprobs, np.float32)
    kept = r_flat != pad_token_id
    kept_before = np.zeros(len(r_flat) + 1, dtype=np.int64)
    np.cumsum(kept, out=kept_before[1:])
    r_len = kept_before[r_off[1:]] - kept_before[r_off[:-1]]
    seq_len = (q_off[1:] - q_off[:-1]) + r_len
    if n and int(seq_len.min()) < 1:
        raise ValueError("every sequence needs at least one token")
    total_tokens = int(seq_len.sum())
    if total_tokens > 0 and min_num_batches > 1:
        effective = min(total_tokens // min_num_batches, pack_length)
    else:
        effective = pack_length
    # greedy row assignment: O(n) scalar work
    row_first = [0] if n else []  # index of the first sequence of each row
    mask_base = np.zeros(n, dtype=np.int32)
    cur = 0
    for i, length in enumerate(seq_len.tolist()):
        if length + cur > effective and cur > 0:
            row_first.append(i)
            cur = 0
        mask_base[i] = row_first[-1]
        cur += length
    dst = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(seq_len, out=dst[1:])

    def up(a):
        return torch.from_numpy(np.ascontiguousarray(a)).to(dev)

    out_i64 = torch.empty(5, max(total_tokens, 1), dtype=torch.int64, device=dev)
    out_f32 = torch.empty(2, max(total_tokens, 1), dtype=torch.float32, device=dev)
    adv_dev = None
    if advantages is not None:
        adv_np = np.asarray(advantages, dtype=np.float32).reshape(-1)
        if adv_np.shape[0] != n:
            raise ValueError(f"advantages has {adv_np.shape[0]} entries for {n} sequences")
        adv_dev = up(adv_np)
    lens_dev = up(np.stack([r_len, seq_len])) if n else torch.zeros(2, 0, dtype=torch.int64, device=dev)
    if n:
        tool = up(m_flat != 0).view(torch.uint8) if mask_tool_use else None
        ins = [up(q_flat), up(q_off), up(r_flat), up(r_off), tool, up(lp_flat), up(dst[:-1]), up(mask_base)]
        _lib.call(
            "oi_pack_sequences", ins[0].data_ptr(), ins[1].data_ptr(), ins[2].data_ptr(), ins[3].data_ptr(),
            _lib.ptr(ins[4]), ins[5].data_ptr(), _lib.ptr(adv_dev), ins[6].data_ptr(), ins[7].data_ptr(), n,
            int(pad_token_id), int(bool(mask_tool_use)), out_i64[0].data_ptr(), out_i64[1].data_ptr(),
            out_i64[2].data_ptr(), out_i64[3].data_ptr(), out_i64[4].data_ptr(), out_f32[0].data_ptr(),
            out_f32[1].data_ptr() if adv_dev is not None else None, torch.cuda.current_stream(dev).cuda_stream,
        )  # fmt: skip
    bounds = [int(dst[i]) for i in row_first] + [total_tokens]
    seq_bounds = row_first + [n]

    def rows(flat):
        return [flat[bounds[k] : bounds[k + 1]] for k in range(len(row_first))]

    def seq_rows(flat):
        return [flat[seq_bounds[k] : seq_bounds[k + 1]] for k in range(len(row_first))]

    return PackedSequences(
        query_responses=rows(out_i64[0]),
        attention_masks=rows(out_i64[1]),
        position_ids=rows(out_i64[2]),
        response_masks=rows(out_i64[3]),
        original_responses=responses,
        num_actions=seq_rows(lens_dev[0]),
        packed_seq_lens=seq_rows(lens_dev[1]),
        dones=rows(out_i64[4]),
        vllm_logprobs=rows(out_f32[0]),
        advantages=rows(out_f32[1]) if adv_dev is not None else None,
    )
