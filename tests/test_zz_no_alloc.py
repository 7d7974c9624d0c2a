"""The statistics entry point that allocates nothing (``oi_grpo_fused_fwd_static``) through the raw
C-ABI against ``oi_grpo_fused_fwd``: same kernels, same order of summation, so every output must be
bit-identical.  Two calls in a row, the second on a smaller input (the static scratch keeps the
first call's partial sums), then the size limit."""

import pytest
import torch

from open_instruct_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
N_STATS = 16
MAX_BLOCKS = 8192


def _inputs(rows, cols, seed):
    g = torch.Generator().manual_seed(seed)
    new = -torch.rand(rows, cols, generator=g) * 5
    t = {
        "new": new,
        "old": new + 0.3 * torch.randn(rows, cols, generator=g),
        "ref": new + 0.5 * torch.randn(rows, cols, generator=g),
        "adv": torch.randn(rows, cols, generator=g),
        "rho": torch.rand(rows, cols, generator=g) * 2,
        "ent": torch.rand(rows, cols, generator=g) * 3,
        "drop": (torch.rand(rows, cols, generator=g) < 0.1).float(),
        "low": (torch.rand(rows, cols, generator=g) < 0.05).float(),
        "high": (torch.rand(rows, cols, generator=g) < 0.05).float(),
        "clip": (torch.rand(rows, cols, generator=g) < 0.2).float(),
    }
    t = {k: v.to(DEV).contiguous() for k, v in t.items()}
    mask = (torch.rand(rows, cols, generator=g) > 0.3).to(DEV).contiguous().view(torch.uint8)
    return t, mask


def _both(rows, cols, seed, axis_mode, denominator):
    lib = _lib.load()
    t, mask = _inputs(rows, cols, seed)
    stream = torch.cuda.current_stream().cuda_stream
    head = [t[k].data_ptr() for k in ("new", "old", "ref", "adv")] + [mask.data_ptr()]
    head += [t[k].data_ptr() for k in ("rho", "ent", "drop", "low", "high", "clip")]
    scalars = [rows, cols, 0, 0.8, 1.28, 2, 0.05, axis_mode, denominator, 2.0]
    outs = []
    for static in (False, True):
        stats = torch.full((N_STATS,), float("nan"), device=DEV)
        denoms = torch.full((rows,), float("nan"), device=DEV)
        if static:
            rc = lib.oi_grpo_fused_fwd_static(*head, *scalars, stats.data_ptr(), denoms.data_ptr(), stream)
        else:
            ws_bytes = lib.oi_grpo_fused_workspace_bytes(rows, cols)
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
            rc = lib.oi_grpo_fused_fwd(*head, *scalars, stats.data_ptr(), denoms.data_ptr(), ws.data_ptr(), ws_bytes, stream)
        assert rc == 0, rc
        torch.cuda.synchronize()
        outs.append((stats.cpu(), denoms.cpu()))
    return outs


def test_static_scratch_entry_matches_workspace_entry_twice_in_a_row():
    print("case static scratch: [64, 2100] then [3, 300]", flush=True)
    for rows, cols, seed, axis_mode, denominator in [(64, 2100, 1, 0, 0.0), (3, 300, 2, 1, 0.0), (7, 1024, 3, 0, 500.0)]:
        (s_ws, d_ws), (s_st, d_st) = _both(rows, cols, seed, axis_mode, denominator)
        assert torch.isfinite(s_ws).all() and torch.isfinite(d_ws).all()
        assert torch.equal(s_ws, s_st), (rows, cols, s_ws, s_st)
        assert torch.equal(d_ws, d_st)


def test_static_scratch_entry_limits():
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    # exactly at the limit: 8 rows x 1024 chunks of 1024 columns
    (s_ws, d_ws), (s_st, d_st) = _both(8, 1024 * 1024, 4, 1, 0.0)
    assert torch.equal(s_ws, s_st) and torch.equal(d_ws, d_st)
    # one block more: refused with the dedicated code, nothing launched, outputs untouched
    rows, cols = 8193, 10
    t, mask = _inputs(rows, cols, 5)
    stats = torch.full((N_STATS,), -7.0, device=DEV)
    denoms = torch.full((rows,), -7.0, device=DEV)
    head = [t[k].data_ptr() for k in ("new", "old", "ref", "adv")] + [mask.data_ptr()]
    head += [t[k].data_ptr() for k in ("rho", "ent", "drop", "low", "high", "clip")]
    rc = lib.oi_grpo_fused_fwd_static(
        *head, rows, cols, 0, 0.8, 1.28, 2, 0.05, 0, 0.0, 1.0, stats.data_ptr(), denoms.data_ptr(), stream
    )
    assert rc == -6 and b"static scratch" in lib.oi_error_string(rc)
    torch.cuda.synchronize()
    assert (stats == -7.0).all() and (denoms == -7.0).all()
