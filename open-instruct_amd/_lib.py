"""ctypes binding of ``liboi_kernels.so`` (the C-ABI declared in ``include/oi_kernels.h``).

The library is built in-tree by :mod:`open_instruct_amd.build`.  There is no other code path: if
the shared object is missing, or a tensor is not on a GPU, the call raises.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_double, c_float, c_int, c_int64, c_size_t, c_uint32, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "liboi_kernels.so")

DTYPE_TAGS = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
LOSS_FN_TAGS = {"dapo": 0, "cispo": 1}

_P, _I64, _F, _I, _SZ = c_void_p, c_int64, c_float, c_int, c_size_t

# name -> (restype, argtypes); mirrors include/oi_kernels.h one to one
SIGNATURES: dict[str, tuple] = {
    "oi_version": (_I, []),
    "oi_error_string": (c_char_p, [_I]),
    "oi_lsg_entropy_fwd": (_I, [_P, _I, _I64, _I64, _I64, _I64, _I64, _P, _F, _P, _P, _P, _P]),
    "oi_lsg_bwd": (_I, [_P, _I, _I64, _I64, _I64, _I64, _I64, _P, _P, _P, _F, _P, _I64, _I64, _P]),
    "oi_lsg_grpo_fwd_bwd": (
        _I,
        [_P, _I, _I64, _I64, _I64, _I64, _I64, _P, _F, _P, _P, _P, _P, _P, _I, _F, _F, _I, _F, _P, _P, _P, _P, _I64, _I64, _P],
    ),
    "oi_grpo_terms_fwd": (_I, [_P, _P, _P, _P, _P, _I64, _I, _F, _F, _I, _P, _P, _P, _P]),
    "oi_grpo_terms_bwd": (_I, [_P, _P, _P, _P, _P, _P, _P, _I64, _I, _F, _F, _I, _P, _P, _P]),
    "oi_grpo_fused_workspace_bytes": (_SZ, [_I64, _I64]),
    "oi_grpo_fused_fwd": (
        _I,
        [_P] * 11 + [_I64, _I64, _I, _F, _F, _I, _F, _I, _F, _F, _P, _P, _P, _SZ, _P],
    ),
    "oi_grpo_fused_fwd_static": (
        _I,
        [_P] * 11 + [_I64, _I64, _I, _F, _F, _I, _F, _I, _F, _F, _P, _P, _P],
    ),
    "oi_grpo_stats_from_terms": (_I, [_P] * 12 + [_I64, _I64, _I, _F, _P, _I64, c_uint32, _P, _SZ, _P]),
    "oi_scale_by_device_scalar": (_I, [_P, _I, _I64, _P, _P]),
    "oi_grpo_fused_bwd": (_I, [_P, _P, _P, _P, _P, _P, _I64, _I64, _I, _F, _F, _I, _F, _F, _P, _P, _P, _P]),
    "oi_estimate_kl_fwd": (_I, [_P, _P, _I64, _P, _P]),
    "oi_estimate_kl_bwd": (_I, [_P, _P, _P, _I64, _P, _P, _P]),
    "oi_mask_logprobs_fwd": (_I, [_P, _P, _I64, _F, _P, _P]),
    "oi_mask_logprobs_bwd": (_I, [_P, _P, _P, _I64, _P, _P]),
    "oi_rho_correction": (_I, [_P, _P, _P, _P, _I64, _I64, _I, _I, _F, _F, _F, _F, _P, _P, _P, _P, _P, _P, _P]),
    "oi_group_advantages": (_I, [_P, _I64, _I64, _I, _P, _P]),
    "oi_masked_mean_workspace_bytes": (_SZ, [_I64, _I64, _I64]),
    "oi_masked_mean_fwd": (_I, [_P, _P, _I, _I64, _I64, _I64, _I, _F, _P, _P, _P, _SZ, _P]),
    "oi_masked_mean_bwd": (_I, [_P, _P, _I, _P, _I64, _I64, _I64, _P, _P]),
    "oi_seq_logp_fwd": (_I, [_P, _P, _P, _I64, _I64, _I, _P, _P, _P]),
    "oi_seq_logp_bwd": (_I, [_P, _P, _P, _P, _I64, _I64, _I, _P, _P]),
    "oi_logprob_diff_stats": (_I, [_P, _P, _P, _I64, _P, _P]),
    "oi_dpo_sigmoid_fwd": (_I, [_P, _P, _P, _P, _P, _I64, _F, _F, _F, _P, _P, _P, _P]),
    "oi_dpo_sigmoid_bwd": (_I, [_P, _P, _P, _P, _P, _P, _I64, _F, _F, _F, _P, _P, _P]),
    "oi_pack_sequences": (_I, [_P] * 9 + [_I64, _I64, _I] + [_P] * 8),
    "oi_lmhead_fwd_workspace_bytes": (_SZ, [_I64, _I64, _I64, _I]),
    "oi_lmhead_logp_fwd": (_I, [_P, _P, _P, _P, _I64, _I64, _I64, _F, _P, _P, _P, _P, _SZ, _P]),
    "oi_lmhead_bwd_workspace_bytes": (_SZ, [_I64, _I64, _I64, _I, _I]),
    "oi_lmhead_logp_bwd": (_I, [_P, _P, _P, _P, _P, _P, _I, _I64, _I64, _I64, _F, _P, _P, _P, _P, _SZ, _P]),
    "oi_lmhead_fwd_wsum_workspace_bytes": (_SZ, [_I64, _I64, _I64, _I]),
    "oi_lmhead_logp_fwd_wsum": (_I, [_P, _P, _P, _P, _I64, _I64, _I64, _F, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "oi_lmhead_dh_workspace_bytes": (_SZ, [_I64, _I64, _I64]),
    "oi_lmhead_dh_from_wsum": (_I, [_P] * 10 + [_I64, _I64, _I64, _F, _P, _P, _SZ, _P]),
    "oi_lmhead_grpo_workspace_bytes": (_SZ, [_I64, _I64, _I64, _I64, _I, _I64]),
    "oi_lmhead_grpo_fwd_bwd": (
        _I,
        [_P] * 8 + [_I64, _I64, _I64, _I64, _F, _I, _F, _F, _I, _F, _I, _F, _F] + [_P] * 5 + [_I64, _P, _SZ, _P],
    ),
    "oi_lmhead_dpo_workspace_bytes": (_SZ, [_I64, _I64, _I, _I64, _I64, _I, _I64]),
    "oi_lmhead_dpo_fwd_bwd": (
        _I,
        [_P, _P, _P, _P, _I64, _I64, _I64, _I64, _F, _P, _P, _F, _F, _F, _I, _F] + [_P] * 7 + [_I64, _P, _SZ, _P],
    ),
    "oi_lmhead_probe_arm": (_I, [_I]),
    "oi_lmhead_probe_read": (_I, [_P, _I, _P]),
    "oi_gemm_bf16_tn": (_I, [_P, _I64, _I64, _P, _I64, _I64, _I64, _P, _P, _I64, _I, _P]),
    "oi_gemm_bf16_layouts": (_I, [_P, _I64, _I, _P, _I64, _I, _I64, _I64, _I64, _P, _P, _I64, _I, _P]),
}

_lib: ctypes.CDLL | None = None


class KernelError(RuntimeError):
    """A C-ABI entry point returned a non-zero status."""


def load() -> ctypes.CDLL:
    """Load the shared object once and attach the argument types."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m open_instruct_amd.build` "
                "(hipcc --offload-arch=gfx950). There is no fallback implementation."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def stream_of(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def require_gpu(*tensors: torch.Tensor | None) -> torch.device:
    """All given tensors must live on the same GPU; returns that device."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "open_instruct_amd runs on an AMD GPU only (got a tensor on "
                f"{t.device}); there is no CPU implementation in this package."
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    if dev is None:
        raise RuntimeError("no tensor argument to take the device from")
    return dev


def call(name: str, *args) -> None:
    """Invoke an ``int``-returning entry point and raise on a non-zero status."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.oi_error_string(rc).decode()
        raise KernelError(f"{name} failed with status {rc}: {msg}")


def f32c(t: torch.Tensor | None) -> torch.Tensor | None:
    """fp32 + contiguous view/copy of a side tensor (no-op for the normal case)."""
    if t is None:
        return None
    if t.dtype != torch.float32:
        t = t.float()
    return t if t.is_contiguous() else t.contiguous()


def mask_u8(mask: torch.Tensor) -> torch.Tensor:
    """One byte per token.  A bool tensor is reinterpreted in place, anything else is compared to 0."""
    if mask.dtype == torch.bool:
        m = mask if mask.is_contiguous() else mask.contiguous()
        return m.view(torch.uint8)
    if mask.dtype == torch.uint8:
        return mask if mask.is_contiguous() else mask.contiguous()
    return (mask != 0).contiguous().view(torch.uint8)


__all__ = [
    "DTYPE_TAGS",
    "LOSS_FN_TAGS",
    "KernelError",
    "LIB_PATH",
    "SIGNATURES",
    "c_double",
    "call",
    "f32c",
    "load",
    "mask_u8",
    "ptr",
    "require_gpu",
    "stream_of",
]
