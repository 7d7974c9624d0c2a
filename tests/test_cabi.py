"""The C-ABI library: exported symbols, header/binding agreement, argument validation.

Runs without a GPU: nothing here launches a kernel (rejected calls return before any HIP call).
"""

import ctypes
import os
import re

import pytest
import torch

import open_instruct_amd
from open_instruct_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "oi_kernels.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(?:int|size_t|const char\*)\s+(oi_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        n = 0 if args in ("", "void") else len([a for a in args.split(",") if a.strip()])
        decls[m.group(1)] = n
    return decls


def test_library_is_built_and_loads():
    assert os.path.exists(_lib.LIB_PATH), "build with: python -m open_instruct_amd.build"
    lib = _lib.load()
    assert lib.oi_version() >= 1000


def test_every_declared_symbol_is_exported_and_bound():
    decls = _declared()
    assert len(decls) >= 25
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name, nargs in decls.items():
        assert hasattr(lib, name), f"{name} declared in oi_kernels.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
        assert len(_lib.SIGNATURES[name][1]) == nargs, f"{name}: header has {nargs} args"
    assert set(_lib.SIGNATURES) == set(decls)


def test_error_strings():
    lib = _lib.load()
    assert b"NULL" in lib.oi_error_string(-2)
    assert lib.oi_error_string(0) == b"ok"


def test_rejected_arguments_return_codes_without_launching():
    lib = _lib.load()
    # vocab <= 0
    assert lib.oi_lsg_entropy_fwd(None, 0, 1, 1, 0, 0, 0, None, 1.0, None, None, None, None) == -1
    # null logits with rows > 0
    assert lib.oi_lsg_entropy_fwd(None, 0, 1, 4, 0, 8, 8, None, 1.0, None, None, None, None) == -2
    # bad temperature
    assert lib.oi_lsg_entropy_fwd(None, 0, 1, 4, 0, 8, 8, None, 0.0, None, None, None, None) == -1
    # empty problem is fine
    assert lib.oi_lsg_entropy_fwd(None, 0, 0, 4, 0, 8, 8, None, 1.0, None, None, None, None) == 0
    # hidden size not a multiple of 64
    assert lib.oi_lmhead_logp_fwd(None, None, None, None, 4, 100, 32, 1.0, None, None, None, None, 0, None) == -1
    # unknown loss function / estimator
    assert lib.oi_grpo_terms_fwd(None, None, None, None, None, 4, 7, 0.8, 1.2, 2, None, None, None, None) == -1
    assert lib.oi_grpo_terms_fwd(None, None, None, None, None, 4, 0, 0.8, 1.2, 9, None, None, None, None) == -1
    assert lib.oi_grpo_terms_fwd(None, None, None, None, None, 4, 0, 0.8, 1.2, 2, None, None, None, None) == -2
    assert lib.oi_group_advantages(None, 2, 0, 0, None, None) == -1
    assert lib.oi_seq_logp_fwd(None, None, None, 2, 0, 0, None, None, None) == -1
    # row strides beyond 2^22 elements do not fit the tile engine's 32-bit lane offsets
    big = (1 << 22) + 64
    assert lib.oi_lmhead_logp_fwd(None, None, None, None, 4, big, 32, 1.0, None, None, None, None, 0, None) == -1
    assert lib.oi_lmhead_logp_fwd(None, None, None, None, big, 64, 32, 1.0, None, None, None, None, 0, None) == -1
    assert lib.oi_gemm_bf16_tn(None, big, 4, None, 64, 4, 64, None, None, 4, 0, None) == -1
    assert lib.oi_gemm_bf16_tn(None, 72, 4, None, 72, 4, 72, None, None, 4, 0, None) == -1  # K % 64
    assert lib.oi_gemm_bf16_layouts(None, 72, 1, None, 72, 0, 4, 8, 64, None, None, 8, 0, None) == -1  # M % 8, A k-major
    assert lib.oi_gemm_bf16_layouts(None, 72, 1, None, 72, 0, 8, 8, 64, None, None, 8, 0, None) == -2
    # packing and logprob statistics: missing pointers / sizes
    assert lib.oi_pack_sequences(*([None] * 9), -1, 0, 0, *([None] * 8)) == -1
    assert lib.oi_pack_sequences(*([None] * 9), 3, 0, 0, *([None] * 8)) == -2
    assert lib.oi_pack_sequences(*([None] * 9), 0, 0, 0, *([None] * 8)) == 0
    assert lib.oi_logprob_diff_stats(None, None, None, 4, None, None) == -2
    assert lib.oi_logprob_diff_stats(None, None, None, -1, None, None) == -1
    assert lib.oi_masked_mean_workspace_bytes(4, 2, 3) == (4 + 1) * 2 * 1 * 4
    # the entry point without a workspace refuses what its static scratch cannot hold (the pointers
    # are never dereferenced: the call is rejected before anything touches the GPU)
    fake = [8] * 11
    assert lib.oi_grpo_fused_fwd_static(*fake, 8193, 10, 0, 0.8, 1.2, 2, 0.05, 0, 0.0, 1.0, 8, 8, None) == -6
    assert lib.oi_grpo_fused_fwd_static(*fake, 9, 1024 * 1024, 0, 0.8, 1.2, 2, 0.05, 0, 0.0, 1.0, 8, 8, None) == -6
    assert lib.oi_grpo_fused_fwd_static(*fake, 4, 10, 5, 0.8, 1.2, 2, 0.05, 0, 0.0, 1.0, 8, 8, None) == -1
    assert lib.oi_grpo_fused_fwd_static(*([None] * 11), 4, 10, 0, 0.8, 1.2, 2, 0.05, 0, 0.0, 1.0, 8, 8, None) == -2
    assert lib.oi_lmhead_fwd_workspace_bytes(0, 64, 10, 0) == 0
    # one dZ chunk (bf16), the fp32 d_hidden accumulator, three queues of 8 words; no transposed copies
    plain = 256 * 256 * 2 + 256 * 64 * 4 + 256
    assert lib.oi_lmhead_bwd_workspace_bytes(256, 64, 256, 1, 0) == plain
    assert lib.oi_lmhead_bwd_workspace_bytes(256, 64, 256, 0, 0) == plain
    # a row selection adds the row index, the count, the gathered hidden rows / labels / lse / gradient / logprob
    selection = 256 * 4 + 256 + 256 * 64 * 2 + 256 * 8 + 3 * 256 * 4
    assert lib.oi_lmhead_bwd_workspace_bytes(256, 64, 256, 1, 1) == plain + selection
    assert lib.oi_lmhead_fwd_workspace_bytes(256, 64, 256, 1) == lib.oi_lmhead_fwd_workspace_bytes(256, 64, 256, 0) + 256 * 4 + 256 + 256 * 64 * 2 + 256 * 8
    # the forward that also accumulates the weighted sum of weight rows: the plain forward's buffers (one split per
    # vocabulary tile at this size), one pair of queue sets per vocabulary chunk of 65536 columns and the chunk of
    # exponentials (2 bytes per token and column)
    assert lib.oi_lmhead_fwd_wsum_workspace_bytes(0, 64, 10, 0) == 0
    assert lib.oi_lmhead_fwd_wsum_workspace_bytes(256, 64, 256, 0) == 256 * 16 + 256 * 4 + 256 + 256 * 256 * 2
    assert lib.oi_lmhead_fwd_wsum_workspace_bytes(256, 64, 70000, 0) >= 256 * 65536 * 2
    # its backward: the mask's row index and count, and the recomputing backward (with a row selection) for flagged rows
    assert lib.oi_lmhead_dh_workspace_bytes(0, 64, 256) == 0
    assert lib.oi_lmhead_dh_workspace_bytes(256, 64, 256) == 256 * 4 + 256 + plain + selection
    assert lib.oi_lmhead_logp_fwd_wsum(None, None, None, None, 4, 100, 32, 1.0, *([None] * 7), 0, None) == -1
    assert lib.oi_lmhead_logp_fwd_wsum(16, 32, 8, None, 4, 64, 32, 1.0, *([None] * 7), 0, None) == -2
    assert lib.oi_lmhead_dh_from_wsum(*([None] * 10), 4, 100, 32, 1.0, None, None, 0, None) == -1
    assert lib.oi_lmhead_dh_from_wsum(*([None] * 10), 4, 64, 32, 1.0, None, None, 0, None) == -2
    assert lib.oi_lmhead_dh_from_wsum(*([None] * 10), 0, 64, 32, 1.0, None, None, 0, None) == 0
    # the whole step: recomputing (slab size 0: forward and backward regions side by side), or in slabs of tokens
    # (a slab of exponentials or the recomputing backward for flagged rows, whichever is larger; with d_weight and
    # more than one slab an fp32 d_weight)
    whole = lib.oi_lmhead_grpo_workspace_bytes(4, 4096, 64, 1000, 1, 0)
    assert whole >= lib.oi_lmhead_bwd_workspace_bytes(4 * 4096, 64, 1000, 1, 1)
    slabs = lib.oi_lmhead_grpo_workspace_bytes(4, 4096, 64, 1000, 1, 4096)
    assert slabs >= 4096 * 1024 * 2 + 1000 * 64 * 4
    assert lib.oi_lmhead_grpo_workspace_bytes(4, 4096, 64, 1000, 0, 4096) <= slabs - 1000 * 64 * 4
    assert lib.oi_lmhead_grpo_workspace_bytes(4, 4096, 64, 1000, 1, 16384) < slabs + 12288 * 1024 * 2  # one slab: no fp32 d_weight
    assert lib.oi_lmhead_grpo_fwd_bwd(*([8] * 8), 4, 4096, 64, 1000, 1.0, 0, 0.8, 1.2, 2, 0.05, 0, 0.0, 1.0, *([8] * 5), -1, 8, 0, None) == -1


def test_cpu_tensors_are_refused_loudly():
    logits = torch.randn(2, 8)
    with pytest.raises(RuntimeError, match="GPU only"):
        open_instruct_amd.model_utils.log_softmax_and_gather(logits, torch.zeros(2, dtype=torch.long))
    with pytest.raises(RuntimeError, match="GPU only"):
        open_instruct_amd.rl_utils.masked_mean(torch.ones(2, 3), torch.ones(2, 3))
    with pytest.raises(RuntimeError, match="GPU only"):
        open_instruct_amd.dpo_utils.dpo_loss(torch.zeros(2), torch.zeros(2), torch.zeros(2), torch.zeros(2), 0.1)


def test_missing_library_is_an_error(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/liboi_kernels.so")
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()
