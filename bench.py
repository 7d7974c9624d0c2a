"""Benchmark of the policy-loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c2|c1|c4|c5|...] [--slab-tokens N]

Prints ONE JSON line.  A "step" is one pass of the hot path (forward + backward) over one batch of
synthetic inputs that already live in HBM.  Workloads are the BASELINE configs:

  c3 (default, the headline metric): fused lm_head + logprob + entropy + GRPO loss, fwd + bwd, at
      Llama-3.1-8B shape: hidden bf16 [32768, 4096], W bf16 [128256, 4096], 70 % response tokens,
      through grpo_loss_on_hidden as it runs by default (slabs of tokens, nothing recomputed);
      c3-recompute is the same step through the three differentiable calls whose backward recomputes
      the logits, c3-one-call-recompute the recomputing form of the one-call entry.
  c2: GRPO loss on materialised bf16 logits [64, 1024, 128256], fwd + bwd (HBM-bound), single pass;
      c2-two-pass keeps the reference's order of operations (the logits are read twice).
  c1: logprob + entropy + masked_mean on fp32 logits [4, 512, 32000], forward only.
  c4: packed batch at OLMo-2-7B shape (16 sequences, cu_seqlens, V=100352), per-sequence sums + GRPO loss
      (c4-recompute: through the three differentiable calls).
  c5: DPO at Llama-3.1-70B head shape: hidden [32768, 8192], W [128256, 8192], bwd to dHidden only.
      c5-train-head: the same batch with a trainable head (what the reference's DPO trains), loss and
      both gradients from one no-recompute call (dpo_loss_on_hidden); c5-train-head-recompute: the same
      through the differentiable calls; c5-one-call: the frozen-head batch through dpo_loss_on_hidden;
      ref-cache: the forward-only pass over that batch that fills the reference-logprob cache of a DPO run.
  sft: causal-LM cross-entropy (the supervised fine-tuning loss) at the c3 head shape, fwd + bwd, slab-wise.
  pack: pack_sequences + advantage broadcast for 512 prompt / response pairs (about 1.09 M tokens).

`roofline` describes the dominant kernel of the workload, timed with HIP events on the stream it
runs on inside the timed region (for the slab-wise workloads through the library's own event probe, with
the other two tile kernels of the call timed over three more steps and reported beside it; --one-kernel
leaves those extra steps out); `cpu_baseline` is the oracle's restatement of the reference's
PyTorch path on a bounded sample of the same workload, on this machine's host cores.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time
import types

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0
PEAK_BF16_TFLOPS = 2500.0

# HBM-side bytes per launch of each workload's dominant kernel, from two `rocprofv3 --pmc` runs of
# this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter
# reads for a 1 GiB device copy (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000 on MI355X).  Counters cannot
# be read from inside the process, so the figures are carried here from the committed summaries in
# profiles/; workloads without a counter run report null.
MEASURED_TRAFFIC_BYTES = {
    # gemm_store_kernel<true, true>, the d_weight product of one slab (average of the launches with rows: two of them
    # write fp32, the last one bf16): L2 misses of the tiled operand re-reads + the result
    "c3": 15.75e9 + 1.81e9,
    "c4": 13.68e9 + 1.49e9,
    "c5-train-head": 31.04e9 + 3.57e9,
    # lmhead_fwd_kernel: L2 misses of the tiled operand re-reads (1.24 GB of unique operands at c3) + the partials
    "c3-recompute": 42.57e9 + 0.20e9,
    "c4-recompute": 40.24e9 + 0.20e9,
    # oi_lmhead_logp_fwd_wsum: two launches of lmhead_fwd_kernel<true> and two of gemm_store_kernel<false, true>
    "c5": 2 * (44.80e9 + 3.09e9) + 2 * (40.44e9 + 0.75e9),
    # lsg_grpo_fused_kernel: one read of the logits (the row waits on the CU for the gradient pass) + one write of
    # dlogits
    "c2": 16.88e9 + 16.94e9,
    "c2-two-pass": 16.83e9 + 0.0e9,  # lsg_entropy_fwd_kernel: 1.00x the logits
}


def _cfg():
    return types.SimpleNamespace(loss_fn="dapo", clip_lower=0.2, clip_higher=0.28, beta=0.05, kl_estimator=2)


class EventTimer:
    """Accumulates the duration of one region per step with HIP events on the current stream."""

    def __init__(self, torch):
        self.torch = torch
        self.pairs = []

    def __enter__(self):
        self.a = self.torch.cuda.Event(enable_timing=True)
        self.b = self.torch.cuda.Event(enable_timing=True)
        self.a.record()
        return self

    def __exit__(self, *exc):
        self.b.record()
        self.pairs.append((self.a, self.b))

    def mean_ms(self):
        return sum(a.elapsed_time(b) for a, b in self.pairs) / max(1, len(self.pairs))

    def reset(self):
        self.pairs = []


# ------------------------------------------------------------------------------------------------
# workloads
# ------------------------------------------------------------------------------------------------
class KernelProbe:
    """Times one tile kernel of the slab-wise entry points through the library's own event probe (the
    call launches several kernels, so events around the call would time all of them).  The probe is armed
    by reset() (or by the first step) and read only when the figures are asked for, after the caller has
    synchronised: nothing inside the timed steps waits for the device.  The library records the first
    1024 launches of the kernel; a run with more of them than that is refused."""

    CAPACITY = 1024

    def __init__(self, oi, kernel):
        self.oi, self.kernel, self._samples, self._armed = oi, kernel, [], False

    def __enter__(self):
        if not self._armed:
            self.oi._lib.call("oi_lmhead_probe_arm", self.kernel)
            self._armed = True
        return self

    def __exit__(self, *exc):
        pass

    def _collect(self):
        import ctypes

        if self._armed:
            ms = (ctypes.c_float * self.CAPACITY)()
            n = ctypes.c_int(0)
            self.oi._lib.call("oi_lmhead_probe_read", ms, self.CAPACITY, ctypes.byref(n))
            if n.value >= self.CAPACITY:
                raise SystemExit(f"bench.py: more than {self.CAPACITY} launches of the probed kernel between two readings; use fewer --steps")
            self._samples += [ms[i] for i in range(n.value)]
            self._armed = False

    @property
    def samples(self):
        self._collect()
        return self._samples

    def reset(self):
        """Drops what was recorded so far and arms the probe again (the events are created here, before the
        caller starts its clock)."""
        self._collect()
        self._samples = []
        self.__enter__()

    def threshold(self):
        """A launch without rows (a pass past the last slab) takes microseconds, one with rows milliseconds."""
        return 0.1 * max(self.samples, default=0.0)

    def mean_ms(self):
        """Average over the launches that had rows to work on."""
        real = [x for x in self.samples if x >= self.threshold()]
        return sum(real) / max(1, len(real))


def make_fused(torch, oi, n_tokens, hdim, vocab, w_std, dpo=False, route="slabs", train_head=False, one_call=False):
    """route: "slabs" = grpo_loss_on_hidden as it runs by default, "one-call-recompute" = the same entry with
    token_slabs=False, "recompute" = fused_lm_head_logprobs -> grpo_loss_fused -> backward.  dpo: the frozen
    head of the DPO config unless train_head (then route "slabs" = dpo_loss_on_hidden, else the differentiable
    calls with a recomputing backward)."""
    dev = "cuda:0"
    torch.manual_seed(0)
    hidden = torch.randn(n_tokens, hdim, device=dev).bfloat16().requires_grad_(True)
    weight = (torch.randn(vocab, hdim, device=dev) * w_std).bfloat16().requires_grad_(not dpo or train_head)
    labels = torch.randint(0, vocab, (n_tokens,), device=dev)
    cfg = _cfg()
    if not dpo:
        mask = torch.rand(n_tokens, device=dev) < 0.7
        adv = torch.randn(n_tokens, device=dev)
        with torch.no_grad():
            lp0, _ = oi.fused_lm_head_logprobs(hidden, weight, labels, mask=mask)
        old = lp0 + 0.05 * torch.randn(n_tokens, device=dev)
        ref = lp0 + 0.1 * torch.randn(n_tokens, device=dev)
        n_eff = int(mask.sum().item())
    else:
        # 16 sequences of 2048 tokens, prompt (128..1024 tokens) masked out with -100 labels
        seqs, per = n_tokens // 2048, 2048
        prompt = torch.randint(128, 1025, (seqs,), device=dev)
        pos = torch.arange(per, device=dev).unsqueeze(0).expand(seqs, per)
        lab2 = labels.view(seqs, per).clone()
        lab2[pos < prompt.unsqueeze(1)] = -100
        labels = lab2.view(1, -1)
        cu = torch.arange(0, n_tokens + 1, per, device=dev, dtype=torch.int32)
        shifted = oi.padding_free_collator.shift_labels(labels)
        mask = (shifted != -100).view(-1)
        ref_c = torch.randn(seqs // 2, device=dev) * 50 - 400
        ref_r = torch.randn(seqs // 2, device=dev) * 50 - 400
        n_eff = int(mask.sum().item())
    fwd_timer = EventTimer(torch)
    # the d_weight product: the largest share of the slab-wise step (without d_weight: the d_hidden product)
    probe = KernelProbe(oi, 1 if (dpo and one_call and not train_head) else 2)
    dpo_slab = oi.dpo_utils.DEFAULT_DPO_SLAB_TOKENS

    def step():
        hidden.grad = None
        weight.grad = None
        if dpo and route == "forward":
            # the pass that fills the reference-logprob cache: no gradient, per-sequence sums of the logprobs
            with torch.no_grad():
                with fwd_timer:
                    lp, _ = oi.fused_lm_head_logprobs(hidden, weight, shifted.view(-1), mask=mask)
                logps = oi.padding_free_collator.get_batch_logps(lp.view(1, -1), labels, cu)
            return logps.sum()
        if dpo and route == "slabs" and (train_head or one_call):
            with probe:
                res = oi.dpo_utils.dpo_loss_on_hidden(
                    hidden[None], weight, labels, ref_c, ref_r, 0.1, cu_seq_lens=cu, token_slabs=dpo_slab
                )
            loss = res.loss
        elif dpo:
            with fwd_timer:
                lp, _ = oi.fused_lm_head_logprobs(hidden, weight, shifted.view(-1), mask=mask)
            logps = oi.padding_free_collator.get_batch_logps(lp.view(1, -1), labels, cu)
            bs = logps.shape[0] // 2
            losses, _, _ = oi.dpo_utils.dpo_loss(logps[:bs], logps[bs:], ref_c, ref_r, beta=0.1)
            loss = losses.mean()
        elif route == "slabs":
            with probe:
                loss, _, _, _ = oi.grpo_utils.grpo_loss_on_hidden(
                    hidden[None], weight, labels[None], old[None], ref[None], adv[None], mask[None], cfg
                )
        elif route == "one-call-recompute":
            with fwd_timer:  # the whole step is one C call here: the timer brackets all of it
                loss, _, _, _ = oi.grpo_utils.grpo_loss_on_hidden(
                    hidden[None], weight, labels[None], old[None], ref[None], adv[None], mask[None], cfg,
                    token_slabs=False,
                )
        else:
            with fwd_timer:
                lp, ent = oi.fused_lm_head_logprobs(hidden, weight, labels, mask=mask, return_entropy=True)
            loss, _ = oi.grpo_utils.grpo_loss_fused(
                lp[None], old[None], ref[None], adv[None], mask[None], cfg, entropy=ent[None]
            )
        loss.backward()
        return loss

    flops_fwd = 2.0 * n_eff * hdim * vocab
    info = {
        "tokens": n_tokens,
        "rows_multiplied": n_eff,
        "hdim": hdim,
        "vocab": vocab,
        "flops_step": (2.0 if dpo else 3.0) * flops_fwd,
        "kernel": "lmhead_fwd_kernel (fused lm_head forward: MFMA tiles + online softmax statistics)",
        "alg_per_launch": flops_fwd,
        "bound": "mfma",
        "timer": fwd_timer,
    }
    if dpo and route == "forward":
        info["flops_step"] = flops_fwd
    elif dpo and (train_head or one_call):
        info["flops_step"] = (3.0 if train_head else 2.0) * flops_fwd
        if route == "slabs" and one_call and not train_head:
            info["kernel"] = (
                f"gemm_store_kernel<false, true> (d_hidden product of a slab of whole chosen/rejected pairs, at most {dpo_slab} "
                "scored tokens; timed launch by launch through the library's event probe)"
            )
            info["alg_per_launch"] = None
            info["timer"] = probe
        elif route == "slabs":
            info["kernel"] = (
                f"gemm_store_kernel<true, true> (d_weight product of a slab of whole chosen/rejected pairs, at most {dpo_slab} "
                "scored tokens, added to the fp32 d_weight; timed launch by launch through the library's event probe)"
            )
            info["alg_per_launch"] = None  # filled in from the number of launches that had rows
            info["timer"] = probe
    elif dpo and route != "forward":
        # the weight takes no gradient: the forward call also accumulates the weighted sum of weight rows that
        # the backward to hidden needs (per vocabulary chunk: statistics + exponentials, then E_chunk @ W_chunk)
        info["kernel"] = (
            "oi_lmhead_logp_fwd_wsum (per vocabulary chunk: lmhead_fwd_kernel<true> + gemm_store_kernel<false, true>; "
            "all of the step's matrix work, nothing is recomputed)"
        )
        info["alg_per_launch"] = 2.0 * flops_fwd
    elif route == "slabs":
        slab = oi.grpo_utils.DEFAULT_SLAB_TOKENS
        n_slabs = max(1, -(-n_eff // slab))
        info["kernel"] = (
            f"gemm_store_kernel<true, true> (d_weight product of a slab of {-(-n_eff // n_slabs)} selected tokens, added to the "
            f"fp32 d_weight; {n_slabs} such launches per step, timed one by one through the library's event probe)"
        )
        info["alg_per_launch"] = flops_fwd / n_slabs
        info["timer"] = probe
    elif route == "one-call-recompute":
        info["kernel"] = "oi_lmhead_grpo_fwd_bwd, recomputing (every launch of the step: forward, loss, dZ, dHidden, dW)"
        info["alg_per_launch"] = 3.0 * flops_fwd
    return step, info


def make_c2(torch, oi, rows_b=64, t=1024, vocab=128256, single_pass=True):
    """GRPO loss on materialised logits.  single_pass: forward and gradient in one read and one write
    of the logits (grpo_loss_on_logits); otherwise the reference's order of operations with the
    logits read twice (log_softmax_and_gather -> loss -> backward)."""
    dev = "cuda:0"
    torch.manual_seed(0)
    logits = torch.empty(rows_b, t, vocab, device=dev, dtype=torch.bfloat16)
    for b in range(rows_b):  # generated per row block to bound the fp32 temporary
        logits[b] = (torch.randn(t, vocab, device=dev) * 3.0).bfloat16()
    logits.requires_grad_(True)
    labels = torch.randint(0, vocab, (rows_b, t), device=dev)
    rewards = (torch.rand(rows_b, device=dev) < 0.3).double()
    adv = oi.grpo_utils.group_advantages(rewards, 8).unsqueeze(1).expand(rows_b, t).contiguous()
    mask = torch.ones(rows_b, t, dtype=torch.bool, device=dev)
    with torch.no_grad():
        lp0 = oi.model_utils.log_softmax_and_gather(logits, labels)
    old = lp0 + 0.05 * torch.randn(rows_b, t, device=dev)
    ref = lp0 + 0.1 * torch.randn(rows_b, t, device=dev)
    cfg = _cfg()
    fwd_timer = EventTimer(torch)

    def step_two_pass():
        logits.grad = None
        with fwd_timer:
            lp = oi.model_utils.log_softmax_and_gather(logits, labels)
        loss, _ = oi.grpo_utils.grpo_loss_fused(lp, old, ref, adv, mask, cfg)
        loss.backward()
        return loss

    plain_call = oi._lib.call

    def timed_call(name, *args):
        if name != "oi_lsg_grpo_fwd_bwd":
            return plain_call(name, *args)
        with fwd_timer:
            return plain_call(name, *args)

    def step_single_pass():
        logits.grad = None
        loss, _, _, _ = oi.grpo_utils.grpo_loss_on_logits(logits, labels, old, ref, adv, mask, cfg)
        loss.backward()
        return loss

    n = rows_b * t
    if single_pass:
        oi._lib.call = timed_call
        info = {
            "tokens": n,
            "rows_multiplied": n,
            "bytes_step": 2.0 * n * vocab * 2,
            "kernel": "lsg_grpo_fused_kernel (one resident 1024-thread workgroup per CU: statistics pass, GRPO derivative, gradient pass; the row waits in the LDS and in registers between the passes)",
            "alg_per_launch": 2.0 * n * vocab * 2,
            "bound": "hbm",
            "timer": fwd_timer,
        }
        return step_single_pass, info
    info = {
        "tokens": n,
        "rows_multiplied": n,
        "bytes_step": 3.0 * n * vocab * 2,
        "kernel": "lsg_entropy_fwd_kernel (row-wise log-softmax gather, one read of the logits)",
        "alg_per_launch": 1.0 * n * vocab * 2,
        "bound": "hbm",
        "timer": fwd_timer,
    }
    return step_two_pass, info


def make_c1(torch, oi):
    dev = "cuda:0"
    torch.manual_seed(0)
    logits = (torch.randn(4, 512, 32000) * 2.0).to(dev)
    ids = torch.randint(0, 32000, (4, 512)).to(dev)
    length = torch.randint(64, 513, (4,))
    mask = (torch.arange(512).unsqueeze(0) >= (512 - length).unsqueeze(1)).to(dev)
    timer = EventTimer(torch)

    def step():
        with timer:
            lp, ent = oi.model_utils.logprob_and_entropy(logits, ids)
        return oi.rl_utils.masked_mean(lp, mask) + oi.rl_utils.masked_mean(ent, mask)

    n = 2048
    info = {
        "tokens": n,
        "rows_multiplied": n,
        "bytes_step": 1.0 * n * 32000 * 4,
        "kernel": "lsg_entropy_fwd_kernel (fp32 rows, logprob + entropy in one pass)",
        "alg_per_launch": 1.0 * n * 32000 * 4,
        "bound": "hbm",
        "timer": timer,
    }
    return step, info


def make_c4(torch, oi, hdim=4096, vocab=100352, n_seqs=16, budget=32768, route="slabs"):
    """Packed (padding-free) batch: per-sequence summed logprobs through cu_seqlens plus the GRPO loss
    with masked_mean(axis=1) over the packed row, forward and backward."""
    dev = "cuda:0"
    torch.manual_seed(0)
    lens = torch.randint(128, 4097, (n_seqs,)).tolist()
    kept, total = [], 0
    for n in lens:  # greedy truncation to the token budget
        n = min(n, budget - total)
        if n <= 1:
            break
        kept.append(n)
        total += n
    cu = torch.tensor([0] + list(torch.tensor(kept).cumsum(0)), dtype=torch.int32, device=dev)
    n_tokens = total
    hidden = torch.randn(n_tokens, hdim, device=dev).bfloat16().requires_grad_(True)
    weight = (torch.randn(vocab, hdim, device=dev) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, vocab, (1, n_tokens), device=dev)
    labels[0, cu[:-1].long()] = -100  # first token of every sequence is never a target
    shifted = oi.padding_free_collator.shift_labels(labels)
    mask = (shifted != -100).view(-1)
    adv = torch.randn(n_tokens, device=dev)
    cfg = _cfg()
    with torch.no_grad():
        lp0, _ = oi.fused_lm_head_logprobs(hidden, weight, shifted.view(-1), mask=mask)
    old = lp0 + 0.05 * torch.randn(n_tokens, device=dev)
    ref = lp0 + 0.1 * torch.randn(n_tokens, device=dev)
    n_eff = int(mask.sum().item())
    fwd_timer = EventTimer(torch)
    probe = KernelProbe(oi, 2)

    def step_slabs():
        # the GRPO loss and both gradients in one slab-wise call (nothing recomputed); the per-sequence sums are
        # taken from the returned logprobs (the loss does not depend on them)
        hidden.grad = None
        weight.grad = None
        with probe:
            loss, _, lp, _ = oi.grpo_utils.grpo_loss_on_hidden(
                hidden[None], weight, shifted.view(1, -1), old[None], ref[None], adv[None], mask[None], cfg, axis=1
            )
        oi.padding_free_collator.get_batch_logps(lp.view(1, -1), labels, cu)
        loss.backward()
        return loss

    def step():
        hidden.grad = None
        weight.grad = None
        with fwd_timer:
            lp, ent = oi.fused_lm_head_logprobs(hidden, weight, shifted.view(-1), mask=mask, return_entropy=True)
        seq_logps = oi.padding_free_collator.get_batch_logps(lp.view(1, -1), labels, cu)
        loss, _ = oi.grpo_utils.grpo_loss_fused(
            lp[None], old[None], ref[None], adv[None], mask[None], cfg, entropy=ent[None], axis=1
        )
        (loss + 1e-6 * seq_logps.mean()).backward()
        return loss

    flops_fwd = 2.0 * n_eff * hdim * vocab
    info = {
        "tokens": n_tokens,
        "rows_multiplied": n_eff,
        "hdim": hdim,
        "vocab": vocab,
        "flops_step": 3.0 * flops_fwd,
        "kernel": "lmhead_fwd_kernel (fused lm_head forward: MFMA tiles + online softmax statistics)",
        "alg_per_launch": flops_fwd,
        "bound": "mfma",
        "timer": fwd_timer,
    }
    if route == "slabs":
        slab = oi.grpo_utils.DEFAULT_SLAB_TOKENS
        n_slabs = max(1, -(-n_eff // slab))
        info["kernel"] = (
            f"gemm_store_kernel<true, true> (d_weight product of a slab of {-(-n_eff // n_slabs)} selected tokens, added to the "
            f"fp32 d_weight; {n_slabs} such launches per step, timed one by one through the library's event probe)"
        )
        info["alg_per_launch"] = flops_fwd / n_slabs
        info["timer"] = probe
        return step_slabs, info
    return step, info


def make_sft(torch, oi, batch=8, seq=4096, hdim=4096, vocab=128256):
    """Supervised fine-tuning loss (open_instruct/finetune.py:818-824) at the Llama-3.1-8B head shape: causal-LM
    cross-entropy of 8 sequences of 4096 tokens whose prompts (256..2048 tokens) carry ignored labels, forward and
    backward to the hidden states and the head through fused_linear_cross_entropy(token_slabs=True)."""
    dev = "cuda:0"
    torch.manual_seed(0)
    hidden = torch.randn(batch, seq, hdim, device=dev).bfloat16().requires_grad_(True)
    weight = (torch.randn(vocab, hdim, device=dev) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, vocab, (batch, seq), device=dev)
    prompt = torch.randint(256, 2049, (batch,), device=dev)
    labels[torch.arange(seq, device=dev).unsqueeze(0) < prompt.unsqueeze(1)] = -100
    n_eff = int((labels[:, 1:] != -100).sum().item())
    probe = KernelProbe(oi, 2)

    def step():
        hidden.grad = None
        weight.grad = None
        with probe:
            loss = oi.fused_linear_cross_entropy(hidden, weight, labels, token_slabs=True)
        loss.backward()
        return loss

    flops_fwd = 2.0 * n_eff * hdim * vocab
    info = {
        "tokens": batch * seq,
        "rows_multiplied": n_eff,
        "hdim": hdim,
        "vocab": vocab,
        "flops_step": 3.0 * flops_fwd,
        "kernel": ("gemm_store_kernel<true, true> (d_weight product of a slab of selected tokens, added to the fp32 d_weight; "
                   "timed launch by launch through the library's event probe)"),
        "alg_per_launch": None,
        "bound": "mfma",
        "timer": probe,
    }
    return step, info


def _pack_case(n=512, max_q=512, max_r=3584, pad=0, seed=0):
    import random

    rng = random.Random(seed)
    queries = [[rng.randrange(1, 50000) for _ in range(rng.randrange(1, max_q + 1))] for _ in range(n)]
    responses = [[rng.randrange(1, 50000) for _ in range(rng.randrange(1, max_r + 1))] for _ in range(n)]
    masks = [[1] * len(r) for r in responses]
    lps = [[-rng.random()] * len(r) for r in responses]
    adv = [rng.gauss(0, 1) for _ in range(n)]
    return queries, responses, masks, lps, adv


def make_pack(torch, oi):
    """Packing of 512 query/response pairs (about a million tokens) into rows of 35840 tokens plus the
    advantage broadcast: the step is the whole call (list flattening on the host, upload, one kernel)."""
    queries, responses, masks, lps, adv = _pack_case()
    n_tokens = sum(len(q) + len(r) for q, r in zip(queries, responses))
    timer = EventTimer(torch)
    plain_call = oi._lib.call

    def timed_call(name, *args):
        if name != "oi_pack_sequences":
            return plain_call(name, *args)
        with timer:
            return plain_call(name, *args)

    oi._lib.call = timed_call

    def step():
        packed = oi.rl_utils.pack_sequences(queries, responses, masks, 35840, 0, lps, advantages=adv, device="cuda:0")
        return packed.advantages[0].sum()

    # per token: read id 8 B + logprob 4 B (+ 1 B tool mask, not read here), write 5 x 8 B + 2 x 4 B
    info = {
        "tokens": n_tokens,
        "rows_multiplied": n_tokens,
        "bytes_step": 60.0 * n_tokens,
        "kernel": "pack_scatter_kernel (one workgroup per sequence, seven per-token outputs)",
        "alg_per_launch": 60.0 * n_tokens,
        "bound": "hbm",
        "timer": timer,
    }
    return step, info


# ------------------------------------------------------------------------------------------------
# CPU baseline: the oracle's restatement of the reference path on a bounded sample
# ------------------------------------------------------------------------------------------------
def cpu_baseline(torch, workload):
    from oracle import grpo as o_grpo
    from oracle import logprob as o_lp
    from oracle import reductions as o_red

    threads = torch.get_num_threads()
    cfg = _cfg()
    torch.manual_seed(0)
    workload = {"c3-recompute": "c3", "c3-one-call-recompute": "c3", "sft": "sft", "c4-recompute": "c4", "c5-one-call": "c5", "c5-train-head": "c5t",
                "c5-train-head-recompute": "c5t"}.get(workload, workload)
    train_head = workload == "c5t"
    forward_only = workload == "ref-cache"
    workload = "c5" if train_head or forward_only else workload
    if workload == "c5":
        # one chosen / rejected pair of 2 x 1024 tokens (of the 8 pairs of 2 x 2048), prompts masked out
        from oracle import dpo as o_dpo

        hdim, vocab, per = 8192, 128256, 1024
        n = 2 * per
        hidden = torch.randn(n, hdim).bfloat16().requires_grad_(True)
        weight = (torch.randn(vocab, hdim) * 0.01).bfloat16().requires_grad_(train_head)
        labels = torch.randint(0, vocab, (2, per))
        prompt = torch.randint(64, 513, (2,))
        labels[torch.arange(per).unsqueeze(0) < prompt.unsqueeze(1)] = -100
        ref_c, ref_r = torch.randn(1) * 50 - 400, torch.randn(1) * 50 - 400

        def run():
            hidden.grad = None
            weight.grad = None
            # reference order: bf16 lm_head GEMM, fp32 log_softmax + gather of the shifted labels, per-sequence
            # sums, sigmoid DPO loss, backward to the hidden states
            with torch.set_grad_enabled(not forward_only):
                z = torch.nn.functional.linear(hidden, weight).view(2, per, vocab)
                per_token = o_lp.calculate_per_token_logps(z, labels)
                logps = o_red.get_batch_logps_padded(per_token, labels)
            if forward_only:
                return
            losses, _, _ = o_dpo.dpo_loss(logps[:1], logps[1:], ref_c, ref_r, 0.1)
            losses.mean().backward()

        if forward_only:
            sample = (f"one pair of 2 x {per} tokens (of 8 pairs of 2 x 2048) at full H={hdim}, V={vocab}, W ~ N(0, 0.01); "
                      "forward only, no gradient; bf16 GEMM + fp32 log_softmax + per-sequence sums")
        else:
            sample = (f"one pair of 2 x {per} tokens (of 8 pairs of 2 x 2048) at full H={hdim}, V={vocab}, W ~ N(0, 0.01); "
                      f"fwd + bwd to the hidden states{' and the head' if train_head else ''}; bf16 GEMM + fp32 log_softmax + "
                      "sigmoid DPO loss")
    elif workload in ("c3", "c4"):
        hdim = 4096
        vocab, n = (100352 if workload == "c4" else 128256), 2048
        hidden = torch.randn(n, hdim).bfloat16().requires_grad_(True)
        weight = (torch.randn(vocab, hdim) * 0.02).bfloat16().requires_grad_(True)
        labels = torch.randint(0, vocab, (n,))
        mask = torch.rand(n) < 0.7
        adv, noise = torch.randn(n), torch.randn(n)

        def run():
            hidden.grad = None
            weight.grad = None
            # reference order: bf16 lm_head GEMM, fp32 upcast, log_softmax + gather, entropy (no grad)
            z = torch.nn.functional.linear(hidden, weight)
            lp = o_lp.log_softmax_and_gather(z, labels, torch.float32)
            with torch.no_grad():
                o_lp.entropy_from_logits(z, torch.float32)
            old, ref = lp.detach() + 0.05 * noise, lp.detach() + 0.1 * noise
            loss, *_ = o_grpo.grpo_token_loss(lp[None], old[None], ref[None], adv[None], mask[None], cfg)
            loss.backward()

        sample = f"{n} of 32768 token rows at full H={hdim}, V={vocab}; fwd+bwd; bf16 GEMM + fp32 log_softmax"
    elif workload == "sft":
        hdim, vocab, n = 4096, 128256, 2048
        hidden = torch.randn(1, n, hdim).bfloat16().requires_grad_(True)
        weight = (torch.randn(vocab, hdim) * 0.02).bfloat16().requires_grad_(True)
        labels = torch.randint(0, vocab, (1, n))
        labels[:, : n // 4] = -100

        def run():
            hidden.grad = None
            weight.grad = None
            # the model forward's order: bf16 lm_head GEMM, fp32 upcast, shifted labels, mean cross-entropy
            z = torch.nn.functional.linear(hidden, weight).float()
            shifted = o_lp.shift_labels(labels).reshape(-1)
            torch.nn.functional.cross_entropy(z.view(-1, vocab), shifted, ignore_index=-100).backward()

        sample = (f"one sequence of {n} tokens (of 8 x 4096) at full H={hdim}, V={vocab}, a quarter of it prompt; fwd+bwd; the "
                  "causal-LM loss as the reference's model forward computes it")
    elif workload in ("c2", "c2-two-pass"):
        n, vocab = 8192, 128256
        logits = (torch.randn(n, vocab) * 3.0).bfloat16().requires_grad_(True)
        labels = torch.randint(0, vocab, (n,))
        adv, noise = torch.randn(n), torch.randn(n)
        mask = torch.ones(n, dtype=torch.bool)

        def run():
            logits.grad = None
            lp = o_lp.log_softmax_and_gather(logits, labels, None).float()  # bf16 log_softmax as the reference
            old, ref = lp.detach() + 0.05 * noise, lp.detach() + 0.1 * noise
            loss, *_ = o_grpo.grpo_token_loss(lp[None], old[None], ref[None], adv[None], mask[None], cfg)
            loss.backward()

        sample = f"{n} of 65536 rows of bf16 logits at V={vocab}; fwd+bwd"
    elif workload == "pack":
        from oracle import packing as o_pack

        queries, responses, masks, lps, adv = _pack_case()
        n = sum(len(q) + len(r) for q, r in zip(queries, responses))
        threads = 1

        def run():
            out = o_pack.pack_sequences(queries, responses, masks, 35840, 0, lps)
            o_pack.broadcast_advantages(adv, out["response_masks"])

        sample = "the full workload (512 pairs), list-based restatement of the reference loop, one thread"
    else:
        n = 2048
        logits = torch.randn(4, 512, 32000) * 2.0
        ids = torch.randint(0, 32000, (4, 512))
        mask = torch.ones(4, 512)

        def run():
            lp = o_lp.log_softmax_and_gather(logits, ids, None)
            ent = o_lp.entropy_from_logits(logits, None)
            o_red.masked_mean(lp, mask) + o_red.masked_mean(ent, mask)

        sample = "the full config-1 batch (2048 rows, V=32000, fp32)"
    scaled = {"c3": 32768, "c4": 32768, "c5": 32768, "sft": 32768, "c2": 65536, "c2-two-pass": 65536}.get(workload)
    run()  # warm-up
    times = []
    t_end = time.time() + 20.0
    while len(times) < 3 or (time.time() < t_end and len(times) < 5):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": n / med,
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": sample + f"; median of {len(times)} runs, {med:.3f} s each, torch CPU threads={threads}",
        # a row slice of the workload was timed and tokens/s taken from it (cost is linear in the rows)
        "scaled": scaled is not None,
        "row_fraction": (n / scaled) if scaled else 1.0,
        "os_cpu_count": os.cpu_count(),
        "cpu_model": _cpu_model(),
    }


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def library_gemm_tflops(torch, n, hdim, vocab):
    """bf16 GEMM ceiling of the vendor library at the forward's shape (reported next to the peak)."""
    a = torch.randn(min(n, 8192), hdim, device="cuda:0").bfloat16()
    w = (torch.randn(vocab, hdim, device="cuda:0") * 0.02).bfloat16()
    out = torch.empty(a.shape[0], vocab, device="cuda:0", dtype=torch.bfloat16)
    for _ in range(2):
        torch.matmul(a, w.t(), out=out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reps = 5
    for _ in range(reps):
        torch.matmul(a, w.t(), out=out)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    return 2.0 * a.shape[0] * hdim * vocab / dt / 1e12


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="c3",
                    choices=["c1", "c2", "c2-two-pass", "c3", "c3-recompute", "c3-one-call-recompute", "c4",
                             "c4-recompute", "c5", "c5-one-call", "c5-train-head", "c5-train-head-recompute", "ref-cache",
                             "sft", "pack"])
    ap.add_argument("--slab-tokens", type=int, default=0,
                    help="c3 / c4 / c5-train-head only: slab size of the no-recompute step (0 = the package's default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--one-kernel", action="store_true",
                    help="time only the dominant kernel of a slab-wise call, not the other two tile kernels over extra steps "
                         "(for profiler runs, whose traces should hold the warm-up and timed steps only)")
    ap.add_argument("--no-library-gemm", action="store_true",
                    help="skip the reference points beside the measurement: the vendor bf16 GEMM of the same shape and, "
                         "for c3, the timing of the recomputing route")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy (reference point for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures the one-GPU hot path only: run it with --gpus 1 (no multi-GPU figure exists).")
        sys.exit(2)

    import torch

    import open_instruct_amd as oi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (the package has no CPU path).")
        sys.exit(2)
    oi._lib.load()

    if args.slab_tokens:
        oi.grpo_utils.DEFAULT_SLAB_TOKENS = args.slab_tokens
        oi.dpo_utils.DEFAULT_DPO_SLAB_TOKENS = args.slab_tokens
    slab_note = f"slabs of at most {oi.grpo_utils.DEFAULT_SLAB_TOKENS} selected tokens, nothing recomputed, no [tokens, vocab] tensor"
    if args.workload == "c3":
        step, info = make_fused(torch, oi, 32768, 4096, 128256, 0.02)
        name = ("c3: fused lm_head+logprob+entropy+GRPO loss fwd+bwd, hidden bf16 [32768,4096], W bf16 [128256,4096], 70% "
                f"response tokens (rows selected on the device), through grpo_loss_on_hidden as it runs by default: {slab_note}")
        dtype = "bf16"
    elif args.workload == "c3-recompute":
        step, info = make_fused(torch, oi, 32768, 4096, 128256, 0.02, route="recompute")
        name = ("c3 through the three differentiable calls fused_lm_head_logprobs -> grpo_loss_fused -> backward: the "
                "backward recomputes the logits one vocabulary chunk at a time (8 N H V executed for 6 N H V credited)")
        dtype = "bf16"
    elif args.workload == "c3-one-call-recompute":
        step, info = make_fused(torch, oi, 32768, 4096, 128256, 0.02, route="one-call-recompute")
        name = "c3 through grpo_loss_on_hidden(token_slabs=False): the recomputing step from one C call"
        dtype = "bf16"
    elif args.workload == "c4":
        step, info = make_c4(torch, oi)
        name = ("c4: packed OLMo-2-7B shape, 16 sequences via cu_seqlens, hidden bf16 [N<=32768,4096], W bf16 [100352,4096]; "
                "GRPO loss masked_mean(axis=1) fwd+bwd through grpo_loss_on_hidden as it runs by default "
                f"({slab_note}), per-sequence logprob sums from the returned logprobs")
        dtype = "bf16"
    elif args.workload == "c4-recompute":
        step, info = make_c4(torch, oi, route="recompute")
        name = ("c4 through the three differentiable calls: per-sequence logprob sums + GRPO loss masked_mean(axis=1), "
                "fwd+bwd, recomputing backward")
        dtype = "bf16"
    elif args.workload == "c5":
        step, info = make_fused(torch, oi, 32768, 8192, 128256, 0.01, dpo=True)
        name = "c5: fused lm_head+per-sequence logprob sums+sigmoid DPO loss, hidden bf16 [32768,8192], W bf16 [128256,8192], bwd to dHidden only"
        dtype = "bf16"
    elif args.workload == "ref-cache":
        step, info = make_fused(torch, oi, 32768, 8192, 128256, 0.01, dpo=True, route="forward")
        name = ("ref-cache: the forward-only pass that fills the reference-logprob cache of a DPO run at the c5 shape "
                "(hidden bf16 [32768,8192], W bf16 [128256,8192], 16 sequences): fused lm_head logprobs of the scored "
                "positions + per-sequence sums, no gradient")
        dtype = "bf16"
    elif args.workload == "c5-one-call":
        step, info = make_fused(torch, oi, 32768, 8192, 128256, 0.01, dpo=True, one_call=True)
        name = ("c5 from one call of dpo_loss_on_hidden (frozen head): sigmoid DPO loss and d_hidden, hidden bf16 [32768,8192], "
                f"W bf16 [128256,8192]; slabs of whole chosen/rejected pairs (at most {oi.dpo_utils.DEFAULT_DPO_SLAB_TOKENS} "
                "scored tokens), nothing recomputed, no fp32 sums between the passes")
        dtype = "bf16"
    elif args.workload == "c5-train-head":
        step, info = make_fused(torch, oi, 32768, 8192, 128256, 0.01, dpo=True, train_head=True)
        name = ("c5 with a trainable head: sigmoid DPO loss, d_hidden and d_weight from one call of dpo_loss_on_hidden, "
                "hidden bf16 [32768,8192], W bf16 [128256,8192]; slabs of whole chosen/rejected pairs (at most "
                f"{oi.dpo_utils.DEFAULT_DPO_SLAB_TOKENS} scored tokens), nothing recomputed")
        dtype = "bf16"
    elif args.workload == "c5-train-head-recompute":
        step, info = make_fused(torch, oi, 32768, 8192, 128256, 0.01, dpo=True, train_head=True, route="recompute")
        name = ("c5 with a trainable head through the differentiable calls (DPOLMHead's route): the backward recomputes "
                "the logits (8 N H V executed for 6 N H V credited)")
        dtype = "bf16"
    elif args.workload == "c2":
        step, info = make_c2(torch, oi)
        name = "c2: GRPO loss on materialised bf16 logits [64,1024,128256], fwd+bwd in one read + one write of the logits"
        dtype = "bf16"
    elif args.workload == "c2-two-pass":
        step, info = make_c2(torch, oi, single_pass=False)
        name = "c2: GRPO loss on materialised bf16 logits [64,1024,128256], fwd+bwd, reference order (logits read twice)"
        dtype = "bf16"
    elif args.workload == "sft":
        step, info = make_sft(torch, oi)
        name = ("sft: causal-LM cross-entropy through the fused head, hidden bf16 [8,4096,4096], W bf16 [128256,4096], "
                f"prompts ignored, fwd+bwd to dHidden and dW through fused_linear_cross_entropy(token_slabs=True): {slab_note}")
        dtype = "bf16"
    elif args.workload == "pack":
        step, info = make_pack(torch, oi)
        name = "pack: 512 query/response pairs (~1M tokens) into rows of 35840 tokens + advantage broadcast, whole call from Python lists"
        dtype = "int64"
    else:
        step, info = make_c1(torch, oi)
        name = "c1: logprob+entropy+masked_mean on fp32 logits [4,512,32000], forward"
        dtype = "f32"

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    info["timer"].reset()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    value = info["tokens"] / (elapsed / args.steps)

    kernel_ms = info["timer"].mean_ms()
    if info["alg_per_launch"] is None:  # launches of a probed kernel that had rows, per step
        probe = info["timer"]
        real = [x for x in probe.samples if x >= probe.threshold()]
        info["alg_per_launch"] = 2.0 * info["rows_multiplied"] * info["hdim"] * info["vocab"] / max(1.0, len(real) / args.steps)
    if info["bound"] == "mfma":
        achieved = info["alg_per_launch"] / (kernel_ms * 1e-3) / 1e12
        peak, unit = PEAK_BF16_TFLOPS, "TFLOP/s"
    else:
        achieved = info["alg_per_launch"] / (kernel_ms * 1e-3) / 1e9
        peak, unit = PEAK_HBM_GBS, "GB/s"
    roofline = {
        "bound": info["bound"],
        "achieved": achieved,
        "peak": peak,
        "unit": unit,
        "frac": achieved / peak,
        "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload),
        "traffic_unit": "bytes/launch",
        "kernel": info["kernel"],
        "kernel_ms": kernel_ms,
        "algorithmic_per_launch": info["alg_per_launch"],
    }
    if isinstance(info["timer"], KernelProbe) and not args.one_kernel:
        # the other tile kernels of the slab-wise call, each timed over three more steps (outside the timed region)
        probe, timed_kernel = info["timer"], info["timer"].kernel
        names = {0: "lmhead_fwd_kernel<true> (forward that keeps its exponentials)", 1: "gemm_store_kernel<false, true> (d_hidden product)",
                 2: "gemm_store_kernel<true, true> (d_weight product)"}
        per_kernel = {names[timed_kernel]: {"ms_per_launch": kernel_ms, "frac": achieved / peak}}
        for k in (0, 1, 2):
            if k == timed_kernel or (k == 2 and info["flops_step"] < 2.5 * 2.0 * info["rows_multiplied"] * info["hdim"] * info["vocab"]):
                continue
            probe.kernel = k
            probe.reset()
            for _ in range(3):
                step()
            torch.cuda.synchronize()
            real = [x for x in probe.samples if x >= probe.threshold()]
            if real:
                ms_k = sum(real) / len(real)
                alg_k = 2.0 * info["rows_multiplied"] * info["hdim"] * info["vocab"] / (len(real) / 3.0)
                per_kernel[names[k]] = {"ms_per_launch": ms_k, "frac": alg_k / (ms_k * 1e-3) / 1e12 / PEAK_BF16_TFLOPS}
        probe.kernel = timed_kernel
        roofline["tile_kernels_of_the_call"] = per_kernel
    if "flops_step" in info:
        roofline["whole_step_tflops"] = info["flops_step"] / (ms_per_step * 1e-3) / 1e12
        roofline["whole_step_frac"] = roofline["whole_step_tflops"] / PEAK_BF16_TFLOPS
        if not args.no_library_gemm:
            hdim = 8192 if args.workload.startswith("c5") or args.workload == "ref-cache" else 4096
            vocab = 100352 if args.workload in ("c4", "c4-recompute") else 128256
            roofline["library_bf16_gemm_tflops"] = library_gemm_tflops(torch, 32768, hdim, vocab)
    if "bytes_step" in info:
        roofline["whole_step_gbs"] = info["bytes_step"] / (ms_per_step * 1e-3) / 1e9
        roofline["whole_step_frac"] = roofline["whole_step_gbs"] / PEAK_HBM_GBS

    line = {
        "metric": "tokens/s fused lm_head+logprob+GRPO loss fwd+bwd, V=128k; % MFMA/HBM peak",
        "value": value,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": {
            "workload": name,
            "tokens_per_step": info["tokens"],
            "rows_multiplied": info["rows_multiplied"],
            "loss_value": float(loss.item()) if math.isfinite(float(loss.item())) else None,
        },
        "roofline": roofline,
    }
    if args.workload == "c3" and not args.no_library_gemm:
        # reported beside the headline figure: the same step through the three differentiable calls, whose
        # backward recomputes the logits (what a caller gets who needs the autograd seam between forward and loss)
        del step
        torch.cuda.empty_cache()
        step_r, info_r = make_fused(torch, oi, 32768, 4096, 128256, 0.02, route="recompute")
        for _ in range(args.warmup):
            step_r()
        torch.cuda.synchronize()
        info_r["timer"].reset()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step_r()
        torch.cuda.synchronize()
        ms_r = (time.perf_counter() - t0) * 1e3 / args.steps
        fwd_ms = info_r["timer"].mean_ms()
        line["other_routes"] = {
            "recompute_three_calls": {
                "ms_per_step": ms_r,
                "tokens_per_s": info_r["tokens"] / (ms_r * 1e-3),
                "whole_step_frac": info_r["flops_step"] / (ms_r * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                "forward_kernel_ms": fwd_ms,
                "forward_kernel_frac": info_r["alg_per_launch"] / (fwd_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                "note": "fused_lm_head_logprobs -> grpo_loss_fused -> backward: the backward recomputes the logits "
                        "(8 N H V executed, 6 N H V credited)",
            }
        }
        del step_r
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(torch, args.workload)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
