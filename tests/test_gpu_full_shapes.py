"""The benchmark configurations at their stated shapes, each run once exactly as ``bench.py`` runs it
and compared with the CPU oracle on a sample that the oracle finishes in seconds:

* fused lm_head configs (Llama-3.1-8B head with GRPO, packed OLMo-2-7B head with GRPO, Llama-3.1-70B
  head with DPO): about 200 token rows for logprob / entropy / dHidden (fp32 ``F.linear`` of those rows
  against all of ``W`` on the host) and 64 vocabulary rows of ``dW`` (``dZ[:, v] = g/T (1[v = y] -
  exp(z_v/T - lse))`` with ``z_v`` from an fp32 product on the host and ``lse`` from a chunked fp32
  ``torch`` matmul on the GPU, i.e. a library path).  The samples contain the first and the last
  tile, every vocabulary-chunk boundary of the backward pass, rows left out by the mask and
  vocabulary rows that are some token's label.  The upstream gradient ``g`` of every token comes from
  autograd on the oracle's loss chain.
* GRPO on the full ``[64, 1024, 128256]`` bf16 logits tensor (element offsets beyond 2^32) through
  the single-launch path and through the two-pass kernels, rows 0 / 33792 / 65535 and a few more
  against the oracle.
* the single-launch kernel against the oracle at the full vocabulary (part of every row waits in the
  LDS, the rest is read twice).

Tolerance 2e-3 abs for values (bf16 inputs, fp32 accumulation).  Gradients at these shapes are of the
order of 1e-6 (the loss is a mean over tens of thousands of tokens), so they are also held to a
relative bound: 2 % of the norm of the compared block, which is what bf16 storage of ``dZ`` and of the
results allows.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from conftest import make_grpo_config

from open_instruct_amd import dpo_utils, grpo_utils, lm_head, model_utils, padding_free_collator
from oracle import dpo as o_dpo
from oracle import grpo as o_grpo
from oracle import logprob as o_logprob
from oracle import reductions as o_red

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3
REL = 2e-2
BWD_CHUNK = 32768  # vocabulary columns per chunk of the backward pass


def _cfg():
    return make_grpo_config(loss_fn="dapo", clip_lower=0.2, clip_higher=0.28, beta=0.05, kl_estimator=2)


def _rel(got: torch.Tensor, exp: torch.Tensor) -> float:
    return ((got.double() - exp.double()).norm() / exp.double().norm().clamp(min=1e-30)).item()


def _token_sample(n: int, mask: torch.Tensor, count: int, gen: torch.Generator) -> torch.Tensor:
    """Token rows: both ends, a few rows left out by the mask, random ones."""
    fixed = [0, 1, 255, 256, 257, n - 257, n - 256, n - 2, n - 1]
    off = torch.nonzero(~mask.cpu()).flatten()[:8].tolist()
    rnd = torch.randint(0, n, (count,), generator=gen).tolist()
    return torch.tensor(sorted(set(i for i in fixed + off + rnd if 0 <= i < n)))


def _vocab_sample(v: int, labels_kept: torch.Tensor, gen: torch.Generator) -> torch.Tensor:
    """Vocabulary rows: first and last tile, both sides of every backward chunk boundary, rows that
    are some kept token's label, random ones."""
    fixed = [0, 1, 255, 256, v - 256, v - 2, v - 1]
    for edge in range(BWD_CHUNK, v, BWD_CHUNK):
        fixed += [edge - 1, edge, edge + 255, edge + 256]
    hit = labels_kept.cpu()[torch.randperm(labels_kept.numel(), generator=gen)[:16]].tolist()
    rnd = torch.randint(0, v, (64,), generator=gen).tolist()
    picked = sorted(set(i for i in fixed + hit + rnd if 0 <= i < v))
    return torch.tensor(picked[:96])


def _library_lse(hidden: torch.Tensor, weight: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    """logsumexp of the fp32 logits of ``rows`` through torch's own matmul on the GPU, in row chunks."""
    w32 = weight.float()
    out = []
    for s in range(0, rows.numel(), 2048):
        z = hidden[rows[s : s + 2048]].float() @ w32.t()
        out.append(torch.logsumexp(z, dim=-1))
        del z
    return torch.cat(out)


def _check_fused_head(hidden, weight, labels_eff, mask, g_cpu, lp, ent, d_hidden, d_weight, seed):
    """Sampled comparison of a fused-head forward + backward with the oracle.

    ``labels_eff`` are the labels the head scored (already shifted where the caller shifts),
    ``g_cpu`` the upstream gradient d loss / d logprob of every token (zero off the mask)."""
    gen = torch.Generator().manual_seed(seed)
    n, h = hidden.shape
    v = weight.shape[0]
    mask_c = mask.cpu()
    rows = _token_sample(n, mask_c, 200, gen)
    w_cpu = weight.detach().cpu().float()
    hs = hidden.detach()[rows.to(DEV)].cpu().float().requires_grad_(True)
    safe = labels_eff.cpu()[rows].clamp(min=0)
    z = F.linear(hs, w_cpu)
    lp_o = o_logprob.log_softmax_and_gather(z, safe, None)
    ent_o = o_logprob.entropy_from_logits(z.detach(), None)
    (lp_o * g_cpu[rows]).sum().backward()
    m = mask_c[rows]
    got_lp, got_ent = lp.detach().cpu()[rows], (ent.detach().cpu()[rows] if ent is not None else None)
    assert (got_lp[m] - lp_o.detach()[m]).abs().max().item() <= TOL
    assert (got_lp[~m] == 0).all()
    if got_ent is not None:
        assert (got_ent[m] - ent_o[m]).abs().max().item() <= TOL
    got_dh = d_hidden.detach()[rows.to(DEV)].float().cpu()
    assert (got_dh - hs.grad).abs().max().item() <= TOL
    assert (got_dh[~m] == 0).all()
    assert _rel(got_dh[m], hs.grad[m]) <= REL, _rel(got_dh[m], hs.grad[m])
    # every kept row on its own: no row may hide behind the others
    per_row = (got_dh[m] - hs.grad[m]).norm(dim=1) / hs.grad[m].norm(dim=1).clamp(min=1e-30)
    live = g_cpu[rows][m] != 0
    assert (per_row[live] <= 2 * REL).all(), per_row[live].max().item()
    del z, w_cpu

    if d_weight is None:
        return
    kept = torch.nonzero(mask).flatten()
    vs = _vocab_sample(v, labels_eff[kept].clamp(min=0), gen)
    lse = _library_lse(hidden.detach(), weight.detach(), kept).cpu()
    hk = hidden.detach()[kept].cpu().float()
    zv = hk @ weight.detach()[vs.to(DEV)].cpu().float().t()  # [kept, |vs|]
    yk = labels_eff[kept].clamp(min=0).cpu()
    onehot = (yk.unsqueeze(1) == vs.unsqueeze(0)).float()
    dz = g_cpu[kept.cpu()].unsqueeze(1) * (onehot - torch.exp(zv - lse.unsqueeze(1)))
    dw_o = dz.t() @ hk  # [|vs|, H]
    got_dw = d_weight.detach()[vs.to(DEV)].float().cpu()
    assert (got_dw - dw_o).abs().max().item() <= TOL
    assert _rel(got_dw, dw_o) <= REL, _rel(got_dw, dw_o)
    per_v = (got_dw - dw_o).norm(dim=1) / dw_o.norm(dim=1).clamp(min=1e-30)
    assert (per_v <= 2 * REL).all(), per_v.max().item()


def test_c3_llama8b_head_grpo_in_token_slabs_full_shape():
    """The c3 step through grpo_loss_on_hidden (the benchmark's default step): three equal slabs of
    selected rows, nothing recomputed, d_weight accumulated in fp32 over the slabs."""
    print("case c3 token slabs N=32768 H=4096 V=128256", flush=True)
    torch.manual_seed(0)
    n, h, v = 32768, 4096, 128256
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (n,), device=DEV)
    mask = torch.rand(n, device=DEV) < 0.7
    adv = torch.randn(n, device=DEV)
    cfg = _cfg()
    with torch.no_grad():
        lp0, _ = lm_head.fused_lm_head_logprobs(hidden, weight, labels, mask=mask)
    old = lp0 + 0.05 * torch.randn(n, device=DEV)
    ref = lp0 + 0.1 * torch.randn(n, device=DEV)
    loss, stats, lp, ent = grpo_utils.grpo_loss_on_hidden(
        hidden[None], weight, labels[None], old[None], ref[None], adv[None], mask[None], cfg
    )
    loss.backward()
    torch.cuda.synchronize()
    lp, ent = lp[0], ent[0]
    assert (lp - lp0).abs().max().item() <= 1e-5
    lp_leaf = lp.detach().cpu().requires_grad_(True)
    loss_o, *_ = o_grpo.grpo_token_loss(
        lp_leaf[None], old.cpu()[None], ref.cpu()[None], adv.cpu()[None], mask.cpu()[None].float(), cfg
    )
    loss_o.backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    assert int(stats["num_response_tokens"].item()) == int(mask.sum().item())
    _check_fused_head(hidden, weight, labels, mask, lp_leaf.grad, lp, ent, hidden.grad, weight.grad, seed=5)


def test_qwen25_7b_head_grpo_in_token_slabs_full_shape():
    """A head shape outside the benchmark list, from a model family the reference trains
    (Qwen2.5-7B: H = 3584, V = 152064 with 151665 used ids; here V = 151665, which is not a multiple of
    the 256-row vocabulary tile, so the last tile of every slab's exponentials is partly padding) at
    temperature 0.7, through grpo_loss_on_hidden in three slabs of 4096 selected rows."""
    print("case qwen2.5-7b head, token slabs, N=16384 H=3584 V=151665 T=0.7", flush=True)
    torch.manual_seed(4)
    n, h, v, temperature = 16384, 3584, 151665, 0.7
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (n,), device=DEV)
    labels[:64] = v - 1 - torch.arange(64, device=DEV)  # labels inside the partly filled last tile
    mask = torch.rand(n, device=DEV) < 0.7
    adv = torch.randn(n, device=DEV)
    cfg = _cfg()
    with torch.no_grad():
        lp0, _ = lm_head.fused_lm_head_logprobs(hidden, weight, labels, temperature=temperature, mask=mask)
    old = lp0 + 0.05 * torch.randn(n, device=DEV)
    ref = lp0 + 0.1 * torch.randn(n, device=DEV)
    loss, stats, lp, ent = grpo_utils.grpo_loss_on_hidden(
        hidden[None], weight, labels[None], old[None], ref[None], adv[None], mask[None], cfg,
        temperature=temperature, token_slabs=4096,
    )  # fmt: skip
    loss.backward()
    torch.cuda.synchronize()
    lp, ent = lp[0], ent[0]
    assert (lp - lp0).abs().max().item() <= 1e-5
    lp_leaf = lp.detach().cpu().requires_grad_(True)
    loss_o, *_ = o_grpo.grpo_token_loss(
        lp_leaf[None], old.cpu()[None], ref.cpu()[None], adv.cpu()[None], mask.cpu()[None].float(), cfg
    )
    loss_o.backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    assert int(stats["num_response_tokens"].item()) == int(mask.sum().item())
    # the oracle at temperature T is the oracle at temperature 1 on weights W / T
    # (d_weight by the chain rule through the scaled weights: d/dW = (d/d(W/T)) / T)
    scaled = weight.detach().float() / temperature
    _check_fused_head(hidden, scaled, labels, mask, lp_leaf.grad, lp, ent, hidden.grad, weight.grad.float() * temperature, seed=9)


def test_token_slabs_with_a_small_remainder_slab():
    """8500 selected rows at H = 4096 with slabs of at most 8192: two equal slabs of 4250 rows would take
    four rounds of tiles in their d_hidden products, 8192 + 308 takes three, so the device-side plan picks
    a full slab and a small remainder (whose d_weight product adds 308 rows' worth to the fp32 sum and
    rounds it).  Sampled oracle check like the benchmark shapes, on a small vocabulary."""
    print("case 8500 selected rows, H=4096 V=5000, slabs 8192 + 308", flush=True)
    torch.manual_seed(6)
    n, h, v = 9000, 4096, 5000
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (n,), device=DEV)
    mask = torch.zeros(n, dtype=torch.bool, device=DEV)
    mask[torch.randperm(n, device=DEV)[:8500]] = True
    adv = torch.randn(n, device=DEV)
    cfg = _cfg()
    with torch.no_grad():
        lp0, _ = lm_head.fused_lm_head_logprobs(hidden, weight, labels, mask=mask)
    old = lp0 + 0.05 * torch.randn(n, device=DEV)
    ref = lp0 + 0.1 * torch.randn(n, device=DEV)
    loss, stats, lp, ent = grpo_utils.grpo_loss_on_hidden(
        hidden[None], weight, labels[None], old[None], ref[None], adv[None], mask[None], cfg, token_slabs=8192
    )
    loss.backward()
    torch.cuda.synchronize()
    lp, ent = lp[0], ent[0]
    assert (lp - lp0).abs().max().item() <= 1e-5
    lp_leaf = lp.detach().cpu().requires_grad_(True)
    loss_o, *_ = o_grpo.grpo_token_loss(
        lp_leaf[None], old.cpu()[None], ref.cpu()[None], adv.cpu()[None], mask.cpu()[None].float(), cfg
    )
    loss_o.backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    assert int(stats["num_response_tokens"].item()) == 8500
    _check_fused_head(hidden, weight, labels, mask, lp_leaf.grad, lp, ent, hidden.grad, weight.grad, seed=11)
    # the recomputing form of the same step agrees (different summation order: bf16 rounding of the results)
    h2 = hidden.detach().clone().requires_grad_(True)
    w2 = weight.detach().clone().requires_grad_(True)
    loss2, _, lp2, _ = grpo_utils.grpo_loss_on_hidden(
        h2[None], w2, labels[None], old[None], ref[None], adv[None], mask[None], cfg, token_slabs=False
    )
    loss2.backward()
    assert (lp2[0] - lp).abs().max().item() <= 1e-5
    assert _rel(hidden.grad.float(), h2.grad.float()) <= REL and _rel(weight.grad.float(), w2.grad.float()) <= REL


def test_c3_llama8b_head_grpo_full_shape():
    """hidden bf16 [32768, 4096], W bf16 [128256, 4096], 70 % response rows: fused lm_head + logprob +
    entropy + GRPO loss, forward and backward to dHidden and dW, through the three differentiable
    calls whose backward recomputes every vocabulary chunk (the benchmark's `c3-recompute` step)."""
    print("case c3 N=32768 H=4096 V=128256 three calls, recomputing backward", flush=True)
    torch.manual_seed(0)
    n, h, v = 32768, 4096, 128256
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (n,), device=DEV)
    mask = torch.rand(n, device=DEV) < 0.7
    adv = torch.randn(n, device=DEV)
    cfg = _cfg()
    with torch.no_grad():
        lp0, _ = lm_head.fused_lm_head_logprobs(hidden, weight, labels, mask=mask)
    old = lp0 + 0.05 * torch.randn(n, device=DEV)
    ref = lp0 + 0.1 * torch.randn(n, device=DEV)

    lp, ent = lm_head.fused_lm_head_logprobs(hidden, weight, labels, mask=mask, return_entropy=True)
    loss, stats = grpo_utils.grpo_loss_fused(lp[None], old[None], ref[None], adv[None], mask[None], cfg, entropy=ent[None])
    loss.backward()
    torch.cuda.synchronize()
    assert torch.equal(lp.detach(), lp0)  # deterministic, run to run

    # loss and upstream gradient of every token from the oracle's loss chain on the kernel's logprobs
    lp_leaf = lp.detach().cpu().requires_grad_(True)
    loss_o, *_ = o_grpo.grpo_token_loss(
        lp_leaf[None], old.cpu()[None], ref.cpu()[None], adv.cpu()[None], mask.cpu()[None].float(), cfg
    )
    loss_o.backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    assert int(stats["num_response_tokens"].item()) == int(mask.sum().item())
    _check_fused_head(hidden, weight, labels, mask, lp_leaf.grad, lp, ent, hidden.grad, weight.grad, seed=3)


def test_c4_packed_olmo2_head_grpo_full_shape():
    """16 sequences packed through cu_seqlens into at most 32768 tokens, H = 4096, V = 100352 (three
    backward chunks of 32768 columns and one of 2048): per-sequence summed logprobs and the GRPO loss
    with masked_mean(axis=1), forward and backward."""
    print("case c4 packed H=4096 V=100352", flush=True)
    torch.manual_seed(0)
    h, v, budget = 4096, 100352, 32768
    lens = torch.randint(128, 4097, (16,)).tolist()
    kept_lens, total = [], 0
    for ln in lens:
        ln = min(ln, budget - total)
        if ln <= 1:
            break
        kept_lens.append(ln)
        total += ln
    cu = torch.tensor([0] + list(torch.tensor(kept_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    n = total
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (1, n), device=DEV)
    labels[0, cu[:-1].long()] = -100
    shifted = padding_free_collator.shift_labels(labels)
    mask = (shifted != -100).view(-1)
    adv = torch.randn(n, device=DEV)
    cfg = _cfg()
    with torch.no_grad():
        lp0, _ = lm_head.fused_lm_head_logprobs(hidden, weight, shifted.view(-1), mask=mask)
    old = lp0 + 0.05 * torch.randn(n, device=DEV)
    ref = lp0 + 0.1 * torch.randn(n, device=DEV)

    lp, ent = lm_head.fused_lm_head_logprobs(hidden, weight, shifted.view(-1), mask=mask, return_entropy=True)
    seq = padding_free_collator.get_batch_logps(lp.view(1, -1), labels, cu)
    loss, _ = grpo_utils.grpo_loss_fused(
        lp[None], old[None], ref[None], adv[None], mask[None], cfg, entropy=ent[None], axis=1
    )
    (loss + 1e-3 * seq.mean()).backward()
    torch.cuda.synchronize()

    lp_leaf = lp.detach().cpu().requires_grad_(True)
    seq_o = o_red.get_batch_logps_packed(lp_leaf[None], labels.cpu(), cu.cpu())
    loss_o, *_ = o_grpo.grpo_token_loss(
        lp_leaf[None], old.cpu()[None], ref.cpu()[None], adv.cpu()[None], mask.cpu()[None].float(), cfg, axis=1
    )
    (loss_o + 1e-3 * seq_o.mean()).backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    # sums of up to 4096 logprobs of size ~12: fp32 summation order
    assert (seq.detach().cpu() - seq_o.detach()).abs().max().item() <= 1e-5 * seq_o.detach().abs().max().item()
    _check_fused_head(hidden, weight, shifted.view(-1), mask, lp_leaf.grad, lp, ent, hidden.grad, weight.grad, seed=4)


def test_c4_packed_olmo2_head_grpo_in_token_slabs_full_shape():
    """The packed OLMo-2 shape through grpo_loss_on_hidden(axis=1), as the benchmark's `c4` workload runs
    it: the GRPO loss with masked_mean(axis=1) over the one packed row and both gradients from the
    slab-wise call, the per-sequence sums from the logprobs it returns."""
    print("case c4 packed H=4096 V=100352 token slabs", flush=True)
    torch.manual_seed(0)
    h, v, budget = 4096, 100352, 32768
    lens = torch.randint(128, 4097, (16,)).tolist()
    kept_lens, total = [], 0
    for ln in lens:
        ln = min(ln, budget - total)
        if ln <= 1:
            break
        kept_lens.append(ln)
        total += ln
    cu = torch.tensor([0] + list(torch.tensor(kept_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    n = total
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (1, n), device=DEV)
    labels[0, cu[:-1].long()] = -100
    shifted = padding_free_collator.shift_labels(labels)
    mask = (shifted != -100).view(-1)
    adv = torch.randn(n, device=DEV)
    cfg = _cfg()
    with torch.no_grad():
        lp0, _ = lm_head.fused_lm_head_logprobs(hidden, weight, shifted.view(-1), mask=mask)
    old = lp0 + 0.05 * torch.randn(n, device=DEV)
    ref = lp0 + 0.1 * torch.randn(n, device=DEV)

    loss, _, lp, ent = grpo_utils.grpo_loss_on_hidden(
        hidden[None], weight, shifted, old[None], ref[None], adv[None], mask[None], cfg, axis=1
    )
    seq = padding_free_collator.get_batch_logps(lp.view(1, -1), labels, cu)
    loss.backward()
    torch.cuda.synchronize()
    lp, ent = lp[0], ent[0]
    assert (lp - lp0).abs().max().item() <= 1e-5

    lp_leaf = lp.detach().cpu().requires_grad_(True)
    seq_o = o_red.get_batch_logps_packed(lp_leaf[None], labels.cpu(), cu.cpu())
    loss_o, *_ = o_grpo.grpo_token_loss(
        lp_leaf[None], old.cpu()[None], ref.cpu()[None], adv.cpu()[None], mask.cpu()[None].float(), cfg, axis=1
    )
    loss_o.backward()
    assert abs(loss.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    assert (seq.detach().cpu() - seq_o.detach()).abs().max().item() <= 1e-5 * seq_o.detach().abs().max().item()
    _check_fused_head(hidden, weight, shifted.view(-1), mask, lp_leaf.grad, lp, ent, hidden.grad, weight.grad, seed=6)


def test_c1_plumbing_chain_at_the_stated_config():
    """fp32 logits [4, 512, 32000] ~ N(0, 2), uniform target ids, a response mask of the last L_b
    positions of every row with L_b uniform in 64..512, seed 0: log_softmax_and_gather and
    entropy_from_logits, then masked_mean of both (open_instruct/model_utils.py:587-600, :326-333,
    open_instruct/rl_utils.py:426-448), every number against the oracle to 1e-5."""
    torch.manual_seed(0)
    b, t, v = 4, 512, 32000
    logits = torch.randn(b, t, v) * 2.0
    ids = torch.randint(0, v, (b, t))
    lengths = torch.randint(64, 513, (b,))
    mask = torch.arange(t).unsqueeze(0) >= (t - lengths).unsqueeze(1)
    assert mask.sum(1).tolist() == lengths.tolist()
    lp_o = o_logprob.log_softmax_and_gather(logits, ids)
    ent_o = o_logprob.entropy_from_logits(logits)
    d = lambda x: x.to(DEV)  # noqa: E731
    lp = model_utils.log_softmax_and_gather(d(logits), d(ids))
    ent = model_utils.entropy_from_logits(d(logits))
    assert lp.dtype == torch.float32 and lp.shape == (b, t)
    assert (lp.cpu() - lp_o).abs().max().item() <= 1e-5 and (ent.cpu() - ent_o).abs().max().item() <= 1e-5
    from open_instruct_amd import rl_utils

    for axis in (None, 1):
        for got_t, exp_t in ((lp, lp_o), (ent, ent_o)):
            got = rl_utils.masked_mean(got_t, d(mask), axis=axis)
            exp = o_red.masked_mean(exp_t, mask.float(), axis=axis)
            assert abs(got.item() - exp.item()) <= 1e-5, (axis, got.item(), exp.item())
    # the one-pass form used by the benchmark gives the same numbers
    lp2, ent2 = model_utils.logprob_and_entropy(d(logits), d(ids))
    assert torch.equal(lp2, lp) and (ent2 - ent).abs().max().item() <= 1e-6


@pytest.mark.parametrize("dhidden_in_forward", [True, False])
def test_c5_llama70b_head_dpo_full_shape(dhidden_in_forward):
    """8 chosen / rejected pairs of 2048 tokens with the prompt (128..1024 tokens) masked out, hidden
    bf16 [32768, 8192] (128 k-tiles), W bf16 [128256, 8192] frozen: per-sequence sums, sigmoid DPO loss
    (beta 0.1), backward to dHidden only; with d_hidden prepared in the forward (the default for a
    frozen head) and with the recomputing backward."""
    print(f"case c5 N=32768 H=8192 V=128256 d_hidden in forward={dhidden_in_forward}", flush=True)
    torch.manual_seed(0)
    n, h, v, per = 32768, 8192, 128256, 2048
    seqs = n // per
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.01).bfloat16()
    labels = torch.randint(0, v, (seqs, per), device=DEV)
    prompt = torch.randint(128, 1025, (seqs,), device=DEV)
    pos = torch.arange(per, device=DEV).unsqueeze(0).expand(seqs, per)
    labels[pos < prompt.unsqueeze(1)] = -100
    labels = labels.view(1, -1)
    cu = torch.arange(0, n + 1, per, device=DEV, dtype=torch.int32)
    shifted = padding_free_collator.shift_labels(labels)
    mask = (shifted != -100).view(-1)
    ref_c = torch.randn(seqs // 2, device=DEV) * 50 - 400
    ref_r = torch.randn(seqs // 2, device=DEV) * 50 - 400

    lp, _ = lm_head.fused_lm_head_logprobs(
        hidden, weight, shifted.view(-1), mask=mask, dhidden_in_forward=dhidden_in_forward
    )
    logps = padding_free_collator.get_batch_logps(lp.view(1, -1), labels, cu)
    bs = logps.shape[0] // 2
    losses, cr, rr = dpo_utils.dpo_loss(logps[:bs], logps[bs:], ref_c, ref_r, beta=0.1)
    losses.mean().backward()
    torch.cuda.synchronize()

    lp_leaf = lp.detach().cpu().requires_grad_(True)
    logps_o = o_red.get_batch_logps_packed(lp_leaf[None], labels.cpu(), cu.cpu())
    losses_o, cr_o, rr_o = o_dpo.dpo_loss(logps_o[:bs], logps_o[bs:], ref_c.cpu(), ref_r.cpu(), 0.1)
    losses_o.mean().backward()
    # per-sequence sums of ~1500 logprobs of size ~12 (|sum| ~ 2e4): fp32 summation order
    assert (logps.detach().cpu() - logps_o.detach()).abs().max().item() <= 1e-5 * logps_o.detach().abs().max().item()
    assert (losses.detach().cpu() - losses_o.detach()).abs().max().item() <= 1e-2  # beta * error of x
    assert (cr.cpu() - cr_o).abs().max().item() <= 1e-2 and (rr.cpu() - rr_o).abs().max().item() <= 1e-2
    _check_fused_head(hidden, weight, shifted.view(-1), mask, lp_leaf.grad, lp, None, hidden.grad, None, seed=5)


@pytest.mark.parametrize("average_log_prob", [False, True])
def test_c5_llama70b_head_dpo_with_trainable_head_full_shape(average_log_prob):
    """The c5 batch with a trainable head, as the reference's DPO trains it
    (open_instruct/olmo_core_train_modules.py:190-207): loss, d_hidden and d_weight from one call of
    dpo_loss_on_hidden (slabs of whole pairs, nothing recomputed), sums (`dpo`) and averages (`dpo_norm`)."""
    print(f"case c5 trainable head N=32768 H=8192 V=128256 average={average_log_prob}", flush=True)
    torch.manual_seed(0)
    n, h, v, per = 32768, 8192, 128256, 2048
    seqs = n // per
    hidden = torch.randn(n, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.01).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (seqs, per), device=DEV)
    prompt = torch.randint(128, 1025, (seqs,), device=DEV)
    pos = torch.arange(per, device=DEV).unsqueeze(0).expand(seqs, per)
    labels[pos < prompt.unsqueeze(1)] = -100
    labels = labels.view(1, -1)
    cu = torch.arange(0, n + 1, per, device=DEV, dtype=torch.int32)
    shifted = padding_free_collator.shift_labels(labels)
    mask = (shifted != -100).view(-1)
    bs = seqs // 2
    scale = 1.0 / 1500 if average_log_prob else 1.0
    ref_c = (torch.randn(bs, device=DEV) * 50 - 400) * scale
    ref_r = (torch.randn(bs, device=DEV) * 50 - 400) * scale
    beta = 5.0 if average_log_prob else 0.1

    res = dpo_utils.dpo_loss_on_hidden(
        hidden[None], weight, labels, ref_c, ref_r, beta, cu_seq_lens=cu, average_log_prob=average_log_prob
    )
    res.loss.backward()
    torch.cuda.synchronize()
    lp = res.per_token_logps.view(-1)

    lp_leaf = lp.detach().cpu().requires_grad_(True)
    logps_o = o_red.get_batch_logps_packed(lp_leaf[None], labels.cpu(), cu.cpu(), average_log_prob)
    losses_o, cr_o, rr_o = o_dpo.dpo_loss(logps_o[:bs], logps_o[bs:], ref_c.cpu(), ref_r.cpu(), beta)
    losses_o.mean().backward()
    got_logps = torch.cat([res.chosen_logps, res.rejected_logps]).cpu()
    assert (got_logps - logps_o.detach()).abs().max().item() <= 1e-5 * logps_o.detach().abs().max().item()
    assert (res.losses.cpu() - losses_o.detach()).abs().max().item() <= 1e-2
    assert abs(res.loss.item() - losses_o.detach().mean().item()) <= 1e-2
    assert (res.chosen_rewards.cpu() - cr_o).abs().max().item() <= 1e-2
    _check_fused_head(hidden, weight, shifted.view(-1), mask, lp_leaf.grad, lp, None, hidden.grad, weight.grad, seed=7)


def _oracle_rows(logits, labels, rows_b, rows_t, temperature=1.0):
    """fp32 oracle logprob / entropy / softmax of single rows of a device logits tensor."""
    out = []
    for b, t in zip(rows_b, rows_t):
        z = logits[b, t].detach().float().cpu()
        y = labels[b, t].cpu()
        lp = o_logprob.log_softmax_and_gather(z[None], y[None], None, temperature)[0]
        ent = o_logprob.entropy_from_logits(z[None], None, temperature)[0]
        p = torch.softmax(z / temperature, dim=-1)
        out.append((lp, ent, p, int(y)))
    return out


def test_c2_grpo_on_logits_full_tensor():
    """bf16 logits [64, 1024, 128256] (8.4e9 elements): the single-launch path and the two-pass kernels
    over the whole tensor, a sample of rows against the oracle (first row, the first row past element
    offset 2^32, the last row, a few random ones), everything else through properties."""
    print("case c2 logits [64,1024,128256] bf16", flush=True)
    torch.manual_seed(0)
    b, t, v = 64, 1024, 128256
    logits = torch.empty(b, t, v, device=DEV, dtype=torch.bfloat16)
    for i in range(b):
        logits[i] = (torch.randn(t, v, device=DEV) * 3.0).bfloat16()
    labels = torch.randint(0, v, (b, t), device=DEV)
    rewards = (torch.rand(b, device=DEV) < 0.3).double()
    adv = grpo_utils.group_advantages(rewards, 8).unsqueeze(1).expand(b, t).contiguous()
    mask = torch.ones(b, t, dtype=torch.bool, device=DEV)
    cfg = _cfg()
    with torch.no_grad():
        lp0 = model_utils.log_softmax_and_gather(logits, labels)
    old = lp0 + 0.05 * torch.randn(b, t, device=DEV)
    ref = lp0 + 0.1 * torch.randn(b, t, device=DEV)

    one = logits.detach().requires_grad_(True)
    loss1, stats1, lp1, ent1 = grpo_utils.grpo_loss_on_logits(one, labels, old, ref, adv, mask, cfg)
    loss1.backward()
    two = logits.detach().requires_grad_(True)
    lp2 = model_utils.log_softmax_and_gather(two, labels)
    loss2, _ = grpo_utils.grpo_loss_fused(lp2, old, ref, adv, mask, cfg)
    loss2.backward()
    torch.cuda.synchronize()

    # oracle loss chain on the kernel's logprobs gives the loss and every token's upstream gradient
    lp_leaf = lp1.detach().cpu().requires_grad_(True)
    loss_o, *_ = o_grpo.grpo_token_loss(lp_leaf, old.cpu(), ref.cpu(), adv.cpu(), mask.cpu().float(), cfg)
    loss_o.backward()
    g = lp_leaf.grad
    assert abs(loss1.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    assert abs(loss2.item() - loss_o.item()) <= 1e-5 + 1e-5 * abs(loss_o.item())
    assert (lp1 - lp2.detach()).abs().max().item() <= 1e-5
    assert int(stats1["num_response_tokens"].item()) == b * t

    gen = torch.Generator().manual_seed(2)
    rows_b = [0, 33, 63] + torch.randint(0, b, (5,), generator=gen).tolist()
    rows_t = [0, 0, 1023] + torch.randint(0, t, (5,), generator=gen).tolist()
    assert 33 * t * v > 2**32  # row (33, 0) starts beyond the 32-bit element range
    for (bi, ti), (lp_o, ent_o, p, y) in zip(zip(rows_b, rows_t), _oracle_rows(logits, labels, rows_b, rows_t)):
        assert abs(lp1[bi, ti].item() - lp_o.item()) <= TOL and abs(lp2[bi, ti].item() - lp_o.item()) <= TOL
        assert abs(ent1[bi, ti].item() - ent_o.item()) <= TOL
        onehot = torch.zeros(v)
        onehot[y] = 1.0
        exp_row = g[bi, ti] * (onehot - p)
        for grad in (one.grad, two.grad):
            got = grad[bi, ti].float().cpu()
            assert (got - exp_row).abs().max().item() <= TOL
            if g[bi, ti] != 0:
                assert _rel(got, exp_row) <= REL, (bi, ti, _rel(got, exp_row))
            else:
                assert (got == 0).all()
    # whole-tensor properties: both paths agree row by row, every gradient row sums to ~0
    for i in range(0, b, 8):
        ga, gc = one.grad[i].float(), two.grad[i].float()
        assert (ga - gc).abs().max().item() <= 2.0**-7 * max(gc.abs().max().item(), 1e-12)
        row_sum, row_abs = ga.sum(-1).abs(), ga.abs().sum(-1)
        assert (row_sum <= 2e-2 * row_abs + 1e-12).all()


@pytest.mark.parametrize("loss_fn", ["dapo", "cispo"])
def test_grpo_on_logits_full_vocabulary_against_oracle(loss_fn):
    """V = 128256 bf16: more than half of every row waits in the LDS between the statistics pass and the
    gradient pass, the rest is read a second time; logprob, entropy, loss and the whole gradient
    against the oracle's autograd (open_instruct/grpo_utils.py:541-574 -> :504-538 ->
    open_instruct/grpo_fast.py:702-724)."""
    g = torch.Generator().manual_seed(43)
    b, t, v = 2, 48, 128256
    logits = (torch.randn(b, t + 1, v, generator=g) * 3.0).bfloat16()
    labels = torch.randint(0, v, (b, t), generator=g)
    labels[0, 0], labels[0, 1], labels[1, 0] = 0, v - 1, 9216 * 8  # ends of the row, first element past the LDS part
    adv = torch.randn(b, t, generator=g)
    mask = torch.rand(b, t, generator=g) > 0.25
    rho = torch.rand(b, t, generator=g) + 0.5
    cfg = make_grpo_config(loss_fn=loss_fn, beta=0.05, kl_estimator=2, clip_higher=0.28)
    temperature = 0.8
    ref_in = logits.float().clone().requires_grad_(True)
    lp_o = o_logprob.log_softmax_and_gather(ref_in[:, :-1], labels, None, temperature)
    ent_o = o_logprob.entropy_from_logits(ref_in[:, :-1].detach(), None, temperature)
    old = lp_o.detach() + 0.05 * torch.randn(b, t, generator=g)
    ref = lp_o.detach() + 0.1 * torch.randn(b, t, generator=g)
    loss_o, *_ = o_grpo.grpo_token_loss(lp_o, old, ref, adv, mask.float(), cfg, rho_weights=rho)
    loss_o.backward()

    lg = logits.to(DEV).requires_grad_(True)
    loss, _, lp, ent = grpo_utils.grpo_loss_on_logits(
        lg, labels.to(DEV), old.to(DEV), ref.to(DEV), adv.to(DEV), mask.to(DEV), cfg, temperature=temperature,
        rho_weights=rho.to(DEV), drop_last=True,
    )  # fmt: skip
    loss.backward()
    assert (lp.cpu() - lp_o.detach()).abs().max().item() <= TOL
    assert (ent.cpu() - ent_o).abs().max().item() <= TOL
    assert abs(loss.item() - loss_o.item()) <= TOL
    got = lg.grad.float().cpu()
    assert (got - ref_in.grad).abs().max().item() <= TOL
    assert _rel(got, ref_in.grad) <= REL
    assert (got[:, -1] == 0).all() and (got[:, :-1][~mask] == 0).all()
    assert math.isfinite(loss.item())
