"""GPU parity of whole call chains of the hot path, small enough for the CPU oracle:

* packed (padding-free) batch: fused lm_head -> per-sequence sums through cu_seqlens + GRPO loss
  with a per-row masked mean, forward and backward;
* DPO: fused lm_head -> per-sequence sums -> sigmoid preference loss, backward to the hidden states;
* the plain product entry point of the MFMA tile engine;
* size-independent properties of the fused kernels at the full Llama-3.1-8B head shape.

Tolerance 2e-3 abs (bf16 inputs, fp32 accumulation) unless a test says otherwise.
"""

import math

import pytest
import torch

from conftest import make_grpo_config

from open_instruct_amd import _lib, dpo_utils, grpo_utils, lm_head, model_utils, padding_free_collator
from oracle import dpo as o_dpo
from oracle import grpo as o_grpo
from oracle import lm_head as o_lm
from oracle import logprob as o_logprob
from oracle import reductions as o_red

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3


def _bf16_tol(ref: torch.Tensor) -> float:
    """Absolute tolerance plus one bf16 rounding of the largest expected entry."""
    return TOL + ref.abs().max().item() * 2**-7


def test_packed_grpo_chain_matches_oracle():
    """Shape of open_instruct/padding_free_collator.py:202-229 callers: one packed row, ragged
    sequences, first token of each sequence never a target."""
    torch.manual_seed(5)
    h, v = 128, 3000
    lens = [37, 1, 250, 2, 129, 64]
    total = sum(lens)
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    hidden = torch.randn(total, h).bfloat16()
    weight = (torch.randn(v, h) * 2.0 / math.sqrt(h)).bfloat16()
    labels = torch.randint(0, v, (1, total))
    labels[0, cu[:-1].long()] = -100
    labels[0, 40:45] = -100  # a prompt stretch inside a sequence
    shifted = o_logprob.shift_labels(labels)
    mask = (shifted != -100).view(-1)
    adv = torch.randn(total)
    cfg = make_grpo_config(loss_fn="dapo", beta=0.05, kl_estimator=2)

    # oracle chain, fp32 on the upcast inputs
    rh = hidden.float().requires_grad_(True)
    rw = weight.float().requires_grad_(True)
    lp_o, ent_o = o_lm.lm_head_logprobs(rh, rw, shifted.view(-1), 1.0, True)
    old = (lp_o.detach() + 0.05 * torch.randn(total)) * mask
    ref = (lp_o.detach() + 0.10 * torch.randn(total)) * mask
    lp_o = lp_o * mask
    seq_o = o_red.get_batch_logps_packed(lp_o[None], labels, cu)
    loss_o, *_ = o_grpo.grpo_token_loss(lp_o[None], old[None], ref[None], adv[None], mask[None].float(), cfg, axis=1)
    (loss_o + 0.01 * seq_o.mean()).backward()

    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(True)
    lp, ent = lm_head.fused_lm_head_logprobs(dh, dw, shifted.view(-1).to(DEV), mask=mask.to(DEV), return_entropy=True)
    seq = padding_free_collator.get_batch_logps(lp.view(1, -1), labels.to(DEV), cu.to(DEV))
    loss, stats = grpo_utils.grpo_loss_fused(
        lp[None], old.to(DEV)[None], ref.to(DEV)[None], adv.to(DEV)[None], mask.to(DEV)[None], cfg,
        entropy=ent[None], axis=1,
    )  # fmt: skip
    (loss + 0.01 * seq.mean()).backward()

    assert (lp.cpu() - lp_o.detach()).abs().max().item() <= TOL
    assert ((ent.cpu() - ent_o) * mask).abs().max().item() <= TOL
    # sums over up to 250 tokens: tolerance per token times the kept count
    counts = torch.tensor([int(mask[cu[i] : cu[i + 1] - 1].sum()) for i in range(len(lens))]).clamp(min=1)
    assert ((seq.cpu() - seq_o.detach()).abs() <= TOL * counts).all()
    assert abs(loss.item() - loss_o.item()) <= TOL
    assert (dh.grad.float().cpu() - rh.grad).abs().max().item() <= _bf16_tol(rh.grad)
    assert (dw.grad.float().cpu() - rw.grad).abs().max().item() <= _bf16_tol(rw.grad)
    assert ((dh.grad.float().cpu() - rh.grad).norm() / rh.grad.norm()).item() <= 2e-2
    assert ((dw.grad.float().cpu() - rw.grad).norm() / rw.grad.norm()).item() <= 2e-2
    assert (dh.grad.cpu()[~mask] == 0).all()
    assert math.isfinite(stats["policy/entropy_avg"].item())


@pytest.mark.parametrize("packed", [False, True])
def test_dpo_chain_matches_oracle(packed):
    """Fused head -> per-sequence logps -> sigmoid preference loss (open_instruct/dpo_utils.py:523-563,
    open_instruct/dpo_utils.py:826-878), gradient to the hidden states only (frozen head)."""
    torch.manual_seed(6)
    h, v, pairs, t = 64, 2000, 3, 48
    b = 2 * pairs  # chosen rows first, rejected rows after, as concatenated_inputs lays them out
    hidden = torch.randn(b, t, h).bfloat16()
    weight = (torch.randn(v, h) * 2.0 / math.sqrt(h)).bfloat16()
    labels = torch.randint(0, v, (b, t))
    labels[:, :7] = -100  # prompt
    labels[1, 30:] = -100  # padding tail
    labels[4, 20:] = -100
    ref_c, ref_r = -torch.rand(pairs) * 40, -torch.rand(pairs) * 40
    beta = 0.1

    rh = hidden.float().requires_grad_(True)
    if packed:
        flat_lab = labels.reshape(1, -1)
        cu = torch.arange(0, b * t + 1, t, dtype=torch.int32)
        lp_o = o_logprob.calculate_per_token_logps(o_lm.lm_head_logits(rh.reshape(1, b * t, h), weight.float()), flat_lab)
        seq_o = o_red.get_batch_logps_packed(lp_o, flat_lab, cu)
    else:
        lp_o = o_logprob.calculate_per_token_logps(o_lm.lm_head_logits(rh, weight.float()), labels)
        seq_o = o_red.get_batch_logps_padded(lp_o, labels)
    losses_o, cr_o, rr_o = o_dpo.dpo_loss(seq_o[:pairs], seq_o[pairs:], ref_c, ref_r, beta, label_smoothing=0.05)
    losses_o.mean().backward()

    dh = hidden.to(DEV).requires_grad_(True)
    w = weight.to(DEV)
    if packed:
        flat_lab_d = labels.reshape(1, -1).to(DEV)
        shifted = padding_free_collator.shift_labels(flat_lab_d)
        lp, _ = lm_head.fused_lm_head_logprobs(dh.reshape(1, b * t, h), w, shifted, mask=shifted != -100)
        seq = padding_free_collator.get_batch_logps(lp, flat_lab_d, cu.to(DEV))
    else:
        shifted = padding_free_collator.shift_labels(labels.to(DEV))
        lp, _ = lm_head.fused_lm_head_logprobs(dh, w, shifted, mask=shifted != -100)
        seq = dpo_utils._get_batch_logps(lp, labels.to(DEV))
    losses, cr, rr = dpo_utils.dpo_loss(seq[:pairs], seq[pairs:], ref_c.to(DEV), ref_r.to(DEV), beta, label_smoothing=0.05)
    losses.mean().backward()

    n_kept = (labels[:, 1:] != -100).sum(-1).clamp(min=1).float()
    assert ((seq.cpu() - seq_o.detach()).abs() <= TOL * n_kept).all()
    # loss = f(beta * x): the error of x (two sequence sums) is scaled by beta
    assert (losses.cpu() - losses_o.detach()).abs().max().item() <= TOL * beta * 2 * n_kept.max().item() + 1e-5
    assert (cr.cpu() - cr_o).abs().max().item() <= TOL * beta * n_kept.max().item() + 1e-5
    assert (rr.cpu() - rr_o).abs().max().item() <= TOL * beta * n_kept.max().item() + 1e-5
    assert (dh.grad.float().cpu() - rh.grad).abs().max().item() <= _bf16_tol(rh.grad)
    assert ((dh.grad.float().cpu() - rh.grad).norm() / rh.grad.norm()).item() <= 2e-2


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("loss_type,slabs,want_dw,w_scale", [
    ("dpo", True, True, 2.0),  # every pair in one slab
    ("dpo_norm", 1024, True, 2.0),  # slabs of whole pairs (two or three pairs each), d_weight accumulates over them
    ("simpo", 512, False, 2.0),  # one pair per slab; no reference model, a margin, averages
    ("dpo", 256, True, 2.0),  # every pair is larger than a slab: cut across slabs, recomputing backward
    ("dpo", 1024, True, 40.0),  # logits of +-100: most labels too unlikely for kept exponentials, flagged and recomputed
    ("dpo_reference_free", True, True, 2.0),
])  # fmt: skip
def test_dpo_loss_on_hidden_whole_step(packed, loss_type, slabs, want_dw, w_scale):
    """One C call for DPOLMHead -> per-sequence logps -> preference loss -> losses.mean().backward()
    (open_instruct/olmo_core_train_modules.py:71-76, :190-207, open_instruct/padding_free_collator.py:202-229,
    open_instruct/dpo_utils.py:523-563, :617-642, :689-712) with a trainable head and nothing recomputed,
    against the oracle chain: padded and packed batches, sums and averages, pair-aligned slabs."""
    torch.manual_seed(16)
    h, v, pairs = 128, 3000, 5
    n_seqs = 2 * pairs
    beta, ls = 0.1, 0.05
    if packed:
        lens = torch.randint(40, 260, (n_seqs,)).tolist()
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
        total = int(cu[-1])
        labels = torch.randint(0, v, (1, total))
        for i in range(n_seqs):
            labels[0, cu[i] : cu[i] + min(lens[i] - 1, 5 + 3 * i)] = -100  # prompts
        hidden = torch.randn(1, total, h).bfloat16()
    else:
        cu, total = None, 220
        labels = torch.randint(0, v, (n_seqs, total))
        for i in range(n_seqs):
            labels[i, : 5 + 3 * i] = -100  # prompts
            labels[i, total - 7 * i :] = -100 if i else labels[i, total:]  # padding tails of different lengths
        hidden = torch.randn(n_seqs, total, h).bfloat16()
    weight = (torch.randn(v, h) * w_scale / math.sqrt(h)).bfloat16()
    ref_c, ref_r = -torch.rand(pairs) * 300, -torch.rand(pairs) * 300
    average = loss_type in ("dpo_norm", "simpo")

    rh = hidden.double().requires_grad_(True)
    rw = weight.double().requires_grad_(True)
    z = o_lm.lm_head_logits(rh, rw, torch.float64)
    lp_o = o_logprob.calculate_per_token_logps(z, labels)
    seq_o = o_red.get_batch_logps_packed(lp_o, labels, cu, average) if packed else o_red.get_batch_logps_padded(lp_o, labels, average)
    if loss_type == "simpo":
        losses_o, cr_o, rr_o = o_dpo.simpo_loss(seq_o[:pairs], seq_o[pairs:], beta, 0.3, ls)
    else:
        losses_o, cr_o, rr_o = o_dpo.dpo_loss(
            seq_o[:pairs], seq_o[pairs:], ref_c.double(), ref_r.double(), beta, loss_type == "dpo_reference_free", ls
        )
    losses_o.mean().backward()

    d = lambda x: None if x is None else x.to(DEV)  # noqa: E731
    dh = d(hidden).requires_grad_(True)
    dw = d(weight).requires_grad_(want_dw)
    res = dpo_utils.dpo_loss_on_hidden(
        dh, dw, d(labels), None if loss_type == "simpo" else d(ref_c), None if loss_type == "simpo" else d(ref_r), beta,
        cu_seq_lens=d(cu), average_log_prob=average, reference_free=loss_type == "dpo_reference_free",
        label_smoothing=ls, gamma_beta_ratio=0.3 if loss_type == "simpo" else 0.0, token_slabs=slabs,
    )  # fmt: skip
    (2.0 * res.loss).backward()  # an upstream gradient other than 1 is applied on the device
    keep = o_logprob.shift_labels(labels) != -100
    size = lp_o.detach().abs().max().item()
    assert ((res.per_token_logps.cpu().double() - lp_o.detach()) * keep).abs().max().item() <= TOL + 1e-6 * size
    assert (res.per_token_logps.cpu()[~keep] == 0).all()
    n_kept = keep.sum().item() / n_seqs
    got_seq = torch.cat([res.chosen_logps, res.rejected_logps]).cpu().double()
    seq_tol = TOL * (1.0 if average else 2.0 * n_kept) + 1e-6 * seq_o.detach().abs().max().item()
    assert (got_seq - seq_o.detach()).abs().max().item() <= seq_tol
    assert (res.losses.cpu().double() - losses_o.detach()).abs().max().item() <= beta * 2 * seq_tol + 1e-5
    assert abs(res.loss.item() - losses_o.detach().mean().item()) <= beta * 2 * seq_tol + 1e-5
    assert (res.chosen_rewards.cpu().double() - cr_o).abs().max().item() <= beta * seq_tol + 1e-4
    assert (res.rejected_rewards.cpu().double() - rr_o).abs().max().item() <= beta * seq_tol + 1e-4
    got = dh.grad.double().cpu()
    exp_dh, exp_dw = 2.0 * rh.grad, 2.0 * rw.grad
    assert torch.isfinite(got).all() and (got[~keep] == 0).all()
    assert ((got - exp_dh).norm() / exp_dh.norm()).item() <= 2e-2
    err, norm = (got - exp_dh).flatten(0, 1).norm(dim=1), exp_dh.flatten(0, 1).norm(dim=1)
    assert (err - 3e-2 * norm).max().item() <= 1e-4 * norm.max().item()
    if want_dw:
        gw = dw.grad.double().cpu()
        assert torch.isfinite(gw).all()
        assert ((gw - exp_dw).norm() / exp_dw.norm()).item() <= 2e-2
    else:
        assert dw.grad is None
    # the differentiable route through the head's per-token logps gives the same numbers
    dh2 = d(hidden).requires_grad_(True)
    shifted = padding_free_collator.shift_labels(d(labels))
    lp2, _ = lm_head.fused_lm_head_logprobs(dh2, d(weight), shifted, mask=shifted != -100)
    assert (lp2.detach() - res.per_token_logps).abs().max().item() <= 1e-5 + 1e-6 * size
    # no gradient wanted: forward only, same values
    with torch.no_grad():
        res0 = dpo_utils.dpo_loss_on_hidden(
            dh, dw, d(labels), None if loss_type == "simpo" else d(ref_c), None if loss_type == "simpo" else d(ref_r),
            beta, cu_seq_lens=d(cu), average_log_prob=average, reference_free=loss_type == "dpo_reference_free",
            label_smoothing=ls, gamma_beta_ratio=0.3 if loss_type == "simpo" else 0.0,
        )  # fmt: skip
    assert not res0.loss.requires_grad and abs(res0.loss.item() - res.loss.item()) <= 1e-5 + 1e-6 * abs(res.loss.item())


class _OlmoStyleModel(torch.nn.Module):
    """Stand-in with the olmo-core interface: the labels go into the model, ``lm_head`` is a DPOLMHead."""

    def __init__(self, vocab, hidden):
        super().__init__()
        from open_instruct_amd.olmo_core_train_modules import DPOLMHead

        self.embed = torch.nn.Embedding(vocab, hidden, dtype=torch.bfloat16)
        self.mix = torch.nn.Linear(hidden, hidden, bias=False, dtype=torch.bfloat16)
        self.lm_head = DPOLMHead(hidden, vocab)

    def forward(self, input_ids, labels=None, position_ids=None, doc_lens=None, max_doc_lens=None):
        x = self.embed(input_ids)
        x = x + torch.tanh(self.mix(x))
        return self.lm_head(x, labels=labels)


@pytest.mark.parametrize("packing", [False, True])
@pytest.mark.parametrize("loss_type", ["dpo_norm", "simpo"])
def test_fused_loss_olmo_matches_the_reference_sequence(packing, loss_type):
    """fused_loss_olmo against concatenated_forward_olmo -> compute_loss -> losses.mean().backward()
    (open_instruct/olmo_core_train_modules.py:190-207) of this package on the same model: loss, logps and
    the gradient of every parameter (trunk and head)."""
    import types

    from open_instruct_amd import model_utils as mu

    torch.manual_seed(26)
    vocab, hid, bs = 400, 64, 3
    model = _OlmoStyleModel(vocab, hid).to(DEV)
    args = types.SimpleNamespace(loss_type=loss_type, beta=5.0, label_smoothing=0.0, gamma_beta_ratio=0.3)
    cache = mu.TensorCache(tensors={"chosen_logps": -torch.rand(8, device=DEV) * 3, "rejected_logps": -torch.rand(8, device=DEV) * 3})
    if packing:
        def side(lens):
            ids = torch.randint(1, vocab, (1, sum(lens)), device=DEV)
            cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=DEV)
            lab = ids.clone()
            for i in range(len(lens)):
                lab[0, cu[i] : cu[i] + 4] = -100
            return ids, lab, cu
        c_ids, c_lab, c_cu = side([20, 33, 17])
        r_ids, r_lab, r_cu = side([25, 19, 30])
        batch = {
            "chosen_input_ids": c_ids, "chosen_labels": c_lab, "chosen_cu_seq_lens_k": c_cu, "chosen_cu_seq_lens_q": c_cu,
            "chosen_max_length_q": 33, "chosen_max_length_k": 33,
            "rejected_input_ids": r_ids, "rejected_labels": r_lab, "rejected_cu_seq_lens_k": r_cu,
            "rejected_cu_seq_lens_q": r_cu, "rejected_max_length_q": 30, "rejected_max_length_k": 30,
            "index": torch.tensor([5, 1, 6], device=DEV),
        }  # fmt: skip
    else:
        batch = {
            "chosen_input_ids": torch.randint(1, vocab, (bs, 30), device=DEV),
            "rejected_input_ids": torch.randint(1, vocab, (bs, 24), device=DEV),
            "index": torch.tensor([5, 1, 6], device=DEV),
        }
        batch["chosen_labels"] = batch["chosen_input_ids"].clone()
        batch["rejected_labels"] = batch["rejected_input_ids"].clone()
        batch["chosen_labels"][:, :6] = -100
        batch["rejected_labels"][:, :4] = -100
    average = loss_type in ("dpo_norm", "simpo")
    c0, r0, _ = dpo_utils.concatenated_forward_olmo(model, batch, average_log_prob=average, packing=packing)
    losses0, cr0, rr0 = dpo_utils.compute_loss(args, batch, c0, r0, cache)
    losses0.mean().backward()
    g0 = [p.grad.float().clone() for p in model.parameters()]
    model.zero_grad()
    res = dpo_utils.fused_loss_olmo(model, batch, args, cache, packing=packing)
    res.loss.backward()
    g1 = [p.grad.float().clone() for p in model.parameters()]
    assert model.lm_head.fused_loss is None and model.lm_head.fused_result is None
    assert (res.chosen_logps - c0.detach()).abs().max().item() <= 1e-4 and (res.rejected_logps - r0.detach()).abs().max().item() <= 1e-4
    assert (res.losses - losses0.detach()).abs().max().item() <= 1e-3
    assert (res.chosen_rewards - cr0).abs().max().item() <= 1e-3 and (res.rejected_rewards - rr0).abs().max().item() <= 1e-3
    for x, y in zip(g0, g1):
        assert (x - y).abs().max().item() <= 2e-2 * max(1e-4, x.abs().max().item()), (x - y).abs().max().item()
    with pytest.raises(ValueError):
        dpo_utils.fused_loss_olmo(model, batch, types.SimpleNamespace(loss_type="ipo", beta=0.1), cache, packing=packing)


def test_fused_loss_olmo_serves_wpo_through_the_differentiable_calls():
    """loss_type wpo has no one-call form: fused_loss_olmo runs concatenated_forward_olmo -> compute_loss ->
    losses.mean() itself (open_instruct/olmo_core_train_modules.py:190-207, open_instruct/dpo_utils.py:566-613)
    and returns the same result type.  One pair per batch: the reference's weight broadcasts the [bs] sequence
    sums against the [bs, T] label masks, which only lines up for bs = 1."""
    import types

    from open_instruct_amd import model_utils as mu

    torch.manual_seed(27)
    vocab, hid = 400, 64
    model = _OlmoStyleModel(vocab, hid).to(DEV)
    args = types.SimpleNamespace(loss_type="wpo", beta=0.5, label_smoothing=0.05, gamma_beta_ratio=0.0)
    cache = mu.TensorCache(tensors={"chosen_logps": -torch.rand(4, device=DEV) * 3, "rejected_logps": -torch.rand(4, device=DEV) * 3})
    batch = {
        "chosen_input_ids": torch.randint(1, vocab, (1, 12), device=DEV),
        "rejected_input_ids": torch.randint(1, vocab, (1, 9), device=DEV),
        "index": torch.tensor([2], device=DEV),
    }
    batch["chosen_labels"] = batch["chosen_input_ids"].clone()
    batch["rejected_labels"] = batch["rejected_input_ids"].clone()
    batch["chosen_labels"][:, :11] = -100  # one scored token each: the weight exp(sum_c + sum_r) stays well above 0
    batch["rejected_labels"][:, :8] = -100
    c0, r0, _ = dpo_utils.concatenated_forward_olmo(model, batch, average_log_prob=False)
    losses0, cr0, rr0 = dpo_utils.compute_loss(args, batch, c0, r0, cache)
    losses0.mean().backward()
    g0 = [p.grad.float().clone() for p in model.parameters()]
    model.zero_grad()
    res = dpo_utils.fused_loss_olmo(model, batch, args, cache)
    res.loss.backward()
    g1 = [p.grad.float().clone() for p in model.parameters()]
    assert res.per_token_logps is None and model.lm_head.fused_loss is None
    assert torch.equal(res.losses, losses0.detach()) and torch.equal(res.chosen_logps, c0.detach())
    assert torch.equal(res.chosen_rewards, cr0) and torch.equal(res.rejected_rewards, rr0)
    assert res.loss.item() == losses0.mean().item() and losses0.abs().max().item() > 1e-7
    for x, y in zip(g0, g1):
        assert torch.equal(x, y)


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (300, 515, 192), (1, 70, 128), (1030, 257, 4096)])
def test_gemm_bf16_tn_entry_point(m, n, k):
    """out[m, n] = sum_k A[m, k] * B[n, k] through the raw C-ABI, bf16 and fp32 outputs, accumulate."""
    torch.manual_seed(7)
    a = torch.randn(m, k).bfloat16()
    b = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    exp = o_lm.lm_head_logits(a, b, torch.float64)
    lib = _lib.load()
    ad, bd = a.to(DEV), b.to(DEV)
    out32 = torch.full((m, n), 0.5, dtype=torch.float32, device=DEV)
    out16 = torch.zeros(m, n, dtype=torch.bfloat16, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.oi_gemm_bf16_tn(ad.data_ptr(), k, m, bd.data_ptr(), k, n, k, out32.data_ptr(), None, n, 1, stream)
    assert rc == 0
    rc = lib.oi_gemm_bf16_tn(ad.data_ptr(), k, m, bd.data_ptr(), k, n, k, None, out16.data_ptr(), n, 0, stream)
    assert rc == 0
    torch.cuda.synchronize()
    # fp32 accumulation of k products of O(1/sqrt k) terms: 1e-4 abs covers k = 4096
    assert (out32.cpu().double() - 0.5 - exp).abs().max().item() <= 1e-4
    assert (out16.cpu().double() - exp).abs().max().item() <= exp.abs().max().item() * 2**-8 + 1e-4
    # rejected arguments launch nothing
    assert lib.oi_gemm_bf16_tn(ad.data_ptr(), k, m, bd.data_ptr(), k, n, k + 8, out32.data_ptr(), None, n, 0, stream) == -1
    assert lib.oi_gemm_bf16_tn(None, k, m, bd.data_ptr(), k, n, k, out32.data_ptr(), None, n, 0, stream) == -2
    assert lib.oi_gemm_bf16_tn(ad.data_ptr(), k, m, bd.data_ptr(), k, n, k, None, None, n, 0, stream) != 0


@pytest.mark.parametrize("a_km,b_km", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (304, 520, 192), (8, 72, 128), (1032, 264, 1024), (64, 64, 4096)])
def test_gemm_bf16_operand_layouts(m, n, k, a_km, b_km):
    """Every combination of k-contiguous and k-major operands through the raw C-ABI: one, two, three
    and many k-tiles, ragged tile edges in both dimensions, padded leading dimensions."""
    print(f"case M={m} N={n} K={k} A k-major={a_km} B k-major={b_km}", flush=True)
    torch.manual_seed(11)
    a = torch.randn(m, k).bfloat16()
    b = (torch.randn(n, k) / math.sqrt(k)).bfloat16()
    exp = o_lm.lm_head_logits(a, b, torch.float64)
    lib = _lib.load()

    def device_operand(x, k_major):
        rows, cols = (x.shape[1], x.shape[0]) if k_major else x.shape
        ld = cols + 16  # padded rows, filled with a value that must never be read as data
        buf = torch.full((rows, ld), 77.0, dtype=torch.bfloat16, device=DEV)
        buf[:, :cols] = (x.t() if k_major else x).to(DEV)
        return buf, ld

    ad, lda = device_operand(a, a_km)
    bd, ldb = device_operand(b, b_km)
    out32 = torch.full((m, n), -0.25, dtype=torch.float32, device=DEV)
    out16 = torch.zeros(m, n, dtype=torch.bfloat16, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    args = (ad.data_ptr(), lda, a_km, bd.data_ptr(), ldb, b_km, m, n, k)
    assert lib.oi_gemm_bf16_layouts(*args, out32.data_ptr(), None, n, 1, stream) == 0
    assert lib.oi_gemm_bf16_layouts(*args, None, out16.data_ptr(), n, 0, stream) == 0
    torch.cuda.synchronize()
    assert (out32.cpu().double() + 0.25 - exp).abs().max().item() <= 1e-4
    assert (out16.cpu().double() - exp).abs().max().item() <= exp.abs().max().item() * 2**-8 + 1e-4
    # the two layouts of the same numbers give the same bits (same products, same order of summation)
    if a_km or b_km:
        ref32 = torch.zeros(m, n, dtype=torch.float32, device=DEV)
        a0, b0 = a.to(DEV).contiguous(), b.to(DEV).contiguous()
        assert lib.oi_gemm_bf16_layouts(a0.data_ptr(), k, 0, b0.data_ptr(), k, 0, m, n, k, ref32.data_ptr(), None, n, 0, stream) == 0
        got32 = torch.zeros(m, n, dtype=torch.float32, device=DEV)
        assert lib.oi_gemm_bf16_layouts(*args, got32.data_ptr(), None, n, 0, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(ref32, got32)
    # rejected arguments launch nothing
    assert lib.oi_gemm_bf16_layouts(ad.data_ptr(), lda, a_km, bd.data_ptr(), ldb, b_km, m, n, k + 8, out32.data_ptr(), None, n, 0, stream) == -1
    assert lib.oi_gemm_bf16_layouts(ad.data_ptr(), 4, a_km, bd.data_ptr(), ldb, b_km, m, n, k, out32.data_ptr(), None, n, 0, stream) == -1
    if a_km:
        assert lib.oi_gemm_bf16_layouts(ad.data_ptr(), lda, 1, bd.data_ptr(), ldb, b_km, m - 1, n, k, out32.data_ptr(), None, n, 0, stream) == -1


def test_full_size_properties_fused_head():
    """Llama-3.1-8B head shape (H = 4096, V = 128256), 1500 rows: properties that need no oracle.

    * zero hidden states -> uniform distribution: logprob = -ln V and entropy = ln V (closed form);
    * hidden * 2 at temperature 2 equals hidden at temperature 1 (power-of-two scaling is exact in bf16);
    * permuting the vocabulary (rows of W and the labels with them) leaves every result unchanged
      up to summation order;
    * every row of dZ sums to zero, so the column sums of dW vanish and, with all rows of W equal,
      dHidden vanishes: a checksum over the whole backward;
    * the fused kernel agrees with the row-wise kernel on library-made fp32 logits.
    """
    torch.manual_seed(8)
    n, h, v = 1500, 4096, 128256
    hidden = torch.randn(n, h, device=DEV).bfloat16()
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16()
    labels = torch.randint(0, v, (n,), device=DEV)

    lp0, ent0 = lm_head.fused_lm_head_logprobs(torch.zeros_like(hidden), weight, labels, return_entropy=True)
    assert (lp0 + math.log(v)).abs().max().item() <= 1e-5
    assert (ent0 - math.log(v)).abs().max().item() <= 1e-5

    lp, ent = lm_head.fused_lm_head_logprobs(hidden, weight, labels, return_entropy=True)
    assert (lp <= 0).all() and (ent >= 0).all() and (ent <= math.log(v) + 1e-4).all()
    lp2, ent2 = lm_head.fused_lm_head_logprobs(hidden * 2, weight, labels, temperature=2.0, return_entropy=True)
    assert (lp2 - lp).abs().max().item() <= 1e-5 and (ent2 - ent).abs().max().item() <= 1e-5

    perm = torch.randperm(v, device=DEV)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(v, device=DEV)
    lpp, entp = lm_head.fused_lm_head_logprobs(hidden, weight[perm], inv[labels], return_entropy=True)
    assert (lpp - lp).abs().max().item() <= 1e-4 and (entp - ent).abs().max().item() <= 1e-4

    logits = hidden[:512].float() @ weight.float().t()
    exp_lp, exp_ent = model_utils.logprob_and_entropy(logits, labels[:512])
    assert (lp[:512] - exp_lp).abs().max().item() <= TOL
    assert (ent[:512] - exp_ent).abs().max().item() <= TOL
    del logits

    dh = hidden.clone().requires_grad_(True)
    dw = weight.clone().requires_grad_(True)
    up = torch.randn(n, device=DEV)
    out, _ = lm_head.fused_lm_head_logprobs(dh, dw, labels, temperature=0.8)
    out.backward(up)
    col_sums = dw.grad.float().sum(0)  # = sum_n (sum_v dZ[n, v]) h_n = 0 up to bf16 rounding of dW and dZ
    scale = dw.grad.float().abs().sum(0)
    assert (col_sums.abs() <= 2e-2 * scale + 1e-3).all(), (col_sums.abs() / (scale + 1e-9)).max().item()
    # dW row of a label that occurs once, for a token with tiny softmax mass there, is ~ g/T * h_n
    assert dh.grad.isfinite().all() and dw.grad.isfinite().all()

    same = weight[:1].expand(4096, h).contiguous()  # all vocabulary rows equal -> dHidden = 0
    dh2 = hidden[:300].clone().requires_grad_(True)
    out2, _ = lm_head.fused_lm_head_logprobs(dh2, same, labels[:300] % 4096)
    out2.backward(up[:300])
    # every dZ entry of a row is the same number g/V and rounds to bf16 the same way, so the row sum
    # of dZ is off by up to one bf16 rounding of g: |dHidden| <= 2^-8 |g| max|w|
    bound = 2**-8 * up[:300].abs().max().item() * same.float().abs().max().item() + 1e-6
    assert dh2.grad.float().abs().max().item() <= bound


@pytest.mark.parametrize("packing", [False, True])
@pytest.mark.parametrize("average_log_prob", [False, True])
def test_concatenated_forward_olmo_through_dpo_lm_head(packing, average_log_prob):
    """Call stack of the olmo-core DPO trainer (open_instruct/olmo_core_train_modules.py:190-207):
    concatenated_forward_olmo (open_instruct/dpo_utils.py:959-1019) -> model(ids, labels=...) whose LM
    head is DPOLMHead (open_instruct/olmo_core_train_modules.py:48-85) -> per-sequence logps -> dpo_loss,
    forward and backward, against the oracle chain on materialised fp32 logits."""
    from open_instruct_amd.olmo_core_train_modules import DPOLMHead

    torch.manual_seed(31)
    d_model, vocab, pairs = 64, 1500, 2

    class TinyOlmo(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.embed = torch.nn.Embedding(vocab, d_model, dtype=torch.bfloat16)
            self.lm_head = DPOLMHead(d_model=d_model, vocab_size=vocab)
            self.seen = {}

        def forward(self, input_ids, labels=None, position_ids=None, doc_lens=None, max_doc_lens=None):
            self.seen = {"doc_lens": doc_lens, "max_doc_lens": max_doc_lens, "position_ids": position_ids}
            return self.lm_head(self.embed(input_ids), labels=labels)

    model = TinyOlmo().to(DEV)
    with torch.no_grad():
        model.lm_head.w_out.weight.mul_(6.0)

    def side(lengths, prompt):
        ids = [torch.randint(1, vocab, (n,)) for n in lengths]
        labs = [t.clone() for t in ids]
        for lab in labs:
            lab[:prompt] = -100
        return ids, labs

    c_ids, c_labs = side([11, 17], 4)
    r_ids, r_labs = side([9, 23], 4)
    if packing:
        def pack(ids, labs):
            lens = torch.tensor([len(t) for t in ids])
            cu = torch.cat([torch.zeros(1, dtype=torch.long), lens.cumsum(0)]).to(torch.int32)
            pos = torch.cat([torch.arange(n) for n in lens.tolist()])
            return {"input_ids": torch.cat(ids)[None], "labels": torch.cat(labs)[None], "cu_seq_lens_q": cu,
                    "cu_seq_lens_k": cu, "max_length_q": int(lens.max()), "max_length_k": int(lens.max()),
                    "position_ids": pos[None]}  # fmt: skip

        batch = {f"chosen_{k}": v for k, v in pack(c_ids, c_labs).items()}
        batch |= {f"rejected_{k}": v for k, v in pack(r_ids, r_labs).items()}
    else:
        def pad(seqs, value):
            width = max(len(t) for t in seqs)
            return torch.stack([torch.cat([t, torch.full((width - len(t),), value)]) for t in seqs])

        batch = {"chosen_input_ids": pad(c_ids, 0), "chosen_labels": pad(c_labs, -100),
                 "rejected_input_ids": pad(r_ids, 0), "rejected_labels": pad(r_labs, -100)}  # fmt: skip
    batch = {k: (v.to(DEV) if torch.is_tensor(v) else v) for k, v in batch.items()}
    ref_c, ref_r = -torch.rand(pairs) * 30, -torch.rand(pairs) * 30
    beta = 0.1

    chosen, rejected, aux = dpo_utils.concatenated_forward_olmo(model, batch, average_log_prob=average_log_prob, packing=packing)
    assert aux is None and chosen.shape == (pairs,) and rejected.shape == (pairs,)
    if packing:
        assert model.seen["doc_lens"].tolist() == [[11, 17, 9, 23]] and model.seen["max_doc_lens"] == [23]
        assert model.seen["position_ids"].shape == (1, 60)
    losses, _, _ = dpo_utils.dpo_loss(chosen, rejected, ref_c.to(DEV), ref_r.to(DEV), beta)
    losses.mean().backward()

    # oracle: the same embedding rows and head weights in fp32, logits materialised
    emb = model.embed.weight.detach().float().cpu().requires_grad_(True)
    w = model.lm_head.w_out.weight.detach().float().cpu().requires_grad_(True)
    if packing:
        concat, _ = padding_free_collator.concatenated_inputs({k: (v.cpu() if torch.is_tensor(v) else v) for k, v in batch.items()})
    else:
        concat = dpo_utils.concatenated_inputs({k: v.cpu() for k, v in batch.items()})
    ids, labels = concat["concatenated_input_ids"], concat["concatenated_labels"]
    logits = torch.nn.functional.linear(emb[ids], w)
    per_token = o_logprob.calculate_per_token_logps(logits, labels)
    if packing:
        seq_o = o_red.get_batch_logps_packed(per_token, labels, concat["concatenated_cu_seq_lens_k"], average_log_prob)
    else:
        seq_o = o_red.get_batch_logps_padded(per_token, labels, average_log_prob)
    losses_o, _, _ = o_dpo.dpo_loss(seq_o[:pairs], seq_o[pairs:], ref_c, ref_r, beta)
    losses_o.mean().backward()

    n_kept = 1.0 if average_log_prob else 23.0
    assert (torch.cat([chosen, rejected]).detach().cpu() - seq_o.detach()).abs().max().item() <= TOL * n_kept
    assert (losses.detach().cpu() - losses_o.detach()).abs().max().item() <= TOL * beta * 2 * n_kept + 1e-5
    for got, exp in ((model.lm_head.w_out.weight.grad, w.grad), (model.embed.weight.grad, emb.grad)):
        got = got.float().cpu()
        assert (got - exp).abs().max().item() <= _bf16_tol(exp)
        assert ((got - exp).norm() / exp.norm()).item() <= 2e-2
    if packing:
        return
    # the two-forward variant of the same stack (open_instruct/dpo_utils.py:1022-1054): same sums, same gradients
    model.zero_grad()
    chosen2, rejected2, aux2 = dpo_utils.separate_forward_olmo(model, batch, average_log_prob=average_log_prob)
    assert aux2 is None and chosen2.shape == (pairs,) and rejected2.shape == (pairs,)
    assert (chosen2 - chosen).abs().max().item() <= 1e-4 and (rejected2 - rejected).abs().max().item() <= 1e-4
    losses2, _, _ = dpo_utils.dpo_loss(chosen2, rejected2, ref_c.to(DEV), ref_r.to(DEV), beta)
    losses2.mean().backward()
    for got, exp in ((model.lm_head.w_out.weight.grad, w.grad), (model.embed.weight.grad, emb.grad)):
        got = got.float().cpu()
        assert (got - exp).abs().max().item() <= _bf16_tol(exp)
        assert ((got - exp).norm() / exp.norm()).item() <= 2e-2


@pytest.mark.parametrize("b,t,h,v,axis,want_dw,slabs", [
    (3, 130, 128, 40000, None, True, True),  # one slab, two vocabulary chunks
    (5, 2500, 64, 700, None, True, True),  # 8000 selected tokens: one slab, d_weight stored directly
    (5, 2500, 64, 700, 1, False, 4096),  # two equal slabs
    (9, 2000, 64, 300, None, True, True),  # 12800 selected tokens: two equal slabs, one pass stays empty
    (9, 2000, 64, 300, None, True, 2048),  # seven slabs in nine passes, d_weight accumulates over them
    (3, 700, 64, 300, None, True, 300),  # a slab size that is rounded up to whole token tiles (512)
])  # fmt: skip
def test_grpo_loss_on_hidden_in_token_slabs(b, t, h, v, axis, want_dw, slabs):
    """The whole step without recomputation (equal slabs of selected tokens made on the device, the
    exponentials of one slab at a time) against the oracle chain."""
    print(f"case b={b} t={t} h={h} v={v} axis={axis} dW={want_dw} slabs={slabs}", flush=True)
    torch.manual_seed(41)
    hidden = torch.randn(b, t, h).bfloat16()
    weight = (torch.randn(v, h) * 3.0 / math.sqrt(h)).bfloat16()
    labels = torch.randint(0, v, (b, t))
    mask = torch.rand(b, t) < 0.8
    mask[1, :] = False
    adv = torch.randn(b, 1)
    cfg = make_grpo_config(loss_fn="dapo", beta=0.05, kl_estimator=2, clip_higher=0.28)
    rh = hidden.float().requires_grad_(True)
    rw = weight.float().requires_grad_(True)
    lp_o, ent_o = o_lm.lm_head_logprobs(rh.reshape(b * t, h), rw, labels.reshape(-1), 1.0, True)
    lp_o, ent_o = lp_o.reshape(b, t), ent_o.reshape(b, t)
    old = lp_o.detach() + 0.05 * torch.randn(b, t)
    ref = lp_o.detach() + 0.1 * torch.randn(b, t)
    loss_o, *_ = o_grpo.grpo_token_loss(lp_o, old, ref, adv.expand(b, t), mask.float(), cfg, axis=axis)
    torch.nan_to_num(loss_o, nan=0.0).backward()
    exp_dh, exp_dw = torch.nan_to_num(rh.grad, nan=0.0), torch.nan_to_num(rw.grad, nan=0.0)

    d = lambda x: x.to(DEV)  # noqa: E731
    dh = d(hidden).requires_grad_(True)
    dw = d(weight).requires_grad_(want_dw)
    loss, stats, lp, ent = grpo_utils.grpo_loss_on_hidden(
        dh, dw, d(labels), d(old), d(ref), d(adv), d(mask), cfg, axis=axis, token_slabs=slabs
    )
    loss.backward()
    assert ((lp.cpu() - lp_o.detach()) * mask).abs().max().item() <= TOL and (lp.cpu()[~mask] == 0).all()
    assert ((ent.cpu() - ent_o) * mask).abs().max().item() <= TOL and (ent.cpu()[~mask] == 0).all()
    if axis is None:
        assert abs(loss.item() - loss_o.item()) <= TOL
    got = dh.grad.float().cpu()
    assert (got - exp_dh).abs().max().item() <= _bf16_tol(exp_dh)
    assert ((got - exp_dh).norm() / exp_dh.norm()).item() <= 2e-2
    assert (dh.grad.cpu()[~mask] == 0).all()
    if want_dw:
        gw = dw.grad.float().cpu()
        assert (gw - exp_dw).abs().max().item() <= _bf16_tol(exp_dw)
        assert ((gw - exp_dw).norm() / exp_dw.norm()).item() <= 2e-2
    else:
        assert dw.grad is None
    # the statistics are those of the recomputing step
    dh2 = d(hidden).requires_grad_(True)
    loss2, stats2, lp2, _ = grpo_utils.grpo_loss_on_hidden(
        dh2, d(weight).requires_grad_(want_dw), d(labels), d(old), d(ref), d(adv), d(mask), cfg, axis=axis,
        token_slabs=False,
    )  # fmt: skip
    # (not to the last bit: a slab's forward merges its vocabulary splits in another order)
    assert (lp - lp2).abs().max().item() <= 1e-5 and abs(loss.item() - loss2.item()) <= 1e-6
    for k in stats2:
        assert torch.allclose(stats[k], stats2[k], rtol=1e-4, atol=1e-6, equal_nan=True), k
    with pytest.raises(ValueError):
        grpo_utils.grpo_loss_on_hidden(dh2, d(weight), d(labels), d(old), d(ref), d(adv), d(mask), cfg, token_slabs=100)
    # the gradients are handed out once
    with pytest.raises(RuntimeError, match="handed out"):
        dh6 = d(hidden).requires_grad_(True)
        loss6, *_ = grpo_utils.grpo_loss_on_hidden(dh6, d(weight), d(labels), d(old), d(ref), d(adv), d(mask), cfg, axis=axis)
        (0.5 * loss6).backward(retain_graph=True)
        (0.5 * loss6).backward()


@pytest.mark.parametrize("slabs,temperature,want_dw", [
    (True, 1.0, True),  # one slab: flagged tokens are added to the bf16 d_weight that the slab stored
    (512, 0.5, True),  # three slabs, fp32 d_weight: flagged tokens are added before it is rounded
    (512, 1.0, False),
    (False, 0.5, True),  # the recomputing step has no such limit to begin with
])  # fmt: skip
def test_grpo_loss_on_hidden_for_logits_of_any_size(slabs, temperature, want_dw):
    """The slab-wise step keeps its exponentials relative to each token's own label logit, and tokens whose
    label is too unlikely for that (more than 44 nats below the row's largest logit) take a recomputing
    backward inside the same call: values and both gradients against the fp64 oracle chain for rows whose
    largest logit / temperature runs from 0 to 600 nats, rows whose logits are all near -100 nats, likely
    and hopeless labels.  The reference's log_softmax is exact at any of these
    (open_instruct/padding_free_collator.py:10-16, open_instruct/model_utils.py:587-600)."""
    from test_gpu_lmhead import _rows_of_any_logit_size

    b, t, h, v = 3, 400, 128, 3000
    hidden, weight, labels, z = _rows_of_any_logit_size(b * t, h, v, seed=71)
    hidden, labels = hidden.view(b, t, h), labels.view(b, t)
    g = torch.Generator().manual_seed(72)
    mask = torch.rand(b, t, generator=g) < 0.8
    adv = torch.randn(b, t, generator=g)
    cfg = make_grpo_config(loss_fn="dapo", beta=0.05, kl_estimator=2, clip_higher=0.28)
    rh = hidden.double().requires_grad_(True)
    rw = weight.double().requires_grad_(True)
    lp_o, ent_o = o_lm.lm_head_logprobs(
        rh.reshape(b * t, h), rw, labels.reshape(-1), temperature, True, compute_dtype=torch.float64
    )
    lp_o, ent_o = lp_o.reshape(b, t), ent_o.reshape(b, t)
    # (off the mask the fused head returns 0, so the behaviour logprobs are 0 there as well: a ratio of
    # exp(0 - (-600)) would be an infinity times the mask's zero in the reference just the same)
    old = ((lp_o.detach() + 0.05 * torch.randn(b, t, generator=g).double()) * mask).float()
    ref = ((lp_o.detach() + 0.1 * torch.randn(b, t, generator=g).double()) * mask).float()
    loss_o, *_ = o_grpo.grpo_token_loss(lp_o * mask, old.double(), ref.double(), adv.double(), mask.double(), cfg)
    loss_o.backward()
    gap = (z / temperature).max(dim=1).values - (z / temperature).gather(1, labels.reshape(-1, 1))[:, 0]
    assert (gap[mask.reshape(-1)] > 60.0).sum() >= 40  # hopeless labels are among the selected rows

    d = lambda x: x.to(DEV)  # noqa: E731
    dh = d(hidden).requires_grad_(True)
    dw = d(weight).requires_grad_(want_dw)
    loss, _, lp, ent = grpo_utils.grpo_loss_on_hidden(
        dh, dw, d(labels), d(old), d(ref), d(adv), d(mask), cfg, temperature=temperature, token_slabs=slabs
    )
    loss.backward()
    size = lp_o.detach().abs().max().item()
    assert ((lp.cpu().double() - lp_o.detach()) * mask).abs().max().item() <= TOL + 1e-6 * size
    assert ((ent.cpu().double() - ent_o.detach()) * mask).abs().max().item() <= TOL
    assert abs(loss.item() - loss_o.item()) <= TOL + 1e-6 * abs(loss_o.item())
    got = dh.grad.double().cpu()
    assert torch.isfinite(got).all() and (got[~mask] == 0).all()
    err, ref_norm = (got - rh.grad).flatten(0, 1).norm(dim=1), rh.grad.flatten(0, 1).norm(dim=1)
    # per row: 3 % of the row's own gradient, plus an absolute part for rows whose gradient is next to nothing
    assert (err - 3e-2 * ref_norm).max().item() <= 1e-4 * ref_norm.max().item()
    assert ((got - rh.grad).norm() / rh.grad.norm()).item() <= 2e-2
    if want_dw:
        gw = dw.grad.double().cpu()
        assert torch.isfinite(gw).all()
        assert ((gw - rw.grad).norm() / rw.grad.norm()).item() <= 2e-2
        errw, normw = (gw - rw.grad).norm(dim=1), rw.grad.norm(dim=1)
        assert (errw - 3e-2 * normw).max().item() <= 2e-3 * normw.max().item()


@pytest.mark.parametrize("loss_fn,axis,denominator,with_old,want_dw", [
    ("dapo", None, None, True, True),
    ("dapo", 1, None, True, False),
    ("cispo", None, 300.0, False, True),
])  # fmt: skip
def test_grpo_loss_on_hidden_whole_step(loss_fn, axis, denominator, with_old, want_dw):
    """One C call for lm_head -> logprob / entropy -> GRPO loss -> backward
    (open_instruct/grpo_utils.py:558-572 -> :504-538 -> open_instruct/grpo_fast.py:702-724), the
    recomputing form of it, against the oracle chain and against the three-call chain of this package."""
    torch.manual_seed(33)
    b, t, h, v = 3, 130, 128, 40000  # two vocabulary chunks, two token tiles
    hidden = torch.randn(b, t, h).bfloat16()
    weight = (torch.randn(v, h) * 3.0 / math.sqrt(h)).bfloat16()
    labels = torch.randint(0, v, (b, t))
    mask = torch.rand(b, t) < 0.7
    mask[1, :] = False  # a row without response tokens
    adv = torch.randn(b, 1)  # broadcast along the tokens
    rho = torch.rand(b, t) + 0.5
    cfg = make_grpo_config(loss_fn=loss_fn, beta=0.05, kl_estimator=2, clip_higher=0.28)
    temperature = 0.9

    rh = hidden.float().requires_grad_(True)
    rw = weight.float().requires_grad_(True)
    lp_o, ent_o = o_lm.lm_head_logprobs(rh.reshape(b * t, h), rw, labels.reshape(-1), temperature, True)
    lp_o, ent_o = lp_o.reshape(b, t), ent_o.reshape(b, t)
    old = lp_o.detach() + 0.05 * torch.randn(b, t)
    ref = lp_o.detach() + 0.1 * torch.randn(b, t)
    loss_o, *_ = o_grpo.grpo_token_loss(
        lp_o, old if with_old else lp_o.detach(), ref, adv.expand(b, t), mask.float(), cfg, rho_weights=rho,
        loss_denominator=denominator, axis=axis, dp_scale=2.0,
    )  # fmt: skip
    torch.nan_to_num(loss_o, nan=0.0).backward()
    exp_dh, exp_dw = torch.nan_to_num(rh.grad, nan=0.0), torch.nan_to_num(rw.grad, nan=0.0)

    d = lambda x: x.to(DEV)  # noqa: E731
    dh = d(hidden).requires_grad_(True)
    dw = d(weight).requires_grad_(want_dw)
    loss, stats, lp, ent = grpo_utils.grpo_loss_on_hidden(
        dh, dw, d(labels), d(old) if with_old else None, d(ref), d(adv), d(mask), cfg, temperature=temperature,
        rho_weights=d(rho), loss_denominator=denominator, axis=axis, dp_scale=2.0, token_slabs=False,
    )  # fmt: skip
    loss.backward()
    assert ((lp.cpu() - lp_o.detach()) * mask).abs().max().item() <= TOL and (lp.cpu()[~mask] == 0).all()
    assert ((ent.cpu() - ent_o) * mask).abs().max().item() <= TOL
    if axis is None:
        assert abs(loss.item() - loss_o.item()) <= TOL
    assert (dh.grad.float().cpu() - exp_dh).abs().max().item() <= _bf16_tol(exp_dh)
    assert ((dh.grad.float().cpu() - exp_dh).norm() / exp_dh.norm()).item() <= 2e-2
    assert (dh.grad.cpu()[~mask] == 0).all()
    if want_dw:
        assert (dw.grad.float().cpu() - exp_dw).abs().max().item() <= _bf16_tol(exp_dw)
        assert ((dw.grad.float().cpu() - exp_dw).norm() / exp_dw.norm()).item() <= 2e-2
    else:
        assert dw.grad is None

    # the three-call chain of this package gives the same numbers
    dh2 = d(hidden).requires_grad_(True)
    dw2 = d(weight).requires_grad_(want_dw)
    # (the recomputing backward on both sides: the one-call entry has no other)
    lp2, ent2 = lm_head.fused_lm_head_logprobs(
        dh2, dw2, d(labels), temperature, mask=d(mask), return_entropy=True, dhidden_in_forward=False
    )
    loss2, stats2 = grpo_utils.grpo_loss_fused(
        lp2, d(old) if with_old else None, d(ref), d(adv), d(mask), cfg, rho_weights=d(rho), entropy=ent2,
        loss_denominator=denominator, axis=axis, dp_scale=2.0,
    )  # fmt: skip
    loss2.backward()
    assert torch.equal(lp, lp2.detach()) and torch.equal(ent, ent2)
    assert loss.item() == loss2.item()
    for k in stats2:
        assert stats[k].item() == stats2[k].item(), k
    assert torch.equal(dh.grad, dh2.grad)
    if want_dw:
        assert torch.equal(dw.grad, dw2.grad)
    # an upstream gradient other than 1 is applied on the device
    dh3 = d(hidden).requires_grad_(True)
    loss3, *_ = grpo_utils.grpo_loss_on_hidden(
        dh3, d(weight), d(labels), d(old) if with_old else None, d(ref), d(adv), d(mask), cfg, temperature=temperature,
        rho_weights=d(rho), loss_denominator=denominator, axis=axis, dp_scale=2.0, token_slabs=False,
    )  # fmt: skip
    (loss3 * 0.5).backward()
    assert (dh3.grad.float() - 0.5 * dh.grad.float()).abs().max().item() <= 2.0**-8 * dh.grad.float().abs().max().item()
    # no gradient wanted: forward only, same loss
    with torch.no_grad():
        loss4, _, lp4, _ = grpo_utils.grpo_loss_on_hidden(
            dh, dw, d(labels), d(old) if with_old else None, d(ref), d(adv), d(mask), cfg, temperature=temperature,
            rho_weights=d(rho), loss_denominator=denominator, axis=axis, dp_scale=2.0,
        )  # fmt: skip
    assert not loss4.requires_grad and loss4.item() == loss.item() and torch.equal(lp4, lp)



@pytest.mark.parametrize("slabs,t", [(False, 140), (2048, 3000)])
def test_entry_points_replay_from_a_hip_graph(slabs, t):
    """The C entry points enqueue kernels only (no allocation, no synchronisation, no memset nodes), so a
    caller may capture them in a HIP graph.  Two launch-bound cases: logprob + entropy + masked means on
    small logits, and the whole GRPO step on hidden states in one call (recomputing, and in two token slabs
    whose d_weight accumulates in fp32 from one slab to the next).  Every replay is compared with the eager result on
    inputs that eager work changed between the replays."""
    torch.manual_seed(51)
    logits = (torch.randn(4, 128, 8000, device=DEV) * 2.0)
    ids = torch.randint(0, 8000, (4, 128), device=DEV)
    mask = torch.rand(4, 128, device=DEV) > 0.3
    b, h, v = 2, 128, 3000
    hidden = torch.randn(b, t, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.2).bfloat16().requires_grad_(True)
    labels = torch.randint(0, v, (b, t), device=DEV)
    rmask = torch.rand(b, t, device=DEV) < 0.7
    adv = torch.randn(b, t, device=DEV)
    cfg = make_grpo_config(loss_fn="dapo", beta=0.05, kl_estimator=2, clip_higher=0.28)

    def small_step():
        lp, ent = model_utils.logprob_and_entropy(logits, ids)
        from open_instruct_amd import rl_utils

        return rl_utils.masked_mean(lp, mask) + rl_utils.masked_mean(ent, mask)

    def grpo_step():
        hidden.grad = None
        weight.grad = None
        loss, _, lp, _ = grpo_utils.grpo_loss_on_hidden(
            hidden, weight, labels, None, None, adv, rmask, cfg, token_slabs=slabs
        )
        loss.backward()
        return loss.detach(), hidden.grad, weight.grad

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            small_step()
            grpo_step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_small = small_step()
        g_loss, g_dh, g_dw = grpo_step()
    for i in range(4):
        with torch.no_grad():  # eager work between the replays changes the inputs in place
            logits.mul_(1.02)
            hidden.mul_(0.97)
        graph.replay()
        torch.cuda.synchronize()
        got = (g_small.clone(), g_loss.clone(), g_dh.clone(), g_dw.clone())
        e_small = small_step()
        e_loss, e_dh, e_dw = grpo_step()
        torch.cuda.synchronize()
        assert torch.equal(got[0], e_small), i
        assert torch.equal(got[1], e_loss) and torch.equal(got[2], e_dh) and torch.equal(got[3], e_dw), i


@pytest.mark.parametrize("slabs", [True, 512])
def test_dpo_step_replays_from_a_hip_graph(slabs):
    """The one-call DPO step (open_instruct/olmo_core_train_modules.py:190-207 as one C call: head, per-sequence
    sums, pair loss, both gradients) enqueues kernels only, so it can be captured: a packed batch with every pair
    in one slab, and in slabs of one or two pairs whose d_weight accumulates from slab to slab.  Every replay is
    compared with the eager result on inputs that eager work changed between the replays."""
    torch.manual_seed(52)
    h, v, pairs = 128, 3000, 4
    lens = torch.randint(60, 240, (2 * pairs,))
    cu = torch.tensor([0] + lens.cumsum(0).tolist(), dtype=torch.int32, device=DEV)
    total = int(cu[-1])
    labels = torch.randint(0, v, (1, total), device=DEV)
    for i in range(2 * pairs):
        labels[0, int(cu[i]) : int(cu[i]) + 4 + i] = -100
    hidden = torch.randn(1, total, h, device=DEV).bfloat16().requires_grad_(True)
    weight = (torch.randn(v, h, device=DEV) * 0.2).bfloat16().requires_grad_(True)
    ref_c, ref_r = -torch.rand(pairs, device=DEV) * 300, -torch.rand(pairs, device=DEV) * 300

    def step():
        hidden.grad = None
        weight.grad = None
        res = dpo_utils.dpo_loss_on_hidden(
            hidden, weight, labels, ref_c, ref_r, 0.1, cu_seq_lens=cu, label_smoothing=0.05, token_slabs=slabs
        )
        res.loss.backward()
        return res.loss.detach(), res.chosen_logps, res.rejected_rewards, hidden.grad, weight.grad

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for i in range(4):
        with torch.no_grad():  # eager work between the replays changes the inputs in place
            hidden.mul_(0.97)
            ref_c.add_(1.5)
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in captured]
        eager = step()
        torch.cuda.synchronize()
        for a, b in zip(got, eager):
            assert torch.equal(a, b), i


class _TinyCausalLM(torch.nn.Module):
    """HuggingFace-shaped stand-in: ``base_model`` returns ``last_hidden_state``, ``get_output_embeddings``
    the bias-free lm_head, the model itself ``.logits`` (and ``.aux_loss``)."""

    class _Out:
        def __init__(self, **kw):
            self.__dict__.update(kw)

    class _Trunk(torch.nn.Module):
        def __init__(self, vocab, hidden):
            super().__init__()
            self.embed = torch.nn.Embedding(vocab, hidden, dtype=torch.bfloat16)
            self.mix = torch.nn.Linear(hidden, hidden, bias=False, dtype=torch.bfloat16)

        def forward(self, input_ids, attention_mask=None, position_ids=None):
            h = self.embed(input_ids)
            h = h + torch.tanh(self.mix(h)) + (0.01 * position_ids.unsqueeze(-1).to(h.dtype) if position_ids is not None else 0)
            return _TinyCausalLM._Out(last_hidden_state=h)

    def __init__(self, vocab=300, hidden=64):
        super().__init__()
        self.model = self._Trunk(vocab, hidden)
        self.lm_head = torch.nn.Linear(hidden, vocab, bias=False, dtype=torch.bfloat16)

    @property
    def base_model(self):
        return self.model

    def get_output_embeddings(self):
        return self.lm_head

    def forward(self, input_ids, attention_mask=None, position_ids=None, output_router_logits=False):
        h = self.model(input_ids, attention_mask, position_ids).last_hidden_state
        return self._Out(logits=self.lm_head(h), aux_loss=None)


def test_fused_head_option_of_the_huggingface_call_paths():
    """``fused_head=True`` in forward_for_logprobs (open_instruct/grpo_utils.py:541-574), concatenated_forward
    and separate_forward (open_instruct/dpo_utils.py:826-956): trunk + fused lm_head instead of the model's
    logits, against the default routes and against the oracle on the model's own (bf16) logits, values and
    gradients of the trunk and of the lm_head weight."""
    torch.manual_seed(31)
    vocab, b, t = 300, 3, 17
    model = _TinyCausalLM(vocab).to(DEV)
    qr = torch.randint(1, vocab, (b, t), device=DEV)
    qr[0, -4:] = 0  # padding
    pos = torch.arange(t, device=DEV).unsqueeze(0).expand(b, -1)
    att = (qr != 0).long()
    resp = torch.zeros(b, t, dtype=torch.bool, device=DEV)
    resp[:, 6:] = True
    resp &= qr != 0

    def grads():
        out = [p.grad.float().clone() for p in model.parameters()]
        model.zero_grad()
        return out

    # GRPO: logprob / entropy of the next token
    lp_a, ent_a = grpo_utils.forward_for_logprobs(model, qr, att, pos, 0, 0.8, return_entropy=True)
    w = torch.randn(b, t - 1, device=DEV) * resp[:, 1:]
    (lp_a * w).sum().backward()
    g_a = grads()
    lp_b, ent_b = grpo_utils.forward_for_logprobs(
        model, qr, att, pos, 0, 0.8, return_entropy=True, fused_head=True, response_mask=resp
    )
    (lp_b * w).sum().backward()
    g_b = grads()
    keep = resp[:, 1:]
    with torch.no_grad():
        logits = model(qr, att, pos).logits
    e_lp, e_ent = o_grpo.forward_for_logprobs(logits.float().cpu(), qr.cpu(), 0, 0.8, True)
    # the default route rounds the logits to bf16 (the model's output dtype), the fused head does not
    assert (lp_a.detach().cpu() - e_lp).abs().max().item() <= 2e-3
    assert ((lp_b.detach() - lp_a.detach()) * keep).abs().max().item() <= 3e-2
    assert ((ent_b - ent_a) * keep).abs().max().item() <= 3e-2
    assert (lp_b[~keep] == 0).all() and (ent_b[~keep] == 0).all()
    for x, y in zip(g_a, g_b):
        assert (x - y).abs().max().item() <= 2e-2 * max(1e-3, x.abs().max().item())
    # fp32 check of the fused route against the same trunk output multiplied in fp32
    with torch.no_grad():
        h = model.base_model(qr, att, pos).last_hidden_state[:, :-1].float()
        z = (h @ model.lm_head.weight.float().T) / 0.8
        labels = qr[:, 1:].clone()
        ref = torch.log_softmax(z, -1).gather(-1, labels[..., None])[..., 0]
    assert ((lp_b.detach() - ref) * keep).abs().max().item() <= 2e-3

    # DPO: per-sequence logps, two forwards or one
    batch = {
        "chosen_input_ids": torch.randint(1, vocab, (2, 12), device=DEV), "rejected_input_ids": torch.randint(1, vocab, (2, 9), device=DEV),
        "chosen_attention_mask": torch.ones(2, 12, dtype=torch.long, device=DEV),
        "rejected_attention_mask": torch.ones(2, 9, dtype=torch.long, device=DEV),
    }  # fmt: skip
    batch["chosen_labels"] = batch["chosen_input_ids"].clone()
    batch["rejected_labels"] = batch["rejected_input_ids"].clone()
    batch["chosen_labels"][:, :4] = -100
    batch["rejected_labels"][:, :3] = -100
    for fn in (dpo_utils.concatenated_forward, dpo_utils.separate_forward):
        c0, r0, _ = fn(model, batch)
        (c0.sum() - r0.sum()).backward()
        g0 = grads()
        c1, r1, aux = fn(model, batch, fused_head=True)
        (c1.sum() - r1.sum()).backward()
        g1 = grads()
        assert aux is None and c1.requires_grad
        assert (c0 - c1).abs().max().item() <= 0.1 and (r0 - r1).abs().max().item() <= 0.1  # bf16 logits on one side
        for x, y in zip(g0, g1):
            assert (x - y).abs().max().item() <= 2e-2 * max(1e-3, x.abs().max().item())
        with pytest.raises(ValueError):
            fn(model, batch, output_router_logits=True, fused_head=True)
    with pytest.raises(TypeError):
        grpo_utils.forward_for_logprobs(torch.nn.Linear(4, 4), qr, att, pos, 0, 1.0, fused_head=True)
