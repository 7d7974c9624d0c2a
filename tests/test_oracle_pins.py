"""Pins the CPU oracle: reference known-answer vectors, closed forms, brute force in pure Python.

None of these tests retypes an oracle formula with the same library calls: brute force uses
``math`` on Python floats, closed forms are facts of the mathematics, and the known answers are
the reference's own test data (tests/golden/reference_known_answers.json).
"""

import math
import types

import numpy as np
import pytest
import torch

from conftest import make_grpo_config
from oracle import dpo, grpo, lm_head, logprob, reductions


# ---------------------------------------------------------------- logprob / entropy / kl
def _brute_logprob_entropy(row, idx, temperature=1.0):
    z = [float(v) / temperature for v in row]
    m = max(z)
    tot = sum(math.exp(v - m) for v in z)
    lse = m + math.log(tot)
    p = [math.exp(v - lse) for v in z]
    ent = -sum(pi * math.log(pi) for pi in p if pi > 0)
    return z[idx] - lse, ent


@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_logprob_and_entropy_brute_force(temperature):
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(3, 5, 11, generator=g, dtype=torch.float64) * 3
    idx = torch.randint(0, 11, (3, 5), generator=g)
    lp = logprob.log_softmax_and_gather(logits, idx, torch.float64, temperature)
    ent = logprob.entropy_from_logits(logits, torch.float64, temperature)
    for b in range(3):
        for t in range(5):
            e_lp, e_ent = _brute_logprob_entropy(logits[b, t].tolist(), int(idx[b, t]), temperature)
            assert abs(lp[b, t].item() - e_lp) < 1e-12
            assert abs(ent[b, t].item() - e_ent) < 1e-12


def test_logprob_invariants():
    g = torch.Generator().manual_seed(2)
    logits = torch.randn(4, 7, generator=g, dtype=torch.float64) * 5
    # probabilities over all indices sum to one; shifting the logits changes nothing
    all_lp = torch.stack([logprob.log_softmax_and_gather(logits, torch.full((4,), j), torch.float64) for j in range(7)])
    assert torch.allclose(all_lp.exp().sum(0), torch.ones(4, dtype=torch.float64), atol=1e-13)
    idx = torch.tensor([0, 3, 6, 2])
    a = logprob.log_softmax_and_gather(logits, idx, torch.float64)
    b = logprob.log_softmax_and_gather(logits + 123.25, idx, torch.float64)
    assert torch.allclose(a, b, atol=1e-12)
    assert (a <= 0).all()


def test_logprob_sliced_view_like_reference_test():
    # shape / sign / finiteness invariants of open_instruct/test_model_utils.py:49-64 at a smaller vocab
    g = torch.Generator().manual_seed(3)
    full = torch.randn(2, 17, 1000, generator=g)
    logits = full[:, :-1, :]
    index = torch.randint(0, 1000, (2, 17), generator=g)[:, 1:].clone()
    assert not logits.is_contiguous()
    out = logprob.log_softmax_and_gather(logits, index)
    assert out.shape == (2, 16) and (out <= 0).all() and torch.isfinite(out).all()


def test_entropy_closed_forms():
    v = 37
    uniform = torch.full((2, v), 1.5, dtype=torch.float64)
    assert torch.allclose(logprob.entropy_from_logits(uniform, torch.float64), torch.full((2,), math.log(v), dtype=torch.float64))
    peaked = torch.zeros(1, v, dtype=torch.float64)
    peaked[0, 4] = 200.0
    assert logprob.entropy_from_logits(peaked, torch.float64).item() == pytest.approx(0.0, abs=1e-12)
    g = torch.Generator().manual_seed(4)
    rnd = torch.randn(50, v, generator=g, dtype=torch.float64) * 4
    ent = logprob.entropy_from_logits(rnd, torch.float64)
    assert (ent >= 0).all() and (ent <= math.log(v) + 1e-12).all()


def test_estimate_kl_closed_forms_and_brute_force():
    d = torch.tensor([0.0, 0.3, -1.7, 40.0, -40.0], dtype=torch.float64)
    ratio = torch.tensor([1.0, 0.5, 2.0, 1.5, 0.1], dtype=torch.float64)
    k = logprob.estimate_kl(d, ratio)
    assert k.shape == (4, 5)
    assert k[:, 0].abs().max() == 0  # d = 0 -> every estimator is 0
    for i in range(5):
        di, ri = d[i].item(), ratio[i].item()
        assert k[0, i].item() == pytest.approx(di, abs=0)
        assert k[1, i].item() == pytest.approx(di * di / 2, rel=1e-15)
        assert k[2, i].item() == pytest.approx(math.expm1(-di) + di, rel=1e-14)
        assert k[3, i].item() == pytest.approx(ri * di, rel=1e-15)
    assert (k[2] >= 0).all()
    small = torch.tensor([1e-4], dtype=torch.float64)
    assert logprob.estimate_kl(small, small)[2].item() == pytest.approx(1e-8 / 2, rel=1e-3)  # Taylor: d^2/2


def test_calculate_per_token_logps_shift_brute_force():
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(2, 6, 9, generator=g)
    labels = torch.randint(0, 9, (2, 6), generator=g)
    labels[0, 3] = -100
    labels[1, -2:] = -100
    out = logprob.calculate_per_token_logps(logits, labels, torch.float64)
    assert out.dtype == torch.float64
    for b in range(2):
        for i in range(6):
            nxt = int(labels[b, i + 1]) if i + 1 < 6 else -100
            tgt = max(nxt, 0)  # ignored labels and the last position score token 0
            e_lp, _ = _brute_logprob_entropy(logits[b, i].double().tolist(), tgt)
            assert abs(out[b, i].item() - e_lp) < 1e-12
    # the reference always upcasts: fp32 result for bf16 logits
    assert logprob.calculate_per_token_logps(logits.bfloat16(), labels).dtype == torch.float32


# ---------------------------------------------------------------- reductions
def test_masked_mean_reference_known_answers(golden):
    for case in golden["masked_mean"]:
        out = reductions.masked_mean(torch.tensor(case["values"]), torch.tensor(case["mask"]), axis=case["axis"])
        exp = torch.tensor(case["expected"])
        assert out.shape == exp.shape, case["source"]
        assert torch.allclose(out, exp, rtol=1e-6, atol=0), case["source"]


def test_masked_mean_denominator_and_bool_mask():
    v = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    m = torch.tensor([[True, True, False], [True, False, False]])
    assert reductions.masked_mean(v, m, None, 10.0).item() == pytest.approx(0.7)
    assert reductions.masked_mean(v, m, None, 0.0).item() == 0.0
    assert reductions.masked_mean(v, m, 1, 2.0).item() == pytest.approx((3.0 / 2 + 4.0 / 2) / 2)
    assert reductions.masked_mean(v, m, -1).item() == pytest.approx(2.75)


def test_get_batch_logps_padded_known_answers(golden):
    for case in golden["get_batch_logps_padded_average"]:
        out = reductions.get_batch_logps_padded(
            torch.tensor(case["per_token_logps"]), torch.tensor(case["labels"]), average_log_prob=True
        )
        assert torch.equal(out, torch.tensor(case["expected"])), case["source"]


def _brute_packed(per_token, labels, cu, average):
    t_total = len(per_token)
    bounds = [c - 1 for c in cu]
    bounds[0] = 0
    s_count = len(cu) - 1
    sums, counts = [0.0] * s_count, [0.0] * s_count
    for t in range(t_total - 1):
        seg = sum(1 for b in bounds[1:] if b <= t)
        seg = min(seg, s_count - 1)
        if labels[t + 1] != -100:
            sums[seg] += per_token[t]
            counts[seg] += 1
    return [s / max(c, 1) for s, c in zip(sums, counts)] if average else sums


@pytest.mark.parametrize("average", [False, True])
def test_get_batch_logps_packed_brute_force_and_padded_equivalence(average):
    g = torch.Generator().manual_seed(6)
    lens = [5, 1, 9, 3, 7]
    rows, labs = [], []
    for n in lens:
        rows.append(torch.randn(n, generator=g, dtype=torch.float64))
        lab = torch.randint(0, 50, (n,), generator=g)
        lab[: max(1, n // 3)] = -100  # prompt part, first label always masked as in real DPO batches
        labs.append(lab)
    per_token = torch.cat(rows).unsqueeze(0)
    labels = torch.cat(labs).unsqueeze(0)
    cu = torch.tensor([0] + list(np.cumsum(lens)), dtype=torch.int32)
    packed = reductions.get_batch_logps_packed(per_token, labels, cu, average)
    brute = _brute_packed(per_token[0].tolist(), labels[0].tolist(), cu.tolist(), average)
    assert torch.allclose(packed, torch.tensor(brute, dtype=torch.float64), atol=1e-12)
    # same sequences as a padded batch give the same per-sequence values
    tmax = max(lens)
    pt = torch.zeros(len(lens), tmax, dtype=torch.float64)
    lb = torch.full((len(lens), tmax), -100)
    for i, n in enumerate(lens):
        pt[i, :n], lb[i, :n] = rows[i], labs[i]
    padded = reductions.get_batch_logps_padded(pt, lb, average)
    assert torch.allclose(packed, padded, atol=1e-12)


def test_packed_all_masked_segment_has_no_nan(golden):
    case = golden["packed_cu_seq_lens"]
    g = torch.Generator().manual_seed(7)
    logits = torch.randn(1, case["seq_len"], 100, generator=g)
    labels = torch.ones(1, case["seq_len"], dtype=torch.long)
    lo, hi = case["masked_label_range"]
    labels[0, lo:hi] = -100
    per_token = logprob.calculate_per_token_logps(logits, labels)
    out = reductions.get_batch_logps_packed(per_token, labels, torch.tensor(case["cu_seq_lens"]), True)
    assert out.shape[0] == case["expected_num_outputs"] and not torch.isnan(out).any()


# ---------------------------------------------------------------- grpo
def test_dapo_known_answers(golden):
    case = golden["dapo_clipping"]
    cfg = make_grpo_config(clip_lower=case["clip_lower"], clip_higher=case["clip_higher"])
    ratio = torch.tensor(case["ratio"])
    pg, clipfrac, kl = grpo.compute_grpo_loss(
        torch.randn(1, 3), ratio, torch.tensor(case["advantages"]), None, cfg, torch.ones_like(ratio)
    )
    assert torch.allclose(pg, torch.tensor(case["expected_pg_loss"]))
    assert torch.equal(clipfrac, torch.tensor(case["expected_clipfrac"]))
    assert torch.equal(kl, torch.zeros_like(kl))

    case = golden["dapo_negative_advantages"]
    cfg = make_grpo_config(clip_lower=case["clip_lower"], clip_higher=case["clip_higher"])
    ratio = torch.tensor(case["ratio"])
    adv = torch.full_like(ratio, case["advantage"])
    pg, _, _ = grpo.compute_grpo_loss(torch.zeros_like(ratio), ratio, adv, None, cfg, torch.ones_like(ratio))
    assert torch.allclose(pg, torch.tensor(case["expected_pg_loss"]))


def test_dapo_branch_grid_brute_force():
    lo_eps, hi_eps = 0.2, 0.28
    cfg = make_grpo_config(clip_lower=lo_eps, clip_higher=hi_eps)
    ratios = [0.5, 0.8, 0.9, 1.0, 1.28, 1.3, 2.0]
    advs = [-1.5, 0.0, 2.0]
    for a in advs:
        for r in ratios:
            rt = torch.tensor([[r]], dtype=torch.float64)
            pg, cf, _ = grpo.compute_grpo_loss(
                torch.zeros(1, 1, dtype=torch.float64), rt, torch.tensor([[a]], dtype=torch.float64), None, cfg,
                torch.ones(1, 1, dtype=torch.float64),
            )  # fmt: skip
            clamped = min(max(r, 1.0 - lo_eps), 1.0 + hi_eps)
            assert pg.item() == pytest.approx(max(-a * r, -a * clamped), abs=1e-15)
            assert cf.item() == (1.0 if -a * clamped > -a * r else 0.0)


def test_cispo_known_answers(golden):
    case = golden["cispo"]
    cfg = make_grpo_config(loss_fn="cispo", clip_higher=case["clip_higher"])
    ratio = torch.tensor(case["ratio"], requires_grad=True)
    new = torch.randn(1, 3, requires_grad=True)
    pg, clipfrac, _ = grpo.compute_grpo_loss(new, ratio, torch.tensor(case["advantages"]), None, cfg, torch.ones(1, 3))
    pg.sum().backward()
    assert (ratio.grad is not None) == case["ratio_gets_grad"]
    assert (new.grad is not None) == case["new_logprobs_gets_grad"]
    assert torch.equal(clipfrac, torch.tensor(case["expected_clipfrac"]))
    # value: -A * min(r, 1 + eps) * logp
    exp = -torch.tensor([[1.2, 0.5, 1.0]]) * new.detach()
    assert torch.allclose(pg.detach(), exp)


def test_grpo_rho_weights_kl_and_invalid_loss_fn():
    g = torch.Generator().manual_seed(8)
    new, adv = torch.randn(2, 4, generator=g), torch.randn(2, 4, generator=g)
    ratio = torch.randn(2, 4, generator=g).exp()
    cfg = make_grpo_config()
    pg1, cf1, kl0 = grpo.compute_grpo_loss(new, ratio, adv, None, cfg, torch.ones(2, 4))
    pg2, cf2, _ = grpo.compute_grpo_loss(new, ratio, adv, None, cfg, torch.full((2, 4), 2.0))
    assert torch.allclose(pg2, pg1 * 2) and torch.equal(cf1, cf2) and torch.equal(kl0, torch.zeros(2, 4))
    w = torch.tensor([[1.0, 0.0, 1.0, 1.0]] * 2)
    pg3, cf3, _ = grpo.compute_grpo_loss(new, ratio, adv, None, cfg, w)
    assert (pg3[:, 1] == 0).all() and (cf3[:, 1] == 0).all()
    ref = torch.randn(2, 4, generator=g)
    _, _, kl = grpo.compute_grpo_loss(new, ratio, adv, ref, cfg, torch.ones(2, 4))
    assert not (kl == 0).all() and (kl >= 0).all()
    with pytest.raises(ValueError):
        grpo.compute_grpo_loss(new, ratio, adv, None, make_grpo_config(loss_fn="invalid"), torch.ones(2, 4))


def test_rho_correction_known_answers(golden):
    case = golden["rho_mask"]
    cfg = make_grpo_config(use_rho_correction=True, rho_mask_lower_bound=case["mask_lower"], rho_mask_upper_bound=case["mask_upper"])
    old = torch.log(torch.tensor(case["rho"]))
    zeros, ones = torch.zeros_like(old), torch.ones_like(old)
    c = grpo.compute_rho_correction(old, zeros, torch.tensor(case["response_mask"]), ones, cfg)
    assert torch.allclose(c.weights, torch.tensor(case["expected_weights"]))
    assert torch.equal(c.metrics["val/rho_drop_low_frac"], torch.tensor(case["expected_drop_low"]))
    assert torch.equal(c.metrics["val/rho_drop_high_frac"], torch.tensor(case["expected_drop_high"]))
    c = grpo.compute_rho_correction(old, zeros, torch.tensor(case["response_mask_with_pad"]), ones, cfg)
    assert torch.allclose(c.weights, torch.tensor(case["expected_weights_with_pad"]))
    assert torch.equal(c.metrics["val/rho_drop_low_frac"], torch.tensor(case["expected_drop_low_with_pad"]))
    assert torch.equal(c.metrics["val/rho_drop_high_frac"], torch.tensor(case["expected_drop_high_with_pad"]))

    case = golden["rho_mask_sequence_level"]
    cfg = make_grpo_config(
        use_rho_correction=True, rho_mask_lower_bound=case["mask_lower"], rho_mask_upper_bound=case["mask_upper"],
        rho_mask_sequence_level=True,
    )  # fmt: skip
    old = torch.log(torch.tensor(case["rho"]))
    c = grpo.compute_rho_correction(old, torch.zeros_like(old), torch.ones_like(old, dtype=torch.bool), torch.ones_like(old), cfg)
    assert torch.allclose(c.weights, torch.tensor(case["expected_weights"]))
    assert torch.equal(c.metrics["val/rho_drop_low_frac"], torch.tensor(case["expected_drop_low"]))
    assert torch.equal(c.metrics["val/rho_drop_high_frac"], torch.tensor(case["expected_drop_high"]))

    case = golden["rho_mask_tv_divergence"]
    cfg = make_grpo_config(
        use_rho_correction=True, rho_mask_lower_bound=case["mask_lower"], rho_mask_upper_bound=case["mask_upper"],
        rho_mask_tv_divergence=True,
    )  # fmt: skip
    old = torch.log(torch.tensor(case["rho"]))
    c = grpo.compute_rho_correction(old, torch.zeros_like(old), torch.ones_like(old, dtype=torch.bool), torch.ones_like(old), cfg)
    assert torch.allclose(c.weights, torch.tensor(case["expected_weights"]))
    assert torch.equal(c.metrics["val/rho_drop_high_frac"], torch.tensor(case["expected_drop_high"]))


def test_rho_correction_disabled_and_properties():
    g = torch.Generator().manual_seed(9)
    old, vl = torch.randn(3, 6, generator=g), torch.randn(3, 6, generator=g)
    mask = torch.rand(3, 6, generator=g) > 0.3
    c = grpo.compute_rho_correction(old, vl, mask, torch.ones(3, 6), make_grpo_config())
    assert torch.equal(c.weights, torch.ones(3, 6)) and c.metrics == {}
    assert c.histogram_metrics["val/rho_hist"].numel() == int(mask.sum())
    cfg = make_grpo_config(use_rho_correction=True, rho_clamp_lower_bound=0.5, rho_clamp_upper_bound=2.0,
                           rho_mask_lower_bound=0.1, rho_mask_upper_bound=8.0)  # fmt: skip
    c = grpo.compute_rho_correction(old, vl, mask, torch.ones(3, 6), cfg)
    w = c.weights
    assert (w[~mask] == 0).all() and ((w == 0) | ((w >= 0.5) & (w <= 2.0))).all()


def test_mask_logprobs_all_masked_is_sentinel():
    lp = torch.tensor([[0.5, float("nan"), -3.0]])
    out = grpo.mask_logprobs(lp, torch.zeros(1, 3, dtype=torch.bool))
    assert (out == 1.0).all()
    out = grpo.mask_logprobs(lp, torch.ones(1, 3, dtype=torch.bool))
    assert out.tolist() == [[0.5, 1.0, -3.0]]


def test_group_advantages_against_loops():
    rng = np.random.default_rng(0)
    scores = (rng.random(64) < 0.3).astype(np.float64)
    scores[8:16] = 1.0  # a zero-variance group
    adv = grpo.group_advantages(scores, 8, "standard")
    for gidx in range(8):
        grp = scores[gidx * 8 : (gidx + 1) * 8].tolist()
        mean = sum(grp) / 8
        std = math.sqrt(sum((x - mean) ** 2 for x in grp) / 8)
        for k, x in enumerate(grp):
            assert adv[gidx * 8 + k] == pytest.approx((x - mean) / (std + 1e-8), rel=1e-12, abs=1e-15)
    assert (adv[8:16] == 0).all()
    cen = grpo.group_advantages(scores, 8, "centered")
    assert cen[0] == pytest.approx(scores[0] - scores[:8].mean())
    with pytest.raises(ValueError):
        grpo.group_advantages(scores, 8, "other")


def test_grpo_token_loss_composition_and_gradient():
    g = torch.Generator().manual_seed(10)
    new = torch.randn(3, 5, generator=g, dtype=torch.float64, requires_grad=True)
    old = new.detach() + 0.05 * torch.randn(3, 5, generator=g, dtype=torch.float64)
    ref = new.detach() + 0.1 * torch.randn(3, 5, generator=g, dtype=torch.float64)
    adv = torch.randn(3, 5, generator=g, dtype=torch.float64)
    mask = torch.rand(3, 5, generator=g) > 0.3
    cfg = make_grpo_config(clip_higher=0.28)
    loss, pg, _, kl, ratio = grpo.grpo_token_loss(new, old, ref, adv, mask, cfg)
    manual = ((pg + 0.05 * kl) * mask).sum() / mask.sum()
    assert loss.item() == pytest.approx(manual.item(), rel=1e-14)
    loss.backward()
    # hand-derived gradient: -A r on the unclipped branch (0 when clipped) + beta (1 - exp(-d))
    lo, hi = 0.8, 1.28
    r, a = ratio.detach(), adv
    clipped_active = (-a * r.clamp(lo, hi)) > (-a * r)
    dpg = torch.where(clipped_active, torch.zeros_like(r), -a * r)
    d = (new.detach() - ref).clamp(-40, 40)
    expect = mask * (dpg + 0.05 * (1 - torch.exp(-d))) / mask.sum()
    assert torch.allclose(new.grad, expect, atol=1e-14)


def test_forward_for_logprobs_shift_and_pad():
    g = torch.Generator().manual_seed(11)
    logits = torch.randn(2, 5, 10, generator=g, dtype=torch.float64)
    ids = torch.randint(1, 10, (2, 5), generator=g)
    ids[0, -1] = 7
    pad = 7
    lp, ent = grpo.forward_for_logprobs(logits, ids, pad, 0.8, True, torch.float64)
    assert lp.shape == (2, 4) and ent.shape == (2, 4) and (ent >= 0).all()
    for b in range(2):
        for i in range(4):
            tgt = int(ids[b, i + 1])
            tgt = 0 if tgt == pad else tgt
            e_lp, e_ent = _brute_logprob_entropy(logits[b, i].tolist(), tgt, 0.8)
            assert abs(lp[b, i].item() - e_lp) < 1e-12 and abs(ent[b, i].item() - e_ent) < 1e-12


# ---------------------------------------------------------------- dpo
def _brute_dpo(pc, pr, rc, rr, beta, ls):
    x = (pc - pr) - (rc - rr)
    lsig = lambda u: -math.log1p(math.exp(-u)) if u > -30 else u  # noqa: E731
    return -lsig(beta * x) * (1 - ls) - lsig(-beta * x) * ls


def test_dpo_loss_closed_forms_and_brute_force(golden):
    case = golden["dpo_loss_zero_margin"]
    losses, cr, rj = dpo.dpo_loss(
        torch.tensor(case["policy_chosen"]), torch.tensor(case["policy_rejected"]), torch.tensor(case["ref_chosen"]),
        torch.tensor(case["ref_rejected"]), beta=case["beta"],
    )  # fmt: skip
    assert torch.allclose(losses, torch.tensor(case["expected_losses"]), atol=1e-7)
    assert torch.equal(cr, torch.zeros(3)) and torch.equal(rj, torch.zeros(3))
    g = torch.Generator().manual_seed(12)
    pc, pr, rc, rr = (torch.randn(6, generator=g, dtype=torch.float64) * 20 - 300 for _ in range(4))
    for ls in (0.0, 0.1):
        out, _, _ = dpo.dpo_loss(pc, pr, rc, rr, beta=0.1, label_smoothing=ls)
        for i in range(6):
            assert out[i].item() == pytest.approx(_brute_dpo(pc[i].item(), pr[i].item(), rc[i].item(), rr[i].item(), 0.1, ls), rel=1e-12)
        # symmetry L(x, ls) = L(-x, 1 - ls)
        swapped, _, _ = dpo.dpo_loss(pr, pc, rr, rc, beta=0.1, label_smoothing=1 - ls)
        assert torch.allclose(out, swapped, atol=1e-13)


def test_dpo_loss_reference_test_properties():
    good, _, _ = dpo.dpo_loss(torch.tensor([0.0]), torch.tensor([-5.0]), torch.tensor([-1.0]), torch.tensor([-1.0]), 0.1)
    bad, _, _ = dpo.dpo_loss(torch.tensor([-5.0]), torch.tensor([0.0]), torch.tensor([-1.0]), torch.tensor([-1.0]), 0.1)
    assert good.item() < bad.item()
    a, _, _ = dpo.dpo_loss(torch.tensor([0.0]), torch.tensor([-1.0]), torch.tensor([-5.0]), torch.tensor([-10.0]), 0.1)
    b, _, _ = dpo.dpo_loss(torch.tensor([0.0]), torch.tensor([-1.0]), torch.tensor([-5.0]), torch.tensor([-10.0]), 0.1, reference_free=True)
    assert a.item() != b.item()
    pc = torch.tensor([0.0], requires_grad=True)
    pr = torch.tensor([-1.0], requires_grad=True)
    _, cr, rj = dpo.dpo_loss(pc, pr, torch.tensor([-1.0]), torch.tensor([-1.0]), 0.1)
    assert not cr.requires_grad and not rj.requires_grad


def _py_pair_loss(x: float, beta: float, ls: float) -> float:
    """-(1 - ls) log sigmoid(beta x) - ls log sigmoid(-beta x) on Python floats."""
    neg_log_sigmoid = lambda u: math.log1p(math.exp(-u)) if u > 0 else -u + math.log1p(math.exp(u))  # noqa: E731
    return (1 - ls) * neg_log_sigmoid(beta * x) + ls * neg_log_sigmoid(-beta * x)


def test_simpo_and_wpo_closed_forms():
    pc, pr = torch.tensor([-2.0, -1.0]), torch.tensor([-3.0, -4.0])
    out, cr, rj = dpo.simpo_loss(pc, pr, beta=2.0, gamma_beta_ratio=1.0)
    assert out[0].item() == pytest.approx(math.log(2.0), rel=1e-6)  # margin exactly cancels: x = 0
    assert torch.allclose(cr, 2.0 * pc) and torch.allclose(rj, 2.0 * pr)
    assert not cr.requires_grad and not rj.requires_grad


@pytest.mark.parametrize("label_smoothing", [0.0, 0.1, 0.5])
def test_simpo_loss_against_python_floats(label_smoothing):
    """open_instruct/dpo_utils.py:617-642 away from x = 0, with label smoothing, on both sides of the
    margin: every pair against a ``math.log1p`` evaluation on Python floats."""
    pc = [-2.0, -1.0, -30.0, -0.25, -7.5]
    pr = [-3.0, -4.0, -2.0, -0.75, -7.5]
    beta, gbr = 2.5, 0.6
    out, cr, rj = dpo.simpo_loss(torch.tensor(pc), torch.tensor(pr), beta, gbr, label_smoothing)
    for i in range(len(pc)):
        exp = _py_pair_loss(pc[i] - pr[i] - gbr, beta, label_smoothing)
        assert out[i].item() == pytest.approx(exp, rel=2e-6, abs=1e-6), i
        assert cr[i].item() == pytest.approx(beta * pc[i]) and rj[i].item() == pytest.approx(beta * pr[i])
    # the margin enters as a plain shift of the log-ratio
    shifted, _, _ = dpo.simpo_loss(torch.tensor(pc) - gbr, torch.tensor(pr), beta, 0.0, label_smoothing)
    assert torch.allclose(out, shifted, atol=1e-6)


@pytest.mark.parametrize("label_smoothing", [0.0, 0.2])
def test_wpo_loss_against_python_floats(label_smoothing):
    """open_instruct/dpo_utils.py:566-613 for one pair (the reference broadcasts the [bs] logps against
    the [bs, T] token masks, which only works for bs == 1, its shipped setting; there the "average"
    is logp * count / count = logp).  Cases on both sides of the clamp: exp(avg_c + avg_r) below 1
    (negative logps) and above 1 (a positive sum, where the weight must stop at 1); expected values
    from Python floats."""
    mask_c = torch.tensor([[True, True, False, True]])
    mask_r = torch.tensor([[True, False, False, False]])
    beta = 0.3
    for pc, pr, rc, rr in [(-0.2, -0.5, -0.4, -0.1), (0.9, -0.3, 0.1, -0.2), (1.5, 2.0, 1.0, 0.0), (-6.0, -9.0, -5.0, -5.0)]:
        out, cr, rj = dpo.wpo_loss(
            torch.tensor([pc]), torch.tensor([pr]), torch.tensor([rc]), torch.tensor([rr]), beta, mask_c, mask_r,
            label_smoothing,
        )  # fmt: skip
        weight = min(1.0, math.exp(pc + pr))
        exp = _py_pair_loss((pc - pr) - (rc - rr), beta, label_smoothing) * weight
        assert out.shape == (1,) and out.item() == pytest.approx(exp, rel=2e-6, abs=1e-7), (pc, pr)
        assert cr.item() == pytest.approx(beta * (pc - rc), abs=1e-6) and rj.item() == pytest.approx(beta * (pr - rr), abs=1e-6)
    # the weight is not detached in the reference: its gradient reaches the policy logps
    pc_t = torch.tensor([-0.2], requires_grad=True)
    out, _, _ = dpo.wpo_loss(pc_t, torch.tensor([-0.5]), torch.tensor([-0.4]), torch.tensor([-0.1]), beta, mask_c, mask_r)
    out.sum().backward()
    x = (-0.2 + 0.5) - (-0.4 + 0.1)
    w = math.exp(-0.7)
    d_loss_dx = -beta / (1 + math.exp(beta * x))
    assert pc_t.grad.item() == pytest.approx(w * d_loss_dx + w * _py_pair_loss(x, beta, 0.0), rel=1e-5)


# ---------------------------------------------------------------- lm_head
def test_lm_head_oracle_matches_materialised_product():
    g = torch.Generator().manual_seed(13)
    hidden = torch.randn(7, 16, generator=g).bfloat16()
    weight = (torch.randn(29, 16, generator=g) * 0.3).bfloat16()
    labels = torch.randint(0, 29, (7,), generator=g)
    labels[2] = -100
    lp, ent = lm_head.lm_head_logprobs(hidden, weight, labels, 0.9, True, torch.float64, row_chunk=3)
    for n in range(7):
        z = [sum(float(hidden[n, k]) * float(weight[v, k]) for k in range(16)) for v in range(29)]
        e_lp, e_ent = _brute_logprob_entropy(z, max(int(labels[n]), 0), 0.9)
        assert abs(lp[n].item() - e_lp) < 1e-10 and abs(ent[n].item() - e_ent) < 1e-10


def test_oracle_gradients_gradcheck():
    g = torch.Generator().manual_seed(14)
    logits = torch.randn(2, 3, 6, generator=g, dtype=torch.float64, requires_grad=True)
    idx = torch.randint(0, 6, (2, 3), generator=g)
    assert torch.autograd.gradcheck(lambda z: logprob.log_softmax_and_gather(z, idx, None, 0.7), (logits,))
    # closed form: d logp / d z_j = (1[j == y] - p_j) / T
    lp = logprob.log_softmax_and_gather(logits, idx, None, 0.7)
    (grad,) = torch.autograd.grad(lp.sum(), logits)
    p = torch.softmax(logits.detach() / 0.7, -1)
    onehot = torch.nn.functional.one_hot(idx, 6).double()
    assert torch.allclose(grad, (onehot - p) / 0.7, atol=1e-13)
    pc = torch.randn(4, generator=g, dtype=torch.float64, requires_grad=True)
    pr = torch.randn(4, generator=g, dtype=torch.float64, requires_grad=True)
    rc, rr = torch.randn(4, generator=g, dtype=torch.float64), torch.randn(4, generator=g, dtype=torch.float64)
    assert torch.autograd.gradcheck(lambda a, b: dpo.dpo_loss(a, b, rc, rr, 0.5, False, 0.1)[0], (pc, pr))


def test_linear_cross_entropy_against_hf_loss_and_brute_force():
    """The SFT loss is computed inside third-party code in the reference (HF model forward,
    open_instruct/finetune.py:818-824).  transformers ships in this image, so the oracle is pinned
    against ``ForCausalLMLoss`` itself, and against an explicit per-token loop."""
    import math

    g = torch.Generator().manual_seed(21)
    b, t, h, v = 2, 7, 8, 11
    hidden = torch.randn(b, t, h, generator=g)
    weight = torch.randn(v, h, generator=g)
    labels = torch.randint(0, v, (b, t), generator=g)
    labels[0, :3] = -100
    labels[1, -1] = -100
    got_mean = lm_head.linear_cross_entropy(hidden, weight, labels)
    got_sum = lm_head.linear_cross_entropy(hidden, weight, labels, num_items_in_batch=5)
    # brute force: position i predicts labels[i + 1]
    total, count = 0.0, 0
    for bi in range(b):
        for i in range(t - 1):
            y = int(labels[bi, i + 1])
            if y == -100:
                continue
            z = [sum(float(hidden[bi, i, k]) * float(weight[j, k]) for k in range(h)) for j in range(v)]
            mx = max(z)
            lse = mx + math.log(sum(math.exp(x - mx) for x in z))
            total += lse - z[y]
            count += 1
    assert abs(got_mean.item() - total / count) < 1e-5
    assert abs(got_sum.item() - total / 5) < 1e-5
    hf = pytest.importorskip("transformers.loss.loss_utils")
    logits = lm_head.lm_head_logits(hidden, weight)
    assert abs(hf.ForCausalLMLoss(logits, labels, v).item() - got_mean.item()) < 1e-6
    assert abs(hf.ForCausalLMLoss(logits, labels, v, num_items_in_batch=5).item() - got_sum.item()) < 1e-6


def test_vllm_local_debug_metrics_against_python_statistics():
    """open_instruct/grpo_utils.py:345-369 restated; checked with the statistics module."""
    import math
    import statistics

    g = torch.Generator().manual_seed(22)
    local = -torch.rand(3, 9, generator=g) * 5
    vllm = local + 0.1 * torch.randn(3, 9, generator=g)
    vllm[0, 2] = float("nan")
    mask = torch.rand(3, 9, generator=g) > 0.3
    mask[0, 2] = True
    got = grpo.compute_vllm_local_debug_metrics(local, vllm, mask)
    diffs, rkls = [], []
    for i in range(3):
        for j in range(9):
            if mask[i, j] and not math.isnan(float(vllm[i, j])):
                lo, vl = float(local[i, j]), float(vllm[i, j])
                diffs.append(abs(lo - vl))
                rkls.append(math.exp(vl) * (vl - lo))
    assert abs(got["debug/vllm_vs_local_logprob_diff_mean"] - statistics.fmean(diffs)) < 1e-6
    assert abs(got["debug/vllm_vs_local_logprob_diff_max"] - max(diffs)) < 1e-6
    assert abs(got["debug/vllm_vs_local_logprob_diff_std"] - statistics.stdev(diffs)) < 1e-6
    assert abs(got["debug/vllm_local_reverse_kl"] - statistics.fmean(rkls)) < 1e-6
    empty = grpo.compute_vllm_local_debug_metrics(local, vllm, torch.zeros_like(mask))
    assert all(x == 0.0 for x in empty.values())
    one = torch.zeros_like(mask)
    one[1, 1] = True
    single = grpo.compute_vllm_local_debug_metrics(local, vllm, one)
    assert single["debug/vllm_vs_local_logprob_diff_std"] == 0.0
    assert abs(single["debug/vllm_vs_local_logprob_diff_mean"] - abs(float(local[1, 1] - vllm[1, 1]))) < 1e-7


def test_pack_sequences_reference_vectors_and_properties(golden):
    """open_instruct/test_rl_utils.py:98-158,299-334: known masks of the tool-use test, packed rows
    hold query + response back to back, min_num_batches splits further without losing tokens."""
    from oracle import packing

    case = golden["pack_sequences_mask_tool_use"]
    args = (case["queries"], case["responses"], case["masks"], case["pack_length"], case["pad_token_id"], case["vllm_logprobs"])
    for flag, key in ((True, "with_masking"), (False, "without_masking")):
        out = packing.pack_sequences(*args, mask_tool_use=flag)
        assert out["query_responses"] == case["expected_query_responses"]
        assert [[m != 0 for m in row] for row in out["response_masks"]] == case[key]
    # three pairs; the first two fit one row, the third starts a new one (test_rl_utils.py:98-115)
    queries = [[5, 6, 7, 8], [9, 10, 11], [12, 13]]
    responses = [[20, 21, 22], [23], [24, 25, 26, 27]]
    masks = [[1] * len(r) for r in responses]
    lps = [[-0.5] * len(r) for r in responses]
    out = packing.pack_sequences(queries, responses, masks, 12, 0, lps)
    assert out["query_responses"] == [[5, 6, 7, 8, 20, 21, 22, 9, 10, 11, 23], [12, 13, 24, 25, 26, 27]]
    assert out["attention_masks"] == [[1] * 7 + [2] * 4, [1] * 6]
    assert out["position_ids"] == [[0, 1, 2, 3, 4, 5, 6, 0, 1, 2, 3], [0, 1, 2, 3, 4, 5]]
    assert out["response_masks"] == [[0, 0, 0, 0, 1, 1, 1, 0, 0, 0, 2], [0, 0, 3, 3, 3, 3]]
    assert out["dones"] == [[0, 0, 0, 0, 0, 0, 1, 0, 0, 0, 2], [0, 0, 0, 0, 0, 3]]
    assert out["num_actions"] == [[3, 1], [4]] and out["packed_seq_lens"] == [[7, 4], [6]]
    assert all(math.isnan(x) for x in out["vllm_logprobs"][0][:4]) and out["vllm_logprobs"][0][4:7] == [-0.5] * 3
    split = packing.pack_sequences(queries, responses, masks, 12, 0, lps, min_num_batches=3)
    assert len(split["query_responses"]) == 3 and all(len(r) > 0 for r in split["query_responses"])
    assert sum(len(r) for r in split["query_responses"]) == sum(len(r) for r in out["query_responses"])
    # padding tokens inside a response are dropped together with their mask and logprob entries
    padded = packing.pack_sequences([[1]], [[7, 0, 8, 0]], [[1, 1, 0, 1]], 16, 0, [[-1.0, -2.0, -3.0, -4.0]], mask_tool_use=True)
    assert padded["query_responses"] == [[1, 7, 8]] and padded["response_masks"] == [[0, 1, 0]]
    assert padded["vllm_logprobs"][0][1:] == [-1.0, -3.0] and padded["num_actions"] == [[2]]
    # a sequence longer than the row length still gets a row of its own
    long = packing.pack_sequences([[1, 2]], [[3, 4, 5, 6]], [[1] * 4], 3, 0, [[0.0] * 4])
    assert long["query_responses"] == [[1, 2, 3, 4, 5, 6]]
    assert packing.broadcast_advantages([0.5, -1.5, 2.0], out["response_masks"]) == [
        [0, 0, 0, 0, 0.5, 0.5, 0.5, 0, 0, 0, -1.5], [0, 0, 2.0, 2.0, 2.0, 2.0],
    ]  # fmt: skip


def test_loss_stat_helpers_by_hand():
    """open_instruct/grpo_utils.py:674-742 on numbers small enough to average by hand: three kept
    tokens, KL entries only with a reference policy, rho entries only when given, weighted summary."""
    cfg = types.SimpleNamespace(load_ref_policy=True, kl_estimator=1, beta=0.5)
    mask = torch.tensor([[True, True, False, True]])
    pg = torch.tensor([[1.0, 2.0, 100.0, 6.0]])
    clip = torch.tensor([[1.0, 0.0, 1.0, 0.0]])
    ratio = torch.tensor([[1.0, 2.0, 50.0, 3.0]])
    new = torch.tensor([[0.0, -1.0, 0.0, -2.0]])
    ref = torch.tensor([[-1.0, -1.0, 5.0, 0.0]])  # d = [1, 0, ., -2]
    ent = torch.tensor([[3.0, 3.0, 9.0, 6.0]])
    stats = grpo.create_loss_stats(2, record_entropy=True)
    assert set(stats) == set(grpo.LOSS_STAT_KEYS) | {"policy/entropy_avg"} and len(stats) == 15
    grpo.populate_sample_loss_stats(stats, 1, pg, clip, ratio, torch.tensor(7.5), mask, new, ref, ent, cfg)
    exp = {
        "loss/policy_avg": 3.0, "policy/clipfrac_avg": 1 / 3, "val/ratio": 2.0, "loss/total_avg": 7.5,
        "policy/entropy_avg": 4.0, "objective/kl0_avg": (1 + 0 - 2) / 3, "objective/kl1_avg": (0.5 + 0 + 2.0) / 3,
        "objective/kl2_avg": (math.expm1(-1) + 1 + 0 + math.expm1(2) - 2) / 3,
        "objective/kl3_avg": (1 * 1 + 2 * 0 + 3 * -2) / 3, "loss/kl_avg": 0.5 * (0.5 + 0 + 2.0) / 3,
    }  # fmt: skip
    for key, value in stats.items():
        assert value[0].item() == 0.0, key  # the other sample is untouched
        assert value[1].item() == pytest.approx(exp.get(key, 0.0), rel=1e-6, abs=1e-7), key
    # without a reference policy the KL entries stay zero even when reference logprobs are passed
    cfg2 = types.SimpleNamespace(load_ref_policy=False, kl_estimator=1, beta=0.5)
    stats2 = grpo.create_loss_stats(1)
    rho = {"val/rho_weight": torch.tensor([[2.0, 0.0, 9.0, 1.0]]), "val/rho_drop_frac": torch.tensor([[0.0, 1.0, 1.0, 0.0]])}
    grpo.populate_sample_loss_stats(stats2, 0, pg, clip, ratio, torch.tensor(1.0), mask, new, ref, None, cfg2, rho)
    assert stats2["objective/kl1_avg"][0].item() == 0.0 and stats2["loss/kl_avg"][0].item() == 0.0
    assert "policy/entropy_avg" not in stats2
    assert stats2["val/rho_weight"][0].item() == pytest.approx(1.0)
    assert stats2["val/rho_drop_frac"][0].item() == pytest.approx(1 / 3)
    assert stats2["val/rho_clipfrac"][0].item() == 0.0
    summary = grpo.compute_metrics_from_loss_stats(
        {"val/ratio": torch.tensor([1.0, 3.0]), "loss/total_avg": torch.tensor([2.0, 4.0])}, torch.tensor([1.0, 3.0])
    )
    assert summary["val/ratio"] == pytest.approx(2.5) and summary["loss/total_avg"] == pytest.approx(3.5)
    assert summary["val/ratio_var"] == pytest.approx(0.25 * 1.5**2 + 0.75 * 0.5**2)
    assert grpo.compute_metrics_from_loss_stats({"val/ratio": torch.ones(2)}, torch.zeros(2))["val/ratio"] == 0.0
