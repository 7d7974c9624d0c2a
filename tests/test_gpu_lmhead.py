"""GPU parity: fused lm_head + logprob/entropy (bf16 MFMA, logits never materialised), forward and
backward, against the CPU oracle (fp32 F.linear on the upcast bf16 inputs + logsumexp).

Tolerance 2e-3 abs for logprob / entropy / gradients (bf16 inputs, fp32 accumulation).
"""

import math

import pytest
import torch

from open_instruct_amd import _lib, lm_head
from open_instruct_amd.olmo_core_train_modules import DPOLMHead
from oracle import lm_head as o_lm
from oracle import logprob as o_logprob

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 2e-3


def _case(n, h, v, seed, w_scale=None):
    g = torch.Generator().manual_seed(seed)
    hidden = torch.randn(n, h, generator=g).bfloat16()
    weight = (torch.randn(v, h, generator=g) * (w_scale or 1.0 / math.sqrt(h))).bfloat16()
    labels = torch.randint(0, v, (n,), generator=g)
    return hidden, weight, labels


@pytest.mark.parametrize(
    "n,h,v",
    [
        (256, 64, 256),  # exactly one tile
        (300, 128, 1000),  # ragged tokens and vocabulary
        (1, 64, 50),  # single row, tiny vocabulary
        (700, 256, 5000),  # several token tiles, partial last vocabulary tile
        (513, 192, 20000),  # several splits of the vocabulary
    ],
)
@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_forward_matches_oracle(n, h, v, temperature):
    print(f"case N={n} H={h} V={v} T={temperature}", flush=True)
    hidden, weight, labels = _case(n, h, v, seed=0, w_scale=3.0 / math.sqrt(h))
    labels[0] = v - 1
    if n > 2:
        labels[1], labels[2] = 0, -100
    exp_lp, exp_ent = o_lm.lm_head_logprobs(hidden, weight, labels, temperature, True)
    lp, ent = lm_head.fused_lm_head_logprobs(hidden.to(DEV), weight.to(DEV), labels.to(DEV), temperature, return_entropy=True)
    assert lp.dtype == torch.float32 and lp.shape == (n,)
    assert (lp.cpu() - exp_lp).abs().max().item() <= TOL
    assert (ent.cpu() - exp_ent).abs().max().item() <= TOL
    lp2, none = lm_head.fused_lm_head_logprobs(hidden.to(DEV), weight.to(DEV), labels.to(DEV), temperature)
    assert none is None and torch.equal(lp2, lp)  # deterministic, run to run


@pytest.mark.parametrize(
    "n,h,v",
    [
        (256, 64, 256),
        (300, 128, 1000),
        (700, 256, 5000),
        (260, 64, 17000),
        (260, 64, 33000),  # two vocabulary chunks, the second with 232 of 256 real rows
        (260, 64, 70000),  # three chunks: d_hidden accumulates in fp32 over a middle chunk
        (130, 128, 100000),  # four chunks, the last with 1696 columns
        (40, 64, 50),  # one k-tile in both backward products, most of its rows missing
        (100, 64, 100),  # two k-tiles
        (130, 128, 150),  # three k-tiles
        (2, 64, 7),
        (300, 320, 1000),  # hidden size between one and two tiles wide: clamped column chunks
        (130, 192, 300),
    ],
)
@pytest.mark.parametrize("route", ["d_weight", "d_hidden_recomputed", "d_hidden_in_forward"])
def test_backward_matches_oracle(n, h, v, route):
    """d_hidden and d_weight by recomputation, d_hidden alone by recomputation, and d_hidden alone
    from the weighted sum of weight rows that the forward accumulates (the default without d_weight)."""
    print(f"case N={n} H={h} V={v} route={route}", flush=True)
    want_dw = route == "d_weight"
    hidden, weight, labels = _case(n, h, v, seed=1, w_scale=3.0 / math.sqrt(h))
    g = torch.Generator().manual_seed(2)
    upstream = torch.randn(n, generator=g)
    upstream[::3] = 0.0  # masked-out tokens
    rh = hidden.float().requires_grad_(True)
    rw = weight.float().requires_grad_(True)
    lp, _ = o_lm.lm_head_logprobs(rh, rw, labels, 0.9)
    lp.backward(upstream)
    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(want_dw)
    out, ent = lm_head.fused_lm_head_logprobs(
        dh, dw, labels.to(DEV), 0.9, return_entropy=True, dhidden_in_forward=route == "d_hidden_in_forward"
    )
    assert (out.detach().cpu() - lp.detach()).abs().max().item() <= TOL
    exp_ent = o_lm.lm_head_logprobs(hidden, weight, labels, 0.9, True)[1]
    assert (ent.cpu() - exp_ent).abs().max().item() <= TOL
    out.backward(upstream.to(DEV))
    assert dh.grad.dtype == torch.bfloat16 and dh.grad.shape == hidden.shape
    # bf16 outputs: allow one bf16 rounding of the largest entry on top of the absolute tolerance
    tol_h = TOL + rh.grad.abs().max().item() * 2**-7
    assert (dh.grad.float().cpu() - rh.grad).abs().max().item() <= tol_h
    assert (dh.grad[::3] == 0).all()
    if want_dw:
        tol_w = TOL + rw.grad.abs().max().item() * 2**-7
        err = (dw.grad.float().cpu() - rw.grad).abs().max().item()
        assert err <= tol_w, (err, tol_w)
        # relative check on the aggregate, so a dropped chunk or a transposed operand cannot hide
        rel = (dw.grad.float().cpu() - rw.grad).norm() / rw.grad.norm()
        assert rel.item() <= 2e-2, rel.item()
    else:
        assert dw.grad is None
    rel = (dh.grad.float().cpu() - rh.grad).norm() / rh.grad.norm()
    assert rel.item() <= 2e-2, rel.item()


def test_mask_compaction_and_leading_shape():
    hidden, weight, labels = _case(6 * 50, 64, 700, seed=3)
    hidden3, labels2 = hidden.reshape(6, 50, 64), labels.reshape(6, 50)
    g = torch.Generator().manual_seed(4)
    mask = torch.rand(6, 50, generator=g) > 0.3
    exp_lp, exp_ent = o_lm.lm_head_logprobs(hidden, weight, labels, 1.0, True)
    dh = hidden3.to(DEV).requires_grad_(True)
    lp, ent = lm_head.fused_lm_head_logprobs(dh, weight.to(DEV), labels2.to(DEV), mask=mask.to(DEV), return_entropy=True)
    assert lp.shape == (6, 50) and ent.shape == (6, 50)
    assert ((lp.cpu() - exp_lp.reshape(6, 50)) * mask).abs().max().item() <= TOL
    assert ((ent.cpu() - exp_ent.reshape(6, 50)) * mask).abs().max().item() <= TOL
    assert (lp.cpu()[~mask] == 0).all()
    lp.sum().backward()
    assert (dh.grad.cpu()[~mask] == 0).all() and dh.grad.cpu()[mask].abs().sum() > 0


@pytest.mark.parametrize("n,h,v", [(300, 128, 1000), (520, 64, 40000)])
def test_d_hidden_in_forward_with_mask_and_confident_tokens(n, h, v):
    """The d_hidden-only route with a row mask (compact rows of the weighted sum, rebuilt selection in
    the backward) and with tokens whose label has probability close to 1 (their gradient is the small
    difference 1 - p: the label's term is evaluated from the fp32 logprob, not from bf16 exponentials)."""
    print(f"case N={n} H={h} V={v}", flush=True)
    hidden, weight, labels = _case(n, h, v, seed=11, w_scale=2.0 / math.sqrt(h))
    # make every fifth token confident: its hidden row points along its label's weight row
    for i in range(0, n, 5):
        wy = weight[labels[i]].float()
        hidden[i] = (wy * (math.log(300.0 * v) / wy.pow(2).sum())).bfloat16()  # p(label) around 0.97-0.99
    g = torch.Generator().manual_seed(12)
    mask = torch.rand(n, generator=g) > 0.35
    upstream = torch.randn(n, generator=g)
    rh = hidden.float().requires_grad_(True)
    lp, _ = o_lm.lm_head_logprobs(rh, weight.float(), labels, 1.0)
    (lp * mask).backward(upstream)
    p_conf = lp.detach()[::5].exp()
    assert 0.9 < p_conf.min().item() and p_conf.max().item() < 0.9999  # confident, and 1 - p still well inside fp32
    for route in (True, False):
        dh = hidden.to(DEV).requires_grad_(True)
        out, _ = lm_head.fused_lm_head_logprobs(
            dh, weight.to(DEV), labels.to(DEV), mask=mask.to(DEV), dhidden_in_forward=route
        )
        assert ((out.detach().cpu() - lp.detach()) * mask).abs().max().item() <= TOL
        out.backward(upstream.to(DEV))
        got = dh.grad.float().cpu()
        assert (got[~mask] == 0).all()
        tol = TOL + rh.grad.abs().max().item() * 2**-7
        assert (got - rh.grad).abs().max().item() <= tol, route
        # relative, per confident token: the small gradient itself must be right, not only small
        conf = torch.arange(0, n, 5)
        conf = conf[mask[conf]]
        rel = (got[conf] - rh.grad[conf]).norm(dim=1) / rh.grad[conf].norm(dim=1).clamp(min=1e-12)
        assert rel.max().item() <= 3e-2, (route, rel.max().item())


def test_d_hidden_in_forward_is_the_default_without_d_weight():
    hidden, weight, labels = _case(300, 64, 700, seed=13)
    grads = {}
    for route in ("auto", True, False):
        dh = hidden.to(DEV).requires_grad_(True)
        out, _ = lm_head.fused_lm_head_logprobs(dh, weight.to(DEV), labels.to(DEV), dhidden_in_forward=route)
        out.sum().backward()
        grads[route] = dh.grad.clone()
    assert torch.equal(grads["auto"], grads[True])  # bit-equal: the same kernels ran
    assert not torch.equal(grads[True], grads[False])  # the recomputing route rounds differently ...
    assert (grads[True].float() - grads[False].float()).abs().max().item() <= TOL  # ... and agrees
    with pytest.raises(ValueError):
        lm_head.fused_lm_head_logprobs(
            hidden.to(DEV).requires_grad_(True), weight.to(DEV), labels.to(DEV), dhidden_in_forward=True,
            compact_backward=True,
        )


def test_no_grad_forward_prepares_nothing_for_a_backward():
    """Under torch.no_grad() (scoring passes, the reference-logprob cache build: open_instruct/dpo_utils.py:405-520)
    the forward is the plain one even when ``hidden`` is a tensor that requires a gradient and the weight is
    frozen: the weighted sum for a backward that never comes would double the matrix work.  Seen through the
    scratch it would allocate (a [tokens, 65536] bf16 chunk and an fp32 [tokens, hidden] sum)."""
    hidden, weight, labels = _case(2048, 256, 70000, seed=14)
    dh, w, lab = hidden.to(DEV).requires_grad_(True), weight.to(DEV), labels.to(DEV)
    out_grad, _ = lm_head.fused_lm_head_logprobs(dh, w, lab)
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    before = torch.cuda.memory_allocated()
    with torch.no_grad():
        out, _ = lm_head.fused_lm_head_logprobs(dh, w, lab)
    torch.cuda.synchronize()
    assert torch.cuda.max_memory_allocated() - before < 64 << 20  # the chunk alone would be 268 MB
    assert not out.requires_grad and (out - out_grad.detach()).abs().max().item() <= 1e-5


def test_dpo_lm_head_matches_calculate_per_token_logps():
    """open_instruct/test_padding_free_collator.py:366-399 with the fused head."""
    torch.manual_seed(42)
    d_model, vocab, seq, batch = 64, 320, 10, 2
    head = DPOLMHead(d_model=d_model, vocab_size=vocab, bias=False).to(DEV)
    x = torch.randn(batch, seq, d_model, device=DEV).bfloat16()
    labels = torch.randint(0, vocab, (batch, seq), device=DEV)
    labels[0, -2:] = -100
    output = head(x, labels=labels)
    with torch.no_grad():
        raw = head.w_out(x)
    expected = o_logprob.calculate_per_token_logps(
        torch.nn.functional.linear(x.float().cpu(), head.w_out.weight.detach().float().cpu()), labels.cpu()
    )
    assert output.logits is None and output.z_loss is None
    assert output.loss.shape == (batch, seq) and output.loss.requires_grad and not output.ce_loss.requires_grad
    # positions whose next label is ignored are not multiplied: 0 there, the reference's value elsewhere
    kept = (o_logprob.shift_labels(labels.cpu()) != -100)
    assert ((output.loss.detach().cpu() - expected) * kept).abs().max().item() <= TOL
    assert (output.loss.detach().cpu()[~kept] == 0).all() and (~kept).sum() == 2 + batch
    head.score_ignored_positions = True  # the reference's numbers at the ignored positions too
    assert (head(x, labels=labels).loss.detach().cpu() - expected).abs().max().item() <= TOL
    head.score_ignored_positions = False
    logits = head(x[:1], labels=None)
    assert isinstance(logits, torch.Tensor) and logits.shape == (1, seq, vocab) and torch.equal(logits, raw[:1])


def test_fused_equals_materialised_path_on_device():
    """A mid-sized shape where the CPU oracle would be slow: the fused kernel must agree with the
    row-wise kernel run on logits materialised by a library GEMM in fp32."""
    from open_instruct_amd import model_utils

    n, h, v = 2048, 1024, 32000
    torch.manual_seed(0)
    hidden = torch.randn(n, h, device=DEV).bfloat16()
    weight = (torch.randn(v, h, device=DEV) * 0.02).bfloat16()
    labels = torch.randint(0, v, (n,), device=DEV)
    logits = hidden.float() @ weight.float().t()
    exp_lp, exp_ent = model_utils.logprob_and_entropy(logits, labels)
    lp, ent = lm_head.fused_lm_head_logprobs(hidden, weight, labels, return_entropy=True)
    assert (lp - exp_lp).abs().max().item() <= TOL
    assert (ent - exp_ent).abs().max().item() <= TOL


@pytest.mark.parametrize("num_items", [None, 37])
def test_fused_linear_cross_entropy_matches_oracle(num_items):
    """Supervised fine-tuning loss through the fused head (open_instruct/finetune.py:818-824):
    value and both gradients against F.cross_entropy on the fp32 product."""
    from oracle import lm_head as o_head

    torch.manual_seed(9)
    b, t, h, v = 3, 40, 128, 3000
    hidden = torch.randn(b, t, h).bfloat16()
    weight = (torch.randn(v, h) * 2.0 / math.sqrt(h)).bfloat16()
    labels = torch.randint(0, v, (b, t))
    labels[:, :6] = -100
    labels[2, 25:] = -100
    rh = hidden.float().requires_grad_(True)
    rw = weight.float().requires_grad_(True)
    exp = o_head.linear_cross_entropy(rh, rw, labels, num_items_in_batch=num_items)
    exp.backward()
    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(True)
    got = lm_head.fused_linear_cross_entropy(dh, dw, labels.to(DEV), num_items_in_batch=num_items)
    got.backward()
    assert got.dtype == torch.float32 and got.ndim == 0
    assert abs(got.item() - exp.item()) <= TOL
    assert (dh.grad.float().cpu() - rh.grad).abs().max().item() <= TOL + rh.grad.abs().max().item() * 2**-7
    assert (dw.grad.float().cpu() - rw.grad).abs().max().item() <= TOL + rw.grad.abs().max().item() * 2**-7
    assert ((dw.grad.float().cpu() - rw.grad).norm() / rw.grad.norm()).item() <= 2e-2
    # the same loss and gradients in token slabs (one call, nothing recomputed)
    dh3 = hidden.to(DEV).requires_grad_(True)
    dw3 = weight.to(DEV).requires_grad_(True)
    got3 = lm_head.fused_linear_cross_entropy(dh3, dw3, labels.to(DEV), num_items_in_batch=num_items, token_slabs=True)
    got3.backward()
    assert abs(got3.item() - exp.item()) <= TOL
    assert (dh3.grad.float().cpu() - rh.grad).abs().max().item() <= TOL + rh.grad.abs().max().item() * 2**-7
    assert (dw3.grad.float().cpu() - rw.grad).abs().max().item() <= TOL + rw.grad.abs().max().item() * 2**-7
    assert ((dw3.grad.float().cpu() - rw.grad).norm() / rw.grad.norm()).item() <= 2e-2
    assert ((dh3.grad.float().cpu() - rh.grad).norm() / rh.grad.norm()).item() <= 2e-2
    # already shifted labels give the same loss
    shifted = torch.full_like(labels, -100)
    shifted[:, :-1] = labels[:, 1:]
    again = lm_head.fused_linear_cross_entropy(dh, dw, shift_labels=shifted.to(DEV), num_items_in_batch=num_items)
    assert torch.equal(again, got)
    with pytest.raises(ValueError):
        lm_head.fused_linear_cross_entropy(dh, dw)
    # nothing to score: zero loss, no NaN
    empty = lm_head.fused_linear_cross_entropy(dh, dw, torch.full_like(labels, -100).to(DEV))
    assert empty.item() == 0.0


def test_compact_backward_leaves_gradients_unchanged():
    """Rows with an exactly zero upstream gradient may be left out of the backward products."""
    hidden, weight, labels = _case(600, 128, 3000, seed=11, w_scale=3.0 / math.sqrt(128))
    g = torch.Generator().manual_seed(12)
    upstream = torch.randn(600, generator=g)
    upstream[torch.rand(600, generator=g) < 0.6] = 0.0
    grads = []
    for compact in (False, True):
        dh = hidden.to(DEV).requires_grad_(True)
        dw = weight.to(DEV).requires_grad_(True)
        out, _ = lm_head.fused_lm_head_logprobs(dh, dw, labels.to(DEV), 0.9, compact_backward=compact)
        out.backward(upstream.to(DEV))
        grads.append((dh.grad.float().cpu(), dw.grad.float().cpu()))
    (h0, w0), (h1, w1) = grads
    assert torch.equal(h0[upstream == 0], torch.zeros_like(h0[upstream == 0])) and torch.equal(h1[upstream == 0], h0[upstream == 0])
    assert (h0 - h1).abs().max().item() <= h0.abs().max().item() * 2**-7
    assert (w0 - w1).abs().max().item() <= w0.abs().max().item() * 2**-7 + 1e-6
    # nothing to propagate at all
    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(True)
    out, _ = lm_head.fused_lm_head_logprobs(dh, dw, labels.to(DEV), compact_backward=True)
    out.backward(torch.zeros(600, device=DEV))
    assert not dh.grad.any() and not dw.grad.any()


@pytest.mark.parametrize("keep", ["none", "one", "all", "random", "last_tile_only"])
@pytest.mark.parametrize("want_dw", [True, False])
def test_row_selection_on_device(keep, want_dw):
    """The mask is turned into a row index on the device (no host read of the count): forward and
    backward against the oracle for an empty selection, a single row, every row, a random subset and a
    subset that lives in the last token tile; rows left out return 0 and get a zero gradient, and an
    upstream gradient on a row that was left out must be ignored."""
    n, h, v = 700, 128, 3000
    hidden, weight, labels = _case(n, h, v, seed=21, w_scale=3.0 / math.sqrt(h))
    g = torch.Generator().manual_seed(22)
    mask = {
        "none": torch.zeros(n, dtype=torch.bool),
        "one": torch.arange(n) == 377,
        "all": torch.ones(n, dtype=torch.bool),
        "random": torch.rand(n, generator=g) < 0.6,
        "last_tile_only": torch.arange(n) >= 690,
    }[keep]
    upstream = torch.randn(n, generator=g)  # non-zero also on the rows that are left out
    rh = hidden.float().requires_grad_(True)
    rw = weight.float().requires_grad_(True)
    lp_o, ent_o = o_lm.lm_head_logprobs(rh, rw, labels, 0.9, True)
    (lp_o * mask).backward(upstream)
    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(want_dw)
    lp, ent = lm_head.fused_lm_head_logprobs(dh, dw, labels.to(DEV), 0.9, mask=mask.to(DEV), return_entropy=True)
    lp.backward(upstream.to(DEV))
    assert ((lp.detach().cpu() - lp_o.detach()) * mask).abs().max().item() <= TOL
    assert ((ent.cpu() - ent_o) * mask).abs().max().item() <= TOL
    assert (lp.detach().cpu()[~mask] == 0).all() and (ent.cpu()[~mask] == 0).all()
    assert (dh.grad.cpu()[~mask] == 0).all()
    assert (dh.grad.float().cpu() - rh.grad).abs().max().item() <= TOL + rh.grad.abs().max().item() * 2**-7
    if mask.any():
        assert ((dh.grad.float().cpu() - rh.grad).norm() / rh.grad.norm()).item() <= 2e-2
    if want_dw:
        assert (dw.grad.float().cpu() - rw.grad).abs().max().item() <= TOL + rw.grad.abs().max().item() * 2**-7
        if mask.any():
            assert ((dw.grad.float().cpu() - rw.grad).norm() / rw.grad.norm()).item() <= 2e-2
        else:
            assert not dw.grad.any()


def test_row_selection_with_compact_backward_and_mask():
    """Mask and zero-gradient rows together: the backward selects rows that are in the mask AND carry
    a gradient."""
    n, h, v = 900, 64, 40000  # two vocabulary chunks
    hidden, weight, labels = _case(n, h, v, seed=23, w_scale=3.0 / math.sqrt(h))
    g = torch.Generator().manual_seed(24)
    mask = torch.rand(n, generator=g) < 0.7
    upstream = torch.randn(n, generator=g)
    upstream[torch.rand(n, generator=g) < 0.5] = 0.0
    rh = hidden.float().requires_grad_(True)
    rw = weight.float().requires_grad_(True)
    lp_o, _ = o_lm.lm_head_logprobs(rh, rw, labels, 1.0)
    (lp_o * mask).backward(upstream)
    dh = hidden.to(DEV).requires_grad_(True)
    dw = weight.to(DEV).requires_grad_(True)
    lp, _ = lm_head.fused_lm_head_logprobs(dh, dw, labels.to(DEV), mask=mask.to(DEV), compact_backward=True)
    lp.backward(upstream.to(DEV))
    dead = ~mask | (upstream == 0)
    assert (dh.grad.cpu()[dead] == 0).all()
    assert ((dh.grad.float().cpu() - rh.grad).norm() / rh.grad.norm()).item() <= 2e-2
    assert ((dw.grad.float().cpu() - rw.grad).norm() / rw.grad.norm()).item() <= 2e-2
    assert (dw.grad.float().cpu() - rw.grad).abs().max().item() <= TOL + rw.grad.abs().max().item() * 2**-7


def _rows_of_any_logit_size(n, h, v, seed):
    """Token rows whose logits cover what a float can hold: the largest logit / temperature of a row near
    0, 60, 85, 100 and 300 nats (the kept exponentials of such rows would overflow bf16 were they not taken
    relative to the label's own logit), rows whose logits are all near -120 nats, labels that are the row's
    most likely token, ordinary labels, and labels more than 44 nats below the row's maximum (which the
    kernels flag and recompute).  Returns ``(hidden, weight, labels, flagged)``; `flagged` marks the rows
    whose label is that unlikely, computed here in fp64."""
    g = torch.Generator().manual_seed(seed)
    u = torch.nn.functional.normalize(torch.randn(h, generator=g), dim=0)
    weight = (torch.randn(v, h, generator=g) / math.sqrt(h) + 2.0 * u).bfloat16()
    hidden = torch.randn(n, h, generator=g)
    hidden -= (hidden @ u)[:, None] * u  # no component along the common direction of the weight rows ...
    z = hidden.double() @ weight.double().T
    targets = torch.tensor([0.0, 60.0, 85.0, 100.0, 300.0, -120.0])
    group = torch.arange(n) % len(targets)
    top = z.max(dim=1).values
    scale = torch.where(targets[group] > 0, targets[group] / top, torch.ones(n, dtype=torch.float64))
    hidden = hidden * scale.float()[:, None]
    hidden += torch.where(targets[group] < 0, targets[group] / 2.0, torch.zeros(n))[:, None] * u  # ... except here
    hidden = hidden.bfloat16()
    z = hidden.double() @ weight.double().T
    labels = torch.randint(0, v, (n,), generator=g)
    likely = (torch.arange(n) // len(targets)) % 3 == 0
    labels[likely] = z.argmax(dim=1)[likely]
    return hidden, weight, labels, z


@pytest.mark.parametrize("temperature", [1.0, 0.5])
@pytest.mark.parametrize("masked", [False, True])
def test_d_hidden_in_forward_for_logits_of_any_size(temperature, masked):
    """The forward that prepares d_hidden keeps its exponentials relative to each token's own label logit:
    logprob, entropy and d_hidden against the oracle for rows whose largest logit / temperature runs from 0
    to 600 nats and for rows whose logits are all very negative; rows whose label is too unlikely for that
    are flagged on the device (checked through the C-ABI below) and recomputed, with the same results."""
    n, h, v = 600, 128, 3000
    hidden, weight, labels, z = _rows_of_any_logit_size(n, h, v, seed=61)
    g = torch.Generator().manual_seed(62)
    mask = (torch.rand(n, generator=g) < 0.7) if masked else torch.ones(n, dtype=torch.bool)
    upstream = torch.randn(n, generator=g)
    rh = hidden.double().requires_grad_(True)
    # the oracle in fp64: at logits of several hundred the fp32 form of the reference's entropy,
    # lse - sum p z, cancels two numbers of that size and is itself off by more than the tolerance
    lp_o, ent_o = o_lm.lm_head_logprobs(rh, weight.double(), labels, temperature, True, compute_dtype=torch.float64)
    (lp_o * mask).backward(upstream.double())
    zt = z / temperature
    gap = zt.max(dim=1).values - zt.gather(1, labels[:, None])[:, 0]
    assert zt.max().item() >= 299.0 and zt.max(dim=1).values.min().item() <= -90.0
    assert (gap > 60.0).sum() >= 20 and (gap < 1e-9).sum() >= 50  # both kinds of label are there
    grads = {}
    for route in (True, False):
        dh = hidden.to(DEV).requires_grad_(True)
        lp, ent = lm_head.fused_lm_head_logprobs(
            dh, weight.to(DEV), labels.to(DEV), temperature, mask=mask.to(DEV) if masked else None,
            return_entropy=True, dhidden_in_forward=route,
        )  # fmt: skip
        lp.backward(upstream.to(DEV))
        # logprobs of several hundred nats: fp32 results, so the bound is relative to their size
        assert ((lp.detach().cpu().double() - lp_o.detach()) * mask).abs().max().item() <= TOL + 1e-6 * lp_o.abs().max().item()
        assert ((ent.cpu().double() - ent_o.detach()) * mask).abs().max().item() <= TOL
        got = dh.grad.double().cpu()
        assert torch.isfinite(got).all() and (got[~mask] == 0).all()
        # per row: 3 % of the row's own gradient; the absolute part covers rows whose label holds nearly all
        # of the probability (a gradient of 1e-30 is met to the rounding of the fp32 logprob, not relatively)
        err, size = (got - rh.grad).norm(dim=1), rh.grad.norm(dim=1)
        worst = (err - 3e-2 * size)[mask].max().item()
        assert worst <= 1e-4, (route, worst)
        assert (err[mask & (size > 1e-2)] / size[mask & (size > 1e-2)]).max().item() <= 3e-2
        grads[route] = got
    assert not torch.equal(grads[True], grads[False])  # the two routes are different code

    # the flags, read through the C-ABI: exactly the rows whose label is more than 64 binary orders down
    lib = _lib.load()
    hid, w, lab = hidden.to(DEV), weight.to(DEV), labels.to(DEV)
    m = mask.to(DEV).view(torch.uint8) if masked else None
    out = {k: torch.empty(n, dtype=torch.float32, device=DEV) for k in ("lp", "lse", "xref")}
    wsum = torch.empty(n, h, dtype=torch.float32, device=DEV)
    unsafe = torch.full((n,), 7, dtype=torch.uint8, device=DEV)
    ws_bytes = lib.oi_lmhead_fwd_wsum_workspace_bytes(n, h, v, int(masked))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=DEV)
    _lib.call(
        "oi_lmhead_logp_fwd_wsum", hid.data_ptr(), w.data_ptr(), lab.data_ptr(), _lib.ptr(m), n, h, v, 1.0 / temperature,
        out["lp"].data_ptr(), None, out["lse"].data_ptr(), wsum.data_ptr(), out["xref"].data_ptr(), unsafe.data_ptr(),
        ws.data_ptr(), ws_bytes, _lib.stream_of(hid),
    )  # fmt: skip
    torch.cuda.synchronize()
    gap2 = gap * math.log2(math.e)
    flagged = unsafe.cpu().bool()
    assert set(unsafe.cpu().unique().tolist()) <= {0, 1}
    clear = (gap2 - 64.0).abs() > 0.5  # away from the threshold the flag is determined
    assert torch.equal(flagged[clear & mask], (gap2 > 64.0)[clear & mask]) and not flagged[~mask].any()
    assert flagged.sum() >= 20
