"""Host-side plumbing that needs no GPU: row layouts, reshapes, label shifts, batch concatenation."""

import contextlib

import pytest
import torch

from conftest import make_grpo_config
from open_instruct_amd import dpo_utils, grpo_utils, model_utils, padding_free_collator, rl_utils


def test_row_layout_contiguous_and_sliced():
    full = torch.zeros(3, 6, 16)
    t, no, ni, so, si = model_utils._row_layout(full)
    assert (no, ni, so, si) == (3, 6, 96, 16) and t.data_ptr() == full.data_ptr()
    view = full[:, :-1]
    t, no, ni, so, si = model_utils._row_layout(view)
    assert (no, ni, so, si) == (3, 5, 96, 16) and t.data_ptr() == full.data_ptr()
    t, no, ni, so, si = model_utils._row_layout(torch.zeros(7, 16))
    assert (no, ni, so, si) == (1, 7, 0, 16)
    t, no, ni, so, si = model_utils._row_layout(torch.zeros(16))
    assert (no, ni) == (1, 1)
    four = torch.zeros(2, 3, 5, 8)
    t, no, ni, so, si = model_utils._row_layout(four)
    assert (no, ni, so, si) == (6, 5, 40, 8)
    # not collapsible -> copied to a contiguous layout with the same row counts
    odd = torch.zeros(2, 4, 5, 8)[:, :3]
    t, no, ni, so, si = model_utils._row_layout(odd)
    assert (no, ni, so, si) == (6, 5, 40, 8) and t.is_contiguous()
    # transposed last dim / expanded rows are copied too
    t, *_ = model_utils._row_layout(torch.zeros(8, 4).t())
    assert t.is_contiguous()
    t, no, ni, so, si = model_utils._row_layout(torch.zeros(1, 8).expand(5, 8))
    assert t.is_contiguous() and si == 8


def test_masked_mean_reshape_rules():
    v = torch.arange(24.0).reshape(4, 2, 3)
    m = torch.ones(2, 3)
    v3, m2, extra_dims, mode = rl_utils._as_rows(v, m, None)
    assert v3.shape == (4, 1, 6) and m2.shape == (1, 6) and extra_dims == 1 and mode == 0
    v3, m2, extra_dims, mode = rl_utils._as_rows(v, m, 1)
    assert v3.shape == (4, 2, 3) and m2.shape == (2, 3) and mode == 1
    v3, m2, _, _ = rl_utils._as_rows(v, m, 0)
    assert v3.shape == (4, 3, 2) and m2.shape == (3, 2)
    assert torch.equal(v3[1, 2], v[1, :, 2])
    with pytest.raises(IndexError):
        rl_utils._as_rows(v, m, 2)
    with pytest.raises(ValueError):
        rl_utils._as_rows(torch.ones(2, 4), torch.ones(2, 3), None)


def test_shift_labels_bit_exact():
    labels = torch.tensor([[5, -100, 7, 9], [1, 2, 3, -100]])
    assert padding_free_collator.shift_labels(labels).tolist() == [[-100, 7, 9, -100], [2, 3, -100, -100]]


def test_packed_concatenated_inputs_offsets():
    batch = {
        "chosen_input_ids": torch.arange(10).unsqueeze(0),
        "chosen_labels": torch.arange(10).unsqueeze(0),
        "chosen_cu_seq_lens_q": torch.tensor([0, 4, 10], dtype=torch.int32),
        "chosen_cu_seq_lens_k": torch.tensor([0, 4, 10], dtype=torch.int32),
        "chosen_max_length_q": 6,
        "chosen_max_length_k": 6,
        "rejected_input_ids": torch.arange(7).unsqueeze(0),
        "rejected_labels": torch.arange(7).unsqueeze(0),
        "rejected_cu_seq_lens_q": torch.tensor([0, 3, 7], dtype=torch.int32),
        "rejected_cu_seq_lens_k": torch.tensor([0, 3, 7], dtype=torch.int32),
        "rejected_max_length_q": 4,
        "rejected_max_length_k": 4,
    }
    out, bs = padding_free_collator.concatenated_inputs(batch)
    assert bs == 2
    assert out["concatenated_input_ids"].shape == (1, 17)
    assert out["concatenated_cu_seq_lens_k"].tolist() == [0, 4, 10, 13, 17]
    assert len(out["concatenated_cu_seq_lens_k"]) == 2 * bs + 1
    assert out["concatenated_max_length_k"] == 6


def test_padded_concatenated_inputs_pad_values():
    batch = {
        "chosen_input_ids": torch.ones(2, 5, dtype=torch.long),
        "chosen_labels": torch.ones(2, 5, dtype=torch.long),
        "rejected_input_ids": torch.ones(2, 3, dtype=torch.long),
        "rejected_labels": torch.ones(2, 3, dtype=torch.long),
        "index": torch.tensor([4, 5]),
    }
    out = dpo_utils.concatenated_inputs(batch)
    assert out["concatenated_input_ids"].shape == (4, 5)
    assert (out["concatenated_input_ids"][2:, 3:] == 0).all()
    assert (out["concatenated_labels"][2:, 3:] == -100).all()


def test_invalid_loss_fn_raises_before_any_kernel():
    cfg = make_grpo_config(loss_fn="invalid")
    with pytest.raises(ValueError, match="Invalid loss function"):
        grpo_utils.compute_grpo_loss(torch.randn(2, 4), torch.ones(2, 4), torch.randn(2, 4), None, cfg, torch.ones(2, 4))


def test_resolve_old_logprob_bookkeeping():
    cache = [None, None]
    new = torch.tensor([1.0, 2.0], requires_grad=True)
    vl = torch.tensor([3.0, 4.0])
    out = grpo_utils.resolve_old_logprob(cache, 0, 0, 1, False, vl, new)
    assert not out.requires_grad and torch.equal(out, new.detach())
    assert grpo_utils.resolve_old_logprob(cache, 0, 1, 1, False, vl, new * 2) is out
    out = grpo_utils.resolve_old_logprob(cache, 1, 0, 1, True, vl, new)
    assert out is vl
    cache2 = [torch.tensor([9.0])]
    assert grpo_utils.resolve_old_logprob(cache2, 0, 0, 2, False, vl, new) is cache2[0]


def test_metrics_from_loss_stats():
    stats = {"val/ratio": torch.tensor([1.0, 3.0]), "loss/total_avg": torch.tensor([2.0, 4.0])}
    out = grpo_utils.compute_metrics_from_loss_stats(stats, torch.tensor([1.0, 3.0]))
    assert out["val/ratio"] == pytest.approx(2.5)
    assert out["loss/total_avg"] == pytest.approx(3.5)
    assert out["val/ratio_var"] == pytest.approx(0.25 * 1.5**2 + 0.75 * 0.5**2)


def test_tensor_cache_roundtrip_and_reference_cache_builder(tmp_path):
    """open_instruct/model_utils.py:92-115 and open_instruct/dpo_utils.py:405-520 (one-process form):
    scatter by index, padding batches skipped, missing indices raise, disk round trip."""
    cache = model_utils.TensorCache(tensors={"chosen_logps": torch.arange(5.0), "rejected_logps": -torch.arange(5.0)})
    picked = cache[torch.tensor([3, 1])]
    assert picked["chosen_logps"].tolist() == [3.0, 1.0] and picked["rejected_logps"].tolist() == [-3.0, -1.0]
    path = tmp_path / "sub" / "cache.pt"
    cache.to_disk(path)
    again = model_utils.TensorCache.from_disk(path, device=torch.device("cpu"))
    assert torch.equal(again.tensors["chosen_logps"], cache.tensors["chosen_logps"])

    calls = []

    def forward_fn(model, batch, average_log_prob=False, scale=1.0):
        calls.append((model.training, average_log_prob, torch.is_grad_enabled()))
        idx = batch["index"].float()
        return idx * scale, -idx * scale, None

    model = torch.nn.Linear(2, 2)
    batches = [
        {"index": torch.tensor([2, 0])},
        {"index": torch.tensor([1, 3])},
        {"index": torch.tensor([0, 0]), "is_padding": True},
    ]
    # called as open_instruct/dpo_tune_cache.py:522-534 calls it (every argument by keyword)
    built = dpo_utils.build_reference_logprobs_cache(
        model=model,
        dataloader=batches,
        average_log_prob=True,
        forward_fn=forward_fn,
        full_dataset_size=4,
        device=torch.device("cpu"),
        cache_path=tmp_path / "deep" / "ref.pt",
        is_main_process=True,
        model_dims=object(),
        use_lora=False,
        disable_adapter_context=None,
    )
    assert built.tensors["chosen_logps"].tolist() == [0.0, 1.0, 2.0, 3.0]
    assert built.tensors["rejected_logps"].tolist() == [0.0, -1.0, -2.0, -3.0]
    assert calls == [(False, True, False)] * 3 and model.training
    assert (tmp_path / "deep" / "ref.pt").exists()
    # an existing file is loaded, not recomputed
    n_calls = len(calls)
    loaded = dpo_utils.build_reference_logprobs_cache(
        model, batches, True, forward_fn, 4, torch.device("cpu"), tmp_path / "deep" / "ref.pt", True, None
    )
    assert len(calls) == n_calls and torch.equal(loaded.tensors["chosen_logps"], built.tensors["chosen_logps"])
    # the keyword dictionary of open_instruct/dpo.py:310 (`model=..., **cache_kwargs`), extra forward arguments
    # included; a process that is not the main one computes the cache and writes nothing
    cache_kwargs = dict(
        dataloader=batches, average_log_prob=False, forward_fn=forward_fn, full_dataset_size=4,
        device=torch.device("cpu"), cache_path=tmp_path / "other" / "ref.pt", is_main_process=False,
        model_dims=None, forward_kwargs={"scale": 2.0},
    )  # fmt: skip
    model.eval()
    quiet = dpo_utils.build_reference_logprobs_cache(model=model, **cache_kwargs)
    assert quiet.tensors["chosen_logps"].tolist() == [0.0, 2.0, 4.0, 6.0] and model.training
    assert not (tmp_path / "other").exists()
    # with LoRA the forward runs inside the context that switches the adapter off
    entered = []

    @contextlib.contextmanager
    def adapter_off():
        entered.append("in")
        yield
        entered.append("out")

    dpo_utils.build_reference_logprobs_cache(
        model, batches, False, forward_fn, 4, torch.device("cpu"), tmp_path / "lora.pt", True, None,
        use_lora=True, disable_adapter_context=adapter_off,
    )  # fmt: skip
    assert entered == ["in", "out"] * 3
    entered.clear()
    dpo_utils.build_reference_logprobs_cache(
        model, batches, False, forward_fn, 4, torch.device("cpu"), tmp_path / "nolora.pt", True, None,
        use_lora=False, disable_adapter_context=adapter_off,
    )  # fmt: skip
    assert entered == []
    with pytest.raises(RuntimeError, match="Missing 1 indices"):
        dpo_utils.build_reference_logprobs_cache(
            model, batches[:2], False, forward_fn, 5, torch.device("cpu"), tmp_path / "miss.pt", True, None
        )
    assert not (tmp_path / "miss.pt").exists()


def test_collation_of_packed_rows_for_workers():
    """open_instruct/data_loader.py:636-641,1205-1289: rank split, per-rank shuffle from numpy's
    global generator, right padding (pad id for tokens, 0 elsewhere), uneven tails dropped."""
    import numpy as np

    from open_instruct_amd import data_loader
    from open_instruct_amd.rl_utils import PackedSequences

    lens = [5, 3, 7, 2, 4]
    rows = lambda fill, dtype: [torch.full((n,), fill(k), dtype=dtype) for k, n in enumerate(lens)]  # noqa: E731
    packed = PackedSequences(
        query_responses=rows(lambda k: 10 + k, torch.long), attention_masks=rows(lambda k: 1, torch.long),
        response_masks=rows(lambda k: k + 1, torch.long), original_responses=[],
        advantages=rows(lambda k: 0.5 * k, torch.float32), position_ids=[torch.arange(n) for n in lens],
        vllm_logprobs=rows(lambda k: -1.0 * k, torch.float32),
    )  # fmt: skip
    np.random.seed(3)
    got = data_loader.prepare_collated_data_for_workers(packed, 2, 2, pad_token_id=99)
    np.random.seed(3)
    orders = [np.random.permutation(2), np.random.permutation(2)]
    assert len(got) == 2 and all(len(c) == 1 for c in got)  # 5 rows -> 4 kept, 2 per rank, one micro-batch each
    for rank, (coll, order) in enumerate(zip(got, orders)):
        src = [2 * rank + int(i) for i in order]
        qr = coll.query_responses[0]
        width = max(lens[i] for i in src)
        assert qr.shape == (2, width)
        for r, i in enumerate(src):
            assert qr[r, : lens[i]].tolist() == [10 + i] * lens[i] and qr[r, lens[i] :].tolist() == [99] * (width - lens[i])
            assert coll.attention_masks[0][r].tolist() == [1] * lens[i] + [0] * (width - lens[i])
            assert coll.position_ids[0][r, : lens[i]].tolist() == list(range(lens[i]))
            assert coll.response_masks[0][r].tolist() == [i + 1] * lens[i] + [0] * (width - lens[i])
            assert coll.advantages[0][r, : lens[i]].tolist() == [0.5 * i] * lens[i]
            assert coll.vllm_logprobs[0][r, lens[i] :].tolist() == [0.0] * (width - lens[i])
    single = data_loader.prepare_collated_data_for_workers(packed, 1, 1, pad_token_id=0)
    assert len(single) == 1 and len(single[0]) == 5 and all(t.shape[0] == 1 for t in single[0].query_responses)
    assert data_loader.collate_fn([torch.tensor([1, 2, 3])], 0).shape == (1, 3)


def test_side_tensors_that_do_not_broadcast_are_rejected_before_any_kernel():
    cfg = make_grpo_config()
    logits = torch.randn(2, 3, 16).requires_grad_(True)
    labels = torch.zeros(2, 3, dtype=torch.int64)
    mask = torch.ones(2, 3, dtype=torch.bool)
    with pytest.raises(ValueError, match="advantages of shape"):
        grpo_utils.grpo_loss_on_logits(logits, labels, None, None, torch.zeros(3, 2), mask, cfg)
    with pytest.raises(ValueError, match="advantages of shape"):
        grpo_utils.compute_rho_correction(torch.zeros(2, 3), torch.zeros(2, 3), mask, torch.zeros(5), cfg)


def test_doc_lens_from_attention_mask_reference_vectors(golden):
    """open_instruct/test_grpo_utils.py:9-48: run lengths per row, padding runs kept as segments, rows
    padded with zeros to the widest row, row sums equal the sequence length."""
    from open_instruct_amd import olmo_core_utils

    for case in golden["doc_lens_from_attention_mask"]["cases"]:
        mask = torch.tensor(case["attention_mask"], dtype=torch.long)
        doc_lens, max_doc_lens = olmo_core_utils.doc_lens_from_attention_mask(mask)
        assert doc_lens.dtype == torch.int32, case["name"]
        assert doc_lens.tolist() == case["doc_lens"], case["name"]
        assert max_doc_lens == case["max_doc_lens"], case["name"]
        assert doc_lens.sum(dim=1).tolist() == [mask.shape[1]] * mask.shape[0]
    # against a plain Python run-length encoding on random masks with non-monotonic ids
    g = torch.Generator().manual_seed(0)
    mask = torch.randint(0, 3, (5, 40), generator=g).sort(dim=1).values.roll(7, dims=1)
    doc_lens, max_doc_lens = olmo_core_utils.doc_lens_from_attention_mask(mask)
    for row, got, longest in zip(mask.tolist(), doc_lens.tolist(), max_doc_lens):
        runs, prev = [], object()
        for v in row:
            if v == prev:
                runs[-1] += 1
            else:
                runs.append(1)
                prev = v
        assert got[: len(runs)] == runs and not any(got[len(runs) :]) and longest == max(runs)


def test_loss_type_enums():
    """open_instruct/dpo_utils.py:76-92, open_instruct/grpo_utils.py:69-71: string enums whose members equal
    their names; which DPO losses average the sequence logprobs, need a reference model, report rewards."""
    import types

    from open_instruct_amd import dpo_utils, grpo_utils

    T = dpo_utils.DPOLossType
    assert [m.value for m in T] == ["dpo", "dpo_norm", "simpo", "wpo"]
    assert T.dpo_norm == "dpo_norm" and T("wpo") is T.wpo and str(T.simpo) == "simpo"
    table = {"dpo": (False, True, True), "dpo_norm": (True, True, True), "simpo": (True, False, False), "wpo": (False, True, False)}
    for name, (avg, needs_ref, rewards) in table.items():
        assert (T(name).is_average_loss, T(name).needs_reference_model, T(name).computes_reward_metrics) == (avg, needs_ref, rewards)
    G = grpo_utils.GRPOLossType
    assert [m.value for m in G] == ["dapo", "cispo"] and G.cispo == "cispo"
    # a config may hold the member or its name
    for loss_fn in (G.dapo, "dapo"):
        assert grpo_utils._loss_fn_tag(types.SimpleNamespace(loss_fn=loss_fn)) == grpo_utils._loss_fn_tag(types.SimpleNamespace(loss_fn="dapo"))
    with pytest.raises(ValueError):
        grpo_utils._loss_fn_tag(types.SimpleNamespace(loss_fn="ppo"))


def test_batch_counters_reference_vectors(golden):
    """open_instruct/test_padding_free_collator.py:399-419: sequences of a packed batch are the strictly
    increasing boundary steps of every *cu_seq_lens_k, of a padded one the rows of every *input_ids; padded
    token positions are the elements of every *input_ids."""
    from open_instruct_amd import padding_free_collator as pfc

    vec = golden["batch_counters"]
    for case in vec["num_sequences"]:
        batch = {k: torch.tensor(v) for k, v in case.get("batch", {}).items()}
        batch.update({k: torch.zeros(*shape) for k, shape in case.get("batch_shapes", {}).items()})
        got = pfc.get_num_sequences(batch)
        assert isinstance(got, torch.Tensor) and got.ndim == 0, case["name"]
        assert int(got) == case["expected"], case["name"]
    for case in vec["num_padded_tokens"]:
        batch = {k: torch.zeros(*shape) for k, shape in case["batch_shapes"].items()}
        assert pfc.get_num_padded_tokens(batch) == case["expected"]
    # repeated boundaries (a packed row padded to a fixed number of sequences) do not count
    assert int(pfc.get_num_sequences({"cu_seq_lens_k": torch.tensor([0, 3, 7, 7, 7])})) == 2
    # real tokens (open_instruct/padding_free_collator.py:232-249): the last boundaries of a packed batch, the
    # attention-mask sums of a padded one, else every input id; non-tensor entries are skipped
    packed = {"chosen_cu_seq_lens_k": torch.tensor([0, 3, 7]), "rejected_cu_seq_lens_k": torch.tensor([0, 4]),
              "chosen_input_ids": torch.zeros(1, 9), "rejected_input_ids": torch.zeros(1, 6)}  # fmt: skip
    assert pfc.get_num_tokens(packed) == 11 and pfc.get_num_padded_tokens(packed) == 15
    padded = {"chosen_attention_mask": torch.tensor([[1, 1, 0], [1, 0, 0]]), "rejected_attention_mask": torch.tensor([[1, 1, 1]]),
              "chosen_input_ids": torch.zeros(2, 3), "rejected_input_ids": torch.zeros(1, 3), "index": [4, 5]}  # fmt: skip
    assert pfc.get_num_tokens(padded) == 6 and pfc.get_num_padded_tokens(padded) == 9
    assert pfc.get_num_tokens({"input_ids": torch.zeros(2, 7), "note": "x"}) == 14


def test_doc_lens_from_cu_seq_lens():
    """open_instruct/olmo_core_utils.py:650-665: differences of the offsets; a padded tail becomes a
    segment of its own so the lengths cover the whole row (the reference holds no vector for it;
    expected values follow from the definition)."""
    from open_instruct_amd import olmo_core_utils

    cu = torch.tensor([0, 50, 100, 550, 600], dtype=torch.int32)  # open_instruct/test_padding_free_collator.py:348-363
    doc_lens, longest = olmo_core_utils.doc_lens_from_cu_seq_lens(cu, seq_len=600)
    assert doc_lens.dtype == torch.int32 and doc_lens.tolist() == [[50, 50, 450, 50]] and longest == [450]
    doc_lens, longest = olmo_core_utils.doc_lens_from_cu_seq_lens(cu, seq_len=1000)
    assert doc_lens.tolist() == [[50, 50, 450, 50, 400]] and longest == [450]
    doc_lens, longest = olmo_core_utils.doc_lens_from_cu_seq_lens(torch.tensor([0, 3]), seq_len=10)
    assert doc_lens.tolist() == [[3, 7]] and longest == [7]


def test_olmo_forward_plumbing_passes_labels_and_doc_lens():
    """concatenated_forward_olmo (open_instruct/dpo_utils.py:959-1019) hands the labels to the model and,
    for packed batches, position ids and document lengths; forward_for_logprobs with
    pass_olmo_core_doc_lens (open_instruct/grpo_utils.py:551-557) replaces the attention mask by them.
    Checked with a recording stand-in model up to the first kernel call (which needs a GPU)."""
    calls = []

    class Recorder(torch.nn.Module):
        def forward(self, *args, **kwargs):
            calls.append((args, kwargs))
            raise RuntimeError("recorded")

    chosen = {"input_ids": torch.ones(1, 5, dtype=torch.long), "labels": torch.ones(1, 5, dtype=torch.long),
              "cu_seq_lens_q": torch.tensor([0, 2, 5]), "cu_seq_lens_k": torch.tensor([0, 2, 5]),
              "max_length_q": 3, "max_length_k": 3, "position_ids": torch.tensor([[0, 1, 0, 1, 2]])}  # fmt: skip
    rejected = {"input_ids": torch.ones(1, 4, dtype=torch.long), "labels": torch.ones(1, 4, dtype=torch.long),
                "cu_seq_lens_q": torch.tensor([0, 1, 4]), "cu_seq_lens_k": torch.tensor([0, 1, 4]),
                "max_length_q": 3, "max_length_k": 3, "position_ids": torch.tensor([[0, 0, 1, 2]])}  # fmt: skip
    batch = {f"chosen_{k}": v for k, v in chosen.items()} | {f"rejected_{k}": v for k, v in rejected.items()}
    with pytest.raises(RuntimeError, match="recorded"):
        dpo_utils.concatenated_forward_olmo(Recorder(), batch, packing=True)
    args, kwargs = calls.pop()
    assert args[0].shape == (1, 9) and kwargs["labels"].shape == (1, 9)
    assert kwargs["doc_lens"].tolist() == [[2, 3, 1, 3]] and kwargs["max_doc_lens"] == [3]
    assert kwargs["position_ids"].tolist() == [[0, 1, 0, 1, 2, 0, 0, 1, 2]]
    padded = {"chosen_input_ids": torch.ones(2, 5, dtype=torch.long), "chosen_labels": torch.ones(2, 5, dtype=torch.long),
              "rejected_input_ids": torch.ones(2, 3, dtype=torch.long), "rejected_labels": torch.ones(2, 3, dtype=torch.long)}  # fmt: skip
    with pytest.raises(RuntimeError, match="recorded"):
        dpo_utils.concatenated_forward_olmo(Recorder(), padded, packing=False)
    args, kwargs = calls.pop()
    assert args[0].shape == (4, 5) and set(kwargs) == {"labels"} and (kwargs["labels"][2:, 3:] == -100).all()
    mask = torch.tensor([[1, 1, 2, 2, 2, 0]])
    with pytest.raises(RuntimeError, match="recorded"):
        grpo_utils.forward_for_logprobs(Recorder(), torch.ones(1, 6, dtype=torch.long), mask, mask, 0, 1.0, pass_olmo_core_doc_lens=True)
    _, kwargs = calls.pop()
    assert kwargs["attention_mask"] is None and kwargs["doc_lens"].tolist() == [[2, 3, 1]] and kwargs["max_doc_lens"] == [3]
    with pytest.raises(AssertionError):
        grpo_utils.forward_for_logprobs(Recorder(), torch.ones(1, 6, dtype=torch.long), None, mask, 0, 1.0, pass_olmo_core_doc_lens=True)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures the one-GPU hot path only: any other GPU count ends with a message, before
    torch or the library are touched."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)  # fmt: skip
    assert res.returncode == 2
    assert "one-GPU" in res.stdout
    env = dict(os.environ, WORLD_SIZE="4")
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py")], capture_output=True, text=True, env=env,
                         timeout=120)  # fmt: skip
    assert res.returncode == 2 and "one-GPU" in res.stdout
