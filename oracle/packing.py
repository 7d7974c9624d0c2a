"""Oracle: packing of query/response pairs into training rows (test infrastructure only).

Plain Python lists, token by token, following the reference's own loop order.
"""

from __future__ import annotations

import math


def pack_sequences(
    queries, responses, masks, pack_length, pad_token_id, vllm_logprobs, min_num_batches=1, mask_tool_use=False
) -> dict[str, list[list]]:
    """Restates open_instruct/rl_utils.py:227-375 with list outputs (one inner list per packed row).

    Keys: query_responses, attention_masks, response_masks, position_ids, num_actions,
    packed_seq_lens, dones, vllm_logprobs.  Position ids restart at 0 for every sequence inside a
    row (open_instruct/rl_utils.py:215-224, applied to the per-row attention ids).
    """
    assert not any(pad_token_id in q for q in queries)
    total = sum(len(q) + sum(1 for t in r if t != pad_token_id) for q, r in zip(queries, responses))
    effective = min(total // min_num_batches, pack_length) if (total > 0 and min_num_batches > 1) else pack_length
    keys = ("query_responses", "attention_masks", "response_masks", "position_ids", "num_actions",
            "packed_seq_lens", "dones", "vllm_logprobs")  # fmt: skip
    out = {k: [] for k in keys}
    cur = {k: [] for k in keys}
    offset = 0
    for i, (query, response, mask, logprobs) in enumerate(zip(queries, responses, masks, vllm_logprobs)):
        assert len(logprobs) == len(response)
        kept = [(t, m, lp) for t, m, lp in zip(response, mask, logprobs) if t != pad_token_id]
        resp = [t for t, _, _ in kept]
        seq = list(query) + resp
        if len(seq) + len(cur["query_responses"]) > effective and len(cur["query_responses"]) > 0:
            for k in keys:
                out[k].append(cur[k])
            cur = {k: [] for k in keys}
            offset = i
        cur["query_responses"].extend(seq)
        cur["vllm_logprobs"].extend([math.nan] * len(query) + [lp for _, _, lp in kept])
        cur["num_actions"].append(len(resp))
        cur["packed_seq_lens"].append(len(seq))
        resp_mask = [i + 1 if m else 0 for _, m, _ in kept] if mask_tool_use else [i + 1] * len(resp)
        cur["response_masks"].extend([0] * len(query) + resp_mask)
        cur["attention_masks"].extend([i + 1 - offset] * len(seq))
        cur["position_ids"].extend(range(len(seq)))
        cur["dones"].extend([0] * (len(seq) - 1) + [i + 1])
    if len(cur["query_responses"]) > 0:
        for k in keys:
            out[k].append(cur[k])
    return out


def broadcast_advantages(advantages, response_masks) -> list[list[float]]:
    """Restates open_instruct/data_loader.py:1509-1514: ``lookup[0] = 0``, ``lookup[i + 1] =
    advantages[i]``, gathered with the document-id response mask of every row."""
    lookup = [0.0] + [float(a) for a in advantages]
    return [[lookup[m] for m in row] for row in response_masks]
