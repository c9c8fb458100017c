"""Integer routing oracle (numpy).  Test infrastructure only.

Notation: ``R`` routed rows with flat index ``t`` (token-major ``t = i*k + j``,
disagmoe/frontend/engine.py:668-671), ``E`` experts.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np


def _as_ids(exp_ids) -> np.ndarray:
    if hasattr(exp_ids, "detach"):
        exp_ids = exp_ids.detach().cpu().reshape(-1).numpy()
    return np.asarray(exp_ids, dtype=np.int64).reshape(-1)


def histogram_offsets(exp_ids, num_experts: int) -> Tuple[np.ndarray, np.ndarray]:
    """``(exp_cnt[E], offsets[E+1])``: per-expert row counts and their exclusive
    scan.  Follows the count loop and running sum of
    disagmoe/ops/memory.py:38-46 (there as an inclusive sum)."""
    ids = _as_ids(exp_ids)
    cnt = np.bincount(ids, minlength=num_experts).astype(np.int64)
    assert cnt.shape[0] == num_experts, "expert id out of range"
    offsets = np.zeros(num_experts + 1, dtype=np.int64)
    np.cumsum(cnt, out=offsets[1:])
    return cnt, offsets


def _rank_within_expert(ids: np.ndarray, offsets: np.ndarray) -> np.ndarray:
    """rank[t] = #{t' < t : ids[t'] == ids[t]} via a stable sort."""
    order = np.argsort(ids, kind="stable")
    rank = np.empty_like(ids)
    rank[order] = np.arange(ids.shape[0], dtype=np.int64) - offsets[ids[order]]
    return rank


def get_mappings_from_exp_ids(exp_ids, num_experts: int) -> Tuple[List[int], List[int]]:
    """Destination row of every routed row, reference order.

    disagmoe/ops/memory.py:34-54: counting sort whose second pass walks ``t``
    upwards and hands out slots from the END of each expert's range
    (``cumsum[id] -= 1; mappings[t] = cumsum[id]``, :50-52).  Hence
    ``mappings[t] = offsets[e] + cnt[e] - 1 - rank[t]``: experts ascending,
    DESCENDING ``t`` inside an expert.  Returns Python lists like the reference.
    """
    ids = _as_ids(exp_ids)
    cnt, offsets = histogram_offsets(ids, num_experts)
    if ids.shape[0] == 0:
        return [], cnt.tolist()
    rank = _rank_within_expert(ids, offsets)
    mappings = offsets[ids] + cnt[ids] - 1 - rank
    return mappings.tolist(), cnt.tolist()


def get_mappings_stable(exp_ids, num_experts: int) -> np.ndarray:
    """Device-variant order: inverse permutation of a sort of the ids
    (disagmoe/ops/memory.py:57-69: ``_, rank = ids.sort(); mappings[rank] =
    arange``).  torch's default sort does not promise stability; the contract
    adopted here is the stable one, ``mappings[t] = offsets[e] + rank[t]``.
    Returns int32 like the reference (:68)."""
    ids = _as_ids(exp_ids)
    _, offsets = histogram_offsets(ids, num_experts)
    if ids.shape[0] == 0:
        return np.zeros(0, dtype=np.int32)
    rank = _rank_within_expert(ids, offsets)
    return (offsets[ids] + rank).astype(np.int32)


def merge_by_exp_ids(batches: Sequence[Sequence[int]], num_experts: int) -> Tuple[List[int], List[int]]:
    """Expert-side merge of several incoming batches.

    csrc/include/datatypes.hpp:288-337 runs the same decrement-then-assign
    counting sort (:321-323) over the batches in arrival order, i.e. over their
    concatenation; ``mappings[idx] = j`` is the destination row of the idx-th
    row of the concatenated stream.  The reference caps experts at 32 (:291);
    the cap is not reproduced."""
    flat = np.concatenate([_as_ids(b) for b in batches]) if len(batches) else np.zeros(0, np.int64)
    return get_mappings_from_exp_ids(flat, num_experts)


def expert_batch_sizes(exp_ids, n_expert: int, inner_exp_rank: Sequence[int] | None = None) -> np.ndarray:
    """int64 rows per LOCAL expert: histogram over global experts, then select
    ``inner_exp_rank`` (csrc/include/datatypes.hpp:228-247; the selection list is
    built at disagmoe/frontend/engine.py:151-154)."""
    cnt, _ = histogram_offsets(exp_ids, n_expert)
    if inner_exp_rank is None:
        return cnt
    sel = np.asarray(list(inner_exp_rank), dtype=np.int64)
    assert ((0 <= sel) & (sel < n_expert)).all()
    return cnt[sel]


def sort_by_prefill_order(req_ids: Sequence[int], attn_dp_ranks: Sequence[int],
                          init_prefill_lens: Sequence[int]) -> List[int]:
    """Return mapping of the expert worker (csrc/include/datatypes.hpp:411-433).

    Rows are ranked by attention DP rank, then prefill rows (``init_prefill_len
    != -1``) before decode rows (``== -1``), prefill rows by request id;
    ``mapping[rank[i]] = i``.  The reference's comparator leaves decode/decode
    pairs (and mixed pairs with equal lens) unordered under a non-stable
    ``std::sort``; this restatement keeps their original order (stable), which is
    one of the orders the reference may produce."""
    n = len(req_ids)
    assert len(attn_dp_ranks) == n and len(init_prefill_lens) == n

    import functools

    def before(i: int, j: int) -> bool:
        if attn_dp_ranks[i] != attn_dp_ranks[j]:
            return attn_dp_ranks[i] < attn_dp_ranks[j]
        if init_prefill_lens[i] == -1 or init_prefill_lens[j] == -1:
            return init_prefill_lens[i] > init_prefill_lens[j]
        return req_ids[i] < req_ids[j]

    def cmp(i: int, j: int) -> int:
        if before(i, j):
            return -1
        if before(j, i):
            return 1
        return 0

    rank = sorted(range(n), key=functools.cmp_to_key(cmp))
    mapping = [0] * n
    for i, r in enumerate(rank):
        mapping[r] = i
    return mapping


def apply_row_mapping(values: Sequence, mapping: Sequence[int]) -> list:
    """``out[mapping[i]] = values[i]`` -- how the reference moves per-row metadata
    (csrc/include/datatypes.hpp:377-409)."""
    out = [None] * len(values)
    for i, m in enumerate(mapping):
        out[m] = values[i]
    return out


def fused_topk(gating_output, topk: int, renormalize: bool = True):
    """Routing producer ``fused_topk(hidden_states, gating_output, topk,
    renormalize)`` of vllm 0.6.2 (requirements.txt:5; not present in this
    checkout), as called at disagmoe/models/attention.py:228-231.  Its published
    definition: ``w = softmax(gating_output.float(), dim=-1)``; the ``topk``
    largest ``w`` per token with their expert ids; with ``renormalize`` divide
    the kept weights by their sum.  Ties go to the lower expert id (vllm's
    ``topk_softmax`` kernel scans experts upwards and replaces only on a strictly
    larger value).  The order is taken on the logits, which is the order of the
    probabilities wherever their fp32 rounding keeps distinct logits apart.
    Returns ``(weights [n, topk] float32, ids [n, topk] int32)``."""
    x = gating_output
    if hasattr(x, "detach"):
        x = x.detach().cpu().float().numpy()
    x = np.asarray(x, dtype=np.float32)
    n, E = x.shape
    assert 1 <= topk <= E
    order = np.argsort(-x.astype(np.float64), axis=1, kind="stable")[:, :topk]   # stable: lower id first among equals
    m = x.max(axis=1, keepdims=True)
    p = np.exp((x - m).astype(np.float32)).astype(np.float32)
    p = p / p.sum(axis=1, keepdims=True, dtype=np.float32)
    w = np.take_along_axis(p, order, axis=1).astype(np.float32)
    if renormalize:
        w = w / w.sum(axis=1, keepdims=True, dtype=np.float32)
    return w.astype(np.float32), order.astype(np.int32)
