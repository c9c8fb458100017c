"""Per-row bookkeeping of a batch on the expert worker.

Mirror of the part of the reference's ``Metadata`` (csrc/include/datatypes.hpp:135-501) that the
expert step reads and writes (disagmoe/frontend/engine.py:683-739): the lists live on the host as
they do there, the sorting and moving runs in the C++ library (no Python loops over rows), and what
reaches the device is a row mapping for ``permute_tokens``.  The wire format (cereal field order,
datatypes.hpp:223-226) belongs to the transport and is not part of this package.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import numpy as np

from .. import _lib


def _i32(values: Sequence[int]) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(values, dtype=np.int32))


def _ptr(a: np.ndarray) -> int:
    return a.ctypes.data


def sort_by_prefill_order(req_ids: Sequence[int], attn_dp_ranks: Sequence[int],
                          init_prefill_lens: Sequence[int]) -> List[int]:
    """Return mapping ``mapping[rank[i]] = i`` of the rows ranked by DP rank, prefill before
    decode, request id (datatypes.hpp:411-433); rows that compare equal keep their order."""
    n = len(req_ids)
    assert len(attn_dp_ranks) == n and len(init_prefill_lens) == n
    r, a, p = _i32(req_ids), _i32(attn_dp_ranks), _i32(init_prefill_lens)
    mapping = np.empty(n, dtype=np.int64)
    _lib.call("dmoe_sort_by_prefill_order", _ptr(r), _ptr(a), _ptr(p), n, _ptr(mapping))
    return mapping.tolist()


def move_row_infos(values: Sequence, mapping: Sequence[int], dtype=np.int32) -> list:
    """``out[mapping[i]] = values[i]`` for one per-row list (permute_token_infos, datatypes.hpp:377-409)."""
    n = len(values)
    assert len(mapping) == n
    v = np.ascontiguousarray(np.asarray(values, dtype=dtype))
    m = np.ascontiguousarray(np.asarray(mapping, dtype=np.int64))
    out = np.empty_like(v)
    _lib.call("dmoe_move_row_infos", _ptr(v), v.dtype.itemsize, _ptr(m), n, _ptr(out))
    return out.tolist()


def expert_batch_sizes(exp_ids: Sequence[int], n_expert: int,
                       inner_exp_rank: Optional[Sequence[int]] = None) -> List[int]:
    """Rows per expert (get_expert_batch_sizes, datatypes.hpp:228-234); with ``inner_exp_rank`` the
    counts of those experts in that order (:236-247)."""
    ids = _i32(exp_ids)
    if inner_exp_rank is None:
        out = np.empty(n_expert, dtype=np.int64)
        _lib.call("dmoe_expert_batch_sizes", _ptr(ids), ids.size, n_expert, None, 0, _ptr(out))
    else:
        sel = _i32(inner_exp_rank)
        out = np.empty(sel.size, dtype=np.int64)
        _lib.call("dmoe_expert_batch_sizes", _ptr(ids), ids.size, n_expert, _ptr(sel), sel.size, _ptr(out))
    return out.tolist()


@dataclass
class Metadata:
    """Field names and method names of the reference's ``Metadata`` as the expert step uses them."""
    shape: List[int]
    dtype: str = "bf16"
    layer_id: int = 0
    req_ids: List[int] = field(default_factory=list)
    exp_ids: List[int] = field(default_factory=list)
    attn_dp_ranks: List[int] = field(default_factory=list)
    init_prefill_lens: List[int] = field(default_factory=list)
    topk_weights: List[float] = field(default_factory=list)

    def __post_init__(self):
        n = len(self.req_ids)
        if not self.attn_dp_ranks:
            self.attn_dp_ranks = [0] * n
        if not self.init_prefill_lens:
            self.init_prefill_lens = [-1] * n

    def num_tokens(self) -> int:
        return self.shape[0]

    def step_layer(self) -> None:
        self.layer_id += 1

    def get_expert_batch_sizes(self, n_expert: int) -> List[int]:
        assert n_expert > 0
        return expert_batch_sizes(self.exp_ids, n_expert)

    def permute_token_infos(self, exp_mappings: Sequence[int]) -> None:
        """Every per-row list moves along: ``list[mapping[i]] = list[i]`` (datatypes.hpp:377-409)."""
        if len(exp_mappings) == 0:
            return
        assert len(self.req_ids) == len(exp_mappings)
        if self.exp_ids:
            self.exp_ids = move_row_infos(self.exp_ids, exp_mappings)
        self.req_ids = move_row_infos(self.req_ids, exp_mappings)
        self.attn_dp_ranks = move_row_infos(self.attn_dp_ranks, exp_mappings)
        self.init_prefill_lens = move_row_infos(self.init_prefill_lens, exp_mappings)
        if self.topk_weights:
            self.topk_weights = move_row_infos(self.topk_weights, exp_mappings, dtype=np.float32)

    def update_exp_ids(self, new_exp_ids: Sequence[int], exp_mappings: Sequence[int]) -> None:
        """datatypes.hpp:343-347: the expert ids are replaced first, then everything is moved."""
        self.exp_ids = list(new_exp_ids)
        self.permute_token_infos(exp_mappings)

    def sort_by_prefill_order(self) -> List[int]:
        """datatypes.hpp:411-433: returns the mapping and applies it to the lists (the expert ids
        are dropped: ``update_exp_ids({}, mapping)``)."""
        mapping = sort_by_prefill_order(self.req_ids, self.attn_dp_ranks, self.init_prefill_lens)
        self.update_exp_ids([], mapping)
        return mapping

    def duplicate_topk(self, topk: int) -> None:
        """datatypes.hpp:354-375: the per-request lists are repeated k-major (copy ``j`` of request
        ``i`` at ``j * n + i``).  The routed ROWS are token-major (``i * k + j``,
        disagmoe/frontend/engine.py:668-676), so for k > 1 these labels do not line up with the rows:
        the reference's behaviour, kept; the tensors do not depend on it."""
        if topk == 1:
            return
        self.req_ids = list(self.req_ids) * topk
        self.init_prefill_lens = list(self.init_prefill_lens) * topk
        self.attn_dp_ranks = list(self.attn_dp_ranks) * topk
        self.shape = [self.shape[0] * topk] + list(self.shape[1:])

    def shrink_topk(self, topk: int) -> None:
        """datatypes.hpp:349-352: only the row count shrinks."""
        if topk == 1:
            return
        self.shape = [self.shape[0] // topk] + list(self.shape[1:])
