"""Per-row bookkeeping of a batch on the expert worker.

Mirror of the part of the reference's ``Metadata`` (csrc/include/datatypes.hpp:135-501) that the
expert step reads and writes (disagmoe/frontend/engine.py:683-739): the lists live on the host as
they do there, the sorting and moving runs in the C++ library (no Python loops over rows), and what
reaches the device is a row mapping for ``permute_tokens``.  ``serialize`` / ``deserialize`` read and
write the bytes the reference's workers exchange for a batch (cereal field order, datatypes.hpp:223-226).
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


def host_mappings(exp_ids: Sequence[int], n_expert: int):
    """``(mappings, exp_cnt)`` of the reference's counting sort (memory.py:38-52, datatypes.hpp:303-324)
    computed on the host lists: experts ascending, inside an expert the first row takes the last slot."""
    ids = _i32(exp_ids)
    mappings = np.empty(ids.size, dtype=np.int64)
    cnt = np.empty(n_expert, dtype=np.int64)
    _lib.call("dmoe_host_mappings", _ptr(ids), ids.size, n_expert, _ptr(mappings), _ptr(cnt))
    return mappings.tolist(), cnt.tolist()


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

    def serialize(self) -> bytes:
        """The bytes the reference's workers exchange for this Metadata: cereal's binary archive of the fields in the
        order of ``Metadata::serialize`` (datatypes.hpp:223-226; ``cerealize``, utils.hpp:150-157)."""
        import ctypes
        keep = [np.ascontiguousarray(np.asarray(self.shape, dtype=np.uint64)), np.frombuffer(self.dtype.encode(), dtype=np.uint8),
                _i32(self.req_ids), _i32(self.exp_ids), _i32(self.attn_dp_ranks), _i32(self.init_prefill_lens),
                np.ascontiguousarray(np.asarray(self.topk_weights, dtype=np.float32))]
        p = [a.ctypes.data if a.size else None for a in keep]
        view = _lib.MetadataView(p[0], keep[0].size, p[1], keep[1].size, int(self.layer_id), p[2], keep[2].size, p[3],
                                 keep[3].size, p[4], keep[4].size, p[5], keep[5].size, p[6], keep[6].size)
        need = ctypes.c_size_t(0)
        _lib.call("dmoe_metadata_wire_bytes", ctypes.byref(view), ctypes.byref(need))
        out = ctypes.create_string_buffer(need.value)
        _lib.call("dmoe_metadata_serialize", ctypes.byref(view), out, need.value)
        return out.raw

    @staticmethod
    def deserialize(blob: bytes) -> "Metadata":
        """Inverse of :meth:`serialize` (``decerealize``, utils.hpp:167-174).  Raises ``DmoeError`` on a blob that ends
        early or has bytes left over."""
        import ctypes
        lay = _lib.MetadataLayout()
        buf = (ctypes.c_char * len(blob)).from_buffer_copy(blob)
        _lib.call("dmoe_metadata_parse", buf, len(blob), ctypes.byref(lay))

        def take(off, n, dtype):
            return np.frombuffer(blob, dtype=dtype, count=int(n), offset=int(off)).tolist()

        return Metadata(shape=take(lay.off_shape, lay.n_shape, "<u8"),
                        dtype=bytes(blob[lay.off_dtype:lay.off_dtype + lay.n_dtype]).decode(), layer_id=int(lay.layer_id),
                        req_ids=take(lay.off_req_ids, lay.n_req_ids, "<i4"), exp_ids=take(lay.off_exp_ids, lay.n_exp_ids, "<i4"),
                        attn_dp_ranks=take(lay.off_attn_dp_ranks, lay.n_attn_dp_ranks, "<i4"),
                        init_prefill_lens=take(lay.off_init_prefill_lens, lay.n_init_prefill_lens, "<i4"),
                        topk_weights=take(lay.off_topk_weights, lay.n_topk_weights, "<f4"))

    @staticmethod
    def merge_by_exp_ids(metas: Sequence["Metadata"], n_expert: Optional[int] = None):
        """datatypes.hpp:287-337: the batches are concatenated and sorted by expert id with the rule of
        ``host_mappings``; returns ``(merged, mappings)`` with ``mappings[idx]`` = row of the idx-th
        incoming row in the merged batch.  ``n_expert`` defaults to the largest id + 1 (the reference
        sizes its table for 32 experts)."""
        assert len(metas) > 0
        cat = lambda name: [v for m in metas for v in getattr(m, name)]
        exp_ids = cat("exp_ids")
        total = sum(m.num_tokens() for m in metas)
        assert len(exp_ids) == total
        if n_expert is None:
            n_expert = max(exp_ids) + 1 if exp_ids else 1
        mappings, _ = host_mappings(exp_ids, n_expert)
        # the merged batch always carries one weight per row; batches without weights contribute zeros (:301, :327-329)
        weights = [w for m in metas for w in (m.topk_weights if len(m.topk_weights) else [0.0] * m.num_tokens())]
        merged = Metadata(shape=[total] + list(metas[0].shape[1:]), dtype=metas[0].dtype, layer_id=metas[0].layer_id,
                          req_ids=move_row_infos(cat("req_ids"), mappings) if total else [],
                          exp_ids=move_row_infos(exp_ids, mappings) if total else [],
                          attn_dp_ranks=move_row_infos(cat("attn_dp_ranks"), mappings) if total else [],
                          init_prefill_lens=move_row_infos(cat("init_prefill_lens"), mappings) if total else [],
                          topk_weights=move_row_infos(weights, mappings, dtype=np.float32) if total else [])
        return merged, mappings


@dataclass
class TensorBatch:
    """Rows on the device with their bookkeeping (datatypes.hpp:503-506)."""
    data: "torch.Tensor"
    metadata: Metadata

    @staticmethod
    def merge(batches: Sequence["TensorBatch"], n_expert: Optional[int] = None) -> "TensorBatch":
        """The expert worker's merge of the batches it received (datatypes.hpp:508-549): metadata by
        ``merge_by_exp_ids``, rows gathered through a table of row pointers.  The table is built on the
        device (one address per incoming row, scattered by the mapping), so nothing waits for the
        stream, where the reference fills it in a host loop and synchronises after the gather
        (csrc/cuda_ops/permute.cu:151).  The incoming tensors must stay alive until the gather has run."""
        import torch
        from . import memory
        assert len(batches) > 0
        meta, mappings = Metadata.merge_by_exp_ids([b.metadata for b in batches], n_expert)
        first = batches[0].data
        dev, hidden, dtype = first.device, first.shape[1], first.dtype
        row_bytes = hidden * first.element_size()
        addrs = []
        for b in batches:
            assert b.data.is_contiguous() and b.data.shape[1] == hidden and b.data.dtype == dtype
            assert b.data.shape[0] == b.metadata.num_tokens()
            addrs.append(b.data.data_ptr() + torch.arange(b.data.shape[0], dtype=torch.int64, device=dev) * row_bytes)
        table = torch.empty(meta.num_tokens(), dtype=torch.int64, device=dev)
        table[torch.tensor(mappings, dtype=torch.int64).to(dev, non_blocking=True)] = torch.cat(addrs)
        return TensorBatch(memory.gather_row_ptrs(table, hidden, dtype), meta)
