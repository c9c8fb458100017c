"""The whole expert-worker step on one device: route -> permute -> SwiGLU FFN ->
gate-weighted combine.

Single-GPU statement of the reference's attention-side dispatch
(disagmoe/frontend/engine.py:663-680: mappings from the top-k ids, then the
duplicating permute), expert step (:683-739: batch sizes, executor, weight scale,
return permute) and top-k sum (:624-628), with every stage on the device and no
host synchronisation between them.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from . import _lib
from .ops import memory
from .ops.metadata import Metadata


def expert_layer_forward(experts: torch.nn.Module, x: torch.Tensor, topk_ids: torch.Tensor,
                         topk_weights: torch.Tensor, stages: Optional[Dict[str, torch.Tensor]] = None,
                         order: int = _lib.ORDER_REFERENCE, fetch_rows: Optional[bool] = None) -> torch.Tensor:
    """``x [T, d]`` bf16, ``topk_ids [T, k]`` int, ``topk_weights [T, k]`` fp32 ->
    ``[T, d]``: ``out[i] = sum_j w[i, j] * FFN_{ids[i, j]}(x[i])``.  ``stages`` (if
    given) receives the intermediate tensors of the kernels that ran; it does not change which
    kernels run.  ``fetch_rows``: whether the gate-up kernel fetches the tokens' rows by their
    place in the expert-sorted order (no permute launch, no ``[R, d]`` copy of the rows; same
    result bit for bit) instead of reading a permuted copy; ``None`` takes it where the experts
    say it is the faster form (``MoEExperts.takes_rows``)."""
    T, k = topk_ids.shape
    num_experts = experts.num_experts
    if hasattr(experts, "forward_quantized"):
        # fp8 experts: the routed rows are quantised on their way into the expert-sorted buffer
        mappings, batch_sizes, offsets = memory.route_tokens(topk_ids, num_experts, order)
        xq, xs = memory.permute_quantize(x, mappings)
        expert_out = experts.forward_quantized(T * k, xq, xs, batch_sizes)
        out = memory.combine_tokens(expert_out, mappings, topk_weights)
        if stages is not None:
            stages.update(mappings=mappings, batch_sizes=batch_sizes, offsets=offsets, permuted_q=xq,
                          permuted_scale=xs, expert_out=expert_out)
        return out
    if fetch_rows is None:
        fetch_rows = hasattr(experts, "forward_rows") and x.dtype == torch.bfloat16 and experts.takes_rows(T, T * k)
    if fetch_rows:
        mappings, batch_sizes, offsets, row_token = memory.route_tokens_with_sources(topk_ids, num_experts, order)
        expert_out = experts.forward_rows(x, row_token, batch_sizes)
        out = memory.combine_tokens(expert_out, mappings, topk_weights)
        if stages is not None:
            stages.update(mappings=mappings, batch_sizes=batch_sizes, offsets=offsets, row_token=row_token,
                          expert_out=expert_out)
        return out
    mappings, batch_sizes, offsets = memory.route_tokens(topk_ids, num_experts, order)
    permuted = memory.permute_tokens_cuda(x, mappings)
    expert_out = experts.forward(T * k, permuted, batch_sizes)
    out = memory.combine_tokens(expert_out, mappings, topk_weights)
    if stages is not None:
        stages.update(mappings=mappings, batch_sizes=batch_sizes, offsets=offsets, permuted=permuted,
                      expert_out=expert_out)
    return out


class ExpertWorker:
    """The expert worker's step with the static buffers of the reference's engine
    (disagmoe/frontend/engine.py:263 ``static_mappings_gpu``, :374 ``_static_bs_cuda``, :305-307 the
    host-to-device stream, :713-729 the pinned staging): nothing is allocated per step for batches of
    up to ``max_batch_size`` rows.

    ``process_batch_expert(meta, x)`` is the reference's ``Engine.process_batch_expert`` (:683-739).  It
    is ``stage(meta)`` (host: batch sizes, the return mapping and the weights go into pinned staging;
    the bookkeeping lists are reordered and the layer stepped) followed by ``run(layer_id, x)`` (device:
    uploads from the staging into the static buffers, FFN, scale + return permute in one kernel).
    ``run`` touches no Python-side data, so it can be recorded into a HIP graph and replayed after each
    ``stage`` of a batch of the same row count; a replay reads the pinned staging when it executes, so the
    caller waits for it (the graph's stream) before staging the next batch.  In eager use ``stage``
    waits by itself for the uploads of the step before.

    ``reference_weight_pairing=True`` reproduces the reference's scale exactly: it builds the weight
    tensor from the lists AFTER ``sort_by_prefill_order`` has reordered them (:715, then :726) and
    multiplies rows that are still in expert order (:732), i.e. row ``r`` is scaled by the weight of
    the row that ends up at position ``r``.  The default scales every row by its own weight."""

    def __init__(self, executor, top_k: int = 1, inner_exp_rank=None, max_batch_size: Optional[int] = None,
                 device: Optional[torch.device] = None, reference_weight_pairing: bool = False):
        cfg = executor.model_config
        self.executor = executor
        self.top_k = top_k
        self.num_experts = cfg.num_experts
        self.inner_exp_rank = list(inner_exp_rank) if inner_exp_rank is not None else None
        self.reference_weight_pairing = reference_weight_pairing
        self.max_batch_size = int(max_batch_size or cfg.max_batch_size_expert)
        dev = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        self.device = dev
        n_local = len(self.inner_exp_rank) if self.inner_exp_rank is not None else self.num_experts
        n = self.max_batch_size
        self.static_batch_sizes = torch.zeros(n_local, dtype=torch.int64, device=dev)
        self.static_mappings = torch.zeros(n, dtype=torch.int64, device=dev)
        self.static_weights = torch.zeros(n, dtype=torch.bfloat16, device=dev)
        self._host_batch_sizes = torch.zeros(n_local, dtype=torch.int64, pin_memory=True)
        self._host_mappings = torch.zeros(n, dtype=torch.int64, pin_memory=True)
        self._host_weights = torch.zeros(n, dtype=torch.bfloat16, pin_memory=True)
        self.h2d_stream = torch.cuda.Stream(device=dev)
        self._uploaded = torch.cuda.Event()       # the staged mapping and weights have been read: they may be rewritten
        self._sizes_uploaded = torch.cuda.Event() # the staged batch sizes have been read (they travel on the step's stream)
        self._consumed = torch.cuda.Event()       # the static buffers have been read: they may be rewritten
        self._uploaded.record(torch.cuda.current_stream(dev))
        self._sizes_uploaded.record(torch.cuda.current_stream(dev))
        self._consumed.record(torch.cuda.current_stream(dev))
        self._rows = 0
        self._overflow = None                     # (mappings, weights) of a batch beyond max_batch_size

    def stage(self, meta: Metadata) -> int:
        """Host half of the step; returns the row count."""
        rows = meta.num_tokens()
        sizes = meta.get_expert_batch_sizes(self.num_experts)
        if self.inner_exp_rank is not None:
            sizes = [sizes[i] for i in self.inner_exp_rank]
        own_weights = list(meta.topk_weights) if self.top_k > 1 else None
        mapping = meta.sort_by_prefill_order()
        weights = None
        if self.top_k > 1:
            weights = list(meta.topk_weights) if self.reference_weight_pairing else own_weights
            assert len(weights) == rows, f"{len(weights)} top-k weights for {rows} rows"
        self._uploaded.synchronize()              # the previous step's uploads have left the staging
        self._sizes_uploaded.synchronize()
        self._host_batch_sizes.copy_(torch.tensor(sizes, dtype=torch.int64))
        if rows <= self.max_batch_size:
            self._host_mappings[:rows].copy_(torch.tensor(mapping, dtype=torch.int64))
            if weights is not None:
                self._host_weights[:rows].copy_(torch.tensor(weights, dtype=torch.bfloat16))
            self._overflow = None
        else:   # larger than the static buffers: one-off tensors, as engine.py:720-721
            m = torch.tensor(mapping, dtype=torch.int64, pin_memory=True)
            wt = torch.tensor(weights, dtype=torch.bfloat16, pin_memory=True) if weights is not None else None
            self._overflow = (m, wt)
        self._rows = rows
        meta.step_layer()
        return rows

    def run(self, layer_id: int, input_tensor: torch.Tensor) -> torch.Tensor:
        """Device half of the step on the batch staged last."""
        rows = self._rows
        assert input_tensor.shape[0] == rows, f"{input_tensor.shape[0]} rows, {rows} staged"
        dev = self.device
        cur = torch.cuda.current_stream(dev)
        self.static_batch_sizes.copy_(self._host_batch_sizes, non_blocking=True)
        if not torch.cuda.is_current_stream_capturing():
            self._sizes_uploaded.record(cur)
        if self._overflow is not None:
            mappings = self._overflow[0].to(dev, non_blocking=True)
            weights = self._overflow[1].to(dev, non_blocking=True) if self._overflow[1] is not None else None
            output = self.executor.execute(layer_id, rows, input_tensor, self.static_batch_sizes,
                                               host_batch_sizes=self._host_batch_sizes)
        else:
            mappings = self.static_mappings[:rows]
            weights = self.static_weights[:rows] if self.top_k > 1 else None
            if torch.cuda.is_current_stream_capturing():
                # one stream inside a recording: the uploads become nodes of the graph
                mappings.copy_(self._host_mappings[:rows], non_blocking=True)
                if weights is not None:
                    weights.copy_(self._host_weights[:rows], non_blocking=True)
                output = self.executor.execute(layer_id, rows, input_tensor, self.static_batch_sizes,
                                               host_batch_sizes=self._host_batch_sizes)
            else:
                # the mapping and the weights travel on the upload stream while the FFN runs (engine.py:717-729)
                self.h2d_stream.wait_event(self._consumed)
                with torch.cuda.stream(self.h2d_stream):
                    mappings.copy_(self._host_mappings[:rows], non_blocking=True)
                    if weights is not None:
                        weights.copy_(self._host_weights[:rows], non_blocking=True)
                    self._uploaded.record(self.h2d_stream)
                output = self.executor.execute(layer_id, rows, input_tensor, self.static_batch_sizes,
                                               host_batch_sizes=self._host_batch_sizes)
                cur.wait_event(self._uploaded)
        output = memory.permute_tokens_cuda(output, mappings, row_scale=weights)
        if not torch.cuda.is_current_stream_capturing():
            if self._overflow is not None:
                self._uploaded.record(cur)
            self._consumed.record(cur)
        return output

    def process_batch_expert(self, meta: Metadata, input_tensor: torch.Tensor):
        layer_id = meta.layer_id
        self.stage(meta)
        return self.run(layer_id, input_tensor), meta


def process_batch_expert(executor, meta: Metadata, input_tensor: torch.Tensor,
                         inner_exp_rank=None, top_k: int = 1, reference_weight_pairing: bool = False):
    """``Engine.process_batch_expert`` (disagmoe/frontend/engine.py:683-739) as a function: the step of
    an :class:`ExpertWorker` that is created on first use and kept on ``executor`` (one per
    ``top_k`` / ``inner_exp_rank`` / pairing), so that later calls find its static buffers.
    Returns ``(output, meta)`` like the reference."""
    key = (top_k, tuple(inner_exp_rank) if inner_exp_rank is not None else None, reference_weight_pairing,
           input_tensor.device)
    workers = executor.__dict__.setdefault("_expert_workers", {})
    worker = workers.get(key)
    if worker is None:
        worker = ExpertWorker(executor, top_k=top_k, inner_exp_rank=inner_exp_rank, device=input_tensor.device,
                              reference_weight_pairing=reference_weight_pairing)
        workers[key] = worker
    return worker.process_batch_expert(meta, input_tensor)
