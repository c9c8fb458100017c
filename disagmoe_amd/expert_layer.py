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
                         order: int = _lib.ORDER_REFERENCE) -> torch.Tensor:
    """``x [T, d]`` bf16, ``topk_ids [T, k]`` int, ``topk_weights [T, k]`` fp32 ->
    ``[T, d]``: ``out[i] = sum_j w[i, j] * FFN_{ids[i, j]}(x[i])``.  ``stages`` (if
    given) receives the intermediate tensors of the kernels that ran; it does not change which
    kernels run."""
    T, k = topk_ids.shape
    num_experts = experts.num_experts
    mappings, batch_sizes, offsets = memory.route_tokens(topk_ids, num_experts, order)
    if hasattr(experts, "forward_quantized"):
        # fp8 experts: the routed rows are quantised on their way into the expert-sorted buffer
        xq, xs = memory.permute_quantize(x, mappings)
        expert_out = experts.forward_quantized(T * k, xq, xs, batch_sizes)
        out = memory.combine_tokens(expert_out, mappings, topk_weights)
        if stages is not None:
            stages.update(mappings=mappings, batch_sizes=batch_sizes, offsets=offsets, permuted_q=xq,
                          permuted_scale=xs, expert_out=expert_out)
        return out
    permuted = memory.permute_tokens_cuda(x, mappings)
    expert_out = experts.forward(T * k, permuted, batch_sizes)
    out = memory.combine_tokens(expert_out, mappings, topk_weights)
    if stages is not None:
        stages.update(mappings=mappings, batch_sizes=batch_sizes, offsets=offsets, permuted=permuted,
                      expert_out=expert_out)
    return out


def process_batch_expert(executor, meta: Metadata, input_tensor: torch.Tensor,
                         inner_exp_rank=None, top_k: int = 1):
    """The expert worker's step on a batch that arrives sorted by expert id
    (disagmoe/frontend/engine.py:683-739): batch sizes of the local experts from the
    bookkeeping, the FFN, then the rows go back to prefill-then-decode order, scaled by
    their top-k weights on the way (one kernel: the scale is an argument of the permute).
    ``executor`` is an ``ExpertsExecutor``; returns ``(output, meta)`` like the reference.

    A row is scaled by its own weight.  The reference builds the weight tensor from the lists
    after ``sort_by_prefill_order`` has reordered them (engine.py:715, then :726) and multiplies
    rows that are still in expert order (:732), which pairs rows with other rows' weights
    whenever the return mapping is not the identity; that is not reproduced."""
    num_tokens = meta.num_tokens()
    dev = input_tensor.device
    num_experts = executor.model_config.num_experts
    sizes = meta.get_expert_batch_sizes(num_experts)
    if inner_exp_rank is not None:
        sizes = [sizes[i] for i in inner_exp_rank]
    batch_sizes = torch.tensor(sizes, dtype=torch.int64).to(dev, non_blocking=True)
    output = executor.execute(meta.layer_id, num_tokens, input_tensor, batch_sizes)
    # the weights travel with the rows: read them before the lists are reordered
    weights = None
    if top_k > 1:
        weights = torch.tensor(meta.topk_weights, dtype=output.dtype).to(dev, non_blocking=True)
    new_mappings = meta.sort_by_prefill_order()
    mappings = torch.tensor(new_mappings, dtype=torch.int64).to(dev, non_blocking=True)
    output = memory.permute_tokens_cuda(output, mappings, row_scale=weights)
    meta.update_exp_ids([], [])
    meta.step_layer()
    return output, meta
