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


def expert_layer_forward(experts: torch.nn.Module, x: torch.Tensor, topk_ids: torch.Tensor,
                         topk_weights: torch.Tensor, stages: Optional[Dict[str, torch.Tensor]] = None,
                         order: int = _lib.ORDER_REFERENCE) -> torch.Tensor:
    """``x [T, d]`` bf16, ``topk_ids [T, k]`` int, ``topk_weights [T, k]`` fp32 ->
    ``[T, d]``: ``out[i] = sum_j w[i, j] * FFN_{ids[i, j]}(x[i])``.  ``stages`` (if
    given) receives the intermediate tensors."""
    T, k = topk_ids.shape
    num_experts = experts.num_experts
    mappings, batch_sizes, offsets = memory.route_tokens(topk_ids, num_experts, order)
    permuted = memory.permute_tokens_cuda(x, mappings)
    expert_out = experts.forward(T * k, permuted, batch_sizes)
    out = memory.combine_tokens(expert_out, mappings, topk_weights)
    if stages is not None:
        stages.update(mappings=mappings, batch_sizes=batch_sizes, offsets=offsets, permuted=permuted,
                      expert_out=expert_out)
    return out
