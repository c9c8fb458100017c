"""Routing producer on the device: what the attention side of the reference gets
from vllm's ``fused_topk`` (disagmoe/models/attention.py:228-231), with the same
name, argument order and return types, computed by ``dmoe_topk_softmax`` of
libdmoe_hip.so on the current stream.  ``route_from_logits`` chains it with the
row mapping so that the expert ids never visit the host (the reference moves them
through ``.tolist()``: disagmoe/frontend/engine.py:668-675).
"""
from __future__ import annotations

from typing import Tuple

import torch

from .. import _lib
from .memory import _device_of, _stream, route_tokens

_LOGIT_DTYPES = {torch.float32: _lib.FP32, torch.bfloat16: _lib.BF16, torch.float16: _lib.FP16}


def fused_topk(hidden_states: torch.Tensor, gating_output: torch.Tensor, topk: int,
               renormalize: bool = True, ids_dtype: torch.dtype = torch.int32) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(topk_weights [n, topk] fp32, topk_ids [n, topk] int32)``: softmax over
    the experts in fp32, the ``topk`` largest (ties to the lower expert id) and,
    with ``renormalize``, the weights divided by their sum.  ``hidden_states`` is
    only checked for its token count, as in vllm."""
    if gating_output.dim() != 2:
        raise ValueError(f"gating_output must be [tokens, experts], got {tuple(gating_output.shape)}")
    if hidden_states is not None and hidden_states.shape[0] != gating_output.shape[0]:
        raise ValueError("Number of tokens mismatch")
    if gating_output.dtype not in _LOGIT_DTYPES:
        raise TypeError(f"router logits must be fp32, bf16 or fp16, got {gating_output.dtype}")
    if ids_dtype not in (torch.int32, torch.int64):
        raise TypeError(f"ids_dtype must be int32 or int64, got {ids_dtype}")
    device = _device_of(gating_output)
    logits = gating_output.to(device).contiguous()
    n, E = logits.shape
    with torch.cuda.device(device):
        weights = torch.empty(n, topk, dtype=torch.float32, device=device)
        ids = torch.empty(n, topk, dtype=ids_dtype, device=device)
        _lib.call("dmoe_topk_softmax", logits.data_ptr(), _LOGIT_DTYPES[logits.dtype], n, E, topk, int(bool(renormalize)),
                  weights.data_ptr(), ids.data_ptr(), _lib.I32 if ids_dtype == torch.int32 else _lib.I64,
                  _stream(device))
    return weights, ids


def route_from_logits(gating_output: torch.Tensor, topk: int, renormalize: bool = True,
                      order: int = _lib.ORDER_REFERENCE):
    """Router logits to everything the expert step needs, all on the device:
    ``(topk_weights [n, k] fp32, topk_ids [n, k] int32, mappings [n*k] int64,
    batch_sizes [E] int64, offsets [E+1] int64)``."""
    weights, ids = fused_topk(None, gating_output, topk, renormalize)
    mappings, batch_sizes, offsets = route_tokens(ids, gating_output.shape[1], order)
    return weights, ids, mappings, batch_sizes, offsets
