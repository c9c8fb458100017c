from .memory import (combine_tokens, gather_row_ptrs, gather_rows, get_mappings_from_exp_ids,
                     get_mappings_from_exp_ids_cuda, permute_quantize, permute_tokens_cuda, permute_tokens_triton,
                     route_tokens)

from .metadata import Metadata, TensorBatch, expert_batch_sizes, host_mappings, move_row_infos, sort_by_prefill_order
from .routing import fused_topk, route_from_logits

permute_tokens = permute_tokens_cuda

__all__ = [
    "get_mappings_from_exp_ids", "get_mappings_from_exp_ids_cuda", "permute_tokens_cuda", "permute_tokens_triton",
    "permute_tokens", "permute_quantize", "route_tokens", "gather_rows", "gather_row_ptrs", "combine_tokens",
    "fused_topk", "route_from_logits", "Metadata", "TensorBatch", "host_mappings", "sort_by_prefill_order", "move_row_infos", "expert_batch_sizes",
]
