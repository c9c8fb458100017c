from .memory import (combine_tokens, gather_row_ptrs, gather_rows, get_mappings_from_exp_ids,
                     get_mappings_from_exp_ids_cuda, permute_tokens_cuda, permute_tokens_triton, route_tokens)

permute_tokens = permute_tokens_cuda

__all__ = [
    "get_mappings_from_exp_ids", "get_mappings_from_exp_ids_cuda", "permute_tokens_cuda", "permute_tokens_triton",
    "permute_tokens", "route_tokens", "gather_rows", "gather_row_ptrs", "combine_tokens",
]
