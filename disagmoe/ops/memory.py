"""disagmoe/ops/memory.py of the reference: get_mappings_from_exp_ids, get_mappings_from_exp_ids_cuda, permute_tokens_cuda, permute_tokens_triton (same module object as disagmoe_amd.ops.memory)."""
import sys

import disagmoe_amd.ops.memory as _impl

sys.modules[__name__] = _impl
