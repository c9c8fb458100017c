"""The fields of the reference's ``ModelConfig`` that the expert path reads
(disagmoe/config.py:9-39) and its Mixtral preset (:70-80)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, List


@dataclass
class ModelConfig:
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    num_experts: int
    intermediate_size: int
    dtype: object = None
    ep_size: int = 1
    tp_size: int = 1
    dp_size: int = 1
    rank: int = 0
    layer_ids: Optional[List[int]] = None
    top_k: int = 1
    enable_grouped_gemm: bool = True
    max_batch_size_expert: int = 512

    @property
    def num_experts_per_rank(self) -> int:
        return self.num_experts // self.ep_size


def mixtral_config() -> ModelConfig:
    import torch
    return ModelConfig(hidden_size=4096, num_layers=32, num_heads=32, num_kv_heads=8, num_experts=8,
                       intermediate_size=14336, dtype=torch.bfloat16, top_k=2)
