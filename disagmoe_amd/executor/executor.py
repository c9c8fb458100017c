"""``ExpertsExecutor`` with the interface of the reference
(disagmoe/executor/executor.py:349-370; layer id mapping :28-33)."""
from __future__ import annotations

from typing import Optional

import torch

from ..config import ModelConfig
from ..models.experts import MoEExperts, MoEExpertsSerial


class ExpertsExecutor:

    def __init__(self, model_config: ModelConfig, device: Optional[torch.device] = None, init_std: float = 1.0):
        self.model_config = model_config
        layer_ids = model_config.layer_ids if model_config.layer_ids is not None else list(range(model_config.num_layers))
        self.num_layers = len(layer_ids)
        # physical layer id -> index of the local operator
        self.layer_mappings = [0] * (max(layer_ids) + 1 if layer_ids else 0)
        for i, lid in enumerate(layer_ids):
            self.layer_mappings[lid] = i
        expert_cls = MoEExperts if model_config.enable_grouped_gemm else MoEExpertsSerial
        self.operators = [
            expert_cls(model_config.hidden_size, model_config.intermediate_size, model_config.num_experts_per_rank,
                       max_batch_size=model_config.max_batch_size_expert, device=device, init_std=init_std)
            for _ in range(self.num_layers)
        ]

    def execute(self, layer_id: int, num_tokens: int, hidden_states: torch.Tensor,
                batch_sizes: torch.Tensor, host_batch_sizes: Optional[torch.Tensor] = None) -> torch.Tensor:
        operator = self.operators[self.layer_mappings[layer_id]]
        if host_batch_sizes is None:
            return operator.forward(num_tokens, hidden_states, batch_sizes)
        return operator.forward(num_tokens, hidden_states, batch_sizes, host_batch_sizes=host_batch_sizes)
