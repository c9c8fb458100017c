"""The reference's own import lines and call shapes run unchanged against this tree.

The import statements are the literal lines of the reference's callers
(disagmoe/frontend/engine.py:6-7,13, disagmoe/executor/executor.py:14-15,
disagmoe/models/experts.py:3,7, tests/ops/test_gemm.py:1, tests/ops/test_mappings.py:1)
with the names this path does not build (attention, transport) left out of the tuple.
"""
import pytest
import torch

IMPORT_LINES = [
    "from disagmoe.ops.memory import permute_tokens_cuda as permute_tokens, get_mappings_from_exp_ids",   # engine.py:13
    "from disagmoe.ops.memory import get_mappings_from_exp_ids_cuda, permute_tokens_triton",
    "from grouped_gemm.backend import gmm",                                                              # experts.py:3
    "from grouped_gemm.backend import gmm, get_arguments, gmm_with_arguments",
    "from disagmoe.models.experts import MoEExperts, MoEExpertsSerial",                                  # executor.py:14
    "from disagmoe.executor.executor import ExpertsExecutor",                                            # engine.py:6
    "from disagmoe.config import ModelConfig",                                                           # engine.py:7
    "from disagmoe.utils.constants import MAX_BATCH_SIZE",                                               # experts.py:7
    "from disagmoe.frontend.datatypes import Metadata, TensorBatch",                                     # engine.py:9
]


@pytest.mark.parametrize("line", IMPORT_LINES)
def test_reference_import_line(line):
    scope = {}
    exec(line, scope)
    assert all(v is not None for k, v in scope.items() if not k.startswith("__"))


def test_aliases_are_the_same_modules():
    import disagmoe.ops.memory
    import disagmoe_amd.ops.memory
    import grouped_gemm.backend
    import disagmoe_amd.grouped_gemm.backend
    assert disagmoe.ops.memory is disagmoe_amd.ops.memory
    assert grouped_gemm.backend is disagmoe_amd.grouped_gemm.backend


def test_host_call_shape_of_the_dispatch_step():
    # engine.py:668-677: ids as a Python list -> (mappings list, counts) without a device
    from disagmoe.ops.memory import get_mappings_from_exp_ids
    expert_ids = torch.tensor([[2, 0], [2, 1], [0, 2]]).view(-1).tolist()
    exp_mappings, cnt = get_mappings_from_exp_ids(expert_ids, 3)
    assert exp_mappings == [5, 1, 4, 2, 0, 3] and cnt == [2, 1, 3]


@pytest.mark.gpu
def test_call_shapes_of_the_expert_step():
    # engine.py:675-677 (dispatch), :705 (execute), :734 (return permute), with the names the engine binds
    from disagmoe.ops.memory import permute_tokens_cuda as permute_tokens, get_mappings_from_exp_ids
    from disagmoe.executor.executor import ExpertsExecutor
    from disagmoe.config import ModelConfig
    from oracle import ffn, rows
    dev = torch.device("cuda", 0)
    cfg = ModelConfig(hidden_size=256, num_layers=1, num_heads=1, num_kv_heads=1, num_experts=4, intermediate_size=384,
                      dtype=torch.bfloat16, top_k=1)
    executor = ExpertsExecutor(cfg, device=dev, init_std=0.05)
    g = torch.Generator().manual_seed(2)
    hiddens = torch.randn(50, 256, generator=g).to(torch.bfloat16).to(dev)
    expert_ids = torch.randint(0, 4, (50,), generator=g).tolist()
    exp_mappings, cnt = get_mappings_from_exp_ids(expert_ids, cfg.num_experts)
    permuted = permute_tokens(hiddens, exp_mappings)
    assert torch.equal(permuted.cpu(), rows.permute_tokens(hiddens.cpu(), exp_mappings))
    batch_sizes = torch.tensor(cnt, dtype=torch.int64, device="cuda")
    output = executor.execute(0, 50, permuted, batch_sizes)
    op = executor.operators[0]
    ref = ffn.moe_experts_forward(permuted.cpu(), op.w13_weight.cpu(), op.w2_weight.cpu(), cnt)
    assert ffn.max_rel_err(output, ref) <= 1e-2
    inverse = [0] * 50
    for t, m in enumerate(exp_mappings):
        inverse[m] = t
    back = permute_tokens(output, torch.tensor(inverse, dtype=torch.int64, device="cuda"))
    assert torch.equal(back, output[torch.tensor(exp_mappings, device="cuda")])     # row t is back at position t
