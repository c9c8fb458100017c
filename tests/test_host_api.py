"""Host-side logic that needs no GPU: workload recipes, API surface, and that the
operators refuse to run without a HIP device instead of falling back."""
import inspect

import pytest
import torch

from disagmoe_amd import workloads
from disagmoe_amd.config import mixtral_config
from disagmoe_amd.grouped_gemm import backend as gg
from disagmoe_amd.models import experts
from disagmoe_amd.ops import memory


def test_workload_table_matches_the_five_configs():
    w = workloads.WORKLOADS
    assert (w["C1"].E, w["C1"].d, w["C1"].I, w["C1"].T, w["C1"].k) == (8, 1024, 2816, 512, 2)
    assert (w["C2"].E, w["C2"].d, w["C2"].I, w["C2"].T, w["C2"].k) == (8, 4096, 14336, 4096, 2)
    assert (w["C3"].T, w["C3"].routing) == (256, "zipf")
    assert (w["C4"].E, w["C4"].d, w["C4"].I, w["C4"].T, w["C4"].k) == (64, 2048, 1408, 8192, 6)
    assert (w["C5"].d, w["C5"].I, w["C5"].T, w["C5"].fp8) == (6144, 16384, 16384, True)
    assert abs(w["C2"].gemm_flops - 2.886e12) / 2.886e12 < 1e-3
    assert abs(w["C2"].permute_bytes - 1.343e8) / 1.343e8 < 1e-3


@pytest.mark.parametrize("name", ["C1", "C3", "C4"])
def test_routing_recipe(name):
    w = workloads.WORKLOADS[name]
    ids, gates = workloads.make_routing(w)
    assert ids.shape == (w.T, w.k) and ids.dtype == torch.int32
    assert int(ids.min()) >= 0 and int(ids.max()) < w.E
    srt = ids.sort(dim=1).values
    assert (srt[:, 1:] != srt[:, :-1]).all()          # without replacement
    assert torch.allclose(gates.sum(dim=1), torch.ones(w.T))
    ids2, gates2 = workloads.make_routing(w)
    assert torch.equal(ids, ids2) and torch.equal(gates, gates2)
    if w.routing == "zipf":
        cnt = torch.bincount(ids.view(-1).long(), minlength=w.E)
        assert cnt[0] > 3 * cnt[-1]


def test_reference_signatures():
    assert list(inspect.signature(memory.get_mappings_from_exp_ids).parameters) == ["exp_ids", "num_experts"]
    assert list(inspect.signature(memory.get_mappings_from_exp_ids_cuda).parameters) == ["exp_ids", "num_experts"]
    assert list(inspect.signature(memory.permute_tokens_cuda).parameters)[:2] == ["tokens", "mappings"]
    assert list(inspect.signature(memory.permute_tokens_triton).parameters) == ["tokens", "mappings"]
    p = inspect.signature(gg.gmm).parameters
    # the reference's five parameters first, in its order; the workspace pair behind them is keyword-only in practice
    assert list(p)[:5] == ["a", "b", "batch_sizes", "trans_b", "c"] and p["trans_b"].default is False
    assert all(p[k].default is None for k in list(p)[4:])
    assert list(inspect.signature(gg.gmm_with_arguments).parameters)[:5] == ["a", "b", "batch_sizes", "workspace", "arguments_ptr"]
    p = inspect.signature(experts.MoEExperts.__init__).parameters
    assert list(p)[1:7] == ["hidden_size", "intermediate_size", "num_experts", "tp_size", "enable_cutlass_cache", "max_batch_size"]
    # the reference's parameters in its order; what follows them is optional (the sizes in host memory beside a device tensor)
    p = inspect.signature(experts.MoEExperts.forward).parameters
    assert list(p)[:4] == ["self", "bs", "hiddens", "batch_sizes"] and all(p[k].default is None for k in list(p)[4:])
    cfg = mixtral_config()
    assert (cfg.hidden_size, cfg.intermediate_size, cfg.num_experts, cfg.top_k) == (4096, 14336, 8, 2)


@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the no-device behaviour")
def test_no_cpu_fallback():
    x = torch.zeros(4, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        memory.permute_tokens_cuda(x, [0, 1, 2, 3])
    # ids that live on the host are sorted by the library's host code, as the reference's host loop does: no device
    assert memory.get_mappings_from_exp_ids([2, 0, 2, 1, 0, 2], 3) == ([5, 1, 4, 2, 0, 3], [2, 1, 3])
    with pytest.raises(IndexError):
        memory.get_mappings_from_exp_ids([0, 3], 3)
    with pytest.raises(RuntimeError):
        memory.route_tokens(torch.tensor([0, 1]), 2)
    with pytest.raises(RuntimeError):
        gg.gmm(x, torch.zeros(1, 8, 8, dtype=torch.bfloat16), torch.tensor([4]))
