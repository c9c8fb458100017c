"""The whole expert step (router logits -> top-k -> route -> permute -> FFN ->
combine) recorded once as a HIP graph over static buffers and replayed
(reference precedent: tests/cg/test_expert.py:27-57, static buffers of
disagmoe/frontend/engine.py:263,374).  Every replay is checked bit for bit
against the eager result of the same inputs, with eager work and
synchronisations between the replays."""
import pytest
import torch

from disagmoe_amd import workloads
from disagmoe_amd.expert_layer import expert_layer_forward
from disagmoe_amd.ops import routing as dev_routing
from helpers import announce, dev
from test_gpu_layer import _layer_from

pytestmark = pytest.mark.gpu


def _step(layer, x, logits, k):
    weights, ids = dev_routing.fused_topk(x, logits, k, True)
    return expert_layer_forward(layer, x, ids, weights)


@pytest.mark.parametrize("name,T,fp8", [("C1", 512, False), ("C3", 256, False), ("C4", 1024, False), ("C1", 512, True)])
def test_graph_replays_equal_eager(name, T, fp8):
    w = workloads.WORKLOADS[name]
    announce(test="graph_replay", config=name, T=T, d=w.d, I=w.I, E=w.E, k=w.k, fp8=fp8)
    w13, w2 = workloads.make_weights(w, dev())
    if fp8:   # the fp8 step: rows quantised inside the permute, the intermediate quantised between the GEMMs
        from disagmoe_amd.models.experts import MoEExpertsFP8
        layer = MoEExpertsFP8(w13, w2)
    else:
        layer = _layer_from(w13, w2)
    g = torch.Generator().manual_seed(77)
    x_static = torch.zeros(T, w.d, dtype=torch.bfloat16, device=dev())
    logits_static = torch.zeros(T, w.E, dtype=torch.float32, device=dev())

    def fresh():
        return torch.randn(T, w.d, generator=g).to(torch.bfloat16), torch.randn(T, w.E, generator=g) * 2.0

    # warm up on a side stream (allocator pools, lazy kernel attributes), then record
    x0, l0 = fresh()
    x_static.copy_(x0)
    logits_static.copy_(l0)
    side = torch.cuda.Stream(device=dev())
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            _step(layer, x_static, logits_static, w.k)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = _step(layer, x_static, logits_static, w.k)

    for rep in range(4):
        xr, lr = fresh()
        x_static.copy_(xr)
        logits_static.copy_(lr)
        graph.replay()
        torch.cuda.synchronize()
        got = out_static.clone()
        eager = _step(layer, xr.to(dev()), lr.to(dev()), w.k)   # eager work between replays, different routing
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {rep} differs from the eager step"


def test_expert_worker_step_recorded_once():
    # the device half of process_batch_expert (uploads from pinned staging into the static buffers, FFN, scale + return
    # permute) recorded once; every replay follows the host half of a new batch of the same size
    from disagmoe_amd.config import ModelConfig
    from disagmoe_amd.executor import ExpertsExecutor
    from disagmoe_amd.expert_layer import ExpertWorker
    from test_gpu_layer import _expert_step_case, _expert_step_reference
    announce(test="graph_expert_worker")
    E, d, I, top_k, R = 8, 512, 768, 2, 192
    cfg = ModelConfig(hidden_size=d, num_layers=1, num_heads=8, num_kv_heads=8, num_experts=E, intermediate_size=I,
                      layer_ids=[0], top_k=top_k, max_batch_size_expert=256)
    ex = ExpertsExecutor(cfg, init_std=0.02)
    worker = ExpertWorker(ex, top_k=top_k)
    x_static = torch.zeros(R, d, dtype=torch.bfloat16, device=dev())
    meta, x, *case = _expert_step_case(E, d, R, top_k, seed=100)
    x_static.copy_(x)
    side = torch.cuda.Stream(device=dev())
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        worker.process_batch_expert(meta, x_static)                    # warm-up outside the recording
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    meta, x, *case = _expert_step_case(E, d, R, top_k, seed=101)
    x_static.copy_(x)
    worker.stage(meta)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = worker.run(0, x_static)
    for rep in range(4):
        meta, x, *case = _expert_step_case(E, d, R, top_k, seed=200 + rep)
        x_static.copy_(x)
        worker.stage(meta)
        graph.replay()
        torch.cuda.synchronize()
        got = out_static.clone()
        ref = _expert_step_reference(ex.operators[0], x, *case, E, False)      # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(got, ref), f"replay {rep}"
