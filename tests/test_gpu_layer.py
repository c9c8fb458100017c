"""Whole expert-layer parity on the benchmark configurations.

C1 is checked in full against the oracle.  C2/C3/C4 run at full size; the FFN is
compared on a sample of rows of every expert (the oracle needs seconds for
those), against the library matmul loop on the device, and the data-movement
stages through exact properties."""
import pytest
import torch

from disagmoe_amd import workloads
from disagmoe_amd.expert_layer import expert_layer_forward
from disagmoe_amd.models.experts import MoEExperts, MoEExpertsSerial
from oracle import cpu_path, ffn, routing
from helpers import TOL_BF16, announce, dev, max_rel_err

pytestmark = pytest.mark.gpu


def _layer_from(w13, w2):
    E, d, two_i = w13.shape
    layer = MoEExperts.__new__(MoEExperts)
    torch.nn.Module.__init__(layer)
    layer.hidden_size, layer.intermediate_size, layer.num_experts, layer.tp_size = d, two_i // 2, E, 1
    layer.w13_weight = torch.nn.Parameter(w13, requires_grad=False)
    layer.w2_weight = torch.nn.Parameter(w2, requires_grad=False)
    layer.act_fn = torch.nn.SiLU(inplace=True)
    layer.enable_cache = False
    layer.gmm_cache_max_batch_size = 0
    from disagmoe_amd.grouped_gemm import backend as gg
    layer.gmm = gg.gmm
    layer._init_gemm_state(w13.device)
    return layer


def test_c1_full_layer_against_oracle():
    w = workloads.WORKLOADS["C1"]
    announce(test="layer_c1", T=w.T, d=w.d, I=w.I, E=w.E)
    ids, gates = workloads.make_routing(w)
    x = workloads.make_activations(w)
    w13, w2 = workloads.make_weights(w, "cpu")
    layer = _layer_from(w13.to(dev()), w2.to(dev()))
    stages = {}
    out = expert_layer_forward(layer, x.to(dev()), ids.to(dev()), gates.to(dev()), stages=stages, fetch_rows=False)
    # the form without a permute launch (the gate-up kernel fetches the tokens' rows itself): the same bits
    st2 = {}
    out2 = expert_layer_forward(layer, x.to(dev()), ids.to(dev()), gates.to(dev()), stages=st2, fetch_rows=True)
    assert torch.equal(out2, out) and torch.equal(st2["expert_out"], stages["expert_out"])
    assert torch.equal(st2["row_token"].cpu().long(), torch.argsort(stages["mappings"].cpu()) // w.k)
    m_ref, cnt = routing.get_mappings_from_exp_ids(ids, w.E)
    assert stages["mappings"].cpu().tolist() == m_ref and stages["batch_sizes"].cpu().tolist() == cnt
    from oracle import rows
    xp = rows.permute_tokens(x, m_ref)
    assert torch.equal(stages["permuted"].cpu(), xp)
    y_ref = ffn.moe_experts_forward(xp, w13, w2, cnt)
    assert max_rel_err(stages["expert_out"], y_ref) <= TOL_BF16
    ref = ffn.combine(y_ref, m_ref, gates)
    assert max_rel_err(out, ref) <= TOL_BF16, max_rel_err(out, ref)
    # the CPU baseline path computes the same function
    assert max_rel_err(cpu_path.expert_layer(x, ids, gates, w13, w2), ref) <= 2e-2


@pytest.mark.parametrize("name,rows_per_expert", [("C2", 12), ("C3", 8), ("C4", 4)])
def test_full_size_layer(name, rows_per_expert):
    w = workloads.WORKLOADS[name]
    announce(test="layer_full_size", config=name, T=w.T, d=w.d, I=w.I, E=w.E, k=w.k)
    ids, gates = workloads.make_routing(w)
    x = workloads.make_activations(w).to(dev())
    w13, w2 = workloads.make_weights(w, dev())
    layer = _layer_from(w13, w2)
    stages = {}
    out = expert_layer_forward(layer, x, ids.to(dev()), gates.to(dev()), stages=stages, fetch_rows=False)
    # the default form for these sizes, which may leave the permute to the gate-up kernel: the same bits
    assert torch.equal(expert_layer_forward(layer, x, ids.to(dev()), gates.to(dev())), out)
    assert torch.equal(expert_layer_forward(layer, x, ids.to(dev()), gates.to(dev()), fetch_rows=True), out)
    torch.cuda.synchronize()
    m_ref, cnt = routing.get_mappings_from_exp_ids(ids, w.E)
    assert stages["mappings"].cpu().tolist() == m_ref and stages["batch_sizes"].cpu().tolist() == cnt
    xp, y = stages["permuted"], stages["expert_out"]
    # (1) sampled rows of every expert against the fp32 oracle
    off = stages["offsets"].cpu().tolist()
    worst = 0.0
    for e in range(w.E):
        n = cnt[e]
        if n == 0:
            continue
        pick = sorted(set([off[e], off[e] + n - 1] + [off[e] + (i * 7919) % n for i in range(rows_per_expert)]))
        sel = torch.tensor(pick, device=dev())
        ref = ffn.moe_experts_forward(xp[sel].cpu(), w13[e:e + 1].cpu(), w2[e:e + 1].cpu(), [len(pick)])
        worst = max(worst, max_rel_err(y[sel], ref))
    assert worst <= TOL_BF16, worst
    # (2) the whole FFN output against the per-expert library matmul loop on the device
    serial = MoEExpertsSerial.__new__(MoEExpertsSerial)
    serial.__dict__.update(layer.__dict__)
    y_lib = serial.forward(w.R, xp, stages["batch_sizes"].cpu())
    assert max_rel_err(y, y_lib) <= TOL_BF16, max_rel_err(y, y_lib)
    # (3) combine of the kernel's own FFN output against the oracle's combine
    ref_out = ffn.combine(y.cpu(), m_ref, gates)
    assert max_rel_err(out, ref_out) <= 2 ** -7
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("top_k", [1, 2])
def test_process_batch_expert(top_k):
    # the expert worker's step on an expert-sorted batch (engine.py:683-739): FFN, scale by the row's top-k weight,
    # rows back to prefill-then-decode order; lists of the bookkeeping moved along
    from disagmoe_amd.config import ModelConfig
    from disagmoe_amd.executor import ExpertsExecutor
    from disagmoe_amd.expert_layer import process_batch_expert
    from disagmoe_amd.ops.metadata import Metadata
    announce(test="process_batch_expert", top_k=top_k)
    E, d, I, R = 4, 512, 768, 300
    cfg = ModelConfig(hidden_size=d, num_layers=1, num_heads=8, num_kv_heads=8, num_experts=E, intermediate_size=I,
                      layer_ids=[0], top_k=top_k)
    ex = ExpertsExecutor(cfg, init_std=0.02)
    g = torch.Generator().manual_seed(5)
    exp_ids = torch.sort(torch.randint(0, E, (R,), generator=g)).values.tolist()          # arrives sorted by expert
    req_ids = torch.randperm(R, generator=g).tolist()
    lens = torch.where(torch.rand(R, generator=g) < 0.5, -1, 8).tolist()
    dp = torch.randint(0, 2, (R,), generator=g).tolist()
    weights = torch.rand(R, generator=g).tolist() if top_k > 1 else []
    x = torch.randn(R, d, generator=g).to(torch.bfloat16)
    meta = Metadata(shape=[R, d], layer_id=0, req_ids=list(req_ids), exp_ids=list(exp_ids), attn_dp_ranks=list(dp),
                    init_prefill_lens=list(lens), topk_weights=list(weights))
    out, new_meta = process_batch_expert(ex, meta, x.to(dev()), top_k=top_k)

    op = ex.operators[0]
    sizes = routing.expert_batch_sizes(exp_ids, E).tolist()
    y = ffn.moe_experts_forward(x, op.w13_weight.cpu(), op.w2_weight.cpu(), sizes)
    if top_k > 1:
        y = (y.float() * torch.tensor(weights).to(torch.bfloat16).float().view(-1, 1)).to(torch.bfloat16)
    mapping = routing.sort_by_prefill_order(req_ids, dp, lens)
    ref = torch.empty_like(y)
    ref[torch.tensor(mapping)] = y
    assert out.shape == (R, d)
    assert max_rel_err(out, ref) <= TOL_BF16, max_rel_err(out, ref)
    # bookkeeping: lists in the new order, expert ids dropped, layer stepped
    assert new_meta.req_ids == routing.apply_row_mapping(req_ids, mapping)
    assert new_meta.init_prefill_lens == routing.apply_row_mapping(lens, mapping)
    assert new_meta.exp_ids == [] and new_meta.layer_id == 1
    order = [(a, p == -1) for a, p in zip(new_meta.attn_dp_ranks, new_meta.init_prefill_lens)]
    assert order == sorted(order)
    # the data movement alone is exact: same FFN output scaled and moved by torch
    y_dev = op.forward(R, x.to(dev()), torch.tensor(sizes, device=dev()))
    if top_k > 1:
        y_dev = y_dev * torch.tensor(weights, dtype=torch.bfloat16, device=dev()).view(-1, 1)
    moved = torch.empty_like(y_dev)
    moved[torch.tensor(mapping, device=dev())] = y_dev
    assert torch.equal(out, moved)


def _expert_step_case(E, d, R, top_k, seed):
    from disagmoe_amd.ops.metadata import Metadata
    g = torch.Generator().manual_seed(seed)
    exp_ids = torch.sort(torch.randint(0, E, (R,), generator=g)).values.tolist()
    req_ids = torch.randperm(R, generator=g).tolist()
    lens = torch.where(torch.rand(R, generator=g) < 0.5, -1, 8).tolist()
    dp = torch.randint(0, 2, (R,), generator=g).tolist()
    weights = torch.rand(R, generator=g).tolist() if top_k > 1 else []
    x = torch.randn(R, d, generator=g).to(torch.bfloat16)
    meta = Metadata(shape=[R, d], layer_id=0, req_ids=list(req_ids), exp_ids=list(exp_ids), attn_dp_ranks=list(dp),
                    init_prefill_lens=list(lens), topk_weights=list(weights))
    return meta, x, exp_ids, req_ids, lens, dp, weights


def _expert_step_reference(op, x, exp_ids, req_ids, lens, dp, weights, E, pairing):
    """Statement by statement what engine.py:705-734 computes, with torch on the device: the FFN of the layer under
    test, the scale, the scatter to the return order."""
    sizes = routing.expert_batch_sizes(exp_ids, E).tolist()
    y = op.forward(len(exp_ids), x.to(dev()), torch.tensor(sizes, device=dev()))
    mapping = routing.sort_by_prefill_order(req_ids, dp, lens)
    if weights:
        w = list(weights)
        if pairing:   # the lists were reordered before the weights were read: position r holds the weight of the row that moves there
            w = routing.apply_row_mapping(weights, mapping)
        y = y * torch.tensor(w, dtype=torch.bfloat16, device=dev()).view(-1, 1)
    moved = torch.empty_like(y)
    moved[torch.tensor(mapping, device=dev())] = y
    return moved


@pytest.mark.parametrize("pairing", [False, True])
def test_expert_worker_static_buffers(pairing):
    # consecutive steps of different sizes through one worker's static buffers, one of them larger than the buffers;
    # with the reference's weight pairing and with each row's own weight
    from disagmoe_amd.config import ModelConfig
    from disagmoe_amd.executor import ExpertsExecutor
    from disagmoe_amd.expert_layer import ExpertWorker
    announce(test="expert_worker", pairing=pairing)
    E, d, I, top_k = 4, 512, 768, 2
    cfg = ModelConfig(hidden_size=d, num_layers=1, num_heads=8, num_kv_heads=8, num_experts=E, intermediate_size=I,
                      layer_ids=[0], top_k=top_k, max_batch_size_expert=256)
    ex = ExpertsExecutor(cfg, init_std=0.02)
    worker = ExpertWorker(ex, top_k=top_k, reference_weight_pairing=pairing)
    buffers = (worker.static_mappings.data_ptr(), worker.static_batch_sizes.data_ptr(), worker.static_weights.data_ptr())
    for seed, R in [(1, 200), (2, 256), (3, 90), (4, 300), (5, 120)]:          # 300 rows: beyond max_batch_size_expert
        meta, x, exp_ids, req_ids, lens, dp, weights = _expert_step_case(E, d, R, top_k, seed)
        out, new_meta = worker.process_batch_expert(meta, x.to(dev()))
        ref = _expert_step_reference(ex.operators[0], x, exp_ids, req_ids, lens, dp, weights, E, pairing)
        assert torch.equal(out, ref), (seed, R)
        assert new_meta.layer_id == 1 and new_meta.exp_ids == []
    assert buffers == (worker.static_mappings.data_ptr(), worker.static_batch_sizes.data_ptr(),
                       worker.static_weights.data_ptr())
    if not pairing:      # the two pairings differ whenever the return mapping moves rows
        meta, x, exp_ids, req_ids, lens, dp, weights = _expert_step_case(E, d, 100, top_k, 9)
        other = _expert_step_reference(ex.operators[0], x, exp_ids, req_ids, lens, dp, weights, E, True)
        out, _ = worker.process_batch_expert(meta, x.to(dev()))
        assert not torch.equal(out, other)
