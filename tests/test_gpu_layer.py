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
    return layer


def test_c1_full_layer_against_oracle():
    w = workloads.WORKLOADS["C1"]
    announce(test="layer_c1", T=w.T, d=w.d, I=w.I, E=w.E)
    ids, gates = workloads.make_routing(w)
    x = workloads.make_activations(w)
    w13, w2 = workloads.make_weights(w, "cpu")
    layer = _layer_from(w13.to(dev()), w2.to(dev()))
    stages = {}
    out = expert_layer_forward(layer, x.to(dev()), ids.to(dev()), gates.to(dev()), stages=stages)
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
    out = expert_layer_forward(layer, x, ids.to(dev()), gates.to(dev()), stages=stages)
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
