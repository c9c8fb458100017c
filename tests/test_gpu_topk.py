"""Routing producer on the device against the oracle: ids bit-exact, weights to
fp32 round-off (tolerance 1e-5 relative: hardware exponential and reciprocal)."""
import numpy as np
import pytest
import torch

from disagmoe_amd import _lib
from disagmoe_amd.ops import routing as dev_routing
from oracle import routing
from helpers import announce, dev

pytestmark = pytest.mark.gpu

TOL_TOPK = 1e-5


def _check(x_cpu: torch.Tensor, k: int, renorm: bool, ids_dtype=torch.int32):
    w_ref, ids_ref = routing.fused_topk(x_cpu, k, renorm)
    hidden = torch.empty(x_cpu.shape[0], 1, device=dev())
    w, ids = dev_routing.fused_topk(hidden, x_cpu.to(dev()), k, renorm, ids_dtype=ids_dtype)
    assert w.dtype == torch.float32 and ids.dtype == ids_dtype and tuple(w.shape) == (x_cpu.shape[0], k)
    assert ids.cpu().tolist() == ids_ref.tolist()
    np.testing.assert_allclose(w.cpu().numpy(), w_ref, rtol=TOL_TOPK, atol=1e-30)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,E,k", [(1, 8, 2), (4096, 8, 2), (8192, 64, 6), (257, 5, 5), (100, 16, 1), (63, 32, 4),
                                   (300, 160, 8), (77, 1000, 32), (50, 256, 3), (31, 65, 7),
                                   # many tokens: narrow lane groups with several logits per lane
                                   (20000, 16, 2), (10000, 32, 4), (3000, 100, 8), (2500, 160, 6), (2100, 256, 32),
                                   (2049, 65, 7)])
def test_fused_topk(n, E, k, dtype):
    announce(test="fused_topk", n=n, E=E, k=k, dtype=str(dtype))
    g = torch.Generator().manual_seed(n * 131 + E)
    x = torch.randn(n, E, generator=g).to(dtype)
    _check(x, k, True)
    _check(x, k, False, ids_dtype=torch.int64)


def test_ties_and_masked_experts():
    announce(test="fused_topk_ties")
    x = torch.tensor([[1, 5, 5, 0, 5, 5, 5, 5], [0, 0, 0, 0, 0, 0, 0, 0]], dtype=torch.float32)
    _check(x, 3, True)
    x = torch.randint(-2, 3, (500, 12), generator=torch.Generator().manual_seed(3)).float()
    _check(x, 4, True)
    x = torch.randint(-2, 3, (10000, 12), generator=torch.Generator().manual_seed(5)).float()   # the narrow form
    _check(x, 4, True)
    x = torch.randn(64, 16, generator=torch.Generator().manual_seed(4))
    x[:, ::3] = float("-inf")                   # masked experts: probability 0, never ahead of a finite logit
    _check(x, 4, True)


def test_closed_form():
    announce(test="fused_topk_closed_form")
    x = torch.log(torch.arange(1, 5, dtype=torch.float64)).float()[None, :].to(dev())
    w, ids = dev_routing.fused_topk(None, x, 2, True)
    assert ids.cpu().tolist() == [[3, 2]]
    np.testing.assert_allclose(w.cpu().numpy(), [[4 / 7, 3 / 7]], rtol=1e-5)


def test_route_from_logits_matches_two_step():
    announce(test="route_from_logits")
    x = torch.randn(4096, 8, generator=torch.Generator().manual_seed(11))
    w, ids, mappings, bs, off = dev_routing.route_from_logits(x.to(dev()), 2)
    w_ref, ids_ref = routing.fused_topk(x, 2, True)
    m_ref, cnt_ref = routing.get_mappings_from_exp_ids(ids_ref.reshape(-1), 8)
    assert ids.cpu().tolist() == ids_ref.tolist()
    assert mappings.cpu().tolist() == m_ref and bs.cpu().tolist() == cnt_ref


def test_errors():
    x = torch.randn(4, 8, device=dev())
    for bad_k in (0, 9):
        with pytest.raises(_lib.DmoeError):
            dev_routing.fused_topk(None, x, bad_k)
    with pytest.raises(TypeError):
        dev_routing.fused_topk(None, x.double(), 2)
    with pytest.raises(ValueError):
        dev_routing.fused_topk(torch.empty(3, 1, device=dev()), x, 2)
    w, ids = dev_routing.fused_topk(None, x[:0], 2)
    assert tuple(w.shape) == (0, 2) and tuple(ids.shape) == (0, 2)
