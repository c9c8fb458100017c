"""Routing parity (bit-exact) of the HIP counting sort against the oracle."""
import json
import os

import numpy as np
import pytest
import torch

from disagmoe_amd import _lib, workloads
from disagmoe_amd.ops import memory
from oracle import routing
from helpers import announce, dev

pytestmark = pytest.mark.gpu


def _check(ids_cpu: torch.Tensor, E: int):
    R = ids_cpu.numel()
    m_ref, cnt_ref = routing.get_mappings_from_exp_ids(ids_cpu, E)
    _, off_ref = routing.histogram_offsets(ids_cpu, E)
    st_ref = routing.get_mappings_stable(ids_cpu, E)
    for map_dtype in (torch.int64, torch.int32):
        m, bs, off = memory.route_tokens(ids_cpu.to(dev()), E, _lib.ORDER_REFERENCE, map_dtype=map_dtype)
        assert m.dtype == map_dtype and bs.dtype == torch.int64 and off.dtype == torch.int64
        assert m.cpu().tolist() == m_ref
        assert bs.cpu().tolist() == cnt_ref
        assert off.cpu().tolist() == off_ref.tolist()
    m, bs, off = memory.route_tokens(ids_cpu.to(dev()), E, _lib.ORDER_STABLE)
    assert m.cpu().tolist() == st_ref.tolist()
    assert R == 0 or sorted(m.cpu().tolist()) == list(range(R))


def test_known_answers(golden_dir):
    with open(os.path.join(golden_dir, "routing_kat.json")) as f:
        cases = json.load(f)["cases"]
    for case in cases:
        announce(test="route_kat", ids=case["ids"], E=case["E"])
        m, cnt = memory.get_mappings_from_exp_ids(case["ids"], case["E"])
        assert isinstance(m, list) and isinstance(cnt, list)
        assert m == case["mappings"] and cnt == case["exp_cnt"]
        m32, empty = memory.get_mappings_from_exp_ids_cuda(torch.tensor(case["ids"], dtype=torch.int64, device=dev()), case["E"])
        assert empty == [] and m32.dtype == torch.int32 and m32.cpu().tolist() == case["stable"]


@pytest.mark.parametrize("R", [1, 63, 64, 65, 511, 512, 513, 1024, 5000, 6144, 6145, 16384, 16385, 16897, 49152, 300007])
@pytest.mark.parametrize("E", [1, 2, 8, 64, 100])
def test_random_ids(R, E):
    announce(test="route_random", R=R, E=E)
    g = torch.Generator().manual_seed(R * 131 + E)
    for dtype in (torch.int32, torch.int64):
        ids = torch.randint(0, E, (R,), generator=g).to(dtype)
        _check(ids, E)


def test_empty_experts_and_skew():
    announce(test="route_skew")
    g = torch.Generator().manual_seed(7)
    ids = torch.randint(2, 8, (64,), generator=g)           # tests/ops/test_memory.py:14: experts 0, 1 empty
    _check(ids, 8)
    ids = torch.full((3000,), 5, dtype=torch.int64)          # everything on one expert
    _check(ids, 8)
    ids = torch.cat([torch.zeros(700, dtype=torch.int64), torch.full((900,), 299, dtype=torch.int64)])
    _check(ids, 300)                                          # E > 64: several scan rounds


def test_tensor_shapes_and_lists():
    announce(test="route_shapes")
    ids = torch.tensor([[2, 0], [2, 1], [0, 2]], dtype=torch.int32)
    m, cnt = memory.get_mappings_from_exp_ids(ids, 3)         # [T, k] input is flattened token-major
    assert m == [5, 1, 4, 2, 0, 3] and cnt == [2, 1, 3]
    m2, _ = memory.get_mappings_from_exp_ids(ids.to(dev()), 3)
    assert m2 == m
    assert memory.get_mappings_from_exp_ids([], 4) == ([], [0, 0, 0, 0])
    with pytest.raises(IndexError):
        memory.get_mappings_from_exp_ids([0, 3], 3)


def test_invalid_ids_are_marked_not_written():
    announce(test="route_invalid")
    ids = torch.tensor([1, 9, 0, -4, 1], dtype=torch.int64, device=dev())
    m, bs, off = memory.route_tokens(ids, 2)
    assert m.cpu().tolist() == [2, -1, 0, -1, 1]
    assert bs.cpu().tolist() == [1, 2] and off.cpu().tolist() == [0, 1, 3]


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_benchmark_configs(name):
    w = workloads.WORKLOADS[name]
    announce(test="route_config", config=name, R=w.R, E=w.E)
    ids, _ = workloads.make_routing(w)
    _check(ids.view(-1), w.E)


def test_merge_of_several_batches():
    announce(test="route_merge")
    rng = np.random.default_rng(3)
    batches = [rng.integers(0, 8, size=n).tolist() for n in (700, 0, 33, 1200)]
    m_ref, cnt_ref = routing.merge_by_exp_ids(batches, 8)
    flat = torch.tensor([v for b in batches for v in b], dtype=torch.int32, device=dev())
    m, bs, _ = memory.route_tokens(flat, 8)
    assert m.cpu().tolist() == m_ref and bs.cpu().tolist() == cnt_ref


def test_expert_count_limits():
    # the routing tables of E entries live in LDS: up to 4096 experts, more is refused
    announce(test="route_max_experts")
    from disagmoe_amd._lib import DmoeError
    g = torch.Generator().manual_seed(11)
    _check(torch.randint(0, 4096, (10000,), generator=g), 4096)
    _check(torch.randint(4000, 4096, (300,), generator=g), 4096)      # one chunk, nearly all experts empty
    _check(torch.randint(0, 4096, (40000,), generator=g), 4096)       # scanned histograms, 64 workgroups of experts
    _check(torch.randint(0, 4096, (1000,), generator=g), 4096)        # two chunks in one workgroup: 64 KiB of LDS
    _check(torch.randint(0, 4096, (1500,), generator=g), 4096)        # three chunks: their tables no longer fit
    with pytest.raises(DmoeError):
        memory.route_tokens(torch.zeros(8, dtype=torch.int64, device=dev()), 4097)
