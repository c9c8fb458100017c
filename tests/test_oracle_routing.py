"""Pins the integer routing oracle without using its own formula: hand-derived
known answers, brute-force rank counting, library routines and invariants."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import routing


def _load(golden_dir, name):
    with open(os.path.join(golden_dir, name)) as f:
        return json.load(f)


def test_known_answers(golden_dir):
    for case in _load(golden_dir, "routing_kat.json")["cases"]:
        m, cnt = routing.get_mappings_from_exp_ids(case["ids"], case["E"])
        assert m == case["mappings"], case
        assert cnt == case["exp_cnt"], case
        assert routing.get_mappings_stable(case["ids"], case["E"]).tolist() == case["stable"], case
        c, off = routing.histogram_offsets(case["ids"], case["E"])
        assert off.tolist() == case["offsets"] and c.tolist() == case["exp_cnt"]


def _brute_force(ids, E):
    """Definition by counting: slot = offset + cnt - 1 - #{earlier rows of the same expert}."""
    R = len(ids)
    cnt = [sum(1 for v in ids if v == e) for e in range(E)]
    off = [sum(cnt[:e]) for e in range(E)]
    out = []
    for t in range(R):
        earlier = sum(1 for u in range(t) if ids[u] == ids[t])
        out.append(off[ids[t]] + cnt[ids[t]] - 1 - earlier)
    return out, cnt


@pytest.mark.parametrize("R,E,seed", [(1, 1, 0), (7, 3, 1), (64, 8, 2), (65, 8, 3), (200, 5, 4), (257, 64, 5), (300, 2, 6)])
def test_brute_force(R, E, seed):
    rng = np.random.default_rng(seed)
    ids = rng.integers(0, E, size=R).tolist()
    m, cnt = routing.get_mappings_from_exp_ids(ids, E)
    bm, bcnt = _brute_force(ids, E)
    assert m == bm and cnt == bcnt


@pytest.mark.parametrize("R,E,lo", [(4096, 8, 0), (5000, 64, 0), (64, 8, 2), (1000, 100, 37)])
def test_invariants(R, E, lo):
    # lo > 0 leaves the first experts empty, like tests/ops/test_memory.py:14 (ids in [2, 8))
    g = torch.Generator().manual_seed(R + E)
    ids = torch.randint(lo, E, (R,), generator=g)
    m, cnt = routing.get_mappings_from_exp_ids(ids, E)
    m = np.asarray(m)
    assert sorted(m.tolist()) == list(range(R))                 # a permutation
    assert sum(cnt) == R and all(c == 0 for c in cnt[:lo])
    placed = np.empty(R, dtype=np.int64)
    placed[m] = ids.numpy()
    assert (np.diff(placed) >= 0).all()                         # experts ascending in the sorted buffer
    src = np.empty(R, dtype=np.int64)
    src[m] = np.arange(R)
    same = placed[1:] == placed[:-1]
    assert (np.diff(src)[same] < 0).all()                       # descending t inside an expert
    # tensor input of any shape is flattened (memory.py:35-36)
    if R % 2 == 0:
        m2, _ = routing.get_mappings_from_exp_ids(ids.view(-1, 2), E)
        assert m2 == m.tolist()


@pytest.mark.parametrize("R,E", [(1, 1), (100, 8), (4097, 64)])
def test_stable_variant_is_inverse_of_stable_sort(R, E):
    g = torch.Generator().manual_seed(R)
    ids = torch.randint(0, E, (R,), generator=g)
    _, order = torch.sort(ids, stable=True)
    inv = torch.empty(R, dtype=torch.int64)
    inv[order] = torch.arange(R)
    got = routing.get_mappings_stable(ids, E)
    assert got.dtype == np.int32
    assert got.tolist() == inv.tolist()


def test_merge_equals_single_stream():
    rng = np.random.default_rng(9)
    batches = [rng.integers(0, 6, size=n).tolist() for n in (5, 0, 17, 1)]
    m, cnt = routing.merge_by_exp_ids(batches, 6)
    flat = [v for b in batches for v in b]
    bm, bcnt = _brute_force(flat, 6)
    assert m == bm and cnt == bcnt
    assert routing.merge_by_exp_ids([], 3) == ([], [0, 0, 0])


def test_expert_batch_sizes():
    ids = [5, 1, 1, 7, 5, 5]
    full = routing.expert_batch_sizes(ids, 8)
    assert full.dtype == np.int64 and full.tolist() == np.bincount(ids, minlength=8).tolist()
    # EP rank 1 of 2 owns experts 4..7 (engine.py:151-154)
    assert routing.expert_batch_sizes(ids, 8, [4, 5, 6, 7]).tolist() == [0, 3, 0, 1]


def test_prefill_order_known_answer(golden_dir):
    kat = _load(golden_dir, "prefill_kat.json")
    mapping = routing.sort_by_prefill_order(kat["req_ids"], kat["attn_dp_ranks"], kat["init_prefill_lens"])
    assert mapping == kat["mapping"]
    assert routing.apply_row_mapping(kat["init_prefill_lens"], mapping) == kat["sorted_init_prefill_lens"]


def test_prefill_order_dp_rank_first():
    mapping = routing.sort_by_prefill_order([3, 2, 1, 0], [1, 0, 1, 0], [4, -1, 4, 7])
    # dp 0: prefill req 0 then decode req 2; dp 1: prefill req 1 then req 3
    assert routing.apply_row_mapping([3, 2, 1, 0], mapping) == [0, 2, 1, 3]
